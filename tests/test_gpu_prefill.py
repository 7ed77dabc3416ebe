"""Prompt ingestion in one pass per layer (vui_prefill) against the oracle's bf16 regime and against the
position-by-position path of the same library.  Reference: Decoder.forward_flash with T > 1 /
Engine._prefill_emb (src/vui/model.py:534-549, engine.py:674-694)."""
import pytest
import torch

from oracle import vui_oracle as O
from tests.util import TINY_SD, make_model, rel_err

pytestmark = pytest.mark.gpu
BF, F32 = torch.bfloat16, torch.float32
BF16_TOL = 2.0 ** -5  # 8 bf16 ulps of the largest value, as for the decode step


def _dims(kv):
    # head_dim 32 (the pass needs multiples of 32), ffn 512
    return O.Dims(d_model=128, n_layers=3, n_heads=4, n_kv_heads=kv, n_quantizers=4, codebook_size=32, rq_d_model=64,
                  rq_n_layers=1, rq_n_heads=2, vocab_size=50, max_seqlen=256)


@pytest.mark.parametrize("kv", [4, 2])
def test_prefill_pass_vs_oracle_and_stepwise(kv):
    d = _dims(kv)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    sdb = {k: O.rnd(v, BF) for k, v in sd.items()}
    o = O.OracleModel(d, sdb, BF, n_slots=2, max_seqlen=256)
    of = O.OracleModel(d, sdb, F32, n_slots=2, max_seqlen=256)
    m = make_model(d, sd, BF, max_seqlen=256)
    m.decoder.allocate_flash_kv_cache(2, m.device, BF)
    seq = m.decoder.flash_kv_caches[0].seq_lens
    g = torch.Generator().manual_seed(11)
    blocks = [O.rnd(torch.randn(T, d.d_model, generator=g) * 0.5, BF) for T in (37, 70, 5)]  # 70 crosses a 64-row tile
    slot = torch.tensor([1], dtype=torch.int32, device="cuda")
    pos = 0
    for emb in blocks:
        ref = o.prefill(emb, slot=1)
        ref32 = of.prefill(emb, slot=1)
        got = m.decoder.forward_flash(emb[None].to(BF).cuda(), None, slot_idx=slot)[0]
        pos += emb.shape[0]
        assert int(seq[1]) == pos and int(seq[0]) == 0
        assert rel_err(got, ref) <= BF16_TOL, rel_err(got, ref)
        assert rel_err(got, ref32) <= 1.3 * rel_err(ref, ref32) + 2.0 ** -8
    # cache rows written by the pass: in layer 0 only the summation order inside the dot products differs from
    # the oracle (a bf16 rounding flips here and there, by one ulp), deeper layers within the tolerance
    for l in range(d.n_layers):
        for mine, theirs in ((m.decoder._k, o.k_cache), (m.decoder._v, o.v_cache)):
            a, b = mine[l, 1, :pos].float().cpu(), theirs[l, 1, :pos]
            if l == 0:
                assert float((a != b).float().mean()) < 0.01
                assert float(((a - b).abs() / b.abs().clamp_min(1e-3)).max()) <= 2.0 ** -7
            assert rel_err(a, b) <= BF16_TOL
    assert float(m.decoder._k[:, 0].abs().sum()) == 0  # the other slot is untouched

    # the same blocks position by position through the decode step
    m2 = make_model(d, sd, BF, max_seqlen=256)
    m2.decoder.allocate_flash_kv_cache(2, m2.device, BF)
    m2.decoder.PREFILL_MIN = 10 ** 9
    outs = [m2.decoder.forward_flash(e[None].to(BF).cuda(), None, slot_idx=slot)[0] for e in blocks]
    m.decoder.flash_kv_caches[0].seq_lens[1] = 0
    m.decoder.PREFILL_CHUNK = 32  # several chunks per block
    for e, want in zip(blocks, outs):
        got = m.decoder.forward_flash(e[None].to(BF).cuda(), None, slot_idx=slot)[0]
        assert rel_err(got, want) <= BF16_TOL, rel_err(got, want)
    # a decode step after either prefill sees equivalent caches
    codes = torch.randint(0, d.codebook_size, (1, d.n_quantizers), generator=g).cuda()
    res = []
    for mm in (m, m2):
        cb0 = torch.empty(1, d.codebook_size, dtype=BF, device="cuda")
        mm.decoder._step(codes=codes, emb=None, slot_idx=slot, seq_inc=None, B=1, hidden_out=None, cb0_out=cb0, eos_out=None,
                         n_splits=4, stream=torch.cuda.current_stream().cuda_stream)
        res.append(cb0.float().cpu())
    assert rel_err(res[0], res[1]) <= BF16_TOL


def test_prefill_window_and_errors():
    d = _dims(4)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    from tests.util import dims_to_config
    from vui_amd.model import Vui

    cfg = dims_to_config(d, 256)
    cfg.model.window_size = 16
    m = Vui(cfg, sd, device="cuda", dtype=BF)
    m.decoder.allocate_flash_kv_cache(1, m.device, BF)
    g = torch.Generator().manual_seed(2)
    emb = O.rnd(torch.randn(1, 50, d.d_model, generator=g) * 0.5, BF).to(BF).cuda()
    a = m.decoder.forward_flash(emb, None)
    m.decoder.flash_kv_caches[0].seq_lens.zero_()
    m.decoder.PREFILL_MIN = 10 ** 9
    b = m.decoder.forward_flash(emb, None)
    assert rel_err(a, b) <= BF16_TOL  # sliding window: same visible range as the decode step
    m.decoder.PREFILL_MIN = 4
    with pytest.raises(ValueError):
        m.decoder.forward_flash(torch.zeros(1, 300, d.d_model, dtype=BF, device="cuda"), None)


@pytest.mark.parametrize("int8", [False, True])
def test_prefill_nano_576_positions(int8):
    """The benchmark's prompt (512 audio frames + 64 text tokens) at Vui Nano dims, with bf16 and with weight-only
    int8 matrices: the pass against the oracle (which evaluates the same int8 weights) on the first 96 positions,
    its last hidden state and the cache it leaves against the position-by-position path."""
    d = O.Dims()
    sd = O.synthetic_state_dict(d, seed=0)
    m = make_model(d, sd, BF, int8=int8, max_seqlen=1408)
    m.decoder.allocate_flash_kv_cache(1, m.device, BF, max_seqlen=1408)
    assert m.decoder._prefill_available()
    g = torch.Generator().manual_seed(0)
    emb = O.rnd(torch.randn(1, 576, d.d_model, generator=g) * 0.02 * 4, BF).to(BF).cuda()
    o = O.OracleModel(d, sd, BF, n_slots=1, max_seqlen=128, int8=int8)
    ref96 = o.prefill(emb[0, :96].float().cpu(), slot=0)
    got96 = m.decoder.forward_flash(emb[:, :96].contiguous(), None)[0]
    assert rel_err(got96, ref96) <= BF16_TOL, rel_err(got96, ref96)
    m.decoder.flash_kv_caches[0].seq_lens.zero_()
    a = m.decoder.forward_flash(emb, None)
    ka = m.decoder._k[:, 0, :576].clone()
    m.decoder.flash_kv_caches[0].seq_lens.zero_()
    m.decoder.PREFILL_MIN = 10 ** 9
    b = m.decoder.forward_flash(emb, None)
    assert int(m.decoder.flash_kv_caches[0].seq_lens[0]) == 576
    assert rel_err(a[0, -1], b[0, -1]) <= BF16_TOL, rel_err(a[0, -1], b[0, -1])
    assert rel_err(a, b) <= 2 * BF16_TOL
    assert rel_err(ka, m.decoder._k[:, 0, :576]) <= BF16_TOL
    k0a, k0b = ka[0].float(), m.decoder._k[0, 0, :576].float()  # layer 0 keys: only the summation order differs
    assert float((k0a != k0b).float().mean()) < 0.01


@pytest.mark.parametrize("heads,kv,rope_dim", [(4, 2, 64), (2, 1, 64), (2, 2, 128)])
def test_prefill_other_head_dims(heads, kv, rope_dim):
    """head_dim 64 and 128 (other instantiations of the attention kernel; 128 runs four waves per workgroup), grouped
    KV heads, a rotation that covers only part of the head: the pass against the oracle's bf16 regime, and the
    cache it leaves against the position-by-position path, across a block boundary of the staged keys."""
    d = O.Dims(d_model=256, n_layers=2, n_heads=heads, n_kv_heads=kv, n_quantizers=4, codebook_size=32, rq_d_model=64,
               rq_n_layers=1, rq_n_heads=2, vocab_size=50, max_seqlen=192, rope_dim=rope_dim)
    assert d.head_dim in (64, 128)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    sdb = {k: O.rnd(v, BF) for k, v in sd.items()}
    o = O.OracleModel(d, sdb, BF, n_slots=1, max_seqlen=192)
    m = make_model(d, sd, BF, max_seqlen=192)
    m.decoder.allocate_flash_kv_cache(1, m.device, BF)
    assert m.decoder._prefill_available()
    m2 = make_model(d, sd, BF, max_seqlen=192)
    m2.decoder.allocate_flash_kv_cache(1, m2.device, BF)
    m2.decoder.PREFILL_MIN = 10 ** 9
    g = torch.Generator().manual_seed(3)
    pos = 0
    for T in (45, 83):  # 45 + 83 = 128 positions: the second block starts inside a staged block of 32 keys
        emb = O.rnd(torch.randn(T, d.d_model, generator=g) * 0.5, BF)
        ref = o.prefill(emb, slot=0)
        got = m.decoder.forward_flash(emb[None].to(BF).cuda(), None)[0]
        want = m2.decoder.forward_flash(emb[None].to(BF).cuda(), None)[0]
        pos += T
        assert int(m.decoder.flash_kv_caches[0].seq_lens[0]) == pos
        assert rel_err(got, ref) <= BF16_TOL, rel_err(got, ref)
        assert rel_err(got, want) <= BF16_TOL, rel_err(got, want)
    for mine, theirs in ((m.decoder._k, m2.decoder._k), (m.decoder._v, m2.decoder._v)):
        assert rel_err(mine[:, 0, :pos], theirs[:, 0, :pos]) <= BF16_TOL
