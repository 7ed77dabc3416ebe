"""Dimension-generic claim of the kernels: randomly drawn architectures (head_dim 8..128, grouped KV heads, partial
rotation, sliding window with global layers, 2..16 codebooks of 16..2048 entries, depth heads 8..512 wide) through
both forms of the bf16 decode step, the prompt pass and the depth head, against the oracle's bf16 regime."""
import random

import pytest
import torch

from oracle import vui_oracle as O
from tests.util import TINY_SD, make_model, rel_err

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
TOL = 2.0 ** -5  # the stated bf16 tolerance (tests/test_gpu_model.py)


def _dims(rnd: random.Random) -> O.Dims:
    hd = rnd.choice([8, 16, 24, 32, 48, 64, 96, 128])
    H = rnd.choice([1, 2, 3, 4, 6, 8])
    while hd * H > 1024:
        H = max(1, H // 2)
    kv = rnd.choice([k for k in (1, 2, 3, 4, 6, 8) if H % k == 0])
    rh = rnd.choice([1, 2, 4, 8])
    rhd = rnd.choice([8, 16, 32, 64])
    kw = dict(d_model=hd * H, n_layers=rnd.randint(1, 4), n_heads=H, n_kv_heads=kv, n_quantizers=rnd.choice([2, 3, 4, 8, 16]),
              codebook_size=rnd.choice([16, 32, 100, 256, 1024, 2048]), rq_d_model=rh * rhd, rq_n_layers=rnd.randint(1, 3),
              rq_n_heads=rh, vocab_size=50, max_seqlen=96, intermediate_size=rnd.choice([None, 8 * rnd.randint(2, 40)]))
    if rnd.random() < 0.4:
        kw["rope_dim"] = rnd.choice([x for x in (4, 8, 16, 32) if x <= hd])
    if rnd.random() < 0.4:
        kw["window_size"] = rnd.choice([3, 6, 17])
        kw["global_every"] = rnd.choice([None, 2, 3])
        if rnd.random() < 0.5:
            kw["global_rope_dim"] = rnd.choice([x for x in (4, 8, 16) if x <= hd])
    return O.Dims(**kw)


@pytest.mark.parametrize("seed", range(24))
def test_random_architecture_vs_oracle(seed):
    rnd = random.Random(seed)
    d = _dims(rnd)
    sdkw = dict(TINY_SD)
    sdkw["std"] = 0.15 * (64.0 / max(64, d.d_model)) ** 0.5  # keeps the activations' range independent of the width
    sd = O.synthetic_state_dict(d, **sdkw)
    g = torch.Generator().manual_seed(seed)
    T = rnd.choice([1, 2, 3, 5, 9, 20, 33])
    ids = torch.randint(0, d.vocab_size, (T,), generator=g)
    for fused in (1, 0):
        m = make_model(d, sd, BF)
        o = O.OracleModel(d, sd, BF)
        m.decoder.allocate_flash_kv_cache(1, m.device, BF)
        if bool(m._native.fused(fused)) != bool(fused):
            continue  # the one-launch form does not take this architecture: the kernel sequence is checked below
        h_pre = m.decoder.forward_flash(m.token_emb(ids.cuda()[None]), torch.arange(T, device="cuda"))
        assert rel_err(h_pre[0], o.prefill(o.embed_text(ids))) <= TOL, (d, fused, "prompt pass")
        hid = torch.empty(1, d.d_model, dtype=BF, device="cuda")
        cb0 = torch.empty(1, d.codebook_size, dtype=BF, device="cuda")
        for i in range(8):
            codes = torch.randint(0, d.codebook_size, (1, d.n_quantizers), generator=g)
            h_ref, cb_ref, _ = o.decode_step(codes)
            m.decoder._step(codes=codes.cuda(), emb=None, slot_idx=None, seq_inc=None, B=1, hidden_out=hid, cb0_out=cb0,
                            eos_out=None, n_splits=4, stream=torch.cuda.current_stream().cuda_stream)
            assert rel_err(hid, h_ref) <= TOL and rel_err(cb0, cb_ref) <= TOL, (d, fused, i)
        hidden = O.rnd(torch.randn(1, d.d_model, generator=g), BF)
        c0 = torch.randint(0, d.codebook_size, (1,), generator=g)
        want, logits = o.rq_generate(hidden, c0, 1.0, 1, return_logits=True)
        got = m.rq_transformer.generate(hidden.to(BF).cuda(), c0.cuda(), temperature=1.0, top_k=1).cpu()
        for i in range(d.n_quantizers - 1):
            if got[0, i + 1] != want[0, i + 1]:
                top2 = torch.topk(logits[0, i], 2).values
                assert float(top2[0] - top2[1]) <= 2 * TOL * float(logits[0, i].abs().max()), (d, fused, "depth head", i)
                break  # later codebooks are conditioned on a different token
        m._native.status()


@pytest.mark.parametrize("seed", range(16))
def test_random_architecture_batch_vs_oracle(seed):
    """2..16 rows over shuffled cache slots with ragged lengths, bf16 or weight-only int8: four decode steps (hidden
    state, code-0 logits, positions) and the depth head of the batch against the oracle."""
    rnd = random.Random(1000 + seed)
    d = _dims(rnd)
    sdkw = dict(TINY_SD)
    sdkw["std"] = 0.15 * (64.0 / max(64, d.d_model)) ** 0.5
    sd = O.synthetic_state_dict(d, **sdkw)
    g = torch.Generator().manual_seed(seed)
    int8 = rnd.random() < 0.4
    B = rnd.choice([2, 3, 4, 5, 8, 9, 12, 16])
    n_slots = B + rnd.randint(0, 3)
    S = d.max_seqlen
    m = make_model(d, sd, BF, int8=int8)
    o = O.OracleModel(d, sd, BF, n_slots=n_slots, int8=int8)
    m.decoder.allocate_flash_kv_cache(n_slots, m.device, BF)
    lens = torch.randint(0, S - 12, (n_slots,), generator=g)
    kc = O.rnd(0.5 * torch.randn(d.n_layers, n_slots, S, d.n_kv_heads, d.head_dim, generator=g), BF)
    vc = O.rnd(0.5 * torch.randn(d.n_layers, n_slots, S, d.n_kv_heads, d.head_dim, generator=g), BF)
    m.decoder._k.copy_(kc.to(BF))
    m.decoder._v.copy_(vc.to(BF))
    m.decoder.flash_kv_caches[0].seq_lens.copy_(lens.to(torch.int32))
    o.k_cache.copy_(kc)
    o.v_cache.copy_(vc)
    o.seq_lens.copy_(lens)
    slots = torch.randperm(n_slots, generator=g)[:B]
    hid = torch.empty(B, d.d_model, dtype=BF, device="cuda")
    cb0 = torch.empty(B, d.codebook_size, dtype=BF, device="cuda")
    for i in range(4):
        codes = torch.randint(0, d.codebook_size, (B, d.n_quantizers), generator=g)
        h_ref, cb_ref, _ = o.decode_step(codes, slots)
        m.decoder._step(codes=codes.cuda(), emb=None, slot_idx=slots.to(torch.int32).cuda(), seq_inc=None, B=B, hidden_out=hid,
                        cb0_out=cb0, eos_out=None, n_splits=rnd.choice([1, 2, 4, 8]), stream=torch.cuda.current_stream().cuda_stream)
        assert rel_err(hid, h_ref) <= TOL and rel_err(cb0, cb_ref) <= TOL, (d, B, int8, i)
        assert m.decoder.flash_kv_caches[0].seq_lens.cpu().tolist() == o.seq_lens.tolist()
    hidden = O.rnd(torch.randn(B, d.d_model, generator=g), BF)
    c0 = torch.randint(0, d.codebook_size, (B,), generator=g)
    want, logits = o.rq_generate(hidden, c0, 1.0, 1, return_logits=True)
    got = m.rq_transformer.generate(hidden.to(BF).cuda(), c0.cuda(), temperature=1.0, top_k=1).cpu()
    for b in range(B):
        for i in range(d.n_quantizers - 1):
            if got[b, i + 1] != want[b, i + 1]:
                top2 = torch.topk(logits[b, i], 2).values
                assert float(top2[0] - top2[1]) <= 2 * TOL * float(logits[b, i].abs().max()), (d, B, "depth head", b, i)
                break
    m._native.status()


def _dims64(rnd: random.Random) -> O.Dims:
    """Architectures the persistent batched backbone kernel takes: widths in multiples of 64 (heads x head_dim equal to
    d_model), a codebook in multiples of 16, rotated widths in fours; grouped KV heads, windows and global layers drawn."""
    hd = rnd.choice([16, 32, 64, 96, 128])
    H = rnd.choice([h for h in (2, 4, 6, 8, 12, 16) if (h * hd) % 64 == 0 and h * hd <= 1024])
    kv = rnd.choice([k for k in (1, 2, 3, 4, 6, 8, 16) if H % k == 0 and (k * hd) % 16 == 0])
    kw = dict(d_model=hd * H, n_layers=rnd.randint(1, 3), n_heads=H, n_kv_heads=kv, n_quantizers=rnd.choice([2, 4, 8, 16]),
              codebook_size=rnd.choice([16, 64, 256, 2048]), rq_d_model=64, rq_n_layers=1, rq_n_heads=2, vocab_size=50,
              max_seqlen=rnd.choice([96, 300]), intermediate_size=64 * rnd.randint(1, 12))
    if rnd.random() < 0.5:
        kw["rope_dim"] = rnd.choice([x for x in (4, 8, 16, 32) if x <= hd])
    if rnd.random() < 0.5:
        kw["window_size"] = rnd.choice([3, 17, 70])
        kw["global_every"] = rnd.choice([None, 2, 3])
        if rnd.random() < 0.5:
            kw["global_rope_dim"] = rnd.choice([x for x in (4, 8, 16) if x <= hd])
    return O.Dims(**kw)


@pytest.mark.parametrize("seed", range(12))
def test_persistent_batched_backbone_vs_oracle(seed):
    """The backbone step of 2..16 rows as one persistent kernel (row groups by cache length, key ranges dealt by
    length, the general instantiation with conditional steps): hidden state, code-0 logits, end-of-turn logit, cache
    rows and positions of three steps against the oracle, bf16 and int8 weights, shuffled slots, ragged caches; and
    within the tolerance of the kernel sequence on the same inputs."""
    rnd = random.Random(7000 + seed)
    d = _dims64(rnd)
    sdkw = dict(TINY_SD)
    sdkw["std"] = 0.15 * (64.0 / max(64, d.d_model)) ** 0.5
    sd = O.synthetic_state_dict(d, **sdkw)
    g = torch.Generator().manual_seed(seed)
    int8 = seed % 2 == 1
    B = [2, 3, 4, 5, 8, 9, 12, 13, 16, 16, 7, 2][seed]
    n_slots = B + rnd.randint(0, 2)
    S = d.max_seqlen
    lens = torch.randint(0, S - 8, (n_slots,), generator=g)
    lens[0] = 0  # an empty cache among them
    kc = O.rnd(0.5 * torch.randn(d.n_layers, n_slots, S, d.n_kv_heads, d.head_dim, generator=g), BF)
    vc = O.rnd(0.5 * torch.randn(d.n_layers, n_slots, S, d.n_kv_heads, d.head_dim, generator=g), BF)
    slots = torch.randperm(n_slots, generator=g)[:B]
    codes_all = torch.randint(0, d.codebook_size, (3, B, d.n_quantizers), generator=g)
    o = O.OracleModel(d, sd, BF, n_slots=n_slots, int8=int8)
    o.k_cache.copy_(kc)
    o.v_cache.copy_(vc)
    o.seq_lens.copy_(lens)
    refs = [o.decode_step(codes_all[i], slots) for i in range(3)]
    outs = {}
    for fused in (1, 0):
        m = make_model(d, sd, BF, int8=int8)
        m.decoder.allocate_flash_kv_cache(n_slots, m.device, BF)
        m._native.fused(fused)
        if fused:
            assert m._native.bb_batch(), (d, "the persistent batched backbone kernel must take this architecture")
        m.decoder._k.copy_(kc.to(BF))
        m.decoder._v.copy_(vc.to(BF))
        m.decoder.flash_kv_caches[0].seq_lens.copy_(lens.to(torch.int32))
        hid = torch.empty(B, d.d_model, dtype=BF, device="cuda")
        cb0 = torch.empty(B, d.codebook_size, dtype=BF, device="cuda")
        eos = torch.empty(B, 1, dtype=BF, device="cuda")
        for i in range(3):
            m.decoder._step(codes=codes_all[i].cuda(), emb=None, slot_idx=slots.to(torch.int32).cuda(), seq_inc=None, B=B,
                            hidden_out=hid, cb0_out=cb0, eos_out=eos, n_splits=4, stream=torch.cuda.current_stream().cuda_stream)
            h_ref, cb_ref, eos_ref = refs[i]
            assert rel_err(hid, h_ref) <= TOL and rel_err(cb0, cb_ref) <= TOL, (d, B, int8, fused, i, rel_err(hid, h_ref), rel_err(cb0, cb_ref))
            assert float((eos.float().cpu() - eos_ref).abs().max()) <= TOL * max(1.0, float(cb_ref.abs().max())), (d, B, fused, i)
            outs[(fused, i)] = (hid.clone(), cb0.clone())
        m._native.status()
        assert m.decoder.flash_kv_caches[0].seq_lens.cpu().tolist() == o.seq_lens.tolist()
        # the three appended positions of every row, layer 0 and the last layer
        for b in range(B):
            s = int(slots[b])
            for l in (0, d.n_layers - 1):
                got = m.decoder._k[l, s, int(lens[s]):int(lens[s]) + 3].float().cpu()
                assert rel_err(got, o.k_cache[l, s, int(lens[s]):int(lens[s]) + 3]) <= TOL, (d, b, l)
                got = m.decoder._v[l, s, int(lens[s]):int(lens[s]) + 3].float().cpu()
                assert rel_err(got, o.v_cache[l, s, int(lens[s]):int(lens[s]) + 3]) <= TOL, (d, b, l)
    for i in range(3):
        assert rel_err(outs[(1, i)][0], outs[(0, i)][0]) <= TOL and rel_err(outs[(1, i)][1], outs[(0, i)][1]) <= TOL
