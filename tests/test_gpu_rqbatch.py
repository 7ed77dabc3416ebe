"""The depth head of a batch as one persistent kernel against the oracle and against the kernel sequence.
Reference: RQTransformer._generate_graph_body_kv / generate_cuda_graph_kv (src/vui/model.py:908-1016)."""
import pytest
import torch

from oracle import vui_oracle as O
from tests.util import TINY_SD, make_model

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
BF16_TOL = 2.0 ** -5


def _check_greedy(got, ref, logits, d):
    """Tokens equal the oracle's wherever its top-2 logit margin exceeds the bf16 tolerance."""
    n_exact = 0
    for b in range(got.shape[0]):
        assert int(got[b, 0]) == int(ref[b, 0])
        for i in range(d.n_quantizers - 1):
            if got[b, i + 1] != ref[b, i + 1]:
                top2 = torch.topk(logits[b, i], 2).values
                assert float(top2[0] - top2[1]) <= 2 * BF16_TOL * float(logits[b, i].abs().max()), (b, i)
                break  # later codebooks are conditioned on a different token
        else:
            n_exact += 1
    return n_exact


def _small_dims():
    # depth head 64-d x 2 layers, 4 heads of 16; every vector length a multiple of 32
    return O.Dims(d_model=128, n_layers=1, n_heads=4, n_kv_heads=4, n_quantizers=6, codebook_size=64, rq_d_model=64,
                  rq_n_layers=2, rq_n_heads=4, vocab_size=50, max_seqlen=64)


def _wide_dims():
    # a 640-d depth head: 80 chunks of 8 (a lane of the fused wait + norm holds a second, partly filled chunk) and
    # 40 out_proj / W2 tiles (more than half of a row group's workgroups: every tile takes all rows)
    return O.Dims(d_model=128, n_layers=1, n_heads=4, n_kv_heads=4, n_quantizers=5, codebook_size=64, rq_d_model=640,
                  rq_n_layers=2, rq_n_heads=8, vocab_size=50, max_seqlen=64)


def _preset_b_dims():
    # the 768-wide, 5-layer depth head: 144 QKV tiles, so the first 16 workgroups of a row group take a third one
    return O.Dims(d_model=128, n_layers=1, n_heads=4, n_kv_heads=4, n_quantizers=16, codebook_size=2048, rq_d_model=768,
                  rq_n_layers=5, rq_n_heads=8, vocab_size=50, max_seqlen=64)


@pytest.mark.parametrize("dims", ["small", "wide", "preset_b", "nano"])
def test_batched_depth_head_vs_oracle_and_sequence(dims):
    if dims in ("small", "wide", "preset_b"):
        d = {"small": _small_dims, "wide": _wide_dims, "preset_b": _preset_b_dims}[dims]()
        sdkw = dict(TINY_SD)
        if dims == "preset_b":
            sdkw["std"] = 0.04  # keeps the logits of a 768-wide head in the range the tiny ones have
        sd = O.synthetic_state_dict(d, **sdkw)
    else:
        d = O.Dims()
        sd = O.synthetic_state_dict(d, seed=0)
    m = make_model(d, sd, BF, max_seqlen=64)
    o = O.OracleModel(d, sd, BF, max_seqlen=64)
    g = torch.Generator().manual_seed(21)
    B = 16
    hidden = O.rnd(torch.randn(B, d.d_model, generator=g), BF)
    code0 = torch.randint(0, d.codebook_size, (B,), generator=g)
    ref, logits = o.rq_generate(hidden, code0, 1.0, 1, return_logits=True)
    hd_, c0_ = hidden.to(BF).cuda(), code0.cuda()
    rq = m.rq_transformer
    m._native.fused(1)
    assert m._native.rq_batch(), "the batched depth-head kernel must be available on an MI355X"
    for nb in (16, 5, 2):
        got = rq.generate(hd_[:nb], c0_[:nb], temperature=1.0, top_k=1).cpu()
        m._native.status()
        assert got.shape == (nb, d.n_quantizers)
        exact = _check_greedy(got, ref[:nb], logits[:nb], d)
        assert exact >= nb // 2  # most rows have no near-tie at all
        if nb == 16:
            full = got
        else:
            assert torch.equal(got, full[:nb])  # a row's result does not depend on the batch around it
    # the kernel sequence on the same inputs
    m._native.fused(0)
    assert not m._native.rq_batch()
    seq = rq.generate(hd_, c0_, temperature=1.0, top_k=1).cpu()
    _check_greedy(seq, ref, logits, d)
    m._native.fused(1)
    # fewer codebooks through the captured-graph entry point (a view of the static output buffer)
    nq = d.n_quantizers - 2
    rq.setup_cuda_graph_kv(m.device, BF, top_k=1, batch_sizes=(3,))
    out = rq.generate_cuda_graph_kv(hd_[:3], c0_[:3], 1.0, n_quantizers=nq).cpu()
    m._native.status()
    assert out.shape == (3, nq) and torch.equal(out, full[:3, :nq])


def test_batched_depth_head_sampling_is_per_row_deterministic():
    d = O.Dims()
    sd = O.synthetic_state_dict(d, seed=0)
    m = make_model(d, sd, BF, max_seqlen=64)
    g = torch.Generator().manual_seed(4)
    hidden = torch.randn(16, d.d_model, generator=g).to(BF).cuda()
    code0 = torch.randint(0, d.codebook_size, (16,), generator=g).cuda()
    rq = m.rq_transformer
    rq.seed = 7
    res = []
    for n in (16, 16, 6):
        rq._ctr.zero_()  # the draw counter advances per call: same counter, same draws
        res.append(rq.generate(hidden[:n], code0[:n], temperature=0.8, top_k=50).cpu())
    a, b, c = res
    m._native.status()
    assert torch.equal(a, b) and torch.equal(a[:6], c)
    assert int(a.min()) >= 0 and int(a.max()) < d.codebook_size
    # sixteen different rows do not all draw the same thing
    assert len({tuple(r.tolist()) for r in a}) > 8
