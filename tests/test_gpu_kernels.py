"""Single-kernel parity through the C ABI against the CPU oracle (needs an MI355X)."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import vui_oracle as O

pytestmark = pytest.mark.gpu

BF, F32 = torch.bfloat16, torch.float32


@pytest.fixture(scope="module")
def lib():
    from vui_amd import _lib

    return _lib.load()


def stream():
    return torch.cuda.current_stream().cuda_stream


def dcode(dt):
    return 1 if dt == F32 else 0


@pytest.mark.parametrize("dt", [F32, BF])
@pytest.mark.parametrize("B,N,K,norm", [(1, 2304, 768, True), (1, 768, 2048, False), (3, 50, 64, True),
                                        (16, 2048, 768, True), (16, 768, 2048, False), (5, 1408, 512, True),
                                        (2, 512, 1408, False), (1, 6, 4096, True)])
def test_rmsnorm_gemv(lib, dt, B, N, K, norm):
    from vui_amd import _lib

    g = torch.Generator().manual_seed(B * 1000 + N + K)
    x = O.rnd(torch.randn(B, K, generator=g) * 2, dt)
    W = O.rnd(torch.randn(N, K, generator=g) / K ** 0.5, dt)
    nw = O.rnd(1 + 0.2 * torch.randn(K, generator=g), dt) if norm else None
    ref = O.linear(O.rmsnorm(x, nw, 1e-5, dt) if norm else x, W, dt)
    xd, Wd = x.to(dt).cuda(), W.to(dt).cuda()
    nwd = nw.to(dt).cuda() if norm else None
    y = torch.empty(B, N, dtype=dt, device="cuda")
    _lib.check(lib.vui_rmsnorm_gemv(dcode(dt), xd.data_ptr(), _lib.ptr(nwd), 1e-5, Wd.data_ptr(), None, 0,
                                    y.data_ptr(), B, N, K, stream()), "gemv")
    got = y.float().cpu()
    if dt == F32:
        np.testing.assert_allclose(got.numpy(), ref.numpy(), rtol=2e-5, atol=2e-5)
    else:
        # both sides round an fp32 sum to bf16; sums differ by order -> at most one bf16 ulp on a few entries
        ulp = (ref.abs() * 2.0 ** -7).clamp_min(2e-5 * float(ref.abs().max()))
        assert ((got - ref).abs() <= ulp).all()
        assert (got != ref).float().mean() < 0.05


@pytest.mark.parametrize("B,N,K", [(1, 2304, 768), (16, 768, 2048), (4, 2048, 768),
                                   (3, 288, 288), (16, 56, 272), (2, 480, 352), (16, 16, 144), (5, 32, 56)])
def test_gemv_int8(lib, B, N, K):
    """Weight-only int8 against dequantise-then-matmul in fp32 on the same int8 weights.  The small shapes have a K that
    is no multiple of 64: on the matrix-core form the last K step is then partly beyond the row (lanes with zero
    weights), and K = 56 takes the one-wave-per-row-pair form."""
    from vui_amd import _lib
    from vui_amd.model import quantize_int8

    g = torch.Generator().manual_seed(N + K + B)
    x = O.rnd(torch.randn(B, K, generator=g), BF)
    W = torch.randn(N, K, generator=g) * 0.02
    q_o, s_o = O.quantize_int8(W)
    q, s = quantize_int8(W)
    assert torch.equal(q, q_o) and torch.equal(s.float(), s_o)
    ref = O.linear_int8(x, q_o, s_o, BF)
    y = torch.empty(B, N, dtype=BF, device="cuda")
    qd, sd_, xd = q.cuda(), s.cuda(), x.to(BF).cuda()
    _lib.check(lib.vui_rmsnorm_gemv(0, xd.data_ptr(), None, 0.0, qd.data_ptr(), sd_.data_ptr(), 1, y.data_ptr(),
                                    B, N, K, stream()), "gemv int8")
    got = y.float().cpu()
    ulp = (ref.abs() * 2.0 ** -7).clamp_min(2e-5 * float(ref.abs().max()))
    assert ((got - ref).abs() <= ulp).all()
    # and the quantisation itself is close to the unquantised product (sanity, not parity)
    full = O.linear(x, W, F32)
    assert (got - full).abs().max() <= 0.02 * full.abs().max()


@pytest.mark.parametrize("dt", [F32, BF])
@pytest.mark.parametrize("hd,rope_dim", [(96, 96), (16, 8)])
def test_rope(lib, dt, hd, rope_dim):
    from vui_amd import _lib

    g = torch.Generator().manual_seed(hd)
    B, nh, S = 5, 3, 64
    table = O.precompute_freqs_cis(rope_dim, S, 10000.0, 1.0)
    pos = torch.tensor([0, 1, 7, 33, 63], dtype=torch.int32)
    x = O.rnd(torch.randn(B, nh, hd, generator=g), dt)
    ref = O.apply_rotary_emb(table[pos.long()][:, None], x, dt)
    xd, td, pd = x.to(dt).cuda(), table.cuda(), pos.cuda()  # keep the device copies alive past the launch
    _lib.check(lib.vui_rope(dcode(dt), xd.data_ptr(), td.data_ptr(), pd.data_ptr(), B, nh, hd,
                            rope_dim, stream()), "rope")
    np.testing.assert_array_equal(xd.float().cpu().numpy(), ref.numpy())
    # position 0 is the identity; each pair keeps its norm
    np.testing.assert_array_equal(xd[0].float().cpu().numpy(), x[0].numpy())


@pytest.mark.parametrize("dt", [F32, BF])
@pytest.mark.parametrize("H,KV,hd,S,lens,splits,window", [
    (8, 8, 96, 4608, [255, 1023, 4095], 32, 0),
    (8, 8, 96, 2304, [127, 2047, 600, 1, 0, 999], 4, 0),
    (4, 2, 16, 64, [0, 5, 63], 3, 0),
    (4, 2, 16, 64, [40, 5, 63], 2, 7),
    (8, 8, 96, 512, [300], 1, 0),
    # many rows, many pieces, short and empty pieces
    (8, 8, 96, 2304, [127, 2047, 600, 1, 0, 999, 1500, 64], 32, 0),
    (4, 4, 16, 256, [0, 5, 63, 255, 100, 31, 32, 33], 32, 0),
    (2, 2, 32, 256, [200, 5, 63, 255, 100, 31, 32, 33], 64, 50),
])
def test_decode_attn(lib, dt, H, KV, hd, S, lens, splits, window):
    """Append + attention over ragged lengths with slot indirection, against the textbook softmax."""
    from vui_amd import _lib

    B = len(lens)
    n_slots = B + 2
    g = torch.Generator().manual_seed(S + hd + B)
    slot_idx = torch.randperm(n_slots, generator=g)[:B].to(torch.int32)
    kc = O.rnd(torch.randn(n_slots, S, KV, hd, generator=g), dt)
    vc = O.rnd(torch.randn(n_slots, S, KV, hd, generator=g), dt)
    q = O.rnd(torch.randn(B, H, hd, generator=g), dt)
    kn = O.rnd(torch.randn(B, KV, hd, generator=g), dt)
    vn = O.rnd(torch.randn(B, KV, hd, generator=g), dt)
    seq_lens = torch.zeros(n_slots, dtype=torch.int32)
    for b, L in enumerate(lens):
        seq_lens[slot_idx[b]] = L
    ref = torch.zeros(B, H, hd)
    for b, L in enumerate(lens):
        s = int(slot_idx[b])
        kk = torch.cat([kc[s, :L], kn[b][None]], 0).transpose(0, 1)  # (KV, L+1, hd)
        vv = torch.cat([vc[s, :L], vn[b][None]], 0).transpose(0, 1)
        if window > 0:
            lo = max(0, L - window)
            kk, vv = kk[:, lo:], vv[:, lo:]
        kk = kk.repeat_interleave(H // KV, 0)
        vv = vv.repeat_interleave(H // KV, 0)
        ref[b] = O.attention(q[b][:, None], kk, vv, hd ** -0.5, dt)[:, 0]
    kcd, vcd = kc.to(dt).cuda(), vc.to(dt).cuda()
    out = torch.empty(B, H, hd, dtype=dt, device="cuda")
    scratch = torch.zeros(lib.vui_attn_scratch_bytes(B, H, hd, splits), dtype=torch.uint8, device="cuda")
    sl, qd, knd, vnd, sid = seq_lens.cuda(), q.to(dt).cuda(), kn.to(dt).cuda(), vn.to(dt).cuda(), slot_idx.cuda()
    for rep in range(2):  # twice: the merge counters must come back to zero
        out.zero_()
        _lib.check(lib.vui_decode_attn(dcode(dt), qd.data_ptr(), knd.data_ptr(), vnd.data_ptr(), kcd.data_ptr(),
                                       vcd.data_ptr(), sl.data_ptr(), sid.data_ptr(), out.data_ptr(), B, H, KV, hd,
                                       S, window, splits, scratch.data_ptr(), stream()), "attn")
        got = out.float().cpu()
        tol = 2e-5 if dt == F32 else 2.0 ** -7
        assert (got - ref).abs().max() <= tol * max(1.0, float(ref.abs().max())), rep
    # the new rows landed at seq_lens[slot]
    for b, L in enumerate(lens):
        s = int(slot_idx[b])
        np.testing.assert_array_equal(kcd[s, L].float().cpu().numpy(), kn[b].numpy())
        np.testing.assert_array_equal(vcd[s, L].float().cpu().numpy(), vn[b].numpy())


def _sample(lib, logits, bias, temperature, top_k, seed, frame, codebook):
    from vui_amd import _lib

    B, CS = logits.shape
    sp = _lib.SampleParamsC()
    sp.temperature, sp.top_k, sp.seed = temperature, top_k, seed
    ctr = torch.tensor([frame], dtype=torch.int32, device="cuda")
    sp.frame_ctr = ctr.data_ptr()
    out = torch.empty(B, dtype=torch.long, device="cuda")
    ld = logits.cuda()
    bd = bias.cuda() if bias is not None else None
    _lib.check(lib.vui_sample_logits(ld.data_ptr(), _lib.ptr(bd), CS, C.byref(sp), codebook, out.data_ptr(), B,
                                     stream()), "sample")
    return out.cpu()


def test_sampler_greedy_and_ties(lib):
    g = torch.Generator().manual_seed(0)
    lg = torch.randn(16, 2048, generator=g)
    lg[3, 100] = lg[3, 900] = lg[3].max() + 1  # tie: lowest index wins
    got = _sample(lib, lg, None, 0.8, 1, 0, 0, 1)
    assert torch.equal(got, lg.argmax(-1))
    assert got[3] == 100
    got = _sample(lib, lg, None, 0.0, 50, 0, 0, 1)  # temperature <= 0 is greedy too
    assert torch.equal(got, lg.argmax(-1))


@pytest.mark.parametrize("CS,top_k", [(2048, 50), (2048, 0), (32, 5), (4096, 100), (100, 100)])
def test_sampler_matches_oracle_draws(lib, CS, top_k):
    """Same logits, same (seed, frame, row, codebook): the device pick equals the oracle's
    inverse-CDF pick except where the uniform falls within rounding of a CDF step."""
    g = torch.Generator().manual_seed(CS + top_k)
    B = 16
    lg = torch.randn(B, CS, generator=g) * 3
    bias = torch.randn(CS, generator=g)
    n_match = n = 0
    for frame in range(40):
        got = _sample(lib, lg, bias, 0.8, top_k, 1234, frame, 3)
        for b in range(B):
            exp = O.sample_rq(lg[b] + bias, 0.8, top_k, O.uniform01(1234, frame, b, 3))
            n_match += int(got[b] == exp)
            n += 1
            kept = O.topk_threshold_probs(lg[b] + bias, 0.8, top_k)
            assert kept[int(got[b])] > 0  # never outside the kept set
    assert n_match >= 0.995 * n, (n_match, n)


def _sample_cb0_rows(lib, logits_bf, temperature, top_k, top_p, seed, frame):
    """vui_sample_cb0 over bf16 rows with the ties-kept rule (what inference.stream_frames calls)."""
    from vui_amd import _lib

    B, CS = logits_bf.shape
    cfgc = _lib.VuiConfigC()
    cfgc.dtype, cfgc.d_model, cfgc.n_layers, cfgc.n_heads, cfgc.n_kv_heads, cfgc.head_dim, cfgc.ffn = 0, 64, 1, 4, 4, 16, 64
    cfgc.n_quantizers, cfgc.codebook_size, cfgc.rq_dim, cfgc.rq_layers, cfgc.rq_heads, cfgc.rq_ffn = 4, CS, 64, 0, 1, 8
    cfgc.rope_dim, cfgc.max_seqlen, cfgc.n_slots, cfgc.norm_eps, cfgc.rq_norm_eps = 16, 16, 1, 1e-5, 1e-6
    n = lib.vui_workspace_bytes(C.byref(cfgc), 16)
    assert n > 0, _lib.last_error()
    ws = torch.zeros(n + 256, dtype=torch.uint8, device="cuda")
    dummy = torch.zeros(64, dtype=torch.float32, device="cuda")
    w = _lib.WeightsC()
    for f in ("audio_emb", "final_norm", "codec_head", "eos_w", "eos_b", "rope_table"):
        setattr(w, f, dummy.data_ptr())
    for f in ("attn_norm", "wqkv", "wo", "mlp_norm", "w1", "w3", "w2"):
        setattr(w.layers[0], f, dummy.data_ptr())
    h = C.c_void_p()
    _lib.check(lib.vui_ctx_create(C.byref(cfgc), C.byref(w), (ws.data_ptr() + 255) & ~255, n, 16, C.byref(h)), "ctx")
    ctr = torch.tensor([frame], dtype=torch.int32, device="cuda")
    sp = _lib.SampleParamsC()
    sp.temperature, sp.top_k, sp.seed, sp.frame_ctr, sp.keep_ties, sp.top_p = temperature, top_k, seed, ctr.data_ptr(), 1, top_p
    out = torch.empty(B, dtype=torch.long, device="cuda")
    ld = logits_bf.cuda()
    _lib.check(lib.vui_sample_cb0(h, ld.data_ptr(), None, None, None, 1.0, 0, C.byref(sp), out.data_ptr(), B, stream()), "cb0")
    torch.cuda.synchronize()
    lib.vui_ctx_destroy(h)
    return out.cpu()


@pytest.mark.parametrize("CS,top_k,top_p", [(2048, 0, 0.9), (2048, 50, 0.8), (2048, 100, 0.3), (32, 0, 0.5), (32, 5, 0.7),
                                            (4096, 0, 0.95), (100, 10, 1.0), (2048, 0, 0.05)])
def test_sampler_nucleus_matches_oracle_draws(lib, CS, top_k, top_p):
    """The nucleus cut of sampling.sample_top_p / sample_top_p_top_k on the device: fp32 logits through
    vui_sample_logits (32-bit keys) and bf16 logits through vui_sample_cb0 (16-bit keys) give the oracle's pick on
    the same uniform except where it falls within rounding of a CDF step or the budget within rounding of a
    boundary; no pick lies outside a kept set widened by the boundary's own neighbours."""
    from vui_amd import _lib

    g = torch.Generator().manual_seed(CS * 3 + top_k + int(top_p * 100))
    B = 16
    lg = torch.randn(B, CS, generator=g) * 3
    lg[5, : CS // 4] = lg[5, 0]  # a row whose boundary falls into a run of equal values
    k_or = top_k if top_k > 0 else None
    n_match = n = 0
    for frame in range(12):
        sp = _lib.SampleParamsC()
        ctr = torch.tensor([frame], dtype=torch.int32, device="cuda")
        sp.temperature, sp.top_k, sp.seed, sp.frame_ctr, sp.top_p = 0.8, top_k, 4321, ctr.data_ptr(), top_p
        out = torch.empty(B, dtype=torch.long, device="cuda")
        ld = lg.cuda()
        _lib.check(lib.vui_sample_logits(ld.data_ptr(), None, CS, C.byref(sp), 2, out.data_ptr(), B, stream()), "sample")
        got32 = out.cpu()
        lgb = lg.to(BF)
        got16 = _sample_cb0_rows(lib, lgb, 0.8, top_k, top_p, 4321, frame)
        for b in range(B):
            for got, src, cb in ((got32, lg[b], 2), (got16, lgb[b].float(), 0)):
                u = O.uniform01(4321, frame, b, cb)
                kept = O.sample_codes_probs(src, 0.8, k_or, top_p)
                exp = O._inverse_cdf(kept, u)
                n_match += int(got[b] == exp)
                n += 1
                # the pick is a kept entry, or (budget within rounding of a boundary) no smaller than the smallest kept one
                pr = torch.softmax(src / 0.8, -1).numpy()
                assert kept[int(got[b])] > 0 or pr[int(got[b])] >= pr[kept > 0].min() * (1 - 1e-5), (b, int(got[b]))
    assert n_match >= 0.99 * n, (n_match, n)


def test_sampler_nucleus_keeps_lowest_indices_of_a_tie(lib):
    """Eight equal logits, temperature 1: probabilities of 1/8 each.  top_p = 0.3 keeps the entries with 0, 1/8 and
    2/8 ahead of them - the three lowest indices - whatever the uniform."""
    from vui_amd import _lib

    lg = torch.full((16, 8), 0.5)
    seen = set()
    for frame in range(30):
        sp = _lib.SampleParamsC()
        ctr = torch.tensor([frame], dtype=torch.int32, device="cuda")
        sp.temperature, sp.top_k, sp.seed, sp.frame_ctr, sp.top_p = 1.0, 0, 9, ctr.data_ptr(), 0.3
        out = torch.empty(16, dtype=torch.long, device="cuda")
        ld = lg.cuda()
        _lib.check(lib.vui_sample_logits(ld.data_ptr(), None, 8, C.byref(sp), 1, out.data_ptr(), 16, stream()), "sample")
        seen |= set(out.cpu().tolist())
    assert seen == {0, 1, 2}
    assert set(np.nonzero(O.sample_codes_probs(lg[0], 1.0, None, 0.3))[0]) == {0, 1, 2}


def test_sampler_histogram(lib):
    """Chi-square of 20000 device draws against the analytic top-k softmax (benchmark configuration 3's
    distribution-level check)."""
    g = torch.Generator().manual_seed(5)
    CS, k = 2048, 50
    row = torch.randn(CS, generator=g) * 2
    lg = row.repeat(16, 1)
    hist = np.zeros(CS)
    for frame in range(1250):
        got = _sample(lib, lg, None, 0.8, k, 7, frame, 2)
        for c in got.tolist():
            hist[c] += 1
    w = O.topk_threshold_probs(row, 0.8, k)
    assert set(np.nonzero(hist)[0]) <= set(np.nonzero(w)[0])
    exp = w / w.sum() * hist.sum()
    keep = exp > 5
    chi2 = (((hist - exp) ** 2)[keep] / exp[keep]).sum()
    dof = keep.sum() - 1
    assert chi2 < dof + 5 * (2 * dof) ** 0.5, (chi2, dof)


@pytest.mark.parametrize("CS,top_k", [(2048, 100), (2048, 1000), (32, 5), (1000, 37)])
def test_sampler_16bit_key_search_equals_32bit(lib, CS, top_k):
    """bf16 logits take the two-round 8-bit histogram search for the k-th largest key; with a
    repetition state attached (all counts zero, so values are unchanged) the same logits take the
    generic 32-bit search.  Same (seed, frame) -> same picks, and the picks lie in the oracle's kept set."""
    from vui_amd import _lib

    B = 16
    g = torch.Generator().manual_seed(CS * 7 + top_k)
    lg = (torch.randn(B, CS, generator=g) * 2).to(BF)
    lg[2, :CS // 2] = lg[2, 0]  # heavy ties around the cut
    cfgc = _lib.VuiConfigC()
    cfgc.dtype, cfgc.d_model, cfgc.n_layers, cfgc.n_heads, cfgc.n_kv_heads, cfgc.head_dim, cfgc.ffn = 0, 64, 1, 4, 4, 16, 64
    cfgc.n_quantizers, cfgc.codebook_size, cfgc.rq_dim, cfgc.rq_layers, cfgc.rq_heads, cfgc.rq_ffn = 4, CS, 64, 0, 1, 8
    cfgc.rope_dim, cfgc.max_seqlen, cfgc.n_slots, cfgc.norm_eps, cfgc.rq_norm_eps = 16, 16, 1, 1e-5, 1e-6
    n = lib.vui_workspace_bytes(C.byref(cfgc), 16)
    assert n > 0, _lib.last_error()
    ws = torch.zeros(n + 256, dtype=torch.uint8, device="cuda")
    dummy = torch.zeros(64, dtype=torch.float32, device="cuda")
    w = _lib.WeightsC()
    for f in ("audio_emb", "final_norm", "codec_head", "eos_w", "eos_b", "rope_table"):
        setattr(w, f, dummy.data_ptr())
    for f in ("attn_norm", "wqkv", "wo", "mlp_norm", "w1", "w3", "w2"):
        setattr(w.layers[0], f, dummy.data_ptr())
    h = C.c_void_p()
    _lib.check(lib.vui_ctx_create(C.byref(cfgc), C.byref(w), (ws.data_ptr() + 255) & ~255, n, 16, C.byref(h)), "ctx")
    ld = lg.cuda()
    counts = torch.zeros(B, CS, dtype=torch.float32, device="cuda")
    n_match = n_all = 0
    for frame in range(20):
        ctr = torch.tensor([frame], dtype=torch.int32, device="cuda")
        sp = _lib.SampleParamsC()
        sp.temperature, sp.top_k, sp.seed, sp.frame_ctr = 0.9, top_k, 99, ctr.data_ptr()
        a = torch.empty(B, dtype=torch.long, device="cuda")
        b = torch.empty(B, dtype=torch.long, device="cuda")
        _lib.check(lib.vui_sample_cb0(h, ld.data_ptr(), None, None, None, 1.0, 0, C.byref(sp), a.data_ptr(), B, stream()), "a")
        counts.zero_()
        _lib.check(lib.vui_sample_cb0(h, ld.data_ptr(), counts.data_ptr(), None, None, 1.0001, 0, C.byref(sp), b.data_ptr(), B,
                                      stream()), "b")
        assert torch.equal(a, b), frame
        for r in range(B):
            # the code-0 rule keeps exactly top_k entries: of row 2's ties only the lowest indices survive
            kept = O.cb0_probs(lg[r].float(), 0.9, top_k)
            assert (kept > 0).sum() == min(top_k, CS)
            assert kept[int(a[r])] > 0
            n_match += int(a[r]) == O.sample_cb0(lg[r].float(), torch.zeros(CS), 1.0, 0.9, top_k, O.uniform01(99, frame, r, 0))
            n_all += 1
    assert n_match >= 0.99 * n_all, (n_match, n_all)
    lib.vui_ctx_destroy(h)
