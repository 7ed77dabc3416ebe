"""The CPU oracle against golden vectors written from the reference's own classes
(tests/golden/make_golden.py).  No GPU needed."""
import os

import numpy as np
import pytest
import torch

from oracle import vui_oracle as O
from tests.conftest import GOLDEN

TINY_SD = dict(seed=7, std=0.15, norm_jitter=0.1, bias_std=0.1)


def tiny_dims(kv):
    return O.Dims(d_model=64, n_layers=2, n_heads=4, n_kv_heads=kv, n_quantizers=4, codebook_size=32,
                  rq_d_model=48, rq_n_layers=2, rq_n_heads=4, vocab_size=50, max_seqlen=32)


def load(name):
    return np.load(os.path.join(GOLDEN, name))


def T(a):
    return torch.from_numpy(np.asarray(a))


def test_freqs_table():
    g = load("rope.npz")
    np.testing.assert_array_equal(O.precompute_freqs_cis(96, 40).numpy(), g["plain"])
    np.testing.assert_allclose(O.precompute_freqs_cis(8, 24, 500.0, 1.7).numpy(), g["rescaled"], rtol=0, atol=1e-6)


def test_apply_rotary():
    g = load("rope.npz")
    pos = T(g["pos"])
    t = T(g["t"])
    full = O.precompute_freqs_cis(16, 24)[pos]
    part = O.precompute_freqs_cis(8, 24, 500.0, 1.7)[pos]
    np.testing.assert_allclose(O.apply_rotary_emb(full, t, torch.float32).numpy(), g["rot_full"], rtol=0, atol=1e-6)
    np.testing.assert_allclose(O.apply_rotary_emb(part, t, torch.float32).numpy(), g["rot_part"], rtol=0, atol=1e-6)
    t3 = T(g["t3"])
    np.testing.assert_allclose(O.apply_rotary_emb(full[:, None], t3, torch.float32).numpy(), g["rot3"], rtol=0, atol=1e-6)
    got = O.apply_rotary_emb(full[:, None], O.rnd(t3, torch.bfloat16), torch.bfloat16).numpy()
    np.testing.assert_array_equal(got, g["rot3_bf16"])


def test_rmsnorm_and_embedding():
    g = load("pieces.npz")
    y = O.rmsnorm(T(g["norm_x"]), T(g["norm_w"]), 1e-5, torch.float32)
    np.testing.assert_allclose(y.numpy(), g["norm_y"], rtol=1e-6, atol=1e-6)
    yb = O.rmsnorm(O.rnd(T(g["norm_x"]), torch.bfloat16), O.rnd(T(g["norm_w"]), torch.bfloat16), 1e-5, torch.bfloat16)
    np.testing.assert_array_equal(yb.numpy(), g["norm_y_bf16"])
    tab, codes = T(g["ae_table"]), T(g["ae_codes"])
    np.testing.assert_allclose(O.audio_embedding(tab, codes, 8, torch.float32).numpy(), g["ae_full"], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(O.audio_embedding(tab, codes[:, :2], 8, torch.float32).numpy(), g["ae_q2"], rtol=1e-6, atol=1e-6)


def test_top_k_kept_set_matches_reference_histogram():
    g = load("pieces.npz")
    p = T(g["tk_probs"])
    k = int(g["tk_k"])
    hist = g["tk_hist"].astype(np.float64)
    kept = O.cb0_probs(torch.log(p), 1.0, k)  # softmax(log p) == p
    assert set(np.nonzero(kept)[0]) == set(np.nonzero(hist)[0])  # ties at the k-th place are kept
    exp = kept / kept.sum() * hist.sum()
    chi2 = (((hist - exp) ** 2)[exp > 0] / exp[exp > 0]).sum()
    assert chi2 < 30, chi2  # 4 dof


@pytest.mark.parametrize("kv,name", [(4, "tiny_backbone_mha.npz"), (2, "tiny_backbone_gqa.npz")])
def test_tiny_backbone(kv, name):
    g = load(name)
    d = tiny_dims(kv)
    m = O.OracleModel(d, O.synthetic_state_dict(d, **TINY_SD), torch.float32)
    ids, codes = T(g["ids"]), T(g["codes"])
    h_pre = m.prefill(m.embed_text(ids))
    np.testing.assert_allclose(h_pre.numpy(), g["h_prefill"], rtol=2e-5, atol=2e-5)
    for i in range(codes.shape[0]):
        h, cb0, eos = m.decode_step(codes[i][None])
        np.testing.assert_allclose(h[0].numpy(), g["hidden"][i], rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(cb0[0].numpy(), g["cb0"][i], rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(eos[0].numpy(), g["eos"][i], rtol=2e-5, atol=2e-5)
    assert int(m.seq_lens[0]) == 9
    # reference KVCache is (B, KV, S, hd); ours (slots, S, KV, hd)
    np.testing.assert_allclose(m.k_cache[0, 0, :9].transpose(0, 1).numpy(), g["k_layer0"], rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(m.v_cache[1, 0, :9].transpose(0, 1).numpy(), g["v_layer1"], rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_tiny_backbone_global_layers(name):
    """Which layers are global, their own rotation table (width and derived base) and which table rotates which
    layer, against the reference's Decoder (its CPU path applies no window, so neither does the oracle here)."""
    g = load(f"tiny_backbone_global_{name}.npz")
    d = tiny_dims(2)
    for k, v in zip(g["kw_keys"], g["kw_vals"]):
        setattr(d, str(k), float(v) if str(k) == "global_rope_theta" else int(v))
    assert d.block_is_global() == [bool(x) for x in g["is_global"]]
    m = O.OracleModel(d, O.synthetic_state_dict(d, **TINY_SD), torch.float32, apply_window=False)
    if "freqs_global" in g.files:
        np.testing.assert_allclose(m.freqs_global.numpy(), g["freqs_global"], rtol=1e-6, atol=1e-6)
    else:
        assert m.freqs_global is None
    ids, codes = T(g["ids"]), T(g["codes"])
    np.testing.assert_allclose(m.prefill(m.embed_text(ids)).numpy(), g["h_prefill"], rtol=2e-5, atol=2e-5)
    for i in range(codes.shape[0]):
        h, cb0, _ = m.decode_step(codes[i][None])
        np.testing.assert_allclose(h[0].numpy(), g["hidden"][i], rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(cb0[0].numpy(), g["cb0"][i], rtol=2e-5, atol=2e-5)
    # a plausible mistake must fail: the common table on the global layers gives other hidden states
    d2 = tiny_dims(2)
    d2.n_layers = d.n_layers
    m2 = O.OracleModel(d2, O.synthetic_state_dict(d, **TINY_SD), torch.float32)
    assert float((m2.prefill(m2.embed_text(ids)) - T(g["h_prefill"])).abs().max()) > 1e-3


def test_window_mask_of_local_layers():
    """flash-attn's window (w, 0) on the local layers only: a query at position i sees keys i-w .. i
    (MHA.forward_flash model.py:242-257).  One layer, window 3, against the textbook attention over the last 4 keys."""
    d = tiny_dims(2)
    d.n_layers, d.window_size = 1, 3
    sd = O.synthetic_state_dict(d, **TINY_SD)
    assert d.block_is_global() == [False]
    m = O.OracleModel(d, sd, torch.float32)
    d_full = tiny_dims(2)
    d_full.n_layers = 1
    full = O.OracleModel(d_full, sd, torch.float32)
    g_ = torch.Generator().manual_seed(1)
    emb = torch.randn(9, d.d_model, generator=g_) * 0.5
    a, b = m.prefill(emb), full.prefill(emb)
    assert torch.allclose(a[:4], b[:4], atol=1e-6)  # positions 0..3 see at most 4 keys either way
    assert float((a[4:] - b[4:]).abs().max()) > 1e-4  # from position 4 on the window cuts keys off
    # position 8 from scratch: keys 5..8 only
    H, KV, hd = d.n_heads, d.n_kv_heads, d.head_dim
    p = "decoder.blocks.0."
    x = emb[8:9]
    h = O.rmsnorm(x, sd[p + "attn_norm.weight"], d.norm_eps, torch.float32)
    q = O.linear(h, sd[p + "attn.Wqkv.weight"], torch.float32)[:, :H * hd].view(1, H, hd)
    q = O.apply_rotary_emb(m.freqs[8][None, None], q, torch.float32)
    kk = m.k_cache[0, 0, 5:9].transpose(0, 1).repeat_interleave(H // KV, 0)
    vv = m.v_cache[0, 0, 5:9].transpose(0, 1).repeat_interleave(H // KV, 0)
    att = O.attention(q.transpose(0, 1), kk, vv, hd ** -0.5, torch.float32).transpose(0, 1).reshape(1, H * hd)
    x1 = x + O.linear(att, sd[p + "attn.out_proj.weight"], torch.float32)
    h2 = O.rmsnorm(x1, sd[p + "mlp_norm.weight"], d.norm_eps, torch.float32)
    x2 = x1 + O.swiglu(h2, sd[p + "mlp.w1.weight"], sd[p + "mlp.w3.weight"], sd[p + "mlp.w2.weight"], torch.float32)
    want = O.rmsnorm(x2, sd["decoder.norm.weight"], d.norm_eps, torch.float32)
    assert torch.allclose(a[8:9], want, atol=2e-5)


def test_tiny_rq_forward_and_greedy():
    g = load("tiny_rq.npz")
    d = tiny_dims(4)
    m = O.OracleModel(d, O.synthetic_state_dict(d, **TINY_SD), torch.float32)
    hidden, codes = T(g["hidden"]), T(g["codes"])
    np.testing.assert_allclose(m.rq_forward(hidden, codes).numpy(), g["forward_logits"], rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(m.rq_forward(hidden, codes[:, :3]).numpy(), g["forward_logits_q3"], rtol=2e-5, atol=2e-5)
    np.testing.assert_array_equal(m.rq_generate(hidden, codes[:, 0], 1.0, 1).numpy(), g["greedy"])
    np.testing.assert_array_equal(m.rq_generate_full(hidden, codes[:, 0], 1.0, 1).numpy(), g["greedy"])
    bias = T(g["bias"])
    np.testing.assert_array_equal(m.rq_generate(hidden, codes[:, 0], 0.7, 1, bias).numpy(), g["greedy_bias"])
    np.testing.assert_array_equal(m.rq_generate_full(hidden, codes[:, 0], 0.7, 1, bias).numpy(), g["greedy_bias"])
    # n_quantizers < Q: a prefix of the full greedy frame (model.py:860-877, 1001)
    np.testing.assert_array_equal(m.rq_generate(hidden, codes[:, 0], 1.0, 1, n_quantizers=3).numpy(), g["greedy"][:, :3])


def test_tiny_rq_sampling_histogram():
    """The reference's top-k/temperature draw of codebook 1 (20000 rows, torch RNG) against the
    oracle's analytic kept distribution and against the oracle's own Philox-driven draws."""
    g = load("tiny_rq.npz")
    d = tiny_dims(4)
    m = O.OracleModel(d, O.synthetic_state_dict(d, **TINY_SD), torch.float32)
    hidden, codes = T(g["hidden"])[:1], T(g["codes"])[:1]
    _, lg = m.rq_generate(hidden, codes[:, 0], 1.0, 1, return_logits=True)
    w = O.topk_threshold_probs(lg[0, 0], 0.8, 5)
    hist = g["samp_hist_cb1"].astype(np.float64)
    assert set(np.nonzero(w)[0]) == set(np.nonzero(hist)[0])
    exp = w / w.sum() * hist.sum()
    chi2 = (((hist - exp) ** 2)[exp > 0] / exp[exp > 0]).sum()
    assert chi2 < 30, chi2  # 4 dof
    mine = np.zeros_like(hist)
    for f in range(20000):
        mine[O.sample_rq(lg[0, 0], 0.8, 5, O.uniform01(0, f, 0, 1))] += 1
    chi2 = (((mine - exp) ** 2)[exp > 0] / exp[exp > 0]).sum()
    assert chi2 < 30, chi2


def test_tiny_bf16_within_tolerance():
    """bf16 regime: the reference's CPU bf16 run and the oracle round at the same places but sum in
    different orders, so results agree to a few bf16 ulps, not bit for bit."""
    g = load("tiny_bf16.npz")
    d = tiny_dims(2)
    m = O.OracleModel(d, O.synthetic_state_dict(d, **TINY_SD), torch.bfloat16)
    ids, codes = T(g["ids"]), T(g["codes"])
    h_pre = m.prefill(m.embed_text(ids))
    tol = 0.04  # CPU bf16 SDPA rounds scores and probabilities to bf16, the oracle keeps them fp32
    assert np.abs(h_pre.numpy() - g["h_prefill"]).max() <= tol * np.abs(g["h_prefill"]).max()
    for i in range(codes.shape[0]):
        h, cb0, eos = m.decode_step(codes[i][None])
        assert np.abs(cb0[0].numpy() - g["cb0"][i]).max() <= tol * np.abs(g["cb0"][i]).max()
        assert np.abs(h[0].numpy() - g["hidden"][i]).max() <= tol * np.abs(g["hidden"][i]).max()
    lg = m.rq_forward(T(g["rq_hidden"]), codes[:3])
    assert np.abs(lg.numpy() - g["rq_logits"]).max() <= tol * np.abs(g["rq_logits"]).max()


@pytest.mark.slow
def test_nano_grid_config1():
    """Benchmark config 1 on the oracle: identical 64x16 greedy token grid to the reference's classes."""
    path = os.path.join(GOLDEN, "nano_grid.npz")
    if not os.path.exists(path):
        pytest.skip("nano_grid.npz not generated")
    g = np.load(path)
    d = O.Dims()
    sd = O.synthetic_state_dict(d, seed=0)
    keys = list(g["weight_checksum_keys"])
    for k, c in zip(keys, g["weight_checksums"]):
        assert int(sd[str(k)].view(torch.int32).to(torch.int64).sum()) == int(c), f"synthetic weights differ from the fixture's at {k}"
    n_frames = int(os.environ.get("VUI_GRID_FRAMES", "64"))
    m = O.OracleModel(d, sd, torch.float32, max_seqlen=128)
    h = m.prefill(m.embed_text(T(g["ids"])))[-1:]
    np.testing.assert_allclose(h[0].numpy(), g["first_hidden"], rtol=1e-4, atol=1e-5)
    grid = m.generate_frames(h, n_frames, top_k=1, temperature=1.0)[:, 0]
    np.testing.assert_array_equal(grid.numpy(), g["grid"][:n_frames])
