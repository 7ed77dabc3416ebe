"""The vocoder oracle against vectors written from the reference's own classes, and against the
properties its streaming design rests on (CPU only)."""
import os

import numpy as np
import pytest
import torch

from oracle import codec_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def load(name):
    return {k: torch.from_numpy(v) for k, v in np.load(os.path.join(GOLD, name)).items()}


def weights(fx, prefix, add=""):
    p = prefix + ".w."
    return {add + k[len(p):]: v for k, v in fx.items() if k.startswith(p)}


def chunks(fn, x, cuts, dim=-1):
    outs, lo = [], 0
    for hi in list(cuts) + [x.shape[dim]]:
        outs.append(fn(x.narrow(dim, lo, hi - lo)))
        lo = hi
    return torch.cat(outs, dim=dim)


def close(a, b, tol=2e-5):
    scale = max(1.0, float(b.abs().max()))
    assert a.shape == b.shape
    assert float((a - b).abs().max()) <= tol * scale, float((a - b).abs().max())


@pytest.fixture(scope="module")
def fx():
    return load("codec_pieces.npz")


@pytest.mark.parametrize("name,dil,groups", [("conv_dil", 2, 1), ("conv_dw", 1, 6), ("conv_k1", 1, 1)])
def test_causal_conv(fx, name, dil, groups):
    w = weights(fx, name)
    x = fx[name + ".x"]
    close(O.causal_conv(x, w["conv.weight"], w["conv.bias"], dil, groups, None, "c"), fx[name + ".offline"])
    st = {}
    close(chunks(lambda c: O.causal_conv(c, w["conv.weight"], w["conv.bias"], dil, groups, st, "c"), x, (1, 4, 5)),
          fx[name + ".stream"])
    # the streamed form is the offline form
    close(fx[name + ".stream"], fx[name + ".offline"])


@pytest.mark.parametrize("name,stride", [("tconv_2s", 3), ("tconv_s", 2)])
def test_causal_transconv(fx, name, stride):
    w = weights(fx, name)
    x = fx[name + ".x"]
    close(O.causal_transconv(x, w["conv.weight"], w["conv.bias"], stride, None, "t"), fx[name + ".offline"])
    st = {}
    close(chunks(lambda c: O.causal_transconv(c, w["conv.weight"], w["conv.bias"], stride, st, "t"), x, (2, 3, 6)),
          fx[name + ".stream"])


def test_snake(fx):
    w = weights(fx, "snake")
    close(O.snake_beta(fx["snake.x"], w["alpha"], w["beta"]), fx["snake.y"])
    # closed form at one point
    x, a, b = 0.7, float(w["alpha"][2]), float(w["beta"][2])
    ref = x + np.sin(x * np.exp(a)) ** 2 / (np.exp(b) + 1e-9)
    got = O.snake_beta(torch.full((1, 6, 1), x), w["alpha"], w["beta"])[0, 2, 0]
    assert abs(float(got) - ref) < 1e-6


def test_convnext(fx):
    w = weights(fx, "convnext")
    x = fx["convnext.x"]
    close(O.convnext_block(x, w, "", None), fx["convnext.offline"])
    st = {}
    close(chunks(lambda c: O.convnext_block(c, w, "", st), x, (1, 2, 6)), fx["convnext.stream"])


def test_decoder_block(fx):
    w = weights(fx, "block")
    x = fx["block.x"]
    close(O.decoder_block(x, w, "block.", 3, None), fx["block.offline"])
    st = {}
    close(chunks(lambda c: O.decoder_block(c, w, "block.", 3, st), x, (1, 2, 5)), fx["block.stream"])


def test_vq_decode(fx):
    w = weights(fx, "vq", add="quantizer.")
    d = O.CodecDims(n_codebooks=4, codebook_size=16, codebook_dim=4, vq_dim=6, n_semantic=1)
    codes = fx["vq.codes"]
    close(O.vq_decode(codes, w, d), fx["vq.y4"])
    close(O.vq_decode(codes[:, :2], w, d), fx["vq.y2"])
    close(O.vq_decode(codes[:, :1], w, d), fx["vq.y1"])


def test_dec_transformer(fx):
    w = weights(fx, "xf", add="pre_transformer.")
    d = O.CodecDims(latent_dim=12, d_model=8, n_layers=2, n_heads=2, head_dim=4, mlp_dim=12, max_seq=20)
    x = fx["xf.x"]
    close(O.dec_transformer(x, w, d, None), fx["xf.offline"])
    st = {}
    close(chunks(lambda c: O.dec_transformer(c, w, d, st), x, (3, 4, 8), dim=1), fx["xf.stream"])
    assert st["pos"] == 9
    with pytest.raises(IndexError):
        O.dec_transformer(torch.zeros(1, 12, 12), w, d, st)


def test_rope_tables_closed_form():
    cos, sin = O.rope_tables(5, 8, 10000.0)
    assert cos.shape == (5, 8)
    for t in (0, 3):
        for i in range(4):
            ang = t * 10000.0 ** (-2 * i / 8)
            assert abs(float(cos[t, i]) - np.cos(ang)) < 1e-6 and abs(float(sin[t, i + 4]) - np.sin(ang)) < 1e-6


@pytest.fixture(scope="module")
def full():
    fxf = load("codec_full.npz")
    d = O.CodecDims()
    dec = O.CodecDecoderOracle(d, O.synthetic_codec_state_dict(d, seed=0))
    return fxf, dec


def test_full_decoder_offline_and_streamed(full):
    fxf, dec = full
    codes = fxf["codes"]
    close(dec.forward(codes), fxf["offline"], 1e-4)
    dec.open_stream()
    st = torch.cat([dec.forward(codes[:, :, i:i + 1]) for i in range(codes.shape[2])], dim=-1)
    dec.close_stream()
    close(st, fxf["stream"], 1e-4)
    close(dec.forward(codes[:, :8, :2]), fxf["offline_q8"], 1e-4)
    assert fxf["offline"].shape[-1] == 4 * O.CodecDims().hop == 4 * 1920


def _digest(a):
    a = a.reshape(-1).double()
    return np.array([a.sum().item(), a.abs().sum().item(), *a[:4].tolist(), *a[-4:].tolist()])


def test_codec_ctx_session(full):
    """Prompt of 30 frames + 10 added, prefill (seeds 40 frames), 90 streamed frames: the decoder
    state restarts cold when 125 frames have passed since the seed."""
    fxf, dec = full
    ctx = O.CodecCtxOracle(dec)
    ctx.set_prompt(fxf["ctx_prompt"])
    ctx.add(fxf["ctx_extra"])
    ctx.prefill()
    assert ctx._frames_since_prefill == 40
    frames = fxf["ctx_frames"]
    for t in range(frames.shape[0]):
        a = ctx.decode_frame(frames[t].view(1, -1, 1))
        assert ctx._frames_since_prefill == int(fxf["ctx_fsp"][t])
        got, ref = _digest(a), fxf["ctx_digest"][t].numpy()
        assert abs(got[0] - ref[0]) < 0.05 and abs(got[1] - ref[1]) < 0.05, (t, got[:2], ref[:2])
        assert np.abs(got[2:] - ref[2:]).max() < 2e-4, t
    assert ctx.n_frames == 130
    assert int(fxf["ctx_fsp"][84]) == 125 and int(fxf["ctx_fsp"][85]) == 1
    ctx.reset()
    assert not dec.is_streaming


def test_streaming_equals_offline_small():
    d = O.tiny_dims()
    dec = O.CodecDecoderOracle(d, O.synthetic_codec_state_dict(d, seed=3))
    g = torch.Generator().manual_seed(2)
    codes = torch.randint(0, d.codebook_size, (2, d.n_codebooks, 13), generator=g)
    off = dec.forward(codes)
    assert off.shape == (2, 1, 13 * d.hop)
    for cuts in ((), tuple(range(1, 13)), (2, 3, 9)):
        dec.open_stream()
        st = chunks(dec.forward, codes, cuts)
        dec.close_stream()
        close(st, off, 1e-4)


def test_ctx_buffer_rules():
    """Buffer trimming keeps the prompt and the newest frames (qwen_codec.py:490-502)."""
    d = O.tiny_dims()
    dec = O.CodecDecoderOracle(d, O.synthetic_codec_state_dict(d, seed=3))
    ctx = O.CodecCtxOracle(dec, max_ctx_secs=0.8)  # 10 frames
    assert ctx.max_ctx == 10
    ctx.set_prompt(torch.zeros(1, 4, 3, dtype=torch.long))
    ctx.add(torch.arange(1, 31).view(1, 1, 30).expand(1, 4, 30))
    assert ctx.n_frames == 20
    assert ctx._buf[0, 0, :3].tolist() == [0, 0, 0] and ctx._buf[0, 0, 3:].tolist() == list(range(14, 31))
    ctx.add(torch.zeros(1, 2, 1, dtype=torch.long))  # fewer codebooks: both sides cut to the smaller count
    assert ctx._buf.shape[1] == 2
    ctx.prefill()  # 20 % 10 == 0 -> cold, nothing fed
    assert ctx._frames_since_prefill == 0 and dec.state == {}
