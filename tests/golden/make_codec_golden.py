"""Writes the vocoder golden vectors under tests/golden/ from the reference's own classes.

Run once, in the build container only (the reference checkout does not travel):

    PYTHONPATH=/root/reference/src python tests/golden/make_codec_golden.py

It imports the reference's `vui.qwen_codec`, fills its modules with deterministic weights and
records small input/output vectors as .npz files.  The fixtures are data only.

Fixtures:
  codec_pieces.npz  CausalConv1d (dilated, depthwise), CausalTransConv1d (kernel = 2*stride and
                    kernel = stride), SnakeBeta, ConvNeXtBlock, DecoderBlock, SplitResidualVQ.decode,
                    DecTransformer - each offline and streamed in ragged chunks; weights inside
  codec_full.npz    QwenCodecDecoder at its real dims with oracle.codec_oracle.synthetic_codec_state_dict
                    (seed 0): offline and frame-by-frame audio of 4 frames, 2 frames with 8 codebooks,
                    and a CodecCtx session (prompt, add, prefill, 90 streamed frames across the
                    125-frame restart) as per-frame digests
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle.codec_oracle import CodecDims, synthetic_codec_state_dict  # noqa: E402

import vui.qwen_codec as Q  # noqa: E402  (reference)
from vui.streaming import StreamingContainer  # noqa: E402  (reference)


def randomize(mod, seed):
    """Every parameter and codebook ~ N(0, 0.5) (the reference initialises several to zero); the RoPE
    frequency table is a derived buffer and stays."""
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for n, p in list(mod.named_parameters()) + list(mod.named_buffers()):
            if p.dtype.is_floating_point and not n.endswith("inv_freq"):
                p.copy_(0.5 * torch.randn(p.shape, generator=g))


def put(out, prefix, mod):
    for k, v in mod.state_dict().items():
        out[f"{prefix}.w.{k}"] = v.detach().numpy().copy()


class Box(StreamingContainer):
    """Gives a plain nn.Module with streaming children the reference's streaming() context."""

    def __init__(self, m):
        super().__init__()
        self.m = m

    def forward(self, x):
        return self.m(x)


def streamed(mod, x, cuts, dim=-1):
    """Feed x in chunks cut at `cuts` along dim inside mod.streaming(1)."""
    outs = []
    if not hasattr(mod, "streaming"):
        mod = Box(mod)
    with torch.inference_mode(), mod.streaming(x.shape[0]):
        lo = 0
        for hi in list(cuts) + [x.shape[dim]]:
            outs.append(mod(x.narrow(dim, lo, hi - lo)).clone())
            lo = hi
    return torch.cat(outs, dim=dim)


def digest(a):
    a = a.reshape(-1).double()
    return np.array([a.sum().item(), a.abs().sum().item(), *a[:4].tolist(), *a[-4:].tolist()])


@torch.inference_mode()
def pieces():
    out = {}
    g = torch.Generator().manual_seed(11)
    # CausalConv1d: dilated, and depthwise
    for name, kw, cin in (("conv_dil", dict(in_ch=5, out_ch=6, kernel=3, dilation=2), 5),
                          ("conv_dw", dict(in_ch=6, out_ch=6, kernel=7, groups=6), 6),
                          ("conv_k1", dict(in_ch=4, out_ch=3, kernel=1), 4)):
        m = Q.CausalConv1d(**kw)
        randomize(m, 1)
        x = torch.randn(1, cin, 11, generator=g)
        put(out, name, m)
        out[name + ".x"] = x.numpy()
        out[name + ".offline"] = m(x).numpy()
        out[name + ".stream"] = streamed(m, x, (1, 4, 5)).numpy()
    for name, kw in (("tconv_2s", dict(in_ch=4, out_ch=3, kernel=6, stride=3)),
                     ("tconv_s", dict(in_ch=4, out_ch=5, kernel=2, stride=2))):
        m = Q.CausalTransConv1d(**kw)
        randomize(m, 2)
        x = torch.randn(1, 4, 7, generator=g)
        put(out, name, m)
        out[name + ".x"] = x.numpy()
        out[name + ".offline"] = m(x).numpy()
        out[name + ".stream"] = streamed(m, x, (2, 3, 6)).numpy()
    m = Q.SnakeBeta(6)
    randomize(m, 3)
    x = 2.0 * torch.randn(1, 6, 9, generator=g)
    put(out, "snake", m)
    out["snake.x"] = x.numpy()
    out["snake.y"] = m(x).numpy()
    m = Q.ConvNeXtBlock(8)
    randomize(m, 4)
    x = torch.randn(1, 8, 9, generator=g)
    put(out, "convnext", m)
    out["convnext.x"] = x.numpy()
    out["convnext.offline"] = m(x).numpy()
    out["convnext.stream"] = streamed(m, x, (1, 2, 6)).numpy()
    m = Q.DecoderBlock(8, 4, 3)
    randomize(m, 5)
    x = torch.randn(1, 8, 8, generator=g)
    put(out, "block", m)
    out["block.x"] = x.numpy()
    out["block.offline"] = m(x).numpy()
    out["block.stream"] = streamed(m, x, (1, 2, 5)).numpy()
    m = Q.SplitResidualVQ(input_dim=6, codebook_dim=4, codebook_size=16, n_semantic=1, n_acoustic=3)
    randomize(m, 6)
    codes = torch.randint(0, 16, (2, 4, 5), generator=g)
    put(out, "vq", m)
    out["vq.codes"] = codes.numpy()
    out["vq.y4"] = m.decode(codes).numpy()
    out["vq.y2"] = m.decode(codes[:, :2]).numpy()
    out["vq.y1"] = m.decode(codes[:, :1]).numpy()
    m = Q.DecTransformer(latent_dim=12, d_model=8, n_layers=2, n_heads=2, head_dim=4, mlp_dim=12, max_seq=20)
    randomize(m, 7)
    x = torch.randn(1, 9, 12, generator=g)
    put(out, "xf", m)
    out["xf.x"] = x.numpy()
    out["xf.offline"] = m(x).numpy()
    out["xf.stream"] = streamed(m, x, (3, 4, 8), dim=1).numpy()
    np.savez_compressed(os.path.join(HERE, "codec_pieces.npz"), **out)
    print("codec_pieces.npz", len(out), "arrays")


@torch.inference_mode()
def full():
    d = CodecDims()
    sd = synthetic_codec_state_dict(d, seed=0)
    dec = Q.QwenCodecDecoder().eval()
    dec.load_state_dict(sd, strict=True)
    g = torch.Generator().manual_seed(5)
    codes = torch.randint(0, d.codebook_size, (1, d.n_codebooks, 4), generator=g)
    out = {"codes": codes.numpy()}
    out["offline"] = dec(codes).numpy()
    out["stream"] = streamed(dec, codes, (1, 2, 3)).numpy()
    out["offline_q8"] = dec(codes[:, :8, :2]).numpy()
    # CodecCtx session
    prompt = torch.randint(0, d.codebook_size, (1, d.n_codebooks, 30), generator=g)
    extra = torch.randint(0, d.codebook_size, (1, d.n_codebooks, 10), generator=g)
    frames = torch.randint(0, d.codebook_size, (90, d.n_codebooks), generator=g)
    ctx = Q.CodecCtx(dec)
    ctx.set_prompt(prompt)
    ctx.add(extra)
    ctx.prefill(n_codebooks=0, device="cpu")
    dig, fsp = [], []
    for t in range(frames.shape[0]):
        a = ctx.decode_frame(frames[t].view(1, -1, 1))
        dig.append(digest(a))
        fsp.append(ctx._frames_since_prefill)
    ctx.reset()
    out["ctx_prompt"] = prompt.numpy()
    out["ctx_extra"] = extra.numpy()
    out["ctx_frames"] = frames.numpy()
    out["ctx_digest"] = np.stack(dig)
    out["ctx_fsp"] = np.array(fsp)
    np.savez_compressed(os.path.join(HERE, "codec_full.npz"), **out)
    print("codec_full.npz", {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    torch.manual_seed(0)
    pieces()
    full()
