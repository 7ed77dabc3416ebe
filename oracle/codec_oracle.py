"""CPU oracle for the streaming vocoder frame step.  TEST INFRASTRUCTURE ONLY.

Restates, with plain PyTorch CPU ops in fp32 (the reference's codec regime,
`codec_dtype=torch.float32`, src/vui/engine.py:302), the decoder half of the reference's codec:
codes (B, n_q, T) -> audio (B, 1, T * 1920), both as the stateless offline forward and as the
stateful streaming forward that the reference runs one frame at a time.  Only tests, the smoke
check and the CPU-baseline leg of the benchmark may import it; the product package never does.

Every function cites the reference lines it follows (paths relative to the reference checkout).

How each function is pinned (tests/test_codec_oracle.py):

* causal_conv, causal_transconv, snake_beta, convnext_block, res_unit, decoder_block,
  vq_decode, DecTransformer (offline and streaming, chunked feeding), the whole decoder at small
  dims and at the real dims: golden vectors written from the reference's own classes by
  tests/golden/make_codec_golden.py (weights from `synthetic_codec_state_dict`).
* streaming == offline: feeding the frames one by one (or in ragged chunks) through the
  streaming form reproduces the offline forward (the property the reference's streaming design
  is built on, qwen_codec.py:410-427), checked on random inputs.
* CodecCtx bookkeeping (window, re-seed, cold restart every 125 frames): restated rule by rule
  from qwen_codec.py:429-668 and pinned by goldens of the reference class driving the reference
  decoder.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

Tensor = torch.Tensor

SAMPLE_RATE = 24000  # qwen_codec.py:27-30
FRAME_RATE = 12.5


@dataclass
class CodecDims:
    """Architecture numbers of QwenCodecDecoder.__init__ (qwen_codec.py:1080-1125)."""

    n_codebooks: int = 16
    codebook_size: int = 2048
    codebook_dim: int = 256
    vq_dim: int = 512
    n_semantic: int = 1
    latent_dim: int = 1024
    d_model: int = 512
    n_layers: int = 8
    n_heads: int = 16
    head_dim: int = 64
    mlp_dim: int = 1024
    max_seq: int = 250
    rope_theta: float = 10000.0
    up_ratios: tuple = (2, 2)
    decoder_dim: int = 1536
    rates: tuple = (8, 5, 4, 3)

    @property
    def hop(self) -> int:
        return math.prod(self.up_ratios) * math.prod(self.rates)

    @property
    def n_acoustic(self) -> int:
        return self.n_codebooks - self.n_semantic


def tiny_dims() -> CodecDims:
    return CodecDims(n_codebooks=4, codebook_size=32, codebook_dim=8, vq_dim=16, latent_dim=24, d_model=16,
                     n_layers=2, n_heads=2, head_dim=8, mlp_dim=24, max_seq=40, up_ratios=(2, 2),
                     decoder_dim=32, rates=(3, 2))


# --------------------------------------------------------------------------------------
# weights
# --------------------------------------------------------------------------------------
def codec_state_dict_shapes(d: CodecDims) -> dict[str, tuple[int, ...]]:
    """Keys and shapes of QwenCodecDecoder.state_dict() (qwen_codec.py:1080-1125, 185-253, 832-1000)."""
    sh: dict[str, tuple[int, ...]] = {}
    for name, n in (("semantic", d.n_semantic), ("acoustic", d.n_acoustic)):
        p = f"quantizer.{name}."
        sh[p + "input_proj.weight"] = (d.codebook_dim, d.vq_dim, 1)
        sh[p + "output_proj.weight"] = (d.vq_dim, d.codebook_dim, 1)
        for i in range(n):
            sh[p + f"codebooks.{i}.embed"] = (d.codebook_size, d.codebook_dim)
    sh["pre_conv.conv.weight"] = (d.latent_dim, d.vq_dim, 3)
    sh["pre_conv.conv.bias"] = (d.latent_dim,)
    A = d.n_heads * d.head_dim
    sh["pre_transformer.input_proj.weight"] = (d.d_model, d.latent_dim)
    sh["pre_transformer.input_proj.bias"] = (d.d_model,)
    for i in range(d.n_layers):
        p = f"pre_transformer.layers.{i}."
        sh[p + "input_layernorm.weight"] = (d.d_model,)
        sh[p + "q_proj.weight"] = (A, d.d_model)
        sh[p + "k_proj.weight"] = (A, d.d_model)
        sh[p + "v_proj.weight"] = (A, d.d_model)
        sh[p + "o_proj.weight"] = (d.d_model, A)
        sh[p + "attn_scale"] = (d.d_model,)
        sh[p + "post_attention_layernorm.weight"] = (d.d_model,)
        sh[p + "gate_proj.weight"] = (d.mlp_dim, d.d_model)
        sh[p + "up_proj.weight"] = (d.mlp_dim, d.d_model)
        sh[p + "down_proj.weight"] = (d.d_model, d.mlp_dim)
        sh[p + "mlp_scale"] = (d.d_model,)
    sh["pre_transformer.norm.weight"] = (d.d_model,)
    sh["pre_transformer.output_proj.weight"] = (d.latent_dim, d.d_model)
    sh["pre_transformer.output_proj.bias"] = (d.latent_dim,)
    L = d.latent_dim
    for i, r in enumerate(d.up_ratios):
        p = f"upsample.{i}."
        sh[p + "0.conv.weight"] = (L, L, r)
        sh[p + "0.conv.bias"] = (L,)
        sh[p + "1.dwconv.conv.weight"] = (L, 1, 7)
        sh[p + "1.dwconv.conv.bias"] = (L,)
        sh[p + "1.norm.weight"] = (L,)
        sh[p + "1.norm.bias"] = (L,)
        sh[p + "1.pwconv1.weight"] = (4 * L, L)
        sh[p + "1.pwconv1.bias"] = (4 * L,)
        sh[p + "1.pwconv2.weight"] = (L, 4 * L)
        sh[p + "1.pwconv2.bias"] = (L,)
        sh[p + "1.gamma"] = (L,)
    dim = d.decoder_dim
    sh["decoder.0.conv.weight"] = (dim, L, 7)
    sh["decoder.0.conv.bias"] = (dim,)
    for i, rate in enumerate(d.rates):
        out = dim // 2
        p = f"decoder.{i + 1}.block."
        sh[p + "0.alpha"] = (dim,)
        sh[p + "0.beta"] = (dim,)
        sh[p + "1.conv.weight"] = (dim, out, 2 * rate)
        sh[p + "1.conv.bias"] = (out,)
        for j in (2, 3, 4):
            q = p + f"{j}."
            sh[q + "act1.alpha"] = (out,)
            sh[q + "act1.beta"] = (out,)
            sh[q + "conv1.conv.weight"] = (out, out, 7)
            sh[q + "conv1.conv.bias"] = (out,)
            sh[q + "act2.alpha"] = (out,)
            sh[q + "act2.beta"] = (out,)
            sh[q + "conv2.conv.weight"] = (out, out, 1)
            sh[q + "conv2.conv.bias"] = (out,)
        dim = out
    n = len(d.rates)
    sh[f"decoder.{n + 1}.alpha"] = (dim,)
    sh[f"decoder.{n + 1}.beta"] = (dim,)
    sh[f"decoder.{n + 2}.conv.weight"] = (1, dim, 7)
    sh[f"decoder.{n + 2}.conv.bias"] = (1,)
    return sh


def synthetic_codec_state_dict(d: CodecDims, seed: int = 0) -> dict[str, Tensor]:
    """Deterministic fp32 weights that keep activations O(1) through the ~60 layers: linear and
    conv weights N(0, 1/fan_in), biases N(0, 0.05), norm weights 1 + N(0, 0.1), snake log-rates
    N(0, 0.3), residual scales (attn_scale, mlp_scale, gamma) N(0.3, 0.1), codebooks N(0, 1); the closing
    1x1 conv of every residual unit is scaled by 0.3 and the last conv by 0.12 so that the residual stream does
    not grow and the audio is not clamped everywhere.  Each key draws from its own CPU generator seeded with (seed, key index)."""
    sd = {}
    for idx, (k, shape) in enumerate(codec_state_dict_shapes(d).items()):
        g = torch.Generator().manual_seed(seed * 1000003 + 7919 + idx)
        r = torch.randn(shape, generator=g)
        if k.endswith("embed"):
            t = r
        elif k.endswith(("alpha", "beta")):
            t = 0.3 * r
        elif k.endswith(("attn_scale", "mlp_scale", "gamma")):
            t = 0.3 + 0.1 * r
        elif k.endswith("layernorm.weight") or k.endswith("norm.weight"):
            t = 1.0 + 0.1 * r
        elif k.endswith(".bias"):
            t = 0.05 * r
        elif len(shape) == 3 and ".block.1." in k or (len(shape) == 3 and k.startswith("upsample") and ".0.conv" in k):
            # ConvTranspose1d (in, out, k): each output sample sums in * k/stride terms (stride = k or k/2)
            stride = shape[2] if k.startswith("upsample") else shape[2] // 2
            t = r / math.sqrt(shape[0] * shape[2] / stride)
        elif len(shape) == 3:
            t = r / math.sqrt(shape[1] * shape[2])
            if "conv2.conv" in k:
                t = 0.3 * t
            elif shape[0] == 1:
                t = 0.12 * t
        else:
            t = r / math.sqrt(shape[-1])
        sd[k] = t.contiguous()
    return sd


# --------------------------------------------------------------------------------------
# building blocks; `state` is a dict name -> tensor (None = offline)
# --------------------------------------------------------------------------------------
def causal_conv(x: Tensor, w: Tensor, b: Tensor | None, dilation: int, groups: int, state: dict | None, key: str) -> Tensor:
    """CausalConv1d.forward, stride 1 (qwen_codec.py:92-101): left context of (k-1)*dilation columns,
    zeros offline / at stream start, the previous input tail while streaming."""
    pad = (w.shape[2] - 1) * dilation
    if pad > 0:
        if state is None:
            x = F.pad(x, (pad, 0))
        else:
            prev = state.get(key)
            if prev is None:
                prev = torch.zeros(x.shape[0], x.shape[1], pad, dtype=x.dtype)
            x = torch.cat([prev, x], dim=-1)
            state[key] = x[..., -pad:].clone()
    return F.conv1d(x, w, b, dilation=dilation, groups=groups)


def causal_transconv(x: Tensor, w: Tensor, b: Tensor | None, stride: int, state: dict | None, key: str) -> Tensor:
    """CausalTransConv1d.forward (qwen_codec.py:140-158): the kernel-stride trailing samples are
    dropped offline; while streaming they are kept (without the bias) and added to the head of the
    next call's output."""
    y = F.conv_transpose1d(x, w, b, stride=stride)
    pt = w.shape[2] - stride
    if pt == 0:
        return y
    if state is None:
        return y[..., :-pt]
    part = state.get(key)
    y = y.clone()
    if part is not None:
        y[..., :pt] = y[..., :pt] + part
    tail = y[..., -pt:].clone()
    if b is not None:
        tail = tail - b[:, None]
    state[key] = tail
    return y[..., :-pt]


def snake_beta(x: Tensor, alpha: Tensor, beta: Tensor) -> Tensor:
    """SnakeBeta.forward (qwen_codec.py:826-829): x + sin^2(x e^alpha) / (e^beta + 1e-9), per channel."""
    a = alpha[None, :, None].exp()
    bb = beta[None, :, None].exp()
    return x + (1.0 / (bb + 1e-9)) * torch.sin(x * a).pow(2)


def rms_norm(x: Tensor, w: Tensor, eps: float = 1e-6) -> Tensor:
    """RMSNorm.forward (qwen_codec.py:813-817), fp32."""
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def convnext_block(x: Tensor, sd: dict, p: str, state: dict | None) -> Tensor:
    """ConvNeXtBlock.forward (qwen_codec.py:841-848): depthwise k=7 causal conv, LayerNorm over
    channels, Linear -> GELU (erf) -> Linear, per-channel gamma, residual."""
    C = x.shape[1]
    h = causal_conv(x, sd[p + "dwconv.conv.weight"], sd[p + "dwconv.conv.bias"], 1, C, state, p + "dwconv")
    h = h.transpose(1, 2)
    h = F.layer_norm(h, (C,), sd[p + "norm.weight"], sd[p + "norm.bias"], 1e-6)
    h = F.gelu(F.linear(h, sd[p + "pwconv1.weight"], sd[p + "pwconv1.bias"]))
    h = sd[p + "gamma"] * F.linear(h, sd[p + "pwconv2.weight"], sd[p + "pwconv2.bias"])
    return x + h.transpose(1, 2)


def res_unit(x: Tensor, sd: dict, p: str, dilation: int, state: dict | None) -> Tensor:
    """DecoderResUnit.forward (qwen_codec.py:859-860)."""
    h = snake_beta(x, sd[p + "act1.alpha"], sd[p + "act1.beta"])
    h = causal_conv(h, sd[p + "conv1.conv.weight"], sd[p + "conv1.conv.bias"], dilation, 1, state, p + "conv1")
    h = snake_beta(h, sd[p + "act2.alpha"], sd[p + "act2.beta"])
    h = causal_conv(h, sd[p + "conv2.conv.weight"], sd[p + "conv2.conv.bias"], 1, 1, state, p + "conv2")
    return x + h


def decoder_block(x: Tensor, sd: dict, p: str, stride: int, state: dict | None) -> Tensor:
    """DecoderBlock.forward (qwen_codec.py:864-879): snake, transposed conv (kernel 2*stride), three
    residual units with dilations 1, 3, 9."""
    h = snake_beta(x, sd[p + "0.alpha"], sd[p + "0.beta"])
    h = causal_transconv(h, sd[p + "1.conv.weight"], sd[p + "1.conv.bias"], stride, state, p + "1")
    for j, dil in ((2, 1), (3, 3), (4, 9)):
        h = res_unit(h, sd, p + f"{j}.", dil, state)
    return h


def vq_decode(codes: Tensor, sd: dict, d: CodecDims) -> Tensor:
    """SplitResidualVQ.decode (qwen_codec.py:231-238, 263-270): codes (B, n_q, T) -> (B, vq_dim, T);
    codebook rows are summed per group, each group has its own 1x1 output projection."""
    out = None
    n_q = codes.shape[1]
    for name, lo, hi in (("semantic", 0, d.n_semantic), ("acoustic", d.n_semantic, n_q)):
        if hi <= lo:
            continue
        q = 0
        for i in range(lo, hi):
            q = q + F.embedding(codes[:, i], sd[f"quantizer.{name}.codebooks.{i - lo}.embed"]).transpose(1, 2)
        y = F.conv1d(q, sd[f"quantizer.{name}.output_proj.weight"])
        out = y if out is None else out + y
    return out


def rope_tables(n: int, head_dim: int, theta: float) -> tuple[Tensor, Tensor]:
    """RoPE.forward (qwen_codec.py:161-171): angles t * theta^(-2i/dim), the half-table repeated twice."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    fr = torch.outer(torch.arange(n, dtype=torch.float32), inv)
    emb = torch.cat([fr, fr], dim=-1)
    return emb.cos(), emb.sin()


def _rot_half(x: Tensor) -> Tensor:
    x1, x2 = x.chunk(2, dim=-1)
    return torch.cat((-x2, x1), dim=-1)


def dec_transformer(x: Tensor, sd: dict, d: CodecDims, state: dict | None) -> Tensor:
    """DecTransformer.forward / _forward_streaming with DecTransformerBlock.forward
    (qwen_codec.py:940-974, 1034-1076): x (B, T, latent) -> (B, T, latent).  Rotate-half RoPE at the
    absolute position, attention over every earlier position of the stream, residual branches scaled
    per channel (attn_scale, mlp_scale)."""
    p = "pre_transformer."
    B, T, _ = x.shape
    H, hd = d.n_heads, d.head_dim
    x = F.linear(x, sd[p + "input_proj.weight"], sd[p + "input_proj.bias"])
    pos0 = 0 if state is None else state.get("pos", 0)
    if pos0 + T > d.max_seq and state is not None:
        raise IndexError(f"stream position {pos0}+{T} beyond max_seq {d.max_seq}")
    cos, sin = rope_tables(pos0 + T, hd, d.rope_theta)
    cos, sin = cos[pos0:], sin[pos0:]
    for i in range(d.n_layers):
        q_ = p + f"layers.{i}."
        h = rms_norm(x, sd[q_ + "input_layernorm.weight"])
        q = F.linear(h, sd[q_ + "q_proj.weight"]).view(B, T, H, hd).transpose(1, 2)
        k = F.linear(h, sd[q_ + "k_proj.weight"]).view(B, T, H, hd).transpose(1, 2)
        v = F.linear(h, sd[q_ + "v_proj.weight"]).view(B, T, H, hd).transpose(1, 2)
        q = q * cos + _rot_half(q) * sin
        k = k * cos + _rot_half(k) * sin
        if state is not None:
            pk, pv = state.get(f"k{i}"), state.get(f"v{i}")
            if pk is not None:
                k = torch.cat([pk, k], dim=2)
                v = torch.cat([pv, v], dim=2)
            state[f"k{i}"], state[f"v{i}"] = k, v
        S = k.shape[2]
        sc = torch.matmul(q, k.transpose(-1, -2)) / math.sqrt(hd)
        qpos = torch.arange(S - T, S)[:, None]
        mask = torch.arange(S)[None, :] <= qpos
        sc = sc.masked_fill(~mask, float("-inf"))
        a = torch.matmul(torch.softmax(sc, dim=-1), v)
        a = a.transpose(1, 2).reshape(B, T, H * hd)
        x = x + sd[q_ + "attn_scale"] * F.linear(a, sd[q_ + "o_proj.weight"])
        h = rms_norm(x, sd[q_ + "post_attention_layernorm.weight"])
        m = F.silu(F.linear(h, sd[q_ + "gate_proj.weight"])) * F.linear(h, sd[q_ + "up_proj.weight"])
        x = x + sd[q_ + "mlp_scale"] * F.linear(m, sd[q_ + "down_proj.weight"])
    if state is not None:
        state["pos"] = pos0 + T
    x = rms_norm(x, sd[p + "norm.weight"])
    return F.linear(x, sd[p + "output_proj.weight"], sd[p + "output_proj.bias"])


class CodecDecoderOracle:
    """QwenCodecDecoder (qwen_codec.py:1079-1227): `forward(codes)` is the offline pass while no
    stream is open and the stateful pass inside `open_stream()` ... `close_stream()` (the reference's
    `with decoder.streaming(1)`)."""

    def __init__(self, dims: CodecDims, sd: dict[str, Tensor]):
        self.d = dims
        self.sd = {k: v.float() for k, v in sd.items()}
        self.state: dict | None = None

    def open_stream(self) -> None:
        self.state = {}

    def close_stream(self) -> None:
        self.state = None

    @property
    def is_streaming(self) -> bool:
        return self.state is not None

    @torch.no_grad()
    def forward(self, codes: Tensor) -> Tensor:
        d, sd, st = self.d, self.sd, self.state
        h = vq_decode(codes.long(), sd, d)
        h = causal_conv(h, sd["pre_conv.conv.weight"], sd["pre_conv.conv.bias"], 1, 1, st, "pre_conv")
        h = dec_transformer(h.transpose(1, 2), sd, d, st).transpose(1, 2)
        return self.vocoder_chain(h)

    def vocoder_chain(self, h: Tensor) -> Tensor:
        """_vocoder_chain (qwen_codec.py:1217-1224)."""
        d, sd, st = self.d, self.sd, self.state
        for i, r in enumerate(d.up_ratios):
            p = f"upsample.{i}."
            h = causal_transconv(h, sd[p + "0.conv.weight"], sd[p + "0.conv.bias"], r, st, p + "0")
            h = convnext_block(h, sd, p + "1.", st)
        h = causal_conv(h, sd["decoder.0.conv.weight"], sd["decoder.0.conv.bias"], 1, 1, st, "decoder.0")
        for i, rate in enumerate(d.rates):
            h = decoder_block(h, sd, f"decoder.{i + 1}.block.", rate, st)
        n = len(d.rates)
        h = snake_beta(h, sd[f"decoder.{n + 1}.alpha"], sd[f"decoder.{n + 1}.beta"])
        h = causal_conv(h, sd[f"decoder.{n + 2}.conv.weight"], sd[f"decoder.{n + 2}.conv.bias"], 1, 1, st, f"decoder.{n + 2}")
        return h.clamp(-1, 1)


class CodecCtxOracle:
    """CodecCtx (qwen_codec.py:410-668), streaming side: rolling code buffer, seeding of a new
    stream with the last `n_frames % max_ctx` buffered frames, cold restart of the decoder state
    every `max_ctx` frames."""

    def __init__(self, decoder: CodecDecoderOracle, max_ctx_secs: float = 10.0):
        self.decoder = decoder
        self.max_ctx = int(max_ctx_secs * FRAME_RATE)
        self._prompt_len = 0
        self._buf: Tensor | None = None
        self._open = False
        self._frames_since_prefill = 0
        self._prefill_n_codebooks = 0

    def set_prompt(self, codes: Tensor) -> None:  # :438-445
        if codes.dim() == 2:
            codes = codes.unsqueeze(0)
        self._prompt_len = codes.shape[2]
        self._buf = codes
        self._close()

    def add(self, codes: Tensor) -> None:  # :447-451
        if codes.dim() == 2:
            codes = codes.unsqueeze(0)
        self._append(codes)

    @property
    def n_frames(self) -> int:
        return self._buf.shape[2] if self._buf is not None else 0

    def _append(self, codes: Tensor) -> None:  # :476-502
        if self._buf is None:
            self._buf = codes
        else:
            if codes.shape[1] != self._buf.shape[1]:
                mq = min(codes.shape[1], self._buf.shape[1])
                self._buf = self._buf[:, :mq].contiguous()
                codes = codes[:, :mq].contiguous()
            self._buf = torch.cat([self._buf, codes], dim=2)
        limit = self.max_ctx * 2
        if self._buf.shape[2] > limit:
            if 0 < self._prompt_len < limit:
                self._buf = torch.cat([self._buf[:, :, : self._prompt_len], self._buf[:, :, -(limit - self._prompt_len):]], dim=2)
            else:
                self._buf = self._buf[:, :, -limit:]

    def prefill(self, n_codebooks: int = 0) -> None:  # :558-607
        self._prefill_n_codebooks = n_codebooks
        self._cold()
        if self._buf is None or self._buf.shape[2] == 0:
            return
        n = self._buf.shape[2] % self.max_ctx
        if n == 0:
            return
        seed = self._buf[:, :, -n:]
        if n_codebooks > 0:
            seed = seed[:, :n_codebooks]
        self.decoder.forward(seed)
        self._frames_since_prefill = n

    def _cold(self) -> None:  # _hard_reset :609-623
        self._close()
        self.decoder.open_stream()
        self._open = True
        self._frames_since_prefill = 0

    def _close(self) -> None:
        if self._open:
            self.decoder.close_stream()
            self._open = False

    def decode_frame(self, codes: Tensor, store_codes: Tensor | None = None) -> Tensor:  # :625-657
        if codes.dim() == 2:
            codes = codes.unsqueeze(0)
        if not self._open or self._frames_since_prefill >= self.max_ctx:
            self._cold()
        audio = self.decoder.forward(codes)
        self._append(store_codes if store_codes is not None else codes)
        self._frames_since_prefill += 1
        return audio

    def reset(self) -> None:  # :664-668
        self._prompt_len = 0
        self._buf = None
        self._frames_since_prefill = 0
        self._close()
