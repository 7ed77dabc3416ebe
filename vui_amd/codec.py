"""Host-side mirror of the reference's codec decoder and its streaming driver
(src/vui/qwen_codec.py: QwenCodecDecoder :1079-1293, CodecCtx :410-668) over the native vocoder
frame step (include/vui_codec.h).  There is no CPU or PyTorch fallback: a missing library raises.

Differences from the reference surface, both forced by the native state living in one place:
an offline `forward` (no stream open) runs the frames through a cold stream and leaves the state
cold again, and it refuses to run while a stream is open instead of leaving that stream untouched.
"""
from __future__ import annotations

import ctypes as C
import math
from dataclasses import dataclass

import torch
from torch import Tensor

from . import _lib

SAMPLE_RATE = 24000
DOWNSAMPLE_RATE = 1920
FRAME_RATE = SAMPLE_RATE / DOWNSAMPLE_RATE  # 12.5
N_CODEBOOKS = 16


@dataclass
class CodecConfig:
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

    def to_c(self) -> _lib.CodecConfigC:
        c = _lib.CodecConfigC()
        for n in ("n_codebooks", "codebook_size", "codebook_dim", "vq_dim", "n_semantic", "latent_dim", "d_model",
                  "n_layers", "n_heads", "head_dim", "mlp_dim", "max_seq", "decoder_dim"):
            setattr(c, n, int(getattr(self, n)))
        c.rope_theta = float(self.rope_theta)
        c.n_up = len(self.up_ratios)
        for i, r in enumerate(self.up_ratios):
            c.up_ratios[i] = int(r)
        c.n_rates = len(self.rates)
        for i, r in enumerate(self.rates):
            c.rates[i] = int(r)
        return c


def codec_state_dict_shapes(d: CodecConfig) -> dict[str, tuple[int, ...]]:
    """Keys and shapes of QwenCodecDecoder.state_dict(), in the order the native library takes them."""
    sh: dict[str, tuple[int, ...]] = {}
    for name, n in (("semantic", d.n_semantic), ("acoustic", d.n_codebooks - d.n_semantic)):
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
        for n in ("q_proj", "k_proj", "v_proj"):
            sh[p + n + ".weight"] = (A, d.d_model)
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


def hf_key_map(d: CodecConfig) -> dict[str, str]:
    """state-dict key -> key of the published tokenizer checkpoint, `decoder.` prefix removed
    (_decoder_key_map, qwen_codec.py:1391-1480).  Codebooks are stored there as running sums and are
    rebuilt by `from_hf_state` (qwen_codec.py:1321-1322, 1483-1496)."""
    m = {}
    for k in codec_state_dict_shapes(d):
        if ".codebooks." in k or k.endswith("input_proj.weight") and k.startswith("quantizer"):
            continue
        h = k
        h = h.replace("quantizer.semantic.", "quantizer.rvq_first.").replace("quantizer.acoustic.", "quantizer.rvq_rest.")
        if k.startswith("pre_transformer.layers."):
            for n in ("q_proj", "k_proj", "v_proj", "o_proj"):
                h = h.replace(f".{n}.", f".self_attn.{n}.")
            for n in ("gate_proj", "up_proj", "down_proj"):
                h = h.replace(f".{n}.", f".mlp.{n}.")
            h = h.replace(".attn_scale", ".self_attn_layer_scale.scale").replace(".mlp_scale", ".mlp_layer_scale.scale")
        m[k] = h
    return m


class _Stream:
    """The object `QwenCodecDecoder.streaming()` returns: closing it ends the stream."""

    def __init__(self, dec: "QwenCodecDecoder"):
        self.dec = dec

    def close(self) -> None:
        self.dec._streaming = False

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False


class QwenCodecDecoder:
    """Codes (1, n_q, T) -> audio (1, 1, T * 1920), fp32, on the native frame step."""

    def __init__(self, state_dict: dict[str, Tensor], cfg: CodecConfig | None = None, device: str | torch.device = "cuda"):
        self.cfg = cfg or CodecConfig()
        self.device = torch.device(device)
        lib = _lib.load()
        self.lib = lib
        cc = self.cfg.to_c()
        shapes = codec_state_dict_shapes(self.cfg)
        n = lib.vui_codec_n_tensors(C.byref(cc))
        if n < 0:
            raise ValueError(_lib.last_error())
        assert n == len(shapes)
        missing = [k for k in shapes if k not in state_dict]
        if missing:
            raise KeyError(f"codec state dict lacks {missing[:4]}{'...' if len(missing) > 4 else ''}")
        tensors = []
        for k, shp in shapes.items():
            t = state_dict[k]
            if tuple(t.shape) != tuple(shp):
                raise ValueError(f"Shape mismatch: {k} {tuple(t.shape)} vs {shp}")
            tensors.append(t.to(device=self.device, dtype=torch.float32).contiguous())
        need = lib.vui_codec_workspace_bytes(C.byref(cc))
        if need < 0:
            raise ValueError(_lib.last_error())
        self._ws = torch.empty(need, dtype=torch.uint8, device=self.device)
        arr = (C.c_void_p * n)(*[t.data_ptr() for t in tensors])
        h = C.c_void_p()
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.vui_codec_init(C.byref(cc), arr, n, self._ws.data_ptr(), need, st, C.byref(h)), "vui_codec_init")
        torch.cuda.current_stream().synchronize()  # the caller's tensors may go away now
        self.handle = h
        self.hop = self.cfg.hop
        self._streaming = False
        self._cap_stream = torch.cuda.Stream(device=self.device)
        self._graphs: dict[int, object] = {}
        self._stream_codes_in = torch.zeros(self.cfg.n_codebooks, dtype=torch.long, device=self.device)
        self._stream_out = torch.zeros(1, 1, self.hop, dtype=torch.float32, device=self.device)

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                self.lib.vui_codec_destroy(self.handle)
                self.handle = None
        except Exception:
            pass

    # ---- loading ----
    @classmethod
    def from_hf_state(cls, hf_state: dict[str, Tensor], cfg: CodecConfig | None = None, device="cuda") -> "QwenCodecDecoder":
        """From the tensors of the published tokenizer checkpoint with the `decoder.` prefix removed
        (QwenCodecDecoder.from_pretrained, qwen_codec.py:1278-1293)."""
        cfg = cfg or CodecConfig()
        sd = {}
        for ours, theirs in hf_key_map(cfg).items():
            sd[ours] = hf_state[theirs]
        for name, hf, n in (("semantic", "rvq_first", cfg.n_semantic), ("acoustic", "rvq_rest", cfg.n_codebooks - cfg.n_semantic)):
            sd[f"quantizer.{name}.input_proj.weight"] = hf_state.get(
                f"quantizer.{hf}.input_proj.weight", torch.zeros(cfg.codebook_dim, cfg.vq_dim, 1))
            for i in range(n):
                usage = hf_state[f"quantizer.{hf}.vq.layers.{i}._codebook.cluster_usage"].float()
                esum = hf_state[f"quantizer.{hf}.vq.layers.{i}._codebook.embedding_sum"].float()
                sd[f"quantizer.{name}.codebooks.{i}.embed"] = esum / usage.clamp(min=1e-5).unsqueeze(1)
        return cls(sd, cfg, device)

    @classmethod
    def from_pretrained(cls, path: str, cfg: CodecConfig | None = None, device="cuda") -> "QwenCodecDecoder":
        """From local .safetensors files of the tokenizer checkpoint (a directory or one file); nothing
        is downloaded."""
        import glob
        import os

        from safetensors import safe_open

        files = sorted(glob.glob(os.path.join(path, "*.safetensors"))) if os.path.isdir(path) else [path]
        if not files:
            raise FileNotFoundError(f"no .safetensors under {path}")
        state = {}
        for f in files:
            with safe_open(f, framework="pt", device="cpu") as st:
                for k in st.keys():
                    if k.startswith("decoder."):
                        state[k[len("decoder."):]] = st.get_tensor(k)
        return cls.from_hf_state(state, cfg, device)

    # ---- streaming state ----
    @property
    def is_streaming(self) -> bool:
        return self._streaming

    def streaming(self, batch_size: int = 1) -> _Stream:
        """Opens a cold stream (StreamingModule.streaming, src/vui/streaming.py:74-87); one row."""
        if batch_size != 1:
            raise ValueError("the native vocoder step decodes one stream at a time")
        assert not self._streaming, "already streaming"
        self.reset_streaming()
        self._streaming = True
        return _Stream(self)

    def reset_streaming(self) -> None:
        _lib.check(self.lib.vui_codec_reset(self.handle, torch.cuda.current_stream().cuda_stream), "vui_codec_reset")

    def frames_since_reset(self) -> int:
        n = self.lib.vui_codec_status(self.handle, torch.cuda.current_stream().cuda_stream)
        if n < 0:
            raise RuntimeError(_lib.last_error())
        return int(n)

    def persistent(self, enable: int = -1) -> bool:
        """Whether the one-column steps of a frame run as one persistent kernel; enable = 1/0 switches it
        (captured graphs keep the form they were captured with)."""
        return bool(self.lib.vui_codec_persistent(self.handle, int(enable)))

    def workgroups(self, n: int) -> None:
        """The persistent form of the one-column steps on n workgroups (vui_codec_workgroups): for a vocoder that
        runs on a stream bound to part of the GPU.  Captured graphs are dropped: they hold the old width."""
        _lib.check(self.lib.vui_codec_workgroups(self.handle, int(n)), "vui_codec_workgroups")
        self._graphs.clear()

    def setup_streaming_graph(self, batch_size: int = 1, n_q: int | None = None, **_) -> None:
        """Captures the one-frame step as a HIP graph over static in/out buffers
        (setup_streaming_graph, qwen_codec.py:1138-1189).  The capture itself advances nothing."""
        from .model import Graph

        if batch_size != 1:
            raise ValueError("the native vocoder step decodes one stream at a time")
        n_q = int(n_q or self.cfg.n_codebooks)
        if n_q in self._graphs:
            return

        def body(st):
            _lib.check(self.lib.vui_codec_decode_frame(self.handle, self._stream_codes_in.data_ptr(), n_q,
                                                       self._stream_out.data_ptr(), st), "vui_codec_decode_frame")

        self._graphs[n_q] = Graph(self, body, warmup=0)

    # ---- forward ----
    def _frame(self, codes_q: Tensor, out: Tensor) -> None:
        n_q = codes_q.shape[0]
        g = self._graphs.get(n_q)
        if g is not None:
            self._stream_codes_in[:n_q].copy_(codes_q)
            g.replay()
            out.copy_(self._stream_out.view(-1))
            return
        _lib.check(self.lib.vui_codec_decode_frame(self.handle, codes_q.data_ptr(), n_q, out.data_ptr(),
                                                   torch.cuda.current_stream().cuda_stream), "vui_codec_decode_frame")

    @torch.inference_mode()
    def forward(self, codes: Tensor) -> Tensor:
        """codes (1, n_q, T) long -> audio (1, 1, T * hop).  Inside `streaming()` the call continues the
        stream; outside it decodes the T frames from a cold state (the offline forward)."""
        if codes.dim() != 3 or codes.shape[0] != 1:
            raise ValueError("codes must be (1, n_q, T)")
        n_q, T = codes.shape[1], codes.shape[2]
        if n_q < 1 or n_q > self.cfg.n_codebooks:
            raise ValueError(f"n_q={n_q} outside [1, {self.cfg.n_codebooks}]")
        offline = not self._streaming
        if offline:
            if T > self.cfg.max_seq:
                raise ValueError(f"{T} frames exceed the decoder's window of {self.cfg.max_seq}; decode in chunks")
            self.reset_streaming()
        ct = codes[0].to(device=self.device, dtype=torch.long).t().contiguous()  # (T, n_q)
        if T == 1 and not offline and n_q in self._graphs:
            self._frame(ct[0], self._stream_out.view(-1))
            return self._stream_out
        audio = torch.empty(1, 1, T * self.hop, dtype=torch.float32, device=self.device)
        flat = audio.view(-1)
        for t in range(T):
            self._frame(ct[t], flat[t * self.hop:(t + 1) * self.hop])
        if offline:
            self.reset_streaming()
        return audio

    __call__ = forward

    def decode(self, codes: Tensor) -> Tensor:
        return self.forward(codes)


class CodecCtx:
    """Managed decode with the 10 s context window (CodecCtx, qwen_codec.py:410-668): rolling code
    buffer shared by the full-decode and the streaming mode; a new stream is seeded with the last
    `n_frames % max_ctx` buffered frames and restarts cold every `max_ctx` frames."""

    def __init__(self, decoder: QwenCodecDecoder, max_ctx_secs: float = 10.0):
        self.decoder = decoder
        self.max_ctx = int(max_ctx_secs * FRAME_RATE)
        self._prompt_len = 0
        self._buf: Tensor | None = None
        self._stack: _Stream | None = None
        self._frames_since_prefill = 0
        self._prefill_n_codebooks = 0

    def set_prompt(self, codes: Tensor) -> None:
        if codes.dim() == 2:
            codes = codes.unsqueeze(0)
        self._prompt_len = codes.shape[2]
        self._buf = codes
        self._close_stack()

    def add(self, codes: Tensor) -> None:
        if codes.dim() == 2:
            codes = codes.unsqueeze(0)
        self._append(codes)

    @property
    def n_frames(self) -> int:
        return self._buf.shape[2] if self._buf is not None else 0

    def get_context(self, max_frames: int | None = None) -> Tensor | None:
        if self._buf is None:
            return None
        limit = max_frames or self.max_ctx
        T = self._buf.shape[2]
        if T <= limit:
            return self._buf
        if 0 < self._prompt_len < limit:
            avail = limit - self._prompt_len
            return torch.cat([self._buf[:, :, : self._prompt_len], self._buf[:, :, -avail:]], dim=2)
        return self._buf[:, :, -limit:]

    def _append(self, codes: Tensor) -> None:
        if self._buf is None:
            self._buf = codes
        else:
            if codes.shape[1] != self._buf.shape[1]:
                min_q = min(codes.shape[1], self._buf.shape[1])
                if self._buf.shape[1] != min_q:
                    self._buf = self._buf[:, :min_q].contiguous()
                if codes.shape[1] != min_q:
                    codes = codes[:, :min_q].contiguous()
            self._buf = torch.cat([self._buf, codes.to(self._buf.device)], dim=2)
        limit = self.max_ctx * 2
        if self._buf.shape[2] > limit:
            if 0 < self._prompt_len < limit:
                self._buf = torch.cat([self._buf[:, :, : self._prompt_len], self._buf[:, :, -(limit - self._prompt_len):]], dim=2)
            else:
                self._buf = self._buf[:, :, -limit:]

    # --- full decode (rolling window) ---
    @torch.inference_mode()
    def __call__(self, codes: Tensor) -> Tensor:
        if codes.dim() == 2:
            codes = codes.unsqueeze(0)
        T_new = codes.shape[2]
        ctx = self.get_context()
        ctx_t = ctx.shape[2] if ctx is not None else 0
        if ctx_t + T_new <= self.max_ctx:
            if ctx is not None:
                audio = self.decoder(torch.cat([ctx.to(codes.device), codes], dim=2))
                self._append(codes)
                return audio[..., ctx_t * self.decoder.hop:]
            audio = self.decoder(codes)
            self._append(codes)
            return audio
        return self._decode_chunked(codes)

    def _decode_chunked(self, codes: Tensor) -> Tensor:
        ctx = self.get_context(self.max_ctx // 2)
        T = codes.shape[2]
        wavs, pos = [], 0
        while pos < T:
            ctx_t = ctx.shape[2] if ctx is not None else 0
            end = min(pos + self.max_ctx - ctx_t, T)
            chunk = codes[:, :, pos:end]
            if ctx is not None:
                audio = self.decoder(torch.cat([ctx.to(codes.device), chunk], dim=2))
                wavs.append(audio[..., ctx_t * self.decoder.hop:])
            else:
                wavs.append(self.decoder(chunk))
            ctx_limit = min(self.max_ctx // 2, end)
            ctx = codes[:, :, end - ctx_limit: end]
            pos = end
        self._append(codes)
        return torch.cat(wavs, dim=-1)

    # --- streaming ---
    def prefill(self, n_codebooks: int = 0, device: str | torch.device = "cuda") -> None:
        self._prefill_n_codebooks = n_codebooks
        self._hard_reset()
        self._reseed()

    def _reseed(self) -> None:
        if self._buf is None or self._buf.shape[2] == 0:
            self._frames_since_prefill = 0
            return
        n = self._buf.shape[2] % self.max_ctx
        if n == 0:
            self._frames_since_prefill = 0
            return
        seed = self._buf[:, :, -n:]
        if self._prefill_n_codebooks > 0:
            seed = seed[:, : self._prefill_n_codebooks]
        self.decoder(seed)
        self._frames_since_prefill = n

    def _hard_reset(self) -> None:
        self._close_stack()
        self._stack = self.decoder.streaming(1)
        self._frames_since_prefill = 0

    def decode_frame(self, codes: Tensor, vocoder_ctx: int | None = None, store_codes: Tensor | None = None) -> Tensor:
        """One frame (1, n_q, 1) -> audio (1, 1, hop) inside the active stream; cold restart every
        `max_ctx` frames (qwen_codec.py:625-657).  The returned tensor is a static buffer when the
        step runs from its captured graph."""
        if codes.dim() == 2:
            codes = codes.unsqueeze(0)
        if self._stack is None or self._frames_since_prefill >= self.max_ctx:
            self._hard_reset()
        audio = self.decoder(codes)
        self._append(store_codes if store_codes is not None else codes)
        self._frames_since_prefill += 1
        return audio

    def _close_stack(self) -> None:
        if self._stack is not None:
            self._stack.close()
            self._stack = None

    def reset(self) -> None:
        self._prompt_len = 0
        self._buf = None
        self._frames_since_prefill = 0
        self._close_stack()
