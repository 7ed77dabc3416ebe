"""Host-side mirror of the reference's model surface for the per-frame decode path.

Same names, argument meaning and error behaviour as src/vui/model.py (Vui, Decoder,
FlashKVCache, AudioEmbedding, RQTransformer), but every GPU computation on the decode path is
one of the HIP kernels behind libvui_amd.so.  PyTorch is used for device memory, streams and
for the off-path embedding lookups of prompt ingestion.
"""
from __future__ import annotations

import ctypes as C
import json
import math
import os

import torch
import torch.nn.functional as F
from torch import Tensor

from . import _lib
from .config import Config, VuiConfig

MAX_BATCH = _lib.VUI_MAX_BATCH


def precompute_freqs_cis(dim: int, max_seqlen: int, theta: float = 10_000.0,
                         theta_rescale_factor: float = 1.0) -> Tensor:
    """(max_seqlen, dim, 2) fp32 cos/sin table with every frequency repeated twice
    (interleaved pairs).  Same construction as src/vui/rope.py:60-77, on the CPU."""
    theta = theta * theta_rescale_factor ** (dim / (dim - 2))
    pos = torch.arange(max_seqlen, dtype=torch.float32)
    inv_freqs = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))
    freqs = torch.outer(pos, inv_freqs).repeat_interleave(2, dim=-1)
    return torch.stack((freqs.cos(), freqs.sin()), dim=-1)


def quantize_int8(W: Tensor):
    """Weight-only int8, symmetric per output row: scale = max|w|/127 (stored bf16),
    q = clamp(round(w/scale), -127, 127)."""
    Wf = W.float()
    s = (Wf.abs().amax(dim=1) / 127.0).clamp_min(1e-12).to(torch.bfloat16)
    q = torch.clamp(torch.round(Wf / s.float()[:, None]), -127, 127).to(torch.int8)
    return q.contiguous(), s.contiguous()


class FlashKVCache:
    """One layer's view of the shared caches: k_cache/v_cache (slots, S, KV, hd) and the
    seq_lens tensor shared by all layers (src/vui/model.py:71-99, 492-495)."""

    def __init__(self, k_cache: Tensor, v_cache: Tensor, seq_lens: Tensor):
        self.k_cache = k_cache
        self.v_cache = v_cache
        self.seq_lens = seq_lens


class _Linear:
    """Callable weight holder with nn.Linear's attributes; evaluated by the fused GEMV kernel."""

    def __init__(self, weight: Tensor, bias: Tensor | None = None):
        self.weight = weight
        self.bias = bias

    def __call__(self, x: Tensor) -> Tensor:
        lib = _lib.load()
        shp = x.shape
        x2 = x.reshape(-1, shp[-1]).contiguous()
        N, K = self.weight.shape
        y = torch.empty(x2.shape[0], N, device=x.device, dtype=x.dtype)
        dt = _lib.DTYPE_F32 if x.dtype == torch.float32 else _lib.DTYPE_BF16
        st = torch.cuda.current_stream().cuda_stream
        for b0 in range(0, x2.shape[0], MAX_BATCH):
            xb = x2[b0:b0 + MAX_BATCH]
            _lib.check(lib.vui_rmsnorm_gemv(dt, xb.data_ptr(), None, 0.0, self.weight.data_ptr(), None, 0,
                                            y[b0:].data_ptr(), xb.shape[0], N, K, st), "vui_rmsnorm_gemv")
        if self.bias is not None:
            y = (y.float() + self.bias.float()).to(x.dtype)
        return y.reshape(*shp[:-1], N)


class _Embedding:
    def __init__(self, weight: Tensor):
        self.weight = weight

    def __call__(self, ids: Tensor) -> Tensor:
        return F.embedding(ids, self.weight)


class AudioEmbedding:
    """codes (*, Q') -> (*, d): sum over q of table[code_q + q*CS]  (src/vui/model.py:552-563).
    Used for prompt ingestion; the decode step gathers inside the native backbone step."""

    def __init__(self, n_quantizers: int, codebook_size: int, weight: Tensor):
        self.n_quantizers = n_quantizers
        self.codebook_size = codebook_size
        self.embedding = _Embedding(weight)

    def __call__(self, codes: Tensor) -> Tensor:
        Q = codes.shape[-1]
        offsets = torch.arange(Q, device=codes.device) * self.codebook_size
        return self.embedding(codes + offsets).sum(dim=-2)


class _Native:
    """Owns the native context (configuration + device pointers) and its workspace."""

    def __init__(self, model: "Vui", n_slots: int, max_seqlen: int):
        lib = _lib.load()
        m = model.config.model
        c = _lib.VuiConfigC()
        c.dtype = _lib.DTYPE_F32 if model.dtype == torch.float32 else _lib.DTYPE_BF16
        c.d_model, c.n_layers, c.n_heads, c.n_kv_heads = m.d_model, m.n_layers, m.n_heads, m.kv_heads
        c.head_dim, c.ffn = m.head_dim, m.ffn
        c.n_quantizers, c.codebook_size = m.n_quantizers, m.codebook_size
        has_rq = model.rq_transformer is not None
        c.rq_dim = m.rq_d_model if has_rq else m.d_model
        c.rq_layers = m.rq_n_layers if has_rq else 0
        c.rq_heads = m.rq_n_heads if has_rq else 1
        c.rq_ffn = m.rq_ffn if has_rq else 8
        c.rope_dim = (m.rope_dim or m.head_dim) if m.use_rotary_emb else 0
        c.max_seqlen, c.n_slots = max_seqlen, n_slots
        c.window = m.window_size or 0
        dec = model.decoder
        c.global_layers = sum(1 << i for i, g in enumerate(dec.block_is_global) if g)
        c.global_rope_dim = dec.global_rope_dim if (dec.freqs_cis_global is not None and m.use_rotary_emb) else 0
        c.norm_eps, c.rq_norm_eps = 1e-5, 1e-6  # Decoder default / RMSNorm default, model.py:391,287
        c.int8_backbone = 1 if model.int8 else 0
        self.cfg = c
        sd = model.sd
        w = _lib.WeightsC()
        w.audio_emb = sd["audio_emb.embedding.weight"].data_ptr()
        w.final_norm = sd["decoder.norm.weight"].data_ptr()
        w.codec_head = sd["codec_head.weight"].data_ptr()
        w.eos_w = sd["eos_head.weight"].data_ptr()
        w.eos_b = sd["eos_head.bias"].data_ptr()
        w.rope_table = model.decoder.freqs_cis.data_ptr()
        if dec.freqs_cis_global is not None and m.use_rotary_emb:
            w.rope_table_global = dec.freqs_cis_global.data_ptr()
        for i in range(m.n_layers):
            p = f"decoder.blocks.{i}."
            L = w.layers[i]
            L.attn_norm = sd[p + "attn_norm.weight"].data_ptr()
            L.mlp_norm = sd[p + "mlp_norm.weight"].data_ptr()
            for fld, key, sfld in (("wqkv", "attn.Wqkv", "s_qkv"), ("wo", "attn.out_proj", "s_o"),
                                   ("w1", "mlp.w1", "s_1"), ("w3", "mlp.w3", "s_3"), ("w2", "mlp.w2", "s_2")):
                if model.int8:
                    q, s = model.q8[p + key + ".weight"]
                    setattr(L, fld, q.data_ptr())
                    setattr(L, sfld, s.data_ptr())
                else:
                    setattr(L, fld, sd[p + key + ".weight"].data_ptr())
        if has_rq:
            r = "rq_transformer."
            if r + "backbone_proj.weight" in sd:
                w.rq_backbone_proj = sd[r + "backbone_proj.weight"].data_ptr()
            w.rq_code_emb = sd[r + "code_emb.embedding.weight"].data_ptr()
            w.rq_pos_emb = sd[r + "pos_emb.weight"].data_ptr()
            w.rq_head_w = sd[r + "head_W"].data_ptr()
            w.rq_norm = sd[r + "norm.weight"].data_ptr()
            for i in range(m.rq_n_layers):
                p = f"{r}blocks.{i}."
                L = w.rq_layers[i]
                for fld, key in (("attn_norm", "attn_norm"), ("wqkv", "Wqkv"), ("wo", "out_proj"),
                                 ("mlp_norm", "mlp_norm"), ("w1", "w1"), ("w3", "w3"), ("w2", "w2")):
                    setattr(L, fld, sd[p + key + ".weight"].data_ptr())
        self.weights = w
        nbytes = lib.vui_workspace_bytes(C.byref(c), MAX_BATCH)
        if nbytes < 0:
            raise RuntimeError(f"vui_workspace_bytes: {_lib.last_error()}")
        self.workspace = torch.zeros(nbytes + 256, dtype=torch.uint8, device=model.device)
        base = (self.workspace.data_ptr() + 255) & ~255
        h = C.c_void_p()
        _lib.check(lib.vui_ctx_create(C.byref(c), C.byref(w), base, nbytes, MAX_BATCH, C.byref(h)), "vui_ctx_create")
        self.handle = h
        self.lib = lib
        _lib.check(lib.vui_ctx_init(h, torch.cuda.current_stream().cuda_stream), "vui_ctx_init")

    def fused(self, enable: int = -1) -> bool:
        """Query (-1) or switch (1/0) the one-kernel form of the batch-1 bf16 calls."""
        return bool(self.lib.vui_ctx_fused(self.handle, enable))

    def rq_batch(self) -> bool:
        """True when the depth head of 2..16 rows runs as one persistent kernel."""
        return bool(self.lib.vui_ctx_rq_batch(self.handle))

    def bb_batch(self) -> bool:
        """True when the backbone step of 2..16 rows runs as one persistent kernel."""
        return bool(self.lib.vui_ctx_bb_batch(self.handle))

    def workgroups(self, n: int) -> None:
        """The batch-1 one-launch kernel on n workgroups instead of one per compute unit (vui_ctx_workgroups)."""
        _lib.check(self.lib.vui_ctx_workgroups(self.handle, int(n)), "vui_ctx_workgroups")

    def status(self) -> None:
        _lib.check(self.lib.vui_ctx_status(self.handle), "vui_ctx_status")

    def reinit(self) -> None:
        """vui_ctx_init again: clears a raised error word (and rewrites the workspace's derived weight copies)."""
        _lib.check(self.lib.vui_ctx_init(self.handle, torch.cuda.current_stream().cuda_stream), "vui_ctx_init")

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                self.lib.vui_ctx_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class Graph:
    """A captured HIP graph of native calls (stands for torch.cuda.CUDAGraph in the reference)."""

    def __init__(self, model: "Vui", fn, warmup: int = 1):
        lib = _lib.load()
        s = model._cap_stream
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for _ in range(warmup):
                fn(s.cuda_stream)
        s.synchronize()
        _lib.check(lib.vui_graph_begin(s.cuda_stream), "vui_graph_begin")
        try:
            fn(s.cuda_stream)
        finally:
            h = C.c_void_p()
            rc = lib.vui_graph_end(s.cuda_stream, C.byref(h))
        _lib.check(rc, "vui_graph_end")
        self.handle = h
        self.lib = lib
        torch.cuda.current_stream().wait_stream(s)

    def replay(self) -> None:
        _lib.check(self.lib.vui_graph_launch(self.handle, torch.cuda.current_stream().cuda_stream), "vui_graph_launch")

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                self.lib.vui_graph_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class SampleDev:
    """vui_sample_dev: temperature, top-k and seed in 16 bytes of device memory that captured steps read when they
    run.  `set` is a stream-ordered copy (it waits for the copy on the host), skipped when nothing changed."""

    def __init__(self, device):
        self.buf = torch.zeros(16, dtype=torch.uint8, device=device)
        self._cur = None

    def set(self, temperature: float, top_k: "int | None", seed: int) -> "SampleDev":
        import struct

        val = (float(temperature), int(top_k) if top_k is not None else 0, int(seed) & 0xFFFFFFFFFFFFFFFF)
        if val != self._cur:
            self.buf.copy_(torch.frombuffer(bytearray(struct.pack("<fiQ", *val)), dtype=torch.uint8))
            self._cur = val
        return self

    def data_ptr(self) -> int:
        return self.buf.data_ptr()


def make_sample_params(temperature: float, top_k: int | None, seed: int, frame_ctr: Tensor | None,
                       state_rows: Tensor | None = None, keep_ties: bool = False, top_p: float = 0.0,
                       dev: "SampleDev | None" = None):
    sp = _lib.SampleParamsC()
    sp.top_p = float(top_p)
    sp.dev = dev.data_ptr() if dev is not None else None
    sp.keep_ties = 1 if keep_ties else 0
    sp.state_rows = state_rows.data_ptr() if state_rows is not None else None
    sp.temperature = float(temperature)
    sp.top_k = int(top_k) if top_k is not None else 0
    sp.seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    sp.frame_ctr = frame_ctr.data_ptr() if frame_ctr is not None else None
    return sp


class Decoder:
    """Backbone.  Mirrors Decoder in src/vui/model.py:378-549 for the flash/KV-cache path."""

    def __init__(self, model: "Vui", max_seqlen: int):
        m = model.config.model
        self._model = model
        self.max_seqlen = max_seqlen
        self.use_rotary_emb = m.use_rotary_emb
        self.window_size = m.window_size
        self.n_kv_heads = m.kv_heads
        self.head_dim = m.head_dim
        self.n_layers = m.n_layers
        rope_dim = m.rope_dim or m.head_dim
        self.freqs_cis = precompute_freqs_cis(rope_dim, max_seqlen, m.rope_theta,
                                              m.rope_theta_rescale_factor).to(model.device)

        # Global-attention layers (src/vui/model.py:406-468): without a window every layer is global; with one,
        # the last layer and every global_every-th are.  Global layers attend over the whole cache and may rotate
        # with a table of their own (other width and/or base; the base defaults to theta * max_seqlen / window).
        def _is_global(idx: int) -> bool:
            if m.window_size is None:
                return True
            if m.global_every is not None:
                if idx == m.n_layers - 1 or (idx + 1) % m.global_every == 0:
                    return True
            return False

        self.block_is_global = [_is_global(i) for i in range(m.n_layers)]
        g_dim = m.global_rope_dim or rope_dim
        if m.global_rope_theta is not None:
            g_theta = m.global_rope_theta
        elif m.window_size is not None and any(self.block_is_global):
            g_theta = m.rope_theta * (max_seqlen / m.window_size)
        else:
            g_theta = m.rope_theta
        self.global_rope_dim = g_dim
        self.freqs_cis_global = None
        if g_dim != rope_dim or g_theta != m.rope_theta:
            if g_dim > m.head_dim:
                raise ValueError(f"global_rope_dim={g_dim} exceeds head_dim={m.head_dim}")
            self.freqs_cis_global = precompute_freqs_cis(g_dim, max_seqlen, g_theta,
                                                         m.rope_theta_rescale_factor).to(model.device)
        self.flash_kv_caches: list[FlashKVCache] | None = None
        self._k = self._v = None
        self._prefill_scratch: dict[int, Tensor] = {}  # one buffer per lane (stream) that ingests prompts
        self._prefill_ok: bool | None = None

    def allocate_flash_kv_cache(self, batch_size: int, device, dtype=torch.bfloat16, max_seqlen: int | None = None):
        """src/vui/model.py:473-495.  One allocation per K and V, laid out (layers, slots, S, KV, hd);
        flash_kv_caches[l] holds layer l's (slots, S, KV, hd) views and the shared seq_lens."""
        model = self._model
        if dtype != model.dtype:
            raise ValueError(f"KV cache dtype {dtype} must equal the model dtype {model.dtype}")
        seqlen = max_seqlen or self.max_seqlen
        if seqlen > self.max_seqlen:
            raise ValueError(f"max_seqlen={seqlen} exceeds the RoPE table length {self.max_seqlen}")
        shape = (self.n_layers, batch_size, seqlen, self.n_kv_heads, self.head_dim)
        self._k = torch.zeros(shape, dtype=dtype, device=device)
        self._v = torch.zeros(shape, dtype=dtype, device=device)
        seq_lens = torch.zeros(batch_size, dtype=torch.int32, device=device)
        self.flash_kv_caches = [FlashKVCache(self._k[l], self._v[l], seq_lens) for l in range(self.n_layers)]
        self.kv_seqlen = seqlen
        model._invalidate_graphs()  # captured graphs point into the previous context's workspace
        model._native = _Native(model, batch_size, seqlen)

    def deallocate_kv_cache(self):
        self.flash_kv_caches = None
        self._k = self._v = None

    def _step(self, *, codes: Tensor | None, emb: Tensor | None, slot_idx: Tensor | None, seq_inc: Tensor | None,
              B: int, hidden_out: Tensor | None, cb0_out: Tensor | None, eos_out: Tensor | None, n_splits: int,
              stream: int) -> None:
        if self.flash_kv_caches is None:
            raise RuntimeError("allocate_flash_kv_cache() must be called before decoding")
        nat = self._model._native
        _lib.check(nat.lib.vui_backbone_step(
            nat.handle, _lib.ptr(codes), _lib.ptr(emb), _lib.ptr(slot_idx), self.flash_kv_caches[0].seq_lens.data_ptr(),
            _lib.ptr(seq_inc), B, self._k.data_ptr(), self._v.data_ptr(), _lib.ptr(hidden_out), _lib.ptr(cb0_out),
            _lib.ptr(eos_out), n_splits, stream), "vui_backbone_step")

    def default_splits(self, B: int) -> int:
        """Key-range pieces per (row, head): about 1024 workgroups over the launch (measured on 16 ragged
        rows of 128..2048 keys), at most 32 pieces."""
        H = self._model.config.model.n_heads
        return max(1, min(32, 1024 // max(1, B * H)))

    def forward_flash(self, x: Tensor, positions: Tensor, per_sample_positions: bool = False,
                      slot_idx: Tensor | None = None, known: "tuple[int, int] | None" = None, lane: int = 0) -> Tensor:
        """x (B, T, d) appended at seq_lens[slot]; returns the final-norm output (B, T, d) and advances
        seq_lens by T (src/vui/model.py:534-549).  The native step rotates at the position it writes
        to, so `positions` must be the cache positions (seq_lens .. seq_lens+T-1), as in every
        reference call site (engine.py:683, inference.py:741, model.py:1283)."""
        B, T, d = x.shape
        if B > MAX_BATCH:
            raise ValueError(f"batch {B} > {MAX_BATCH}")
        model = self._model
        if B == 1 and T >= self.PREFILL_MIN and self._prefill_available():
            return self._prefill(x, slot_idx, known, lane)
        out = torch.empty_like(x)
        st = torch.cuda.current_stream().cuda_stream
        ns = self.default_splits(B)
        for t in range(T):
            xt = x[:, t].contiguous()
            ht = torch.empty(B, d, device=x.device, dtype=x.dtype)
            self._step(codes=None, emb=xt, slot_idx=slot_idx, seq_inc=None, B=B, hidden_out=ht, cb0_out=None,
                       eos_out=None, n_splits=ns, stream=st)
            out[:, t] = ht
        return out

    PREFILL_MIN = 4      # shorter blocks go position by position through the decode step
    PREFILL_CHUNK = 1024  # positions per pass: bounds the activation scratch (about 15 KB per position)

    def _prefill_available(self) -> bool:
        """The one-pass form takes bf16 weights and dims that are multiples of 64, head_dim of 32 (the library decides)."""
        if self._prefill_ok is None:
            nat = self._model._native
            self._prefill_ok = nat.lib.vui_prefill_scratch_bytes(C.byref(nat.cfg), 1, 1) >= 0
        return self._prefill_ok

    def _prefill(self, x: Tensor, slot_idx: Tensor | None, known: "tuple[int, int] | None" = None, lane: int = 0) -> Tensor:
        """One row, T positions: the matrix-core pass of the native library, in chunks.  known = (slot, length
        of the slot) from a caller that keeps count: otherwise both are read back from the device.  lane: which
        scratch buffer to use; passes of different rows that run on different streams at once take different lanes."""
        model = self._model
        nat = model._native
        seq_lens = self.flash_kv_caches[0].seq_lens
        if known is not None:
            slot, pos = known
        else:
            slot = 0 if slot_idx is None else int(slot_idx[0])
            pos = int(seq_lens[slot])
        T = x.shape[1]
        if pos + T > self._k.shape[2]:
            raise ValueError(f"prefill of {T} positions at offset {pos} exceeds the cache length {self._k.shape[2]}")
        out = torch.empty_like(x)
        st = torch.cuda.current_stream().cuda_stream
        for t0 in range(0, T, self.PREFILL_CHUNK):
            n = min(self.PREFILL_CHUNK, T - t0)
            need = nat.lib.vui_prefill_scratch_bytes(C.byref(nat.cfg), n, pos + n)
            if need < 0:
                raise RuntimeError(f"vui_prefill_scratch_bytes failed: {_lib.last_error()}")
            buf = self._prefill_scratch.get(lane)
            if buf is None or buf.numel() < need + 256:
                buf = self._prefill_scratch[lane] = torch.empty(need + 256, dtype=torch.uint8, device=x.device)
            base = (buf.data_ptr() + 255) & ~255
            xc = x[0, t0:t0 + n].contiguous()
            _lib.check(nat.lib.vui_prefill(nat.handle, xc.data_ptr(), n, slot, pos, seq_lens.data_ptr(), self._k.data_ptr(),
                                           self._v.data_ptr(), out[0, t0:t0 + n].data_ptr(), base, need, st), "vui_prefill")
            pos += n
        return out


class RQTransformer:
    """Depth head.  Mirrors RQTransformer's generation API (src/vui/model.py:638-1016)."""

    def __init__(self, model: "Vui"):
        m = model.config.model
        self._model = model
        self.rq_dim = m.rq_d_model
        self.n_quantizers = m.n_quantizers
        self.codebook_size = m.codebook_size
        self.seed = 0
        self._gkv_graphs: dict = {}
        self._gkv_batch_sizes: tuple[int, ...] = ()
        self._ctr = torch.zeros(1, dtype=torch.int32, device=model.device)
        self._gkv_dev = None

    def _call(self, hidden, code0, bias, n_q, sp, codes_out, B, stream):
        nat = self._model._native
        _lib.check(nat.lib.vui_rq_generate(nat.handle, hidden.data_ptr(), code0.data_ptr(), _lib.ptr(bias), n_q,
                                           C.byref(sp), codes_out.data_ptr(), codes_out.stride(0), 0, B, stream),
                   "vui_rq_generate")

    @torch.inference_mode()
    def generate(self, backbone_hidden: Tensor, code_0: Tensor, temperature: float = 0.7,
                 top_k: int | None = None, logit_bias: Tensor | None = None) -> Tensor:
        """Eager form (src/vui/model.py:686-728): (B, Q) int64.  The draw uses the library's
        counter-based generator keyed by (self.seed, call number, row, codebook)."""
        B = backbone_hidden.shape[0]
        Q = self.n_quantizers
        out = torch.zeros(B, Q, dtype=torch.long, device=backbone_hidden.device)
        bias = None
        if logit_bias is not None:
            bias = torch.zeros(Q - 1, self.codebook_size, dtype=torch.float32, device=out.device)
            bias[: logit_bias.size(0)].copy_(logit_bias)
        sp = make_sample_params(temperature, top_k, self.seed, self._ctr)
        st = torch.cuda.current_stream().cuda_stream
        for b0 in range(0, B, MAX_BATCH):
            nb = min(MAX_BATCH, B - b0)
            self._call(backbone_hidden[b0:b0 + nb].contiguous(), code_0[b0:b0 + nb].contiguous(), bias, Q, sp,
                       out[b0:], nb, st)
            self._ctr.add_(1)  # a new draw index per call (and per 16-row chunk of a large batch)
        return out

    def generate_kv_compilable(self, backbone_hidden: Tensor, code_0: Tensor, temperature, logit_bias: Tensor,
                               top_k: int = 100) -> Tensor:
        """The entry the reference hands to torch.compile (src/vui/model.py:730-811; temperature as a tensor,
        logit_bias always given, top_k a Python int).  There is no compiler here: it is the eager form on the same
        kernels, and a temperature tensor is read on the host (one synchronisation per distinct call site; callers
        in a loop pass a float, as InferenceState's wrapper does)."""
        t = float(temperature.item()) if isinstance(temperature, Tensor) else float(temperature)
        return self.generate(backbone_hidden, code_0, t, top_k, logit_bias)

    def setup_cuda_graph_kv(self, device, dtype=torch.bfloat16, top_k: int = 100, pool=None,
                            batch_sizes: tuple[int, ...] = (1,)):
        """Static buffers for graph replay at the given batch sizes (src/vui/model.py:814-881).
        Graphs are captured on first use of a (batch, Q', temperature) combination."""
        Q = self.n_quantizers
        self._gkv_top_k = top_k
        self._gkv_batch_sizes = tuple(sorted(set(batch_sizes)))
        B_max = max(self._gkv_batch_sizes)
        if B_max > MAX_BATCH:
            raise ValueError(f"batch size {B_max} > {MAX_BATCH}")
        self._gkv_backbone = torch.zeros(B_max, self._model.config.model.d_model, device=device, dtype=dtype)
        self._gkv_code0 = torch.zeros(B_max, device=device, dtype=torch.long)
        self._gkv_logit_bias = torch.zeros(Q - 1, self.codebook_size, device=device, dtype=torch.float32)
        self._gkv_codes_out = torch.zeros(B_max, Q, device=device, dtype=torch.long)
        self._gkv_graphs = {}

    def generate_cuda_graph_kv(self, backbone_hidden: Tensor, code_0: Tensor, temperature: float = 0.7,
                               logit_bias: Tensor | None = None, n_quantizers: int = 0) -> Tensor:
        """(B, Q') int64 VIEW of the static output buffer (src/vui/model.py:988-1016)."""
        B = backbone_hidden.shape[0]
        Q = n_quantizers if n_quantizers > 0 else self.n_quantizers
        if B not in self._gkv_batch_sizes or not (2 <= Q <= self.n_quantizers):
            raise KeyError(f"No RQ CUDA graph captured for batch_size={B}, Q={Q}. "
                           f"Call setup_cuda_graph_kv(batch_sizes=(1,2,4,...)) to capture.")
        self._gkv_backbone[:B].copy_(backbone_hidden)
        self._gkv_code0[:B].copy_(code_0)
        self._gkv_logit_bias.zero_()
        if logit_bias is not None:
            self._gkv_logit_bias[: logit_bias.size(0)].copy_(logit_bias)
        # temperature, top-k and seed sit in a device block that the captured launch reads at each replay (the
        # reference fills a 0-d temperature tensor before its replay, model.py:1011): one graph per (B, Q')
        if self._gkv_dev is None:
            self._gkv_dev = SampleDev(self._gkv_codes_out.device)
        self._gkv_dev.set(temperature, self._gkv_top_k, self.seed)
        key = (B, Q)
        g = self._gkv_graphs.get(key)
        if g is None:
            sp = make_sample_params(temperature, self._gkv_top_k, self.seed, self._ctr, dev=self._gkv_dev)
            g = Graph(self._model, lambda st: self._call(self._gkv_backbone, self._gkv_code0, self._gkv_logit_bias,
                                                         Q, sp, self._gkv_codes_out, B, st))
            g._sp = sp
            self._gkv_graphs[key] = g
        g.replay()
        self._ctr.add_(1)
        return self._gkv_codes_out[:B, :Q]


class Vui:
    """Model shell.  Mirrors Vui in src/vui/model.py:1054-1311 for inference."""

    VUI2 = "vui-nano.safetensors"

    def __init__(self, config: Config, state_dict: dict[str, Tensor], device="cuda", dtype=torch.bfloat16,
                 int8: bool = False):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("dtype must be bfloat16 or float32")
        self.config = config
        self.device = torch.device(device)
        self.dtype = dtype
        self.int8 = int8
        cfg = config.model
        self.use_rotary_emb = cfg.use_rotary_emb
        self.sd = {k: (v.to(self.device, dtype).contiguous() if v.is_floating_point() else v.to(self.device))
                   for k, v in state_dict.items()}
        sd = self.sd
        if not cfg.vocab_size:
            cfg.vocab_size = sd["token_emb.weight"].shape[0]
        self.q8 = {}
        if int8:
            for i in range(cfg.n_layers):
                for nm in ("attn.Wqkv", "attn.out_proj", "mlp.w1", "mlp.w3", "mlp.w2"):
                    key = f"decoder.blocks.{i}.{nm}.weight"
                    self.q8[key] = quantize_int8(sd[key])
        self.token_emb = _Embedding(sd["token_emb.weight"])
        self.audio_emb = AudioEmbedding(cfg.n_quantizers, cfg.codebook_size, sd["audio_emb.embedding.weight"])
        self.codec_head = _Linear(sd["codec_head.weight"])
        self.eos_head = _Linear(sd["eos_head.weight"], sd["eos_head.bias"])
        self.spk_proj = _Linear(sd["spk_proj.weight"]) if "spk_proj.weight" in sd else None
        max_seqlen = config.max_seq_len if config.max_seq_len > 0 else cfg.max_text_tokens + cfg.max_audio_tokens
        self._cap_stream = torch.cuda.Stream(device=self.device)
        self.decoder = Decoder(self, max_seqlen + cfg.n_quantizers)
        self.rq_transformer = RQTransformer(self) if cfg.use_rq_transformer else None
        self._cond_bias = torch.zeros(1, 1, cfg.d_model, device=self.device, dtype=dtype)
        self._native = _Native(self, 1, self.decoder.max_seqlen)
        self._decode_graph = None

    # -- construction ------------------------------------------------------------------
    @staticmethod
    def from_pretrained(checkpoint_path: str | dict, device="cuda", dtype=torch.float32, **config_kwargs) -> "Vui":
        """Local checkpoints only: a dict {"config", "model"}, a .safetensors file whose metadata
        carries the JSON config, or a torch file loaded with weights_only=True
        (src/vui/model.py:1154-1219)."""
        if isinstance(checkpoint_path, dict):
            config = {**checkpoint_path["config"], **config_kwargs}
            state_dict = checkpoint_path["model"]
        else:
            if not os.path.exists(checkpoint_path):
                raise FileNotFoundError(f"{checkpoint_path}: only local checkpoints can be loaded")
            if checkpoint_path.endswith(".safetensors"):
                from safetensors.torch import load_file, safe_open

                with safe_open(checkpoint_path, framework="pt") as f:
                    metadata = f.metadata()
                config = {**json.loads(metadata["config"]), **config_kwargs}
                state_dict = load_file(checkpoint_path)
            else:
                ck = torch.load(checkpoint_path, map_location="cpu", weights_only=True)
                config = {**ck["config"], **config_kwargs}
                state_dict = ck["model"]
        state_dict = {k.replace("module.", "").replace("text_embedding.", "token_emb."): v
                      for k, v in state_dict.items()}
        # older checkpoints carry the optional projections without their config flags
        # (infer_optional_modules, src/vui/config.py:81-101); a flag present in the config wins
        mcfg = dict(config.get("model") or {})
        for flag, sentinel in (("has_sq_proj", "sq_proj.proj.0.weight"), ("has_wps_proj", "wps_proj.proj.0.weight"),
                               ("has_spk_proj", "spk_proj.weight")):
            if sentinel in state_dict and flag not in mcfg:
                mcfg[flag] = True
        cfg = Config.from_dict({**config, "model": mcfg})
        return Vui(cfg, state_dict, device=device, dtype=dtype)

    @staticmethod
    def from_pretrained_inf(checkpoint_path: str | dict, device="cuda", **config_kwargs) -> "Vui":
        """bf16 inference model (src/vui/model.py:1221-1226)."""
        return Vui.from_pretrained(checkpoint_path, device=device, dtype=torch.bfloat16, **config_kwargs)

    def _invalidate_graphs(self):
        self._decode_graph = None
        if self.rq_transformer is not None:
            self.rq_transformer._gkv_graphs = {}

    # -- B=1 decode graph ----------------------------------------------------------------
    def setup_decode_graph(self, pool=None):
        """src/vui/model.py:1228-1256: a one-slot KV cache, static in/out buffers and the captured step."""
        cfg = self.config.model
        dev, dt = self.device, self.dtype
        self.decoder.allocate_flash_kv_cache(1, dev, dt)
        self._decode_code_in = torch.zeros(cfg.n_quantizers, device=dev, dtype=torch.long)
        self._decode_hidden_out = torch.zeros(1, cfg.d_model, device=dev, dtype=dt)
        self._decode_codec_logits = torch.zeros(1, cfg.codebook_size, device=dev, dtype=dt)
        self._decode_eos_logit = torch.zeros(1, 1, device=dev, dtype=dt)
        seq_lens = self.decoder.flash_kv_caches[0].seq_lens
        ns = self.decoder.default_splits(1)

        def body(st):
            self.decoder._step(codes=self._decode_code_in, emb=None, slot_idx=None, seq_inc=None, B=1,
                               hidden_out=self._decode_hidden_out, cb0_out=self._decode_codec_logits,
                               eos_out=self._decode_eos_logit, n_splits=ns, stream=st)

        self._decode_graph = Graph(self, body)
        seq_lens.zero_()

    @torch.inference_mode()
    def decode_step(self, codes: Tensor, pos: int) -> tuple[Tensor, Tensor, Tensor]:
        """src/vui/model.py:1289-1300: returns the static (hidden, codec logits, eos logit) buffers."""
        if self._decode_graph is None:
            raise RuntimeError("setup_decode_graph() must be called first")
        self._decode_code_in.copy_(codes)
        self.decoder.flash_kv_caches[0].seq_lens[:1].fill_(pos)
        self._decode_graph.replay()
        return self._decode_hidden_out, self._decode_codec_logits, self._decode_eos_logit

    # -- conditioning --------------------------------------------------------------------
    def embed_audio(self, codes: Tensor) -> Tensor:
        return self.audio_emb(codes)

    def embed_speaker(self, spk_emb: Tensor) -> Tensor:
        """(1, 1, d) speaker token for prefill (src/vui/model.py:1276-1278)."""
        if self.spk_proj is None:
            raise RuntimeError("checkpoint has no spk_proj")
        return self.spk_proj(spk_emb.to(self.device, self.dtype).reshape(1, -1)).reshape(1, 1, -1)

    def set_cond_bias(self, sq_scores=None, wps_score: float = 0.0):
        """src/vui/model.py:1258-1274.  The SQ/WPS projection heads are not part of the decode step;
        without them the bias stays zero, as in the reference when the modules are absent."""
        self._cond_bias.zero_()
        if "sq_proj.weight" in self.sd and sq_scores is not None:
            v = torch.tensor([sq_scores], device=self.device, dtype=self.dtype)
            self._cond_bias.add_(F.linear(v, self.sd["sq_proj.weight"]).reshape(1, 1, -1))
