"""CPU oracle for the Vui per-frame decode step.  TEST INFRASTRUCTURE ONLY.

This file restates, with plain PyTorch CPU ops, the arithmetic of the reference's
per-frame decode path so that the HIP kernels can be checked against it.  Only tests,
the smoke check and the CPU-baseline leg of the benchmark may import it; the product
package never does.

Every function cites the reference lines it follows (paths relative to the reference
checkout, `src/vui/...`).  Two arithmetic regimes are provided:

* ``dt=torch.float32`` - the reference's CPU regime: no intermediate rounding.
* ``dt=torch.bfloat16`` - the reference's GPU regime: every value the reference
  materialises as a bf16 tensor is rounded to bf16 here at the same point, while the
  accumulations stay fp32.  Tensors are carried as fp32 holding bf16-representable values.

How each function is pinned (see tests/test_oracle_golden.py, tests/test_oracle_math.py):

* precompute_freqs_cis, apply_rotary_emb, rmsnorm, audio_embedding, backbone forward
  (prefill + decode against the reference's SDPA/KVCache path), rq_forward, rq_generate
  (full-recompute and KV-cached forms), sample_top_k_probs, the 64x16 greedy token grid:
  golden vectors written from the reference's own classes by tests/golden/make_golden.py.
* attention: additionally brute force against an explicit softmax on tiny sizes.
* philox4x32_10: Random123 known-answer vectors.
* sample_rq / sample_cb0 selection rule: exhaustive small cases (ties at the k-th place kept
  by the depth-head rule, cut to exactly k in index order by the code-0 rule) + chi-square against
  the analytic top-k softmax; the *random stream* itself has no counterpart in the reference
  (torch.multinomial's CUDA generator is third-party) -> "parity unpinned" for the
  drawn token under sampling, pinned for greedy.
* top_p_probs / top_p_top_k_probs (nucleus cut, alone and with top-k): brute force over every ordering of small
  probability vectors written out as exact binary fractions, including mass exactly at top_p, ties
  across the boundary and top_p >= 1; parity of which of several EQUAL probabilities survives is
  unpinned (torch.sort leaves it open), the lowest indices are kept.
* rep_penalty: closed form + ring-buffer invariant (counts == histogram of the window).
* int8 weight-only quantisation: closed form (scale = max|w|/127 per output row); the
  format is defined by the benchmark config, it has no reference implementation on this
  path -> "parity unpinned" against the reference, pinned against dequantise-then-matmul.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np
import torch
import torch.nn.functional as F

Tensor = torch.Tensor


# --------------------------------------------------------------------------------------
# dims
# --------------------------------------------------------------------------------------
@dataclass
class Dims:
    """Architecture numbers (reference: src/vui/config.py:16-52, model.py:1061-1136)."""

    d_model: int = 768
    n_layers: int = 22
    n_heads: int = 8
    n_kv_heads: int = 8
    intermediate_size: int | None = None
    n_quantizers: int = 16
    codebook_size: int = 2048
    rq_d_model: int = 512
    rq_n_layers: int = 4
    rq_n_heads: int = 8
    vocab_size: int = 100554
    max_seqlen: int = 10576
    rope_dim: int | None = None
    rope_theta: float = 10000.0
    rope_theta_rescale_factor: float = 1.0
    norm_eps: float = 1e-5  # Decoder default, model.py:391
    rq_norm_eps: float = 1e-6  # RMSNorm default used by RQBlock, model.py:287,583
    # sliding window and global-attention layers (config.py:36-41, model.py:396-468)
    window_size: int | None = None
    global_every: int | None = None
    global_rope_dim: int | None = None
    global_rope_theta: float | None = None
    trained_max_seqlen: int | None = None  # Decoder.max_seqlen, the length the global base is derived from

    def block_is_global(self) -> list[bool]:
        """model.py:406-418: without a window every layer is global; with one, the last layer and every
        global_every-th are."""
        def g(idx: int) -> bool:
            if self.window_size is None:
                return True
            if self.global_every is not None:
                if idx == self.n_layers - 1 or (idx + 1) % self.global_every == 0:
                    return True
            return False
        return [g(i) for i in range(self.n_layers)]

    def global_rope(self, max_seqlen: int):
        """(dim, theta) of the global layers' own table or None when they share the common one (model.py:449-468)."""
        rope_dim = self.rope_dim or self.head_dim
        g_dim = self.global_rope_dim or rope_dim
        if self.global_rope_theta is not None:
            g_theta = self.global_rope_theta
        elif self.window_size is not None and any(self.block_is_global()):
            g_theta = self.rope_theta * (max_seqlen / self.window_size)
        else:
            g_theta = self.rope_theta
        if g_dim != rope_dim or g_theta != self.rope_theta:
            return g_dim, g_theta
        return None

    @property
    def head_dim(self) -> int:
        return self.d_model // self.n_heads

    @property
    def ffn(self) -> int:
        # model.py:272-277
        if self.intermediate_size is not None:
            return self.intermediate_size
        h = 4 * self.d_model
        h = int(2 * h / 3)
        return 256 * ((h + 255) // 256)

    @property
    def rq_ffn(self) -> int:
        # model.py:587-588
        h = int(self.rq_d_model * 8 / 3)
        return 64 * ((h + 63) // 64)

    @property
    def rq_head_dim(self) -> int:
        return self.rq_d_model // self.rq_n_heads


def rnd(t: Tensor, dt: torch.dtype) -> Tensor:
    """Round to `dt` and come back to fp32 (identity for fp32)."""
    if dt == torch.float32:
        return t.float()
    return t.to(dt).float()


# --------------------------------------------------------------------------------------
# elementary pieces
# --------------------------------------------------------------------------------------
def precompute_freqs_cis(dim: int, max_seqlen: int, theta: float = 10000.0,
                         theta_rescale_factor: float = 1.0) -> Tensor:
    """cos/sin table (max_seqlen, dim, 2) fp32, each frequency repeated twice.

    Reference: rope.py:60-77.  theta <- theta * rescale**(dim/(dim-2)); angle(p, i) =
    p * theta**(-(2*(i//2))/dim).
    """
    theta = theta * theta_rescale_factor ** (dim / (dim - 2))
    pos = torch.arange(max_seqlen, dtype=torch.float32)
    inv = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))
    fr = pos[:, None] * inv[None, :]
    fr = fr.repeat_interleave(2, dim=-1)
    return torch.stack((fr.cos(), fr.sin()), dim=-1)


def apply_rotary_emb(freqs: Tensor, t: Tensor, dt: torch.dtype) -> Tensor:
    """Interleaved (GPT-J) rotation of the first rot_dim features.

    Reference: rope.py:16-57.  `freqs` (..., rot_dim, 2) is already gathered per position
    and broadcast against `t` (..., head_dim).  fp32 arithmetic, one rounding at the end.
    """
    rot = freqs.shape[-2]
    cos, sin = freqs[..., 0], freqs[..., 1]
    x = t[..., :rot].float()
    x1, x2 = x[..., 0::2], x[..., 1::2]
    rh = torch.stack((-x2, x1), dim=-1).flatten(-2)
    out = x * cos + rh * sin
    if rot < t.shape[-1]:
        out = torch.cat((out, t[..., rot:].float()), dim=-1)
    return rnd(out, dt)


def rmsnorm(x: Tensor, w: Tensor, eps: float, dt: torch.dtype) -> Tensor:
    """Reference: model.py:286-297.  Normalise in fp32, round, scale by weight, round."""
    xf = x.float()
    n = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return rnd(rnd(n, dt) * w.float(), dt)


def linear(x: Tensor, W: Tensor, dt: torch.dtype, bias: Tensor | None = None) -> Tensor:
    """y = x W^T (+ b): fp32 accumulate over `dt`-valued operands, one rounding."""
    y = x.float() @ W.float().t()
    if bias is not None:
        y = y + bias.float()
    return rnd(y, dt)


def swiglu(x: Tensor, w1: Tensor, w3: Tensor, w2: Tensor, dt: torch.dtype) -> Tensor:
    """Reference: model.py:282-283 (and 610).  w2(silu(w1 x) * w3 x), rounding after each op."""
    a = linear(x, w1, dt)
    b = linear(x, w3, dt)
    s = rnd(F.silu(a), dt)
    return linear(rnd(s * b, dt), w2, dt)


def audio_embedding(table: Tensor, codes: Tensor, codebook_size: int, dt: torch.dtype) -> Tensor:
    """Sum over the last axis of table[codes[..., q] + q*CS].  Reference: model.py:559-563.

    The sum accumulates in fp32 and rounds once (torch's bf16 reduction does the same).
    """
    Q = codes.shape[-1]
    off = torch.arange(Q) * codebook_size
    rows = table.float()[codes + off]
    return rnd(rows.sum(dim=-2), dt)


def attention(q: Tensor, k: Tensor, v: Tensor, scale: float, dt: torch.dtype,
              mask: Tensor | None = None) -> Tensor:
    """softmax(q k^T * scale + mask) v with fp32 scores/probabilities, one output rounding.

    q (..., Tq, hd), k/v (..., Tk, hd).  Stands for flash_attn_with_kvcache
    (model.py:247-257) and F.scaled_dot_product_attention (model.py:191-198, 630, 901).
    """
    s = (q.float() @ k.float().transpose(-1, -2)) * scale
    if mask is not None:
        s = s.masked_fill(~mask, float("-inf"))
    p = torch.softmax(s, dim=-1)
    return rnd(p @ v.float(), dt)


# --------------------------------------------------------------------------------------
# counter-based random numbers
# --------------------------------------------------------------------------------------
_PH_M0, _PH_M1 = 0xD2511F53, 0xCD9E8D57
_PH_W0, _PH_W1 = 0x9E3779B9, 0xBB67AE85


def philox4x32_10(counter, key):
    """Philox-4x32 with 10 rounds (Salmon et al., SC'11; Random123).  Returns 4 uint32."""
    c = [int(x) & 0xFFFFFFFF for x in counter]
    k = [int(x) & 0xFFFFFFFF for x in key]
    for _ in range(10):
        p0 = _PH_M0 * c[0]
        p1 = _PH_M1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & 0xFFFFFFFF, p1 & 0xFFFFFFFF,
             ((p0 >> 32) ^ c[3] ^ k[1]) & 0xFFFFFFFF, p0 & 0xFFFFFFFF]
        k = [(k[0] + _PH_W0) & 0xFFFFFFFF, (k[1] + _PH_W1) & 0xFFFFFFFF]
    return c


def uniform01(seed: int, frame: int, row: int, codebook: int) -> float:
    """The uniform in [0,1) that the device sampler draws for (seed, frame, row, codebook).

    key = (seed low 32, seed high 32); counter = (frame, row, codebook, 0); the top 24 bits
    of the first output word, scaled by 2^-24 (exact in fp32).
    """
    out = philox4x32_10((frame, row, codebook, 0), (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))
    return (out[0] >> 8) * (1.0 / 16777216.0)


# --------------------------------------------------------------------------------------
# samplers
# --------------------------------------------------------------------------------------
def _inverse_cdf(p: np.ndarray, u: float) -> int:
    """Smallest index whose running sum (index order, float64) exceeds u * total."""
    c = np.cumsum(p.astype(np.float64))
    j = int(np.searchsorted(c, u * c[-1], side="right"))
    if j >= len(p):  # only reachable through rounding when u is within 2^-24 of 1
        j = int(np.nonzero(p > 0)[0][-1])
    return j


def topk_threshold_probs(logits: Tensor, temperature: float, top_k: int) -> np.ndarray:
    """Unnormalised kept weights of the RQ-head sampler.  Reference: model.py:955-961.

    logits (CS,) fp32 (bias already added); /temperature; values below the k-th largest are
    dropped (ties with the k-th are kept); exp(l - max).  top_k <= 0 keeps everything.
    """
    l = logits.float() / temperature
    if top_k > 0:
        kth = torch.topk(l, min(top_k, l.numel())).values[-1]
        l = torch.where(l < kth, torch.full_like(l, float("-inf")), l)
    return torch.exp(l - l.max()).numpy()


def sample_rq(logits: Tensor, temperature: float, top_k: int, u: float) -> int:
    """One draw of the RQ-head sampler (model.py:955-962) with the uniform `u`.

    top_k == 1 (or temperature <= 0) is greedy: the lowest index attaining the maximum.
    """
    if top_k == 1 or temperature <= 0:
        return int(torch.argmax(logits.float()))
    return _inverse_cdf(topk_threshold_probs(logits, temperature, top_k), u)


def rep_penalise(logits: Tensor, counts: Tensor, penalty: float) -> Tensor:
    """Reference: engine.py:571-576.  factor = penalty**count; positive logits are divided."""
    if penalty <= 1.0:
        return logits.float()
    lf = logits.float()
    factor = torch.pow(torch.tensor(penalty, dtype=torch.float32), counts.float())
    return torch.where(lf > 0, lf / factor, lf * factor)


def cb0_probs(logits: Tensor, temperature: float, top_k: int) -> np.ndarray:
    """Kept weights of the code-0 sampler.  Reference: engine.py:855-863, 1456-1464.

    softmax(logits/T) in fp32, then exactly top_k probabilities are kept (topk + scatter) and
    renormalised.  Where several probabilities tie at the k-th place torch.topk's choice among
    them is unspecified; here, and on the device, the lowest indices among the tied are kept.
    """
    p = torch.softmax(logits.float() / temperature, dim=-1)
    if top_k is not None and 0 < top_k < p.numel():
        order = torch.sort(p, descending=True, stable=True).indices[:top_k]  # stable: ties in index order
        kept = torch.zeros_like(p)
        kept[order] = p[order]
        p = kept
    return p.numpy()


def top_p_probs(probs: Tensor, p: float) -> Tensor:
    """sampling.sample_top_p's kept weights, in index order (src/vui/sampling.py:23-31): probabilities sorted
    largest first, an entry is dropped when the cumulative sum strictly ahead of it exceeds p
    (`probs_sum - probs_sort > p`), the rest renormalised.  torch.sort leaves the order of equal probabilities
    open; here (and on the device) equal ones go by index (stable sort)."""
    ps, idx = torch.sort(probs.float(), dim=-1, descending=True, stable=True)
    csum = torch.cumsum(ps, dim=-1)
    ps = ps * (~(csum - ps > p)).float()
    ps = ps / ps.sum(dim=-1, keepdim=True)
    out = torch.zeros_like(ps)
    out[idx] = ps
    return out


def top_p_top_k_probs(probs: Tensor, p: float, top_k: int) -> Tensor:
    """sampling.sample_top_p_top_k's kept weights, in index order (src/vui/sampling.py:34-43): the nucleus as
    above, then sample_top_k on the renormalised sorted vector (everything >= its k-th largest entry)."""
    ps, idx = torch.sort(probs.float(), dim=-1, descending=True, stable=True)
    csum = torch.cumsum(ps, dim=-1)
    ps = ps * (~(csum - ps > p)).float()
    ps = ps / ps.sum(dim=-1, keepdim=True)
    kth = torch.topk(ps, min(top_k, ps.numel())).values[-1]
    ps = ps * (ps >= kth).float()
    out = torch.zeros_like(ps)
    out[idx] = ps
    return out


def sample_codes_probs(logits: Tensor, temperature: float, top_k: "int | None", top_p: "float | None") -> np.ndarray:
    """Kept, unnormalised weights (index order) of inference._sample_codes (src/vui/inference.py:491-504), which
    picks among sampling.py's rules: sample_top_p_top_k (both given), sample_top_p (top_p alone and > 0),
    sample_top_k (ties with the k-th largest kept), or the plain softmax."""
    probs = torch.softmax(logits.float() / temperature, dim=-1)
    if top_p is not None and top_k is not None:
        return top_p_top_k_probs(probs, top_p, top_k).numpy()
    if top_p is not None and top_p > 0:
        return top_p_probs(probs, top_p).numpy()
    if top_k is not None and top_k > 0:
        kth = torch.topk(probs, min(top_k, probs.numel())).values[-1]
        probs = probs * (probs >= kth).float()
    return probs.numpy()


def sample_codes(logits: Tensor, temperature: float, top_k: "int | None", top_p: "float | None", u: float) -> int:
    """One draw of inference._sample_codes with the uniform `u` (inverse CDF in index order over the kept set)."""
    return _inverse_cdf(sample_codes_probs(logits, temperature, top_k, top_p), u)


def sample_cb0(logits: Tensor, counts: Tensor, penalty: float, temperature: float,
               top_k: int, u: float) -> int:
    l = rep_penalise(logits, counts, penalty)
    if top_k == 1 or temperature <= 0:
        return int(torch.argmax(l))
    return _inverse_cdf(cb0_probs(l, temperature, top_k), u)


class RepState:
    """Rolling code-0 history of one row.  Reference: engine.py:540-590."""

    def __init__(self, codebook_size: int, window: int):
        self.counts = torch.zeros(codebook_size, dtype=torch.float32)
        self.window = window
        self.hist = [0] * max(window, 1)
        self.head = 0
        self.filled = 0

    def push(self, code: int) -> None:
        if self.window > 0:
            if self.filled == self.window:
                self.counts[self.hist[self.head]] -= 1
            self.hist[self.head] = code
            self.head = (self.head + 1) % self.window
            if self.filled < self.window:
                self.filled += 1
        self.counts[code] += 1


# --------------------------------------------------------------------------------------
# int8 weight-only format of the benchmark's quantised config
# --------------------------------------------------------------------------------------
def quantize_int8(W: Tensor):
    """Symmetric per-output-channel int8: scale = max|w_row|/127 rounded to bf16,
    q = clamp(round(w/scale), -127, 127).  Returns (q int8, scale as fp32 holding bf16)."""
    Wf = W.float()
    s = (Wf.abs().amax(dim=1) / 127.0).clamp_min(1e-12)
    s = s.to(torch.bfloat16).float()
    q = torch.clamp(torch.round(Wf / s[:, None]), -127, 127).to(torch.int8)
    return q, s


def linear_int8(x: Tensor, q: Tensor, s: Tensor, dt: torch.dtype) -> Tensor:
    """y[n] = s[n] * sum_k q[n,k] x[k]  (fp32 accumulate, scale applied once per row)."""
    return rnd((x.float() @ q.float().t()) * s.float(), dt)


# --------------------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------------------
class OracleModel:
    """Backbone + RQ depth head on CPU from a reference-keyed state dict.

    State-dict keys are the reference's (model.py:1076-1136, 577-663).
    """

    def __init__(self, dims: Dims, sd: dict[str, Tensor], dt: torch.dtype = torch.float32,
                 n_slots: int = 1, max_seqlen: int | None = None, int8: bool = False, apply_window: bool = True):
        """apply_window=False restates the reference's CPU path (SDPA + KVCache, model.py:146-202), which ignores
        window_size; True the engine's path, where flash-attn applies it per layer (model.py:242-257)."""
        self.dims = dims
        self.apply_window = apply_window
        self.dt = dt
        self.sd = {k: rnd(v, dt) if v.is_floating_point() else v for k, v in sd.items()}
        self.S = max_seqlen or dims.max_seqlen
        d = dims
        rope_dim = d.rope_dim or d.head_dim
        self.freqs = precompute_freqs_cis(rope_dim, self.S, d.rope_theta, d.rope_theta_rescale_factor)
        # per-layer window and rotation table (Decoder._get_freqs model.py:504-509; MHA.forward_flash's window, :256)
        self.is_global = d.block_is_global()
        gr = d.global_rope(d.trained_max_seqlen or d.max_seqlen)
        self.freqs_global = (precompute_freqs_cis(gr[0], self.S, gr[1], d.rope_theta_rescale_factor)
                             if gr is not None else None)
        # FlashKVCache layout (slots, S, KV, hd); one seq_lens shared by all layers (model.py:71-99,492-495)
        self.k_cache = torch.zeros(d.n_layers, n_slots, self.S, d.n_kv_heads, d.head_dim)
        self.v_cache = torch.zeros_like(self.k_cache)
        self.seq_lens = torch.zeros(n_slots, dtype=torch.int32)
        self.int8 = int8
        self.q8 = {}
        if int8:
            for i in range(d.n_layers):
                for nm in ("attn.Wqkv", "attn.out_proj", "mlp.w1", "mlp.w3", "mlp.w2"):
                    key = f"decoder.blocks.{i}.{nm}.weight"
                    self.q8[key] = quantize_int8(self.sd[key])

    # -- linears (bf16/fp32 or int8 weight-only) --
    def _lin(self, x: Tensor, key: str) -> Tensor:
        if self.int8 and key in self.q8:
            q, s = self.q8[key]
            return linear_int8(x, q, s, self.dt)
        return linear(x, self.sd[key], self.dt)

    # -- backbone ---------------------------------------------------------------------
    def forward_flash(self, x: Tensor, slots: Tensor, n_new: int = 1) -> Tensor:
        """T = n_new new positions per row appended at seq_lens[slot]; returns final-norm output.

        x (B, T, d).  Reference: Decoder.forward_flash model.py:534-549, Block.forward_flash
        :359-375, MHA.forward_flash :204-258 (cache append at cache_seqlens, causal attention
        over everything up to and including each new position, slot indirection via
        cache_batch_idx), and the equivalent SDPA path :146-202, 511-532.
        """
        d, dt, sd = self.dims, self.dt, self.sd
        B, T, _ = x.shape
        H, KV, hd = d.n_heads, d.n_kv_heads, d.head_dim
        x = rnd(x, dt)
        start = self.seq_lens[slots.long()].long()  # (B,)
        pos = start[:, None] + torch.arange(T)[None, :]  # (B, T)
        for li in range(d.n_layers):
            p = f"decoder.blocks.{li}."
            table = self.freqs_global if (self.freqs_global is not None and self.is_global[li]) else self.freqs
            fr = table[pos]  # (B, T, rot, 2)
            win = None if (self.is_global[li] or not self.apply_window) else d.window_size  # (w, 0): keys i-w .. i
            h = rmsnorm(x, sd[p + "attn_norm.weight"], d.norm_eps, dt)
            qkv = self._lin(h, p + "attn.Wqkv.weight")
            q, k, v = torch.split(qkv, [H * hd, KV * hd, KV * hd], dim=-1)
            q = q.view(B, T, H, hd)
            k = k.view(B, T, KV, hd)
            v = v.view(B, T, KV, hd)
            q = apply_rotary_emb(fr[:, :, None], q, dt)
            k = apply_rotary_emb(fr[:, :, None], k, dt)
            outs = []
            for b in range(B):
                s, st = int(slots[b]), int(start[b])
                self.k_cache[li, s, st:st + T] = k[b]
                self.v_cache[li, s, st:st + T] = v[b]
                L = st + T
                kk = self.k_cache[li, s, :L].transpose(0, 1)  # (KV, L, hd)
                vv = self.v_cache[li, s, :L].transpose(0, 1)
                if H != KV:  # repeat_kv, model.py:102-110
                    kk = kk.repeat_interleave(H // KV, dim=0)
                    vv = vv.repeat_interleave(H // KV, dim=0)
                qq = q[b].transpose(0, 1)  # (H, T, hd)
                qpos = (st + torch.arange(T))[:, None]
                mask = torch.arange(L)[None, :] <= qpos  # (T, L)
                if win:
                    mask = mask & (torch.arange(L)[None, :] >= qpos - win)
                o = attention(qq, kk, vv, hd ** -0.5, dt, mask[None])
                outs.append(o.transpose(0, 1).reshape(T, H * hd))
            a = torch.stack(outs)
            x = rnd(x + self._lin(a, p + "attn.out_proj.weight"), dt)
            h2 = rmsnorm(x, sd[p + "mlp_norm.weight"], d.norm_eps, dt)
            a1 = self._lin(h2, p + "mlp.w1.weight")
            a3 = self._lin(h2, p + "mlp.w3.weight")
            g = rnd(rnd(F.silu(a1), dt) * a3, dt)
            x = rnd(x + self._lin(g, p + "mlp.w2.weight"), dt)
        return rmsnorm(x, sd["decoder.norm.weight"], d.norm_eps, dt)

    def advance(self, slots: Tensor, n: int = 1) -> None:
        for s in slots.tolist():
            self.seq_lens[s] += n

    def embed_audio(self, codes: Tensor) -> Tensor:
        return audio_embedding(self.sd["audio_emb.embedding.weight"], codes,
                               self.dims.codebook_size, self.dt)

    def embed_text(self, ids: Tensor) -> Tensor:
        return self.sd["token_emb.weight"][ids]

    def heads(self, hidden: Tensor):
        """codec_head / eos_head.  Reference: engine.py:445-448, model.py:1083,1099."""
        cb0 = linear(hidden, self.sd["codec_head.weight"], self.dt)
        eos = linear(hidden, self.sd["eos_head.weight"], self.dt, self.sd["eos_head.bias"])
        return cb0, eos

    def decode_step(self, codes: Tensor, slots: Tensor | None = None):
        """One backbone step for B rows: codes (B, Q') zero-padded to Q (engine.py:473-479).

        Reference: Engine._backbone_decode_body[_b] engine.py:434-449, 485-502.
        Returns hidden (B,d), cb0 logits (B,CS), eos logit (B,1); advances seq_lens.
        """
        B = codes.shape[0]
        Q = self.dims.n_quantizers
        if codes.shape[1] < Q:
            codes = torch.cat([codes, torch.zeros(B, Q - codes.shape[1], dtype=codes.dtype)], 1)
        if slots is None:
            slots = torch.arange(B)
        emb = self.embed_audio(codes)[:, None]
        hidden = self.forward_flash(emb, slots)[:, 0]
        self.advance(slots)
        cb0, eos = self.heads(hidden)
        return hidden, cb0, eos

    def prefill(self, emb: Tensor, slot: int = 0) -> Tensor:
        """Reference: Engine._prefill_emb engine.py:674-694.  emb (T, d) -> (T, d)."""
        s = torch.tensor([slot])
        out = self.forward_flash(emb[None], s, emb.shape[0])[0]
        self.advance(s, emb.shape[0])
        return out

    # -- RQ depth head ------------------------------------------------------------------
    def _rq_block(self, li: int, x: Tensor, k_all: Tensor | None, v_all: Tensor | None, causal: bool):
        """RQBlock on x (B,T,R).  If k_all/v_all are given they are the earlier positions'
        keys/values (B,P,h,hd) and the new ones are appended.  Reference: model.py:599-635."""
        d, dt, sd = self.dims, self.dt, self.sd
        p = f"rq_transformer.blocks.{li}."
        B, T, R = x.shape
        nh, hd = d.rq_n_heads, d.rq_head_dim
        h = rmsnorm(x, sd[p + "attn_norm.weight"], d.rq_norm_eps, dt)
        qkv = linear(h, sd[p + "Wqkv.weight"], dt).view(B, T, 3, nh, hd)
        q, k, v = qkv.unbind(2)
        if k_all is not None:
            k = torch.cat([k_all, k], 1)
            v = torch.cat([v_all, v], 1)
        P = k.shape[1]
        mask = None
        if causal:
            mask = (torch.arange(P)[None, :] <= (P - T + torch.arange(T))[:, None])[None, None]
        o = attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), hd ** -0.5, dt, mask)
        o = o.transpose(1, 2).reshape(B, T, R)
        x = rnd(x + linear(o, sd[p + "out_proj.weight"], dt), dt)
        h2 = rmsnorm(x, sd[p + "mlp_norm.weight"], d.rq_norm_eps, dt)
        x = rnd(x + swiglu(h2, sd[p + "w1.weight"], sd[p + "w3.weight"], sd[p + "w2.weight"], dt), dt)
        return x, k, v

    def _rq_tok0(self, hidden: Tensor) -> Tensor:
        sd, dt = self.sd, self.dt
        if "rq_transformer.backbone_proj.weight" in sd:
            pr = linear(hidden, sd["rq_transformer.backbone_proj.weight"], dt)
        else:  # nn.Identity when backbone_dim == rq_dim, model.py:653-657
            pr = rnd(hidden, dt)
        return rnd(pr + sd["rq_transformer.pos_emb.weight"][0], dt)

    def _rq_tok(self, code: Tensor, i: int) -> Tensor:
        """Token at sequence position i+1 from the code of codebook i.  model.py:703,722-726,967-970."""
        sd = self.sd
        e = sd["rq_transformer.code_emb.embedding.weight"][code + i * self.dims.codebook_size]
        return rnd(e + sd["rq_transformer.pos_emb.weight"][i + 1], self.dt)

    def rq_logits(self, h: Tensor, i: int, logit_bias: Tensor | None) -> Tensor:
        """fp32 logits of codebook i+1 from the hidden at position i+1 (before /temperature).
        Reference: model.py:954-956, 975-979."""
        sd, dt = self.sd, self.dt
        hn = rmsnorm(h, sd["rq_transformer.norm.weight"], self.dims.rq_norm_eps, dt)
        lg = linear(hn, sd["rq_transformer.head_W"][i], dt)
        if logit_bias is not None:
            lg = lg + logit_bias[i].float()
        return lg

    def rq_generate(self, hidden: Tensor, code0: Tensor, temperature: float = 0.7, top_k: int = 100,
                    logit_bias: Tensor | None = None, n_quantizers: int = 0, seed: int = 0,
                    frame: int = 0, return_logits: bool = False):
        """KV-cached depth loop.  Reference: _generate_graph_body_kv model.py:908-986 and
        generate_cuda_graph_kv :988-1016.  Returns codes (B, Q') int64."""
        d = self.dims
        Q = n_quantizers if n_quantizers > 0 else d.n_quantizers
        B = hidden.shape[0]
        seq = torch.stack([self._rq_tok0(hidden), self._rq_tok(code0, 0)], 1)  # (B,2,R)
        ks, vs = [], []
        for li in range(d.rq_n_layers):
            seq, k, v = self._rq_block(li, seq, None, None, causal=True)
            ks.append(k)
            vs.append(v)
        codes = [code0.clone()]
        all_logits = []
        h = seq[:, 1]
        for i in range(Q - 1):
            if i > 0:
                tok = self._rq_tok(codes[-1], i)[:, None]
                for li in range(d.rq_n_layers):
                    tok, ks[li], vs[li] = self._rq_block(li, tok, ks[li], vs[li], causal=False)
                h = tok[:, 0]
            lg = self.rq_logits(h, i, logit_bias)
            all_logits.append(lg)
            nxt = [sample_rq(lg[b], temperature, top_k, uniform01(seed, frame, b, i + 1)) for b in range(B)]
            codes.append(torch.tensor(nxt, dtype=torch.long))
        out = torch.stack(codes, 1)
        if return_logits:
            return out, torch.stack(all_logits, 1)
        return out

    def rq_generate_full(self, hidden: Tensor, code0: Tensor, temperature: float = 0.7, top_k: int = 100,
                         logit_bias: Tensor | None = None, seed: int = 0, frame: int = 0) -> Tensor:
        """Full-recompute depth loop.  Reference: RQTransformer.generate model.py:686-728."""
        d = self.dims
        Q = d.n_quantizers
        B = hidden.shape[0]
        seq = torch.zeros(B, Q, d.rq_d_model)
        seq[:, 0] = self._rq_tok0(hidden)
        seq[:, 1] = self._rq_tok(code0, 0)
        codes = [code0.clone()]
        for i in range(Q - 1):
            h = seq
            for li in range(d.rq_n_layers):
                h, _, _ = self._rq_block(li, h, None, None, causal=True)
            lg = self.rq_logits(h[:, i + 1], i, logit_bias)
            nxt = [sample_rq(lg[b], temperature, top_k, uniform01(seed, frame, b, i + 1)) for b in range(B)]
            codes.append(torch.tensor(nxt, dtype=torch.long))
            if i + 2 < Q:
                seq[:, i + 2] = self._rq_tok(codes[-1], i + 1)
        return torch.stack(codes, 1)

    def rq_forward(self, hidden: Tensor, codes: Tensor) -> Tensor:
        """Teacher-forced logits (N, Q-1, CS).  Reference: RQTransformer.forward model.py:665-684."""
        d, sd, dt = self.dims, self.sd, self.dt
        Q = codes.shape[1]
        toks = [self._rq_tok0(hidden)] + [self._rq_tok(codes[:, i], i) for i in range(Q - 1)]
        seq = torch.stack(toks, 1)
        for li in range(d.rq_n_layers):
            seq, _, _ = self._rq_block(li, seq, None, None, causal=True)
        hn = rmsnorm(seq, sd["rq_transformer.norm.weight"], d.rq_norm_eps, dt)
        return torch.stack([linear(hn[:, i + 1], sd["rq_transformer.head_W"][i], dt) for i in range(Q - 1)], 1)

    # -- whole frames -------------------------------------------------------------------
    def generate_frames(self, first_hidden: Tensor, n_frames: int, *, temperature: float = 0.9,
                        top_k: int = 1, rq_temperature: float | None = None, rq_top_k: int | None = None,
                        rep_penalty: float = 1.0, rep_window: int = 0, n_codebooks: int = 0,
                        seed: int = 0, slots: Tensor | None = None, collect: dict | None = None) -> Tensor:
        """Frame loop of the reference's drivers without EOS/text logic.

        first_hidden (B,d): final-norm hidden of the last prefill position.  Per frame: code0
        from codec_head logits (rep penalty, temperature, top-k), RQ head for the other
        codebooks, feed the frame back through decode_step.  Reference: engine.py:1414-1485,
        inference.py:596-608, 700-726.  Returns (n_frames, B, Q').
        """
        B = first_hidden.shape[0]
        d = self.dims
        rq_t = temperature if rq_temperature is None else rq_temperature
        rq_k = top_k if rq_top_k is None else rq_top_k
        reps = [RepState(d.codebook_size, rep_window) for _ in range(B)]
        hidden = first_hidden
        cb0, eos = self.heads(hidden)
        frames = []
        for f in range(n_frames):
            c0 = []
            for b in range(B):
                c = sample_cb0(cb0[b], reps[b].counts, rep_penalty, temperature, top_k,
                               uniform01(seed, f, b, 0))
                if rep_penalty > 1.0:
                    reps[b].push(c)
                c0.append(c)
            code0 = torch.tensor(c0, dtype=torch.long)
            frame = self.rq_generate(hidden, code0, rq_t, rq_k, None, n_codebooks, seed, f)
            frames.append(frame)
            if collect is not None:
                collect.setdefault("cb0", []).append(cb0.clone())
                collect.setdefault("eos", []).append(eos.clone())
                collect.setdefault("hidden", []).append(hidden.clone())
            if f + 1 < n_frames:
                hidden, cb0, eos = self.decode_step(frame, slots)
        return torch.stack(frames)


# --------------------------------------------------------------------------------------
# streaming control loop of one row
# --------------------------------------------------------------------------------------
FRAME_RATE = 12.5
DEFAULT_WPS = 3.0  # engine.py:41
GATE_RETRY_TEMPS = (0.5, 0.3)  # engine.py:1367


def max_turn_frames(n_words: int, prompt_wps: float, max_turn_secs: float = 15.0, max_turn_wps: float = 0.0) -> int:
    """Reference: GenConfig.max_turn_frames, engine.py:88-103."""
    ceil = int(max_turn_secs * FRAME_RATE)
    wps = max_turn_wps if max_turn_wps > 0 else prompt_wps
    if wps <= 0:
        wps = DEFAULT_WPS
    if n_words <= 0:
        return ceil
    return min(int((n_words / wps * 1.6 + 0.6) * FRAME_RATE), ceil)


def stream_row(model: "OracleModel", chunks, *, temperature: float = 0.9, top_k: int = 100, rq_top_k: int = 100,
               rep_penalty: float = 1.1, rep_window: int = 24, eos_threshold: float = 0.45, min_secs: float = 0.5,
               max_turn_secs: float = 15.0, max_secs: float = 30.0, n_codebooks: int = 0, max_turn_wps: float = 0.0,
               gate_frames: int = 0, gate_entropy_max: float = 1.9, gate_retries: int = 2, seed: int = 0,
               prompt_wps: float = 0.0, max_seq: int | None = None, slot: int = 0, cancel_after: int | None = None,
               log: list | None = None) -> list[Tensor]:
    """Restatement of Engine._stream_row (engine.py:1308-1521) on the oracle model, one turn with a
    fresh repetition state.  chunks: list of (emb (T, d), n_words).  Returns the yielded code
    frames.  The draw for frame f of the turn uses uniform01(seed, f, 0, codebook); a frame whose
    EOS test ends the chunk still consumes its counter (the device step draws it before the test).
    cancel_after: behave as if cancel were set once that many frames have been yielded.
    log: receives ("retry", chunk, temp) / ("eos", chunk, step) / ("cap", chunk) events and the EOS
    probability of every step as ("p", chunk, step, probability)."""
    d = model.dims
    max_frames = int(max_secs * FRAME_RATE)
    min_frames = int(min_secs * FRAME_RATE)
    max_seq = (max_seq if max_seq is not None else d.max_seqlen) - 10
    s = torch.tensor([slot])
    rep = RepState(d.codebook_size, rep_window)
    out: list[Tensor] = []
    fctr = 0

    def cancelled() -> bool:
        return cancel_after is not None and len(out) >= cancel_after

    def probs_of(cb0, temp):
        return torch.softmax(rep_penalise(cb0, rep.counts, rep_penalty) / temp, dim=-1)

    def ent(p):
        return float(-(p * p.clamp_min(1e-9).log()).sum(-1).mean())

    def draw0(cb0, temp, k):
        nonlocal fctr
        c = sample_cb0(cb0, rep.counts, rep_penalty, temp, k, uniform01(seed, fctr, 0, 0))
        if rep_penalty > 1.0:
            rep.push(c)
        return c

    for ci, (emb, n_words) in enumerate(chunks):
        if len(out) >= max_frames or int(model.seq_lens[slot]) >= max_seq or cancelled():
            return out
        use_gate = gate_frames > 0 and ci == 0
        chunk_start = int(model.seq_lens[slot])
        max_per_turn = max_turn_frames(n_words, prompt_wps, max_turn_secs, max_turn_wps)
        retry_idx = 0
        while True:
            cur_temp = temperature
            if retry_idx > 0:
                cur_temp = GATE_RETRY_TEMPS[min(retry_idx - 1, len(GATE_RETRY_TEMPS) - 1)]
                model.seq_lens[slot] = chunk_start
                rep = RepState(d.codebook_size, rep_window)
                if log is not None:
                    log.append(("retry", ci, cur_temp))
            hidden = model.prefill(emb, slot)[-1:]
            cb0, _ = model.heads(hidden)
            held: list[Tensor] = []
            entropies: list[float] = []
            if use_gate:
                entropies.append(ent(probs_of(cb0, cur_temp)))
            rq_k = rq_top_k if top_k != 1 else 1
            c0 = draw0(cb0[0], cur_temp, 1 if top_k == 1 else 0)
            frame = model.rq_generate(hidden, torch.tensor([c0]), cur_temp, rq_k, None, n_codebooks, seed, fctr)[0]
            fctr += 1
            (held if use_gate else out).append(frame)
            retry = False
            for step in range(1, max_per_turn):
                if len(out) >= max_frames or int(model.seq_lens[slot]) >= max_seq:
                    out.extend(held)
                    if log is not None:
                        log.append(("cap", ci))
                    return out
                if cancelled():
                    return out
                hidden, cb0, eos = model.decode_step(frame[None], s)
                gathering = use_gate and len(held) < gate_frames
                if gathering:
                    entropies.append(ent(probs_of(cb0, cur_temp)))
                c0 = draw0(cb0[0], cur_temp, top_k)
                p_eos = float(torch.sigmoid(eos[0, 0].float()))
                if log is not None:
                    log.append(("p", ci, step, p_eos))
                if step >= min_frames and p_eos > eos_threshold:
                    out.extend(held)
                    held = []
                    fctr += 1
                    if log is not None:
                        log.append(("eos", ci, step))
                    break
                frame = model.rq_generate(hidden, torch.tensor([c0]), cur_temp, rq_k, None, n_codebooks, seed, fctr)[0]
                fctr += 1
                if gathering:
                    held.append(frame)
                    if len(held) == gate_frames:
                        if sum(entropies) / len(entropies) > gate_entropy_max and retry_idx < gate_retries:
                            retry = True
                            break
                        out.extend(held)
                        held = []
                        use_gate = False
                else:
                    out.append(frame)
            if retry:
                retry_idx += 1
                continue
            out.extend(held)
            break
    return out


def render_rows(model: "OracleModel", chunk_lists, *, temperature: float = 0.9, top_k: int = 100, rq_top_k: int = 100,
                rep_penalty: float = 1.1, rep_window: int = 24, eos_threshold: float = 0.45, min_secs: float = 0.5,
                max_turn_secs: float = 15.0, max_secs: float = 30.0, n_codebooks: int = 0, max_turn_wps: float = 0.0,
                seed: int = 0, prompt_wps: float = 0.0, max_seq: int | None = None, log: list | None = None):
    """Restatement of Engine._render_rows (engine.py:865-1087) on the oracle model: row r of chunk_lists (a list of
    (emb (T, d), n_words) per row) renders in cache slot r, all rows in lock step.  Returns {row: (T, Q') codes}.

    The frame counter of the random stream advances once per chunk start and once per decode step (the
    device's frame step draws before the end-of-turn test); a chunk start draws code 0 (no top-k cut unless
    greedy) with the repetition state of its own row.  A chunk that ends (EOS or its cap) with fewer than two
    frames per word is rewound and redone colder: 0.5, then 0.3 (engine.py:952-983), which resets every row's
    repetition state as the reference does.  log: ("retry", row, chunk, temp) / ("eos", row, chunk) events."""
    d = model.dims
    N = len(chunk_lists)
    max_frames = int(max_secs * FRAME_RATE)
    min_frames = int(min_secs * FRAME_RATE)
    max_seq = (max_seq if max_seq is not None else d.max_seqlen) - 10
    nq = n_codebooks if n_codebooks > 0 else d.n_quantizers
    greedy = top_k == 1
    rq_k = rq_top_k if not greedy else 1
    reps = [RepState(d.codebook_size, rep_window) for _ in range(N)]
    chunk_idx = [0] * N
    frames: list[list[Tensor]] = [[] for _ in range(N)]
    turn_count = [0] * N
    max_turn = [max_turn_frames(0, prompt_wps, max_turn_secs, max_turn_wps)] * N
    chunk_offset = [0] * N
    retry_idx = [0] * N
    active = [True] * N
    last: list[Tensor | None] = [None] * N
    fctr = 0

    def advance_turn(r: int, temp: float | None = None) -> bool:
        nonlocal fctr
        ci = chunk_idx[r]
        if ci >= len(chunk_lists[r]) or len(frames[r]) >= max_frames:
            return False
        emb, n_words = chunk_lists[r][ci]
        max_turn[r] = max_turn_frames(n_words, prompt_wps, max_turn_secs, max_turn_wps)
        chunk_offset[r] = int(model.seq_lens[r])
        t = temp or temperature
        hidden = model.prefill(emb, r)[-1:]
        cb0, _ = model.heads(hidden)
        c0 = sample_cb0(cb0[0], reps[r].counts, rep_penalty, t, 1 if greedy else 0, uniform01(seed, fctr, r, 0))
        if rep_penalty > 1.0:
            reps[r].push(c0)
        frame = model.rq_generate(hidden, torch.tensor([c0]), t, rq_k, None, n_codebooks, seed, fctr)[0]
        fctr += 1
        last[r] = frame
        frames[r].append(frame)
        turn_count[r] = 1
        return True

    def retry_chunk(r: int) -> bool:
        nonlocal reps
        n_words = chunk_lists[r][chunk_idx[r]][1]
        fpw = turn_count[r] / n_words if n_words > 0 else 999
        if fpw >= 2.0:
            retry_idx[r] = 0
            return False
        ri = retry_idx[r]
        if ri >= len(GATE_RETRY_TEMPS):
            retry_idx[r] = 0
            return False
        retry_idx[r] = ri + 1
        if log is not None:
            log.append(("retry", r, chunk_idx[r], GATE_RETRY_TEMPS[ri]))
        model.seq_lens[r] = chunk_offset[r]
        del frames[r][len(frames[r]) - turn_count[r]:]
        reps = [RepState(d.codebook_size, rep_window) for _ in range(N)]
        advance_turn(r, GATE_RETRY_TEMPS[ri])
        return True

    def next_chunk(r: int) -> None:
        if retry_chunk(r):
            return
        retry_idx[r] = 0
        chunk_idx[r] += 1
        if not advance_turn(r):
            active[r] = False

    for r in range(N):
        if not advance_turn(r):
            active[r] = False
    steps = 0
    while any(active) and steps < max_frames:
        for r in range(N):
            if active[r] and turn_count[r] >= max_turn[r]:
                next_chunk(r)
        if not any(active):
            break
        # every slot steps (the batched graph covers all rows); rows that are over keep feeding their last frame
        rows = list(range(N))
        slots = torch.tensor(rows)
        codes = torch.zeros(N, d.n_quantizers, dtype=torch.long)
        for r in rows:
            if last[r] is not None:
                codes[r, :nq] = last[r]
        hidden, cb0, eos = model.decode_step(codes, slots)
        c0s = []
        for i, r in enumerate(rows):
            c = sample_cb0(cb0[i], reps[r].counts, rep_penalty, temperature, top_k, uniform01(seed, fctr, r, 0))
            if rep_penalty > 1.0:
                reps[r].push(c)
            c0s.append(c)
        new = model.rq_generate(hidden, torch.tensor(c0s), temperature, rq_k, None, n_codebooks, seed, fctr)
        fctr += 1
        steps += 1
        hit = []
        for i, r in enumerate(rows):
            if not active[r]:
                continue
            if int(model.seq_lens[r]) >= max_seq or len(frames[r]) >= max_frames:
                active[r] = False
                continue
            if turn_count[r] >= min_frames and float(torch.sigmoid(eos[i, 0].float())) > eos_threshold:
                if log is not None:
                    log.append(("eos", r, chunk_idx[r]))
                hit.append(r)
                continue
            last[r] = new[i]
            frames[r].append(new[i])
            turn_count[r] += 1
        for r in hit:
            next_chunk(r)
    return {r: torch.stack(frames[r]) for r in range(N) if frames[r]}


def stream_frames(model: "OracleModel", chunks, *, temperature: float = 0.9, top_k: int = 100, rq_top_k: int = 100,
                  rep_penalty: float = 1.0, rep_window: int = 0, max_secs: float = 120.0, max_turn_secs: float = 15.0,
                  eos_threshold: float = 0.45, min_turn_secs: float = 0.5, seed: int = 0, max_seq: int | None = None):
    """Restatement of inference.stream_frames (inference.py:507-734) on the oracle model, from position 0 of
    slot 0.  chunks: list of emb (T, d).  Returns [(frame, turn_end)] with turn_end the chunk index on a turn's
    last frame, else None.  Code 0 is drawn by sampling.sample_top_k's rule (everything >= the k-th largest kept,
    sampling.py:14-20) on every frame; the depth head runs before the end-of-turn test (inference.py:708-720), so
    each rq_sample call consumes one frame number of the random stream."""
    d = model.dims
    max_frames = int(max_secs * FRAME_RATE)
    max_per_turn = int(max_turn_secs * FRAME_RATE)
    min_frames = int(min_turn_secs * FRAME_RATE)
    max_seq = (max_seq if max_seq is not None else d.max_seqlen) - 10
    rep = RepState(d.codebook_size, rep_window)
    s0 = torch.tensor([0])
    out = []
    fctr = 0
    total = 0
    rq_k = rq_top_k if top_k != 1 else 1

    def rq_sample(cb0: Tensor, hidden: Tensor) -> Tensor:
        nonlocal fctr
        l = rep_penalise(cb0, rep.counts, rep_penalty)
        u = uniform01(seed, fctr, 0, 0)
        if top_k == 1 or temperature <= 0:
            c0 = int(torch.argmax(l))
        else:
            c0 = _inverse_cdf(topk_threshold_probs(l, temperature, top_k if top_k else 0), u)
        if rep_penalty > 1.0:
            rep.push(c0)
        frame = model.rq_generate(hidden, torch.tensor([c0]), temperature, rq_k, None, 0, seed, fctr)[0]
        fctr += 1
        return frame

    model.seq_lens[0] = 0
    for ti, emb in enumerate(chunks):
        if int(model.seq_lens[0]) >= max_seq or total >= max_frames:
            break
        if int(model.seq_lens[0]) + emb.shape[0] >= max_seq:
            break
        hidden = model.prefill(emb, 0)[-1:]
        cb0, _ = model.heads(hidden)
        pending = rq_sample(cb0[0], hidden)
        total += 1
        codes_in = pending
        for step in range(1, max_per_turn):
            if int(model.seq_lens[0]) >= max_seq or total >= max_frames:
                break
            hidden, cb0, eos = model.decode_step(codes_in[None], s0)
            nxt = rq_sample(cb0[0], hidden)
            if step >= min_frames and float(torch.sigmoid(eos[0, 0].float())) > eos_threshold:
                break
            out.append((pending, None))
            pending = nxt
            total += 1
            codes_in = nxt
        out.append((pending, ti))
    return out


def _get_bucket(n: int, max_rows: int) -> int:
    """Smallest bucket holding n rows; buckets are the powers of two below max_rows and max_rows itself
    (engine.py:134-154)."""
    b = 1
    while b < n:
        b *= 2
    return min(b, max_rows)


def render_continuous(model: "OracleModel", requests, *, max_rows: int, temperature: float = 0.9, top_k: int = 100,
                      rq_top_k: int = 100, rep_penalty: float = 1.1, eos_threshold: float = 0.45,
                      min_secs: float = 0.5, max_turn_secs: float = 15.0, max_secs: float = 30.0,
                      n_codebooks: int = 0, max_turn_wps: float = 0.0, seed: int = 0, max_seq: int | None = None,
                      log: list | None = None) -> list[Tensor]:
    """Restatement of Engine.render_continuous (engine.py:1112-1302) on the oracle model (n_slots >=
    max_rows).  requests: list of (prompt_emb (T, d) or None, chunks [(emb (T, d), n_words)], prompt_wps).
    Returns the frames (T_i, Q') of every request in input order.

    Rules kept from the reference: the queue is served in order into the lowest free slot; a slot's
    repetition counts start at zero and never age (no window); a chunk's first frame is drawn from the
    text's last hidden state without top-k (unless greedy); every step draws for all active slots, and a slot
    whose EOS flag is up after min_secs or whose chunk reached its frame cap drops that step's frame and
    starts its next chunk; max_secs or the cache limit end the request (that step's frame is dropped too);
    freed slots are refilled before the next step.  The draw of sampling event e (a chunk start or a
    step) for slot s uses uniform01(seed, e, s, 0); the depth head of that event uses frame e with rows
    numbered by position in the sorted slot list.
    log: receives ("start", request, slot) / ("next", request, chunk) / ("end", request, reason, frames)
    and ("step", tuple(sorted slots), bucket)."""
    d = model.dims
    max_frames = int(max_secs * FRAME_RATE)
    min_frames = int(min_secs * FRAME_RATE)
    max_seq = (max_seq if max_seq is not None else d.max_seqlen) - 10
    greedy = top_k == 1
    rq_k = 1 if greedy else rq_top_k
    counts = torch.zeros(max_rows, d.codebook_size)
    frames: list[list[Tensor]] = [[] for _ in requests]
    pending = list(range(len(requests)))
    free = set(range(max_rows))
    active: dict[int, dict] = {}
    event = 0

    def draw(cb0_row: Tensor, slot: int, k: int) -> int:
        c = sample_cb0(cb0_row, counts[slot], rep_penalty, temperature, k, uniform01(seed, event, slot, 0))
        if rep_penalty > 1.0:
            counts[slot, c] += 1.0
        return c

    def advance(info: dict) -> bool:
        nonlocal event
        if info["ci"] >= len(info["chunks"]):
            return False
        emb, n_words = info["chunks"][info["ci"]]
        info["max_turn"] = max_turn_frames(n_words, info["wps"], max_turn_secs, max_turn_wps)
        hidden = model.prefill(emb, info["slot"])[-1:]
        cb0, _ = model.heads(hidden)
        c0 = draw(cb0[0], info["slot"], 1 if greedy else 0)
        info["last"] = model.rq_generate(hidden, torch.tensor([c0]), temperature, rq_k, None, n_codebooks, seed, event)[0]
        event += 1
        frames[info["req"]].append(info["last"])
        info["n"] += 1
        info["turn"] = 1
        info["off"] = int(model.seq_lens[info["slot"]])
        if log is not None:
            log.append(("next", info["req"], info["ci"]))
        return True

    def backfill() -> None:
        while pending and free:
            ri = pending.pop(0)
            prompt, chunks, wps = requests[ri]
            slot = min(free)
            free.remove(slot)
            model.seq_lens[slot] = 0
            counts[slot].zero_()
            if log is not None:
                log.append(("start", ri, slot))
            if prompt is not None and prompt.shape[0] > 0:
                model.prefill(prompt, slot)
            info = dict(req=ri, slot=slot, chunks=chunks, wps=wps, ci=0, n=0, turn=0, max_turn=0, off=0, last=None)
            if not chunks or not advance(info):
                free.add(slot)
                continue
            active[slot] = info

    backfill()
    while active:
        slots = sorted(active)
        if log is not None:
            log.append(("step", tuple(slots), _get_bucket(len(slots), max_rows)))
        codes = torch.stack([active[s]["last"] for s in slots])
        hidden, cb0, eos = model.decode_step(codes, torch.tensor(slots))
        for s in slots:
            active[s]["off"] += 1
        c0 = torch.tensor([draw(cb0[i], s, top_k) for i, s in enumerate(slots)])
        flags = torch.sigmoid(eos.float()).flatten() > eos_threshold
        new = model.rq_generate(hidden, c0, temperature, rq_k, None, n_codebooks, seed, event)
        event += 1
        gone = []
        for i, s in enumerate(slots):
            info = active[s]
            if info["n"] >= max_frames or info["off"] >= max_seq:
                gone.append((s, "cap"))
                continue
            if (info["turn"] >= min_frames and bool(flags[i])) or info["turn"] >= info["max_turn"]:
                info["ci"] += 1
                if not advance(info):
                    gone.append((s, "done"))
                continue
            info["last"] = new[i]
            frames[info["req"]].append(new[i])
            info["n"] += 1
            info["turn"] += 1
        for s, why in gone:
            info = active.pop(s)
            free.add(s)
            if log is not None:
                log.append(("end", info["req"], why, info["n"]))
        backfill()
    q = n_codebooks if n_codebooks > 0 else d.n_quantizers
    return [torch.stack(f) if f else torch.zeros(0, q, dtype=torch.long) for f in frames]


# --------------------------------------------------------------------------------------
# deterministic synthetic weights (the benchmark's "random-init N(0, 0.02) from seed 0")
# --------------------------------------------------------------------------------------
def state_dict_shapes(d: Dims) -> dict[str, tuple[int, ...]]:
    """Shapes per reference state-dict key (model.py:1076-1136, 577-663)."""
    H, KV, hd = d.n_heads, d.n_kv_heads, d.head_dim
    sh: dict[str, tuple[int, ...]] = {}
    sh["token_emb.weight"] = (d.vocab_size, d.d_model)
    sh["audio_emb.embedding.weight"] = (d.n_quantizers * d.codebook_size, d.d_model)
    sh["codec_head.weight"] = (d.codebook_size, d.d_model)
    sh["eos_head.weight"] = (1, d.d_model)
    sh["eos_head.bias"] = (1,)
    for i in range(d.n_layers):
        p = f"decoder.blocks.{i}."
        sh[p + "attn_norm.weight"] = (d.d_model,)
        sh[p + "attn.Wqkv.weight"] = ((H + 2 * KV) * hd, d.d_model)
        sh[p + "attn.out_proj.weight"] = (d.d_model, d.d_model)
        sh[p + "mlp_norm.weight"] = (d.d_model,)
        sh[p + "mlp.w1.weight"] = (d.ffn, d.d_model)
        sh[p + "mlp.w3.weight"] = (d.ffn, d.d_model)
        sh[p + "mlp.w2.weight"] = (d.d_model, d.ffn)
    sh["decoder.norm.weight"] = (d.d_model,)
    R = d.rq_d_model
    if R != d.d_model:
        sh["rq_transformer.backbone_proj.weight"] = (R, d.d_model)
    sh["rq_transformer.code_emb.embedding.weight"] = ((d.n_quantizers - 1) * d.codebook_size, R)
    sh["rq_transformer.pos_emb.weight"] = (d.n_quantizers, R)
    sh["rq_transformer.head_W"] = (d.n_quantizers - 1, d.codebook_size, R)
    sh["rq_transformer.norm.weight"] = (R,)
    for i in range(d.rq_n_layers):
        p = f"rq_transformer.blocks.{i}."
        sh[p + "attn_norm.weight"] = (R,)
        sh[p + "Wqkv.weight"] = (3 * R, R)
        sh[p + "out_proj.weight"] = (R, R)
        sh[p + "mlp_norm.weight"] = (R,)
        sh[p + "w1.weight"] = (d.rq_ffn, R)
        sh[p + "w3.weight"] = (d.rq_ffn, R)
        sh[p + "w2.weight"] = (R, d.rq_ffn)
    return sh


def synthetic_state_dict(d: Dims, seed: int = 0, std: float = 0.02, norm_jitter: float = 0.0,
                         bias_std: float = 0.0) -> dict[str, Tensor]:
    """Per-key seeded N(0, std) fp32 weights; norm weights 1 (+ jitter), eos bias 0 (+ noise).

    Each key draws from its own torch CPU generator seeded with (seed, key index), so a
    tensor's values do not depend on which other keys exist.
    """
    sd = {}
    for idx, (k, shape) in enumerate(state_dict_shapes(d).items()):
        g = torch.Generator().manual_seed(seed * 1000003 + idx)
        if k.endswith("norm.weight"):
            t = torch.ones(shape)
            if norm_jitter:
                t = t + norm_jitter * torch.randn(shape, generator=g)
        elif k.endswith(".bias"):
            t = bias_std * torch.randn(shape, generator=g) if bias_std else torch.zeros(shape)
        else:
            t = std * torch.randn(shape, generator=g)
        sd[k] = t
    return sd
