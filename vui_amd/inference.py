"""The single-stream driver of the reference's `vui.inference` on the native step: `InferenceState`
(position pointer, prompt prefill, checkpoint / rewind) and `stream_frames`, the per-frame code generator
that `render_codes_stream`, `render_audio_stream` and the TTS worker consume (src/vui/inference.py:140-367,
507-734).

It differs from `Engine._stream_row` exactly where the reference's two drivers differ: code 0 is drawn with
`sampling.sample_top_k` (everything >= the k-th largest probability kept) on EVERY frame, the first of a chunk
included; the depth head runs before the end-of-turn test, so a turn's last frame is drawn and then dropped;
the step is `Vui.decode_step(codes, pos)`; a chunk is capped by max_turn_secs alone; `top_p` adds the nucleus
cut of `sampling.sample_top_p` / `sample_top_p_top_k` to the code-0 draw.

Text handling (cleaning, chunking, tokenising) is outside this package: chunks arrive as `Chunk`s whose `emb`
holds the embeddings of `[spk] text` (+ `[SC]` where the next chunk changes speaker, + cond_bias), as the
reference's loop writes them (inference.py:648-666).
"""
from __future__ import annotations

import ctypes as C
from typing import Iterator

import torch
from torch import Tensor

from . import _lib
from .engine import FRAME_RATE, Chunk
from .model import Vui, make_sample_params

CODEC_HZ = FRAME_RATE  # src/vui/inference.py:370


class InferenceState:
    """Graphs and the position pointer of one stream (InferenceState, src/vui/inference.py:140-345).  The
    vocoder part of the reference's class (codec chunk graphs) lives in vui_amd.codec."""

    def __init__(self, model: Vui, codec=None, chunk_frames: int = 7, ctx_frames: int = 3, sq_scores=None,
                 wps_score: float = 1.0, codec_graphs: bool = True, compile_rq: bool = False, rq_top_k: int = 100):
        """Same arguments as the reference's (inference.py:143-166).  chunk_frames / ctx_frames / codec_graphs
        belong to its chunked vocoder graphs and are kept for callers that pass them (the vocoder here streams
        frame by frame); compile_rq selects generate_kv_compilable, which runs the same kernels."""
        self.model = model
        self.codec = codec
        self.chunk_frames = chunk_frames
        self.ctx_frames = ctx_frames
        self._codec_graphs = codec_graphs
        self._compile_rq = compile_rq
        self.device = model.device
        self.dtype = model.dtype
        self.offset = 0
        self._ckpt_offset = 0
        self._ckpt_spk_token: Tensor | None = None
        self._ckpt_spk_token_2: Tensor | None = None
        self._rq_top_k = rq_top_k
        self._setup_graphs()
        self.model.set_cond_bias(sq_scores=sq_scores, wps_score=wps_score)

    def _setup_graphs(self) -> None:
        """src/vui/inference.py:169-197: the one-slot backbone step graph and the depth-head graphs."""
        self.model.setup_decode_graph()
        rq = self.model.rq_transformer
        rq.setup_cuda_graph_kv(self.device, self.dtype, top_k=self._rq_top_k)
        if self._compile_rq:
            top_k = self._rq_top_k
            self._rq_generate = lambda hidden, code0, temperature, bias: rq.generate_kv_compilable(
                hidden, code0, temperature, bias, top_k)
        else:
            self._rq_generate = rq.generate_cuda_graph_kv

    def reset(self) -> None:
        self.rewind(0)

    def teardown(self) -> None:
        self.model.decoder.deallocate_kv_cache()

    def checkpoint(self) -> int:
        self._ckpt_offset = self.offset
        return self.offset

    def rewind(self, offset: int | None = None) -> int:
        """Only the position moves; keys and values beyond it are never cleared (inference.py:325-345)."""
        target = offset if offset is not None else self._ckpt_offset
        if self.model.decoder.flash_kv_caches is None:
            self._setup_graphs()
        self.model.decoder.flash_kv_caches[0].seq_lens[:1].fill_(target)
        self.offset = target
        return target

    @torch.inference_mode()
    def prefill(self, segments: "list[tuple[str, Tensor]]", cond_last: bool = True) -> int:
        """Interleaved ("text", embeddings (1, T, d)) / ("audio", codes (T, Q)) segments (inference.py:236-268);
        cond_bias is added to the last segment only when cond_last."""
        bias = self.model._cond_bias
        for i, (kind, data) in enumerate(segments):
            use_bias = (not cond_last) or i == len(segments) - 1
            if kind == "text":
                emb = data.to(self.device, self.dtype)
            else:
                emb = self.model.embed_audio(data.to(self.device)[None]).to(self.dtype)
            if use_bias:
                emb = emb + bias
            _forward_flash_emb(self, emb)
        return self.offset

    @torch.inference_mode()
    def prefill_prompt(self, prompt_segments=None, prompt_segments_2=None, spk_emb: Tensor | None = None,
                       spk_emb_2: Tensor | None = None) -> int:
        """`[spk] text codes` per segment for one or two speakers from position 0 (inference.py:274-317).
        Segments are (text embeddings (1, T, d) or None, codes (T, Q))."""
        self.reset()
        model = self.model
        spk = model.embed_speaker(spk_emb) if (spk_emb is not None and model.spk_proj is not None) else None
        spk2 = model.embed_speaker(spk_emb_2) if (spk_emb_2 is not None and model.spk_proj is not None) else None
        self._ckpt_spk_token, self._ckpt_spk_token_2 = spk, spk2
        for segs, seg_spk in ((prompt_segments, spk), (prompt_segments_2, spk2)):
            if segs is None:
                continue
            for text_emb, codes in segs:
                if seg_spk is not None:
                    _forward_flash_emb(self, seg_spk.to(self.dtype))
                if text_emb is not None and text_emb.shape[1] > 0:
                    _forward_flash_emb(self, text_emb.to(self.device, self.dtype))
                pc = codes.to(self.device)
                if pc.dim() == 2:
                    pc = pc.unsqueeze(0)
                _forward_flash_emb(self, model.embed_audio(pc).to(self.dtype))
        return self.offset


def _forward_flash_emb(state: InferenceState, emb: Tensor) -> Tensor:
    """src/vui/inference.py:737-744."""
    n = emb.shape[1]
    positions = torch.arange(state.offset, state.offset + n, device=state.device)
    out = state.model.decoder.forward_flash(emb, positions)
    state.offset += n
    return out


@torch.inference_mode()
def stream_frames(state: InferenceState, chunks: "list[Chunk]", *, temperature: float = 0.9, top_k: int | None = 100,
                  top_p: float | None = None, rep_penalty: float = 1.0, rep_window: int = 0,
                  max_secs: float = 120.0, max_turn_secs: float = 15.0, eos_threshold: float = 0.45,
                  min_turn_secs: float = 0.5, resume: bool = False, seed: int = 0) -> Iterator[tuple[Tensor, object]]:
    """Per-frame code generator: yields (code_frame (Q,) int64 on the GPU, turn_end) where turn_end is None
    inside a turn and the chunk (with .frames / .secs set) on its last frame (src/vui/inference.py:507-734).

    resume=False starts from position 0 (a prompt is written by the caller through state.prefill_prompt and
    resume=True, as the reference's low-latency path does)."""
    if not chunks:
        return
    model, nat = state.model, state.model._native
    rq = model.rq_transformer
    Q, CS = rq.n_quantizers, rq.codebook_size
    dev = state.device
    zero_rq_bias = torch.zeros(Q - 1, CS, device=dev, dtype=torch.float32)
    # rolling code-0 counts on the device: what the reference keeps as a deque and a {code: count} dict
    use_rep = rep_penalty > 1.0
    counts = torch.zeros(1, CS, device=dev, dtype=torch.float32)
    hist = torch.zeros(1, max(rep_window, 1), device=dev, dtype=torch.int32)
    pos2 = torch.zeros(1, 2, device=dev, dtype=torch.int32)
    frame_ctr = rq._ctr  # one frame number keys the code-0 draw and the depth head's draws; the depth-head call advances it
    if not resume:
        frame_ctr.zero_()
    code0 = torch.zeros(1, dtype=torch.long, device=dev)
    win = rep_window if (use_rep and rep_window > 0) else 0
    k = 1 if top_k == 1 else (top_k if (top_k is not None and top_k > 0) else 0)
    # _sample_codes (inference.py:491-504): both given -> sample_top_p_top_k, top_p alone (> 0) -> sample_top_p,
    # else top-k or the plain softmax.  A nucleus of top_p <= 0 beside a top_k holds the largest probability alone.
    p = 0.0
    if top_p is not None and (top_k is not None or top_p > 0):
        if top_p <= 0:
            k = 1
        else:
            p = float(top_p)
    sp0 = make_sample_params(temperature, k, seed, frame_ctr, keep_ties=True, top_p=p)
    rq.seed = seed

    def rq_sample(cb0_logits: Tensor, hidden: Tensor) -> Tensor:
        """inference.py:596-608: penalise, draw code 0 (sample_top_k), push it, depth head."""
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(nat.lib.vui_sample_cb0(
            nat.handle, cb0_logits.contiguous().data_ptr(), counts.data_ptr() if use_rep else None,
            hist.data_ptr() if win else None, pos2.data_ptr() if win else None, float(rep_penalty), win,
            C.byref(sp0), code0.data_ptr(), 1, st), "vui_sample_cb0")
        return state._rq_generate(hidden, code0, temperature, zero_rq_bias).clone()  # advances frame_ctr

    max_frames = int(max_secs * CODEC_HZ)
    max_per_turn = int(max_turn_secs * CODEC_HZ)
    min_frames = int(min_turn_secs * CODEC_HZ)
    max_seq = model.decoder.max_seqlen - 10
    if not resume:
        state.reset()
    total_frames = 0
    for turn_idx, chunk in enumerate(chunks):
        if state.offset >= max_seq or total_frames >= max_frames:
            break
        n = chunk.emb.shape[1]
        if state.offset + n >= max_seq:
            break
        out = _forward_flash_emb(state, chunk.emb.to(dev, state.dtype))
        hidden = out[:, -1]
        first_codes = rq_sample(model.codec_head(hidden), hidden)
        pending = first_codes[0]
        turn_frame_count = 1
        total_frames += 1
        codes_in = first_codes[0]
        for step in range(1, max_per_turn):
            if state.offset >= max_seq or total_frames >= max_frames:
                break
            hidden_next, cb0_logits, eos_logit = model.decode_step(codes_in, state.offset)
            state.offset += 1
            next_codes = rq_sample(cb0_logits, hidden_next)
            if step >= min_frames and torch.sigmoid(eos_logit.float()).item() > eos_threshold:
                break
            yield pending, None
            pending = next_codes[0]
            turn_frame_count += 1
            total_frames += 1
            codes_in = next_codes[0]
        chunk.frames = turn_frame_count
        chunk.secs = turn_frame_count / CODEC_HZ
        yield pending, chunk
    nat.status()


def render_codes_stream(state: InferenceState, chunks: "list[Chunk]", **kwargs):
    """Per-turn generator: (turn_codes (T, Q) on the CPU, chunk) (src/vui/inference.py:747-759)."""
    pending: list[Tensor] = []
    for frame, turn_end in stream_frames(state, chunks, **kwargs):
        pending.append(frame.cpu())
        if turn_end is not None:
            yield torch.stack(pending), turn_end
            pending = []


def render_audio_stream(state: InferenceState, chunks: "list[Chunk]", *, chunk_frames: int | None = None,
                        ctx_frames: int | None = None, first_chunk_frames: int | None = None, **kwargs):
    """Low-latency audio: consumes `stream_frames` and yields audio (1, 1, n * hop) every `chunk_frames` frames
    (the first emission after `first_chunk_frames`), flushing at a turn's end (src/vui/inference.py:761-830).

    The reference decodes each emission offline from its frames plus `ctx_frames` of context and cuts the context
    off; the vocoder here streams (its convolution and attention state carries the whole history), so every frame
    is decoded once, in order, and an emission is the concatenation of its frames' audio: the same schedule and the
    same number of samples, without the seam the context window approximates.  `ctx_frames` is accepted for
    callers that pass it."""
    from .codec import CodecCtx

    if state.codec is None:
        raise RuntimeError("render_audio_stream() needs InferenceState(codec=...)")
    chunk_size = chunk_frames if chunk_frames is not None else state.chunk_frames
    first_size = first_chunk_frames if first_chunk_frames is not None else chunk_size
    ctx = getattr(state, "_codec_ctx", None)
    if ctx is None:
        ctx = state._codec_ctx = CodecCtx(state.codec)
    pending: list[Tensor] = []  # audio of the frames not yet emitted
    have_emitted_first = False
    for frame, turn_end in stream_frames(state, chunks, **kwargs):
        pending.append(ctx.decode_frame(frame.view(1, -1, 1)).clone())
        target = chunk_size if have_emitted_first else first_size
        if turn_end is not None or len(pending) >= target:
            yield torch.cat(pending, dim=-1)
            pending = []
            have_emitted_first = True  # the first-chunk size applies to the first emission of the call only

