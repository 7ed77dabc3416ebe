"""Decode-loop driver over the native step.  Mirrors the decode-step surface of the
reference's Engine (src/vui/engine.py): rows/slots over one shared KV cache with a padding
slot, graph-captured batched and bucketed backbone steps, code-0 sampling with the rolling
repetition penalty, the depth-head call, and -- new here -- the whole frame as ONE graph.

Text handling, the codec/vocoder and the serving layers are outside this package: prompts
enter as embeddings or token ids.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, replace
from typing import Iterator

import torch
from torch import Tensor

from . import _lib
from .model import MAX_BATCH, Graph, SampleDev, Vui, make_sample_params

FRAME_RATE = 12.5  # codec frames per second (src/vui/qwen_codec.py:27-30)
DEFAULT_WPS = 3.0  # words per second when the prompt gives none (src/vui/engine.py:41)
GATE_RETRY_TEMPS = (0.5, 0.3)  # src/vui/engine.py:1367


@dataclass(frozen=True)
class GenConfig:
    """Sampling + generation settings; the fields the decode step reads, with the reference's
    defaults (src/vui/engine.py:60-86)."""

    temperature: float = 0.9
    top_k: int | None = 100
    top_p: float | None = None
    rep_penalty: float = 1.1
    rep_window: int = 24
    eos_threshold: float = 0.45
    min_secs: float = 0.5
    max_turn_secs: float = 15.0
    max_secs: float = 30.0
    n_codebooks: int = 0  # 0 = all Q quantizers
    max_turn_wps: float = 0.0  # >0: override the words-per-second of the chunk duration cap
    gate_frames: int = 0  # hallucination gate (engine.py:78-86): 0 = off
    gate_entropy_max: float = 1.9
    gate_retries: int = 2
    rq_top_k: int = 100  # the reference bakes top_k=100 into the RQ graphs (engine.py:393-397)
    seed: int = 0

    def max_turn_frames(self, n_words: int, prompt_wps: float = 0.0) -> int:
        """Frame cap of one chunk from its word count (src/vui/engine.py:88-103)."""
        ceil = int(self.max_turn_secs * FRAME_RATE)
        wps = self.max_turn_wps if self.max_turn_wps > 0 else prompt_wps
        if wps <= 0:
            wps = DEFAULT_WPS
        if n_words <= 0:
            return ceil
        secs = n_words / wps * 1.6 + 0.6
        return min(int(secs * FRAME_RATE), ceil)


@dataclass(frozen=True)
class Segment:
    """One voice-reference unit: a transcript and its codec codes (Segment, src/vui/engine.py:48-58).
    Tokenising is the caller's: `text_emb` (1, T, d) holds the embeddings of the cleaned, tokenised text
    (model.token_emb of its ids); `text` is kept for the words-per-second estimate.  Either part may be missing."""

    text: str = ""
    codes: Tensor | None = None  # (T, Q) long
    text_emb: Tensor | None = None


@dataclass
class Chunk:
    """One text chunk of a turn as the decode loop needs it: the embeddings of `[spk] text` (with
    `[SC]` appended on a turn's last chunk) that Engine._add_agent_text writes (src/vui/engine.py:825-844;
    tokenising and chunking the text is the caller's), the word count that caps the chunk's
    length, and the speaker-change flag of chunk_text."""

    emb: Tensor  # (1, T, d)
    n_words: int = 0
    sc: bool = False


@dataclass
class RenderRequest:
    """One request of `Engine.render_continuous` (RenderRequest, src/vui/engine.py:107-117, with the text
    side already embedded): `prompt_emb` (1, T, d) is what Row.prefill / add_user would have written (voice
    prompt, user turn), `chunks` the agent text chunk by chunk."""

    chunks: "list[Chunk]"
    prompt_emb: Tensor | None = None
    prompt_wps: float = 0.0


@dataclass
class _ActiveSlot:
    row: "Row"
    request_idx: int
    chunks: "list[Chunk]"
    chunk_idx: int = 0
    frame_count: int = 0
    turn_count: int = 0
    max_turn_frames: int = 0
    seq_offset: int = 0
    last_codes: Tensor | None = None


def _make_buckets(max_bs: int) -> list[int]:
    """src/vui/engine.py:134-142."""
    buckets, b = [], 1
    while b < max_bs:
        buckets.append(b)
        b *= 2
    if not buckets or buckets[-1] != max_bs:
        buckets.append(max_bs)
    return buckets


def _get_bucket(batch_size: int, buckets: list[int]) -> int:
    for b in buckets:
        if batch_size <= b:
            return b
    return buckets[-1]


class Row:
    """One conversation slot of the shared KV cache (src/vui/engine.py:157-270)."""

    def __init__(self, engine: "Engine", idx: int):
        self._engine = engine
        self._idx = idx
        self._prompt_offset = 0
        self._spk_token: Tensor | None = None
        self._spk_token_2: Tensor | None = None  # optional second speaker
        self._active_speaker = 0  # flipped on chunks flagged as speaker changes
        self._closed = False
        self.prompt_wps: float = 0.0
        self._slot = torch.tensor([idx], dtype=torch.int32, device=engine.device)
        # rolling vocoder context of the row (src/vui/engine.py:172); None without a codec
        self._codec_ctx = None
        if engine.codec is not None:
            from .codec import CodecCtx

            self._codec_ctx = CodecCtx(engine.codec)

    @property
    def idx(self) -> int:
        return self._idx

    @property
    def offset(self) -> int:
        return int(self._engine.seq_lens[self._idx].item())

    def prefill_emb(self, emb: Tensor) -> Tensor:
        """Write a (1, T, d) embedding block at the row's offset; returns the final-norm output
        (1, T, d).  Engine._prefill_emb, src/vui/engine.py:674-694."""
        return self._engine._prefill_emb(self, emb)

    def prefill(self, segments: "list[Segment]", spk_emb: Tensor | None = None,
                segments_2: "list[Segment] | None" = None, spk_emb_2: Tensor | None = None) -> int:
        """Prefill `[spk] text_i codes_i` for every segment, both speakers in order (Row.prefill,
        src/vui/engine.py:186-202); sets the rewind point and the words-per-second estimate."""
        return self._engine._prefill_row(self, segments, spk_emb, segments_2, spk_emb_2)

    def add_user(self, text_emb: Tensor | None = None, codes: Tensor | None = None, *, final: bool = True) -> int:
        """Write a user turn chunk: text ([SC] when final) codes (Row.add_user, src/vui/engine.py:204-208;
        the text arrives embedded)."""
        return self._engine._add_user(self, text_emb, codes, final=final)

    def render(self, chunks: "list[Chunk]", cfg: GenConfig = GenConfig()) -> "tuple[Tensor, Tensor | None]":
        """A whole turn without streaming: (codes (T, Q) on the CPU, audio (1, 1, S) or None without a vocoder)
        (Row.render, src/vui/engine.py:246-250)."""
        codes = self._engine._render_row(self, chunks, cfg)
        return codes, self._engine._decode_full(codes)

    def stream_codes(self, chunks: "list[Chunk]", cfg: GenConfig = GenConfig(), cancel=None, *, reset_rep: bool = True,
                     final_turn: bool = False) -> Iterator[Tensor]:
        """The code frames (Q',) int64 of one assistant turn, chunk by chunk: Engine._stream_row's frames before
        the vocoder (src/vui/engine.py:1308-1521).  No counterpart of its own in the reference, whose Row.stream
        hands out audio only.  cancel: object with is_set(), polled per frame."""
        if self._engine.max_rows != 1:
            raise RuntimeError(f"stream() requires Engine(max_rows=1), got {self._engine.max_rows}")
        yield from self._engine._stream_row(self, chunks, cfg, cancel, reset_rep=reset_rep, final_turn=final_turn)

    def stream(self, chunks: "list[Chunk]", cfg: GenConfig = GenConfig(), cancel=None, *, reset_rep: bool = True,
               final_turn: bool = False) -> Iterator[Tensor]:
        """Streams one assistant turn as audio, (1, 1, 1920) float per frame, as Row.stream of the reference
        does (src/vui/engine.py:211-244, 1349-1356, 1537-1546): every frame of `stream_codes` goes through the
        row's vocoder context, which is seeded once per session from the row's buffered codes.  An engine built
        without a vocoder has no audio to give: there `stream` yields the code frames themselves."""
        if self._codec_ctx is None:
            yield from self.stream_codes(chunks, cfg, cancel, reset_rep=reset_rep, final_turn=final_turn)
            return
        eng = self._engine
        if eng._split is None:
            if self._codec_ctx._stack is None:
                self._codec_ctx.prefill(n_codebooks=cfg.n_codebooks)
            for codes in self.stream_codes(chunks, cfg, cancel, reset_rep=reset_rep, final_turn=final_turn):
                yield eng._stream_decode_frame(self, codes, cfg.n_codebooks)
            return
        # divided GPU: a frame's codes are complete when stream_codes hands them out (it has waited for the step's
        # event), so the vocoder of frame f is enqueued on its own share at once and runs while the decode step of
        # frame f + 1, already in flight, finishes on the other; its audio is handed out one iteration later.  The
        # audio tensor is the vocoder's static buffer: it is overwritten when the generator is resumed.
        s_dec, s_voc = eng._split
        cur = torch.cuda.current_stream()
        s_dec.wait_stream(cur)
        s_voc.wait_stream(cur)
        with torch.cuda.stream(s_voc):
            if self._codec_ctx._stack is None:
                self._codec_ctx.prefill(n_codebooks=cfg.n_codebooks)
        it = self.stream_codes(chunks, cfg, cancel, reset_rep=reset_rep, final_turn=final_turn)
        pending = None  # (audio, event) of the vocoder step in flight
        first = True    # the first frame's audio is handed out as soon as it is done (time to the first sound)
        try:
            while True:
                with torch.cuda.stream(s_dec):
                    codes = next(it, None)
                if pending is not None:
                    audio, ev = pending
                    pending = None
                    ev.synchronize()
                    yield audio
                if codes is None:
                    break
                with torch.cuda.stream(s_voc):
                    audio = eng._stream_decode_frame(self, codes, cfg.n_codebooks)
                    ev = torch.cuda.Event()
                    ev.record(s_voc)
                if first:
                    first = False
                    ev.synchronize()
                    yield audio
                else:
                    pending = (audio, ev)
        finally:
            it.close()
            cur.wait_stream(s_dec)
            cur.wait_stream(s_voc)

    def stream_audio(self, chunks: "list[Chunk]", cfg: GenConfig = GenConfig(), cancel=None, *, reset_rep: bool = True,
                     final_turn: bool = False) -> Iterator[Tensor]:
        """`stream` on an engine that must have a vocoder (raises otherwise)."""
        if self._codec_ctx is None:
            raise RuntimeError("stream_audio() needs Engine(codec=...)")
        yield from self.stream(chunks, cfg, cancel, reset_rep=reset_rep, final_turn=final_turn)

    def mark_prompt(self) -> int:
        self._prompt_offset = self.offset
        return self._prompt_offset

    def rewind(self) -> int:
        return self._engine._rewind_row(self, self._prompt_offset)

    def reset(self) -> int:
        return self._engine._rewind_row(self, 0)

    def close(self) -> None:
        if not self._closed:
            self._engine._release_row(self)
            self._closed = True

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


_CU_STREAMS: dict = {}  # (device, first compute unit, count) -> stream bound to that range (never destroyed)


class Engine:
    """Streaming (B=1) and batched (B=N) decode over one flash-style KV cache."""

    def __init__(self, name: str | None = None, *, model: Vui | None = None, codec=None, max_rows: int = 1,
                 max_seq: int | None = None, sc_token_id: int | None = None, split_cus: int | None = None):
        if model is None:
            if name is None:
                raise ValueError("pass model= or a local checkpoint path")
            model = Vui.from_pretrained_inf(name)
        if max_rows < 1 or max_rows > MAX_BATCH:
            raise ValueError(f"max_rows must be in [1, {MAX_BATCH}]")
        self.model = model
        self.codec = codec
        self.max_rows = max_rows
        self.device = model.device
        self.dtype = model.dtype
        cfg = model.config.model
        self.Q, self.CS, self.D = cfg.n_quantizers, cfg.codebook_size, cfg.d_model
        trained = model.decoder.max_seqlen
        self.max_seq = max_seq or trained
        if self.max_seq > trained:
            raise ValueError(f"max_seq={self.max_seq} exceeds trained ceiling {trained}")
        self._cond_bias = model._cond_bias
        # embedding of the speaker-change token (src/vui/engine.py:320-324 looks its id up in the tokenizer, which
        # is not part of this package: the caller passes the id; without it no [SC] position is written)
        self._sc_emb = None
        if sc_token_id is not None:
            self._sc_emb = model.token_emb(torch.tensor([[sc_token_id]], device=self.device)).to(self.dtype)
        self._setup_graphs()
        self._setup_rep_state()
        self._free: set[int] = set(range(max_rows))
        self._rows: dict[int, Row] = {}
        self._frame_graphs: dict = {}
        self._lane_streams: list = []
        self._split = None
        if split_cus:
            self._setup_split(int(split_cus))

    # ------------------------------------------------------------------ setup
    def _setup_split(self, n: int) -> None:
        """Audio streaming on a divided GPU: the decode step's one-launch kernel runs on compute units [0, n) and
        the vocoder on the rest, each on a stream that is bound to its share (vui_cu_stream_create), so that the
        vocoder of frame f runs beside the decode step of frame f + 1 (Row.stream).  The context is limited to n
        workgroups for good and the vocoder's persistent kernel to as many as its share has compute units (a
        persistent kernel sized for the whole GPU would wait for workgroups that its share has no room for; where
        the vocoder's rows do not fit that few workgroups it runs as separate launches).  No counterpart in the reference, which
        runs the two one after the other (src/vui/engine.py:1537-1546)."""
        if self.codec is None or self.max_rows != 1:
            raise ValueError("split_cus needs Engine(codec=..., max_rows=1)")
        cus = torch.cuda.get_device_properties(self.device).multi_processor_count
        if not 0 < n < cus:
            raise ValueError(f"split_cus={n} outside (0, {cus})")
        nat = self.model._native
        streams = []
        for first, count in ((0, n), (n, cus - n)):
            key = (torch.device(self.device).index or 0, first, count)
            if key not in _CU_STREAMS:  # bound streams are kept for the life of the process: one per range
                h = C.c_void_p()
                _lib.check(nat.lib.vui_cu_stream_create(first, count, C.byref(h)), "vui_cu_stream_create")
                _CU_STREAMS[key] = torch.cuda.ExternalStream(h.value, device=self.device)
            streams.append(_CU_STREAMS[key])
        nat.workgroups(n)
        self._frame_graphs.clear()  # captured steps hold the width they were captured with
        try:  # the vocoder's persistent kernel on its share, where its rows fit that few workgroups
            self.codec.workgroups(cus - n)
            self.codec.persistent(1)
        except RuntimeError:
            self.codec.persistent(0)
        self.codec._graphs.clear()
        with torch.cuda.stream(streams[1]):
            self.codec.setup_streaming_graph(1)
        torch.cuda.synchronize()
        self._split = tuple(streams)

    def _setup_graphs(self) -> None:
        """src/vui/engine.py:375-432.  KV cache of max_rows + 1 slots (the last one is the write-only
        target of bucket padding rows), static in/out buffers, batched and bucketed step graphs."""
        model, dev, dt = self.model, self.device, self.dtype
        model.decoder.allocate_flash_kv_cache(self.max_rows + 1, dev, dt, max_seqlen=self.max_seq)
        self.seq_lens = model.decoder.flash_kv_caches[0].seq_lens
        self._pad_slot = self.max_rows
        self._buckets = _make_buckets(self.max_rows)
        rq_batch_sizes = tuple(sorted(set(self._buckets) | {1, self.max_rows}))
        model.rq_transformer.setup_cuda_graph_kv(dev, dt, top_k=100, batch_sizes=rq_batch_sizes)
        self._zero_rq_bias = torch.zeros(self.Q - 1, self.CS, device=dev, dtype=torch.float32)
        N = self.max_rows
        self._g_codes_in = torch.zeros(N, self.Q, device=dev, dtype=torch.long)
        self._g_hidden_out = torch.zeros(N, self.D, device=dev, dtype=dt)
        self._g_cb0_out = torch.zeros(N, self.CS, device=dev, dtype=dt)
        self._g_eos_out = torch.zeros(N, 1, device=dev, dtype=dt)
        self._decode_graph = None
        B_max = self._buckets[-1]
        self._gc_codes_in = torch.zeros(B_max, self.Q, device=dev, dtype=torch.long)
        self._gc_hidden_out = torch.zeros(B_max, self.D, device=dev, dtype=dt)
        self._gc_cb0_out = torch.zeros(B_max, self.CS, device=dev, dtype=dt)
        self._gc_eos_out = torch.zeros(B_max, 1, device=dev, dtype=dt)
        self._g_slot_idx = torch.full((B_max,), self._pad_slot, device=dev, dtype=torch.int32)
        self._g_seq_inc = torch.zeros(self.max_rows + 1, device=dev, dtype=torch.int32)
        self._bucketed_graphs: dict[int, Graph] = {}
        # fused frame state
        self._frame_ctr = torch.zeros(1, dtype=torch.int32, device=dev)
        self._code0 = torch.zeros(N, dtype=torch.long, device=dev)
        # device-side end-of-turn test of a streamed turn: {stopped, step}, and what a chunk start resets it to
        self._stop_state = torch.zeros(2, dtype=torch.int32, device=dev)
        self._stop_init = torch.tensor([0, 1], dtype=torch.int32, device=dev)
        self._stop_host = [torch.zeros(1, dtype=torch.int32).pin_memory() for _ in range(2)]
        # sampling settings of the captured frame step (code-0 draw, depth-head draws), read on the device
        self._sdev0, self._sdev1 = SampleDev(dev), SampleDev(dev)

    def _splits(self, B: int) -> int:
        return self.model.decoder.default_splits(B)

    def _backbone_decode_body(self, stream: int) -> None:
        """One decode step across all max_rows slots (src/vui/engine.py:434-449)."""
        B = self.max_rows
        self.model.decoder._step(codes=self._g_codes_in, emb=None, slot_idx=None, seq_inc=None, B=B,
                                 hidden_out=self._g_hidden_out, cb0_out=self._g_cb0_out, eos_out=self._g_eos_out,
                                 n_splits=self._splits(B), stream=stream)

    def _capture(self, body) -> Graph:
        """Warm once and capture; warm-up and capture advance seq_lens, so it is restored
        (src/vui/engine.py:451-471)."""
        saved = self.seq_lens.clone()
        g = Graph(self.model, body, warmup=1)
        torch.cuda.current_stream().synchronize()
        self.seq_lens.copy_(saved)
        return g

    def _decode_step(self) -> tuple[Tensor, Tensor, Tensor]:
        """Replay the batched backbone graph; returns views of the static (hidden, cb0, eos)
        buffers (src/vui/engine.py:850-853)."""
        if self._decode_graph is None:
            self._decode_graph = self._capture(self._backbone_decode_body)
        self._decode_graph.replay()
        return self._g_hidden_out, self._g_cb0_out, self._g_eos_out

    def _set_codes_in(self, row_idx: int, codes: Tensor) -> None:
        """src/vui/engine.py:473-479: frames shorter than Q are zero-padded."""
        Q_out = codes.shape[0]
        if Q_out < self.Q:
            self._g_codes_in[row_idx].zero_()
            self._g_codes_in[row_idx, :Q_out] = codes
        else:
            self._g_codes_in[row_idx] = codes

    def _backbone_decode_body_b(self, B: int, stream: int) -> None:
        """Step for B rows with slot indirection (src/vui/engine.py:485-502)."""
        self.model.decoder._step(codes=self._gc_codes_in, emb=None, slot_idx=self._g_slot_idx,
                                 seq_inc=self._g_seq_inc, B=B, hidden_out=self._gc_hidden_out,
                                 cb0_out=self._gc_cb0_out, eos_out=self._gc_eos_out, n_splits=self._splits(B),
                                 stream=stream)

    def _bucketed_decode_step(self, B_active: int) -> tuple[Tensor, Tensor, Tensor]:
        """src/vui/engine.py:525-534: pad the active rows up to the bucket with rows that write to the
        padding slot, replay that bucket's graph."""
        B_bucket = _get_bucket(B_active, self._buckets)
        self._g_slot_idx[B_active:B_bucket].fill_(self._pad_slot)
        g = self._bucketed_graphs.get(B_bucket)
        if g is None:
            saved_idx, saved_inc = self._g_slot_idx.clone(), self._g_seq_inc.clone()
            self._g_slot_idx[:B_bucket].fill_(self._pad_slot)
            self._g_seq_inc.zero_()
            g = self._capture(lambda st: self._backbone_decode_body_b(B_bucket, st))
            self._g_slot_idx.copy_(saved_idx)
            self._g_seq_inc.copy_(saved_inc)
            self._bucketed_graphs[B_bucket] = g
        g.replay()
        return self._gc_hidden_out[:B_active], self._gc_cb0_out[:B_active], self._gc_eos_out[:B_active]

    # ------------------------------------------------------------------ repetition penalty
    def _setup_rep_state(self) -> None:
        """Device-resident rolling counts (src/vui/engine.py:540-553); the ring position lives on the
        device too so that the sampler can run inside a captured graph."""
        N = self.max_rows
        self._rep_counts = torch.zeros(N, self.CS, device=self.device, dtype=torch.float32)
        self._rep_history: Tensor | None = None
        self._rep_pos = torch.zeros(N, 2, device=self.device, dtype=torch.int32)
        self._rep_window_cur = 0

    def _rep_reset(self, penalty: float, window: int) -> None:
        """src/vui/engine.py:555-569."""
        self._rep_counts.zero_()
        self._rep_pos.zero_()
        if penalty <= 1.0:
            return
        if window > 0 and (self._rep_history is None or self._rep_window_cur != window):
            self._rep_history = torch.zeros(self.max_rows, window, device=self.device, dtype=torch.int32)
            self._rep_window_cur = window
            self._frame_graphs = {}
        elif window > 0:
            self._rep_history.zero_()

    def _sample_cb0(self, logits: Tensor, cfg: GenConfig, *, top_k: int | None = -1, frame_ctr: Tensor | None = None,
                    out: Tensor | None = None) -> Tensor:
        """Penalise (when cfg.rep_penalty > 1), sample and push: the three steps of
        src/vui/engine.py:571-590 and 855-863 in one kernel.  (N, CS) -> (N,)."""
        B = logits.shape[0]
        nat = self.model._native
        k = cfg.top_k if top_k == -1 else top_k
        sp = make_sample_params(cfg.temperature, k, cfg.seed, frame_ctr if frame_ctr is not None else self._frame_ctr)
        out = out if out is not None else torch.empty(B, dtype=torch.long, device=self.device)
        use_rep = cfg.rep_penalty > 1.0
        win = cfg.rep_window if (use_rep and self._rep_history is not None) else 0
        _lib.check(nat.lib.vui_sample_cb0(
            nat.handle, logits.contiguous().data_ptr(), self._rep_counts.data_ptr() if use_rep else None,
            _lib.ptr(self._rep_history) if win else None, self._rep_pos.data_ptr() if win else None,
            float(cfg.rep_penalty), win, C.byref(sp), out.data_ptr(), B, torch.cuda.current_stream().cuda_stream),
            "vui_sample_cb0")
        return out

    # ------------------------------------------------------------------ rows
    def new_row(self) -> Row:
        if not self._free:
            raise RuntimeError(f"No free rows (max_rows={self.max_rows} all in use)")
        idx = min(self._free)
        self._free.remove(idx)
        row = Row(self, idx)
        self._rows[idx] = row
        self.seq_lens[idx] = 0
        return row

    def _release_row(self, row: Row) -> None:
        self._rows.pop(row.idx, None)
        self._free.add(row.idx)
        if row._codec_ctx is not None:
            row._codec_ctx.reset()

    def _stream_decode_frame(self, row: Row, frame_codes: Tensor, n_codebooks: int) -> Tensor:
        """One frame of codes (Q',) -> audio through the row's vocoder context; fewer codebooks are
        decoded as such but stored zero-padded to Q (src/vui/engine.py:1537-1546)."""
        if frame_codes.shape[0] < self.Q:
            padded = torch.zeros(self.Q, device=self.device, dtype=frame_codes.dtype)
            padded[: frame_codes.shape[0]] = frame_codes
            frame_codes = padded
        codes_t = frame_codes.unsqueeze(0).unsqueeze(-1)
        decode_codes = codes_t[:, :n_codebooks] if n_codebooks > 0 else codes_t
        return row._codec_ctx.decode_frame(decode_codes, store_codes=codes_t)

    def reset(self) -> None:
        for row in list(self._rows.values()):
            row.close()
        self.seq_lens.zero_()

    def _rewind_row(self, row: Row, offset: int) -> int:
        """KV rewind = overwrite one int32; K/V beyond it are never cleared (engine.py:651-654)."""
        self.seq_lens[row.idx] = offset
        return offset

    def _prefill_emb(self, row: Row, emb: Tensor, offset: int | None = None, lane: int = 0) -> Tensor:
        """offset: the row's current length when the caller keeps count of it (saves reading it back from
        the device, a synchronisation).  lane: see Decoder._prefill."""
        T = emb.shape[1]
        off = row.offset if offset is None else offset
        if off + T > self.max_seq:
            raise ValueError(f"prefill of {T} positions at offset {off} exceeds max_seq={self.max_seq}")
        pos = torch.arange(off, off + T, device=self.device)
        return self.model.decoder.forward_flash(emb.to(self.dtype), pos, slot_idx=row._slot,
                                                known=(row.idx, off) if offset is not None else None, lane=lane)

    max_frame_graphs = 32  # captured frame graphs kept (oldest dropped first)
    prefill_lanes = 4  # streams that ingest the blocks of different rows at once (1: one after the other)

    def _prefill_many(self, jobs: "list[tuple[Row, Tensor, int]]") -> "list[Tensor]":
        """Blocks (row, embeddings, the row's length) of different rows through the prompt-ingestion pass.  Rows
        share nothing but read-only weights, and a short block's kernels fill a fraction of the GPU, so several
        blocks go out on side streams (default priority, a scratch buffer each) and the calling stream waits for
        all of them.  The results do not depend on how many lanes there are."""
        dec = self.model.decoder
        lanes = min(self.prefill_lanes, len(jobs))
        if lanes < 2 or not dec._prefill_available() or any(e.shape[1] < dec.PREFILL_MIN for _, e, _ in jobs):
            return [self._prefill_emb(r, e, offset=o) for r, e, o in jobs]
        main = torch.cuda.current_stream()
        if len(self._lane_streams) < lanes:
            self._lane_streams += [torch.cuda.Stream(device=self.device) for _ in range(lanes - len(self._lane_streams))]
        used = self._lane_streams[:lanes]
        start = main.record_event()
        for s in used:
            s.wait_event(start)
        outs = []
        for i, (r, e, o) in enumerate(jobs):
            with torch.cuda.stream(used[i % lanes]):
                h = self._prefill_emb(r, e, offset=o, lane=1 + i % lanes)
                h.record_stream(main)
            outs.append(h)
        for s in used:
            main.wait_stream(s)
        return outs

    def set_conditioning(self, *, sq_scores=None, wps_score: float = 0.0) -> None:
        self.model.set_cond_bias(sq_scores=sq_scores, wps_score=wps_score)
        self._cond_bias = self.model._cond_bias

    # ------------------------------------------------------------------ fused frame loop
    def _frame_graph(self, B: int, cfg: GenConfig, slot_idx: Tensor | None, max_frames: int,
                     stop: "tuple[float, int] | None" = None):
        """One HIP graph holding a whole frame: backbone step on the previous frame, code-0
        sampling with repetition penalty, the depth head, frame log, counters.  stop = (eos_threshold,
        min_frames): the step also runs the end-of-turn test on the device (self._stop_state)."""
        nq = cfg.n_codebooks if cfg.n_codebooks > 0 else self.Q
        # temperature, top-k values and seed live in two device blocks the step reads when it runs, so that a
        # request with another seed or temperature replays the same graph (the reference captures once, too)
        self._sdev0.set(cfg.temperature, cfg.top_k, cfg.seed)
        self._sdev1.set(cfg.temperature, cfg.rq_top_k if cfg.top_k != 1 else 1, cfg.seed)
        # the frame log is sized in powers of two from 256 frames, so that runs of different lengths share a graph
        max_frames = 0 if max_frames <= 0 else max(256, 1 << (max_frames - 1).bit_length())
        key = (B, nq, cfg.rep_penalty, cfg.rep_window, None if slot_idx is None else tuple(slot_idx.tolist()), max_frames, stop)
        hit = self._frame_graphs.get(key)
        if hit is not None:
            self._frame_graphs[key] = self._frame_graphs.pop(key)  # most recently used last
            return hit
        nat = self.model._native
        dec = self.model.decoder
        # max_frames == 0: no frame log, eos holds the (B) probabilities of the latest step
        frames = torch.zeros(max_frames, B, self.Q, dtype=torch.long, device=self.device) if max_frames else None
        eos = torch.zeros(max(max_frames, 1), B, dtype=torch.float32, device=self.device)
        sp0 = make_sample_params(cfg.temperature, cfg.top_k, cfg.seed, self._frame_ctr, dev=self._sdev0)
        sp1 = make_sample_params(cfg.temperature, cfg.rq_top_k if cfg.top_k != 1 else 1, cfg.seed, self._frame_ctr, dev=self._sdev1)
        use_rep = cfg.rep_penalty > 1.0
        win = cfg.rep_window if (use_rep and self._rep_history is not None) else 0
        codes_io = self._gc_codes_in if slot_idx is not None else self._g_codes_in
        ns = self._splits(B)
        stop_c = None
        if stop is not None:
            stop_c = _lib.EosStopC()
            stop_c.threshold, stop_c.min_frames, stop_c.state = float(stop[0]), int(stop[1]), self._stop_state.data_ptr()

        def body(st):
            _lib.check(nat.lib.vui_frame_step(
                nat.handle, codes_io.data_ptr(), _lib.ptr(slot_idx), self.seq_lens.data_ptr(), None, B,
                dec._k.data_ptr(), dec._v.data_ptr(), self._rep_counts.data_ptr() if use_rep else None,
                _lib.ptr(self._rep_history) if win else None, self._rep_pos.data_ptr() if win else None,
                float(cfg.rep_penalty), win, C.byref(sp0), C.byref(sp1), None, nq, self._g_hidden_out.data_ptr(),
                self._g_cb0_out.data_ptr(), eos.data_ptr(), _lib.ptr(frames), max_frames,
                self._frame_ctr.data_ptr(), ns, C.byref(stop_c) if stop_c is not None else None, st), "vui_frame_step")

        # captured without a warm-up run: the step mutates seq_lens, the rep state and the counter
        g = Graph(self.model, body, warmup=0)
        entry = (g, frames, eos, (sp0, sp1, slot_idx, stop_c))
        if len(self._frame_graphs) >= self.max_frame_graphs:  # shapes, not settings, key a graph; still bounded
            self._frame_graphs.pop(next(iter(self._frame_graphs)))
        self._frame_graphs[key] = entry
        return entry

    @torch.inference_mode()
    def generate(self, rows: list[Row], first_hidden: Tensor, n_frames: int, cfg: GenConfig = GenConfig(),
                 *, sync_every: int = 0) -> tuple[Tensor, Tensor]:
        """Generate n_frames codec frames for the given rows, starting from the final-norm hidden
        of each row's last prefill position (B, d).

        Frame 0 follows src/vui/engine.py:1414-1433 (code 0 from codec_head(hidden), sampled without
        top-k unless greedy; depth head; feed back); frames 1.. replay the one-graph frame step
        (engine.py:1450-1485).  Returns (frames (n_frames, B, Q') int64, eos_prob (n_frames, B) fp32;
        row 0 of eos_prob is 0).  EOS is reported, not acted on: the caller truncates."""
        B = len(rows)
        nq = cfg.n_codebooks if cfg.n_codebooks > 0 else self.Q
        identity = [r.idx for r in rows] == list(range(B))
        slot_idx = None if identity else torch.tensor([r.idx for r in rows], dtype=torch.int32, device=self.device)
        codes_io = self._g_codes_in if identity else self._gc_codes_in
        self._rep_reset(cfg.rep_penalty, cfg.rep_window)
        self._frame_ctr.zero_()
        # frame 0
        cb0 = self.model.codec_head(first_hidden.to(self.dtype))
        k0 = 1 if cfg.top_k == 1 else 0
        code0 = self._sample_cb0(cb0, cfg, top_k=k0)
        rq = self.model.rq_transformer
        rq.seed = cfg.seed
        sp1 = make_sample_params(cfg.temperature, cfg.rq_top_k if cfg.top_k != 1 else 1, cfg.seed, self._frame_ctr)
        nat = self.model._native
        _lib.check(nat.lib.vui_rq_generate(nat.handle, first_hidden.to(self.dtype).contiguous().data_ptr(),
                                           code0.data_ptr(), None, nq, C.byref(sp1), codes_io.data_ptr(), self.Q, 1, B,
                                           torch.cuda.current_stream().cuda_stream), "vui_rq_generate")
        first = codes_io[:B, :nq].clone()
        self._frame_ctr.fill_(1)
        if n_frames <= 1:
            return first[None], torch.zeros(1, B, device=self.device)
        g, frames, eos, _ = self._frame_graph(B, cfg, slot_idx, max(n_frames, 1))
        # the capture above ran nothing, state is as left by frame 0
        frames[0, :, :nq] = first
        for f in range(1, n_frames):
            g.replay()
            if sync_every and f % sync_every == 0:
                torch.cuda.current_stream().synchronize()
        torch.cuda.current_stream().synchronize()
        nat.status()  # a persistent launch that gave up a wait committed nothing: raise instead of returning stale frames
        return frames[:n_frames, :, :nq].clone(), eos[:n_frames].clone()

    # ------------------------------------------------------------------ prompt, user turn
    def _audio_emb(self, codes: Tensor) -> Tensor:
        pc = codes.to(self.device)
        if pc.dim() == 2:
            pc = pc.unsqueeze(0)
        return self.model.embed_audio(pc).to(self.dtype)

    def _embed_speaker(self, spk_emb: Tensor | None) -> Tensor | None:
        if spk_emb is None or self.model.spk_proj is None:
            return None
        return self.model.embed_speaker(spk_emb).to(self.dtype)

    def _prefill_speaker_segments(self, row: Row, segments: "list[Segment]", spk_token: Tensor | None, *,
                                  final: bool = False) -> None:
        """src/vui/engine.py:725-741: `[spk] text_i ([SC] before the last audio) codes_i` per segment."""
        last = len(segments) - 1
        for i, seg in enumerate(segments):
            if spk_token is not None:
                self._prefill_emb(row, spk_token)
            if seg.text_emb is not None and seg.text_emb.shape[1] > 0:
                self._prefill_emb(row, seg.text_emb.to(self.device, self.dtype))  # prompt text carries no cond_bias
            if final and i == last and self._sc_emb is not None:
                self._prefill_emb(row, self._sc_emb)
            if seg.codes is not None:
                self._prefill_emb(row, self._audio_emb(seg.codes))

    @torch.inference_mode()
    def _prefill_row(self, row: Row, segments: "list[Segment]", spk_emb: Tensor | None,
                     segments_2: "list[Segment] | None" = None, spk_emb_2: Tensor | None = None) -> int:
        """Engine._prefill_row, src/vui/engine.py:743-796."""
        row._spk_token = self._embed_speaker(spk_emb)
        row._spk_token_2 = self._embed_speaker(spk_emb_2)
        row._active_speaker = 0
        all_segs = list(segments) + (list(segments_2) if segments_2 else [])
        all_codes = [seg.codes for seg in all_segs if seg.codes is not None]
        if all_codes and row._codec_ctx is not None:  # seed the row's vocoder context with every prompt code
            row._codec_ctx.set_prompt(torch.cat([c.to(self.device) for c in all_codes], dim=0).T.unsqueeze(0))
        self._prefill_speaker_segments(row, segments, row._spk_token, final=True)
        if segments_2 is not None:
            self._prefill_speaker_segments(row, segments_2, row._spk_token_2, final=True)
        row._prompt_offset = row.offset
        total_words = sum(len(seg.text.split()) for seg in all_segs if seg.text)
        total_frames = sum(seg.codes.shape[0] for seg in all_segs if seg.codes is not None)
        if total_frames > 0 and total_words > 0:
            row.prompt_wps = total_words / (total_frames / FRAME_RATE)
        return row._prompt_offset

    @torch.inference_mode()
    def _add_user(self, row: Row, text_emb: Tensor | None, codes: Tensor | None, *, final: bool = True) -> int:
        """Engine._add_user, src/vui/engine.py:798-826: text ([SC] when final) codes.  The text arrives embedded
        (the reference adds model.noisy_emb to user text; the caller folds it in)."""
        if text_emb is not None and text_emb.shape[1] > 0:
            self._prefill_emb(row, text_emb.to(self.device, self.dtype))
        if final and self._sc_emb is not None:
            self._prefill_emb(row, self._sc_emb)
        if codes is not None:
            self._prefill_emb(row, self._audio_emb(codes))
            if row._codec_ctx is not None:
                row._codec_ctx.add(codes.T.unsqueeze(0).to(self.device))
        return row.offset

    def _decode_full(self, codes: Tensor) -> Tensor | None:
        """(T, Q) codes -> (1, 1, S) audio through the vocoder's offline pass (Engine._decode_full); None when
        the engine has no vocoder."""
        if self.codec is None:
            return None
        if codes.shape[0] == 0:
            return torch.zeros(1, 1, 0, device=self.device)
        return self.codec(codes.to(self.device).T.unsqueeze(0))

    # ------------------------------------------------------------------ batched offline render
    @torch.inference_mode()
    def _render_rows(self, rows: "list[Row]", chunk_lists: "list[list[Chunk]]", cfg: GenConfig) -> "dict[int, Tensor]":
        """Core batched decode loop of render()/render_all() (Engine._render_rows, src/vui/engine.py:865-1087):
        {row.idx: (T, Q) codes on the CPU}.  Every row has been prefilled; per chunk the agent text is written and
        the first frame drawn without a top-k cut, then all max_rows slots step together (one batched backbone
        step, code 0 with each row's rolling repetition state, EOS flags read on the host, one batched depth-head
        call) until every row has used its chunks, max_secs, or the cache.  A chunk that ends with fewer than two
        frames per word is rewound and drawn again colder (0.5, then 0.3).

        Where this differs from the reference, by necessity: texts arrive as chunks of embeddings; draws come from
        the counter-based generator, one counter step per chunk start and per decode step; a chunk start uses the
        repetition state of its own row (the reference broadcasts one row's logits against all rows' counts there,
        which only works for max_rows == 1 or without a penalty).  With max_rows == 1 the step is the one-launch
        frame graph and the frames equal what Row.stream yields for the same chunks (the invariant the reference
        states at engine.py:1001-1008) as long as neither the stream's gate nor this loop's retry fires."""
        model, nat = self.model, self.model._native
        N = self.max_rows
        max_frames = int(cfg.max_secs * FRAME_RATE)
        min_frames = int(cfg.min_secs * FRAME_RATE)
        max_seq = self.max_seq - 10
        nq = cfg.n_codebooks if cfg.n_codebooks > 0 else self.Q
        greedy = cfg.top_k == 1
        use_rep = cfg.rep_penalty > 1.0
        stream = torch.cuda.current_stream()
        row_chunks = {r.idx: list(ch) for r, ch in zip(rows, chunk_lists)}
        row_chunk_idx = {r.idx: 0 for r in rows}
        row_frame_count = {r.idx: 0 for r in rows}
        row_turn_count = {r.idx: 0 for r in rows}
        row_max_turn = {r.idx: cfg.max_turn_frames(0, r.prompt_wps) for r in rows}
        row_offset = {r.idx: r.offset for r in rows}  # host-side count of every row's cache length
        row_chunk_offset: dict[int, int] = {}
        row_retry_idx = {r.idx: 0 for r in rows}
        frame_buf = torch.zeros(N, max(max_frames, 1), self.Q, device=self.device, dtype=torch.long)
        active = {r.idx: True for r in rows}
        self._rep_reset(cfg.rep_penalty, cfg.rep_window)
        self._frame_ctr.zero_()
        MIN_FPW = 2.0
        RETRY_TEMPS = (0.5, 0.3)
        single = N == 1 and nat.fused(-1)  # one row on the one-launch form: the frame graph is the step
        rq_out = torch.zeros(N, self.Q, dtype=torch.long, device=self.device)

        def advance_turn(row: Row, temp: float | None = None) -> bool:
            """Write the next chunk's text and draw its first frame (engine.py:909-950); False without a chunk."""
            ci = row_chunk_idx[row.idx]
            chunks = row_chunks[row.idx]
            if ci >= len(chunks) or row_frame_count[row.idx] >= max_frames:
                return False
            chunk = chunks[ci]
            if chunk.sc and row._spk_token_2 is not None:
                row._active_speaker = 1 - row._active_speaker
            row_max_turn[row.idx] = cfg.max_turn_frames(chunk.n_words, row.prompt_wps)
            row_chunk_offset[row.idx] = row_offset[row.idx]
            t = temp or cfg.temperature
            hidden = self._prefill_emb(row, chunk.emb, offset=row_offset[row.idx])[:, -1]
            row_offset[row.idx] += chunk.emb.shape[1]
            cb0 = model.codec_head(hidden)
            sp0 = make_sample_params(t, 1 if greedy else 0, cfg.seed, self._frame_ctr, state_rows=row._slot)
            code0 = torch.empty(1, dtype=torch.long, device=self.device)
            win = cfg.rep_window if (use_rep and self._rep_history is not None) else 0
            _lib.check(nat.lib.vui_sample_cb0(
                nat.handle, cb0.contiguous().data_ptr(), self._rep_counts.data_ptr() if use_rep else None,
                _lib.ptr(self._rep_history) if win else None, self._rep_pos.data_ptr() if win else None,
                float(cfg.rep_penalty), win, C.byref(sp0), code0.data_ptr(), 1, stream.cuda_stream), "vui_sample_cb0")
            sp1 = make_sample_params(t, cfg.rq_top_k if not greedy else 1, cfg.seed, self._frame_ctr, state_rows=None)
            _lib.check(nat.lib.vui_rq_generate(nat.handle, hidden.contiguous().data_ptr(), code0.data_ptr(), None, nq,
                                               C.byref(sp1), rq_out.data_ptr(), self.Q, 1, 1, stream.cuda_stream),
                       "vui_rq_generate")
            self._frame_ctr += 1
            self._g_codes_in[row.idx] = rq_out[0]
            frame_buf[row.idx, row_frame_count[row.idx]] = rq_out[0]
            row_frame_count[row.idx] += 1
            row_turn_count[row.idx] = 1
            return True

        def retry_chunk(row: Row) -> bool:
            """engine.py:952-983: fewer than two frames per word -> rewind the chunk and draw it again colder."""
            ci = row_chunk_idx[row.idx]
            n_words = row_chunks[row.idx][ci].n_words
            turn_n = row_turn_count[row.idx]
            fpw = turn_n / n_words if n_words > 0 else 999
            if fpw >= MIN_FPW:
                row_retry_idx[row.idx] = 0
                return False
            ri = row_retry_idx[row.idx]
            if ri >= len(RETRY_TEMPS):
                row_retry_idx[row.idx] = 0
                return False
            row_retry_idx[row.idx] = ri + 1
            self.seq_lens[row.idx] = row_chunk_offset[row.idx]
            row_offset[row.idx] = row_chunk_offset[row.idx]
            row_frame_count[row.idx] -= turn_n
            self._rep_reset(cfg.rep_penalty, cfg.rep_window)
            advance_turn(row, temp=RETRY_TEMPS[ri])
            return True

        def next_chunk(row: Row) -> None:
            if retry_chunk(row):
                return
            row_retry_idx[row.idx] = 0
            row_chunk_idx[row.idx] += 1
            if not advance_turn(row):
                active[row.idx] = False

        for r in rows:
            if not advance_turn(r):
                active[r.idx] = False
        g1 = eos1 = None
        if single:
            g1, _, eos1, _ = self._frame_graph(1, cfg, None, 0)
        sp_rq = make_sample_params(cfg.temperature, cfg.rq_top_k if not greedy else 1, cfg.seed, self._frame_ctr)
        total_steps = 0
        while any(active.values()) and total_steps < max_frames:
            # a row whose chunk reached its frame cap moves on before the step (engine.py:1001-1019)
            for r in rows:
                if active[r.idx] and row_turn_count[r.idx] >= row_max_turn[r.idx]:
                    next_chunk(r)
            if not any(active.values()):
                break
            if single:
                g1.replay()  # backbone step, code 0 (+ push), depth head; the new frame is in _g_codes_in
                p0 = eos1[0, 0].item()
                if p0 < 0.0:
                    nat.status()
                    raise RuntimeError("frame step failed without a raised error word")
                eos_cpu = [p0]
                frames_all = self._g_codes_in
            else:
                hidden_all, cb0_all, eos_all = self._decode_step()
                code0s = self._sample_cb0(cb0_all, cfg)
                eos_cpu = torch.sigmoid(eos_all.float()).flatten().cpu().tolist()
                nat.status()
                _lib.check(nat.lib.vui_rq_generate(nat.handle, hidden_all.data_ptr(), code0s.data_ptr(), None, nq,
                                                   C.byref(sp_rq), rq_out.data_ptr(), self.Q, 1, N, stream.cuda_stream),
                           "vui_rq_generate")
                self._frame_ctr += 1
                frames_all = rq_out
            total_steps += 1
            for r in rows:
                row_offset[r.idx] += 1  # every slot of the batched step advances
            hit = []
            for r in rows:
                if not active[r.idx]:
                    continue
                if row_offset[r.idx] >= max_seq or row_frame_count[r.idx] >= max_frames:
                    active[r.idx] = False
                    continue
                turn_n = row_turn_count[r.idx]
                if turn_n >= min_frames and eos_cpu[r.idx] > cfg.eos_threshold:
                    hit.append(r)
                    continue
                frame_buf[r.idx, row_frame_count[r.idx]] = frames_all[r.idx]
                if not single:
                    self._g_codes_in[r.idx] = frames_all[r.idx]
                row_frame_count[r.idx] += 1
                row_turn_count[r.idx] += 1
            for r in hit:
                next_chunk(r)
        # the batched depth head of the last step (or of a chunk start behind it) has not been checked yet: a
        # persistent launch that gave up a wait raised the error word, and its codes must not be returned as results
        stream.synchronize()
        nat.status()
        result: dict[int, Tensor] = {}
        for r in rows:
            n = row_frame_count[r.idx]
            if n > 0:
                result[r.idx] = frame_buf[r.idx, :n, :nq].cpu()
        return result

    def _render_row(self, row: Row, chunks: "list[Chunk]", cfg: GenConfig) -> Tensor:
        """Engine._render_row, src/vui/engine.py:1089-1092."""
        nq = cfg.n_codebooks if cfg.n_codebooks > 0 else self.Q
        return self._render_rows([row], [chunks], cfg).get(row.idx, torch.zeros(0, nq, dtype=torch.long))

    def render_all(self, rows: "list[Row]", chunk_lists: "list[list[Chunk]]", cfg: GenConfig = GenConfig()) -> list:
        """Batched non-streaming render (Engine.render_all, src/vui/engine.py:1094-1106): one audio tensor per row
        when the engine has a vocoder, else the (T, Q) codes of every row."""
        results = self._render_rows(rows, chunk_lists, cfg)
        nq = cfg.n_codebooks if cfg.n_codebooks > 0 else self.Q
        out = []
        for r in rows:
            codes = results.get(r.idx, torch.zeros(0, nq, dtype=torch.long))
            out.append(self._decode_full(codes) if self.codec is not None else codes)
        return out

    # ------------------------------------------------------------------ continuous batching
    @torch.inference_mode()
    def render_continuous(self, requests: "list[RenderRequest]", cfg: GenConfig = GenConfig()) -> list[Tensor]:
        """Continuous batching over bucketed step graphs (Engine.render_continuous,
        src/vui/engine.py:1112-1302): more requests than rows are accepted, a slot is freed when its
        request ends and refilled from the queue at once.  Per step: one bucketed backbone step with slot
        indirection (padding rows write to the spare slot), code 0 per active slot with the slot's own
        repetition counts (no window here, engine.py:594-616), EOS flags, one batched depth-head call at the
        bucket size, then per-slot bookkeeping (EOS after min_secs or the chunk's frame cap start the next
        chunk; max_secs or the cache limit end the request).  Returns the codes (T_i, Q') of every request in
        input order (the reference decodes them to audio with the offline vocoder pass)."""
        if not requests:
            return []
        model, nat = self.model, self.model._native
        max_frames = int(cfg.max_secs * FRAME_RATE)
        min_frames = int(cfg.min_secs * FRAME_RATE)
        max_seq = self.max_seq - 10
        nq = cfg.n_codebooks if cfg.n_codebooks > 0 else self.Q
        greedy = cfg.top_k == 1
        use_rep = cfg.rep_penalty > 1.0
        frame_bufs: list[list[Tensor]] = [[] for _ in requests]
        pending = list(range(len(requests)))
        active: dict[int, _ActiveSlot] = {}
        self._rep_counts.zero_()
        self._frame_ctr.zero_()
        stream = torch.cuda.current_stream()
        sp_rq = make_sample_params(cfg.temperature, cfg.rq_top_k if not greedy else 1, cfg.seed, self._frame_ctr)
        one_slot = torch.zeros(1, dtype=torch.int32, device=self.device)
        rq_code0 = torch.zeros(self._buckets[-1], dtype=torch.long, device=self.device)
        rq_out = torch.zeros(self._buckets[-1], self.Q, dtype=torch.long, device=self.device)
        # the latest frame of every slot (zero beyond nq), so that a step's input is one gather; the host keeps
        # count of every row's length instead of reading it back
        last = torch.zeros(self.max_rows + 1, self.Q, dtype=torch.long, device=self.device)

        def sample(cb0: Tensor, slots: Tensor, top_k: int, out: Tensor | None = None) -> Tensor:
            B = cb0.shape[0]
            sp = make_sample_params(cfg.temperature, top_k, cfg.seed, self._frame_ctr, state_rows=slots)
            out = out if out is not None else torch.empty(B, dtype=torch.long, device=self.device)
            _lib.check(nat.lib.vui_sample_cb0(nat.handle, cb0.contiguous().data_ptr(),
                                              self._rep_counts.data_ptr() if use_rep else None, None, None,
                                              float(cfg.rep_penalty), 0, C.byref(sp), out.data_ptr(), B, stream.cuda_stream),
                       "vui_sample_cb0")
            return out

        def depth_head(hidden: Tensor, code0: Tensor, B: int) -> Tensor:
            _lib.check(nat.lib.vui_rq_generate(nat.handle, hidden.contiguous().data_ptr(), code0.data_ptr(), None, nq,
                                               C.byref(sp_rq), rq_out.data_ptr(), self.Q, 1, B, stream.cuda_stream),
                       "vui_rq_generate")
            return rq_out[:B, :nq]

        def advance_slots(infos: "list[_ActiveSlot]") -> "list[bool]":
            """Write the next chunk's text of every given slot and draw its first frame; False where no chunk is
            left.  The slots that advance in the same step share one codec-head call, one code-0 draw and one
            depth-head call (rows are independent: a burst of sixteen costs one batched depth head instead of
            sixteen single ones)."""
            ok = [info.chunk_idx < len(info.chunks) for info in infos]
            ready = [info for info, k in zip(infos, ok) if k]
            if not ready:
                return ok
            jobs = []
            for info in ready:
                chunk = info.chunks[info.chunk_idx]
                info.max_turn_frames = cfg.max_turn_frames(chunk.n_words, info.row.prompt_wps)
                jobs.append((info.row, chunk.emb, info.seq_offset))
                info.seq_offset += chunk.emb.shape[1]
            hiddens = [h[:, -1] for h in self._prefill_many(jobs)]
            n = len(ready)
            hidden = hiddens[0] if n == 1 else torch.cat(hiddens, dim=0)
            cb0 = model.codec_head(hidden)
            slots = torch.tensor([info.row.idx for info in ready], dtype=torch.int32, device=self.device)
            code0 = sample(cb0, slots, 1 if greedy else 0)
            frames = depth_head(hidden, code0, n)[:n].clone()
            last[slots.long(), :nq] = frames
            self._frame_ctr += 1
            for i, info in enumerate(ready):
                info.last_codes = frames[i]
                frame_bufs[info.request_idx].append(info.last_codes)
                info.frame_count += 1
                info.turn_count = 1
            return ok

        def backfill() -> None:
            while pending and self._free:  # again while rows closed below leave room for waiting requests
                prompts, taken = [], []
                while pending and self._free:
                    req_idx = pending.pop(0)
                    req = requests[req_idx]
                    row = self.new_row()
                    self._rep_counts[row.idx].zero_()
                    row.prompt_wps = req.prompt_wps
                    off = 0  # new_row starts the slot at length zero
                    if req.prompt_emb is not None and req.prompt_emb.shape[1] > 0:
                        prompts.append((row, req.prompt_emb, 0))
                        off = req.prompt_emb.shape[1]
                    taken.append((row, req_idx, req, off))
                self._prefill_many(prompts)
                admitted: "list[_ActiveSlot]" = []
                for row, req_idx, req, off in taken:
                    if not req.chunks:
                        row.close()
                        continue
                    admitted.append(_ActiveSlot(row=row, request_idx=req_idx, chunks=req.chunks, seq_offset=off))
                for info, k in zip(admitted, advance_slots(admitted)):
                    if k:
                        active[info.row.idx] = info
                    else:
                        info.row.close()

        backfill()
        prev_slots: list[int] = []
        slots_t = slots_l = None
        while active:
            slot_list = sorted(active)
            B_active = len(slot_list)
            B_bucket = _get_bucket(B_active, self._buckets)
            if slot_list != prev_slots:  # membership changes only when a request ends or starts
                slots_t = torch.tensor(slot_list, dtype=torch.int32, device=self.device)
                slots_l = slots_t.long()
                self._g_slot_idx[:B_active] = slots_t
                self._g_seq_inc.zero_()
                self._g_seq_inc[slots_l] = 1
                prev_slots = slot_list
            torch.index_select(last, 0, slots_l, out=self._gc_codes_in[:B_active])
            hidden_all, cb0_all, eos_all = self._bucketed_decode_step(B_active)
            for slot in slot_list:
                active[slot].seq_offset += 1
            sample(cb0_all, slots_t, cfg.top_k, out=rq_code0[:B_active])
            eos_flags = (torch.sigmoid(eos_all.float()).flatten() > cfg.eos_threshold).cpu()
            nat.status()  # the stream is idle here: the steps so far (persistent depth head included) are complete
            frames_all = depth_head(self._gc_hidden_out[:B_bucket], rq_code0, B_bucket)[:B_active].clone()
            last[slots_l, :nq] = frames_all  # a slot that starts a new chunk below overwrites its row
            self._frame_ctr += 1
            to_remove: list[int] = []
            turning: "list[_ActiveSlot]" = []  # slots whose chunk ended with this step
            for qi, slot in enumerate(slot_list):
                info = active[slot]
                if info.frame_count >= max_frames or info.seq_offset >= max_seq:
                    to_remove.append(slot)
                    continue
                turn_n = info.turn_count
                if (turn_n >= min_frames and bool(eos_flags[qi])) or turn_n >= info.max_turn_frames:
                    info.chunk_idx += 1
                    turning.append(info)
                    continue
                info.last_codes = frames_all[qi]
                frame_bufs[info.request_idx].append(info.last_codes)
                info.frame_count += 1
                info.turn_count += 1
            for info, k in zip(turning, advance_slots(turning)):
                if not k:
                    to_remove.append(info.row.idx)
            for slot in to_remove:
                active.pop(slot).row.close()
            backfill()
        stream.synchronize()
        nat.status()  # the last step's depth head and the chunk starts behind it
        return [torch.stack(b) if b else torch.zeros(0, nq, dtype=torch.long, device=self.device) for b in frame_bufs]

    # ------------------------------------------------------------------ streaming single-row turn
    def _penalised_probs(self, cb0: Tensor, counts: Tensor, cfg: GenConfig, temp: float) -> Tensor:
        """softmax(rep_apply(cb0) / temp) as the reference forms it for the gate statistics
        (src/vui/engine.py:571-576, 1412, 1455)."""
        lf = cb0.float()
        if cfg.rep_penalty > 1.0:
            factor = torch.pow(torch.tensor(cfg.rep_penalty, device=lf.device), counts)
            lf = torch.where(lf > 0, lf / factor, lf * factor)
        return torch.softmax(lf / temp, dim=-1)

    @torch.inference_mode()
    def _stream_row(self, row: Row, chunks: "list[Chunk]", cfg: GenConfig, cancel=None, *, reset_rep: bool = True,
                    final_turn: bool = False) -> Iterator[Tensor]:
        """Per-frame streaming decode of one row; yields (Q',) int64 code frames.

        The control flow of src/vui/engine.py:1308-1521: per chunk write its text, draw frame 0 from
        the text's last hidden state (no top-k, engine.py:1411-1424), then one decode step per frame
        until the EOS probability passes cfg.eos_threshold (after min_secs), the chunk's word-count
        cap, cfg.max_secs or the cache limit; the optional gate holds the first cfg.gate_frames
        frames of the first chunk, and on high mean entropy rewinds the cache to the chunk start and
        retries colder.  A frame step here is one graph replay that also runs the depth head; when
        the EOS test then ends the chunk, that frame is dropped (the reference tests before its depth
        head runs: same frames out).  The EOS test itself runs on the device (vui_eos_stop), the host reads
        its flag one frame late; after a cancel the cache may hold one position more than the reference's
        (a step already in flight), callers rewind after a cancel."""
        if not chunks:
            return
        max_frames = int(cfg.max_secs * FRAME_RATE)
        min_frames = int(cfg.min_secs * FRAME_RATE)
        max_seq = self.max_seq - 10
        nq = cfg.n_codebooks if cfg.n_codebooks > 0 else self.Q
        identity = row.idx == 0
        slot_idx = None if identity else row._slot
        codes_io = self._g_codes_in if identity else self._gc_codes_in
        nat = self.model._native
        stream = torch.cuda.current_stream()
        if reset_rep:
            self._rep_reset(cfg.rep_penalty, cfg.rep_window)
            self._frame_ctr.zero_()  # draws are keyed by (seed, frame of the turn, row, codebook)
        total_frames = 0
        use_rep = cfg.rep_penalty > 1.0

        def cancelled() -> bool:
            return cancel is not None and cancel.is_set()

        def entropy_top1(probs: Tensor) -> tuple[float, float]:
            ent = -(probs * probs.clamp_min(1e-9).log()).sum(-1).mean().item()
            return ent, probs.max(-1).values.mean().item()

        last_idx = len(chunks) - 1
        offset = row.offset
        for ci, chunk in enumerate(chunks):
            if total_frames >= max_frames or offset >= max_seq or cancelled():
                return
            # (speaker alternation on chunk.sc is the caller's: it picks the [spk] token inside chunk.emb)
            use_gate = cfg.gate_frames > 0 and ci == 0 and reset_rep
            chunk_start = offset
            gate_target = cfg.gate_frames
            max_per_turn = cfg.max_turn_frames(chunk.n_words, row.prompt_wps)
            retry_idx = 0
            while True:  # retry loop: a single pass unless the gate asks for a colder one
                cur_temp = cfg.temperature
                if retry_idx > 0:
                    cur_temp = GATE_RETRY_TEMPS[min(retry_idx - 1, len(GATE_RETRY_TEMPS) - 1)]
                    self.seq_lens[row.idx] = chunk_start
                    self._rep_reset(cfg.rep_penalty, cfg.rep_window)
                cfg_t = replace(cfg, temperature=cur_temp)
                hidden = self._prefill_emb(row, chunk.emb)[:, -1]  # (1, d)
                offset = chunk_start + chunk.emb.shape[1]
                cb0 = self.model.codec_head(hidden)
                held: list[Tensor] = []
                entropies: list[float] = []
                top1s: list[float] = []
                if use_gate:
                    e, p1 = entropy_top1(self._penalised_probs(cb0, self._rep_counts[row.idx:row.idx + 1], cfg, cur_temp))
                    entropies.append(e)
                    top1s.append(p1)
                # frame 0 of the chunk: no top-k cut unless greedy
                code0 = self._sample_cb0(cb0, cfg_t, top_k=1 if cfg.top_k == 1 else 0)
                sp1 = make_sample_params(cur_temp, cfg.rq_top_k if cfg.top_k != 1 else 1, cfg.seed, self._frame_ctr)
                _lib.check(nat.lib.vui_rq_generate(nat.handle, hidden.contiguous().data_ptr(), code0.data_ptr(), None, nq,
                                                   C.byref(sp1), codes_io.data_ptr(), self.Q, 1, 1, stream.cuda_stream),
                           "vui_rq_generate")
                self._frame_ctr += 1
                frame = codes_io[0, :nq].clone()
                if self._split is not None:
                    stream.synchronize()  # the vocoder reads this frame on another stream
                if use_gate:
                    held.append(frame)
                else:
                    yield frame
                    total_frames += 1
                # Frames 1.. of the chunk: one graph replay each (backbone step on the previous frame, code-0 draw
                # + push, depth head, and the end-of-turn test of src/vui/engine.py:1468-1471 on the device).  The
                # one-launch form does nothing once the test has fired, so the next step is enqueued before this
                # step's flag is read (one frame late: the GPU never waits for the host between frames); the
                # kernel-sequence form, and the gate while it gathers (it reads every step's logits), go one
                # step at a time.
                g, _, _, _ = self._frame_graph(1, cfg_t, slot_idx, 0, stop=(cfg.eos_threshold, min_frames))
                self._stop_state.copy_(self._stop_init)
                ahead = nat.fused(-1)
                retry_triggered = False
                pending = None  # (frame, event, pinned flag, gathering) of the step whose flag is still unread
                step = 1
                while True:
                    launched = None
                    reason = None
                    if pending is None or (ahead and not use_gate):
                        # the reference's tests at the top of an iteration, in its order (engine.py:1441-1449); a
                        # step in flight counts as kept (if it turns out to be the last, the loop ends anyway)
                        counted = total_frames + (1 if pending is not None else 0)
                        if step >= max_per_turn:
                            reason = "cap"
                        elif counted >= max_frames or offset >= max_seq:
                            reason = "limit"
                        elif cancelled():
                            return  # a step already in flight is dropped: no frame is yielded after a cancel
                        else:
                            gathering = use_gate and len(held) < gate_target
                            counts_before = self._rep_counts[row.idx:row.idx + 1].clone() if (gathering and use_rep) else None
                            g.replay()
                            offset += 1
                            if gathering:
                                cnt = counts_before if counts_before is not None else self._rep_counts[row.idx:row.idx + 1]
                                e, p1 = entropy_top1(self._penalised_probs(self._g_cb0_out[0:1], cnt, cfg, cur_temp))
                                entropies.append(e)
                                top1s.append(p1)
                            flag_t = self._stop_host[step & 1]
                            flag_t.copy_(self._stop_state[:1], non_blocking=True)
                            frame_t = codes_io[0, :nq].clone()  # before the event: a frame handed out is complete
                            ev = torch.cuda.Event()
                            ev.record(stream)
                            launched = (frame_t, ev, flag_t, gathering)
                            step += 1
                    if pending is not None:
                        frame, ev, flag_t, was_gathering = pending
                        pending = None
                        ev.synchronize()
                        flag = int(flag_t[0])
                        if flag == 2:  # the step's persistent launch failed and committed nothing
                            nat.status()
                            raise RuntimeError("frame step failed without a raised error word")
                        if flag == 1:  # end of turn: this frame is dropped; a step enqueued behind it did nothing
                            if launched is not None:
                                offset -= 1
                            for hc in held:
                                yield hc
                                total_frames += 1
                            held = []
                            break
                        if was_gathering:
                            held.append(frame)
                            if len(held) == gate_target:
                                avg_e = sum(entropies) / len(entropies)
                                if avg_e > cfg.gate_entropy_max and retry_idx < cfg.gate_retries:
                                    retry_triggered = True
                                    break
                                for hc in held:
                                    yield hc
                                    total_frames += 1
                                held = []
                                use_gate = False
                        else:
                            yield frame
                            total_frames += 1
                    pending = launched
                    if pending is None and reason is not None:
                        if reason == "cap":  # the chunk's step cap: on to the next chunk
                            break
                        for hc in held:  # max_secs or the cache limit: the turn is over
                            yield hc
                            total_frames += 1
                        return
                if retry_triggered:
                    retry_idx += 1
                    continue
                for hc in held:  # chunk shorter than the gate: flushed without a decision
                    yield hc
                    total_frames += 1
                break
