"""The offline render loop (reference: Engine._render_rows / render_all / Row.render, src/vui/engine.py:865-1110)
and the single-stream driver (reference: inference.stream_frames, src/vui/inference.py:507-734).

CPU: the oracle's restatements against the rules the reference's loops implement.  GPU: the Engine and
vui_amd.inference through the native step against the oracle, token for token, in fp32 greedy mode, and the
invariant the reference states for its two loops (render == stream, engine.py:1001-1008) on the bf16 path."""
import pytest
import torch

from oracle import vui_oracle as O
from tests.util import TINY_SD, tiny_dims


def _model(eos_bias=None):
    d = tiny_dims(max_seqlen=400)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    if eos_bias is not None:
        sd["eos_head.bias"] = torch.tensor([float(eos_bias)])
        sd["eos_head.weight"] = sd["eos_head.weight"] * 0.0
    return d, sd


def _chunks(d, n, T=5, words=2, seed=3):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(T, d.d_model, generator=g) * 0.5, words) for _ in range(n)]


def _mid_threshold(d, sd, ch, **kw):
    """An EOS threshold inside the range this model's eos head produces, and the distance of the closest
    probability from it."""
    log = []
    O.stream_row(O.OracleModel(d, sd), ch, log=log, eos_threshold=2.0, **kw)
    ps = sorted(e[3] for e in log if e[0] == "p")
    i = int(0.85 * len(ps))
    return 0.5 * (ps[i] + ps[i + 1])


# ------------------------------------------------------------------ CPU: render_rows
def test_render_of_one_row_equals_stream():
    # engine.py:1001-1008: render is kept equal to stream across chunk boundaries (same draws, same cache)
    d, sd = _model()
    ch = _chunks(d, 3)
    kw = dict(top_k=1, rep_penalty=1.2, rep_window=4, min_secs=0.2)
    thr = _mid_threshold(d, sd, ch, **kw)
    a, b = O.OracleModel(d, sd), O.OracleModel(d, sd)
    log = []
    ref = O.stream_row(a, ch, eos_threshold=thr, log=log, **kw)
    assert any(e[0] == "eos" for e in log)
    got = O.render_rows(b, [ch], eos_threshold=thr, **kw)[0]
    assert len(ref) == got.shape[0] and all(torch.equal(x, y) for x, y in zip(ref, got))
    assert int(a.seq_lens[0]) == int(b.seq_lens[0])
    # and sampled: one frame number per chunk start and per decode step in both loops
    kw = dict(top_k=5, rq_top_k=5, rep_penalty=1.2, rep_window=4, eos_threshold=2.0, seed=11)
    ref = O.stream_row(O.OracleModel(d, sd), ch, **kw)
    got = O.render_rows(O.OracleModel(d, sd), [ch], **kw)[0]
    assert len(ref) == got.shape[0] and all(torch.equal(x, y) for x, y in zip(ref, got))


def test_render_caps():
    d, sd = _model(eos_bias=-20.0)  # never EOS
    cap = O.max_turn_frames(2, 0.0)  # 20 frames per chunk of two words
    out = O.render_rows(O.OracleModel(d, sd), [_chunks(d, 2)], top_k=1)
    assert out[0].shape[0] == 2 * cap
    out = O.render_rows(O.OracleModel(d, sd), [_chunks(d, 3)], top_k=1, max_secs=2.0)
    assert out[0].shape[0] == 25  # int(2.0 * 12.5) frames in total
    m = O.OracleModel(d, sd)
    out = O.render_rows(m, [_chunks(d, 4, words=30)], top_k=1, max_seq=60)
    assert 0 < out[0].shape[0] < 60 and int(m.seq_lens[0]) <= 60 - 10 + 1


def test_render_retries_short_chunks_colder():
    # engine.py:952-983: a chunk that ends with fewer than two frames per word is rewound and redone at 0.5, then
    # 0.3, then accepted.  EOS always on: every attempt ends at min_frames = 6 frames for 10 words.
    d, sd = _model(eos_bias=20.0)
    ch = _chunks(d, 2, words=10)
    m = O.OracleModel(d, sd)
    log = []
    out = O.render_rows(m, [ch], top_k=1, rep_penalty=1.0, log=log)  # (a retry also clears the repetition state)
    assert [e for e in log if e[0] == "retry"] == [("retry", 0, 0, 0.5), ("retry", 0, 0, 0.3), ("retry", 0, 1, 0.5),
                                                   ("retry", 0, 1, 0.3)]
    # greedy draws ignore the temperature and every retry starts from the rewound cache: the frames and the cache
    # length are those of chunks whose word count asks for no retry
    base = O.OracleModel(d, sd)
    ref = O.render_rows(base, [[(e, 0) for e, _ in ch]], top_k=1, rep_penalty=1.0)
    assert torch.equal(out[0], ref[0]) and out[0].shape[0] == 12
    assert int(m.seq_lens[0]) == int(base.seq_lens[0]) == 2 * (5 + 6)


def test_render_rows_are_independent_under_greedy():
    d, sd = _model()
    chs = [_chunks(d, 2, seed=s) for s in (3, 4, 5)]
    chs[1] = chs[1][:1]  # rows of different lengths: one finishes early and idles
    kw = dict(top_k=1, rep_penalty=1.2, rep_window=4, eos_threshold=2.0)
    together = O.render_rows(O.OracleModel(d, sd, n_slots=3), chs, **kw)
    for r in range(3):
        alone = O.render_rows(O.OracleModel(d, sd), [chs[r]], **kw)[0]
        assert torch.equal(together[r], alone), r
    assert O.render_rows(O.OracleModel(d, sd, n_slots=2), [[], _chunks(d, 1)], **kw).keys() == {1}


# ------------------------------------------------------------------ CPU: stream_frames
def test_stream_frames_rules():
    d, sd = _model(eos_bias=20.0)
    ch = [e for e, _ in _chunks(d, 3)]
    m = O.OracleModel(d, sd)
    out = O.stream_frames(m, ch, top_k=1, min_turn_secs=0.5)
    # every turn: the first frame, then steps 1..5 each release one frame; step 6 >= min_frames ends the turn
    assert len(out) == 3 * 6
    assert [t for _, t in out] == ([None] * 5 + [0]) + ([None] * 5 + [1]) + ([None] * 5 + [2])
    assert int(m.seq_lens[0]) == 3 * (5 + 6)  # 5 text positions + 6 decode steps per turn
    # never EOS: a turn runs to max_turn_secs; the total cap ends the stream inside a turn
    d, sd = _model(eos_bias=-20.0)
    out = O.stream_frames(O.OracleModel(d, sd), ch, top_k=1, max_turn_secs=1.0)
    assert len(out) == 3 * 12
    out = O.stream_frames(O.OracleModel(d, sd), ch, top_k=1, max_turn_secs=1.0, max_secs=1.6)
    assert len(out) == 20 and out[-1][1] == 1


def test_stream_frames_draws_code0_with_ties_kept_on_every_frame():
    # sampling.sample_top_k keeps everything >= the k-th largest probability; Engine._stream_row draws a chunk's
    # first frame without any cut.  With top_k=1 both are greedy and the two drivers give the same frames as long
    # as no turn ends by EOS (the drivers differ in what they do with the last frame) and the caps agree.
    d, sd = _model(eos_bias=-20.0)
    ch = _chunks(d, 2, words=0)
    a = O.stream_row(O.OracleModel(d, sd), ch, top_k=1, rep_penalty=1.2, rep_window=4, max_turn_secs=1.0)
    b = O.stream_frames(O.OracleModel(d, sd), [e for e, _ in ch], top_k=1, rep_penalty=1.2, rep_window=4,
                        max_turn_secs=1.0)
    assert len(a) == len(b) == 24 and all(torch.equal(x, y[0]) for x, y in zip(a, b))


# ------------------------------------------------------------------ GPU
def _engine(d, sd, dt, rows, **kw):
    from tests.util import make_model
    from vui_amd.engine import Engine

    model = make_model(d, sd, dt, max_seqlen=400)
    return model, Engine(model=model, max_rows=rows, max_seq=400, **kw)


def _cfg(**kw):
    from vui_amd.engine import GenConfig

    return GenConfig(temperature=0.9, **kw)


@pytest.mark.gpu
@pytest.mark.parametrize("rows,empty", [(1, False), (3, False), (3, True)])
def test_engine_render_equals_oracle(rows, empty):
    """empty: the last row has no chunks at all (it yields no frames and the others are not disturbed)."""
    from vui_amd.engine import Chunk

    d, sd = _model()
    chs = [_chunks(d, 2 + (r == 0), seed=3 + r) for r in range(rows)]
    if empty:
        chs[-1] = []
    kw = dict(top_k=1, rep_penalty=1.2, rep_window=4, min_secs=0.2)
    thr = _mid_threshold(d, sd, chs[0], **kw)
    om = O.OracleModel(d, sd, n_slots=rows)
    log = []
    ref = O.render_rows(om, chs, eos_threshold=thr, log=log, **kw)
    assert any(e[0] == "eos" for e in log)
    model, eng = _engine(d, sd, torch.float32, rows)
    rws = [eng.new_row() for _ in range(rows)]
    cfg = _cfg(eos_threshold=thr, **kw)
    got = eng._render_rows(rws, [[Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch] for ch in chs], cfg)
    assert got.keys() == ref.keys()
    for r in ref:
        assert got[r].shape == ref[r].shape and torch.equal(got[r], ref[r]), r
    if empty:  # a row without frames has no entry (src/vui/engine.py:1082-1087); render_all gives it (0, Q)
        assert (rows - 1) not in ref
    # Row.render / render_all return what _render_rows found (no vocoder here: codes)
    for r in rws:
        r.reset()
    outs = eng.render_all(rws, [[Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch] for ch in chs], cfg)
    none = torch.zeros(0, d.n_quantizers, dtype=torch.long)
    assert all(torch.equal(o.cpu(), ref.get(i, none)) for i, o in enumerate(outs))


@pytest.mark.gpu
def test_engine_render_retry_rewinds():
    from vui_amd.engine import Chunk

    d, sd = _model(eos_bias=20.0)
    ch = _chunks(d, 2, words=10)
    om = O.OracleModel(d, sd)
    ref = O.render_rows(om, [ch], top_k=1, rep_penalty=1.3, rep_window=4)[0]
    model, eng = _engine(d, sd, torch.float32, 1)
    row = eng.new_row()
    codes, audio = row.render([Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch],
                              _cfg(top_k=1, rep_penalty=1.3, rep_window=4))
    assert audio is None and torch.equal(codes, ref)
    assert row.offset == int(om.seq_lens[0])


@pytest.mark.gpu
def test_render_equals_stream_on_the_one_launch_path():
    """bf16, sampling on, one row: Row.render goes through the same one-launch frame graph as Row.stream and the
    same frame numbers, so the two give the same frames (engine.py:1001-1008)."""
    from vui_amd.engine import Chunk

    d, sd = _model(eos_bias=-20.0)
    model, eng = _engine(d, sd, torch.bfloat16, 1)
    assert model._native.fused(-1)
    ch = [Chunk(emb=e[None].cuda().to(torch.bfloat16), n_words=w) for e, w in _chunks(d, 3)]
    cfg = _cfg(top_k=5, rq_top_k=5, rep_penalty=1.2, rep_window=4, seed=5)
    row = eng.new_row()
    streamed = torch.stack([f.cpu() for f in row.stream(ch, cfg)])
    off = row.offset
    row.reset()
    rendered, _ = row.render(ch, cfg)
    assert rendered.shape[0] == 3 * cfg.max_turn_frames(2) and torch.equal(rendered, streamed)
    assert row.offset == off
    model._native.status()


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [1, 0])
def test_device_end_of_turn_test(fused):
    """The end-of-turn test inside the frame step (vui_eos_stop): the step whose EOS probability passes the
    threshold at step >= min_frames sets the flag and still commits; on the one-launch form every step enqueued
    behind it does nothing at all (position, repetition state, frame number, codes stay), the kernel sequence only
    maintains the flag."""
    from vui_amd.engine import Chunk

    d, sd = _model(eos_bias=20.0)  # EOS probability 1 on every step
    model, eng = _engine(d, sd, torch.bfloat16, 1)
    assert model._native.fused(fused) == bool(fused)
    row = eng.new_row()
    ch = _chunks(d, 1)[0]
    h = row.prefill_emb(ch[0][None].cuda().to(torch.bfloat16))[:, -1]
    cfg = _cfg(top_k=5, rq_top_k=5, rep_penalty=1.2, rep_window=4)
    eng.generate([row], h, 1, cfg)  # frame 0 into the step's input buffer
    g, _, _, _ = eng._frame_graph(1, cfg, None, 0, stop=(0.5, 3))
    eng._stop_state.copy_(eng._stop_init)
    for step in (1, 2):  # below min_frames: runs, no flag
        g.replay()
        assert eng._stop_state.tolist() == [0, step + 1] and row.offset == 5 + step
    g.replay()  # step 3 >= min_frames: runs (position 8), sets the flag
    assert eng._stop_state.tolist() == [1, 4] and row.offset == 8
    snap = (eng._rep_counts.clone(), eng._frame_ctr.clone(), eng._g_codes_in.clone(), eng._rep_pos.clone())
    for _ in range(3):
        g.replay()
    now = (eng._rep_counts, eng._frame_ctr, eng._g_codes_in, eng._rep_pos)
    if fused:
        assert row.offset == 8 and eng._stop_state.tolist() == [1, 4]
        assert all(torch.equal(a, b) for a, b in zip(snap, now))
    else:
        assert row.offset == 11 and eng._stop_state.tolist() == [1, 7]
    eng._stop_state.copy_(eng._stop_init)  # a new chunk: steps run again
    g.replay()
    assert row.offset == (9 if fused else 12) and eng._stop_state.tolist() == [0, 2]
    model._native.status()
    model._native.fused(1)


@pytest.mark.gpu
def test_stream_reads_the_flag_one_frame_late_with_the_same_result():
    """Row.stream on the one-launch form enqueues the next step before it reads this step's flag; the frames, the
    row's position and its repetition state are those of the same turn streamed a second time, and every chunk
    stops where the EOS probabilities say (a model whose EOS head always fires: min_frames frames per chunk)."""
    from vui_amd.engine import Chunk

    d, sd = _model(eos_bias=20.0)
    model, eng = _engine(d, sd, torch.bfloat16, 1)
    assert model._native.fused(-1)
    chunks = [Chunk(emb=e[None].cuda().to(torch.bfloat16), n_words=w) for e, w in _chunks(d, 3)]
    cfg = _cfg(top_k=5, rq_top_k=5, rep_penalty=1.2, rep_window=4, min_secs=0.5, seed=2)
    row = eng.new_row()
    a = [f.cpu() for f in row.stream(chunks, cfg)]
    assert len(a) == 3 * 6 and row.offset == 3 * (5 + 6)  # the reference's count: 6 frames, 6 decode steps per chunk
    counts = eng._rep_counts.clone()
    row.reset()
    b = [f.cpu() for f in row.stream(chunks, cfg)]
    assert len(b) == len(a) and all(torch.equal(x, y) for x, y in zip(a, b))
    assert row.offset == 3 * (5 + 6) and torch.equal(counts, eng._rep_counts)
    model._native.status()


@pytest.mark.gpu
def test_prefill_segments_and_user_turn_layout():
    """Row.prefill / add_user write `[spk] text [SC] codes` in the reference's order (engine.py:725-826): the
    cache equals the one the same embeddings give when written in that order by hand."""
    from vui_amd.engine import Chunk, Segment

    d, sd = _model()
    g = torch.Generator().manual_seed(8)
    model, eng = _engine(d, sd, torch.float32, 2, sc_token_id=7)
    t1 = torch.randn(1, 4, d.d_model, generator=g) * 0.5
    t2 = torch.randn(1, 3, d.d_model, generator=g) * 0.5
    c1 = torch.randint(0, d.codebook_size, (6, d.n_quantizers), generator=g)
    c2 = torch.randint(0, d.codebook_size, (5, d.n_quantizers), generator=g)
    ut = torch.randn(1, 2, d.d_model, generator=g) * 0.5
    row = eng.new_row()
    n = row.prefill([Segment(text="one two three", codes=c1, text_emb=t1.cuda()),
                     Segment(text="four five", codes=c2, text_emb=t2.cuda())])
    assert n == 4 + 6 + 3 + 1 + 5 == row.offset  # [SC] only before the last segment's audio
    assert abs(row.prompt_wps - 5 / (11 / 12.5)) < 1e-9
    n2 = row.add_user(ut.cuda(), c1[:2], final=True)
    assert n2 == n + 2 + 1 + 2
    assert row.rewind() == n and row.offset == n
    # the same positions written by hand through the oracle
    om = O.OracleModel(d, sd)
    sc = om.embed_text(torch.tensor([7]))
    parts = [t1[0], om.embed_audio(c1), t2[0], sc, om.embed_audio(c2), ut[0], sc, om.embed_audio(c1[:2])]
    om.prefill(torch.cat(parts, 0), 0)
    k = model.decoder.flash_kv_caches[0].k_cache[0, :n2].float().cpu()
    assert torch.allclose(k, om.k_cache[0, 0, :n2], rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("compile_rq", [False, True])
def test_stream_frames_equals_oracle(compile_rq):
    """compile_rq: the depth head through generate_kv_compilable (the entry the reference compiles) instead of the
    captured graphs; same kernels, same frames."""
    from vui_amd.engine import Chunk
    from vui_amd.inference import InferenceState, render_codes_stream, stream_frames

    d, sd = _model()
    ch = _chunks(d, 3)
    kw = dict(top_k=1, rep_penalty=1.2, rep_window=4, min_turn_secs=0.2, max_turn_secs=2.0)
    # threshold inside the model's range (stream_row's probe sees the same probabilities: same greedy frames)
    thr = _mid_threshold(d, sd, ch, top_k=1, rep_penalty=1.2, rep_window=4, min_secs=0.2)
    om = O.OracleModel(d, sd)
    ref = O.stream_frames(om, [e for e, _ in ch], eos_threshold=thr, **kw)
    assert len(ref) > 10 and [t for _, t in ref if t is not None] == [0, 1, 2]
    from tests.util import make_model

    model = make_model(d, sd, torch.float32, max_seqlen=400)
    # the depth-head graphs bake their top-k in; 1 = greedy, as the oracle run
    state = InferenceState(model, rq_top_k=1, compile_rq=compile_rq, chunk_frames=7, ctx_frames=3, codec_graphs=True)
    chunks = [Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch]
    got = [(f.cpu(), t) for f, t in stream_frames(state, chunks, eos_threshold=thr, **kw)]
    assert len(got) == len(ref)
    for i, ((a, ta), (b, tb)) in enumerate(zip(got, ref)):
        assert torch.equal(a, b), i
        assert (ta is None) == (tb is None) and (ta is None or ta is chunks[tb])
    assert state.offset == int(om.seq_lens[0])
    assert chunks[0].frames == sum(1 for _, t in ref[: [t for _, t in ref].index(0) + 1])
    # checkpoint / rewind / resume: the second turn continues from the stored position
    state.checkpoint()
    turns = list(render_codes_stream(state, chunks[:1], resume=True, eos_threshold=thr, **kw))
    assert len(turns) == 1 and turns[0][0].shape[1] == d.n_quantizers
    assert state.rewind() == int(om.seq_lens[0])
    # the nucleus cut of _sample_codes (inference.py:491-504): a nucleus too small for a second entry holds the
    # largest probability alone, so the turn equals the greedy one frame for frame; a wide one runs, stays inside
    # the codebooks and repeats with the same seed
    kw_p = dict(kw, top_k=None, top_p=1e-6)
    tiny = [(f.cpu(), t) for f, t in stream_frames(state, chunks, eos_threshold=thr, **kw_p)]
    assert len(tiny) == len(got) and all(torch.equal(a, b) for (a, _), (b, _) in zip(tiny, got))
    kw_w = dict(kw, top_k=20, top_p=0.9, temperature=0.9, seed=3)
    wide = [f.cpu() for f, _ in stream_frames(state, chunks, eos_threshold=2.0, **kw_w)]
    again = [f.cpu() for f, _ in stream_frames(state, chunks, eos_threshold=2.0, **kw_w)]
    assert len(wide) == len(again) > 10 and all(torch.equal(a, b) for a, b in zip(wide, again))
    assert all(int(f.min()) >= 0 and int(f.max()) < d.codebook_size for f in wide)


@pytest.mark.gpu
def test_render_audio_stream_schedule_and_samples():
    """Audio emissions of inference.render_audio_stream: first after `first_chunk_frames`, then every `chunk_frames`,
    flushed at a turn's end; concatenated they are the vocoder oracle's streaming decode of the frames that
    stream_frames yields for the same arguments."""
    import dataclasses

    from oracle import codec_oracle as CO
    from tests.util import make_model
    from vui_amd.codec import CodecConfig, QwenCodecDecoder
    from vui_amd.engine import Chunk
    from vui_amd.inference import InferenceState, render_audio_stream, stream_frames

    d, sd = _model()
    ch = _chunks(d, 2)
    cd = CO.CodecDims(n_codebooks=d.n_quantizers, codebook_size=d.codebook_size, codebook_dim=16, vq_dim=32, latent_dim=64,
                      d_model=32, n_layers=2, n_heads=2, head_dim=16, mlp_dim=64, max_seq=130, up_ratios=(2, 2),
                      decoder_dim=128, rates=(3, 2))
    csd = CO.synthetic_codec_state_dict(cd, seed=4)
    dec = QwenCodecDecoder(csd, CodecConfig(**dataclasses.asdict(cd)), device="cuda")
    model = make_model(d, sd, torch.float32, max_seqlen=400)
    state = InferenceState(model, dec, rq_top_k=1)
    chunks = [Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch]
    kw = dict(top_k=1, eos_threshold=2.0, max_turn_secs=1.0)  # no end-of-turn inside the cap: 12 frames per turn
    frames = [(f.cpu(), t) for f, t in stream_frames(state, chunks, **kw)]
    per_turn = int(1.0 * 12.5)
    assert len(frames) == 2 * per_turn
    audio = [a.cpu() for a in render_audio_stream(state, chunks, chunk_frames=5, first_chunk_frames=2, **kw)]
    # turn 1: 2, 5, then the flush of 5; turn 2: 5, 5, flush of 2
    assert [a.shape[-1] // cd.hop for a in audio] == [2, 5, 5, 5, 5, 2]
    ora = CO.CodecDecoderOracle(cd, csd)
    ora.open_stream()
    ref = torch.cat([ora.forward(f.view(1, -1, 1)) for f, _ in frames], dim=-1)
    ora.close_stream()
    got = torch.cat(audio, dim=-1)
    assert got.shape == ref.shape and float((got - ref).abs().max()) < 2e-4
    with pytest.raises(RuntimeError):
        next(render_audio_stream(InferenceState(model, None, rq_top_k=1), chunks, **kw))
