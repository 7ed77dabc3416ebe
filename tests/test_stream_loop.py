"""Control flow of the streaming turn loop (reference: Engine._stream_row, src/vui/engine.py:1308-1521).

CPU: the oracle's restatement against the rules the reference's loop implements (minimum length,
EOS cut, word-count cap, total cap, gate retries with rewind, cancel).  GPU: Engine.stream through
the native frame step against the oracle, token for token, in fp32 greedy mode."""
import pytest
import torch

from oracle import vui_oracle as O
from tests.util import TINY_SD, tiny_dims


def _model(eos_bias=None, seed_sd=None):
    d = tiny_dims(max_seqlen=320)
    sd = O.synthetic_state_dict(d, **(seed_sd or TINY_SD))
    if eos_bias is not None:
        sd["eos_head.bias"] = torch.tensor([float(eos_bias)])
        sd["eos_head.weight"] = sd["eos_head.weight"] * 0.0
    return d, sd


def _chunks(d, n, T=5, words=4, seed=3):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(T, d.d_model, generator=g) * 0.5, words) for _ in range(n)]


def test_max_turn_frames_formula():
    # engine.py:88-103: min(int((n_words / wps * 1.6 + 0.6) * 12.5), int(max_turn_secs * 12.5))
    assert O.max_turn_frames(0, 0.0) == 187
    assert O.max_turn_frames(5, 0.0) == int((5 / 3.0 * 1.6 + 0.6) * 12.5) == 40
    assert O.max_turn_frames(5, 2.0) == int((5 / 2.0 * 1.6 + 0.6) * 12.5) == 57
    assert O.max_turn_frames(1000, 3.0) == 187
    assert O.max_turn_frames(5, 2.0, max_turn_wps=4.0) == int((5 / 4.0 * 1.6 + 0.6) * 12.5)


def test_eos_cut_respects_minimum_length():
    # eos probability 1 at every step: each chunk ends at the first step >= min_frames (the frame of that
    # step is not emitted), so a chunk yields exactly min_frames frames
    d, sd = _model(eos_bias=20.0)
    m = O.OracleModel(d, sd)
    log = []
    out = O.stream_row(m, _chunks(d, 3), top_k=1, min_secs=0.5, log=log)
    assert len(out) == 3 * 6  # int(0.5 * 12.5) = 6
    assert [e for e in log if e[0] == "eos"] == [("eos", 0, 6), ("eos", 1, 6), ("eos", 2, 6)]
    assert all(e[3] > 0.999 for e in log if e[0] == "p")
    # cache: per chunk 5 text positions + 6 decode steps
    assert int(m.seq_lens[0]) == 3 * (5 + 6)


def test_word_count_cap_and_total_cap():
    d, sd = _model(eos_bias=-20.0)  # never EOS
    m = O.OracleModel(d, sd)
    out = O.stream_row(m, _chunks(d, 2, words=2), top_k=1)
    cap = O.max_turn_frames(2, 0.0)  # 20
    assert len(out) == 2 * cap
    m = O.OracleModel(d, sd)
    log = []
    out = O.stream_row(m, _chunks(d, 3, words=2), top_k=1, max_secs=2.0, log=log)  # 25 frames in total
    assert len(out) == 25 and ("cap", 1) in log



def test_cache_limit_stops_the_turn():
    d, sd = _model(eos_bias=-20.0)
    m = O.OracleModel(d, sd)
    out = O.stream_row(m, _chunks(d, 4, words=30), top_k=1, max_seq=60)
    assert int(m.seq_lens[0]) <= 60 - 10 + 1
    assert 0 < len(out) < 60


def test_cancel_stops_between_frames():
    d, sd = _model(eos_bias=-20.0)
    m = O.OracleModel(d, sd)
    out = O.stream_row(m, _chunks(d, 2), top_k=1, cancel_after=7)
    assert len(out) == 7


def test_gate_retries_rewind_and_release():
    d, sd = _model(eos_bias=-20.0)
    ch = _chunks(d, 2, words=3)
    base = O.OracleModel(d, sd)
    ref = O.stream_row(base, ch, top_k=1)
    m = O.OracleModel(d, sd)
    log = []
    out = O.stream_row(m, ch, top_k=1, gate_frames=4, gate_entropy_max=0.0, gate_retries=2, log=log)
    # threshold 0 always fails: two retries at 0.5 and 0.3, then the held frames are released
    assert [e for e in log if e[0] == "retry"] == [("retry", 0, 0.5), ("retry", 0, 0.3)]
    # greedy draws do not depend on the temperature and the cache was rewound to the chunk start:
    # same frames and same cache length as without the gate
    assert len(out) == len(ref) and all(torch.equal(a, b) for a, b in zip(out, ref))
    assert int(m.seq_lens[0]) == int(base.seq_lens[0])
    # a gate that passes holds nothing back either
    m2 = O.OracleModel(d, sd)
    log2 = []
    out2 = O.stream_row(m2, ch, top_k=1, gate_frames=4, gate_entropy_max=1e9, log=log2)
    assert not [e for e in log2 if e[0] != "p"] and all(torch.equal(a, b) for a, b in zip(out2, ref))
    # a chunk shorter than the gate flushes its frames without a decision
    m3 = O.OracleModel(d, sd)
    out3 = O.stream_row(m3, ch, top_k=1, gate_frames=1000, gate_entropy_max=0.0)
    assert all(torch.equal(a, b) for a, b in zip(out3, ref)) and len(out3) == len(ref)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["eos", "caps", "gate"])
def test_engine_stream_equals_oracle(mode):
    from tests.util import make_model
    from vui_amd.engine import Chunk, Engine, GenConfig

    d = tiny_dims(max_seqlen=320)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    kw = dict(top_k=1, rep_penalty=1.2, rep_window=4)
    if mode == "eos":
        # threshold in the middle of what this model's eos head produces, so that some chunks end by EOS
        probe_log = []
        O.stream_row(O.OracleModel(d, sd), _chunks(d, 3, words=2), log=probe_log, eos_threshold=2.0, **kw)
        ps = sorted(e[3] for e in probe_log if e[0] == "p")
        kw.update(eos_threshold=0.5 * (ps[int(0.85 * len(ps))] + ps[int(0.85 * len(ps)) + 1]), min_secs=0.2)
    elif mode == "caps":
        kw.update(eos_threshold=2.0, max_secs=1.9)
    else:
        kw.update(eos_threshold=2.0, gate_frames=3, gate_entropy_max=0.0, gate_retries=2)
    ch = _chunks(d, 3, words=2)
    om = O.OracleModel(d, sd)
    log = []
    ref = O.stream_row(om, ch, log=log, **kw)
    assert len(ref) > 10
    # no EOS probability so close to the threshold that fp32 summation order could flip the test
    assert min(abs(e[3] - kw["eos_threshold"]) for e in log if e[0] == "p") > 1e-5
    if mode == "eos":
        assert any(e[0] == "eos" for e in log)

    model = make_model(d, sd, torch.float32, max_seqlen=320)
    eng = Engine(model=model, max_rows=1, max_seq=320)
    row = eng.new_row()
    cfg = GenConfig(temperature=0.9, top_k=1, rep_penalty=kw["rep_penalty"], rep_window=kw["rep_window"],
                    eos_threshold=kw["eos_threshold"], min_secs=kw.get("min_secs", 0.5), max_secs=kw.get("max_secs", 30.0),
                    gate_frames=kw.get("gate_frames", 0), gate_entropy_max=kw.get("gate_entropy_max", 1.9),
                    gate_retries=kw.get("gate_retries", 2))
    chunks = [Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch]
    got = [f.cpu() for f in row.stream(chunks, cfg)]
    assert len(got) == len(ref), (len(got), len(ref), log)
    for i, (a, b) in enumerate(zip(got, ref)):
        assert torch.equal(a, b), (i, a, b)
    assert row.offset == int(om.seq_lens[0])


@pytest.mark.gpu
def test_engine_stream_sampled_and_cancel():
    """bf16 fused frame step, sampling on: caps hold, frames are valid codes, cancel stops the turn,
    stream() refuses engines with more than one row (src/vui/engine.py:238-241)."""
    import threading

    from tests.util import make_model
    from vui_amd.engine import Chunk, Engine, GenConfig

    d = tiny_dims(max_seqlen=320)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    model = make_model(d, sd, torch.bfloat16, max_seqlen=320)
    eng = Engine(model=model, max_rows=1, max_seq=320)
    row = eng.new_row()
    ch = [Chunk(emb=e[None].cuda(), n_words=w) for e, w in _chunks(d, 2, words=3)]
    cfg = GenConfig(eos_threshold=2.0, rep_window=4, top_k=5)
    frames = list(row.stream(ch, cfg))
    assert len(frames) == 2 * cfg.max_turn_frames(3)
    st = torch.stack(frames)
    assert st.shape[1] == d.n_quantizers and int(st.min()) >= 0 and int(st.max()) < d.codebook_size
    assert row.offset == 2 * (5 + cfg.max_turn_frames(3) - 1)
    # same seed, same turn -> same frames (counter-based draws restart with the turn)
    row.reset()
    again = list(row.stream(ch, cfg))
    assert all(torch.equal(a, b) for a, b in zip(frames, again))
    # cancel after 5 frames
    row.reset()
    ev = threading.Event()
    n = 0
    for _ in row.stream(ch, cfg, cancel=ev):
        n += 1
        if n == 5:
            ev.set()
    assert n == 5
    eng2 = Engine(model=model, max_rows=2, max_seq=320)
    with pytest.raises(RuntimeError):
        next(iter(eng2.new_row().stream(ch, cfg)))


@pytest.mark.gpu
@pytest.mark.parametrize("graph", [False, True, "split"])
def test_stream_audio_equals_vocoder_oracle_on_streamed_codes(graph):
    """Row.stream (= stream_audio) on an engine with a vocoder: every frame of Row.stream_codes passed through the
    row's vocoder context.  Same turn, same seed: the audio is the vocoder oracle's for the codes Row.stream_codes
    yields; an early stop by the consumer leaves the row and the vocoder context usable.  "split": the engine
    with the GPU divided between the decode step (160 compute units) and the vocoder (the rest), the vocoder of
    one frame running beside the decode step of the next."""
    import dataclasses

    from oracle import codec_oracle as CO
    from tests.util import make_model
    from vui_amd.codec import CodecConfig, QwenCodecDecoder
    from vui_amd.engine import Chunk, Engine, GenConfig

    d = tiny_dims(max_seqlen=320)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    cd = CO.CodecDims(n_codebooks=4, codebook_size=32, codebook_dim=16, vq_dim=32, latent_dim=64, d_model=32,
                      n_layers=2, n_heads=2, head_dim=16, mlp_dim=64, max_seq=130, up_ratios=(2, 2),
                      decoder_dim=128, rates=(3, 2))
    csd = CO.synthetic_codec_state_dict(cd, seed=4)
    dec = QwenCodecDecoder(csd, CodecConfig(**dataclasses.asdict(cd)), device="cuda")
    if graph is True:
        dec.setup_streaming_graph(1)
    model = make_model(d, sd, torch.bfloat16, max_seqlen=320)
    ch = [Chunk(emb=e[None].cuda().to(torch.bfloat16), n_words=w) for e, w in _chunks(d, 2, words=3)]
    cfg = GenConfig(eos_threshold=2.0, rep_window=4, top_k=5)
    eng = Engine(model=model, codec=dec, max_rows=1, max_seq=320, split_cus=160 if graph == "split" else None)
    row = eng.new_row()
    audio = [a.clone().cpu() for a in row.stream(ch, cfg)]  # with a vocoder Row.stream hands out audio, as the reference's
    row.reset()
    row._codec_ctx.reset()
    it = row.stream_audio(ch, cfg)  # the consumer walks away after three frames
    for _ in range(3):
        next(it)
    it.close()
    row.reset()
    row._codec_ctx.reset()
    again = [a.clone().cpu() for a in row.stream_audio(ch, cfg)]
    assert len(again) == len(audio) and all(torch.equal(a, b) for a, b in zip(again, audio))
    row.reset()
    row._codec_ctx.reset()
    codes = [f.cpu() for f in row.stream_codes(ch, cfg)]
    n = 2 * cfg.max_turn_frames(3)
    assert len(audio) == len(codes) == n
    ora = CO.CodecDecoderOracle(cd, csd)
    ora.open_stream()
    for i in range(n):  # fewer frames than the context's cold restart after 125
        ref = ora.forward(codes[i].view(1, -1, 1))
        assert audio[i].shape == (1, 1, cd.hop) and float((audio[i] - ref).abs().max()) < 2e-4, i
    ora.close_stream()
    row.close()
