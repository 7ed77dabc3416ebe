"""Randomly drawn scenarios of the four drivers (Row.stream, Engine._render_rows, inference.stream_frames,
Engine.render_continuous) against the oracle's restatements of the reference's loops, fp32 greedy: chunk counts and
lengths, word counts, frame caps, minimum lengths, repetition settings, reduced codebook counts, end-of-turn thresholds
inside the range the model produces, rows and slots, prompts."""
import random

import pytest
import torch

from oracle import vui_oracle as O
from tests.util import TINY_SD, make_model, tiny_dims

pytestmark = pytest.mark.gpu

S = 400


def _chunks(d, g, n, rnd):
    """n text chunks: (embeddings (T, d), word count)."""
    return [(torch.randn(rnd.randint(3, 7), d.d_model, generator=g) * 0.5, rnd.randint(1, 6)) for _ in range(n)]


def _threshold(ps, q, lo_gap=1e-4):
    """A threshold near quantile q of the observed end-of-turn probabilities, in the middle of a gap wide enough that
    fp32 summation order cannot flip a test; 2.0 (never) when there is none."""
    ps = sorted(ps)
    if len(ps) < 2:
        return 2.0
    i = min(len(ps) - 2, int(q * len(ps)))
    for j in list(range(i, len(ps) - 1)) + list(range(i - 1, -1, -1)):
        if ps[j + 1] - ps[j] > 2 * lo_gap:
            return 0.5 * (ps[j] + ps[j + 1])
    return 2.0


def _scenario(seed):
    from vui_amd.engine import Chunk, Engine, GenConfig
    from vui_amd.inference import InferenceState, stream_frames

    rnd = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    d = tiny_dims(max_seqlen=S)
    sdkw = dict(TINY_SD)
    sdkw["seed"] = 7 + seed
    sd = O.synthetic_state_dict(d, **sdkw)
    kw = dict(top_k=1, rep_penalty=rnd.choice([1.0, 1.2, 1.5]), rep_window=rnd.choice([2, 4, 24]),
              min_secs=rnd.choice([0.08, 0.2, 0.5]), max_secs=rnd.choice([1.0, 2.5, 30.0]),
              max_turn_wps=rnd.choice([0.0, 3.0]), n_codebooks=rnd.choice([0, 0, 2, 3]))
    what = rnd.choice(["stream", "render", "render", "frames", "cont"])
    fails = []
    if what == "stream":
        ch = _chunks(d, g, rnd.randint(1, 4), rnd)
        log = []
        O.stream_row(O.OracleModel(d, sd), ch, log=log, eos_threshold=2.0, **kw)
        thr = _threshold([e[3] for e in log if e[0] == "p"], rnd.choice([0.5, 0.8, 0.95]))
        om = O.OracleModel(d, sd)
        log = []
        ref = O.stream_row(om, ch, log=log, eos_threshold=thr, **kw)
        if min([abs(e[3] - thr) for e in log if e[0] == "p"] + [1.0]) < 2e-5:
            return "skip"  # a probability too close to the threshold to call
        model = make_model(d, sd, torch.float32, max_seqlen=S)
        eng = Engine(model=model, max_rows=1, max_seq=S)
        row = eng.new_row()
        cfg = GenConfig(temperature=0.9, eos_threshold=thr, **kw)
        got = [f.cpu() for f in row.stream([Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch], cfg)]
        if len(got) != len(ref) or any(not torch.equal(a, b) for a, b in zip(got, ref)):
            fails.append(("stream", len(got), len(ref)))
        if row.offset != int(om.seq_lens[0]):
            fails.append(("stream offset", row.offset, int(om.seq_lens[0])))
    elif what == "render":
        rows = rnd.randint(1, 3)
        chs = [_chunks(d, g, rnd.randint(0, 3), rnd) for _ in range(rows)]
        log = []
        om0 = O.OracleModel(d, sd, n_slots=rows)
        O.render_rows(om0, chs, eos_threshold=2.0, log=log, **kw)
        thr = 2.0
        if any(chs):
            log = []
            O.stream_row(O.OracleModel(d, sd), [c for c in chs if c][0], log=log, eos_threshold=2.0,
                         **{k: v for k, v in kw.items()})
            thr = _threshold([e[3] for e in log if e[0] == "p"], rnd.choice([0.5, 0.8, 0.95]))
        om = O.OracleModel(d, sd, n_slots=rows)
        ref = O.render_rows(om, chs, eos_threshold=thr, **kw)
        model = make_model(d, sd, torch.float32, max_seqlen=S)
        eng = Engine(model=model, max_rows=rows, max_seq=S)
        rws = [eng.new_row() for _ in range(rows)]
        cfg = GenConfig(temperature=0.9, eos_threshold=thr, **kw)
        got = eng._render_rows(rws, [[Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch] for ch in chs], cfg)
        if got.keys() != ref.keys():
            fails.append(("render keys", sorted(got.keys()), sorted(ref.keys())))
        else:
            for r in ref:
                if got[r].shape != ref[r].shape or not torch.equal(got[r].cpu(), ref[r]):
                    fails.append(("render row", r, tuple(got[r].shape), tuple(ref[r].shape)))
        for i, r in enumerate(rws):
            if r.offset != int(om.seq_lens[i]):
                fails.append(("render offset", i, r.offset, int(om.seq_lens[i])))
    elif what == "frames":
        ch = _chunks(d, g, rnd.randint(1, 3), rnd)
        fkw = dict(top_k=1, rep_penalty=kw["rep_penalty"], rep_window=kw["rep_window"], min_turn_secs=kw["min_secs"],
                   max_turn_secs=rnd.choice([0.5, 1.0, 2.0]), max_secs=kw["max_secs"])
        log = []
        O.stream_row(O.OracleModel(d, sd), ch, log=log, eos_threshold=2.0, top_k=1, rep_penalty=kw["rep_penalty"],
                     rep_window=kw["rep_window"])
        thr = _threshold([e[3] for e in log if e[0] == "p"], rnd.choice([0.5, 0.8, 0.95]))
        om = O.OracleModel(d, sd)
        ref = O.stream_frames(om, [e for e, _ in ch], eos_threshold=thr, **fkw)
        model = make_model(d, sd, torch.float32, max_seqlen=S)
        state = InferenceState(model, rq_top_k=1, compile_rq=rnd.choice([False, True]))
        cks = [Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch]
        got = [(f.cpu(), t) for f, t in stream_frames(state, cks, eos_threshold=thr, **fkw)]
        if len(got) != len(ref):
            fails.append(("frames len", len(got), len(ref)))
        else:
            for i, ((a, ta), (b, tb)) in enumerate(zip(got, ref)):
                if not torch.equal(a, b) or (ta is None) != (tb is None):
                    fails.append(("frames", i))
                    break
        if state.offset != int(om.seq_lens[0]):
            fails.append(("frames offset", state.offset, int(om.seq_lens[0])))
    else:
        from vui_amd.engine import RenderRequest

        rows = rnd.randint(1, 3)
        nreq = rnd.randint(1, 6)
        reqs = []
        for _ in range(nreq):
            pl = rnd.choice([0, 0, 4, 9])
            pe = torch.randn(pl, d.d_model, generator=g) * 0.5 if pl else None
            reqs.append((pe, _chunks(d, g, rnd.randint(0, 3), rnd), rnd.choice([0.0, 2.0])))
        ckw = {k: v for k, v in kw.items() if k != "rep_window"}
        thr = 2.0
        probe = [ch for _, ch, _ in reqs if ch]
        if probe:
            log = []
            O.stream_row(O.OracleModel(d, sd), probe[0], log=log, eos_threshold=2.0, **kw)
            thr = _threshold([e[3] for e in log if e[0] == "p"], rnd.choice([0.5, 0.8, 0.95]))
        om = O.OracleModel(d, sd, n_slots=rows + 1)
        ref = O.render_continuous(om, reqs, max_rows=rows, eos_threshold=thr, **ckw)
        model = make_model(d, sd, torch.float32, max_seqlen=S)
        eng = Engine(model=model, max_rows=rows, max_seq=S)
        cfg = GenConfig(temperature=0.9, eos_threshold=thr, **kw)
        rr = [RenderRequest(chunks=[Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch],
                            prompt_emb=(p[None].cuda() if p is not None else None), prompt_wps=wps) for p, ch, wps in reqs]
        got = eng.render_continuous(rr, cfg)
        if len(got) != len(ref):
            fails.append(("cont n", len(got), len(ref)))
        else:
            for i, (a, b) in enumerate(zip(got, ref)):
                if a.shape != b.shape or not torch.equal(a.cpu(), b):
                    fails.append(("cont req", i, tuple(a.shape), tuple(b.shape)))
    return (what, kw, fails) if fails else "ok " + what


@pytest.mark.parametrize("seed", range(1000, 1024))
def test_random_driver_scenario(seed):
    r = _scenario(seed)
    assert isinstance(r, str), r
