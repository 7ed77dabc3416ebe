"""Continuous batching (reference: Engine.render_continuous, src/vui/engine.py:1112-1302).

CPU: the oracle's restatement against the rules of the reference's loop (queue order, lowest free slot,
refill at once, EOS / frame cap / total cap, empty requests, buckets) and the property that, with greedy
draws, what a request produces does not depend on how many rows are served together.  GPU:
Engine.render_continuous through the bucketed step graphs with slot indirection against the oracle, token
for token, in fp32 greedy mode."""
import pytest
import torch

from oracle import vui_oracle as O
from tests.util import TINY_SD, tiny_dims


def _model(eos_bias=None):
    d = tiny_dims(max_seqlen=320)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    if eos_bias is not None:
        sd["eos_head.bias"] = torch.tensor([float(eos_bias)])
        sd["eos_head.weight"] = sd["eos_head.weight"] * 0.0
    return d, sd


def _requests(d, spec, seed=7):
    """spec: list of (prompt positions, [words per chunk])."""
    g = torch.Generator().manual_seed(seed)
    out = []
    for n_prompt, words in spec:
        prompt = torch.randn(n_prompt, d.d_model, generator=g) * 0.5 if n_prompt else None
        chunks = [(torch.randn(4, d.d_model, generator=g) * 0.5, w) for w in words]
        out.append((prompt, chunks, 0.0))
    return out


SPEC = [(6, [2, 1]), (0, [1]), (9, [3]), (3, []), (5, [1, 1, 1]), (2, [2])]


def test_queue_slots_and_buckets():
    d, sd = _model(eos_bias=-20.0)  # never EOS: every chunk runs to its frame cap
    m = O.OracleModel(d, sd, n_slots=4)
    log = []
    out = O.render_continuous(m, _requests(d, SPEC), max_rows=3, top_k=1, log=log)
    caps = {w: O.max_turn_frames(w, 0.0) for w in (1, 2, 3)}
    assert [len(o) for o in out] == [caps[2] + caps[1], caps[1], caps[3], 0, 3 * caps[1], caps[2]]
    starts = [e for e in log if e[0] == "start"]
    # served in order into the lowest free slot; the empty request takes and returns a slot at once
    assert starts[:3] == [("start", 0, 0), ("start", 1, 1), ("start", 2, 2)]
    assert [e[1] for e in starts] == [0, 1, 2, 3, 4, 5]
    assert starts[3][2] == starts[4][2] == 1  # request 1 is the first to finish; 3 is empty, 4 takes its slot
    assert all(e[2] in (1, 2, 3) for e in log if e[0] == "step")
    steps = [e for e in log if e[0] == "step"]
    assert steps[0] == ("step", (0, 1, 2), 3) and steps[-1][2] == 1
    assert {e[2] for e in log if e[0] == "end"} == {"done"}
    # a chunk of n frames costs 4 text positions + n - 1 steps... plus the step whose frame is dropped
    assert int(m.seq_lens[0]) > 0


def test_eos_and_total_cap():
    d, sd = _model(eos_bias=20.0)  # EOS at every step: each chunk yields exactly min_frames frames
    m = O.OracleModel(d, sd, n_slots=3)
    out = O.render_continuous(m, _requests(d, SPEC), max_rows=2, top_k=1, min_secs=0.5)
    assert [len(o) for o in out] == [12, 6, 6, 0, 18, 6]
    d, sd = _model(eos_bias=-20.0)
    m = O.OracleModel(d, sd, n_slots=3)
    log = []
    out = O.render_continuous(m, _requests(d, [(0, [30, 30]), (0, [1])]), max_rows=2, top_k=1, max_secs=2.0, log=log)
    assert len(out[0]) == 25 and ("end", 0, "cap", 25) in log and len(out[1]) == O.max_turn_frames(1, 0.0)
    m = O.OracleModel(d, sd, n_slots=3)
    out = O.render_continuous(m, _requests(d, [(0, [30, 30, 30])]), max_rows=1, top_k=1, max_seq=90)
    assert 0 < len(out[0]) < 90 and int(m.seq_lens[0]) <= 90 - 10 + 1


def test_result_does_not_depend_on_the_batch():
    d, sd = _model()
    kw = dict(top_k=1, rep_penalty=1.2, eos_threshold=2.0)
    reqs = _requests(d, SPEC)
    ref = O.render_continuous(O.OracleModel(d, sd, n_slots=2), reqs, max_rows=1, **kw)
    for rows in (2, 3, 6):
        got = O.render_continuous(O.OracleModel(d, sd, n_slots=rows + 1), reqs, max_rows=rows, **kw)
        assert all(torch.equal(a, b) for a, b in zip(got, ref)), rows
    assert O._get_bucket(1, 6) == 1 and O._get_bucket(3, 6) == 4 and O._get_bucket(5, 6) == 6 and O._get_bucket(6, 6) == 6


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["caps", "eos"])
def test_engine_render_continuous_equals_oracle(mode):
    from tests.util import make_model
    from vui_amd.engine import Chunk, Engine, GenConfig, RenderRequest

    d = tiny_dims(max_seqlen=320)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    kw = dict(top_k=1, rep_penalty=1.2, eos_threshold=2.0)
    reqs = _requests(d, SPEC)
    if mode == "eos":
        # a threshold inside the range of this model's EOS head, away from every probability it produces
        probs = []
        base = O.OracleModel(d, sd, n_slots=4)
        orig = base.decode_step

        def spy(codes, slots=None):
            h, c, e = orig(codes, slots)
            probs.extend(torch.sigmoid(e.float()).flatten().tolist())
            return h, c, e

        base.decode_step = spy
        O.render_continuous(base, reqs, max_rows=3, **kw)
        ps = sorted(probs)
        i = int(0.8 * len(ps))
        kw.update(eos_threshold=0.5 * (ps[i] + ps[i + 1]), min_secs=0.2)
    om = O.OracleModel(d, sd, n_slots=4)
    log = []
    ref = O.render_continuous(om, reqs, max_rows=3, log=log, **kw)
    assert sum(len(r) for r in ref) > 50
    if mode == "eos":
        caps = [sum(O.max_turn_frames(w, 0.0) for w in words) for _, words in SPEC]
        assert any(len(r) < c for r, c in zip(ref, caps))  # some chunk did end by EOS

    model = make_model(d, sd, torch.float32, max_seqlen=320)
    eng = Engine(model=model, max_rows=3, max_seq=320)
    cfg = GenConfig(temperature=0.9, top_k=1, rep_penalty=1.2, eos_threshold=kw["eos_threshold"], min_secs=kw.get("min_secs", 0.5))
    requests = [RenderRequest(chunks=[Chunk(emb=e[None].cuda(), n_words=w) for e, w in ch],
                              prompt_emb=None if p is None else p[None].cuda()) for p, ch, _ in reqs]
    got = eng.render_continuous(requests, cfg)
    assert [len(g) for g in got] == [len(r) for r in ref]
    for i, (a, b) in enumerate(zip(got, ref)):
        assert torch.equal(a.cpu(), b), i
    assert len(eng._free) == 3  # every slot was returned
    # the engine is reusable: the same requests again give the same codes
    again = eng.render_continuous(requests, cfg)
    assert all(torch.equal(a, b) for a, b in zip(got, again))


@pytest.mark.gpu
def test_engine_render_continuous_sampled_bf16():
    """bf16, sampling on, 16 rows: valid codes, frame caps hold, slots are recycled."""
    from tests.util import make_model
    from vui_amd.engine import Chunk, Engine, GenConfig, RenderRequest

    d = tiny_dims(max_seqlen=320)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    model = make_model(d, sd, torch.bfloat16, max_seqlen=320)
    eng = Engine(model=model, max_rows=4, max_seq=320)
    reqs = _requests(d, [(3, [1, 2])] * 9)
    requests = [RenderRequest(chunks=[Chunk(emb=e[None].cuda().bfloat16(), n_words=w) for e, w in ch],
                              prompt_emb=p[None].cuda().bfloat16()) for p, ch, _ in reqs]
    cfg = GenConfig(eos_threshold=2.0, top_k=5)
    out = eng.render_continuous(requests, cfg)
    want = cfg.max_turn_frames(1) + cfg.max_turn_frames(2)
    assert [len(o) for o in out] == [want] * 9
    st = torch.cat(out)
    assert st.shape[1] == d.n_quantizers and int(st.min()) >= 0 and int(st.max()) < d.codebook_size
    assert len(eng._free) == 4


@pytest.mark.gpu
def test_ingestion_lanes_do_not_change_results():
    """Blocks of different rows are ingested on side streams at once (Engine.prefill_lanes); the frames must not
    depend on it: bf16, sampled, five requests with prompts through three rows, one lane against four, and a
    queue of requests without chunks must drain."""
    import torch

    from oracle import vui_oracle as O
    from tests.util import TINY_SD, make_model, tiny_dims
    from vui_amd.engine import Chunk, Engine, GenConfig, RenderRequest

    # dims the one-pass ingestion accepts (multiples of 64, head_dim 32)
    d = O.Dims(d_model=128, n_layers=3, n_heads=4, n_kv_heads=2, n_quantizers=4, codebook_size=32, rq_d_model=64,
               rq_n_layers=1, rq_n_heads=2, vocab_size=50, max_seqlen=256)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    g = torch.Generator().manual_seed(3)

    def emb(n):
        return (torch.randn(1, n, d.d_model, generator=g) * 0.3).to(torch.bfloat16).cuda()

    reqs = [RenderRequest(chunks=[Chunk(emb=emb(5 + i), n_words=2), Chunk(emb=emb(4), n_words=1)], prompt_emb=emb(9 + 2 * i))
            for i in range(5)]
    cfg = GenConfig(temperature=0.9, top_k=8, rq_top_k=8, eos_threshold=2.0, max_secs=2.0, seed=5)
    outs = {}
    for lanes in (1, 4):
        m = make_model(d, sd, torch.bfloat16, max_seqlen=d.max_seqlen)
        eng = Engine(model=m, max_rows=3, max_seq=d.max_seqlen)
        assert m.decoder._prefill_available()
        eng.prefill_lanes = lanes
        outs[lanes] = [o.cpu() for o in eng.render_continuous(reqs, cfg)]
        m._native.status()
        assert len(eng._free) == 3
        # requests that only carry a prompt: more of them than rows, every one admitted and released
        empty = eng.render_continuous([RenderRequest(chunks=[], prompt_emb=emb(6)) for _ in range(7)], cfg)
        assert all(o.shape[0] == 0 for o in empty) and len(eng._free) == 3
    assert all(o.shape[0] > 0 for o in outs[1])
    for a, b in zip(outs[1], outs[4]):
        assert torch.equal(a, b)
