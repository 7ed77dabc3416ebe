"""Engine-level behaviour on the GPU: the one-graph frame loop against the oracle and against the
step-by-step composition, batched/bucketed steps with slot indirection, int8 weights at batch 16."""
import numpy as np
import pytest
import torch

from oracle import vui_oracle as O
from tests.util import TINY_SD, make_model, rel_err, tiny_dims

pytestmark = pytest.mark.gpu
BF, F32 = torch.bfloat16, torch.float32


def _engine(d, sd, dt, max_rows=1, S=None, int8=False):
    from vui_amd.engine import Engine

    m = make_model(d, sd, dt, int8=int8, max_seqlen=S or d.max_seqlen)
    return m, Engine(model=m, max_rows=max_rows, max_seq=S or d.max_seqlen)


@pytest.mark.parametrize("dt,fused", [(F32, 0), (BF, 0), (BF, 1)])
def test_frame_loop_greedy_matches_oracle_tiny(dt, fused):
    """Prefill + 10 greedy frames at reduced dims: token-exact against the oracle in fp32; in bf16 the
    frames agree until the first near-tie, and the two GPU forms agree with each other exactly."""
    from vui_amd.engine import GenConfig

    d = tiny_dims(2)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    m, eng = _engine(d, sd, dt)
    assert m._native.fused(fused) == bool(fused and dt == BF)
    ids = torch.tensor([3, 11, 42, 7, 19])
    row = eng.new_row()
    h = row.prefill_emb(m.token_emb(ids.cuda()[None]))[:, -1]
    frames, eos = eng.generate([row], h, 10, GenConfig(temperature=1.0, top_k=1, rep_penalty=1.0))
    m._native.status()
    o = O.OracleModel(d, sd, dt)
    ho = o.prefill(o.embed_text(ids))[-1:]
    col = {}
    ref = o.generate_frames(ho, 10, top_k=1, temperature=1.0, collect=col)[:, 0]
    if dt == F32:
        np.testing.assert_array_equal(frames[:, 0].cpu().numpy(), ref.numpy())
        eos_ref = torch.sigmoid(torch.stack(col["eos"])[1:, 0, 0])
        np.testing.assert_allclose(eos[1:, 0].cpu().numpy(), eos_ref.numpy(), rtol=1e-4, atol=1e-5)
    else:
        same = (frames[:, 0].cpu() == ref).all(dim=1)
        assert bool(same[0]) and int(same.sum()) >= 5, same
    assert int(eng.seq_lens[0]) == 5 + 9


def test_frame_graph_equals_stepwise_composition():
    """The fused frame graph reproduces decode_step + code-0 sampling + depth head called one by one
    (same seeds): sampled tokens, rolling repetition counts and positions, over 12 frames."""
    from vui_amd.engine import GenConfig

    d = tiny_dims(2)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    cfg = GenConfig(temperature=0.9, top_k=10, rq_top_k=10, rep_penalty=1.3, rep_window=4, seed=11)
    ids = torch.tensor([1, 2, 3])
    out = {}
    for fused in (0, 1):
        m, eng = _engine(d, sd, BF)
        m._native.fused(fused)
        row = eng.new_row()
        h = row.prefill_emb(m.token_emb(ids.cuda()[None]))[:, -1]
        frames, eos = eng.generate([row], h, 12, cfg)
        m._native.status()
        out[fused] = (frames.cpu(), eos.cpu(), eng._rep_counts.cpu().clone(), eng._rep_pos.cpu().clone())
    assert torch.equal(out[0][0], out[1][0])
    np.testing.assert_allclose(out[0][1].numpy(), out[1][1].numpy(), rtol=0, atol=0)
    assert torch.equal(out[0][2], out[1][2]) and torch.equal(out[0][3], out[1][3])
    # ring-buffer invariant: counts == histogram of the last `window` code-0 values (engine.py:930-934)
    frames, _, counts, pos = out[1]
    last = frames[-4:, 0, 0]
    hist = torch.bincount(last, minlength=d.codebook_size).float()
    assert torch.equal(counts[0], hist)
    assert pos[0].tolist() == [12 % 4, 4]


def test_sampled_frames_follow_oracle_distribution_tiny():
    """Sampling (T=0.9, top-k 8): code 0 of frame 1 over 2000 seeds against the oracle's analytic kept
    distribution (chi-square); every drawn code lies in the kept set."""
    from vui_amd.engine import GenConfig

    d = tiny_dims(2)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    m, eng = _engine(d, sd, F32)
    ids = torch.tensor([5, 6, 7])
    row = eng.new_row()
    h = row.prefill_emb(m.token_emb(ids.cuda()[None]))[:, -1]
    row.mark_prompt()
    o = O.OracleModel(d, sd, F32)
    ho = o.prefill(o.embed_text(ids))[-1:]
    cb0, _ = o.heads(ho)
    w = O.cb0_probs(cb0[0], 0.9, 0)  # frame 0 draws code 0 without top-k (engine.py:1416-1424)
    hist = np.zeros(d.codebook_size)
    for seed in range(2000):
        row.rewind()
        frames, _ = eng.generate([row], h, 1, GenConfig(temperature=0.9, top_k=8, rep_penalty=1.0, seed=seed))
        hist[int(frames[0, 0, 0])] += 1
    exp = w / w.sum() * hist.sum()
    keep = exp > 5
    chi2 = (((hist - exp) ** 2)[keep] / exp[keep]).sum()
    dof = int(keep.sum()) - 1
    assert chi2 < dof + 5 * (2 * dof) ** 0.5, (chi2, dof)


def test_batched_and_bucketed_steps():
    """_decode_step over all rows and _bucketed_decode_step with slot indirection and a padding slot
    (engine.py:434-534) give each row the same result as stepping it alone."""
    d = tiny_dims(2)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    m, eng = _engine(d, sd, BF, max_rows=4)
    g = torch.Generator().manual_seed(2)
    rows = [eng.new_row() for _ in range(4)]
    for i, r in enumerate(rows):  # ragged prompts
        ids = torch.randint(0, d.vocab_size, (2 + i,), generator=g).cuda()
        r.prefill_emb(m.token_emb(ids[None]))
    base = eng.seq_lens.clone()
    assert base.tolist()[:4] == [2, 3, 4, 5]
    codes = torch.randint(0, d.codebook_size, (4, d.n_quantizers), generator=g).cuda()
    # all rows at once (short frame: zero padded, engine.py:473-479)
    for i in range(4):
        eng._set_codes_in(i, codes[i, :3])
    hid, cb0, eos = eng._decode_step()
    ref_h, ref_c = hid.clone(), cb0.clone()
    assert eng.seq_lens.tolist() == [3, 4, 5, 6, 0]
    # rows 3 and 1 only, through the bucket of 2 with slot indirection
    eng.seq_lens.copy_(base)
    eng._gc_codes_in.zero_()
    eng._gc_codes_in[0, :3] = codes[3, :3]
    eng._gc_codes_in[1, :3] = codes[1, :3]
    eng._g_slot_idx[:2] = torch.tensor([3, 1], dtype=torch.int32)
    eng._g_seq_inc.zero_()
    eng._g_seq_inc[3] = 1
    eng._g_seq_inc[1] = 1
    h2, c2, e2 = eng._bucketed_decode_step(2)
    assert torch.equal(h2[0], ref_h[3]) and torch.equal(h2[1], ref_h[1])
    assert torch.equal(c2[0], ref_c[3]) and torch.equal(c2[1], ref_c[1])
    assert eng.seq_lens.tolist() == [2, 4, 4, 6, 0]
    # three active rows in the bucket of 4: the padding row writes to the padding slot only
    eng.seq_lens.copy_(base)
    eng._gc_codes_in.zero_()
    for j, r in enumerate((0, 2, 3)):
        eng._gc_codes_in[j, :3] = codes[r, :3]
    eng._g_slot_idx[:3] = torch.tensor([0, 2, 3], dtype=torch.int32)
    eng._g_seq_inc.zero_()
    eng._g_seq_inc[[0, 2, 3]] = 1
    h3, c3, _ = eng._bucketed_decode_step(3)
    for j, r in enumerate((0, 2, 3)):
        assert torch.equal(h3[j], ref_h[r]) and torch.equal(c3[j], ref_c[r])
    assert eng.seq_lens.tolist() == [3, 3, 5, 6, 0]
    with pytest.raises(RuntimeError, match="No free rows"):
        eng.new_row()


def test_int8_batch16_ragged_vs_oracle():
    """Benchmark configuration 5 at full dims: 16 streams, ragged cache lengths in [128, 2048], backbone linears
    as weight-only int8 (per-row scales): logits against the oracle evaluating the same int8 weights
    (dequantise-then-matmul), tolerance 2^-5 * max|logit|."""
    S = 2112
    d = O.Dims()
    sd = O.synthetic_state_dict(d, seed=0)
    m = make_model(d, sd, BF, int8=True, max_seqlen=S)
    B = 16
    m.decoder.allocate_flash_kv_cache(B, m.device, BF, max_seqlen=S)
    g = torch.Generator().manual_seed(0)
    lens = torch.randint(128, 2049, (B,), generator=g)
    check = [0, 7, 15]  # rows verified against the CPU oracle (each costs a full CPU step)
    kc = O.rnd(0.5 * torch.randn(d.n_layers, B, S, d.n_kv_heads, d.head_dim, generator=g), BF)
    vc = O.rnd(0.5 * torch.randn(d.n_layers, B, S, d.n_kv_heads, d.head_dim, generator=g), BF)
    m.decoder._k.copy_(kc.to(BF))
    m.decoder._v.copy_(vc.to(BF))
    m.decoder.flash_kv_caches[0].seq_lens.copy_(lens.to(torch.int32))
    codes = torch.randint(0, d.codebook_size, (B, d.n_quantizers), generator=g)
    hid = torch.empty(B, d.d_model, dtype=BF, device="cuda")
    cb0 = torch.empty(B, d.codebook_size, dtype=BF, device="cuda")
    m.decoder._step(codes=codes.cuda(), emb=None, slot_idx=None, seq_inc=None, B=B, hidden_out=hid, cb0_out=cb0,
                    eos_out=None, n_splits=4, stream=torch.cuda.current_stream().cuda_stream)
    assert m.decoder.flash_kv_caches[0].seq_lens.cpu().tolist() == (lens + 1).tolist()
    o = O.OracleModel(d, sd, BF, n_slots=1, max_seqlen=S, int8=True)
    for b in check:
        o.k_cache[:, 0] = kc[:, b]
        o.v_cache[:, 0] = vc[:, b]
        o.seq_lens[0] = int(lens[b])
        h_ref, cb_ref, _ = o.decode_step(codes[b:b + 1])
        assert rel_err(cb0[b:b + 1], cb_ref) <= 2.0 ** -5, (b, rel_err(cb0[b:b + 1], cb_ref))
        assert rel_err(hid[b:b + 1], h_ref) <= 2.0 ** -5


@pytest.mark.parametrize("dims", ["tiny", "nano"])
def test_batch12_mfma_rows_match_small_batches(dims):
    """Rows 9..16 of a batch go through the matrix-core GEMM: a 12-row decode step gives every row
    what the same row gets in a 4-row step (row-per-wave GEMV), to bf16 rounding."""
    if dims == "tiny":
        d, S = tiny_dims(2), 32
        sd = O.synthetic_state_dict(d, **TINY_SD)
    else:
        d, S = O.Dims(), 64
        sd = O.synthetic_state_dict(d, seed=0)
    m = make_model(d, sd, BF, max_seqlen=S)
    B = 12
    m.decoder.allocate_flash_kv_cache(B, m.device, BF, max_seqlen=S)
    g = torch.Generator().manual_seed(5)
    m.decoder._k.copy_((0.5 * torch.randn(m.decoder._k.shape, generator=g)).to(BF))
    m.decoder._v.copy_((0.5 * torch.randn(m.decoder._v.shape, generator=g)).to(BF))
    lens = torch.randint(0, S - 2, (B,), generator=g).to(torch.int32)
    codes = torch.randint(0, d.codebook_size, (B, d.n_quantizers), generator=g).cuda()
    seq = m.decoder.flash_kv_caches[0].seq_lens
    st = torch.cuda.current_stream().cuda_stream

    def run(rows):
        n = len(rows)
        idx = torch.tensor(rows, dtype=torch.int32, device="cuda")
        hid = torch.empty(n, d.d_model, dtype=BF, device="cuda")
        cb0 = torch.empty(n, d.codebook_size, dtype=BF, device="cuda")
        eos = torch.empty(n, 1, dtype=BF, device="cuda")
        m.decoder._step(codes=codes[rows].contiguous(), emb=None, slot_idx=idx, seq_inc=None, B=n, hidden_out=hid,
                        cb0_out=cb0, eos_out=eos, n_splits=2, stream=st)
        return hid.float().cpu(), cb0.float().cpu(), eos.float().cpu()

    seq.copy_(lens)
    h12, c12, e12 = run(list(range(B)))
    assert seq.cpu().tolist() == (lens + 1).tolist()
    for r0 in range(0, B, 4):
        seq.copy_(lens)
        h4, c4, e4 = run(list(range(r0, r0 + 4)))
        assert rel_err(c12[r0:r0 + 4], c4) <= 2.0 ** -5 and rel_err(h12[r0:r0 + 4], h4) <= 2.0 ** -5
        assert rel_err(e12[r0:r0 + 4], e4) <= 2.0 ** -4
    # the depth head at 12 rows against 4-row calls (greedy, so directly comparable up to near-ties)
    hidden = (torch.randn(B, d.d_model, generator=g)).to(BF).cuda()
    code0 = torch.randint(0, d.codebook_size, (B,), generator=g).cuda()
    full = m.rq_transformer.generate(hidden, code0, temperature=1.0, top_k=1).cpu()
    part = torch.cat([m.rq_transformer.generate(hidden[r:r + 4], code0[r:r + 4], temperature=1.0, top_k=1).cpu()
                      for r in range(0, B, 4)])
    agree = (full == part).all(dim=1).float().mean()
    assert agree >= 0.75, agree


def test_full_size_streaming_workload_properties():
    """The headline workload at its real size (Vui Nano dims, bf16, a 512-frame voice prefix + 64 text tokens
    ingested, then 750 sampled frames through the one-graph frame step), checked through what does not depend on
    size: a second run from the same seed gives the same 750 x 16 tokens and EOS probabilities, another seed
    does not; every code is inside its codebook; the cache grew by one position per frame; the rolling
    repetition counts equal the histogram of the last `window` code-0 values (engine.py:930-934); and the frames
    the graph logged are the frames it fed back."""
    from vui_amd.engine import Engine, GenConfig
    from vui_amd.model import Vui
    from vui_amd.synthetic import nano_for_cache, synthetic_state_dict

    n_prefix, n_text, n_frames = 512, 64, 750
    max_seq = 64 * ((n_prefix + n_text + n_frames + 2 + 63) // 64)
    d = nano_for_cache("A", 64).model
    sd = synthetic_state_dict(d, seed=0)
    model = Vui(nano_for_cache("A", max_seq), sd, device="cuda", dtype=BF)
    eng = Engine(model=model, max_rows=1, max_seq=max_seq)
    assert model._native.fused(-1), "the one-launch frame kernel must be the path at these dims"
    g = torch.Generator().manual_seed(0)
    prefix = torch.randint(0, d.codebook_size, (n_prefix, d.n_quantizers), generator=g).cuda()
    ids = torch.randint(0, d.vocab_size, (n_text,), generator=g).cuda()
    row = eng.new_row()
    row.prefill_emb(model.embed_audio(prefix[None]).to(BF))
    h = row.prefill_emb(model.token_emb(ids[None]))[:, -1]
    row.mark_prompt()
    assert row.offset == n_prefix + n_text

    def run(seed):
        row.rewind()
        cfg = GenConfig(seed=seed)  # temperature 0.9, top-k 100, repetition penalty 1.1 over 24 frames
        frames, eos = eng.generate([row], h, n_frames, cfg)
        model._native.status()
        return frames.cpu(), eos.cpu(), eng._rep_counts.cpu().clone(), eng._rep_pos.cpu().clone(), cfg

    f0, e0, counts, pos, cfg = run(0)
    assert f0.shape == (n_frames, 1, d.n_quantizers)
    assert int(f0.min()) >= 0 and int(f0.max()) < d.codebook_size
    assert bool(((e0 >= 0) & (e0 <= 1)).all()) and float(e0[0, 0]) == 0.0
    assert row.offset == n_prefix + n_text + n_frames - 1  # the last frame is not fed back
    last = f0[-cfg.rep_window:, 0, 0]
    assert torch.equal(counts[0], torch.bincount(last, minlength=d.codebook_size).float())
    assert pos[0].tolist() == [n_frames % cfg.rep_window, cfg.rep_window]
    # the codes the graph fed back are the codes it logged
    assert torch.equal(eng._g_codes_in[0, :d.n_quantizers].cpu(), f0[-1, 0])
    # the sampler uses its whole support: code 0 is not stuck and no codebook column is constant
    assert all(len(torch.unique(f0[:, 0, q])) > 50 for q in range(d.n_quantizers))
    f1, e1, *_ = run(0)
    assert torch.equal(f0, f1) and torch.equal(e0, e1)
    f2, *_ = run(1)
    assert not torch.equal(f0, f2)


def test_wide_depth_head_runs_in_the_one_launch_kernel():
    """A depth head whose 16-position keys and values exceed LDS together (768 wide, 5 layers: 245 KB) keeps its values
    in LDS and its keys in a per-workgroup scratch area: the whole frame still is one launch.  Greedy depth-head
    codes equal the oracle's bf16 regime up to the first near-tie of every row (this model's logits are about 9
    wide in bf16 steps of 1/16, so near-ties are frequent; the kernel sequence is held to the same bar), and whole
    frames are reproducible and well-formed."""
    from vui_amd.engine import GenConfig

    d = O.Dims(d_model=128, n_layers=2, n_heads=4, n_kv_heads=4, n_quantizers=16, codebook_size=64, rq_d_model=768,
               rq_n_layers=5, rq_n_heads=8, vocab_size=50, max_seqlen=64)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    o = O.OracleModel(d, sd, BF)
    g = torch.Generator().manual_seed(6)
    N = 12
    hidden = O.rnd(torch.randn(N, d.d_model, generator=g), BF)
    code0 = torch.randint(0, d.codebook_size, (N,), generator=g)
    ref, logits = o.rq_generate(hidden, code0, 1.0, 1, return_logits=True)
    for fused in (1, 0):
        m, eng = _engine(d, sd, BF)
        assert m._native.fused(fused) is bool(fused)  # the whole frame fits the one-launch form
        got = torch.cat([m.rq_transformer.generate(hidden[b:b + 1].to(BF).cuda(), code0[b:b + 1].cuda(), temperature=1.0, top_k=1)
                         for b in range(N)]).cpu()
        m._native.status()
        n_equal = 0
        for b in range(N):
            for i in range(d.n_quantizers - 1):
                if got[b, i + 1] != ref[b, i + 1]:
                    top2 = torch.topk(logits[b, i], 2).values
                    assert float(top2[0] - top2[1]) <= 2 * 2.0 ** -5 * float(logits[b, i].abs().max()), (fused, b, i)
                    break  # later codebooks are conditioned on a different token
                n_equal += 1
        assert n_equal >= 0.6 * N * (d.n_quantizers - 1), (fused, n_equal)
    # whole frames through the one-launch form: same seed, same frames; codes inside their codebooks
    cfg = GenConfig(temperature=0.9, top_k=10, rq_top_k=10, rep_penalty=1.2, rep_window=4, seed=3)
    ids = torch.tensor([4, 9, 2, 7])
    runs = []
    for _ in range(2):
        m, eng = _engine(d, sd, BF)
        assert m._native.fused(-1)
        row = eng.new_row()
        h = row.prefill_emb(m.token_emb(ids.cuda()[None]))[:, -1]
        frames, eos = eng.generate([row], h, 8, cfg)
        m._native.status()
        assert row.offset == 4 + 7
        runs.append(frames.cpu())
    assert torch.equal(runs[0], runs[1])
    assert int(runs[0].min()) >= 0 and int(runs[0].max()) < d.codebook_size


def test_failed_persistent_launch_commits_nothing_and_recovers():
    """The failure protocol of the persistent kernels, without making any kernel wait: the host sets the context's
    launch count to 0xFFFFFFFF, so the next launch finds it wrapped, raises the error word and ends at once (every
    wait is skipped).  Nothing is committed by the frame kernel - position, frame counter, repetition state - the
    EOS slot reads -1, vui_ctx_status reports the failure until vui_ctx_init has run, and after that the same
    generation gives the frames of an undisturbed run."""
    from vui_amd import _lib
    from vui_amd.engine import GenConfig

    d = tiny_dims(2)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    cfg = GenConfig(temperature=0.9, top_k=10, rq_top_k=10, rep_penalty=1.2, rep_window=4, seed=5)
    ids = torch.tensor([3, 11, 42, 7, 19])
    m, eng = _engine(d, sd, BF)
    nat = m._native
    assert nat.fused(1)
    row = eng.new_row()
    h = row.prefill_emb(m.token_emb(ids.cuda()[None]))[:, -1]
    good, _ = eng.generate([row], h, 6, cfg)
    nat.status()
    # the same generation again on a context whose launch count is about to wrap
    row.reset()
    h = row.prefill_emb(m.token_emb(ids.cuda()[None]))[:, -1]
    _lib.check(nat.lib.vui_debug_set_epoch(nat.handle, 0xFFFFFFFF), "set_epoch")
    with pytest.raises(RuntimeError, match="wrapped"):
        eng.generate([row], h, 6, cfg)
    torch.cuda.synchronize()
    assert int(eng.seq_lens[0]) == 5          # no position was added by the five failed frame steps
    assert int(eng._frame_ctr[0]) == 1        # the host set it to 1 after frame 0; no failed step advanced it
    assert float(eng._rep_counts.sum()) == 1  # frame 0's stand-alone code-0 draw pushed one code, the failed steps none
    g, frames, eos, _ = eng._frame_graph(1, cfg, None, 6)
    assert float(eos[1, 0]) == -1.0           # a failed step marks its EOS slot
    assert torch.equal(frames[1:6, :, : good.shape[-1]], good[1:])  # and logs no frame: the log still holds the first run's
    with pytest.raises(RuntimeError):
        nat.status()                          # sticky until the context is initialised again
    nat.reinit()
    nat.status()
    row.reset()
    h = row.prefill_emb(m.token_emb(ids.cuda()[None]))[:, -1]
    again, _ = eng.generate([row], h, 6, cfg)
    assert torch.equal(again, good)


def test_one_frame_graph_serves_every_sampling_setting():
    """Temperature, top-k and seed are read by the captured frame step from device memory: requests that differ in
    them (and in length) replay ONE graph, and each gives exactly the frames of an engine that never saw the others."""
    from vui_amd.engine import GenConfig

    d = tiny_dims(2)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    ids = torch.tensor([3, 11, 42, 7, 19])
    cfgs = [GenConfig(temperature=0.9, top_k=10, rq_top_k=10, rep_penalty=1.2, rep_window=4, seed=s) for s in (1, 2, 3)]
    cfgs += [GenConfig(temperature=0.6, top_k=5, rq_top_k=7, rep_penalty=1.2, rep_window=4, seed=2),
             GenConfig(temperature=1.0, top_k=1, rep_penalty=1.2, rep_window=4, seed=9)]
    lengths = [8, 12, 8, 20, 6]

    def run(eng, m, cfg, n):
        row = eng.new_row()
        h = row.prefill_emb(m.token_emb(ids.cuda()[None]))[:, -1]
        frames, _ = eng.generate([row], h, n, cfg)
        row.close()
        return frames.cpu()

    m, eng = _engine(d, sd, BF)
    shared = [run(eng, m, c, n) for c, n in zip(cfgs, lengths)]
    assert len(eng._frame_graphs) == 1
    shared_again = run(eng, m, cfgs[0], lengths[0])
    assert torch.equal(shared_again, shared[0]) and len(eng._frame_graphs) == 1
    for c, n, got in zip(cfgs, lengths, shared):
        m2, eng2 = _engine(d, sd, BF)
        assert torch.equal(run(eng2, m2, c, n), got), (c, n)
    assert not torch.equal(shared[0][:8], shared[1][:8])  # another seed, other frames
    # the depth head's own captured graphs likewise: one per (rows, codebooks)
    rq = m.rq_transformer
    hid = torch.randn(1, d.d_model, device="cuda").to(BF)
    c0 = torch.zeros(1, dtype=torch.long, device="cuda")
    outs = []
    for t, s in ((0.7, 0), (0.9, 0), (0.7, 5)):
        rq.seed = s
        rq._ctr.zero_()
        outs.append(rq.generate_cuda_graph_kv(hid, c0, t).clone())
    assert len(rq._gkv_graphs) == 1
    rq.seed = 0
    rq._ctr.zero_()
    assert torch.equal(rq.generate_cuda_graph_kv(hid, c0, 0.7), outs[0])


def test_compute_unit_ranges_and_context_widths():
    """vui_cu_stream_create takes one contiguous range inside the GPU; vui_ctx_workgroups takes the widths the
    one-launch kernel was run against the oracle with, switches the batched kernels off below the full width and is
    undone by vui_ctx_init.  Frames on 192 workgroups of a bound stream are well-formed and repeatable."""
    import ctypes as C

    from vui_amd import _lib
    from vui_amd.engine import GenConfig

    lib = _lib.load()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    h = C.c_void_p()
    for first, n in ((-1, 8), (0, 0), (cus - 8, 16), (0, cus + 1)):
        assert lib.vui_cu_stream_create(first, n, C.byref(h)) != 0
        assert "compute units" in _lib.last_error()
    assert lib.vui_cu_stream_create(0, 1, None) != 0
    d = tiny_dims(2)
    sd = O.synthetic_state_dict(d, **TINY_SD)
    m, eng = _engine(d, sd, BF)
    nat = m._native
    assert nat.fused(-1)
    batched = (nat.rq_batch(), nat.bb_batch())
    for bad in (0, 144, 152, 200, 257):
        with pytest.raises(RuntimeError, match="workgroups"):
            nat.workgroups(bad)
    nat.workgroups(192)
    assert nat.fused(-1) and not nat.rq_batch() and not nat.bb_batch()
    _lib.check(lib.vui_cu_stream_create(0, 192, C.byref(h)), "vui_cu_stream_create")
    stream = torch.cuda.ExternalStream(h.value)
    cfg = GenConfig(temperature=0.9, top_k=10, rq_top_k=10, seed=2)
    ids = torch.tensor([4, 9, 2, 7])
    runs = []
    for _ in range(2):
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            row = eng.new_row()
            hid = row.prefill_emb(m.token_emb(ids.cuda()[None]))[:, -1]
            frames, _ = eng.generate([row], hid, 6, cfg)
            row.close()
        stream.synchronize()
        nat.status()
        runs.append(frames.cpu())
    assert torch.equal(runs[0], runs[1])
    assert int(runs[0].min()) >= 0 and int(runs[0].max()) < d.codebook_size
    nat.reinit()  # the full width again
    assert (nat.rq_batch(), nat.bb_batch()) == batched
    torch.cuda.synchronize()
    row = eng.new_row()
    hid = row.prefill_emb(m.token_emb(ids.cuda()[None]))[:, -1]
    eng._frame_graphs.clear()
    full, _ = eng.generate([row], hid, 6, cfg)
    nat.status()
    assert full.shape == runs[0].shape
