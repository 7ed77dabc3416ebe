"""CPU pins of the oracle functions that no reference-written golden vector covers.

Each check is independent of the oracle's own formula: published known-answer vectors, per-element
Python loops written from the reference lines, brute force over tiny cases, or invariants.
"""
import itertools
import math

import numpy as np
import pytest
import torch

from oracle import vui_oracle as O

F32, BF = torch.float32, torch.bfloat16


# ---- Philox4x32-10: Random123's published known-answer vectors (kat_vectors, "philox4x32 10") ----
PHILOX_KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
     (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
]


@pytest.mark.parametrize("ctr,key,want", PHILOX_KAT)
def test_philox_known_answers(ctr, key, want):
    assert tuple(O.philox4x32_10(ctr, key)) == want


def test_uniform01_is_top_24_bits_of_word0():
    seen = set()
    for seed, frame, row, cb in itertools.product((0, 1, 2 ** 40 + 5), (0, 7, 749), (0, 15), (0, 1, 15)):
        u = O.uniform01(seed, frame, row, cb)
        w0 = O.philox4x32_10((frame, row, cb, 0), (seed & 0xFFFFFFFF, seed >> 32))[0]
        assert 0.0 <= u < 1.0
        assert u * 2 ** 24 == (w0 >> 8)  # exact: a 24-bit integer times 2^-24
        seen.add(u)
    assert len(seen) == 3 * 3 * 2 * 3  # every (seed, frame, row, codebook) has its own stream position
    # all-zero key and counter: word 0 of the first known-answer vector
    assert O.uniform01(0, 0, 0, 0) == (0x6627E8D5 >> 8) / 2 ** 24


def test_uniform01_is_roughly_uniform():
    u = np.array([O.uniform01(3, f, 0, 1) for f in range(4000)])
    hist, _ = np.histogram(u, bins=16, range=(0, 1))
    chi2 = ((hist - 250.0) ** 2 / 250.0).sum()
    assert chi2 < 45.0  # 15 degrees of freedom, p ~ 1e-4


# ---- repetition penalty (engine.py:571-576) against a per-element loop ----
def test_rep_penalise_elementwise():
    logits = torch.tensor([2.0, -2.0, 0.0, 0.5, -0.5, 3.0, -3.0, 1e-3])
    counts = torch.tensor([0.0, 0.0, 3.0, 1.0, 1.0, 2.0, 2.0, 5.0])
    pen = 1.3
    got = O.rep_penalise(logits, counts, pen)
    for i in range(len(logits)):
        f = np.float32(pen) ** np.float32(counts[i].item())
        l = np.float32(logits[i].item())
        want = l / f if l > 0 else l * f  # a zero logit takes the "multiply" branch and stays zero
        assert abs(got[i].item() - want) <= 1e-6 * max(1.0, abs(want)), i
    # count 0 leaves the logit alone, positive logits shrink, negative ones grow in magnitude
    assert got[0] == 2.0 and got[1] == -2.0 and got[2] == 0.0
    assert 0 < got[5] < logits[5] and got[6] < logits[6] < 0
    # penalty <= 1 switches it off whatever the counts (engine.py:573-574)
    assert torch.equal(O.rep_penalise(logits, counts, 1.0), logits)
    assert torch.equal(O.rep_penalise(logits.to(BF), counts, 0.9), logits.to(BF).float())


@pytest.mark.parametrize("window", [1, 4, 24])
def test_rep_state_counts_equal_window_histogram(window):
    CS = 13
    g = torch.Generator().manual_seed(window)
    codes = torch.randint(0, CS, (200,), generator=g).tolist()
    st = O.RepState(CS, window)
    for t, c in enumerate(codes):
        st.push(c)
        want = np.bincount(codes[max(0, t + 1 - window):t + 1], minlength=CS)
        np.testing.assert_array_equal(st.counts.numpy(), want)  # engine.py:930-934 states this invariant


def test_rep_state_without_window_counts_everything():
    st = O.RepState(5, 0)
    for c in [1, 1, 4, 1]:
        st.push(c)
    np.testing.assert_array_equal(st.counts.numpy(), [0, 3, 0, 0, 1])


# ---- selection rules on tiny vocabularies ----
def _kept(weights):
    return set(np.nonzero(weights > 0)[0].tolist())


def test_rq_rule_keeps_ties_at_kth():
    # model.py:955-961: logits < k-th largest are dropped, so everything equal to the k-th stays
    l = torch.tensor([1.0, 3.0, 2.0, 2.0, 0.5, 2.0])
    assert _kept(O.topk_threshold_probs(l, 1.0, 2)) == {1, 2, 3, 5}
    assert _kept(O.topk_threshold_probs(l, 1.0, 1)) == {1}
    assert _kept(O.topk_threshold_probs(l, 1.0, 4)) == {1, 2, 3, 5}
    assert _kept(O.topk_threshold_probs(l, 1.0, 5)) == {0, 1, 2, 3, 5}
    assert _kept(O.topk_threshold_probs(l, 1.0, 0)) == set(range(6))  # top_k <= 0: no cut (model.py:958)
    assert _kept(O.topk_threshold_probs(l, 1.0, 99)) == set(range(6))  # top_k >= CS
    w = O.topk_threshold_probs(l, 0.5, 2)
    np.testing.assert_allclose(w[[1, 2]], [1.0, math.exp((2.0 - 3.0) / 0.5)], rtol=1e-6)


def test_cb0_rule_keeps_exactly_k():
    # engine.py:855-863: probs.topk(k) + scatter keeps exactly k entries; ties go to the lowest indices
    l = torch.tensor([1.0, 3.0, 2.0, 2.0, 0.5, 2.0])
    assert _kept(O.cb0_probs(l, 1.0, 2)) == {1, 2}
    assert _kept(O.cb0_probs(l, 1.0, 3)) == {1, 2, 3}
    assert _kept(O.cb0_probs(l, 1.0, 4)) == {1, 2, 3, 5}
    assert _kept(O.cb0_probs(l, 1.0, 0)) == set(range(6))
    assert _kept(O.cb0_probs(l, 1.0, 6)) == set(range(6))
    p = O.cb0_probs(l, 0.7, 3)
    full = torch.softmax(l / 0.7, -1).numpy()
    np.testing.assert_allclose(p[[1, 2, 3]], full[[1, 2, 3]], rtol=1e-6)  # kept values are the softmax's own


@pytest.mark.parametrize("rule", ["rq", "cb0"])
def test_rules_against_brute_force(rule):
    """Every vocabulary of 5 values from {0, 1, 2} (so ties everywhere) and every k."""
    for vals in itertools.product((0.0, 1.0, 2.0), repeat=5):
        l = torch.tensor(vals)
        for k in range(1, 6):
            srt = sorted(vals, reverse=True)
            kth = srt[k - 1]
            if rule == "rq":
                want = {i for i, v in enumerate(vals) if v >= kth}
                got = _kept(O.topk_threshold_probs(l, 1.0, k))
            else:
                above = [i for i, v in enumerate(vals) if v > kth]
                tied = [i for i, v in enumerate(vals) if v == kth]
                want = set(above + tied[:k - len(above)])
                got = _kept(O.cb0_probs(l, 1.0, k))
                assert len(got) == k
            assert got == want, (vals, k)


def test_inverse_cdf_edges_and_greedy():
    l = torch.tensor([0.0, math.log(2.0), -50.0, math.log(1.0)])  # weights 1 : 2 : ~0 : 1
    # cumulative thresholds at 1/4 and 3/4 of the kept mass
    assert O.sample_rq(l, 1.0, 0, 0.0) == 0
    assert O.sample_rq(l, 1.0, 0, 0.2499) == 0
    assert O.sample_rq(l, 1.0, 0, 0.2501) == 1
    assert O.sample_rq(l, 1.0, 0, 0.7499) == 1
    assert O.sample_rq(l, 1.0, 0, 0.7501) == 3  # index 2 carries (almost) no mass
    assert O.sample_rq(l, 1.0, 0, 1.0 - 2.0 ** -24) == 3
    # dropped entries are never drawn, whatever u
    for u in np.linspace(0, 1 - 2.0 ** -24, 50):
        assert O.sample_rq(l, 1.0, 2, float(u)) in (1, 0, 3)  # k=2: threshold = 1.0-weight entries tie -> kept
        assert O.sample_rq(l, 1.0, 1, float(u)) == 1
    # greedy: lowest index of the maximum
    t = torch.tensor([1.0, 5.0, 5.0, 2.0])
    assert O.sample_rq(t, 0.8, 1, 0.9) == 1 and O.sample_rq(t, 0.0, 50, 0.9) == 1
    assert O.sample_cb0(t, torch.zeros(4), 1.0, 0.8, 1, 0.9) == 1
    # penalty moves the greedy pick (engine.py:571-576 before the draw)
    assert O.sample_cb0(t, torch.tensor([0.0, 3.0, 3.0, 0.0]), 2.0, 0.8, 1, 0.9) == 3


def test_draw_frequencies_follow_kept_weights():
    l = torch.tensor([0.3, 1.2, -0.4, 0.9, 0.0, 1.2])
    for rule, k in (("rq", 3), ("cb0", 3)):
        w = O.topk_threshold_probs(l, 0.8, k) if rule == "rq" else O.cb0_probs(l, 0.8, k)
        w = w / w.sum()
        n = 6000
        hits = np.zeros(6)
        for f in range(n):
            u = O.uniform01(11, f, 0, 1)
            j = O.sample_rq(l, 0.8, k, u) if rule == "rq" else O.sample_cb0(l, torch.zeros(6), 1.0, 0.8, k, u)
            hits[j] += 1
        assert set(np.nonzero(hits)[0]) == _kept(w)
        exp = w * n
        chi2 = ((hits - exp) ** 2 / np.maximum(exp, 1e-9))[w > 0].sum()
        assert chi2 < 25.0, (rule, chi2)


# ---- attention against an explicit softmax loop ----
@pytest.mark.parametrize("L,hd", [(1, 4), (3, 8), (7, 6)])
def test_attention_against_loops(L, hd):
    g = torch.Generator().manual_seed(L * 10 + hd)
    q, k, v = torch.randn(2, hd, generator=g), torch.randn(L, hd, generator=g), torch.randn(L, hd, generator=g)
    mask = torch.ones(2, L, dtype=torch.bool)
    if L > 1:
        mask[0, L - 1] = False
    got = O.attention(q, k, v, hd ** -0.5, F32, mask)
    for t in range(2):
        s = [sum(q[t, e].item() * k[j, e].item() for e in range(hd)) * hd ** -0.5 for j in range(L)]
        s = [s[j] if mask[t, j] else -math.inf for j in range(L)]
        m = max(s)
        w = [math.exp(x - m) for x in s]
        for e in range(hd):
            want = sum(w[j] * v[j, e].item() for j in range(L)) / sum(w)
            assert abs(got[t, e].item() - want) < 1e-5
    # bf16 regime: the same sums, one rounding at the end
    gb = O.attention(q, k, v, hd ** -0.5, BF, mask)
    assert torch.equal(gb, got.to(BF).float())


# ---- int8 weight-only format ----
def test_quantize_int8_round_trip_and_linear():
    g = torch.Generator().manual_seed(5)
    W = torch.randn(9, 33, generator=g) * 0.05
    W[3] = 0.0  # an all-zero row must not divide by zero
    q, s = O.quantize_int8(W)
    assert q.dtype == torch.int8 and int(q.abs().max()) <= 127
    assert torch.equal(s, s.to(BF).float())  # scales are bf16 values
    raw = W.abs().amax(1) / 127.0
    nz = raw > 0
    assert ((s[nz] - raw[nz]).abs() <= raw[nz] * 2.0 ** -8).all()  # bf16 rounding of max|w|/127
    deq = q.float() * s[:, None]
    # inside the clamp the error is half a step; a scale rounded down can push the row maximum past 127
    inside = (W / s[:, None]).abs() <= 127.0
    assert ((W - deq).abs()[inside] <= (s[:, None] / 2 * (1 + 1e-6)).expand_as(W)[inside]).all()
    assert ((W - deq).abs() <= (s[:, None] * (0.5 + 127 * 2.0 ** -8)).expand_as(W) + 1e-12).all()
    assert torch.equal(q[3], torch.zeros(33, dtype=torch.int8))
    # each row's largest element lands on +-127
    assert (q.abs().amax(1)[nz] == 127).all()
    x = torch.randn(2, 33, generator=g).to(BF).float()
    got = O.linear_int8(x, q, s, F32)
    for b in range(2):
        for n in range(9):
            acc = sum(int(q[n, kk]) * x[b, kk].item() for kk in range(33))
            assert abs(got[b, n].item() - acc * s[n].item()) <= 1e-5 * max(1.0, abs(acc * s[n].item()))
    assert torch.equal(O.linear_int8(x, q, s, BF), got.to(BF).float())


# ---- nucleus cut (sampling.sample_top_p / sample_top_p_top_k) ----
def _nucleus_by_hand(probs, p, top_k=None):
    """The rule read off src/vui/sampling.py:23-43 as plain loops over exact fractions: walk the entries from
    the largest down (equal ones by index), drop an entry when the mass strictly ahead of it exceeds p; with
    top_k, of the survivors keep those not smaller than the k-th largest value of the masked vector."""
    from fractions import Fraction

    fr = [Fraction(x) for x in probs]
    order = sorted(range(len(fr)), key=lambda i: (-fr[i], i))
    ahead, kept = Fraction(0), []
    for i in order:
        if not ahead > Fraction(p):
            kept.append(i)
        ahead += fr[i]
    if top_k is not None:
        masked = sorted((fr[i] if i in kept else Fraction(0) for i in range(len(fr))), reverse=True)
        kth = masked[min(top_k, len(fr)) - 1]
        kept = [i for i in kept if fr[i] >= kth]
    return set(kept)


def test_nucleus_rule_against_brute_force():
    """Every vector of 5 eighths summing to one (all orders, so ties and the index rule are met), every
    p in eighths from 0 to 1 and beyond: sums of eighths are exact in fp32, so "mass exactly at p" is
    decided the same way by the oracle's float arithmetic and by the fractions."""
    n = 0
    for parts in itertools.product(range(0, 9), repeat=5):
        if sum(parts) != 8:
            continue
        probs = [c / 8 for c in parts]
        t = torch.tensor(probs, dtype=F32)
        for p16 in (0, 2, 4, 6, 8, 10, 12, 14, 16, 20):
            want = _nucleus_by_hand(probs, p16 / 16)
            got = O.top_p_probs(t, p16 / 16)
            assert set(torch.nonzero(got).flatten().tolist()) == {i for i in want if probs[i] > 0}, (parts, p16)
            # kept weights are the probabilities renormalised over the kept set
            tot = sum(probs[i] for i in want)
            for i in want:
                assert abs(float(got[i]) - probs[i] / tot) < 1e-6
            for k in (1, 2, 4, 5):
                wantk = _nucleus_by_hand(probs, p16 / 16, k)
                gotk = O.top_p_top_k_probs(t, p16 / 16, k)
                assert set(torch.nonzero(gotk).flatten().tolist()) == {i for i in wantk if probs[i] > 0}, (parts, p16, k)
            n += 1
    assert n == 4950


def test_nucleus_special_cases():
    t = torch.tensor([0.125, 0.5, 0.125, 0.25], dtype=F32)
    # the largest entry always survives (nothing lies ahead of it), also with p = 0
    assert torch.nonzero(O.top_p_probs(t, 0.0)).flatten().tolist() == [1]
    # mass exactly at p: 0.5 is not "> 0.5", so the second entry is kept; the third (0.75 ahead) is not
    assert torch.nonzero(O.top_p_probs(t, 0.5)).flatten().tolist() == [1, 3]
    # equal probabilities across the boundary: the lower index is the one kept
    assert torch.nonzero(O.top_p_probs(t, 0.75)).flatten().tolist() == [0, 1, 3]
    # p >= 1 keeps everything and changes nothing
    assert torch.allclose(O.top_p_probs(t, 1.0), t)
    # _sample_codes' dispatch (inference.py:491-504)
    lg = torch.log(t)
    assert np.count_nonzero(O.sample_codes_probs(lg, 1.0, None, None)) == 4
    assert np.count_nonzero(O.sample_codes_probs(lg, 1.0, 2, None)) == 2
    assert np.count_nonzero(O.sample_codes_probs(lg, 1.0, None, 0.0)) == 4    # top_p = 0 alone: no cut at all
    assert np.count_nonzero(O.sample_codes_probs(lg, 1.0, 3, 0.0)) == 1       # beside a top_k: the nucleus of p = 0
    assert np.count_nonzero(O.sample_codes_probs(lg, 1.0, 1, 0.9)) == 1
