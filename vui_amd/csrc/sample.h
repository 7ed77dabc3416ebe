// Block-wide sampler shared by the stand-alone sampling kernel and the fused frame kernel.
#pragma once
#include "common.h"

// ---- Philox4x32-10 (Salmon et al. 2011) ----
__device__ __forceinline__ uint32_t philox_u32(uint64_t seed, uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3) {
  uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1; c3 = (uint32_t)p0; c0 = n0; c2 = n2;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return c0;
}

__device__ __forceinline__ uint32_t float_key(float f) {  // order-preserving map to uint32
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

#define SAMP_THREADS 256
#define SAMP_MAX_E 32  // elements per thread -> CS <= 8192

struct SampleShared {
  float sred[SAMP_THREADS / WAVE];
  int ired[SAMP_THREADS / WAVE];
  float wsum[SAMP_THREADS / WAVE];
  int cnt[2][3 * SAMP_THREADS / WAVE];
  int pick[2];     // slot codebook % 2: consecutive draws of a workgroup alternate, so a draw needs no barrier after its last read
  int tie[SAMP_THREADS / WAVE];  // per wave: keys above the threshold | keys equal to it << 16 (exact-k cut)
#ifdef VUI_SAMPLE_CLOCK
  unsigned long long ts[8];
#endif
};
#ifdef VUI_SAMPLE_CLOCK
#define SAMP_TS(k) do { if (threadIdx.x == 0) sh.ts[k] = wall_clock64(); } while (0)
#else
#define SAMP_TS(k) do { } while (0)
#endif
// Scratch of the digit search: one 256-bin histogram per 8-bit round (two rounds for keys that come from bf16
// values, four for fp32 keys), so that no round has to wait for the bins of an earlier one to be cleared.
#define HIST_WORDS (4 * 256)

// Every wave calls this after the barrier that completes the round's histogram and finds, for itself, the largest
// digit whose suffix count (keys with digit >= it) reaches `need` and the number of keys above that digit: the
// four waves arrive at the same answer without a word passing between them.
__device__ __forceinline__ void hist_select(const int* hist, int need, int& digit_out, int& over_out) {
  const int lane = threadIdx.x & 63;
  const int4 b = *reinterpret_cast<const int4*>(&hist[4 * lane]);  // bins 4*lane .. 4*lane+3
  const int s3 = b.w, s2 = s3 + b.z, s1 = s2 + b.y, s0 = s1 + b.x;  // suffix sums inside the lane
  // exclusive suffix over the lanes: keys in the bins of higher lanes
  int v = s0;
  v += dpp_i<0x101>(v);  // row_shl:1 (a lane reads from higher lanes of its row, 0 from outside)
  v += dpp_i<0x102>(v);
  v += dpp_i<0x104>(v);
  v += dpp_i<0x108>(v);
  {
    const int t3 = __builtin_amdgcn_readlane(v, 48), t2 = __builtin_amdgcn_readlane(v, 32), t1 = __builtin_amdgcn_readlane(v, 16);
    const int row = lane >> 4;
    v += (row <= 2 ? t3 : 0) + (row <= 1 ? t2 : 0) + (row <= 0 ? t1 : 0);
  }
  const int above = v - s0;
  // bin k of this lane: suffix = above + s_k, suffix beyond it = suffix - bin_k
  int digit = -1, over = 0;
  if (above + s3 >= need && above < need) { digit = 4 * lane + 3; over = above; }
  else if (above + s2 >= need && above + s3 < need) { digit = 4 * lane + 2; over = above + s3; }
  else if (above + s1 >= need && above + s2 < need) { digit = 4 * lane + 1; over = above + s2; }
  else if (above + s0 >= need && above + s1 < need) { digit = 4 * lane; over = above + s1; }
  // exactly one lane holds the answer when the round's keys number at least `need` (they do: need <= top_k < CS)
  const unsigned long long found = __ballot(digit >= 0);
  const int src = found ? (int)__builtin_ctzll(found) : 0;
  digit_out = max(__builtin_amdgcn_readlane(digit, src), 0);
  over_out = __builtin_amdgcn_readlane(over, src);
}

// One draw from the values l[e] (element index tid*E + e, -inf beyond CS) held by a 256-thread
// block.  RQ rule (src/vui/model.py:955-962): drop l < k-th largest, softmax, draw.  code-0 rule
// (src/vui/engine.py:855-863): softmax, keep the top-k probabilities, renormalise, draw.  Both
// are: keep {l >= k-th largest l} (code 0: cut to exactly k, see exact_k), weights exp(l - max), inverse CDF in index order with one
// uniform (rnd: philox_u32(seed, frame, row, codebook, 0), computed by the caller ahead of its last wait; codebook
// also picks the slot of the shared result, see SampleShared).  greedy: the lowest index of the maximum.  Every
// thread returns the same pick.
// hist: HIST_WORDS ints of LDS scratch (16-byte aligned) for the digit histograms.
//
// key[e] orders the elements for the top-k cut (any order-preserving image of l[e]); bits below
// low_bit are known to carry no information (16 when the keys come from bf16 values).  low_bit 16 or 0:
// two or four rounds of an 8-bit digit histogram; otherwise two bits per barrier over bits 31..low_bit,
// stopping as soon as exactly top_k keys lie above the candidate.
//
// exact_k (the code-0 rule: topk + scatter keeps exactly top_k entries): of the keys that tie with the k-th largest
// only as many as fill the quota are kept, lowest indices first (torch.topk leaves the choice among equal values
// open); without it every tie is kept (the depth-head rule drops only l < k-th).
template <int EMAX>
__device__ __forceinline__ int block_sample(const float (&l)[EMAX], const uint32_t (&key)[EMAX], int low_bit, int CS,
                                            int E, bool greedy, int top_k, uint32_t rnd, uint32_t codebook,
                                            SampleShared& sh, int* hist, bool exact_k = false) {
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  SAMP_TS(0);
  const bool digits = top_k > 0 && top_k < CS && (low_bit == 16 || low_bit == 0) && !greedy;
  float m = -INFINITY; int mi = 0x7fffffff;
#pragma unroll
  for (int e = 0; e < EMAX; ++e)
    if (e < E && l[e] > m) { m = l[e]; mi = tid * E + e; }
  {
    const float wm = rows_max(group16_max(m));
    // the index of the maximum is the answer of a greedy draw and the fallback of a sampled one
    const int cand = wave_min_i((m == wm) ? mi : 0x7fffffff);
    if (lane == 0) { sh.sred[wave] = wm; sh.ired[wave] = cand; }
  }
  const int rounds = (32 - low_bit) / 8;
  int* pick_slot = &sh.pick[codebook & 1];
  if (tid == 0) *pick_slot = -1;
  if (digits) {
#pragma unroll
    for (int i = 0; i < 4; ++i) if (i < rounds) hist[tid + SAMP_THREADS * i] = 0;
  }
  __syncthreads();
  float M = sh.sred[0]; int Mi = sh.ired[0];
#pragma unroll
  for (int w = 1; w < SAMP_THREADS / WAVE; ++w) {
    if (sh.sred[w] > M) { M = sh.sred[w]; Mi = sh.ired[w]; }
    else if (sh.sred[w] == M) Mi = min(Mi, sh.ired[w]);
  }
  // Logits that hold no ordinary number (all NaN or all -inf: only a launch that has given up its waits and runs on
  // with unfinished words can produce them) leave no candidate; the pick must still be an index of the codebook,
  // because callers gather embedding rows with it.
  if (Mi < 0 || Mi >= CS) Mi = 0;
  if (greedy) { __syncthreads(); return Mi; }
  SAMP_TS(1);

  // key of the k-th largest value
  uint32_t thr = 0u;
  if (digits) {
    // one byte per round from the top, each among the keys that share the bytes chosen so far
    int need = top_k;
#pragma unroll
    for (int round = 0; round < 4; ++round) {
      if (round >= rounds) break;
      const int shift = 24 - 8 * round;
      int* bins = hist + 256 * round;
#pragma unroll
      for (int e = 0; e < EMAX; ++e)
        if (e < E && tid * E + e < CS && (round == 0 || (key[e] >> (shift + 8)) == (thr >> (shift + 8))))
          atomicAdd(&bins[(key[e] >> shift) & 255], 1);
      __syncthreads();
      SAMP_TS(2 + 2 * round);
      int digit, over;
      hist_select(bins, need, digit, over);
      SAMP_TS(3 + 2 * round);
      thr |= (uint32_t)digit << shift;
      need -= over;
    }
  } else if (top_k > 0 && top_k < CS) {
    int it = 0;
    for (int bit = 30; bit >= low_bit; bit -= 2, ++it) {
      const uint32_t c1 = thr | (1u << bit), c2 = thr | (2u << bit), c3 = thr | (3u << bit);
      // per-lane counts on the vector ALU (three 10-bit fields), one packed wave reduction
      int pk = 0;
#pragma unroll
      for (int e = 0; e < EMAX; ++e)
        if (e < E) pk += (key[e] >= c1 ? 1 : 0) + (key[e] >= c2 ? (1 << 10) : 0) + (key[e] >= c3 ? (1 << 20) : 0);
      pk = wave_sum_i(pk);  // per field at most 64 * EMAX <= 1023 when EMAX <= 15; wider EMAX uses three sums
      int n1 = pk & 1023, n2 = (pk >> 10) & 1023, n3 = (pk >> 20) & 1023;
      if (EMAX > 15) {
        int q1 = 0, q2 = 0, q3 = 0;
#pragma unroll
        for (int e = 0; e < EMAX; ++e)
          if (e < E) { q1 += key[e] >= c1; q2 += key[e] >= c2; q3 += key[e] >= c3; }
        n1 = wave_sum_i(q1); n2 = wave_sum_i(q2); n3 = wave_sum_i(q3);
      }
      int* buf = sh.cnt[it & 1];
      if (lane == 0) { buf[wave * 3] = n1; buf[wave * 3 + 1] = n2; buf[wave * 3 + 2] = n3; }
      __syncthreads();
      int t1 = 0, t2 = 0, t3 = 0;
#pragma unroll
      for (int w = 0; w < SAMP_THREADS / WAVE; ++w) { t1 += buf[w * 3]; t2 += buf[w * 3 + 1]; t3 += buf[w * 3 + 2]; }
      int tsel = CS;
      if (t3 >= top_k) { thr = c3; tsel = t3; }
      else if (t2 >= top_k) { thr = c2; tsel = t2; }
      else if (t1 >= top_k) { thr = c1; tsel = t1; }
      if (tsel == top_k) break;  // exactly k keys are >= thr: the kept set is final
    }
  }
  // exact-k: how many of this thread's ties with the threshold are kept (all of them otherwise)
  int tie_keep = EMAX;
  if (exact_k && top_k > 0 && top_k < CS) {
    const uint32_t tt = thr >> low_bit;
    int gt = 0, eq = 0;
#pragma unroll
    for (int e = 0; e < EMAX; ++e)
      if (e < E && tid * E + e < CS) { gt += (key[e] >> low_bit) > tt; eq += (key[e] >> low_bit) == tt; }
    const int mine = gt | (eq << 16);  // both counts stay below 2^14 (CS <= 8192)
    int incl = mine;
    incl += dpp_i<0x111>(incl);  // row_shr:1 .. 8: inclusive scan inside each row of 16 lanes
    incl += dpp_i<0x112>(incl);
    incl += dpp_i<0x114>(incl);
    incl += dpp_i<0x118>(incl);
    {
      const int t0 = __builtin_amdgcn_readlane(incl, 15), t1 = __builtin_amdgcn_readlane(incl, 31), t2 = __builtin_amdgcn_readlane(incl, 47);
      const int row = lane >> 4;
      incl += (row >= 1 ? t0 : 0) + (row >= 2 ? t1 : 0) + (row >= 3 ? t2 : 0);
    }
    if (lane == WAVE - 1) sh.tie[wave] = incl;
    __syncthreads();
    int before = incl - mine, total = 0;
#pragma unroll
    for (int w = 0; w < SAMP_THREADS / WAVE; ++w) { if (w < wave) before += sh.tie[w]; total += sh.tie[w]; }
    const int quota = top_k - (total & 0xffff);  // ties to keep over the whole block, >= 1
    tie_keep = max(0, min(eq, quota - (before >> 16)));
  }
  // weights, their total, and the inverse CDF in index order
  float wloc = 0.f;
  float pw[EMAX];
  {
    const uint32_t tt = thr >> low_bit;
    int ties_seen = 0;
#pragma unroll
    for (int e = 0; e < EMAX; ++e) {
      pw[e] = 0.f;
      if (e < E && tid * E + e < CS && key[e] >= thr) {
        bool keep = true;
        if (exact_k && (key[e] >> low_bit) == tt) keep = ties_seen++ < tie_keep;
        if (keep) pw[e] = __expf(l[e] - M);
      }
      wloc += pw[e];
    }
  }
  // inclusive scan over the wave: shifts inside each row of 16 lanes, then the row totals
  float incl = wloc;
  incl += dpp_f<0x111>(incl);  // row_shr:1, lanes shifted in from outside the row read 0
  incl += dpp_f<0x112>(incl);  // row_shr:2
  incl += dpp_f<0x114>(incl);  // row_shr:4
  incl += dpp_f<0x118>(incl);  // row_shr:8
  {
    const float t0 = lane_f(incl, 15), t1 = lane_f(incl, 31), t2 = lane_f(incl, 47);
    const int row = lane >> 4;
    incl += (row >= 1 ? t0 : 0.f) + (row >= 2 ? t1 : 0.f) + (row >= 3 ? t2 : 0.f);
  }
  SAMP_TS(6);
  if (lane == WAVE - 1) sh.wsum[wave] = incl;
  __syncthreads();
  float base = 0.f, total = 0.f;
#pragma unroll
  for (int w = 0; w < SAMP_THREADS / WAVE; ++w) { if (w < wave) base += sh.wsum[w]; total += sh.wsum[w]; }
  const float u = (float)(rnd >> 8) * (1.0f / 16777216.0f);
  const float target = u * total;
  const float before = base + incl - wloc;  // sum of everything ahead of this thread
  if (target >= before && target < before + wloc) {
    float run = before; int j = -1;
#pragma unroll
    for (int e = 0; e < EMAX; ++e) {
      if (e < E && j < 0) { run += pw[e]; if (pw[e] > 0.f && run > target) j = tid * E + e; }
    }
    if (j < 0) {  // rounding at the thread's upper edge: take its last kept element
#pragma unroll
      for (int e = 0; e < EMAX; ++e) if (e < E && pw[e] > 0.f) j = tid * E + e;
    }
    if (j >= 0) atomicMax(pick_slot, j);
  }
  __syncthreads();
  const int got = *pick_slot;
  const int pick = (got >= 0) ? got : Mi;
  SAMP_TS(7);
  // no barrier here: the next draw of this workgroup (codebook + 1) uses the other slot, and every other word of the
  // shared state is next written behind a barrier of that draw which this read precedes
  return pick;
}

// ---- nucleus cut (sampling.sample_top_p / sample_top_p_top_k, src/vui/sampling.py:23-43) ----
// In the order "largest probability first, equal ones by index" an element is kept while the probability mass
// strictly ahead of it is <= top_p; everything behind is dropped (l = -inf) before the top-k cut and the draw of
// block_sample.  The masses are summed as integers (weight exp(l - max) in units of 2^-32, 64-bit totals), so the
// kept set does not depend on the order in which threads add: the same logits always give the same set.
// The boundary key is found one byte per round from the top, as the k-th key is in block_sample: per round a
// 256-bin histogram of MASS among the keys that share the bytes chosen so far, and the lowest digit whose mass
// above it still fits the remaining budget.  Of the keys equal to the boundary key (equal probabilities) the
// lowest indices are kept, one more than fit entirely into what is left of the budget.
// mass: 256 words of LDS; ties: one int per wave.  Every thread of the 256 calls this.
struct NucleusShared {
  unsigned long long mass[256];
  unsigned long long tot[SAMP_THREADS / WAVE];
  float mx[SAMP_THREADS / WAVE];
  int ties[SAMP_THREADS / WAVE];
};
__device__ __forceinline__ unsigned long long shfl_down_u64(unsigned long long v, int off) {
  const uint32_t lo = (uint32_t)__shfl_down((int)(uint32_t)v, off), hi = (uint32_t)__shfl_down((int)(uint32_t)(v >> 32), off);
  return ((unsigned long long)hi << 32) | lo;
}
template <int EMAX>
__device__ __forceinline__ void nucleus_cut(float (&l)[EMAX], uint32_t (&key)[EMAX], int low_bit, int CS, int E, float top_p,
                                            NucleusShared& ns) {
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  // maximum, then the integer weights and their total
  float m = -INFINITY;
#pragma unroll
  for (int e = 0; e < EMAX; ++e) if (e < E) m = fmaxf(m, l[e]);
  m = rows_max(group16_max(m));
  if (lane == 0) ns.mx[wave] = m;
  ns.mass[tid] = 0ull;
  __syncthreads();
  float M = ns.mx[0];
#pragma unroll
  for (int w = 1; w < SAMP_THREADS / WAVE; ++w) M = fmaxf(M, ns.mx[w]);
  unsigned long long q[EMAX], mine = 0ull;
#pragma unroll
  for (int e = 0; e < EMAX; ++e) {
    q[e] = 0ull;
    if (e < E && tid * E + e < CS) q[e] = (unsigned long long)(__expf(l[e] - M) * 4294967296.0f);
    mine += q[e];
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) mine += shfl_down_u64(mine, off);
  if (lane == 0) ns.tot[wave] = mine;
  __syncthreads();
  unsigned long long Z = 0ull;
#pragma unroll
  for (int w = 0; w < SAMP_THREADS / WAVE; ++w) Z += ns.tot[w];
  unsigned long long rem = (unsigned long long)((double)top_p * (double)Z);  // the budget: mass allowed strictly ahead
  uint32_t thr = 0u;
  const int rounds = (32 - low_bit) / 8;
  for (int round = 0; round < rounds; ++round) {
    const int shift = 24 - 8 * round;
#pragma unroll
    for (int e = 0; e < EMAX; ++e)
      if (e < E && tid * E + e < CS && q[e] && (round == 0 || (key[e] >> (shift + 8)) == (thr >> (shift + 8))))
        atomicAdd(&ns.mass[(key[e] >> shift) & 255], q[e]);
    __syncthreads();
    // every wave for itself: lane holds bins 4 lane .. 4 lane + 3; mass above each of them inside the round
    const unsigned long long b0 = ns.mass[4 * lane], b1 = ns.mass[4 * lane + 1], b2 = ns.mass[4 * lane + 2], b3 = ns.mass[4 * lane + 3];
    unsigned long long above = b0 + b1 + b2 + b3;  // becomes: mass in the bins of higher lanes
    {
      unsigned long long v = above;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long t = shfl_down_u64(v, off);
        if (lane + off < 64) v += t;
      }
      above = v - above;
    }
    // the lowest digit whose mass above still fits: the lanes' candidates, lowest lane wins
    int digit = -1;
    unsigned long long ab = 0ull;
    if (above + b3 + b2 + b1 <= rem) { digit = 4 * lane; ab = above + b3 + b2 + b1; }
    else if (above + b3 + b2 <= rem) { digit = 4 * lane + 1; ab = above + b3 + b2; }
    else if (above + b3 <= rem) { digit = 4 * lane + 2; ab = above + b3; }
    else if (above <= rem) { digit = 4 * lane + 3; ab = above; }
    const unsigned long long found = __ballot(digit >= 0);  // never empty: nothing lies above digit 255
    const int src = (int)__builtin_ctzll(found);
    digit = __builtin_amdgcn_readlane(digit, src);
    const uint32_t ab_lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)ab, src), ab_hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(ab >> 32), src);
    rem -= ((unsigned long long)ab_hi << 32) | ab_lo;
    thr |= (uint32_t)digit << shift;
    __syncthreads();  // every wave has read the bins
    ns.mass[tid] = 0ull;
    __syncthreads();
  }
  // the boundary class: keys equal to thr (above low_bit); their common weight; ranks in index order
  const uint32_t tt = thr >> low_bit;
  int eq = 0;
  unsigned long long qc = 0ull;
#pragma unroll
  for (int e = 0; e < EMAX; ++e)
    if (e < E && tid * E + e < CS && (key[e] >> low_bit) == tt) { ++eq; qc = q[e]; }
  int incl = eq;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int t = __shfl_up(incl, off);
    if (lane >= off) incl += t;
  }
  if (lane == WAVE - 1) ns.ties[wave] = incl;
  // any member's weight will do (equal keys carry equal values): the largest seen in the wave, then in the block
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) { const unsigned long long t = shfl_down_u64(qc, off); qc = t > qc ? t : qc; }
  if (lane == 0) ns.tot[wave] = qc;
  __syncthreads();
  int before = incl - eq;
  unsigned long long qcl = 0ull;
#pragma unroll
  for (int w = 0; w < SAMP_THREADS / WAVE; ++w) { if (w < wave) before += ns.ties[w]; qcl = ns.tot[w] > qcl ? ns.tot[w] : qcl; }
  // member number r (from 0) has r * qcl ahead of it inside the class
  const unsigned long long fit = qcl ? rem / qcl : 0xffffffffull;
  const unsigned long long n_keep = fit + 1ull;
  int seen = 0;
  const uint32_t dropped = float_key(-INFINITY);
#pragma unroll
  for (int e = 0; e < EMAX; ++e) {
    if (e < E && tid * E + e < CS) {
      const uint32_t k = key[e] >> low_bit;
      bool keep = k > tt;
      if (k == tt) { keep = (unsigned long long)(before + seen) < n_keep; ++seen; }
      if (!keep) { l[e] = -INFINITY; key[e] = dropped; }
    }
  }
  __syncthreads();
}

// penalised, biased, temperature-scaled value of one logit
__device__ __forceinline__ float sample_value(float v, const float* bias, int j, const float* counts, float penalty,
                                              float div) {
  if (bias) v += bias[j];
  if (counts && penalty > 1.0f) {
    const float f = powf(penalty, counts[j]);
    v = (v > 0.f) ? v / f : v * f;
  }
  return v / div;
}

// rolling repetition state of one row (src/vui/engine.py:578-590); one thread
__device__ __forceinline__ void rep_push(float* cnt, int32_t* hist, int32_t* pos2, int window, int pick) {
  if (window > 0 && hist) {
    int head = pos2[0], filled = pos2[1];
    if (filled == window) cnt[hist[head]] -= 1.0f;
    hist[head] = pick;
    head = (head + 1) % window;
    if (filled < window) ++filled;
    pos2[0] = head; pos2[1] = filled;
  }
  cnt[pick] += 1.0f;
}
