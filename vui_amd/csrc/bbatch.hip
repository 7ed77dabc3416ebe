// The backbone decode step for 2..16 rows as ONE persistent kernel (bf16 activations, bf16 or int8 weights).
//
//   Engine._backbone_decode_body / _backbone_decode_body_b  (src/vui/engine.py:434-449, 485-534)
//   Block.forward_flash, MHA.forward_flash, LlamaMLP        (src/vui/model.py:204-258, 282, 359-375)
//
// As a kernel sequence the step is ~110 dependent launches whatever the number of rows, i.e. bound by the cost of a
// kernel boundary.  Here one resident grid (one workgroup per CU) walks the layers and hands the small activation
// vectors from phase to phase through flag-in-data words (ll.h), as the batch-1 frame kernel and the batched depth
// head do, with the matrix cores inside: a workgroup owns tiles of 16 output features of each weight matrix and
// multiplies them with the activations of its rows (v_mfma_f32_16x16x32_bf16, int8 weights widened in registers).
//
// Rows are dealt to min(rows, 4) row groups, sorted by cache length and dealt in serpentine order so that the
// groups carry about the same number of keys; a group is served by NWL = 256 / groups workgroups (128 for 2 rows,
// 64 from 3 rows on), because what a phase costs is the number of exchanged words one workgroup has to wait for:
// four groups of one or two rows beat one or two groups of four (measured: 4 rows 1434 -> 1371 us per frame step,
// 8 rows 1603 -> 1557), although a lone row's keys are then streamed by 64 workgroups instead of 256.
// Per layer and group:
//   A  RMSNorm + QKV tiles, rotation of q and k in the epilogue; k and v of the new position go to the cache and,
//      like q, into the exchange
//   B  attention over the ragged rows: the group's workgroups are dealt to (row, set of HG heads, key range) pieces,
//      long rows getting more key ranges (HG = 2 from 9 rows on: twice as fine a division as one head set per
//      workgroup of a 64-workgroup group allows); keys and values stream from the cache with 16 loads per lane in
//      flight, the new position's come from the exchange
//   C  merge of a (row, head)'s pieces
//   D  out_proj tiles
//   E  residual + RMSNorm + W1/W3 tiles + SwiGLU
//   F  W2 tiles
// then residual + final norm, codec head tiles, eos head, hidden output, position update.
// Rounding points are those of the kernel sequence (gemv_epi.h, attn.hip).
#include "common.h"
#include "internal.h"
#include "ll.h"
#include <stdio.h>
#include <string.h>

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bb_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float bb_floatx4;
union BbU128 { uint4 u; bb_bf16x8 v; };
__device__ __forceinline__ bb_bf16x8 bb_frag(const uint4& x) { BbU128 t; t.u = x; return t.v; }

__device__ __forceinline__ void cvt8(const uint4& r, float* o) {
  o[0] = __uint_as_float(r.x << 16); o[1] = __uint_as_float(r.x & 0xffff0000u);
  o[2] = __uint_as_float(r.y << 16); o[3] = __uint_as_float(r.y & 0xffff0000u);
  o[4] = __uint_as_float(r.z << 16); o[5] = __uint_as_float(r.z & 0xffff0000u);
  o[6] = __uint_as_float(r.w << 16); o[7] = __uint_as_float(r.w & 0xffff0000u);
}

// Keys and values are read once per launch and a batch's caches (1.2 GB for 16 ragged rows) are far larger than the
// memory-side cache, so their loads carry the non-temporal hint and leave the cache to what the step reads again:
// the depth head's matrices of the next launch (16 int8 rows 1726 -> 1650 us per frame step, 8 rows 1546 -> 1507).
// The same hint on the weight tiles - each read by one workgroup of every row group - helped two rows and cost four,
// and is not used.
typedef unsigned int bb_u32x4 __attribute__((ext_vector_type(4)));
template <bool NT> __device__ __forceinline__ uint4 bb_ld16(const void* p) {
  if constexpr (NT) {
    const bb_u32x4 v = __builtin_nontemporal_load((const __attribute__((address_space(1))) bb_u32x4*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
  } else {
    return *reinterpret_cast<const uint4*>(p);
  }
}

#define BB_RG 4        // rows per row group
#define BB_MAXSPL 16   // key ranges per row at most (a merge waits for that many partial results)
#define BB_U 8         // keys per lane group in flight per attention step

struct BbTile { int n0; bool on; };

// Weight fragments of one 16-feature tile, K split over the four waves in steps of 64.  The matrices are read from
// a "tiled" copy: blocks of 16 rows x 64 columns, block (r / 16, k / 64) at ((r / 16) * (K / 64) + k / 64) * 1024
// elements; inside a bf16 block the 8-element piece p = (k % 16) / 8 of lane (r % 16) + 16 * ((k % 64) / 16) sits at
// p * 512 + lane * 8 (the operand layout of the prompt-ingestion GEMMs, whose copy is used), inside an int8 block
// the lane's 16 bytes (k % 16 = 0..15) at lane * 16.  A wave's fragment load is then 1 KiB contiguous.
template <bool I8, int MAXS> struct BbW { uint4 a[I8 ? MAXS : 2 * MAXS]; };

// EXACT: K is MAXS * 256, every wave has exactly MAXS steps and nothing is conditional
template <bool I8, int MAXS, bool EXACT>
__device__ __forceinline__ void bb_prefetch(const void* Wt, int K, const BbTile& t, BbW<I8, MAXS>& r) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (!t.on) return;  // uniform over the workgroup
  const int nsteps = EXACT ? 4 * MAXS : (K >> 6);
  const size_t band = (size_t)(t.n0 >> 4) * nsteps;
#pragma unroll
  for (int i = 0; i < MAXS; ++i) {
    const int s = wave + 4 * i;
    if (EXACT || s < nsteps) {  // uniform over the wave; a step past the end is never used
      if (I8) {
        r.a[i] = bb_ld16<false>((const uint8_t*)Wt + (band + s) * 1024 + lane * 16);
      } else {
        const bf16_t* p = (const bf16_t*)Wt + (band + s) * 1024 + lane * 8;
        r.a[2 * i] = bb_ld16<false>(p);
        r.a[2 * i + 1] = bb_ld16<false>(p + 512);
      }
    }
  }
}

// eight int8 -> four packed bf16 pairs, exact
__device__ __forceinline__ uint4 bb_widen8(uint32_t lo, uint32_t hi) {
  uint4 r;
  r.x = f2bf2((float)(int8_t)(lo & 0xff), (float)(int8_t)((lo >> 8) & 0xff));
  r.y = f2bf2((float)(int8_t)((lo >> 16) & 0xff), (float)(int8_t)(lo >> 24));
  r.z = f2bf2((float)(int8_t)(hi & 0xff), (float)(int8_t)((hi >> 8) & 0xff));
  r.w = f2bf2((float)(int8_t)((hi >> 16) & 0xff), (float)(int8_t)(hi >> 24));
  return r;
}
template <bool I8, int MAXS>
__device__ __forceinline__ void bb_split(const BbW<I8, MAXS>& w, int i, uint4& a0, uint4& a1) {
  if (I8) { const uint4 v = w.a[i]; a0 = bb_widen8(v.x, v.y); a1 = bb_widen8(v.z, v.w); }
  else { a0 = w.a[2 * i]; a1 = w.a[2 * i + 1]; }
}

// NT tiles of one matrix (two matrices when DUAL) against the staged rows in one pass.
// xp: activations as packed bf16 pairs, row stride xs words, row BB_RG all zero (it stands for the columns of the
// matrix-core tile that have no row).  red: NT x 4 x 64 x (4 | 8) floats.  epi(j, n, lr, v[4], u[4]) is called by the
// lanes of wave j for tile j: features n .. n+3 of local row lr (u: second matrix).
template <bool I8, int MAXS, int NT, bool DUAL, bool EXACT, typename Epi>
__device__ __forceinline__ void bb_compute(const uint32_t* xp, int xs, int K, const BbTile (&t)[NT], const BbW<I8, MAXS> (&w)[NT],
                                           const BbW<I8, MAXS> (&w2)[DUAL ? NT : 1], float* red, int nrows, Epi&& epi) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, l16 = lane & 15, kg = lane >> 4;
  if (!t[0].on) return;  // uniform over the workgroup; a later tile is never on without the first
  const int nsteps = EXACT ? 4 * MAXS : (K >> 6);
  bb_floatx4 acc[NT], acc2[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) { acc[j] = bb_floatx4{0.f, 0.f, 0.f, 0.f}; acc2[j] = acc[j]; }
  const uint32_t* xrow = xp + (size_t)min(l16, BB_RG) * xs + 8 * kg;
#pragma unroll
  for (int i = 0; i < MAXS; ++i) {
    const int s = wave + 4 * i;
    if (EXACT || s < nsteps) {  // uniform over the wave: the matrix instructions below run for all 64 lanes
      const uint4 x0 = *reinterpret_cast<const uint4*>(xrow + 32 * s);
      const uint4 x1 = *reinterpret_cast<const uint4*>(xrow + 32 * s + 4);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        if (t[j].on) {
          uint4 a0, a1;
          bb_split<I8, MAXS>(w[j], i, a0, a1);
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bb_frag(a0), bb_frag(x0), acc[j], 0, 0, 0);
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bb_frag(a1), bb_frag(x1), acc[j], 0, 0, 0);
          if (DUAL) {
            bb_split<I8, MAXS>(w2[j], i, a0, a1);
            acc2[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bb_frag(a0), bb_frag(x0), acc2[j], 0, 0, 0);
            acc2[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bb_frag(a1), bb_frag(x1), acc2[j], 0, 0, 0);
          }
        }
      }
    }
  }
  constexpr int per = DUAL ? 8 : 4;
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    if (t[j].on) {
      float* mine = red + ((size_t)(j * 4 + wave) * 64 + lane) * per;
      *reinterpret_cast<bb_floatx4*>(mine) = acc[j];
      if (DUAL) *reinterpret_cast<bb_floatx4*>(mine + 4) = acc2[j];
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    if (wave == j && t[j].on) {
      float v[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int wv = 0; wv < 4; ++wv) {
        const float* src = red + ((size_t)(j * 4 + wv) * 64 + lane) * per;
#pragma unroll
        for (int q = 0; q < 4; ++q) { v[q] += src[q]; if (DUAL) u[q] += src[4 + q]; }
      }
      if (l16 < nrows) epi(j, t[j].n0 + 4 * kg, l16, v, u);
    }
  }
}

struct BbNorm { uint4 w[2]; };  // norm weights of chunks lane, lane + 64 (d <= 1024)
__device__ __forceinline__ BbNorm bb_load_norm(const bf16_t* nw, int d) {
  BbNorm r;
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = min(lane + WAVE * i, d / 8 - 1);
    r.w[i] = *reinterpret_cast<const uint4*>(nw + c * 8);
  }
  return r;
}
// two roundings (src/vui/model.py:292-297): rnd(x * rsqrt(mean x^2 + eps)) then rnd(that * weight); q: the row's
// eight values of chunk ch, r the row's factor
__device__ __forceinline__ uint4 bb_norm8(const float (&q)[8], float r, const uint4& g) {
  uint4 o;
  uint32_t t;
  t = f2bf2(q[0] * r, q[1] * r); o.x = f2bf2(bf_lo(t) * bf_lo(g.x), bf_hi(t) * bf_hi(g.x));
  t = f2bf2(q[2] * r, q[3] * r); o.y = f2bf2(bf_lo(t) * bf_lo(g.y), bf_hi(t) * bf_hi(g.y));
  t = f2bf2(q[4] * r, q[5] * r); o.z = f2bf2(bf_lo(t) * bf_lo(g.z), bf_hi(t) * bf_hi(g.z));
  t = f2bf2(q[6] * r, q[7] * r); o.w = f2bf2(bf_lo(t) * bf_lo(g.w), bf_hi(t) * bf_hi(g.w));
  return o;
}
// RMSNorm of the group's rows of xres (fp32, row stride d) into xp; wave w takes rows w, w + 4, ...
__device__ __forceinline__ void bb_norm_rows(const float* xres, const BbNorm& nw, float eps, int d, int Bg, uint32_t* xp, int xs) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int nch = d / 8;
  for (int b = wave; b < Bg; b += 4) {
    const float* x = xres + (size_t)b * d;
    float q[2][8];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = min(lane + WAVE * i, nch - 1);
      const float4 a = *reinterpret_cast<const float4*>(x + c * 8), bq = *reinterpret_cast<const float4*>(x + c * 8 + 4);
      q[i][0] = a.x; q[i][1] = a.y; q[i][2] = a.z; q[i][3] = a.w; q[i][4] = bq.x; q[i][5] = bq.y; q[i][6] = bq.z; q[i][7] = bq.w;
      const float t = (q[i][0] * q[i][0] + q[i][1] * q[i][1]) + (q[i][2] * q[i][2] + q[i][3] * q[i][3]) +
                      (q[i][4] * q[i][4] + q[i][5] * q[i][5]) + (q[i][6] * q[i][6] + q[i][7] * q[i][7]);
      ss += (lane + WAVE * i < nch) ? t : 0.f;
    }
    ss = wave_sum_v(ss);
    const float r = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = lane + WAVE * i;
      if (c < nch) *reinterpret_cast<uint4*>(xp + (size_t)b * xs + c * 4) = bb_norm8(q[i], r, nw.w[i]);
    }
  }
}
// Residual add of an exchanged vector and the norm that follows, row by row inside one wave (the row never leaves
// the wave: no barrier between wait, add and norm).  Row b of the group sits at buf + rowoff[b] (words).
__device__ __forceinline__ void bb_poll_add_norm_rows(const uint64_t* buf, const int* rowoff, Ctl& c, float* xres, const BbNorm& nw,
                                                      float eps, int d, int Bg, uint32_t* xp, int xs) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int nch = d / 8;
  const int NI = nch > WAVE ? 2 : 1;
  for (int b = wave; b < Bg; b += 4) {
    const uint64_t* row = buf + rowoff[b];
    float* x = xres + (size_t)b * d;
    uint64_t v[2][4] = {};
    int spins = 0;
    while (true) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (i >= NI) break;                            // uniform
        const int ch = min(lane + WAVE * i, nch - 1);  // a chunk past the row repeats the last one and is dropped below
#pragma unroll
        for (int k = 0; k < 4; ++k) v[i][k] = ll_ld(row + 4 * ch + k);
      }
      bool all = true;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int k = 0; k < 4; ++k) all = all && (i >= NI || (uint32_t)(v[i][k] >> 32) == c.epoch);
      if (all || c.dead) break;
      if (++spins > SPIN_LIMIT) {
        c.dead = 1;
        __hip_atomic_store(c.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    float q[2][8];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (i >= NI) break;
      const int ch = min(lane + WAVE * i, nch - 1);
      const float4 o0 = *reinterpret_cast<const float4*>(x + ch * 8), o1 = *reinterpret_cast<const float4*>(x + ch * 8 + 4);
      const float old[8] = {o0.x, o0.y, o0.z, o0.w, o1.x, o1.y, o1.z, o1.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t y = (uint32_t)v[i][k];
        const uint32_t pk = f2bf2(old[2 * k] + bf_lo(y), old[2 * k + 1] + bf_hi(y));  // x = rnd(x + y), model.py:367, 374
        q[i][2 * k] = bf_lo(pk); q[i][2 * k + 1] = bf_hi(pk);
      }
      const float t = (q[i][0] * q[i][0] + q[i][1] * q[i][1]) + (q[i][2] * q[i][2] + q[i][3] * q[i][3]) +
                      (q[i][4] * q[i][4] + q[i][5] * q[i][5]) + (q[i][6] * q[i][6] + q[i][7] * q[i][7]);
      if (lane + WAVE * i < nch) {
        ss += t;
        *reinterpret_cast<float4*>(x + ch * 8) = make_float4(q[i][0], q[i][1], q[i][2], q[i][3]);
        *reinterpret_cast<float4*>(x + ch * 8 + 4) = make_float4(q[i][4], q[i][5], q[i][6], q[i][7]);
      }
    }
    ss = wave_sum_v(ss);
    const float r = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (i >= NI) break;
      const int ch = lane + WAVE * i;
      if (ch < nch) *reinterpret_cast<uint4*>(xp + (size_t)b * xs + ch * 4) = bb_norm8(q[i], r, nw.w[i]);
    }
  }
}

// i / n for 0 <= i < 65536 with inv = ceil(2^32 / n)
__device__ __forceinline__ int bb_div(int i, uint32_t inv) { return (int)__umulhi((uint32_t)i, inv); }

// Wait for `nrows` rows of `len` words each (row b at buf + rowbase(r0 + b), words) and put them into xp rows 0.. as
// they are.  Every thread has NW words in flight per round (one trip to memory for 256 * NW words when the data
// is there).
template <int NW, typename RowBase>
__device__ __forceinline__ void bb_poll_rows_n(const uint64_t* buf, RowBase&& rowbase, int r0, int nrows, int len, uint32_t inv_len, Ctl& c,
                                               uint32_t* xp, int xs) {
  const int n = nrows * len;
  for (int base = 0; base < n; base += FR_THREADS * NW) {
    const uint64_t* p[NW];
    int dst[NW];
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int idx = min(base + (int)threadIdx.x + FR_THREADS * i, n - 1);
      const int lr = bb_div(idx, inv_len), j = idx - lr * len;
      p[i] = buf + rowbase(r0 + lr) + j;
      dst[i] = lr * xs + j;
    }
    uint64_t v[NW];
    int spins = 0;
    while (true) {
#pragma unroll
      for (int i = 0; i < NW; ++i) v[i] = ll_ld(p[i]);
      uint32_t bad = 0;
#pragma unroll
      for (int i = 0; i < NW; ++i) bad |= (uint32_t)(v[i] >> 32) ^ c.epoch;
      if (bad == 0u || c.dead) break;
      if (++spins > SPIN_LIMIT) {
        c.dead = 1;
        __hip_atomic_store(c.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
#pragma unroll
    for (int i = 0; i < NW; ++i)
      if (base + (int)threadIdx.x + FR_THREADS * i < n) xp[dst[i]] = (uint32_t)v[i];
  }
}
// picks the words in flight from the vector length (uniform over the workgroup)
template <typename RowBase>
__device__ __forceinline__ void bb_poll_rows(const uint64_t* buf, RowBase&& rowbase, int r0, int nrows, int len, uint32_t inv_len, Ctl& c,
                                             uint32_t* xp, int xs) {
  const int n = nrows * len;
  if (n <= 2 * FR_THREADS) bb_poll_rows_n<2>(buf, rowbase, r0, nrows, len, inv_len, c, xp, xs);
  else if (n <= 4 * FR_THREADS) bb_poll_rows_n<4>(buf, rowbase, r0, nrows, len, inv_len, c, xp, xs);
  else if (n <= 8 * FR_THREADS) bb_poll_rows_n<8>(buf, rowbase, r0, nrows, len, inv_len, c, xp, xs);
  else bb_poll_rows_n<16>(buf, rowbase, r0, nrows, len, inv_len, c, xp, xs);
}

struct BbArgs {
  int B, d, L, H, KV, hd, F, Q, CS, S, n_slots, window, rope_dim, global_rope_dim;
  unsigned long long global_layers;
  float eps;
  const vui_weights* w;   // device copy of the weight table: norm vectors, embedding table, eos head, rotation tables
  const void* tw;         // tiled matrices of the layers: [wqkv | wo | w1 | w3 | w2] per layer (bf16 or int8)
  const bf16_t* thead;    // tiled codec head (bf16)
  const int64_t* codes_in;
  const uint16_t* emb_in;
  const int32_t* slot_idx;
  int32_t* seq_lens;
  const int32_t* seq_inc;
  uint16_t *kc, *vc, *hidden_out, *cb0_out, *eos_out;
  uint64_t* ll;
  uint32_t *epoch, *arrive, *err;
  int xs;
  int hg;                                  // heads per attention piece (1, 2, 4 or 8; divides H)
  int min_keys;                            // no key range shorter than this is made by splitting
  int off_xp, off_red, off_att, off_misc;  // LDS offsets, bytes (xres at 0)
  unsigned long long* dbg;                 // profiling builds: 256 words for the phase stamps of workgroup dbg_wg
  int dbg_wg;
};

// small per-workgroup state in LDS
struct BbMisc {
  int lens[VUI_MAX_BATCH], slots[VUI_MAX_BATCH], order[VUI_MAX_BATCH];
  int grow[BB_RG], gslot[BB_RG], gpos[BB_RG];  // batch row, cache slot and position of the group's rows
  int off_q[BB_RG], off_d[BB_RG], off_f[BB_RG];  // word offsets of the rows in exchange vectors of nqkv/2, d/2, F/2 words
  int spl[2][BB_RG], poff[2][BB_RG + 1];        // attention plan (0: windowed layers, 1: global layers): key ranges per row, first piece
  int Bg;
  int erow[BB_RG][64];                          // embedding table rows of the group's input codes
};

// SD, SF: K steps (of 64) per wave for K = d_model (and heads x head_dim) and K = ffn.  EXACT: d_model = heads x
// head_dim = SD * 256 and ffn = SF * 256, so no step is conditional (the Vui Nano form).
template <bool I8, int NTQ, int SD, int SF, bool EXACT>
__global__ __launch_bounds__(FR_THREADS, 1) void bb_batch_kernel(const BbArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  float* xres = (float*)smem;                             // [BB_RG][d] residual stream of the group's rows
  uint32_t* xp = (uint32_t*)(smem + a.off_xp);            // [BB_RG + 1][xs] staged activations, the last row stays zero
  float* red = (float*)(smem + a.off_red);                // partial tiles; the merge's pieces
  float* att = (float*)(smem + a.off_att);                // attention role scratch
  BbMisc& ms = *(BbMisc*)(smem + a.off_misc);

  const int wg = blockIdx.x, nwg = gridDim.x, tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int l16 = lane & 15, kg = lane >> 4;
  const int B = a.B, d = a.d, H = a.H, hd = a.hd, F = a.F, S = a.S, xs = a.xs;
  const int nq = H * hd, nkv = a.KV * hd, nqkv = nq + 2 * nkv;
  Ctl c;
  ctl_begin(c, a.epoch, a.err);
  const uint32_t ep = c.epoch;
  const vui_weights& W = *a.w;

  // ---- rows -> groups, roles ----
  const int ngroups = min(B, BB_RG);
  const int NWL = nwg >> (ngroups <= 1 ? 0 : (ngroups <= 2 ? 1 : 2));  // workgroups per group
  const int grp = wg / NWL, wl = wg % NWL;
  if (tid < B) {
    const int slot = a.slot_idx ? a.slot_idx[tid] : tid;
    int len = a.seq_lens[slot];
    len = max(0, min(len, S - 1));
    ms.slots[tid] = slot;
    ms.lens[tid] = len;  // position of the new key = keys already in the cache
  }
  for (int i = tid; i < (BB_RG + 1) * xs; i += FR_THREADS) xp[i] = 0u;
  __syncthreads();
  // every position has been read: only now may this workgroup be counted as arrived (the position update at the end
  // of the launch waits for every workgroup's arrival)
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  if (tid == 0) __hip_atomic_fetch_add(a.arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (tid < B) {  // rank by length, longest first, ties by row index
    int rank = 0;
    const int mine = ms.lens[tid];
    for (int u = 0; u < B; ++u) rank += (ms.lens[u] > mine || (ms.lens[u] == mine && u < tid)) ? 1 : 0;
    ms.order[rank] = tid;
  }
  __syncthreads();
  if (tid == 0) {
    // local row lr of group g is the row of rank lr * ngroups + (lr odd ? ngroups - 1 - g : g)
    int Bg = 0;
    for (int lr = 0; lr < BB_RG; ++lr) {
      const int r = lr * ngroups + ((lr & 1) ? ngroups - 1 - grp : grp);
      if (grp < ngroups && r < B) {
        const int b = ms.order[r];
        ms.grow[Bg] = b; ms.gslot[Bg] = ms.slots[b]; ms.gpos[Bg] = ms.lens[b];
        ms.off_q[Bg] = b * (nqkv / 2); ms.off_d[Bg] = b * (d / 2); ms.off_f[Bg] = b * (F / 2);
        ++Bg;
      }
    }
    for (int lr = Bg; lr < BB_RG; ++lr) { ms.grow[lr] = 0; ms.gslot[lr] = 0; ms.gpos[lr] = 0; ms.off_q[lr] = 0; ms.off_d[lr] = 0; ms.off_f[lr] = 0; }
    ms.Bg = Bg;
    // attention plans: one key range per row to start with (H / HG pieces); the spare workgroups go, one set of
    // pieces at a time, to the row whose ranges are longest (no range below 32 keys)
    for (int v = 0; v < 2; ++v) {
      int nk[BB_RG], sp[BB_RG];
      for (int lr = 0; lr < BB_RG; ++lr) {
        const int len = ms.gpos[lr] + 1;
        const int start = (v == 0 && a.window > 0) ? max(0, len - 1 - a.window) : 0;
        nk[lr] = len - start;
        sp[lr] = lr < Bg ? 1 : 0;
      }
      int spare = NWL / (H / a.hg) - Bg;
      while (spare > 0) {
        int best = -1, bestv = 0;
        for (int lr = 0; lr < Bg; ++lr) {  // the row with the longest ranges that one more range leaves at min_keys or above
          const int per = (nk[lr] + sp[lr] - 1) / sp[lr];
          if (sp[lr] < BB_MAXSPL && nk[lr] >= (sp[lr] + 1) * a.min_keys && per > bestv) { bestv = per; best = lr; }
        }
        if (best < 0) break;
        ++sp[best];
        --spare;
      }
      int off = 0;
      for (int lr = 0; lr < BB_RG; ++lr) { ms.spl[v][lr] = sp[lr]; ms.poff[v][lr] = off; off += sp[lr] * (H / a.hg); }
      ms.poff[v][BB_RG] = off;
    }
  }
  __syncthreads();
  const int Bg = ms.Bg;
  const bool active = Bg > 0;
  const int back = NWL - 1 - wl;
  // tiles
  const int nA = nqkv / 16, nO = d / 16, nS = F / 16, nH = a.CS / 16;
  // out_proj / W2: with several times as many workgroups as tiles the group's rows are split between them, so that
  // a workgroup waits for fewer exchanged words
  int orsplit = 1;
  while (orsplit < BB_RG && 2 * orsplit * nO <= NWL) orsplit *= 2;
  const int out_tile = back % nO, out_part = back / nO;
  const int out_per = BB_RG / orsplit;
  const int out_r0 = out_part * out_per;
  const int out_nr = max(0, min(Bg - out_r0, out_per));
  const bool out_on = active && out_part < orsplit && out_nr > 0;
  // merge role: (local row, head)
  const bool mrg_on = active && back < Bg * H;
  const int mrg_lr = back / H, mrg_h = back % H;
  const uint32_t inv_q2 = 0xFFFFFFFFu / (uint32_t)(nq / 2) + 1u, inv_f2 = 0xFFFFFFFFu / (uint32_t)(F / 2) + 1u;

  // ---- input embedding into the residual stream (every workgroup of the group, redundantly) ----
  if (active) {
    if (a.codes_in) {
      for (int i = tid; i < Bg * a.Q; i += FR_THREADS) {
        const int lr = i / a.Q, q = i - lr * a.Q;
        int64_t cc = a.codes_in[(size_t)ms.grow[lr] * a.Q + q];
        cc = cc < 0 ? 0 : (cc >= a.CS ? a.CS - 1 : cc);
        ms.erow[lr][q] = (int)(cc + (int64_t)q * a.CS);
      }
      __syncthreads();
      const uint32_t* table = (const uint32_t*)W.audio_emb;
      for (int i = tid; i < Bg * (d / 2); i += FR_THREADS) {
        const int lr = i / (d / 2), j = i - lr * (d / 2);
        float s0 = 0.f, s1 = 0.f;
        for (int q0 = 0; q0 < a.Q; q0 += 16) {
          uint32_t r[16];
#pragma unroll
          for (int q = 0; q < 16; ++q) r[q] = table[((size_t)ms.erow[lr][min(q0 + q, a.Q - 1)] * d) / 2 + j];
#pragma unroll
          for (int q = 0; q < 16; ++q) if (q0 + q < a.Q) { s0 += bf_lo(r[q]); s1 += bf_hi(r[q]); }
        }
        const uint32_t pk = f2bf2(s0, s1);
        *reinterpret_cast<float2*>(xres + (size_t)lr * d + 2 * j) = make_float2(bf_lo(pk), bf_hi(pk));
      }
    } else {
      for (int i = tid; i < Bg * (d / 2); i += FR_THREADS) {
        const int lr = i / (d / 2), j = i - lr * (d / 2);
        const uint32_t v = reinterpret_cast<const uint32_t*>(a.emb_in)[(size_t)ms.grow[lr] * (d / 2) + j];
        *reinterpret_cast<float2*>(xres + (size_t)lr * d + 2 * j) = make_float2(bf_lo(v), bf_hi(v));
      }
    }
    __syncthreads();
  }

  auto tile_of = [&](int k, int nT) { BbTile t = {16 * (wl + k * NWL), active && (wl + k * NWL) < nT}; return t; };
  // bytes per weight element of the layers' matrices
  const size_t wsz = I8 ? 1 : 2;
  const size_t layer_elems = (size_t)nqkv * d + (size_t)d * nq + 3 * (size_t)F * d;
  const size_t slab = (size_t)a.n_slots * S * nkv;

#ifdef VUI_BB_CLOCK
  __shared__ unsigned long long dbg_ts[256];
  int dbg_n = 0;
#define BB_TS() do { if (a.dbg && wg == a.dbg_wg && tid == 0 && dbg_n < 255) dbg_ts[dbg_n++] = wall_clock64(); } while (0)
#else
#define BB_TS() do { } while (0)
#endif
  BB_TS();
  uint64_t* llp = a.ll;
  const uint64_t* ybuf = nullptr;  // previous layer's W2 output, still to be added
  for (int l = 0; l < a.L; ++l) {
    const vui_layer_weights& Lw = W.layers[l];
    const char* lw = (const char*)a.tw + layer_elems * wsz * l;
    const void* t_qkv = lw;
    const void* t_o = lw + (size_t)nqkv * d * wsz;
    const void* t_1 = (const char*)t_o + (size_t)d * nq * wsz;
    const void* t_3 = (const char*)t_1 + (size_t)F * d * wsz;
    const void* t_2 = (const char*)t_3 + (size_t)F * d * wsz;
    bf16_t* kcl = a.kc + slab * l;
    bf16_t* vcl = a.vc + slab * l;
    const bool glob = (a.global_layers >> l) & 1ull;
    const int win_l = glob ? 0 : a.window;
    const int plan = (glob || a.window <= 0) ? 1 : 0;
    const float* rope_l = (glob && W.rope_table_global) ? W.rope_table_global : W.rope_table;
    const int rope_dim_l = (glob && W.rope_table_global) ? a.global_rope_dim : a.rope_dim;

    // ---- A: RMSNorm + QKV, rotation, cache append ----
    BB_TS();
    uint64_t* qkvb = llp;
    llp += (size_t)B * (nqkv / 2);
    if (active) {
      BbTile t[NTQ];
      BbW<I8, SD> w[NTQ];
      const BbW<I8, SD> nodual[1] = {};
#pragma unroll
      for (int j = 0; j < NTQ; ++j) { t[j] = tile_of(j, nA); bb_prefetch<I8, SD, EXACT>(t_qkv, d, t[j], w[j]); }
      const BbNorm nw = bb_load_norm((const bf16_t*)Lw.attn_norm, d);
      // what the epilogue of this lane will need (wave j < NTQ: tile j, local row l16, features n .. n + 3): scales,
      // the row's position and its rotation factors, requested now
      int en = 0;
#pragma unroll
      for (int j = 0; j < NTQ; ++j) if (wave == j) en = t[j].n0 + 4 * kg;
      en = min(en, nqkv - 4);
      const int erow_ = min(l16, max(Bg - 1, 0));
      const int epos = ms.gpos[erow_], eslot = ms.gslot[erow_];
      int eregion, em;
      if (en < nq) { eregion = 0; em = en; } else if (en < nq + nkv) { eregion = 1; em = en - nq; } else { eregion = 2; em = en - nq - nkv; }
      const int edd = em % hd;
      const bool erot = eregion != 2 && rope_dim_l >= 4 && edd < rope_dim_l;
      float4 f0 = make_float4(1.f, 0.f, 1.f, 0.f), f1 = f0;
      {
        const float* f = rope_l + ((size_t)epos * max(rope_dim_l, 4) + min(edd, max(rope_dim_l, 4) - 4)) * 2;
        if (rope_dim_l >= 4) { f0 = *reinterpret_cast<const float4*>(f); f1 = *reinterpret_cast<const float4*>(f + 4); }
      }
      uint2 esc = make_uint2(0, 0);
      if (I8) esc = *reinterpret_cast<const uint2*>((const bf16_t*)Lw.s_qkv + en);
      if (ybuf) bb_poll_add_norm_rows(ybuf, ms.off_d, c, xres, nw, a.eps, d, Bg, xp, xs);
      else bb_norm_rows(xres, nw, a.eps, d, Bg, xp, xs);
      __syncthreads();
      bb_compute<I8, SD, NTQ, false, EXACT>(xp, xs, d, t, w, nodual, red, Bg, [&](int, int n, int lr, const float* v, const float*) {
        float o[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = v[r];
        if (I8) { o[0] *= bf_lo(esc.x); o[1] *= bf_hi(esc.x); o[2] *= bf_lo(esc.y); o[3] *= bf_hi(esc.y); }
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = bf2f(f2bf(o[r]));
        if (erot) {  // interleaved pairs (src/vui/rope.py:16-77), products rounded before their sum
          const float r0 = rope_mix(o[0], f0.x, -o[1], f0.y), r1 = rope_mix(o[1], f0.z, o[0], f0.w);
          const float r2 = rope_mix(o[2], f1.x, -o[3], f1.y), r3 = rope_mix(o[3], f1.z, o[2], f1.w);
          o[0] = r0; o[1] = r1; o[2] = r2; o[3] = r3;
        }
        const uint32_t p0 = f2bf2(o[0], o[1]), p1 = f2bf2(o[2], o[3]);
        uint64_t* dst = qkvb + ms.off_q[lr] + n / 2;
        ll_st(dst, p0, ep);
        ll_st(dst + 1, p1, ep);
        if (eregion == 1) *reinterpret_cast<uint2*>(kcl + ((size_t)eslot * S + epos) * nkv + em) = make_uint2(p0, p1);
        if (eregion == 2) *reinterpret_cast<uint2*>(vcl + ((size_t)eslot * S + epos) * nkv + em) = make_uint2(p0, p1);
      });
    }

    // ---- B: attention pieces ----
    BB_TS();
    const int pw_ = hd + 2;                 // words of one head's partial result: max, sum, acc[hd]
    const int HG = a.hg, NHQ = H / HG;      // heads per piece, head sets per row
    uint64_t* part = llp;                   // piece p of group g at (g * NWL + p) * HG * pw_, its head hs at + hs * pw_
    llp += (size_t)nwg * HG * pw_;
    if (active) {
      const int npieces = ms.poff[plan][BB_RG];
      // lane groups of 16: head slot hs = group % HG, key slot ks = group / HG
      const int KP = 16 / HG;  // keys a workgroup takes per step and load round
      const int G = H / a.KV;
      for (int p = wl; p < npieces; p += NWL) {  // uniform over the workgroup; one piece per workgroup as a rule
        int lr = 0;
#pragma unroll
        for (int r = 1; r < BB_RG; ++r) if (p >= ms.poff[plan][r]) lr = r;
        const int rel = p - ms.poff[plan][lr];
        const int sp = rel / NHQ, hq = rel - sp * NHQ;
        const int nsp = ms.spl[plan][lr];
        const int pos = ms.gpos[lr], slot = ms.gslot[lr], len = pos + 1;
        const int start = win_l > 0 ? max(0, len - 1 - win_l) : 0;
        int chunk = (len - start + nsp - 1) / nsp;
        chunk = (chunk + 15) & ~15;
        const int lo = start + sp * chunk, hi = min(lo + chunk, len);
        const bool has_new = pos >= lo && pos < hi;
        const int g = wave * 4 + (lane >> 4);
        const int hs = g & (HG - 1), ks = g / HG;
        const int h = hq * HG + hs;
        const int kvh = h / G, kvh0 = (hq * HG) / G, nkvh = (hq * HG + HG - 1) / G - kvh0 + 1;
        const bool act = l16 * 8 < hd;
        const size_t rowstride = (size_t)nkv;
        const bf16_t* kbase = kcl + ((size_t)slot * S) * rowstride + kvh * hd + (act ? l16 * 8 : 0);
        const bf16_t* vbase = vcl + ((size_t)slot * S) * rowstride + kvh * hd + (act ? l16 * 8 : 0);
        // the first keys and values of this lane group are requested before q is waited for; a key beyond the piece
        // reads the piece's last position instead and gets weight zero below
        uint4 kr[BB_U], vr[BB_U];
#pragma unroll
        for (int u = 0; u < BB_U; ++u) {
          const int j = min(lo + ks + KP * u, hi - 1);  // hi >= 1
          kr[u] = bb_ld16<true>(kbase + (size_t)j * rowstride);
          vr[u] = bb_ld16<true>(vbase + (size_t)j * rowstride);
        }
        uint32_t* qw = (uint32_t*)att;   // q of the piece's heads | new k | new v of their KV heads, packed pairs (<= 1536 words)
        float* gm = att + 1536;          // 16 maxima, 16 sums, 16 weights, 16 head maxima
        float* gacc = att + 1536 + 64;   // 16 x 128
        const int nqw = HG * hd / 2, nkw = nkvh * hd / 2;
        __syncthreads();
        {
          // one wait for everything the piece needs of the row: q of its heads and, where the new position is in the
          // piece, the key and value of their KV heads
          const uint64_t* row = qkvb + ms.off_q[lr];
          const uint64_t* rq_ = row + (hq * HG * hd) / 2;
          const uint64_t* rk_ = row + (nq + kvh0 * hd) / 2 - nqw;
          const uint64_t* rv_ = row + (nq + nkv + kvh0 * hd) / 2 - nqw - nkw;
          const int n = nqw + (has_new ? 2 * nkw : 0);
          for (int base = 0; base < n; base += FR_THREADS * 2) {
            const uint64_t* pp[2];
            int idx[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
              idx[i] = min(base + tid + FR_THREADS * i, n - 1);
              pp[i] = (idx[i] < nqw ? rq_ : (idx[i] < nqw + nkw ? rk_ : rv_)) + idx[i];
            }
            uint64_t v[2];
            int spins = 0;
            while (true) {
#pragma unroll
              for (int i = 0; i < 2; ++i) v[i] = ll_ld(pp[i]);
              const uint32_t bad = ((uint32_t)(v[0] >> 32) ^ ep) | ((uint32_t)(v[1] >> 32) ^ ep);
              if (bad == 0u || c.dead) break;
              if (++spins > SPIN_LIMIT) { c.dead = 1; __hip_atomic_store(c.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
              if (base + tid + FR_THREADS * i < n) qw[idx[i]] = (uint32_t)v[i];
          }
        }
        __syncthreads();
        const float scale = 1.0f / sqrtf((float)hd);
        float q8[8], kn8[8], vn8[8];
        {
          const uint4 z4 = make_uint4(0, 0, 0, 0);
          const uint4 qv = act ? *reinterpret_cast<const uint4*>(qw + (hs * hd + l16 * 8) / 2) : z4;
          cvt8(qv, q8);
          const uint4 kv_ = (act && has_new) ? *reinterpret_cast<const uint4*>(qw + nqw + ((kvh - kvh0) * hd + l16 * 8) / 2) : z4;
          cvt8(kv_, kn8);
          const uint4 vv_ = (act && has_new) ? *reinterpret_cast<const uint4*>(qw + nqw + nkw + ((kvh - kvh0) * hd + l16 * 8) / 2) : z4;
          cvt8(vv_, vn8);
        }
        float m = -INFINITY, lsum = 0.f, acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
        for (int j0 = lo + ks; j0 < hi; j0 += KP * BB_U) {
          // the next step's keys and values go out before this step's arithmetic
          uint4 kn[BB_U], vn[BB_U];
#pragma unroll
          for (int u = 0; u < BB_U; ++u) {
            const int j = min(j0 + KP * BB_U + KP * u, hi - 1);  // past the piece: its last key again, never used
            kn[u] = bb_ld16<true>(kbase + (size_t)j * rowstride);
            vn[u] = bb_ld16<true>(vbase + (size_t)j * rowstride);
          }
          float sc_[BB_U];
          float mn = m;
#pragma unroll
          for (int u = 0; u < BB_U; ++u) {
            const int j = j0 + KP * u;
            float k8[8];
            cvt8(kr[u], k8);
            float dsum = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) dsum = fmaf(q8[e], (j == pos) ? kn8[e] : k8[e], dsum);
            dsum = group16_sum(act ? dsum : 0.f) * scale;
            sc_[u] = j < hi ? dsum : -INFINITY;
            mn = fmaxf(mn, sc_[u]);
          }
          const float r = expf(m - mn);  // 0 on the first step (m = -inf); mn is finite: j0 < hi
          lsum *= r;
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] *= r;
#pragma unroll
          for (int u = 0; u < BB_U; ++u) {
            const int j = j0 + KP * u;
            const float pw = expf(sc_[u] - mn);  // 0 for a key beyond the piece
            lsum += pw;
            float v8[8];
            cvt8(vr[u], v8);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = fmaf(pw, (j == pos) ? vn8[e] : v8[e], acc[e]);
          }
          m = mn;
#pragma unroll
          for (int u = 0; u < BB_U; ++u) { kr[u] = kn[u]; vr[u] = vn[u]; }
        }
        // the key slots of a head -> the head's partial result
        if (l16 == 0) { gm[g] = m; gm[16 + g] = lsum; }
        if (act) {
#pragma unroll
          for (int e = 0; e < 8; ++e) gacc[g * 128 + l16 * 8 + e] = acc[e];
        }
        __syncthreads();
        if (tid < 16) {  // weight of lane group tid inside its head: exp(m - max over the head's key slots)
          const int hs_ = tid & (HG - 1);
          float M = -INFINITY;
          for (int k2 = 0; k2 < KP; ++k2) M = fmaxf(M, gm[hs_ + HG * k2]);
          gm[32 + tid] = (gm[tid] == -INFINITY) ? 0.f : expf(gm[tid] - M);
          gm[48 + tid] = M;
        }
        __syncthreads();
        uint64_t* po = part + ((size_t)grp * NWL + p) * HG * pw_;
        for (int i = tid; i < HG * pw_; i += FR_THREADS) {
          const int hh = i / pw_, j = i - hh * pw_;
          float o;
          if (j == 0) o = gm[48 + hh];
          else if (j == 1) { o = 0.f; for (int k2 = 0; k2 < KP; ++k2) o = fmaf(gm[32 + hh + HG * k2], gm[16 + hh + HG * k2], o); }
          else { o = 0.f; for (int k2 = 0; k2 < KP; ++k2) o = fmaf(gm[32 + hh + HG * k2], gacc[(hh + HG * k2) * 128 + j - 2], o); }
          ll_st(po + i, __float_as_uint(o), ep);
        }
      }
    }

    // ---- C: merge the pieces of (row, head) ----
    BB_TS();
    uint64_t* attb = llp;
    llp += (size_t)B * (nq / 2);
    if (mrg_on) {
      const int nsp = ms.spl[plan][mrg_lr];
      const int mhq = mrg_h / HG, mhs = mrg_h - mhq * HG;
      // key range sp of the head's set is piece poff + sp * NHQ + mhq
      const uint64_t* pb = part + (((size_t)grp * NWL + ms.poff[plan][mrg_lr] + mhq) * HG + mhs) * pw_;
      const size_t pstride = (size_t)NHQ * HG * pw_;
      float* pieces = red;  // nsp x pw_
      const int n = nsp * pw_;
      __syncthreads();
      for (int base = 0; base < n; base += FR_THREADS * 4) {
        const uint64_t* pp[4];
        int idx[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          idx[i] = min(base + tid + FR_THREADS * i, n - 1);
          const int sp = idx[i] / pw_, j = idx[i] - sp * pw_;
          pp[i] = pb + (size_t)sp * pstride + j;
        }
        uint64_t v[4];
        int spins = 0;
        while (true) {
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = ll_ld(pp[i]);
          uint32_t bad = 0;
#pragma unroll
          for (int i = 0; i < 4; ++i) bad |= (uint32_t)(v[i] >> 32) ^ ep;
          if (bad == 0u || c.dead) break;
          if (++spins > SPIN_LIMIT) { c.dead = 1; __hip_atomic_store(c.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (base + tid + FR_THREADS * i < n) pieces[idx[i]] = __uint_as_float((uint32_t)v[i]);
      }
      __syncthreads();
      if (tid < hd) {
        float Mx = -INFINITY;
        for (int s0 = 0; s0 < nsp; ++s0) Mx = fmaxf(Mx, pieces[s0 * pw_]);
        float o = 0.f, Lt = 0.f;
        for (int s0 = 0; s0 < nsp; ++s0) {
          const float m0 = pieces[s0 * pw_];
          const float wgt = (m0 == -INFINITY) ? 0.f : expf(m0 - Mx);
          Lt = fmaf(wgt, pieces[s0 * pw_ + 1], Lt);
          o = fmaf(wgt, pieces[s0 * pw_ + 2 + tid], o);
        }
        const float val = o / Lt;
        const float nb = dpp_f<DPP_QUAD_XOR1>(val);  // the neighbour feature
        if (!(tid & 1)) ll_st(attb + (size_t)ms.grow[mrg_lr] * (nq / 2) + (mrg_h * hd + tid) / 2, f2bf2(val, nb), ep);
      }
    }

    // ---- D: out_proj ----
    BB_TS();
    uint64_t* ob = llp;
    llp += (size_t)B * (d / 2);
    if (out_on) {
      BbTile t[1] = {{16 * out_tile, true}};
      BbW<I8, SD> w[1];
      const BbW<I8, SD> nodual[1] = {};
      bb_prefetch<I8, SD, EXACT>(t_o, nq, t[0], w[0]);
      const int en = t[0].n0 + 4 * kg;
      uint2 esc = make_uint2(0, 0);
      if (I8) esc = *reinterpret_cast<const uint2*>((const bf16_t*)Lw.s_o + en);
      __syncthreads();
      bb_poll_rows(attb, [&](int r) { return (size_t)ms.grow[r] * (nq / 2); }, out_r0, out_nr, nq / 2, inv_q2, c, xp, xs);
      __syncthreads();
      bb_compute<I8, SD, 1, false, EXACT>(xp, xs, nq, t, w, nodual, red, out_nr, [&](int, int n, int lr, const float* v, const float*) {
        float o[4] = {v[0], v[1], v[2], v[3]};
        if (I8) { o[0] *= bf_lo(esc.x); o[1] *= bf_hi(esc.x); o[2] *= bf_lo(esc.y); o[3] *= bf_hi(esc.y); }
        uint64_t* dst = ob + ms.off_d[out_r0 + lr] + n / 2;
        ll_st(dst, f2bf2(o[0], o[1]), ep);
        ll_st(dst + 1, f2bf2(o[2], o[3]), ep);
      });
    }

    // ---- E: residual, RMSNorm, W1/W3, SwiGLU ----
    BB_TS();
    uint64_t* hb = llp;
    llp += (size_t)B * (F / 2);
    if (active) {
      BbTile t[2] = {tile_of(0, nS), tile_of(1, nS)};
      BbW<I8, SD> w[2], w3[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) { bb_prefetch<I8, SD, EXACT>(t_1, d, t[j], w[j]); bb_prefetch<I8, SD, EXACT>(t_3, d, t[j], w3[j]); }
      const BbNorm nw = bb_load_norm((const bf16_t*)Lw.mlp_norm, d);
      int en = 0;
#pragma unroll
      for (int j = 0; j < 2; ++j) if (wave == j) en = t[j].n0 + 4 * kg;
      en = min(en, F - 4);
      uint2 esc = make_uint2(0, 0), esc3 = esc;
      if (I8) { esc = *reinterpret_cast<const uint2*>((const bf16_t*)Lw.s_1 + en); esc3 = *reinterpret_cast<const uint2*>((const bf16_t*)Lw.s_3 + en); }
      bb_poll_add_norm_rows(ob, ms.off_d, c, xres, nw, a.eps, d, Bg, xp, xs);
      __syncthreads();
      bb_compute<I8, SD, 2, true, EXACT>(xp, xs, d, t, w, w3, red, Bg, [&](int, int n, int lr, const float* v, const float* u) {
        float g1[4] = {v[0], v[1], v[2], v[3]}, g3[4] = {u[0], u[1], u[2], u[3]};
        if (I8) {
          g1[0] *= bf_lo(esc.x); g1[1] *= bf_hi(esc.x); g1[2] *= bf_lo(esc.y); g1[3] *= bf_hi(esc.y);
          g3[0] *= bf_lo(esc3.x); g3[1] *= bf_hi(esc3.x); g3[2] *= bf_lo(esc3.y); g3[3] *= bf_hi(esc3.y);
        }
        float hq[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float gq = bf2f(f2bf(g1[q])), up = bf2f(f2bf(g3[q]));
          hq[q] = bf2f(f2bf(gq / (1.0f + expf(-gq)))) * up;
        }
        uint64_t* dst = hb + ms.off_f[lr] + n / 2;
        ll_st(dst, f2bf2(hq[0], hq[1]), ep);
        ll_st(dst + 1, f2bf2(hq[2], hq[3]), ep);
      });
    }

    // ---- F: W2 ----
    BB_TS();
    uint64_t* yb = llp;
    llp += (size_t)B * (d / 2);
    if (out_on) {
      BbTile t[1] = {{16 * out_tile, true}};
      BbW<I8, SF> w[1];
      const BbW<I8, SF> nodual[1] = {};
      bb_prefetch<I8, SF, EXACT>(t_2, F, t[0], w[0]);
      const int en = t[0].n0 + 4 * kg;
      uint2 esc = make_uint2(0, 0);
      if (I8) esc = *reinterpret_cast<const uint2*>((const bf16_t*)Lw.s_2 + en);
      __syncthreads();
      bb_poll_rows(hb, [&](int r) { return (size_t)ms.off_f[r]; }, out_r0, out_nr, F / 2, inv_f2, c, xp, xs);
      __syncthreads();
      bb_compute<I8, SF, 1, false, EXACT>(xp, xs, F, t, w, nodual, red, out_nr, [&](int, int n, int lr, const float* v, const float*) {
        float o[4] = {v[0], v[1], v[2], v[3]};
        if (I8) { o[0] *= bf_lo(esc.x); o[1] *= bf_hi(esc.x); o[2] *= bf_lo(esc.y); o[3] *= bf_hi(esc.y); }
        uint64_t* dst = yb + ms.off_d[out_r0 + lr] + n / 2;
        ll_st(dst, f2bf2(o[0], o[1]), ep);
        ll_st(dst + 1, f2bf2(o[2], o[3]), ep);
      });
    }
    ybuf = yb;
  }

  // ---- final norm, codec head, eos head, hidden output ----
  BB_TS();
  if (active) {
    BbTile t[2] = {tile_of(0, nH), tile_of(1, nH)};
    BbW<false, SD> w[2];
    const BbW<false, SD> nodual[1] = {};
#pragma unroll
    for (int j = 0; j < 2; ++j) bb_prefetch<false, SD, EXACT>(a.thead, d, t[j], w[j]);
    const BbNorm nw = bb_load_norm((const bf16_t*)W.final_norm, d);
    // eos head weights of this lane's pairs (wl < Bg computes row wl's)
    uint32_t eosw[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { const int j = min(lane + WAVE * i, d / 2 - 1); eosw[i] = reinterpret_cast<const uint32_t*>(W.eos_w)[j]; }
    const float eosb = bf2f(*reinterpret_cast<const bf16_t*>(W.eos_b));
    bb_poll_add_norm_rows(ybuf, ms.off_d, c, xres, nw, a.eps, d, Bg, xp, xs);
    __syncthreads();
    if (wl < Bg) {
      const int b = ms.grow[wl];
      const uint32_t* xr = xp + (size_t)wl * xs;
      if (a.hidden_out) for (int j = tid; j < d / 2; j += FR_THREADS) reinterpret_cast<uint32_t*>(a.hidden_out)[(size_t)b * (d / 2) + j] = xr[j];
      if (a.eos_out && wave == 0) {
        float tsum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) { const int j = lane + WAVE * i; if (j < d / 2) tsum = dot2_bf(eosw[i], xr[j], tsum); }
        tsum = wave_sum(tsum);
        if (lane == 0) a.eos_out[b] = f2bf(tsum + eosb);
      }
    }
    bb_compute<false, SD, 2, false, EXACT>(xp, xs, d, t, w, nodual, red, Bg, [&](int, int n, int lr, const float* v, const float*) {
      if (a.cb0_out)
        *reinterpret_cast<uint2*>(a.cb0_out + (size_t)ms.grow[lr] * a.CS + n) = make_uint2(f2bf2(v[0], v[1]), f2bf2(v[2], v[3]));
    });
  }

  // ---- position update and launch handshake by workgroup 0 ----
  __syncthreads();
  BB_TS();
#ifdef VUI_BB_CLOCK
  if (a.dbg && wg == a.dbg_wg && tid == 0) { for (int i = 0; i < dbg_n; ++i) a.dbg[i] = dbg_ts[i]; a.dbg[255] = dbg_n; }
#endif
  if (wg == 0 && tid == 0) {
    // every workgroup has read the positions before it reported its arrival
    int spins = 0;
    bool all = true;
    while (__hip_atomic_load(a.arrive, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (uint32_t)nwg) {
      if (++spins >= SPIN_LIMIT) { __hip_atomic_store(a.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); all = false; break; }
    }
    if (all && !c.dead && !ctl_failed(c)) {
      if (a.seq_inc) { for (int s = 0; s < a.n_slots; ++s) a.seq_lens[s] += a.seq_inc[s]; }
      else { for (int b = 0; b < B; ++b) a.seq_lens[ms.slots[b]] += 1; }
      __hip_atomic_store(a.arrive, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(a.epoch, c.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

int bb_xs(const vui_config& c) {
  int k = c.d_model;
  if (c.ffn > k) k = c.ffn;
  if (c.n_heads * c.head_dim > k) k = c.n_heads * c.head_dim;
  return k / 2 + 4;
}
struct BbLayout { size_t xp, red, att, misc, total; };
BbLayout bb_layout(const vui_config& c) {
  BbLayout l;
  size_t off = (size_t)BB_RG * c.d_model * 4;
  l.xp = off; off += (size_t)(BB_RG + 1) * bb_xs(c) * 4;
  l.red = off; off += 3 * 4 * 64 * 8 * 4;  // three single or two double tiles' partial sums (also: 16 pieces of 130 floats)
  l.att = off; off += (size_t)(1536 + 64 + 2048) * 4;  // the row's q/k/v words, the lane groups' maxima/sums/weights, their accumulators
  l.misc = off; off += (sizeof(BbMisc) + 15) & ~(size_t)15;
  l.total = (off + 15) & ~(size_t)15;
  return l;
}

// row-major int8 (N x K, N % 16 == 0, K % 64 == 0) -> tiled; 16 bytes per thread
__global__ __launch_bounds__(256) void bb_tile8_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, size_t N, int K) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int per_row = K >> 4;
  if (i >= N * per_row) return;
  const size_t n = i / per_row;
  const int k = (int)(i % per_row) * 16;
  const size_t o = ((n >> 4) * (size_t)(K >> 6) + (k >> 6)) * 1024 + (size_t)((n & 15) + 16 * ((k & 63) >> 4)) * 16;
  *reinterpret_cast<uint4*>(dst + o) = *reinterpret_cast<const uint4*>(src + n * K + k);
}
// row-major bf16 -> the 16 x 64 block layout (the prompt-ingestion GEMMs' operand layout); 8 elements per thread
__global__ __launch_bounds__(256) void bb_tile16_kernel(const bf16_t* __restrict__ src, bf16_t* __restrict__ dst, size_t N, int K) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int per_row = K >> 3;
  if (i >= N * per_row) return;
  const size_t n = i / per_row;
  const int k = (int)(i % per_row) * 8;
  const size_t o = ((n >> 4) * (size_t)(K >> 6) + (k >> 6)) * 1024 + (size_t)(((k & 15) >> 3) * 512 + (((k & 63) >> 4) * 16 + (n & 15)) * 8);
  *reinterpret_cast<uint4*>(dst + o) = *reinterpret_cast<const uint4*>(src + n * K + k);
}

}  // namespace

// ---------------------------------------------------------------------------------------------
bool bb_batch_supported(const vui_config& c, int nwg, char* why, size_t why_len) {
  const char* r = nullptr;
  const int nq = c.n_heads * c.head_dim, nkv = c.n_kv_heads * c.head_dim;
  if (c.dtype != VUI_DTYPE_BF16) r = "bf16 activations only";
  else if ((c.d_model % 64) || (c.ffn % 64) || (nq % 64)) r = "d_model, heads x head_dim and ffn must be multiples of 64";
  else if (c.d_model > 1024 || c.ffn > 2048 || nq > 1024) r = "vector longer than the register tile";
  else if ((nq % 16) || (nkv % 16) || (c.head_dim % 8) || c.head_dim > 128) r = "head layout";
  else if ((c.rope_dim % 4) || (c.global_rope_dim % 4)) r = "rotated features must come in fours";
  else if ((c.codebook_size % 16) || c.codebook_size > 2 * 16 * 64) r = "codebook_size must be a multiple of 16, at most 2048";
  else if (c.n_quantizers > 64) r = "too many codebooks";
  else if (nwg != 256) r = "needs 256 resident workgroups";
  else {
    const int NWL = 64;  // the smallest group
    if ((nq + 2 * nkv) / 16 > 3 * NWL || c.ffn / 16 > 2 * NWL || c.d_model / 16 > NWL || BB_RG * c.n_heads > NWL || c.n_heads > 16) r = "more tiles or heads than a row group's workgroups take";
    if (nq + 2 * nkv > 3072) r = "q, k and v of a row longer than the attention staging area";
    if ((size_t)c.ffn / 2 * BB_RG >= 65536) r = "exchange vector too long";
    if (bb_layout(c).total > 160 * 1024) r = "activations do not fit in LDS";
  }
  if (r && why) snprintf(why, why_len, "%s", r);
  return r == nullptr;
}

size_t bb_batch_ll_words(const vui_config& c, int nwg) {
  const size_t B = VUI_MAX_BATCH, nq = (size_t)c.n_heads * c.head_dim, nkv = (size_t)c.n_kv_heads * c.head_dim;
  const size_t layer = B * ((nq + 2 * nkv) / 2 + nq / 2 + c.d_model / 2 + c.ffn / 2 + c.d_model / 2) + (size_t)nwg * 8 * (c.head_dim + 2);  // a piece holds at most 8 heads' partial results
  return layer * c.n_layers + 64;
}
size_t bb_batch_lds_bytes(const vui_config& c) { return bb_layout(c).total; }

// bytes of this kernel's own tiled copy of the layers' matrices: the int8 matrices of an int8 context, the bf16
// matrices where the prompt-ingestion pass (whose copy is used otherwise) does not take the configuration; and of the
// tiled codec head
size_t bb_batch_weight_bytes(const vui_config& c, int nwg) {
  if (!bb_batch_supported(c, nwg, nullptr, 0)) return 0;
  if (!c.int8_backbone && prefill_weight_bytes(c)) return 0;
  const size_t nq = (size_t)c.n_heads * c.head_dim, nkv = (size_t)c.n_kv_heads * c.head_dim, d = c.d_model, F = c.ffn;
  return ((nq + 2 * nkv) * d + d * nq + 3 * F * d) * c.n_layers * (c.int8_backbone ? 1 : 2);
}
size_t bb_batch_head_bytes(const vui_config& c, int nwg) {
  return bb_batch_supported(c, nwg, nullptr, 0) ? (size_t)c.codebook_size * c.d_model * 2 : 0;
}

int bb_batch_tile_weights(const vui_config& c, const vui_weights& w, void* dst_layers, void* dst_head, hipStream_t st) {
  const size_t nq = (size_t)c.n_heads * c.head_dim, nkv = (size_t)c.n_kv_heads * c.head_dim, d = c.d_model, F = c.ffn;
  if (dst_layers) {
    const bool i8 = c.int8_backbone != 0;
    char* o = (char*)dst_layers;
    auto tile = [&](const void* src, size_t N, size_t K) {
      if (i8) {
        const size_t pieces = N * (K / 16);
        hipLaunchKernelGGL(bb_tile8_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, (const uint8_t*)src, (uint8_t*)o, N, (int)K);
      } else {
        const size_t pieces = N * (K / 8);
        hipLaunchKernelGGL(bb_tile16_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, (const bf16_t*)src, (bf16_t*)o, N, (int)K);
      }
      o += N * K * (i8 ? 1 : 2);
    };
    for (int l = 0; l < c.n_layers; ++l) {
      const vui_layer_weights& L = w.layers[l];
      tile(L.wqkv, nq + 2 * nkv, d);
      tile(L.wo, d, nq);
      tile(L.w1, F, d);
      tile(L.w3, F, d);
      tile(L.w2, d, F);
    }
  }
  if (dst_head) {
    const size_t pieces = (size_t)c.codebook_size * (d / 8);
    hipLaunchKernelGGL(bb_tile16_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, (const bf16_t*)w.codec_head, (bf16_t*)dst_head,
                       (size_t)c.codebook_size, (int)d);
  }
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

// the kernel's instantiations: Vui Nano's shape (768 wide, ffn 2048) with nothing conditional, and the general one
static bool bb_exact(const vui_config& c) { return c.d_model == 768 && c.n_heads * c.head_dim == 768 && c.ffn == 2048; }
typedef void (*bb_kernel_t)(const BbArgs);
static bb_kernel_t bb_pick(const vui_config& c) {
  if (bb_exact(c)) return c.int8_backbone ? bb_batch_kernel<true, 3, 3, 8, true> : bb_batch_kernel<false, 3, 3, 8, true>;
  return c.int8_backbone ? bb_batch_kernel<true, 3, 4, 8, false> : bb_batch_kernel<false, 3, 4, 8, false>;
}

int bb_batch_max_resident(const vui_config& c) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, dev));
  const size_t lds = bb_layout(c).total;
  const bb_kernel_t k = bb_pick(c);
  HIP_TRY(hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  int occ = 0;
  HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, k, FR_THREADS, lds));
  return occ * prop.multiProcessorCount;
}

#ifdef VUI_BB_CLOCK
// profiling builds only: where the next launches drop the phase stamps of workgroup wg
static unsigned long long* g_bb_dbg = nullptr;
static int g_bb_dbg_wg = 0;
extern "C" void vui_debug_bb_batch_clock(unsigned long long* buf, int wg) { g_bb_dbg = buf; g_bb_dbg_wg = wg; }
#endif

int launch_bb_batch(const vui_config& c, const vui_weights* wdev, const void* tiled_layers, const void* tiled_head, const int64_t* codes_in,
                    const void* emb_in, const int32_t* slot_idx, int32_t* seq_lens, const int32_t* seq_inc, int B, void* k_cache,
                    void* v_cache, void* hidden_out, void* cb0_out, void* eos_out, uint64_t* ll, uint32_t* ctl, int nwg, hipStream_t st) {
  if (B < 2 || B > VUI_MAX_BATCH) { vui_set_error("batched backbone kernel: B=%d outside [2,%d]", B, VUI_MAX_BATCH); return VUI_EINVAL; }
  BbArgs a;
  memset(&a, 0, sizeof(a));
  a.B = B; a.d = c.d_model; a.L = c.n_layers; a.H = c.n_heads; a.KV = c.n_kv_heads; a.hd = c.head_dim; a.F = c.ffn; a.Q = c.n_quantizers;
  a.CS = c.codebook_size; a.S = c.max_seqlen; a.n_slots = c.n_slots; a.window = c.window; a.rope_dim = c.rope_dim;
  a.global_rope_dim = c.global_rope_dim; a.global_layers = c.global_layers; a.eps = c.norm_eps;
  a.w = wdev; a.tw = tiled_layers; a.thead = (const bf16_t*)tiled_head;
  a.codes_in = codes_in; a.emb_in = (const uint16_t*)emb_in; a.slot_idx = slot_idx; a.seq_lens = seq_lens; a.seq_inc = seq_inc;
  a.kc = (uint16_t*)k_cache; a.vc = (uint16_t*)v_cache; a.hidden_out = (uint16_t*)hidden_out; a.cb0_out = (uint16_t*)cb0_out;
  a.eos_out = (uint16_t*)eos_out; a.ll = ll; a.epoch = ctl; a.arrive = ctl + 1; a.err = ctl + 2;
  const BbLayout l = bb_layout(c);
#ifdef VUI_BB_CLOCK
  a.dbg = g_bb_dbg; a.dbg_wg = g_bb_dbg_wg;
#endif
  // heads per attention piece: two from nine rows on (a group of 64 workgroups then holds three or four rows, and
  // pairs of heads divide their keys twice as finely as whole head sets per key range would; measured for the frame
  // step of 16 rows 1716 against 1728 us, of 8 rows - two rows per group - 1554 against 1548, four heads per piece
  // 1765 / 1588); a key range is not split below 64 keys (32..128 measure the same)
  a.hg = (B > 2 * BB_RG && c.n_heads % 2 == 0) ? 2 : 1;
  a.min_keys = 64;
  a.xs = bb_xs(c); a.off_xp = (int)l.xp; a.off_red = (int)l.red; a.off_att = (int)l.att; a.off_misc = (int)l.misc;
  hipLaunchKernelGGL(bb_pick(c), dim3(nwg), dim3(FR_THREADS), l.total, st, a);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}
