// Prompt ingestion: T > 1 new positions of one row through the backbone in one pass per layer.
//
//   Decoder.forward_flash / Engine._prefill_emb with T > 1  (src/vui/model.py:534-549, engine.py:674-694)
//
// bf16 activations; the layers' matrices bf16, or int8 with per-row scales (widened in registers inside the GEMMs,
// the scale on the finished sum).  Per layer: row RMSNorm, QKV GEMM, one kernel that rotates the new keys, appends keys and values to the
// cache and stages the slot's keys / transposed values in operand layout, causal attention of the new positions
// against them (the same kernel rotates the queries in place; scores never leave the registers; probabilities
// rounded to bf16 before they meet the values), out_proj GEMM with the residual add in its epilogue, row RMSNorm, one GEMM over
// W1 and W3 with the SwiGLU product in its epilogue, W2 GEMM with residual: eight launches.
// Every GEMM is C (M x N) = X (M x K) W^T (N x K) on the matrix cores, both operands in the tiled layout below.
//
// Rounding points are those of the single-position step (one rounding after each linear, two in
// the norm, products of the rotation rounded before their sum, residual sums rounded).
#include "common.h"
#include "internal.h"
#include <stdio.h>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 pf_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float pf_floatx4;
union PfU128 { uint4 u; pf_bf16x8 v; };
__device__ __forceinline__ pf_bf16x8 pf_frag(const uint4& x) { PfU128 t; t.u = x; return t.v; }

enum { PF_BF16 = 0, PF_RESID = 1 };

// Operand layout of the GEMMs ("tiled"): a matrix of R rows x K columns (K a multiple of 64, rows padded to 16) is
// cut into blocks of 16 rows x 64 columns, block (r / 16, k / 64) at element offset ((r / 16) * (K / 64) + k / 64)
// * 1024, and inside a block the 8-element piece p = (k % 16) / 8 of lane (r % 16) + 16 * ((k % 64) / 16) sits at
// p * 512 + lane * 8.  A wave then fetches the operand fragment of a 16 x 64 block with two loads of 1 KiB
// contiguous each (lane l: 16 bytes at 16 l), where the row-major form makes the 16 lanes of a quarter-wave read
// 16 different lines - which the address unit serves at about a quarter of the rate (measured on this machine
// from an L2-sized buffer: 9.6 TB/s over the chip for 16 rows x 64 bytes per instruction, 31 TB/s for 1 KiB
// contiguous).  Weights are brought into this form once per context, activations are written in it by their
// producers.
__host__ __device__ __forceinline__ size_t pf_toff(int r, int k, int K) {
  return ((size_t)(r >> 4) * (K >> 6) + (k >> 6)) * 1024 + (size_t)(((k & 15) >> 3) * 512 + (((k & 63) >> 4) * 16 + (r & 15)) * 8 + (k & 7));
}

struct PfGemm {
  const bf16_t* X;   // activations (M x K), tiled
  const void* W;     // weights (N x K), tiled: bf16, or int8 (the byte form of the layout: block (r / 16, k / 64) at
                     // ((r / 16) * (K / 64) + k / 64) * 1024 bytes, the 16 bytes k % 16 = 0..15 of lane (r % 16) + 16 * ((k % 64) / 16)
                     // at 16 * lane) with the per-row scales sc (and sc2 for the second matrix of a SwiGLU pair)
  const bf16_t *sc, *sc2;
  void* C;           // output (M x N) bf16: row-major with row stride ldc (PF_RESID: in place on the residual), or tiled
  int M, N, K, ldc;
};

// row-major (N x K) -> tiled; one 8-element piece per thread
__global__ __launch_bounds__(256) void pf_tile_kernel(const bf16_t* __restrict__ src, bf16_t* __restrict__ dst, int N, int K) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int per_row = K >> 3;
  if (i >= (size_t)N * per_row) return;
  const int n = (int)(i / per_row), k = (int)(i % per_row) * 8;
  *reinterpret_cast<uint4*>(dst + pf_toff(n, k, K)) = *reinterpret_cast<const uint4*>(src + (size_t)n * K + k);
}

// C = X W^T for the projections (K = d_model ... ffn; 64 x 64 tiles would give only 9 x 12 ... 9 x 64
// workgroups at 576 positions, each a long serial walk over K): a workgroup owns 32 rows x 32 features and its four waves split
// the K steps between them, so a wave's chain of dependent trips to memory is a quarter as long and four times as
// many workgroups are in flight.  The four partial tiles meet in LDS and are added in wave order (a fixed order:
// results do not depend on timing).
// DUAL: two weight matrices against the same activations, h = rnd(rnd(silu(rnd(a))) * rnd(c)) written once
// (SwiGLU, src/vui/model.py:282) instead of two products and a pass over both.
// eight int8 -> four packed bf16 pairs, exact
__device__ __forceinline__ uint4 pf_widen8(uint32_t lo, uint32_t hi) {
  uint4 r;
  r.x = f2bf2((float)(int8_t)(lo & 0xff), (float)(int8_t)((lo >> 8) & 0xff));
  r.y = f2bf2((float)(int8_t)((lo >> 16) & 0xff), (float)(int8_t)(lo >> 24));
  r.z = f2bf2((float)(int8_t)(hi & 0xff), (float)(int8_t)((hi >> 8) & 0xff));
  r.w = f2bf2((float)(int8_t)((hi >> 16) & 0xff), (float)(int8_t)(hi >> 24));
  return r;
}

template <int EPI, bool DUAL, bool I8>
__global__ __launch_bounds__(256) void pf_gemm4_kernel(const PfGemm p, const void* __restrict__ W2, int c_tiled) {
  constexpr int TILE = 1024;  // floats of one partial tile
  constexpr int PW = (DUAL ? 2 : 1) * TILE;
  __shared__ float part[4 * PW];
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int l16 = lane & 15, kg = lane >> 4;
  const int MT = (p.M + 31) >> 5;
  const int id = blockIdx.x;
  const int m0 = (id % MT) * 32, n0 = (id / MT) * 32;
  // A step covers 64 values of k, one block of the tiled operands per 16 rows: the lane's 16-byte piece of half h
  // (k = 64 s + 16 kg + 8 h ...; any assignment of k to lanes is valid as long as both operands share it) is at
  // block + 512 h + 8 lane.
  const int nsteps = p.K >> 6;
  const int s0 = nsteps * wave / 4, s1 = nsteps * (wave + 1) / 4;
  const int MB = (p.M + 15) >> 4, NB = (p.N + 15) >> 4;  // 16-row blocks; a tile past the end reads the last block again
  const bf16_t* xr[2];
  const char* wr[2];  // byte addresses: a block is 2048 bytes of bf16 (two 16-byte pieces per lane) or 1024 of int8 (one)
  const char* vr[2];
  constexpr int WB = I8 ? 1024 : 2048, WL = 16;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    xr[j] = p.X + (size_t)min((m0 >> 4) + j, MB - 1) * nsteps * 1024 + lane * 8;
    const size_t wo = (size_t)min((n0 >> 4) + j, NB - 1) * nsteps * WB + lane * WL;
    wr[j] = (const char*)p.W + wo;
    vr[j] = DUAL ? (const char*)W2 + wo : (const char*)p.W + wo;
  }
  pf_floatx4 acc[2][2], acc2[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) { acc[i][j] = pf_floatx4{0.f, 0.f, 0.f, 0.f}; acc2[i][j] = acc[i][j]; }
  // the residual values this thread will add to (its four outputs, see the epilogue) are requested with the first
  // operands instead of after the last product; clamped to the matrix, unused where the thread has no output
  uint2 old = make_uint2(0, 0);
  if (EPI == PF_RESID) {
    const int em = min(m0 + 16 * (wave & 1) + l16, p.M - 1), en = min(n0 + 16 * (wave >> 1) + 4 * kg, p.N - 4);
    old = *reinterpret_cast<const uint2*>((const bf16_t*)p.C + (c_tiled ? pf_toff(em, en, p.N) : (size_t)em * p.ldc + en));
  }
  for (int s = s0; s < s1; ++s) {
    const int k = s << 10;
    uint4 xa[2][2], wa[2][2], va[2][2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < 2; ++j) xa[j][h] = *reinterpret_cast<const uint4*>(xr[j] + k + 512 * h);
    if (I8) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const uint4 w8 = *reinterpret_cast<const uint4*>(wr[j] + (size_t)s * WB);
        wa[j][0] = pf_widen8(w8.x, w8.y); wa[j][1] = pf_widen8(w8.z, w8.w);
        if (DUAL) {
          const uint4 v8 = *reinterpret_cast<const uint4*>(vr[j] + (size_t)s * WB);
          va[j][0] = pf_widen8(v8.x, v8.y); va[j][1] = pf_widen8(v8.z, v8.w);
        }
      }
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          wa[j][h] = *reinterpret_cast<const uint4*>(wr[j] + (size_t)s * WB + 1024 * h);
          if (DUAL) va[j][h] = *reinterpret_cast<const uint4*>(vr[j] + (size_t)s * WB + 1024 * h);
        }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf_frag(wa[i][h]), pf_frag(xa[j][h]), acc[i][j], 0, 0, 0);
          if (DUAL) acc2[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf_frag(va[i][h]), pf_frag(xa[j][h]), acc2[i][j], 0, 0, 0);
        }
  }
  // partial tiles to LDS: [wave][(i, j)][lane] as float4
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      *reinterpret_cast<pf_floatx4*>(&part[wave * PW + ((i * 2 + j) * 64 + lane) * 4]) = acc[i][j];
      if (DUAL) *reinterpret_cast<pf_floatx4*>(&part[wave * PW + TILE + ((i * 2 + j) * 64 + lane) * 4]) = acc2[i][j];
    }
  __syncthreads();
  // thread: sub-tile (i, j) = its wave's two bits, features n0 + 16 i + 4 kg + r (r = 0..3) of row m0 + 16 j + l16
  const int i = wave >> 1, j = wave & 1;
  const int m = m0 + 16 * j + l16, n = n0 + 16 * i + 4 * kg;
  float v[4], u[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int e = tid * 4 + r;
    v[r] = ((part[e] + part[PW + e]) + part[2 * PW + e]) + part[3 * PW + e];
    if (DUAL) u[r] = ((part[TILE + e] + part[PW + TILE + e]) + part[2 * PW + TILE + e]) + part[3 * PW + TILE + e];
  }
  if (m >= p.M || n >= p.N) return;
  if (I8) {  // y[n] = scale[n] * sum_k q[n, k] x[k]
    for (int r = 0; r < 4; ++r)
      if (n + r < p.N) { v[r] *= bf2f(p.sc[n + r]); if (DUAL) u[r] *= bf2f(p.sc2[n + r]); }
  }
  bf16_t* c = (bf16_t*)p.C + (c_tiled ? pf_toff(m, n, p.N) : (size_t)m * p.ldc + n);  // n % 4 == 0: inside one piece
  if (DUAL) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float a = bf2f(f2bf(v[r])), b = bf2f(f2bf(u[r]));
      v[r] = bf2f(f2bf(a / (1.0f + expf(-a)))) * b;
    }
  }
  if (EPI == PF_RESID) {  // x = rnd(x + rnd(y)), src/vui/model.py:367, 374
    if (n + 3 < p.N) {
      v[0] = bf_lo(old.x) + bf2f(f2bf(v[0])); v[1] = bf_hi(old.x) + bf2f(f2bf(v[1]));
      v[2] = bf_lo(old.y) + bf2f(f2bf(v[2])); v[3] = bf_hi(old.y) + bf2f(f2bf(v[3]));
    } else {
      for (int r = 0; r < 4; ++r) if (n + r < p.N) v[r] = bf2f(c[r]) + bf2f(f2bf(v[r]));
    }
  }
  if (n + 3 < p.N) *reinterpret_cast<uint2*>(c) = make_uint2(f2bf2(v[0], v[1]), f2bf2(v[2], v[3]));
  else for (int r = 0; r < 4; ++r) if (n + r < p.N) c[r] = f2bf(v[r]);
}

// two-rounding RMSNorm of rows (src/vui/model.py:286-297); one wave per row
__global__ __launch_bounds__(256) void pf_rownorm_kernel(const bf16_t* x, const bf16_t* w, bf16_t* y, int M, int K, float eps, int y_tiled) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= M) return;
  const bf16_t* xr = x + (size_t)row * K;
  float ss = 0.f;
  for (int c = lane; c < K / 8; c += WAVE) {
    float v[8];
    El<bf16_t>::ld8(xr + c * 8, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf(v[e], v[e], ss);
  }
  ss = wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)K + eps);
  for (int c = lane; c < K / 8; c += WAVE) {
    float v[8], g[8], o[8];
    El<bf16_t>::ld8(xr + c * 8, v);
    El<bf16_t>::ld8(w + c * 8, g);
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = bf2f(f2bf(v[e] * r)) * g[e];
    El<bf16_t>::st8(y + (y_tiled ? pf_toff(row, c * 8, K) : (size_t)row * K + c * 8), o);
  }
}

// interleaved rotation (src/vui/rope.py:16-77) of the four pairs of an 8-element piece whose first dim is dd (even)
// at position pos; pairs at or beyond rope_dim pass through
__device__ __forceinline__ uint4 pf_rope8(uint4 v, const float* __restrict__ rope, int pos, int rope_dim, int dd) {
  if (rope_dim < 2) return v;  // uniform
  uint32_t w[4] = {v.x, v.y, v.z, v.w};
  // the four factor loads go out together (a pair beyond rope_dim reads the last rotated pair's and ignores it):
  // behind a branch each, every load would be waited for before the next is issued
  float4 f[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) f[i] = *reinterpret_cast<const float4*>(rope + ((size_t)pos * rope_dim + min(dd + 2 * i, rope_dim - 2)) * 2);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float a = bf_lo(w[i]), b = bf_hi(w[i]);  // cos, sin of d2 and d2 + 1
    const uint32_t r = f2bf2(rope_mix(a, f[i].x, -b, f[i].y), rope_mix(b, f[i].z, a, f[i].w));
    w[i] = (dd + 2 * i < rope_dim) ? r : w[i];
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// Attention of the new positions against the row's cache without materialised scores: one workgroup per
// (16 queries, head), its waves (eight, four for head_dim 128) take 32 keys at a time in turn with a running maximum and sum each and
// meet in LDS at the end.  Per step: scores^T (keys x queries) = K q^T on the matrix cores, so that a lane holds
// eight keys of ONE query (its column) and the softmax bookkeeping is per lane plus a fold over the four lane
// rows; the probabilities, rounded to bf16, are then already in operand layout for out^T (dims x queries) =
// V^T p^T, with V^T read from the transposed copy in the same key order (any assignment of k to lanes is valid
// when both operands share it).  HD32 = head_dim / 32.
#define PF_ATT_WAVES (HD32 <= 3 ? 8 : 4)  // the partial outputs of the waves must fit 64 KiB of LDS
template <int HD32>
__global__ __launch_bounds__(64 * PF_ATT_WAVES) void pf_attn_kernel(const bf16_t* __restrict__ qkv, const bf16_t* __restrict__ kt,
                                                      const bf16_t* __restrict__ vt, bf16_t* __restrict__ att, int T, int L,
                                                      int Lpad, int nq, int nkv, int gsz, int pos0, int window, float scale) {
  constexpr int HD = 32 * HD32, DT = 2 * HD32;
  __shared__ float s_acc[PF_ATT_WAVES][DT * 256];
  __shared__ float s_m[PF_ATT_WAVES][16], s_l[PF_ATT_WAVES][16];
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int l16 = lane & 15, kg = lane >> 4;
  const int q0 = blockIdx.x * 16, h = blockIdx.y, kvh = h / gsz;
  const int ldq = nq + 2 * nkv;
  // this lane's query (column of every product below)
  const int tq = min(q0 + l16, T - 1);
  const int qlast = pos0 + tq;                                   // last visible key
  const int qfirst = window > 0 ? max(0, qlast - window) : 0;   // first visible key
  uint4 qf[HD32];
#pragma unroll
  for (int c = 0; c < HD32; ++c)
    qf[c] = *reinterpret_cast<const uint4*>(qkv + (size_t)tq * ldq + h * HD + c * 32 + kg * 8);
  // keys any query of the tile can see
  const int t_hi = min(q0 + 15, T - 1);
  const int kend = pos0 + t_hi + 1;
  const int kbeg = (window > 0 ? max(0, pos0 + q0 - window) : 0) & ~31;
  // staged keys / values of this KV head (pf_stage_kv_kernel): a fragment is 16 bytes per lane, 1 KiB contiguous per wave
  const bf16_t* kb = kt + (size_t)kvh * (Lpad >> 4) * HD32 * 512 + lane * 8;
  const bf16_t* vb = vt + (size_t)kvh * DT * (Lpad >> 5) * 512 + lane * 8;

  pf_floatx4 acc[DT];
#pragma unroll
  for (int d = 0; d < DT; ++d) acc[d] = pf_floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;
  for (int k0 = kbeg + 32 * wave; k0 < kend; k0 += 32 * PF_ATT_WAVES) {
    // every load of the step goes out before the first product (keys and values alike: the values do not depend
    // on the scores), so a step is one trip to memory
    uint4 kf[2][HD32], vf[DT];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int c = 0; c < HD32; ++c)
        kf[kt][c] = *reinterpret_cast<const uint4*>(kb + ((size_t)((k0 >> 4) + kt) * HD32 + c) * 512);
    // V^T of dims 16 d + l16: the lane's eight keys k0 + 4 kg + r and k0 + 16 + 4 kg + r, in the order of its scores
#pragma unroll
    for (int d = 0; d < DT; ++d) vf[d] = *reinterpret_cast<const uint4*>(vb + ((size_t)d * (Lpad >> 5) + (k0 >> 5)) * 512);
    __builtin_amdgcn_sched_barrier(0);
    // scores^T of 32 keys: two tiles of 16 keys x 16 queries
    pf_floatx4 sc[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      sc[kt] = pf_floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < HD32; ++c)
        sc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf_frag(kf[kt][c]), pf_frag(qf[c]), sc[kt], 0, 0, 0);
    }
    // the lane holds keys k0 + 16 kt + 4 kg + r of its query
    float sv[8], mx = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = k0 + 16 * kt + 4 * kg + r;
        const float v = (j >= qfirst && j <= qlast) ? sc[kt][r] * scale : -INFINITY;
        sv[4 * kt + r] = v;
        mx = fmaxf(mx, v);
      }
    mx = rows_max(mx);  // over the four lane rows: every key of the step for this query
    const float m_new = fmaxf(m_run, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // nothing visible yet: every weight below is zero
    const float alpha = expf(m_run - m_use);                  // 0 on the first visible step (m_run = -inf)
    float pv[8], ps = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { pv[e] = expf(sv[e] - m_use); ps += pv[e]; }
    l_run = l_run * alpha + ps;
    m_run = m_new;
    uint4 pf;
    pf.x = f2bf2(pv[0], pv[1]); pf.y = f2bf2(pv[2], pv[3]); pf.z = f2bf2(pv[4], pv[5]); pf.w = f2bf2(pv[6], pv[7]);
#pragma unroll
    for (int d = 0; d < DT; ++d) {
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[d][r] *= alpha;
      acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf_frag(vf[d]), pf_frag(pf), acc[d], 0, 0, 0);
    }
  }
  // the waves' parts meet: lane holds dims 16 d + 4 kg + r of query l16
  l_run = rows_sum(l_run);
  if (kg == 0) { s_m[wave][l16] = m_run; s_l[wave][l16] = l_run; }
#pragma unroll
  for (int d = 0; d < DT; ++d) *reinterpret_cast<pf_floatx4*>(&s_acc[wave][(d * 64 + lane) * 4]) = acc[d];
  __syncthreads();
  for (int sl = tid; sl < DT * 64; sl += 64 * PF_ATT_WAVES) {
    const int d = sl >> 6, ln = sl & 63, q = ln & 15, g4 = ln >> 4;
    const int t = q0 + q;
    if (t >= T) continue;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < PF_ATT_WAVES; ++w) M = fmaxf(M, s_m[w][q]);
    float den = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < PF_ATT_WAVES; ++w) {
      const float f = (s_m[w][q] == -INFINITY) ? 0.f : expf(s_m[w][q] - M);
      den = fmaf(f, s_l[w][q], den);
#pragma unroll
      for (int r = 0; r < 4; ++r) o[r] = fmaf(f, s_acc[w][sl * 4 + r], o[r]);
    }
    const float inv = 1.0f / den;
    bf16_t* dst = att + pf_toff(t, h * HD + 16 * d + 4 * g4, nq);  // tiled: operand of out_proj
    *reinterpret_cast<uint2*>(dst) = make_uint2(f2bf2(o[0] * inv, o[1] * inv), f2bf2(o[2] * inv, o[3] * inv));
  }
}

// Keys and values of one row's cache slab in the operand layouts of pf_attn_kernel, zero beyond position L; the new
// positions pos0 .. L - 1 are taken from the projection output, the keys rotated (src/vui/model.py:234-247), and
// appended to the cache on the way.
// Keys of KV head g: blocks of 16 keys x 32 dims, block ((g * Lpad / 16 + j / 16) * hd / 32 + dim / 32) of 512
// elements, lane (j % 16) + 16 * ((dim % 32) / 8) holds its 8 dims at 8 * lane.  Values, transposed: blocks of 16
// dims x 32 keys, block ((g * hd / 16 + dim / 16) * Lpad / 32 + j / 32), lane (dim % 16) + 16 * ((j % 16) / 4)
// holds keys j % 4 of both halves (j % 32) / 16 of the step at 8 * lane + 4 * half + j % 4 - the order in which a
// lane of the attention kernel holds the scores of a step.  One workgroup: 32 keys x 32 features.
__global__ __launch_bounds__(256) void pf_stage_kv_kernel(bf16_t* __restrict__ qkv, bf16_t* __restrict__ kc, bf16_t* __restrict__ vc,
                                                          bf16_t* __restrict__ kt, bf16_t* __restrict__ vt, const float* __restrict__ rope,
                                                          int L, int Lpad, int nq, int nkv, int hd, int rope_dim, int pos0) {
  __shared__ bf16_t tile[32][34];
  const int tid = threadIdx.x;
  const int ldq = nq + 2 * nkv;
  if ((int)blockIdx.y >= nkv / 32) {
    // the other workgroups rotate the queries in place: 32 rows x 32 dims each
    const int t = blockIdx.x * 32 + (tid >> 2), f = ((int)blockIdx.y - nkv / 32) * 32 + (tid & 3) * 8;
    if (tid < 128 && t < L - pos0) {
      uint4* q = reinterpret_cast<uint4*>(qkv + (size_t)t * ldq + f);
      *q = pf_rope8(*q, rope, pos0 + t, rope_dim, f % hd);
    }
    return;
  }
  const int j0 = blockIdx.x * 32, f0 = blockIdx.y * 32;  // f over nkv (= KV * hd); hd is a multiple of 32
  const int g = f0 / hd, dim0 = f0 % hd;
  if (tid < 128) {  // keys: 32 keys x four 8-dim pieces
    const int key = tid >> 2, pc = tid & 3, j = j0 + key;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (j < pos0) v = *reinterpret_cast<const uint4*>(kc + (size_t)j * nkv + f0 + pc * 8);
    else if (j < L) {
      v = pf_rope8(*reinterpret_cast<const uint4*>(qkv + (size_t)(j - pos0) * ldq + nq + f0 + pc * 8), rope, j, rope_dim, dim0 + pc * 8);
      *reinterpret_cast<uint4*>(kc + (size_t)j * nkv + f0 + pc * 8) = v;
    }
    const size_t blk = ((size_t)g * (Lpad >> 4) + (j >> 4)) * (hd >> 5) + (dim0 >> 5);
    *reinterpret_cast<uint4*>(kt + blk * 512 + ((j & 15) + 16 * pc) * 8) = v;
  }
  {
    const int tx = tid & 31, ty = tid >> 5;  // 32 x 8
    for (int r = ty; r < 32; r += 8) {
      const int j = j0 + r;
      bf16_t v = (bf16_t)0;
      if (j < pos0) v = vc[(size_t)j * nkv + f0 + tx];
      else if (j < L) { v = qkv[(size_t)(j - pos0) * ldq + nq + nkv + f0 + tx]; vc[(size_t)j * nkv + f0 + tx] = v; }
      tile[r][tx] = v;
    }
  }
  __syncthreads();
  {
    // thread: dim dl of the 32, piece q = 4 * half + key group: four consecutive keys
    const int dl = tid >> 3, q = tid & 7, half = q >> 2, kgk = q & 3;
    const int dim = dim0 + dl;
    const int jj = half * 16 + kgk * 4;
    const uint32_t lo = (uint32_t)tile[jj][dl] | ((uint32_t)tile[jj + 1][dl] << 16);
    const uint32_t hi = (uint32_t)tile[jj + 2][dl] | ((uint32_t)tile[jj + 3][dl] << 16);
    const size_t blk = ((size_t)g * (hd >> 4) + (dim >> 4)) * (Lpad >> 5) + (j0 >> 5);
    *reinterpret_cast<uint2*>(vt + blk * 512 + ((dim & 15) + 16 * kgk) * 8 + 4 * half) = make_uint2(lo, hi);
  }
}

__global__ void pf_set_len_kernel(int32_t* seq_lens, int slot, int v) { seq_lens[slot] = v; }

// bf16 out, K split over the waves of a workgroup; W2 != nullptr: the SwiGLU pair; i8: int8 matrices with g.sc / g.sc2
static int pf_gemm4(int epi, const PfGemm& g, const void* W2, int c_tiled, bool i8, hipStream_t st) {
  if (g.K % 64 || g.N % 16 || g.M < 1 || g.N < 1 || (c_tiled && g.N % 64)) { vui_set_error("prefill GEMM: bad shape N=%d K=%d", g.N, g.K); return VUI_EINVAL; }
  const dim3 grid((unsigned)(((g.M + 31) / 32) * ((g.N + 31) / 32)));
  if (i8) {
    if (W2) hipLaunchKernelGGL((pf_gemm4_kernel<PF_BF16, true, true>), grid, dim3(256), 0, st, g, W2, c_tiled);
    else if (epi == PF_RESID) hipLaunchKernelGGL((pf_gemm4_kernel<PF_RESID, false, true>), grid, dim3(256), 0, st, g, W2, c_tiled);
    else hipLaunchKernelGGL((pf_gemm4_kernel<PF_BF16, false, true>), grid, dim3(256), 0, st, g, W2, c_tiled);
  } else {
    if (W2) hipLaunchKernelGGL((pf_gemm4_kernel<PF_BF16, true, false>), grid, dim3(256), 0, st, g, W2, c_tiled);
    else if (epi == PF_RESID) hipLaunchKernelGGL((pf_gemm4_kernel<PF_RESID, false, false>), grid, dim3(256), 0, st, g, W2, c_tiled);
    else hipLaunchKernelGGL((pf_gemm4_kernel<PF_BF16, false, false>), grid, dim3(256), 0, st, g, W2, c_tiled);
  }
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

static size_t pf_align(size_t b) { return (b + 255) & ~(size_t)255; }

// scratch: residual x, normed xn, qkv, attention output, FFN buffer, staged keys and values
size_t prefill_scratch_bytes(const vui_config& c, int T, int L) {
  const size_t d = c.d_model, nq = (size_t)c.n_heads * c.head_dim, nkv = (size_t)c.n_kv_heads * c.head_dim;
  const size_t Lpad = ((size_t)L + 63) & ~(size_t)63;
  const size_t T16 = ((size_t)T + 15) & ~(size_t)15;  // tiled operands come in blocks of 16 rows
  size_t b = 0;
  b += pf_align((size_t)T * d * 2) + pf_align(T16 * d * 2);
  b += pf_align((size_t)T * (nq + 2 * nkv) * 2);
  b += pf_align(T16 * nq * 2);
  b += pf_align(T16 * c.ffn * 2);
  b += pf_align(nkv * Lpad * 2) * 2;
  return b;
}

// elements of one layer's weights in tiled form (wqkv | wo | w1 | w3 | w2), and of all layers
static size_t pf_layer_elems(const vui_config& c) {
  const size_t d = c.d_model, nq = (size_t)c.n_heads * c.head_dim, nkv = (size_t)c.n_kv_heads * c.head_dim, F = c.ffn;
  return (nq + 2 * nkv) * d + d * nq + 2 * F * d + d * F;
}
// the pass's own tiled copy: bf16 matrices only (an int8 context reads the batched backbone kernel's tiled int8 copy)
size_t prefill_weight_bytes(const vui_config& c) {
  char why[96];
  return (!c.int8_backbone && prefill_supported(c, why, sizeof(why))) ? pf_layer_elems(c) * c.n_layers * 2 : 0;
}

// one-time: the layers' projection weights in the GEMMs' operand layout
int prefill_tile_weights(const vui_config& c, const vui_weights& w, void* dst, hipStream_t st) {
  const int d = c.d_model, nq = c.n_heads * c.head_dim, nkv = c.n_kv_heads * c.head_dim, F = c.ffn;
  bf16_t* o = (bf16_t*)dst;
  auto tile = [&](const void* src, int N, int K) {
    const size_t pieces = (size_t)N * (K / 8);
    hipLaunchKernelGGL(pf_tile_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, (const bf16_t*)src, o, N, K);
    o += (size_t)N * K;
  };
  for (int l = 0; l < c.n_layers; ++l) {
    const vui_layer_weights& lw = w.layers[l];
    tile(lw.wqkv, nq + 2 * nkv, d);
    tile(lw.wo, d, nq);
    tile(lw.w1, F, d);
    tile(lw.w3, F, d);
    tile(lw.w2, d, F);
  }
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

bool prefill_supported(const vui_config& c, char* why, size_t why_len) {
  const char* r = nullptr;
  const int nkv = c.n_kv_heads * c.head_dim;
  if (c.dtype != VUI_DTYPE_BF16) r = "bf16 activations only";
  else if (c.int8_backbone && !bb_batch_weight_bytes(c, 256)) r = "int8 weights: no tiled int8 copy (it belongs to the batched backbone kernel, which does not take this configuration)";
  else if ((c.d_model % 64) || (c.ffn % 64) || ((c.n_heads * c.head_dim) % 64) || (c.head_dim % 32) || c.head_dim > 128 || (nkv % 8) || (c.rope_dim & 1))
    r = "d_model, heads x head_dim and ffn must be multiples of 64, head_dim a multiple of 32 up to 128";
  else if (c.n_kv_heads < 1 || c.n_heads % c.n_kv_heads) r = "heads must be a multiple of KV heads";
  if (r && why) snprintf(why, why_len, "%s", r);
  return r == nullptr;
}

int launch_prefill(const vui_config& c, const vui_weights& w, const void* tiled_w, const void* emb, int T, int slot, int pos0,
                   int32_t* seq_lens, void* k_cache, void* v_cache, void* out, void* scratch, size_t scratch_bytes, hipStream_t st) {
  const int d = c.d_model, H = c.n_heads, KV = c.n_kv_heads, hd = c.head_dim, F = c.ffn, S = c.max_seqlen;
  const int nq = H * hd, nkv = KV * hd, L = pos0 + T, Lpad = (L + 63) & ~63;
  char why[96];
  if (!prefill_supported(c, why, sizeof(why))) { vui_set_error("prefill: %s", why); return VUI_EINVAL; }
  if (T < 1 || pos0 < 0 || L > S) { vui_set_error("prefill: positions %d..%d outside the cache (S=%d)", pos0, L, S); return VUI_EINVAL; }
  if (slot < 0 || slot >= c.n_slots) { vui_set_error("prefill: slot %d outside [0,%d)", slot, c.n_slots); return VUI_EINVAL; }
  if (scratch_bytes < prefill_scratch_bytes(c, T, L)) { vui_set_error("prefill: scratch of %zu bytes, %zu needed", scratch_bytes, prefill_scratch_bytes(c, T, L)); return VUI_EINVAL; }
  if (!tiled_w) { vui_set_error("prefill: the context holds no tiled weights"); return VUI_EINVAL; }
  const size_t T16 = ((size_t)T + 15) & ~(size_t)15;
  char* sp = (char*)scratch;
  auto take = [&](size_t bytes) { char* r = sp; sp += pf_align(bytes); return r; };
  bf16_t* x = (bf16_t*)take((size_t)T * d * 2);                 // residual stream, row-major
  bf16_t* xn = (bf16_t*)take(T16 * d * 2);                      // normed rows, tiled (rows past T are never written:
  bf16_t* qkv = (bf16_t*)take((size_t)T * (nq + 2 * nkv) * 2);  //  what a GEMM reads there only reaches output rows it drops)
  bf16_t* att = (bf16_t*)take(T16 * nq * 2);                    // attention output, tiled
  bf16_t* fa = (bf16_t*)take(T16 * F * 2);                      // SwiGLU product, tiled
  bf16_t* kt = (bf16_t*)take((size_t)nkv * Lpad * 2);                // staged keys and values of the slot
  bf16_t* vt = (bf16_t*)take((size_t)nkv * Lpad * 2);
  HIP_TRY(hipMemcpyAsync(x, emb, (size_t)T * d * 2, hipMemcpyDeviceToDevice, st));
  const size_t slab = (size_t)c.n_slots * S * nkv;
  const float scale = 1.0f / sqrtf((float)hd);
  int rc;
  for (int l = 0; l < c.n_layers; ++l) {
    const vui_layer_weights& lw = w.layers[l];
    const bool i8 = c.int8_backbone != 0;
    const size_t wsz = i8 ? 1 : 2;
    const char* t_qkv = (const char*)tiled_w + pf_layer_elems(c) * wsz * l;
    const char* t_o = t_qkv + (size_t)(nq + 2 * nkv) * d * wsz;
    const char* t_1 = t_o + (size_t)d * nq * wsz;
    const char* t_3 = t_1 + (size_t)F * d * wsz;
    const char* t_2 = t_3 + (size_t)F * d * wsz;
    bf16_t* kc = (bf16_t*)k_cache + slab * l;
    bf16_t* vc = (bf16_t*)v_cache + slab * l;
    hipLaunchKernelGGL(pf_rownorm_kernel, dim3((T + 3) / 4), dim3(256), 0, st, x, (const bf16_t*)lw.attn_norm, xn, T, d, c.norm_eps, 1);
    PfGemm g{};
    g.X = xn; g.W = t_qkv; g.C = qkv; g.M = T; g.N = nq + 2 * nkv; g.K = d; g.ldc = nq + 2 * nkv; g.sc = (const bf16_t*)lw.s_qkv;
    if ((rc = pf_gemm4(PF_BF16, g, nullptr, 0, i8, st))) return rc;
    // attention over the L cached positions of this slot
    bf16_t* krow = kc + (size_t)slot * S * nkv;
    bf16_t* vrow = vc + (size_t)slot * S * nkv;
    int rope_dim_l;
    const float* rope_l = layer_rope(c, w, l, &rope_dim_l);
    const int window_l = layer_window(c, l);
    hipLaunchKernelGGL(pf_stage_kv_kernel, dim3(Lpad / 32, (nkv + nq) / 32), dim3(256), 0, st, qkv, krow, vrow, kt, vt, rope_l, L, Lpad, nq, nkv,
                       hd, rope_dim_l, pos0);
    {
      const dim3 grid((T + 15) / 16, H);
      switch (hd / 32) {
        case 1: hipLaunchKernelGGL(pf_attn_kernel<1>, grid, dim3(512), 0, st, qkv, kt, vt, att, T, L, Lpad, nq, nkv, H / KV, pos0, window_l, scale); break;
        case 2: hipLaunchKernelGGL(pf_attn_kernel<2>, grid, dim3(512), 0, st, qkv, kt, vt, att, T, L, Lpad, nq, nkv, H / KV, pos0, window_l, scale); break;
        case 3: hipLaunchKernelGGL(pf_attn_kernel<3>, grid, dim3(512), 0, st, qkv, kt, vt, att, T, L, Lpad, nq, nkv, H / KV, pos0, window_l, scale); break;
        default: hipLaunchKernelGGL(pf_attn_kernel<4>, grid, dim3(256), 0, st, qkv, kt, vt, att, T, L, Lpad, nq, nkv, H / KV, pos0, window_l, scale); break;
      }
    }
    PfGemm wo{};
    wo.X = att; wo.W = t_o; wo.C = x; wo.ldc = d; wo.M = T; wo.N = d; wo.K = nq; wo.sc = (const bf16_t*)lw.s_o;
    if ((rc = pf_gemm4(PF_RESID, wo, nullptr, 0, i8, st))) return rc;
    hipLaunchKernelGGL(pf_rownorm_kernel, dim3((T + 3) / 4), dim3(256), 0, st, x, (const bf16_t*)lw.mlp_norm, xn, T, d, c.norm_eps, 1);
    PfGemm f1{};
    f1.X = xn; f1.W = t_1; f1.C = fa; f1.ldc = F; f1.M = T; f1.N = F; f1.K = d; f1.sc = (const bf16_t*)lw.s_1; f1.sc2 = (const bf16_t*)lw.s_3;
    if ((rc = pf_gemm4(PF_BF16, f1, t_3, 1, i8, st))) return rc;  // written tiled: operand of W2
    PfGemm f2{};
    f2.X = fa; f2.W = t_2; f2.C = x; f2.ldc = d; f2.M = T; f2.N = d; f2.K = F; f2.sc = (const bf16_t*)lw.s_2;
    if ((rc = pf_gemm4(PF_RESID, f2, nullptr, 0, i8, st))) return rc;
  }
  hipLaunchKernelGGL(pf_rownorm_kernel, dim3((T + 3) / 4), dim3(256), 0, st, x, (const bf16_t*)w.final_norm, (bf16_t*)out, T, d, c.norm_eps, 0);
  hipLaunchKernelGGL(pf_set_len_kernel, dim3(1), dim3(1), 0, st, seq_lens, slot, L);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}
