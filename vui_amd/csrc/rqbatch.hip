// The depth head for up to 16 rows as ONE persistent kernel (bf16).
//
//   RQTransformer._generate_graph_body_kv / generate_cuda_graph_kv for B > 1  (src/vui/model.py:908-1016)
//
// As a kernel sequence the depth head of a batch is ~350 launches of a few microseconds each, i.e.
// launch-boundary bound.  Here one resident grid (one workgroup per CU) walks the phase list and
// exchanges activations through flag-in-data words (ll.h), as the batch-1 frame kernel does, with the
// matrix cores inside: a workgroup owns tiles of 16 output features of a weight matrix and multiplies
// them with the activations of its rows in one v_mfma_f32_16x16x32_bf16 per 32 k.
//
// The rows are split into row groups of 4 (up to 4 rows: one row per group), each served by 64 workgroups:
// reading an exchanged vector is
// bound by the number of 8-byte words one CU has to poll (about one per two clocks), so four groups that
// each poll a quarter of the rows beat one group polling all sixteen by ~2x (measured), although the
// weights are then read four times (from L2) and the matrix-core tile is a quarter full.
//
// Roles inside a row group (a workgroup holds several; every workgroup walks the same phases in order):
//   all 64      keep the residual stream of the group's rows in LDS (fp32) and take two tiles (wl, wl + 64)
//               of each matrix that follows an RMSNorm (QKV, W1/W3, logits head; projection of position 0), and a
//               third (wl + 128) of a QKV with more than 128 tiles (depth heads wider than 682)
//   attention   workgroup 63 - task, task = local row * heads + head: that row's head, its keys/values of
//               all layers and positions in LDS
//   out tiles   workgroup 63 - tile - (R/16) * half: out_proj and W2 of tile < R/16 for one half of the group's rows
//               (all rows when R/16 > 32)
//   sampler     workgroup r < rows of the group draws row r's code
// Rounding points are those of the kernel sequence (gemv_epi.h, attn.hip, sample.h).
#include "common.h"
#include "internal.h"
#include "ll.h"
#include "sample.h"
#include <stdio.h>
#include <string.h>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 rb_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float rb_floatx4;
union RbU128 { uint4 u; rb_bf16x8 v; };
__device__ __forceinline__ rb_bf16x8 rb_frag(const uint4& x) { RbU128 t; t.u = x; return t.v; }

struct Tile { int n0, N, K; bool on; };
#define RB_RG 4     // rows per row group
#define RB_NWL 64   // workgroups per row group

// weight fragments of one 16-feature tile, K split over the four waves in steps of 32
template <int MAXS, bool DUAL>
struct TileW { uint4 a[MAXS]; uint4 b[DUAL ? MAXS : 1]; };

// The matrices this kernel multiplies by are read from a copy in "tiled" form (rb_tile_kernel): inside every band of
// 16 rows, the block of columns 32 s .. 32 s + 31 is 512 consecutive elements, the 8 elements of lane
// (row % 16) + 16 * ((col % 32) / 8) at 8 * lane.  A wave's fragment load is then 1 KiB contiguous; from the
// row-major form the 16 lanes of a quarter-wave would read 16 different lines, which the address unit serves at
// about a quarter of the rate.  A band starts where it does in the row-major form (16 rows x K elements each).
template <int MAXS, bool DUAL>
__device__ __forceinline__ void tile_prefetch(const bf16_t* W, const bf16_t* W2, const Tile& t, TileW<MAXS, DUAL>& r) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (!t.on) return;
  const size_t band = (size_t)t.n0 * t.K + lane * 8;  // n0 is a multiple of 16, N as well: the band is inside the matrix
#pragma unroll
  for (int i = 0; i < MAXS; ++i) {
    const int s = wave + 4 * i;
    const bool on = s * 32 < t.K;
    r.a[i] = on ? *reinterpret_cast<const uint4*>(W + band + (size_t)s * 512) : make_uint4(0, 0, 0, 0);
    if (DUAL) r.b[i] = on ? *reinterpret_cast<const uint4*>(W2 + band + (size_t)s * 512) : make_uint4(0, 0, 0, 0);
  }
}

// row-major (N x K, N % 16 == 0, K % 32 == 0) -> tiled; one 8-element piece per thread
__global__ __launch_bounds__(256) void rb_tile_kernel(const bf16_t* __restrict__ src, bf16_t* __restrict__ dst, size_t N, int K) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int per_row = K >> 3;
  if (i >= N * per_row) return;
  const size_t n = i / per_row;
  const int k = (int)(i % per_row) * 8;
  const size_t o = (n >> 4) * 16 * (size_t)K + (size_t)(k >> 5) * 512 + ((n & 15) + 16 * ((k & 31) >> 3)) * 8;
  *reinterpret_cast<uint4*>(dst + o) = *reinterpret_cast<const uint4*>(src + n * K + k);
}

// xp: activations of the group's rows as packed bf16 pairs (row stride xs words) followed by one zero row that
// stands for the other columns of the matrix-core tile.  epi(n, row, v[4], u[4]) is called by
// the lanes of wave 0: features n .. n+3 of `row` (u: second matrix).
template <int MAXS, bool DUAL, typename Epi>
__device__ __forceinline__ void tile_compute(const uint32_t* xp, int xs, const Tile& t, const TileW<MAXS, DUAL>& r, float* red,
                                             int B, Epi&& epi) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, l16 = lane & 15, kg = lane >> 4;
  if (!t.on) return;  // uniform over the workgroup
  rb_floatx4 acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < MAXS; ++i) {
    const int s = wave + 4 * i;
    if (s * 32 < t.K) {
      const uint4 x = *reinterpret_cast<const uint4*>(xp + (size_t)min(l16, RB_RG) * xs + s * 16 + kg * 4);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rb_frag(r.a[i]), rb_frag(x), acc, 0, 0, 0);
      if (DUAL) acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rb_frag(r.b[i]), rb_frag(x), acc2, 0, 0, 0);
    }
  }
  const int per = DUAL ? 8 : 4;
  float* mine = red + ((size_t)wave * 64 + lane) * per;
#pragma unroll
  for (int q = 0; q < 4; ++q) { mine[q] = acc[q]; if (DUAL) mine[4 + q] = acc2[q]; }
  __syncthreads();
  if (wave == 0) {
    float v[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        v[q] += red[((size_t)w * 64 + lane) * per + q];
        if (DUAL) u[q] += red[((size_t)w * 64 + lane) * per + 4 + q];
      }
    const int n = t.n0 + 4 * kg;
    if (l16 < B && n < t.N) epi(n, l16, v, u);
  }
}

// Two tiles of the same matrix against the same activations in one pass: one read of every activation fragment, one
// barrier, and the two epilogues side by side in waves 0 and 1 (as two calls of tile_compute they were a second
// barrier and a second epilogue behind the first).  red: twice the floats of tile_compute.
template <int MAXS, bool DUAL, typename Epi>
__device__ __forceinline__ void tile_compute2(const uint32_t* xp, int xs, const Tile& t0, const TileW<MAXS, DUAL>& r0, const Tile& t1,
                                              const TileW<MAXS, DUAL>& r1, float* red, int B, Epi&& epi) {
  if (!t0.on) return;  // uniform over the workgroup; t1 is never on without t0
  if (!t1.on) { tile_compute<MAXS, DUAL>(xp, xs, t0, r0, red, B, epi); return; }
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, l16 = lane & 15, kg = lane >> 4;
  rb_floatx4 a0 = {0.f, 0.f, 0.f, 0.f}, a0b = a0, a1 = a0, a1b = a0;
#pragma unroll
  for (int i = 0; i < MAXS; ++i) {
    const int s = wave + 4 * i;
    if (s * 32 < t0.K) {
      const uint4 x = *reinterpret_cast<const uint4*>(xp + (size_t)min(l16, RB_RG) * xs + s * 16 + kg * 4);
      a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rb_frag(r0.a[i]), rb_frag(x), a0, 0, 0, 0);
      a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rb_frag(r1.a[i]), rb_frag(x), a1, 0, 0, 0);
      if (DUAL) {
        a0b = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rb_frag(r0.b[i]), rb_frag(x), a0b, 0, 0, 0);
        a1b = __builtin_amdgcn_mfma_f32_16x16x32_bf16(rb_frag(r1.b[i]), rb_frag(x), a1b, 0, 0, 0);
      }
    }
  }
  const int per = DUAL ? 8 : 4, half = 4 * 64 * per;
  float* mine = red + ((size_t)wave * 64 + lane) * per;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    mine[q] = a0[q]; mine[half + q] = a1[q];
    if (DUAL) { mine[4 + q] = a0b[q]; mine[half + 4 + q] = a1b[q]; }
  }
  __syncthreads();
  if (wave < 2) {
    const float* src = red + (wave ? half : 0);
    const Tile& t = wave ? t1 : t0;
    float v[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        v[q] += src[((size_t)w * 64 + lane) * per + q];
        if (DUAL) u[q] += src[((size_t)w * 64 + lane) * per + 4 + q];
      }
    const int n = t.n0 + 4 * kg;
    if (l16 < B && n < t.N) epi(n, l16, v, u);
  }
}

struct NormRegs { uint4 w[2]; };  // norm weights of chunks lane, lane + 64 (R <= 1024)
__device__ __forceinline__ NormRegs load_norm(const bf16_t* nw, int R) {
  NormRegs r;
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = lane + WAVE * i;
    r.w[i] = c < R / 8 ? *reinterpret_cast<const uint4*>(nw + c * 8) : make_uint4(0, 0, 0, 0);
  }
  return r;
}
// two-rounding RMSNorm of the B rows of xres (fp32, row stride R) into xp (packed bf16); wave w takes rows w, w+4, ...
__device__ __forceinline__ void norm_rows(const float* xres, const NormRegs& nw, float eps, int R, int B, uint32_t* xp, int xs) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  for (int b = wave; b < B; b += 4) {
    const float* x = xres + (size_t)b * R;
    float4 q[2][2];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = min(lane + WAVE * i, R / 8 - 1);
      q[i][0] = *reinterpret_cast<const float4*>(x + c * 8);
      q[i][1] = *reinterpret_cast<const float4*>(x + c * 8 + 4);
      const float t = (q[i][0].x * q[i][0].x + q[i][0].y * q[i][0].y) + (q[i][0].z * q[i][0].z + q[i][0].w * q[i][0].w) +
                      (q[i][1].x * q[i][1].x + q[i][1].y * q[i][1].y) + (q[i][1].z * q[i][1].z + q[i][1].w * q[i][1].w);
      ss += (lane + WAVE * i < R / 8) ? t : 0.f;
    }
    ss = wave_sum_v(ss);
    const float r = 1.0f / sqrtf(ss / (float)R + eps);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = lane + WAVE * i;
      if (c < R / 8) {
        const uint4 g = nw.w[i];
        uint4 o;
        uint32_t v;
        v = f2bf2(q[i][0].x * r, q[i][0].y * r); o.x = f2bf2(bf_lo(v) * bf_lo(g.x), bf_hi(v) * bf_hi(g.x));
        v = f2bf2(q[i][0].z * r, q[i][0].w * r); o.y = f2bf2(bf_lo(v) * bf_lo(g.y), bf_hi(v) * bf_hi(g.y));
        v = f2bf2(q[i][1].x * r, q[i][1].y * r); o.z = f2bf2(bf_lo(v) * bf_lo(g.z), bf_hi(v) * bf_hi(g.z));
        v = f2bf2(q[i][1].z * r, q[i][1].w * r); o.w = f2bf2(bf_lo(v) * bf_lo(g.w), bf_hi(v) * bf_hi(g.w));
        *reinterpret_cast<uint4*>(xp + (size_t)b * xs + c * 4) = o;
      }
    }
  }
}

// Residual add of an exchanged vector and the norm that follows it, row by row inside one wave: wave w waits for the
// words of rows w, w + 4, ... (a lane for the four words of chunk lane, and of chunk lane + 64), adds them to the
// residual stream (x = rnd(x + y), written back), and normalises the row at once - the row never leaves the wave, so
// no barrier stands between the wait, the add and the norm.  buf: the group's rows, R/2 words each.
__device__ __forceinline__ void poll_add_norm_rows(const uint64_t* buf, Ctl& c, float* xres, const NormRegs& nw, float eps, int R,
                                                   int B, uint32_t* xp, int xs) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int nch = R / 8;
  const int NI = nch > WAVE ? 2 : 1;  // chunks per lane
  for (int b = wave; b < B; b += 4) {
    const uint64_t* row = buf + (size_t)b * (R / 2);
    float* x = xres + (size_t)b * R;
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
        const uint32_t pk = f2bf2(old[2 * k] + bf_lo(y), old[2 * k + 1] + bf_hi(y));
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
    const float r = 1.0f / sqrtf(ss / (float)R + eps);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int ch = lane + WAVE * i;
      if (ch < nch) {
        const uint4 g = nw.w[i];
        uint4 o;
        uint32_t t;
        t = f2bf2(q[i][0] * r, q[i][1] * r); o.x = f2bf2(bf_lo(t) * bf_lo(g.x), bf_hi(t) * bf_hi(g.x));
        t = f2bf2(q[i][2] * r, q[i][3] * r); o.y = f2bf2(bf_lo(t) * bf_lo(g.y), bf_hi(t) * bf_hi(g.y));
        t = f2bf2(q[i][4] * r, q[i][5] * r); o.z = f2bf2(bf_lo(t) * bf_lo(g.z), bf_hi(t) * bf_hi(g.z));
        t = f2bf2(q[i][6] * r, q[i][7] * r); o.w = f2bf2(bf_lo(t) * bf_lo(g.w), bf_hi(t) * bf_hi(g.w));
        *reinterpret_cast<uint4*>(xp + (size_t)b * xs + ch * 4) = o;
      }
    }
  }
}

// i / nw for i < 65536 with inv = ceil(2^32 / nw)
__device__ __forceinline__ int div_small(int i, uint32_t inv) { return (int)__umulhi((uint32_t)i, inv); }

struct RqBatchArgs {
  int B, d, R, rqH, rqF, rqL, Q, CS, n_q;
  float rq_eps;
  const vui_weights* w;
  const uint16_t* hidden;
  const int64_t* code0;
  int64_t* codes_out;
  int codes_stride, zero_pad;
  const float* logit_bias;
  float temp;
  int topk;
  uint64_t seed;
  const vui_sample_dev* sdev;  // if set: the three above are read from here
  const int32_t* frame_ctr;
  uint64_t* ll;
  uint32_t *epoch, *arrive, *err;
  int xs;                                            // row stride of the staged activations, words
  int off_xp, off_red, off_misc, off_att, off_kv;    // LDS offsets, bytes (xres at 0)
  unsigned long long* dbg;                           // optional 64 stamps of one pass (profiling builds)
  int dbg_wg;
};

struct RbLayer { const bf16_t *attn_norm, *wqkv, *wo, *mlp_norm, *w1, *w3, *w2; };

// Q3: QKV has more than two tiles per workgroup of a row group (see the roles above); a compile-time switch, so that the
// common form carries neither the third tile's registers nor its tests.
template <bool Q3>
__global__ __launch_bounds__(FR_THREADS, 1) void rq_batch_kernel(const RqBatchArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  float* xres = (float*)smem;                             // [RB_RG][R]
  uint32_t* xp = (uint32_t*)(smem + a.off_xp);            // [RB_RG + 1][xs], the last row stays zero
  float* red = (float*)(smem + a.off_red);                // 2 x 4 x 64 x 8 floats; the sampler's histogram
  int* codes_s = (int*)(smem + a.off_misc);               // codes of the group's rows at the current position
  SampleShared& ssh = *(SampleShared*)(smem + a.off_misc + 64);
  uint32_t* aq = (uint32_t*)(smem + a.off_att);           // attention role: q (packed), softmax weights
  bf16_t* pw_hi = (bf16_t*)(smem + a.off_att + 512);
  bf16_t* pw_lo = pw_hi + 64;
  bf16_t* kvbase = (bf16_t*)(smem + a.off_kv);

  const int wg = blockIdx.x, nwg = gridDim.x, tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int B = a.B, R = a.R, d = a.d, CS = a.CS, Q = a.Q, xs = a.xs;
  const int rhd = R / a.rqH, QP8 = (Q + 7) & ~7;
  Ctl c;
  ctl_begin(c, a.epoch, a.err);
  const uint32_t ep = c.epoch;
  const vui_weights& W = *a.w;
  const bf16_t* g_proj = (const bf16_t*)W.rq_backbone_proj;
  const bf16_t* g_emb = (const bf16_t*)W.rq_code_emb;
  const bf16_t* g_pos = (const bf16_t*)W.rq_pos_emb;
  const bf16_t* g_head = (const bf16_t*)W.rq_head_w;
  const bf16_t* g_norm = (const bf16_t*)W.rq_norm;
  const uint32_t frame = a.frame_ctr ? (uint32_t)a.frame_ctr[0] : 0u;
  const float s_temp = a.sdev ? a.sdev->temperature : a.temp;
  const int s_topk = a.sdev ? a.sdev->top_k : a.topk;
  const uint64_t s_seed = a.sdev ? a.sdev->seed : a.seed;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  if (tid == 0) __hip_atomic_fetch_add(a.arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  // row group of this workgroup and its roles inside the group
  const int grp = wg / RB_NWL, wl = wg % RB_NWL;
  // rows per group: up to four rows take a group each (a phase costs what a workgroup waits for: the exchanged
  // words of its group's rows; measured 3-5 % of the step at 2-4 rows).  Eight rows as four groups of two were
  // slower than as two groups of four (all 256 workgroups then stream every weight), so more rows keep groups of four.
  const int rg = B <= RB_RG ? 1 : RB_RG;
  const int b0 = grp * rg, Bg = min(max(B - b0, 0), rg);
  const bool active = Bg > 0;
  const int nA = 3 * R / 16, nS = a.rqF / 16, nH = CS / 16, nO = R / 16;
  const int back = RB_NWL - 1 - wl;
  const bool att_on = active && back < Bg * a.rqH;
  const int att_lr = back / a.rqH, att_h = back % a.rqH;
  // out_proj / W2 tiles: with twice as many workgroups as tiles the rows of the group are split in two halves, so
  // a workgroup waits for half as many exchanged words (the wait, not the product, is what these phases cost)
  const bool out_split = 2 * nO <= RB_NWL;
  const int out_tile = out_split ? back % nO : back;
  const int out_r0 = out_split ? (back / nO) * (RB_RG / 2) : 0;                     // first local row
  const int out_nr = out_split ? max(0, min(Bg - out_r0, RB_RG / 2)) : Bg;          // rows taken
  const bool out_on = active && out_nr > 0 && back < (out_split ? 2 * nO : nO);
  const uint32_t inv_r2 = 0xFFFFFFFFu / (uint32_t)(R / 2) + 1u, inv_f2 = 0xFFFFFFFFu / (uint32_t)(a.rqF / 2) + 1u;

  for (int i = tid; i < (RB_RG + 1) * xs; i += FR_THREADS) xp[i] = 0u;
  // values of positions not yet written are multiplied by weight zero and must be finite
  if (att_on) for (int i = tid; i < a.rqL * rhd * QP8; i += FR_THREADS) reinterpret_cast<uint32_t*>(kvbase)[i] = 0u;
  if (active && wl < Bg && tid == 0) {
    int64_t cc = a.code0[b0 + wl];
    a.codes_out[(size_t)(b0 + wl) * a.codes_stride] = cc < 0 ? 0 : (cc >= CS ? CS - 1 : cc);
  }
  __syncthreads();

#ifdef VUI_RB_CLOCK
  __shared__ unsigned long long dbg_ts[64];
  int dbg_n = 0;
#define RB_TS() do { if (a.dbg && wg == a.dbg_wg && tid == 0 && t == 8 && dbg_n < 64) dbg_ts[dbg_n++] = wall_clock64(); } while (0)
#else
#define RB_TS() do { } while (0)
#endif
  // two tiles per workgroup and matrix: wl and wl + RB_NWL
  auto tile_of = [&](int k, int nT, int N, int K) { Tile t = {16 * (wl + k * RB_NWL), N, K, active && (wl + k * RB_NWL) < nT}; return t; };

  uint64_t* llp = a.ll;
  // ---- position 0: projected hidden + pos_emb[0]
  {
    uint64_t* x0 = llp;
    llp += (size_t)B * (R / 2);
    if (g_proj) {
      const Tile t = tile_of(0, nO, R, d);
      TileW<8, false> wr;
      tile_prefetch<8, false>(g_proj, nullptr, t, wr);
      if (t.on) {
        for (int i = tid; i < Bg * (d / 2); i += FR_THREADS) {
          const int lr = i / (d / 2), j = i - lr * (d / 2);
          xp[(size_t)lr * xs + j] = reinterpret_cast<const uint32_t*>(a.hidden)[(size_t)(b0 + lr) * (d / 2) + j];
        }
      }
      __syncthreads();
      tile_compute<8, false>(xp, xs, t, wr, red, Bg, [&](int n, int lr, const float* v, const float*) {
        const uint2 pe = *reinterpret_cast<const uint2*>(g_pos + n);
        uint64_t* dst = x0 + (size_t)(b0 + lr) * (R / 2) + n / 2;
        ll_st(dst, f2bf2(bf2f(f2bf(v[0])) + bf_lo(pe.x), bf2f(f2bf(v[1])) + bf_hi(pe.x)), ep);
        ll_st(dst + 1, f2bf2(bf2f(f2bf(v[2])) + bf_lo(pe.y), bf2f(f2bf(v[3])) + bf_hi(pe.y)), ep);
      });
      if (active) {
        __syncthreads();
        ll_poll_auto(x0 + (size_t)b0 * (R / 2), Bg * (R / 2), c, [&](int i, uint32_t v) {
          const int lr = div_small(i, inv_r2), j = i - lr * (R / 2);
          *reinterpret_cast<float2*>(xres + (size_t)lr * R + 2 * j) = make_float2(bf_lo(v), bf_hi(v));
        });
        __syncthreads();
        // the staged hidden rows are longer than the depth head's vectors: back to zero beyond R/2
        for (int i = tid; i < RB_RG * xs; i += FR_THREADS) xp[i] = 0u;
        __syncthreads();
      }
    } else if (active) {
      for (int i = tid; i < Bg * (R / 2); i += FR_THREADS) {
        const int lr = div_small(i, inv_r2), j = i - lr * (R / 2);
        const uint32_t h2 = reinterpret_cast<const uint32_t*>(a.hidden)[(size_t)(b0 + lr) * (R / 2) + j];
        const uint32_t p2 = reinterpret_cast<const uint32_t*>(g_pos)[j];
        const uint32_t pk = f2bf2(bf_lo(h2) + bf_lo(p2), bf_hi(h2) + bf_hi(p2));
        *reinterpret_cast<float2*>(xres + (size_t)lr * R + 2 * j) = make_float2(bf_lo(pk), bf_hi(pk));
      }
      __syncthreads();
    }
  }

  uint64_t* codebuf = nullptr;  // sampled codes of the previous pass
  for (int t = 0; t < a.n_q; ++t) {
    if (t >= 1 && active) {
      // token t: code embedding + pos_emb[t] for the group's rows
      __syncthreads();
      if (t == 1) {
        if (tid < Bg) { int64_t cc = a.code0[b0 + tid]; codes_s[tid] = (int)(cc < 0 ? 0 : (cc >= CS ? CS - 1 : cc)); }
      } else {
        // (clamped: after a wait that was given up the word may hold anything, and the code indexes the embedding table)
        ll_poll_auto(codebuf + b0, Bg, c, [&](int i, uint32_t v) { codes_s[i] = (int)min(v, (uint32_t)(CS - 1)); });
      }
      __syncthreads();
      for (int i = tid; i < Bg * (R / 8); i += FR_THREADS) {
        const int lr = i / (R / 8), ch = i - lr * (R / 8);
        float e[8], p[8];
        El<bf16_t>::ld8(g_emb + ((size_t)codes_s[lr] + (size_t)(t - 1) * CS) * R + ch * 8, e);
        El<bf16_t>::ld8(g_pos + (size_t)t * R + ch * 8, p);
        float* o = xres + (size_t)lr * R + ch * 8;
#pragma unroll
        for (int k = 0; k < 8; ++k) o[k] = bf2f(f2bf(e[k] + p[k]));
      }
      __syncthreads();
    }
    const uint64_t* ybuf = nullptr;
    for (int l = 0; l < a.rqL; ++l) {
      const vui_rq_layer_weights& Lw = W.rq_layers[l];
      RB_TS();
      // ---- A: RMSNorm + QKV
      uint64_t* qkvb = llp;
      llp += (size_t)B * (3 * R / 2);
      if (active) {
        // QKV has three times the tiles of the other square matrices: a depth head wider than 2 * 64 * 16 / 3 features
        // gives the first workgroups of a group a third tile (wl + 128)
        const Tile t0 = tile_of(0, nA, 3 * R, R), t1 = tile_of(1, nA, 3 * R, R);
        Tile t2 = {0, 3 * R, R, false};
        TileW<8, false> w0, w1, w2;
        tile_prefetch<8, false>((const bf16_t*)Lw.wqkv, nullptr, t0, w0);
        tile_prefetch<8, false>((const bf16_t*)Lw.wqkv, nullptr, t1, w1);
        if (Q3) {
          t2 = tile_of(2, nA, 3 * R, R);
          tile_prefetch<8, false>((const bf16_t*)Lw.wqkv, nullptr, t2, w2);
        }
        const NormRegs nw = load_norm((const bf16_t*)Lw.attn_norm, R);
        if (ybuf) poll_add_norm_rows(ybuf + (size_t)b0 * (R / 2), c, xres, nw, a.rq_eps, R, Bg, xp, xs);
        else norm_rows(xres, nw, a.rq_eps, R, Bg, xp, xs);
        __syncthreads();
        auto epi = [&](int n, int lr, const float* v, const float*) {
          uint64_t* dst = qkvb + (size_t)(b0 + lr) * (3 * R / 2) + n / 2;
          ll_st(dst, f2bf2(v[0], v[1]), ep);
          ll_st(dst + 1, f2bf2(v[2], v[3]), ep);
        };
        tile_compute2<8, false>(xp, xs, t0, w0, t1, w1, red, Bg, epi);
        if (Q3 && t2.on) {  // uniform over the workgroup
          __syncthreads();  // the partial sums of the first two tiles have been read
          tile_compute<8, false>(xp, xs, t2, w2, red, Bg, epi);
        }
      }
      RB_TS();
      const bool kv_only = (t == 0 && l == a.rqL - 1);  // position 0 only feeds later keys/values
      // ---- B: attention of one (row, head)
      uint64_t* attb = llp;
      if (!kv_only) llp += (size_t)B * (R / 2);
      if (att_on) {
        // keys [rhd/8][QP8][8], values [rhd][QP8] of this layer
        bf16_t* kcache = kvbase + (size_t)l * 2 * rhd * QP8;
        bf16_t* vcache = kcache + (size_t)rhd * QP8;
        const uint64_t* row = qkvb + (size_t)(b0 + att_lr) * (3 * R / 2);
        const int hw = rhd / 2;
        __syncthreads();
        {
          const uint64_t* p0 = tid < hw ? row + (att_h * rhd) / 2 + tid : nullptr;
          const uint64_t* p1 = tid < hw ? row + (R + att_h * rhd) / 2 + tid : nullptr;
          const uint64_t* p2 = tid < hw ? row + (2 * R + att_h * rhd) / 2 + tid : nullptr;
          uint32_t r0, r1, r2;
          poll3(p0, p1, p2, c, r0, r1, r2);
          if (tid < hw) {
            const int f = 2 * tid;
            aq[tid] = r0;
            *reinterpret_cast<uint32_t*>(kcache + ((size_t)(f >> 3) * QP8 + t) * 8 + (f & 7)) = r1;
            vcache[(size_t)f * QP8 + t] = (bf16_t)(r2 & 0xffff);
            vcache[(size_t)(f + 1) * QP8 + t] = (bf16_t)(r2 >> 16);
          }
        }
        __syncthreads();
        if (!kv_only && wave == 0) {
          int PP = Q <= 16 ? 4 : (Q <= 32 ? 2 : 1);
          while (PP > 1 && ((rhd % PP) || ((rhd / PP) & 1))) PP >>= 1;
          const int fpp = rhd / PP, nk = t + 1;
          const int kj = lane / PP, part = lane % PP, kk = min(kj, nk - 1);
          float dsum = 0.f;
          for (int i = 0; i < fpp / 2; ++i) {
            const int f = part * fpp + 2 * i;
            dsum = dot2_bf(*reinterpret_cast<const uint32_t*>(kcache + ((size_t)(f >> 3) * QP8 + kk) * 8 + (f & 7)), aq[f / 2], dsum);
          }
          if (PP >= 2) dsum += dpp_f<DPP_QUAD_XOR1>(dsum);
          if (PP >= 4) dsum += dpp_f<DPP_QUAD_XOR2>(dsum);
          const float sco = (kj < nk) ? dsum * (1.0f / sqrtf((float)rhd)) : -INFINITY;
          const float M = rows_max(group16_max(sco));
          const float pw = (kj < nk) ? __expf(sco - M) : 0.f;
          const float Ls = wave_sum_v(part == 0 ? pw : 0.f);
          if (part == 0) {
            const bf16_t hi = f2bf(pw);
            pw_hi[kj] = hi;
            pw_lo[kj] = f2bf(pw - bf2f(hi));
          }
          float o0 = 0.f, o1 = 0.f;
          const int fa = min(lane, rhd - 1), fb = min(lane + WAVE, rhd - 1);
          for (int j0 = 0; j0 < nk; j0 += 8) {
            const uint4 ph = *reinterpret_cast<const uint4*>(pw_hi + j0), pl = *reinterpret_cast<const uint4*>(pw_lo + j0);
            const uint4 va = *reinterpret_cast<const uint4*>(vcache + (size_t)fa * QP8 + j0);
            o0 = dot8_bf(va, ph, o0);
            o0 = dot8_bf(va, pl, o0);
            if (rhd > WAVE) {
              const uint4 vb = *reinterpret_cast<const uint4*>(vcache + (size_t)fb * QP8 + j0);
              o1 = dot8_bf(vb, ph, o1);
              o1 = dot8_bf(vb, pl, o1);
            }
          }
          const float inv = __builtin_amdgcn_rcpf(Ls);
          o0 *= inv; o1 *= inv;
          const float n0 = dpp_f<DPP_QUAD_XOR1>(o0), n1 = dpp_f<DPP_QUAD_XOR1>(o1);
          uint64_t* dst = attb + (size_t)(b0 + att_lr) * (R / 2) + (att_h * rhd) / 2;
          if (!(lane & 1)) {
            if (lane < rhd) ll_st(dst + lane / 2, f2bf2(o0, n0), ep);
            if (lane + WAVE < rhd) ll_st(dst + (lane + WAVE) / 2, f2bf2(o1, n1), ep);
          }
        }
      }
      RB_TS();
      if (kv_only) break;
      // ---- C: out_proj
      uint64_t* ob = llp;
      llp += (size_t)B * (R / 2);
      if (out_on) {
        const Tile to = {16 * out_tile, R, R, true};
        TileW<8, false> wr;
        tile_prefetch<8, false>((const bf16_t*)Lw.wo, nullptr, to, wr);
        __syncthreads();
        ll_poll_auto(attb + (size_t)(b0 + out_r0) * (R / 2), out_nr * (R / 2), c, [&](int i, uint32_t v) {
          const int lr = div_small(i, inv_r2), j = i - lr * (R / 2);
          xp[(size_t)lr * xs + j] = v;
        });
        __syncthreads();
        tile_compute<8, false>(xp, xs, to, wr, red, out_nr, [&](int n, int lr, const float* v, const float*) {
          uint64_t* dst = ob + (size_t)(b0 + out_r0 + lr) * (R / 2) + n / 2;
          ll_st(dst, f2bf2(v[0], v[1]), ep);
          ll_st(dst + 1, f2bf2(v[2], v[3]), ep);
        });
      }
      RB_TS();
      // ---- D: residual, RMSNorm, W1/W3, SwiGLU
      uint64_t* hb = llp;
      llp += (size_t)B * (a.rqF / 2);
      if (active) {
        const Tile t0 = tile_of(0, nS, a.rqF, R), t1 = tile_of(1, nS, a.rqF, R);
        TileW<8, true> w0, w1;
        tile_prefetch<8, true>((const bf16_t*)Lw.w1, (const bf16_t*)Lw.w3, t0, w0);
        tile_prefetch<8, true>((const bf16_t*)Lw.w1, (const bf16_t*)Lw.w3, t1, w1);
        const NormRegs nw = load_norm((const bf16_t*)Lw.mlp_norm, R);
        poll_add_norm_rows(ob + (size_t)b0 * (R / 2), c, xres, nw, a.rq_eps, R, Bg, xp, xs);
        __syncthreads();
        auto epi = [&](int n, int lr, const float* v, const float* u) {
          float h[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float g = bf2f(f2bf(v[q])), up = bf2f(f2bf(u[q]));
            h[q] = bf2f(f2bf(g / (1.0f + expf(-g)))) * up;
          }
          uint64_t* dst = hb + (size_t)(b0 + lr) * (a.rqF / 2) + n / 2;
          ll_st(dst, f2bf2(h[0], h[1]), ep);
          ll_st(dst + 1, f2bf2(h[2], h[3]), ep);
        };
        tile_compute2<8, true>(xp, xs, t0, w0, t1, w1, red, Bg, epi);
      }
      RB_TS();
      // ---- E: W2
      uint64_t* yb = llp;
      llp += (size_t)B * (R / 2);
      if (out_on) {
        const Tile tw = {16 * out_tile, R, a.rqF, true};
        TileW<16, false> wr;
        tile_prefetch<16, false>((const bf16_t*)Lw.w2, nullptr, tw, wr);
        __syncthreads();
        ll_poll_auto(hb + (size_t)(b0 + out_r0) * (a.rqF / 2), out_nr * (a.rqF / 2), c, [&](int i, uint32_t v) {
          const int lr = div_small(i, inv_f2), j = i - lr * (a.rqF / 2);
          xp[(size_t)lr * xs + j] = v;
        });
        __syncthreads();
        tile_compute<16, false>(xp, xs, tw, wr, red, out_nr, [&](int n, int lr, const float* v, const float*) {
          uint64_t* dst = yb + (size_t)(b0 + out_r0 + lr) * (R / 2) + n / 2;
          ll_st(dst, f2bf2(v[0], v[1]), ep);
          ll_st(dst + 1, f2bf2(v[2], v[3]), ep);
        });
      }
      ybuf = yb;
    }
    RB_TS();
    if (t >= 1) {
      // ---- logits of codebook t, then one sampler workgroup per row
      uint64_t* lgb = llp;
      llp += (size_t)B * (CS / 2);
      uint64_t* cb = llp;
      llp += 16;
      if (active) {
        const Tile t0 = tile_of(0, nH, CS, R), t1 = tile_of(1, nH, CS, R);
        TileW<8, false> w0, w1;
        const bf16_t* hw_ = g_head + (size_t)(t - 1) * CS * R;
        tile_prefetch<8, false>(hw_, nullptr, t0, w0);
        tile_prefetch<8, false>(hw_, nullptr, t1, w1);
        const NormRegs nw = load_norm(g_norm, R);
        poll_add_norm_rows(ybuf + (size_t)b0 * (R / 2), c, xres, nw, a.rq_eps, R, Bg, xp, xs);
        __syncthreads();
        auto epi = [&](int n, int lr, const float* v, const float*) {
          uint64_t* dst = lgb + (size_t)(b0 + lr) * (CS / 2) + n / 2;
          ll_st(dst, f2bf2(v[0], v[1]), ep);
          ll_st(dst + 1, f2bf2(v[2], v[3]), ep);
        };
        tile_compute2<8, false>(xp, xs, t0, w0, t1, w1, red, Bg, epi);
      }
      if (active && wl < Bg) {
        const int b = b0 + wl;
        // the row's logits pass through the first words of the staging area
        uint32_t* lgw = xp;
        const uint32_t rnd = philox_u32(s_seed, frame, (uint32_t)b, (uint32_t)t, 0u);  // ahead of the wait
        __syncthreads();
        ll_poll_auto(lgb + (size_t)b * (CS / 2), CS / 2, c, [&](int i, uint32_t v) { lgw[i] = v; });
        __syncthreads();
        const int E = (CS + FR_THREADS - 1) / FR_THREADS;
        const bool greedy = (s_topk == 1) || !(s_temp > 0.f);
        const float div = greedy ? 1.0f : s_temp;
        const float* bias = a.logit_bias ? a.logit_bias + (size_t)(t - 1) * CS : nullptr;
        float lv[8];
        uint32_t key[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          lv[e] = -INFINITY;
          key[e] = 0u;
          const int j = tid * E + e;
          if (e < E && j < CS) {
            const float raw = bf2f(reinterpret_cast<const bf16_t*>(lgw)[j]);
            lv[e] = sample_value(raw, bias, j, nullptr, 1.0f, div);
            key[e] = float_key(bias ? lv[e] : raw);
          }
        }
        __syncthreads();  // every thread holds its logits: the staging words go back to zero (the spare row must
        for (int i = tid; i < CS / 2; i += FR_THREADS) lgw[i] = 0u;  // read as zero, the others are rewritten by the next norm)
        const int code = block_sample<8>(lv, key, bias ? 0 : 16, CS, E, greedy, s_topk, rnd, (uint32_t)t, ssh, (int*)red);
        if (tid == 0) {
          ll_st(cb + b, (uint32_t)code, ep);
          a.codes_out[(size_t)b * a.codes_stride + t] = code;
        }
      }
      codebuf = cb;
    }
    RB_TS();
  }
#ifdef VUI_RB_CLOCK
  if (a.dbg && wg == a.dbg_wg && tid == 0) { for (int i = 0; i < dbg_n; ++i) a.dbg[i] = dbg_ts[i]; a.dbg[63] = dbg_n; }
#endif
  __syncthreads();
  if (active && wl < Bg && a.zero_pad)
    for (int q = a.n_q + tid; q < a.codes_stride; q += FR_THREADS) a.codes_out[(size_t)(b0 + wl) * a.codes_stride + q] = 0;
  if (wg == 0 && tid == 0) ctl_finish(c, a.epoch, a.arrive, (uint32_t)nwg);
}

// ---------------------------------------------------------------------------------------------
static int rb_xs(const vui_config& c) {
  int k = c.d_model;
  if (c.rq_dim > k) k = c.rq_dim;
  if (c.rq_ffn > k) k = c.rq_ffn;
  return k / 2 + 4;
}
struct RbLayout { size_t xp, red, misc, att, kv, total; };
static RbLayout rb_layout(const vui_config& c) {
  RbLayout l;
  size_t off = (size_t)RB_RG * c.rq_dim * 4;
  l.xp = off; off += (size_t)(RB_RG + 1) * rb_xs(c) * 4;
  l.red = off; off += 2 * 4 * 64 * 8 * 4;  // two tiles' partial sums
  l.misc = off; off += 64 + 512;
  l.att = off; off += 512 + 256;
  l.kv = off;
  const size_t rhd = c.rq_dim / c.rq_heads, qp8 = (c.n_quantizers + 7) & ~7;
  off += (size_t)c.rq_layers * 2 * rhd * qp8 * 2;
  l.total = (off + 15) & ~(size_t)15;
  return l;
}

size_t rq_batch_ll_words(const vui_config& c) {
  const size_t R = c.rq_dim, B = VUI_MAX_BATCH;
  const size_t layer = 3 * R / 2 + R / 2 + R / 2 + c.rq_ffn / 2 + R / 2;
  return B * (R / 2 + (size_t)c.n_quantizers * (layer * c.rq_layers + c.codebook_size / 2)) + 16 * (size_t)c.n_quantizers + 64;
}
size_t rq_batch_lds_bytes(const vui_config& c) { return rb_layout(c).total; }

bool rq_batch_supported(const vui_config& c, int nwg, char* why, size_t why_len) {
  const char* r = nullptr;
  const int R = c.rq_dim, rhd = c.rq_heads ? R / c.rq_heads : 0;
  if (c.dtype != VUI_DTYPE_BF16) r = "bf16 only";
  else if (c.rq_layers < 1) r = "no depth head";
  else if ((R % 32) || (c.rq_ffn % 32) || (c.d_model % 32)) r = "rq_dim, rq_ffn and d_model must be multiples of 32";
  else if (R > 1024 || c.d_model > 1024 || c.rq_ffn > 2048) r = "vector longer than the register tile";
  else if ((c.codebook_size % 16) || c.codebook_size > 2048) r = "codebook_size must be a multiple of 16, at most 2048";
  else if ((rhd & 1) || rhd > 128 || rhd * c.rq_heads != R) r = "depth-head head_dim must be even, at most 128";
  else if (c.n_quantizers > 64) r = "too many codebooks";
  else if (rq_batch_lds_bytes(c) > 160 * 1024) r = "activations of 16 rows do not fit in LDS";
  else {
    int nT = c.rq_ffn / 16;  // two tiles per workgroup of W1/W3 and of a codebook head, three of QKV
    if (c.codebook_size / 16 > nT) nT = c.codebook_size / 16;
    if (nT > 2 * RB_NWL || 3 * R / 16 > 3 * RB_NWL || R / 16 > RB_NWL || RB_RG * c.rq_heads > RB_NWL) r = "more tiles than a row group's workgroups take";
    if (nwg < RB_NWL * ((VUI_MAX_BATCH + RB_RG - 1) / RB_RG)) r = "too few workgroups for the row groups";
    if (c.codebook_size / 2 > RB_RG * (rb_xs(c))) r = "codebook longer than the staging area";
    if ((size_t)VUI_MAX_BATCH * (c.rq_ffn / 2) >= 65536) r = "exchange vector too long";
  }
  if (r && why) snprintf(why, why_len, "%s", r);
  return r == nullptr;
}

// elements of the matrices the kernel multiplies by: the layers, the codebook heads, the hidden-state projection
static size_t rb_weight_elems(const vui_config& c) {
  const size_t R = c.rq_dim, F = c.rq_ffn, d = c.d_model;
  return (size_t)c.rq_layers * (3 * R * R + R * R + 3 * F * R) + (size_t)(c.n_quantizers - 1) * c.codebook_size * R + (R != d ? R * d : 0);
}
size_t rq_batch_weight_bytes(const vui_config& c, int nwg) {
  return rq_batch_supported(c, nwg, nullptr, 0) ? rb_weight_elems(c) * 2 : 0;
}
// One-time: the tiled copies into dst; *tiled = w with those matrices' pointers replaced by the copies'.
int rq_batch_tile_weights(const vui_config& c, const vui_weights& w, void* dst, vui_weights* tiled, hipStream_t st) {
  const size_t R = c.rq_dim, F = c.rq_ffn, d = c.d_model;
  bf16_t* o = (bf16_t*)dst;
  *tiled = w;
  auto tile = [&](const void* src, size_t N, size_t K) -> const void* {
    const size_t pieces = N * (K / 8);
    hipLaunchKernelGGL(rb_tile_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, st, (const bf16_t*)src, o, N, (int)K);
    const void* r = o;
    o += N * K;
    return r;
  };
  for (int l = 0; l < c.rq_layers; ++l) {
    const vui_rq_layer_weights& L = w.rq_layers[l];
    vui_rq_layer_weights& T = tiled->rq_layers[l];
    T.wqkv = tile(L.wqkv, 3 * R, R);
    T.wo = tile(L.wo, R, R);
    T.w1 = tile(L.w1, F, R);
    T.w3 = tile(L.w3, F, R);
    T.w2 = tile(L.w2, R, F);
  }
  tiled->rq_head_w = tile(w.rq_head_w, (size_t)(c.n_quantizers - 1) * c.codebook_size, R);
  if (R != d && w.rq_backbone_proj) tiled->rq_backbone_proj = tile(w.rq_backbone_proj, R, d);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

int rq_batch_max_resident(size_t lds_bytes) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, dev));
  static size_t lds_attr = 0;
  if (lds_bytes > lds_attr) {
    HIP_TRY(hipFuncSetAttribute((const void*)rq_batch_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    HIP_TRY(hipFuncSetAttribute((const void*)rq_batch_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    lds_attr = lds_bytes;
  }
  int occ = 0, occ3 = 0;
  HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, rq_batch_kernel<false>, FR_THREADS, lds_bytes));
  HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ3, rq_batch_kernel<true>, FR_THREADS, lds_bytes));
  return (occ < occ3 ? occ : occ3) * prop.multiProcessorCount;
}

#ifdef VUI_RB_CLOCK
// profiling builds only: where the next launches drop the phase stamps of workgroup wg
static unsigned long long* g_rb_dbg = nullptr;
static int g_rb_dbg_wg = 0;
extern "C" void vui_debug_rq_batch_clock(unsigned long long* buf, int wg) { g_rb_dbg = buf; g_rb_dbg_wg = wg; }
#endif

int launch_rq_batch(const vui_config& c, const vui_weights* wdev, const void* hidden, const int64_t* code0, const float* logit_bias,
                    int n_q, float temp, int topk, uint64_t seed, const vui_sample_dev* sdev, const int32_t* frame_ctr, int64_t* codes_out,
                    int codes_stride, int zero_pad, int B, uint64_t* ll, uint32_t* ctl, int nwg, hipStream_t st) {
  RqBatchArgs a;
  memset(&a, 0, sizeof(a));
  a.B = B; a.d = c.d_model; a.R = c.rq_dim; a.rqH = c.rq_heads; a.rqF = c.rq_ffn; a.rqL = c.rq_layers; a.Q = c.n_quantizers;
  a.CS = c.codebook_size; a.n_q = n_q; a.rq_eps = c.rq_norm_eps; a.w = wdev; a.hidden = (const uint16_t*)hidden; a.code0 = code0;
  a.codes_out = codes_out; a.codes_stride = codes_stride; a.zero_pad = zero_pad; a.logit_bias = logit_bias; a.temp = temp;
  a.topk = topk; a.seed = seed; a.sdev = sdev; a.frame_ctr = frame_ctr; a.ll = ll; a.epoch = ctl; a.arrive = ctl + 1; a.err = ctl + 2;
#ifdef VUI_RB_CLOCK
  a.dbg = g_rb_dbg; a.dbg_wg = g_rb_dbg_wg;
#else
  a.dbg = nullptr; a.dbg_wg = 0;
#endif
  const RbLayout l = rb_layout(c);
  a.xs = rb_xs(c); a.off_xp = (int)l.xp; a.off_red = (int)l.red; a.off_misc = (int)l.misc; a.off_att = (int)l.att; a.off_kv = (int)l.kv;
  if (3 * c.rq_dim / 16 > 2 * RB_NWL) hipLaunchKernelGGL(rq_batch_kernel<true>, dim3(nwg), dim3(FR_THREADS), l.total, st, a);
  else hipLaunchKernelGGL(rq_batch_kernel<false>, dim3(nwg), dim3(FR_THREADS), l.total, st, a);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}
