// Streaming vocoder frame step: codes of one codec frame -> hop audio samples, fp32.
//
// Reference: QwenCodecDecoder.forward in streaming mode (src/vui/qwen_codec.py:1191-1224) with its
// building blocks CausalConv1d (:45-101), CausalTransConv1d (:112-158), SplitResidualVQ.decode (:263-270),
// DecTransformer._forward_streaming (:1048-1076), ConvNeXtBlock (:832-848), DecoderBlock (:863-879),
// SnakeBeta (:820-829).
//
// Layout.  Activations are channel-major (C, columns).  Every conv input lives in a ring of 2^k columns
// per channel that keeps the last `pad` columns of earlier frames in front of the current ones: frame f
// occupies columns (f*T + pad + t) mod 2^k, so no history is ever copied; a device counter holds f.
// The activation that precedes a conv (snake) is applied by the producer's epilogue, which writes the
// raw value (for residuals) and the activated value (into the consumer's ring) in one pass.
//
// One GEMM kernel serves every conv, transposed conv and linear layer: out (M x T) = W (M x taps*Cin) .
// X, X[(tap, ci)][t] = ring[ci][t + tap*dil].  Weights are repacked once to tap-major (taps, M, Cin) so a
// lane reads 32 contiguous bytes of one output row; a transposed conv with kernel 2*stride is the
// two-tap conv over (previous column, current column) with M = Cout*stride rows whose results are
// scattered to column t*stride + r.  A workgroup owns 16 output rows x 16*TT columns; its waves split
// the (tap, 32-channel) units, multiply on v_mfma_f32_16x16x4_f32 with both operands read straight from
// global memory / L2 one step ahead, and add their parts through LDS in a fixed order.
#include "common.h"
#include "internal.h"
#include "../../include/vui_codec.h"

#include <math.h>
#include <new>
#include <stdio.h>
#include <string.h>
#include <vector>

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

struct Ring {
  float* p;
  int rs;     // columns per channel (power of two)
  int mask;   // rs - 1
  int pad;    // history columns in front of a frame
  int tstep;  // columns a frame adds (0: plain buffer, always at column 0)
};

__device__ __forceinline__ int ring_base(const Ring& r, int f) { return (f * r.tstep) & r.mask; }
__device__ __forceinline__ float* ring_ptr(const Ring& r, int base, int c, int col) {
  return r.p + (size_t)c * r.rs + ((base + col) & r.mask);
}

// IN_RMS: the input column is RMS-normalised; the norm weight is folded into W when it is packed and
// 1/rms multiplies the sums.  EPI_SILU_PAIR: rows (2i, 2i+1) hold gate_i and up_i; channel i = silu(gate) * up.
enum { IN_PLAIN = 0, IN_RMS = 1 };
enum { EPI_NONE = 0, EPI_GELU = 1, EPI_RES = 2, EPI_SCALE_RES = 3, EPI_SILU_PAIR = 4 };

struct CvGemm {
  const float* W;     // (taps, M, Cin)
  const float* bias;  // row m uses bias[m / bias_div]; may be null
  int M, Cin, taps, dil, T;
  int bias_div;
  Ring in;
  int in_mode;
  float eps;
  int epi;
  const float* scale;  // per output channel (EPI_SCALE_RES)
  Ring res;
  int tc_stride;  // > 0: row m -> channel m / s, column t*s + m % s
  Ring out_raw;   // p may be null
  Ring out_act;   // p may be null: snake with (ea, ib) of the consumer
  const float* ea;
  const float* ib;
  const int* ctr;  // frames started; this frame is *ctr - 1
  int splits;      // workgroups that share one tile's (tap, channel) units; > 1: parts meet in `part`
  float* part;     // (tiles, splits, TT*64*4) partial sums
  int* cnt;        // (tiles) arrival counters, zero between launches
  int tt;          // 16-column blocks per tile (host side: picks the instantiation)
};

// A vocoder that shares the GPU with other kernels (vui_codec_workgroups) reads its weights - 423 MB per frame, each
// byte once - with non-temporal loads, so that they pass through the caches without pushing out what those kernels
// read again and again.  On its own the vocoder is 4 % slower with the hint (636 against 610 us per frame), so a
// vocoder that owns the GPU does not use it.
typedef float cv_f32x4 __attribute__((ext_vector_type(4)));
template <bool NT> __device__ __forceinline__ float4 cv_ld_w(const float* p) {
  if constexpr (NT) {
    const cv_f32x4 v = __builtin_nontemporal_load((const __attribute__((address_space(1))) cv_f32x4*)p);
    float4 r;
    __builtin_memcpy(&r, &v, sizeof(r));
    return r;
  } else {
    return *reinterpret_cast<const float4*>(p);
  }
}

// units a wave keeps in registers per round: NU * (8 + 8*TT) VGPRs, twice that when the rounds are
// double-buffered (DB: for tiles whose waves need several rounds; one wave per SIMD).  Tiles that fit one
// round use the single-buffered form, which leaves room for two or three waves per SIMD.
template <int TT, bool DB> struct Nu { static constexpr int N = TT == 1 ? 8 : (TT == 2 ? (DB ? 5 : 6) : 3); };

#define CV_NW 4  // waves per workgroup

// One 16-row x 16*TT-column output tile.  `red` is CV_NW * TT * 64 * 4 floats of LDS.
template <int TT, bool DB, bool NT>
__device__ __forceinline__ void cv_gemm_tile(const CvGemm& p, const int m0, const int t0, float* red,
                                             const int tile, const int part_idx) {
  constexpr int NU = Nu<TT, DB>::N;
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int r16 = lane & 15, g = lane >> 4;
  const int G = p.Cin >> 5, Uall = p.taps * G;
  const int M = p.M, Cin = p.Cin;
  // this workgroup's share of the units, and in it this wave's contiguous run [ub, U): a wave walks along
  // its 16 weight rows, 128 bytes of each per unit
  const int per = (Uall + p.splits - 1) / p.splits;
  const int wb = part_idx * per, we = min(Uall, wb + per);
  const int per_wave = (we - wb + CV_NW - 1) / CV_NW;
  const int ub = min(we, wb + wave * per_wave), U = min(we, ub + per_wave);

  float4 a0[NU][2], a1[DB ? NU : 1][2];
  float b0[NU][TT][8], b1[DB ? NU : 1][TT][8];
  floatx4 acc[TT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) acc[tt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // request the operands of units u0, u0 + NW, ... (NU of them); nothing is waited for here.  The weights
  // do not depend on the frame counter, so the first round asks for them before the counter is needed.
  auto load_a = [&](int u0, auto& a) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int u = u0 + i;
      const bool on = u < U;
      const int tap = on ? u / G : 0, grp = on ? u - tap * G : 0;
      const float* wp = p.W + ((size_t)tap * M + m0 + r16) * Cin + grp * 32 + g * 8;
      if constexpr (NT) {
        a[i][0] = on ? cv_ld_w<true>(wp) : make_float4(0.f, 0.f, 0.f, 0.f);
        a[i][1] = on ? cv_ld_w<true>(wp + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
      } else {
        a[i][0] = on ? *reinterpret_cast<const float4*>(wp) : make_float4(0.f, 0.f, 0.f, 0.f);
        a[i][1] = on ? *reinterpret_cast<const float4*>(wp + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
  };
  int ib_ = 0;
  auto load_b = [&](int u0, auto& b) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int u = u0 + i;
      const bool on = u < U;
      const int tap = on ? u / G : 0, grp = on ? u - tap * G : 0;
      const int ci0 = grp * 32 + g * 8;
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        const int t = t0 + tt * 16 + r16;
        const bool bon = on && t < p.T;
        const float* xp = ring_ptr(p.in, ib_, bon ? ci0 : 0, bon ? t + tap * p.dil : 0);
#pragma unroll
        for (int j = 0; j < 8; ++j) b[i][tt][j] = bon ? xp[(size_t)j * p.in.rs] : 0.f;
      }
    }
  };
  auto load = [&](int u0, auto& a, auto& b) { load_a(u0, a); load_b(u0, b); };
  auto mma = [&](const auto& a, const auto& b) {
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const float av[8] = {a[i][0].x, a[i][0].y, a[i][0].z, a[i][0].w, a[i][1].x, a[i][1].y, a[i][1].z, a[i][1].w};
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt)
          acc[tt] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[j], b[i][tt][j], acc[tt], 0, 0, 0);
    }
  };

  constexpr int STEP = NU;
  load_a(ub, a0);
  const int f = *p.ctr - 1;
  ib_ = ring_base(p.in, f);
  load_b(ub, b0);
  // what the epilogue adds is requested now as well
  const int rb = ring_base(p.res, f), ob = ring_base(p.out_raw, f), ab = ring_base(p.out_act, f);
  float e_bias[4] = {0.f, 0.f, 0.f, 0.f}, e_res[4] = {0.f, 0.f, 0.f, 0.f}, e_sc[4] = {1.f, 1.f, 1.f, 1.f};
  float e_ea[4] = {0.f, 0.f, 0.f, 0.f}, e_ib[4] = {0.f, 0.f, 0.f, 0.f};
  if (tid < TT * 64) {
    const int t = t0 + (tid >> 6) * 16 + (tid & 15);
    if (t < p.T) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m0 + 4 * ((tid & 63) >> 4) + r;
        int ch = m, col = t;
        if (p.tc_stride > 0) { ch = m / p.tc_stride; col = t * p.tc_stride + m % p.tc_stride; }
        if (p.bias) e_bias[r] = p.bias[m / p.bias_div];
        if (p.epi == EPI_RES || p.epi == EPI_SCALE_RES) e_res[r] = *ring_ptr(p.res, rb, ch, p.res.pad + col);
        if (p.epi == EPI_SCALE_RES) e_sc[r] = p.scale[ch];
        if (p.out_act.p) { e_ea[r] = p.ea[ch]; e_ib[r] = p.ib[ch]; }
      }
    }
  }
  // 1/rms of the input column while the first operands are in flight; applied to the sums at the end
  float rstd = 1.f;
  if (p.in_mode == IN_RMS) {
    float ss = 0.f;
    for (int c = lane; c < Cin; c += WAVE) {
      const float v = *ring_ptr(p.in, ib_, c, p.in.pad);
      ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    rstd = 1.0f / sqrtf(ss / (float)Cin + p.eps);
  }
  if constexpr (DB) {
    for (int u0 = ub; u0 < U; u0 += 2 * STEP) {
      if (u0 + STEP < U) load(u0 + STEP, a1, b1);
      mma(a0, b0);
      if (u0 + STEP < U) {
        if (u0 + 2 * STEP < U) load(u0 + 2 * STEP, a0, b0);
        mma(a1, b1);
      }
    }
  } else {
    for (int u0 = ub; u0 < U; u0 += STEP) {
      if (u0 != ub) load(u0, a0, b0);
      mma(a0, b0);
    }
  }

  // add the waves' parts in a fixed order
#pragma unroll
  for (int tt = 0; tt < TT; ++tt)
    *reinterpret_cast<float4*>(red + ((size_t)(wave * TT + tt) * 64 + lane) * 4) =
        make_float4(acc[tt][0], acc[tt][1], acc[tt][2], acc[tt][3]);
  __syncthreads();
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (tid < TT * 64) {
#pragma unroll
    for (int w = 0; w < CV_NW; ++w) {
      const float4 q = *reinterpret_cast<const float4*>(red + ((size_t)w * TT * 64 + tid) * 4);
      v[0] += q.x; v[1] += q.y; v[2] += q.z; v[3] += q.w;
    }
  }
  if (p.splits > 1) {
    // parts of a tile meet in memory; the workgroup that arrives last adds them in part order and finishes
    __shared__ int last;
    float* mine = p.part + (((size_t)tile * p.splits + part_idx) * TT * 64 + tid) * 4;
    if (tid < TT * 64) { st_dev(mine, v[0], v[1]); st_dev(mine + 2, v[2], v[3]); }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the write-through stores have completed
    __syncthreads();
    if (tid == 0) {
      const int old = __hip_atomic_fetch_add(p.cnt + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      last = old == p.splits - 1;
      if (last) __hip_atomic_store(p.cnt + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!last) return;
    if (tid < TT * 64) {
      uint64_t q[8][2];
#pragma unroll
      for (int z = 0; z < 8; ++z) {
        const float* src = p.part + (((size_t)tile * p.splits + z) * TT * 64 + tid) * 4;
        q[z][0] = z < p.splits ? ld_dev(src) : 0;
        q[z][1] = z < p.splits ? ld_dev(src + 2) : 0;
      }
      v[0] = v[1] = v[2] = v[3] = 0.f;
#pragma unroll
      for (int z = 0; z < 8; ++z) {
        v[0] += __uint_as_float((uint32_t)q[z][0]); v[1] += __uint_as_float((uint32_t)(q[z][0] >> 32));
        v[2] += __uint_as_float((uint32_t)q[z][1]); v[3] += __uint_as_float((uint32_t)(q[z][1] >> 32));
      }
    }
  }
  if (tid < TT * 64) {
    const int tt = tid >> 6, l = tid & 63;
    const int t = t0 + tt * 16 + (l & 15);
    if (t >= p.T) return;
    if (p.epi == EPI_SILU_PAIR) {  // one column per frame
#pragma unroll
      for (int r = 0; r < 4; r += 2) {
        const float ga = v[r] * rstd, up = v[r + 1] * rstd;
        *ring_ptr(p.out_raw, ob, (m0 + 4 * (l >> 4) + r) >> 1, p.out_raw.pad + t) = ga / (1.0f + expf(-ga)) * up;
      }
      return;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + 4 * (l >> 4) + r;
      float y = v[r] * rstd + e_bias[r];
      int ch = m, col = t;
      if (p.tc_stride > 0) { ch = m / p.tc_stride; col = t * p.tc_stride + m % p.tc_stride; }
      if (p.epi == EPI_GELU) y = 0.5f * y * (1.0f + erff(y * 0.70710678118654752f));
      else if (p.epi == EPI_RES) y = e_res[r] + y;
      else if (p.epi == EPI_SCALE_RES) y = e_res[r] + e_sc[r] * y;
      if (p.out_raw.p) *ring_ptr(p.out_raw, ob, ch, p.out_raw.pad + col) = y;
      if (p.out_act.p) {
        const float s = sinf(y * e_ea[r]);
        *ring_ptr(p.out_act, ab, ch, p.out_act.pad + col) = y + e_ib[r] * s * s;
      }
    }
  }
}

template <int TT, bool NT>
__global__ __launch_bounds__(CV_NW * 64) void cv_gemm_kernel(const CvGemm p) {
  __shared__ __align__(16) float red[CV_NW * TT * 64 * 4];
  cv_gemm_tile<TT, true, NT>(p, blockIdx.x * 16, blockIdx.y * (16 * TT), red, blockIdx.y * gridDim.x + blockIdx.x, blockIdx.z);
}
template <int TT, bool NT>
__global__ __launch_bounds__(CV_NW * 64, 2) void cv_gemm1_kernel(const CvGemm p) {
  __shared__ __align__(16) float red[CV_NW * TT * 64 * 4];
  cv_gemm_tile<TT, false, NT>(p, blockIdx.x * 16, blockIdx.y * (16 * TT), red, blockIdx.y * gridDim.x + blockIdx.x, blockIdx.z);
}

// ---- codebook rows of one frame: [sum of the semantic rows | sum of the acoustic rows]; starts the frame ----
struct CvVq {
  const int64_t* codes;
  int n_q, n_sem, CS, cd;
  const float* embed;  // (n_codebooks, CS, cd)
  float* x;            // (2*cd) as a one-column plain buffer with rs = 1
  int* ctr;
  int* err;
  int max_seq;
};

__global__ __launch_bounds__(256) void cv_vq_kernel(const CvVq p) {
  for (int c = threadIdx.x; c < p.cd; c += blockDim.x) {
    float s0 = 0.f, s1 = 0.f;
    for (int i0 = 0; i0 < p.n_q; i0 += 16) {  // 16 codes, then their 16 rows, are requested together
      long code[16];
      float e[16];
#pragma unroll
      for (int k = 0; k < 16; ++k) code[k] = i0 + k < p.n_q ? p.codes[i0 + k] : 0;
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        if (code[k] < 0 || code[k] >= p.CS) { code[k] = code[k] < 0 ? 0 : p.CS - 1; if (c == 0) *p.err = 1; }
        e[k] = i0 + k < p.n_q ? p.embed[((size_t)(i0 + k) * p.CS + code[k]) * p.cd + c] : 0.f;
      }
#pragma unroll
      for (int k = 0; k < 16; ++k) {  // the reference's order: codebook after codebook
        if (i0 + k < p.n_sem) s0 += e[k]; else s1 += e[k];
      }
    }
    p.x[c] = s0;
    p.x[p.cd + c] = s1;
  }
  if (threadIdx.x == 0) {
    int f = *p.ctr;
    if (f >= p.max_seq) { *p.err = 2; f = p.max_seq - 1; }  // stay on the last position: nothing runs out of bounds
    *p.ctr = f + 1;
  }
}

// ---- pre-transformer attention of one new position: rotate-half RoPE, cache append, softmax, P.V ----
struct CvAttn {
  const float* qkv;  // (3*A): q | k | v
  float* kc;         // (H, max_seq, hd)
  float* vc;
  float* out;        // (A)
  const float* inv_freq;  // (hd/2)
  int H, hd, max_seq;
  const int* ctr;
};

__global__ __launch_bounds__(256) void cv_attn_kernel(const CvAttn p) {
  extern __shared__ float sm[];  // q[hd] | sc[max_seq] | part[4][hd] | red[8]
  float* q = sm;
  float* sc = q + p.hd;
  float* part = sc + p.max_seq;
  float* red = part + 4 * p.hd;
  const int h = blockIdx.x, tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int hd = p.hd, half = hd >> 1, A = p.H * hd;
  const int pos = *p.ctr - 1;
  float* kh = p.kc + (size_t)h * p.max_seq * hd;
  float* vh = p.vc + (size_t)h * p.max_seq * hd;
  if (tid < hd) {
    const float ang = (float)pos * p.inv_freq[tid % half];
    const float cs = cosf(ang), sn = sinf(ang);
    const float* qq = p.qkv + h * hd;
    const float* kk = p.qkv + A + h * hd;
    const float qr = tid < half ? -qq[tid + half] : qq[tid - half];
    const float kr = tid < half ? -kk[tid + half] : kk[tid - half];
    q[tid] = qq[tid] * cs + qr * sn;
    kh[(size_t)pos * hd + tid] = kk[tid] * cs + kr * sn;
    vh[(size_t)pos * hd + tid] = p.qkv[2 * A + h * hd + tid];
  }
  __syncthreads();  // this workgroup's own cache row is visible to all its threads after the barrier
  // scores: a group of 16 lanes per key (features l16, l16 + 16, ...), four keys of a group in flight
  const float scale = 1.0f / sqrtf((float)hd);
  const int grp = tid >> 4, l16 = tid & 15, E = hd >> 4;
  float qe[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) qe[e] = e < E ? q[l16 + 16 * e] : 0.f;
  for (int j0 = grp; j0 <= pos; j0 += 64) {
    float kv[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + 16 * u;
#pragma unroll
      for (int e = 0; e < 4; ++e) kv[u][e] = (j <= pos && e < E) ? kh[(size_t)j * hd + l16 + 16 * e] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + 16 * u;
      float d = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) d = fmaf(qe[e], kv[u][e], d);
      d = group16_sum(d);
      if (l16 == 0 && j <= pos) sc[j] = d * scale;
    }
  }
  __syncthreads();
  float mx = -INFINITY;
  for (int j = tid; j <= pos; j += 256) mx = fmaxf(mx, sc[j]);
  mx = wave_max(mx);
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  float sum = 0.f;
  for (int j = tid; j <= pos; j += 256) { const float e = expf(sc[j] - mx); sc[j] = e; sum += e; }
  sum = wave_sum(sum);
  if (lane == 0) red[4 + wave] = sum;
  __syncthreads();
  sum = (red[4] + red[5]) + (red[6] + red[7]);
  // P.V: wave w takes keys w, w + 4, ...; eight rows in flight
  float o = 0.f;
  if (lane < hd) {
    for (int j0 = wave; j0 <= pos; j0 += 32) {
      float vv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) { const int j = j0 + 4 * u; vv[u] = j <= pos ? vh[(size_t)j * hd + lane] : 0.f; }
#pragma unroll
      for (int u = 0; u < 8; ++u) { const int j = j0 + 4 * u; o = fmaf(j <= pos ? sc[j] : 0.f, vv[u], o); }
    }
    part[wave * hd + lane] = o;
  }
  __syncthreads();
  if (tid < hd) p.out[h * hd + tid] = ((part[tid] + part[hd + tid]) + (part[2 * hd + tid] + part[3 * hd + tid])) / sum;
}

// =============================================================================================
// The one-column trunk as ONE persistent kernel: codebook rows -> quantizer projection -> pre_conv
// -> input_proj -> the transformer layers -> output_proj -> first upsampling transposed conv.
// These 46 steps have one column each (1-3 MB of weights), so as separate launches they run at the
// cost of a dependent launch.  Here 256 workgroups (one per CU) walk the same list of phases; every
// workgroup owns a few rows of every matrix, keeps the residual stream and the current input vector
// in LDS, requests the weights of the next phase before it waits, and passes results as 8-byte
// words = fp32 payload + launch epoch (device-scope relaxed atomics: a word showing the epoch is the
// data).  Exchange buffers are never reused inside a launch.  Every wait is bounded.
// =============================================================================================
#include "ll.h"

struct TrunkLayer {
  const float* Wqkv; const float* Wo; const float* asc; const float* Wgu; const float* Wd; const float* msc;
  float* kc; float* vc;
};

struct CvTrunk {
  const int64_t* codes;
  int n_q, n_sem, CS, cd;
  const float* embed;
  int* ctr;
  int* err;
  int max_seq;
  const float* Wvq; int vq_dim;
  const float* Wpre; const float* bpre; int L;
  Ring pre_in;
  const float* Win; const float* bin; int D;
  int n_layers, H, hd, mlp;
  const TrunkLayer* layers;
  const float* inv_freq;
  const float* Wout; const float* bout;
  const float* Wt0; const float* bt0; int r0;  // Wt0 == nullptr: no upsampling stage, `out` takes the latent
  Ring out;
  uint64_t* ll;
  uint32_t* epoch; uint32_t* arrive; uint32_t* lerr;
  float eps;
};

#define TR_MAXC 6   // float4 chunks per lane and row: K <= 1536
#define TR_REGS 24  // float4 registers of a wave's rows of one phase: rows per wave x chunks per row

// Rows per wave, phase by phase.  The kernel is built for a whole GPU (256 workgroups) and for the share of one that a
// caller leaves to the vocoder beside other work (NARROW: 96 workgroups and more): a workgroup then owns 256 / 96
// times the rows, and every phase keeps its rows x chunks within TR_REGS registers.
template <bool NARROW> struct TrPlan {
  static constexpr int VQ = NARROW ? 2 : 1, PRE = NARROW ? 3 : 1, IN = NARROW ? 2 : 1, QKV = NARROW ? 10 : 4, O = NARROW ? 2 : 1,
                       GU = NARROW ? 6 : 4, DN = NARROW ? 2 : 1, OUT = NARROW ? 3 : 1, UP = NARROW ? 6 : 4;
};

struct TrRows { float4 w[TR_REGS]; };

// rows r_lo + wave, r_lo + wave + 4, ... below r_hi of W (M x K): request them
template <int MAXR, int MAXC>
__device__ __forceinline__ void tr_prefetch(const float* W, int K, int r_lo, int r_hi, TrRows& rr) {
  static_assert(MAXR * MAXC <= TR_REGS, "rows x chunks of a phase exceed the wave's registers");
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int row = r_lo + wave + 4 * i;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
      const int k = (lane + 64 * c) * 4;
      const bool on = row < r_hi && k < K;
      rr.w[i * MAXC + c] = on ? *reinterpret_cast<const float4*>(W + (size_t)row * K + k) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
}
// dot products of those rows with xs (K floats in LDS); epi(row, sum) runs in every lane of the wave
template <int MAXR, int MAXC, typename F>
__device__ __forceinline__ void tr_compute(const float* xs, int K, int r_lo, int r_hi, const TrRows& rr, F&& epi) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int row = r_lo + wave + 4 * i;
    if (row < r_hi) {
      float s = 0.f;
#pragma unroll
      for (int c = 0; c < MAXC; ++c) {
        const int k = (lane + 64 * c) * 4;
        if (k < K) {
          const float4 x = *reinterpret_cast<const float4*>(xs + k);
          const float4 w = rr.w[i * MAXC + c];
          s = fmaf(w.x, x.x, s); s = fmaf(w.y, x.y, s);
          s = fmaf(w.z, x.z, s); s = fmaf(w.w, x.w, s);
        }
      }
      s = wave_sum(s);
      epi(row, s);
    }
  }
}

__device__ __forceinline__ void tr_rows(int M, int wg, int nwg, int& lo, int& hi) {
  const int per = (M + nwg - 1) / nwg;
  lo = min(M, wg * per);
  hi = min(M, lo + per);
}

// q/k/v rows: the head-owning workgroups (the first H) stay out of this phase when enough others exist; they
// use the time to fetch their key / value history
__device__ __forceinline__ void tr_rows_qkv(int M, int wg, int nwg, int H, int& lo, int& hi) {
  if (nwg >= 4 * H) {
    if (wg < H) { lo = hi = M; return; }
    tr_rows(M, wg - H, nwg - H, lo, hi);
  } else {
    tr_rows(M, wg, nwg, lo, hi);
  }
}

__device__ __forceinline__ float tr_rstd(const float* x, int n, float eps, float* red) {
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  float ss = 0.f;
  for (int i = tid; i < n; i += FR_THREADS) ss = fmaf(x[i], x[i], ss);
  ss = wave_sum(ss);
  __syncthreads();
  if (lane == 0) red[wave] = ss;
  __syncthreads();
  return 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)n + eps);
}

template <bool NARROW>
__global__ __launch_bounds__(FR_THREADS) void cv_trunk_kernel(const CvTrunk a) {
  typedef TrPlan<NARROW> P;
  extern __shared__ __align__(16) float tsm[];
  // xs: current input vector (<= 1536) | x: residual stream (D) | q (hd) | sc (max_seq) | part (4*hd) | red (16)
  float* xs = tsm;
  float* x = xs + 1536;
  float* q = x + a.D;
  float* sc = q + 64;  // max_seq + 192: scores, and before them the raw q | k | v of the head
  float* part = sc + a.max_seq + 192;
  float* red = part + 4 * 64;
  const int wg = blockIdx.x, nwg = gridDim.x, tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  Ctl c;
  ctl_begin(c, a.epoch, a.lerr);
  const uint32_t ep = c.epoch;
  int f = *a.ctr;
  const bool over = f >= a.max_seq;
  if (over) f = a.max_seq - 1;  // stay on the last position: nothing runs out of bounds
  // the epoch and the frame counter have been read before this workgroup reports its arrival
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  if (tid == 0) __hip_atomic_fetch_add(a.arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  uint64_t* ll = a.ll;
  auto take = [&](int n) { uint64_t* p = ll; ll += n; return p; };
  auto put = [&](uint64_t* buf, int i, float v) { ll_st(buf + i, __float_as_uint(v), ep); };
  auto get = [&](const uint64_t* buf, int n, float* dst) {
    ll_poll_auto(buf, n, c, [&](int i, uint32_t v) { dst[i] = __uint_as_float(v); });
    __syncthreads();
  };
  TrRows rr;
  int lo, hi;
  const int cd = a.cd, V = a.vq_dim, L = a.L, D = a.D, A = a.H * a.hd, hd = a.hd, mlp = a.mlp;

  // ---- quantizer projection: rows of [W_sem | W_ac] against [sum of semantic rows | sum of acoustic rows] ----
  tr_rows(V, wg, nwg, lo, hi);
  tr_prefetch<P::VQ, 2>(a.Wvq, 2 * cd, lo, hi, rr);
  for (int ch = tid; ch < cd; ch += FR_THREADS) {  // every workgroup sums the codebook rows itself
    float s0 = 0.f, s1 = 0.f;
    for (int i0 = 0; i0 < a.n_q; i0 += 16) {
      long code[16];
      float e[16];
#pragma unroll
      for (int k = 0; k < 16; ++k) code[k] = i0 + k < a.n_q ? a.codes[i0 + k] : 0;
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        if (code[k] < 0 || code[k] >= a.CS) { code[k] = code[k] < 0 ? 0 : a.CS - 1; if (ch == 0 && wg == 0) *a.err = 1; }
        e[k] = i0 + k < a.n_q ? a.embed[((size_t)(i0 + k) * a.CS + code[k]) * cd + ch] : 0.f;
      }
#pragma unroll
      for (int k = 0; k < 16; ++k) { if (i0 + k < a.n_sem) s0 += e[k]; else s1 += e[k]; }
    }
    xs[ch] = s0;
    xs[cd + ch] = s1;
  }
  __syncthreads();
  uint64_t* b_y1 = take(V);
  const int pbase = ring_base(a.pre_in, f);
  tr_compute<P::VQ, 2>(xs, 2 * cd, lo, hi, rr, [&](int row, float s) {
    if (lane == 0) { put(b_y1, row, s); *ring_ptr(a.pre_in, pbase, row, a.pre_in.pad) = s; }
  });
  // ---- pre_conv: three taps = the two previous frames' columns and this one ----
  tr_rows(L, wg, nwg, lo, hi);
#pragma unroll
  for (int i = 0; i < P::PRE; ++i) {
    const int wave_row = lo + wave + 4 * i;  // (3, L, V) tap-major
#pragma unroll
    for (int cc = 0; cc < TR_MAXC; ++cc) {
      const int k = (lane + 64 * cc) * 4;  // index into [tap][ci]
      const int tap = k / V, ci = k - tap * V;
      const bool on = wave_row < hi && k < 3 * V;
      rr.w[i * TR_MAXC + cc] = on ? *reinterpret_cast<const float4*>(a.Wpre + ((size_t)tap * L + wave_row) * V + ci) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
  __syncthreads();  // xs is free again
  for (int i = tid; i < 2 * V; i += FR_THREADS) xs[i] = *ring_ptr(a.pre_in, pbase, i % V, i / V);
  ll_poll_auto(b_y1, V, c, [&](int i, uint32_t v) { xs[2 * V + i] = __uint_as_float(v); });
  __syncthreads();
  uint64_t* b_pre = take(L);
  tr_compute<P::PRE, TR_MAXC>(xs, 3 * V, lo, hi, rr, [&](int row, float s) { if (lane == 0) put(b_pre, row, s + a.bpre[row]); });
  // ---- input_proj ----
  tr_rows(D, wg, nwg, lo, hi);
  tr_prefetch<P::IN, 4>(a.Win, L, lo, hi, rr);
  __syncthreads();
  get(b_pre, L, xs);
  uint64_t* b_x = take(D);
  tr_compute<P::IN, 4>(xs, L, lo, hi, rr, [&](int row, float s) { if (lane == 0) put(b_x, row, s + a.bin[row]); });
  {
    int qlo, qhi;
    tr_rows_qkv(3 * A, wg, nwg, a.H, qlo, qhi);
    tr_prefetch<P::QKV, 2>(a.layers[0].Wqkv, D, qlo, qhi, rr);
  }
  get(b_x, D, x);

  const float att_scale = 1.0f / sqrtf((float)hd);
  // rotation of this position: the same for every layer, computed once and before any q arrives
  float rope_cs = 1.f, rope_sn = 0.f;
  if (wg < a.H && tid < hd) {
    const float ang = (float)f * a.inv_freq[tid % (hd >> 1)];
    rope_cs = cosf(ang);
    rope_sn = sinf(ang);
  }
  for (int l = 0; l < a.n_layers; ++l) {
    const TrunkLayer& W = a.layers[l];
    // The head's workgroup asks for its whole key / value history now (at most 256 earlier positions: 16 per
    // lane group, 4 features per lane), long before the new q arrives: attention then runs from registers,
    // whatever the position.
    float kreg[16][4], vreg[16][4];
    if (wg < a.H) {
      const float* kh = W.kc + (size_t)wg * a.max_seq * hd;
      const float* vh = W.vc + (size_t)wg * a.max_seq * hd;
      const int g16 = tid >> 4, c16 = tid & 15, E = hd >> 4;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = g16 + 16 * i;
#pragma unroll
        for (int e = 0; e < 4; ++e) { kreg[i][e] = 0.f; vreg[i][e] = 0.f; }
        if (16 * i < f) {  // uniform: blocks of 16 positions that do not exist yet cost nothing
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const bool on = j < f && e < E;
            kreg[i][e] = on ? kh[(size_t)j * hd + c16 + 16 * e] : 0.f;
            vreg[i][e] = on ? vh[(size_t)j * hd + c16 + 16 * e] : 0.f;
          }
        }
      }
    }
    // ---- q, k, v rows (norm weight folded in; 1/rms multiplies the sums) ----
    const float r1 = tr_rstd(x, D, a.eps, red);
    tr_rows_qkv(3 * A, wg, nwg, a.H, lo, hi);
    uint64_t* b_qkv = take(3 * A);
    tr_compute<P::QKV, 2>(x, D, lo, hi, rr, [&](int row, float s) { if (lane == 0) put(b_qkv, row, s * r1); });
    uint64_t* b_att = take(A);
    int olo, ohi;
    tr_rows(D, wg, nwg, olo, ohi);
    tr_prefetch<P::O, 4>(W.Wo, A, olo, ohi, rr);
    // ---- attention: workgroup h owns head h ----
    if (wg < a.H) {
      const int h = wg, half = hd >> 1, pos = f;
      float* kh = W.kc + (size_t)h * a.max_seq * hd;
      float* vh = W.vc + (size_t)h * a.max_seq * hd;
      float* kvn = part;  // this position's rotated key | value
      __syncthreads();
      if (tid < 3 * hd) {
        const int which = tid / hd, i = tid - which * hd;
        const uint64_t* src = b_qkv + which * A + h * hd + i;
        uint64_t v = ll_ld(src);
        int spins = 0;
        while ((uint32_t)(v >> 32) != ep && !c.dead) {
          v = ll_ld(src);
          if (++spins > SPIN_LIMIT) { c.dead = 1; __hip_atomic_store(c.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
        }
        sc[which * hd + i] = __uint_as_float((uint32_t)v);  // raw q | k | v
      }
      __syncthreads();
      if (tid < hd) {
        const float cs = rope_cs, sn = rope_sn;
        const float* qq = sc;
        const float* kk = sc + hd;
        const float qr = tid < half ? -qq[tid + half] : qq[tid - half];
        const float kr = tid < half ? -kk[tid + half] : kk[tid - half];
        q[tid] = qq[tid] * cs + qr * sn;
        const float kn = kk[tid] * cs + kr * sn, vn = sc[2 * hd + tid];
        kvn[tid] = kn; kvn[hd + tid] = vn;
        kh[(size_t)pos * hd + tid] = kn;
        vh[(size_t)pos * hd + tid] = vn;
      }
      __syncthreads();
      const int grp = tid >> 4, l16 = tid & 15, E = hd >> 4;
      float qe[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) qe[e] = e < E ? q[l16 + 16 * e] : 0.f;
      __syncthreads();  // sc is rewritten below
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = grp + 16 * i;
        if (j <= pos) {  // uniform over the 16 lanes of a group
          float d = 0.f;
#pragma unroll
          for (int e = 0; e < 4; ++e) d = fmaf(qe[e], (j == pos && e < E) ? kvn[l16 + 16 * e] : kreg[i][e], d);
          d = group16_sum(d);
          if (l16 == 0) sc[j] = d * att_scale;
        }
      }
      __syncthreads();
      float mx = -INFINITY;
      for (int j = tid; j <= pos; j += FR_THREADS) mx = fmaxf(mx, sc[j]);
      mx = wave_max(mx);
      if (lane == 0) red[wave] = mx;
      __syncthreads();
      mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
      float sum = 0.f;
      for (int j = tid; j <= pos; j += FR_THREADS) { const float e = expf(sc[j] - mx); sc[j] = e; sum += e; }
      sum = wave_sum(sum);
      if (lane == 0) red[4 + wave] = sum;
      __syncthreads();
      sum = (red[4] + red[5]) + (red[6] + red[7]);
      // P.V per lane group over its own keys, then the 16 groups are added in order (xs is free here)
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int j = grp + 16 * i;
        if (j <= pos) {
          const float pj = sc[j];
#pragma unroll
          for (int e = 0; e < 4; ++e) o4[e] = fmaf(pj, (j == pos && e < E) ? kvn[hd + l16 + 16 * e] : vreg[i][e], o4[e]);
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) if (e < E) xs[grp * hd + l16 + 16 * e] = o4[e];
      __syncthreads();
      if (tid < hd) {
        float o = 0.f;
#pragma unroll
        for (int gg = 0; gg < 16; ++gg) o += xs[gg * hd + tid];
        part[tid] = o / sum;  // kvn (= part) has been read by everyone
      }
      __syncthreads();
      if (tid < hd) put(b_att, h * hd + tid, part[tid]);
    }
    // ---- out_proj, residual with per-channel scale ----
    // the scales of this thread's channels (tid, tid + 256, ...) are asked for ahead of the waits: fetched when
    // the sums arrive, their pointer and then their value would be two trips to memory on the critical path
    float asc_r[6], msc_r[6];  // d_model <= 1536
#pragma unroll
    for (int k = 0; k < 6; ++k) {
      const int i = tid + FR_THREADS * k;
      asc_r[k] = i < D ? W.asc[i] : 0.f;
      msc_r[k] = i < D ? W.msc[i] : 0.f;
    }
    get(b_att, A, xs);
    uint64_t* b_o = take(D);
    tr_compute<P::O, 4>(xs, A, olo, ohi, rr, [&](int row, float s) { if (lane == 0) put(b_o, row, s); });
    int glo, ghi;
    tr_rows(mlp, wg, nwg, glo, ghi);  // channels; rows 2i, 2i + 1 are gate_i, up_i
    glo *= 2; ghi *= 2;
    tr_prefetch<P::GU, 2>(W.Wgu, D, glo, ghi, rr);
    ll_poll_auto(b_o, D, c, [&](int i, uint32_t v) { x[i] += asc_r[i / FR_THREADS] * __uint_as_float(v); });
    // ---- gate / up rows interleaved: channel i = silu(gate_i) * up_i ----
    const float r2 = tr_rstd(x, D, a.eps, red);
    uint64_t* b_h = take(mlp);
    {
      // a wave's rows glo + wave + 4 i alternate between gate and up of different channels: pair through LDS
      float* pair = part;
      tr_compute<P::GU, 2>(x, D, glo, ghi, rr, [&](int row, float s) { if (lane == 0) pair[row - glo] = s * r2; });
      __syncthreads();
      for (int i = tid; 2 * i + 1 < ghi - glo; i += FR_THREADS) {
        const float ga = pair[2 * i], up = pair[2 * i + 1];
        put(b_h, (glo >> 1) + i, ga / (1.0f + expf(-ga)) * up);
      }
    }
    int dlo, dhi;
    tr_rows(D, wg, nwg, dlo, dhi);
    tr_prefetch<P::DN, 4>(W.Wd, mlp, dlo, dhi, rr);
    get(b_h, mlp, xs);
    uint64_t* b_d = take(D);
    tr_compute<P::DN, 4>(xs, mlp, dlo, dhi, rr, [&](int row, float s) { if (lane == 0) put(b_d, row, s); });
    if (l + 1 < a.n_layers) {
      int qlo, qhi;
      tr_rows_qkv(3 * A, wg, nwg, a.H, qlo, qhi);
      tr_prefetch<P::QKV, 2>(a.layers[l + 1].Wqkv, D, qlo, qhi, rr);
    } else {
      int plo, phi;
      tr_rows(L, wg, nwg, plo, phi);
      tr_prefetch<P::OUT, 2>(a.Wout, D, plo, phi, rr);
    }
    ll_poll_auto(b_d, D, c, [&](int i, uint32_t v) { x[i] += msc_r[i / FR_THREADS] * __uint_as_float(v); });
  }
  // ---- final norm (folded) + output_proj ----
  const float r3 = tr_rstd(x, D, a.eps, red);
  tr_rows(L, wg, nwg, lo, hi);
  const int obase = ring_base(a.out, f);
  if (a.Wt0 == nullptr) {
    tr_compute<P::OUT, 2>(x, D, lo, hi, rr, [&](int row, float s) {
      if (lane == 0) *ring_ptr(a.out, obase, row, a.out.pad) = s * r3 + a.bout[row];
    });
  } else {
    uint64_t* b_lat = take(L);
    tr_compute<P::OUT, 2>(x, D, lo, hi, rr, [&](int row, float s) { if (lane == 0) put(b_lat, row, s * r3 + a.bout[row]); });
    // ---- first upsampling stage: transposed conv with kernel = stride: row m -> channel m / r0, column m % r0 ----
    tr_rows(L * a.r0, wg, nwg, lo, hi);
    tr_prefetch<P::UP, 4>(a.Wt0, L, lo, hi, rr);
    __syncthreads();
    get(b_lat, L, xs);
    tr_compute<P::UP, 4>(xs, L, lo, hi, rr, [&](int row, float s) {
      if (lane == 0) *ring_ptr(a.out, obase, row / a.r0, a.out.pad + row % a.r0) = s + a.bt0[row / a.r0];
    });
  }
  if (wg == 0 && tid == 0) {
    // every workgroup has read the epoch and the frame counter before they may change
    ctl_finish(c, a.epoch, a.arrive, (uint32_t)nwg);
    if (over) *a.err = 2;
    *a.ctr = f + 1;
  }
}

// ---- depthwise causal conv (k taps) + LayerNorm over channels, one workgroup per column ----
struct CvDwLn {
  Ring in;           // pad = k - 1
  const float* w;    // (C, k)
  const float* b;    // (C)
  const float* lnw;
  const float* lnb;
  float* out;        // (C, rs_out) plain
  int rs_out, C, k;
  float eps;
  const int* ctr;
};

#define DW_MAXC 8  // channels per thread

__global__ __launch_bounds__(256) void cv_dwln_kernel(const CvDwLn p) {
  __shared__ float red[8];
  const int t = blockIdx.x, tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int f = *p.ctr - 1, base = ring_base(p.in, f);
  float v[DW_MAXC];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < DW_MAXC; ++i) {
    const int c = tid + 256 * i;
    v[i] = 0.f;
    if (c < p.C) {
      float a = p.b[c];
      for (int k = 0; k < p.k; ++k) a = fmaf(p.w[c * p.k + k], *ring_ptr(p.in, base, c, t + k), a);
      v[i] = a;
      s += a;
    }
  }
  s = wave_sum(s);
  if (lane == 0) red[wave] = s;
  __syncthreads();
  const float mean = ((red[0] + red[1]) + (red[2] + red[3])) / (float)p.C;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < DW_MAXC; ++i) {
    const int c = tid + 256 * i;
    if (c < p.C) { const float d = v[i] - mean; q = fmaf(d, d, q); }
  }
  q = wave_sum(q);
  if (lane == 0) red[4 + wave] = q;
  __syncthreads();
  const float rstd = 1.0f / sqrtf(((red[4] + red[5]) + (red[6] + red[7])) / (float)p.C + p.eps);
#pragma unroll
  for (int i = 0; i < DW_MAXC; ++i) {
    const int c = tid + 256 * i;
    if (c < p.C) p.out[(size_t)c * p.rs_out + t] = (v[i] - mean) * rstd * p.lnw[c] + p.lnb[c];
  }
}

// ---- last conv: one output channel, k taps, clamp to [-1, 1]; 64 samples x 4 channel quarters per workgroup ----
struct CvFinal {
  Ring in;         // pad = k - 1
  const float* w;  // (C, k)
  const float* b;  // (1)
  float* audio;
  int C, k, T;
  const int* ctr;
};

#define FIN_TW 16  // output columns per workgroup: 120 workgroups per frame, and a window small enough that every
                   // thread has all its loads in flight at once (64 columns: 30 workgroups, four rounds of loads)
__global__ __launch_bounds__(256) void cv_final_kernel(const CvFinal p) {
  extern __shared__ float xs[];  // C x (FIN_TW + k - 1) window of the ring | 16 x FIN_TW partial sums | C x k weights
  const int tid = threadIdx.x, qd = tid / FIN_TW, l = tid % FIN_TW;  // 16 channel groups x FIN_TW columns
  const int t0 = blockIdx.x * FIN_TW, W = FIN_TW + p.k - 1;
  const int n = p.C * W;
  float* part = xs + n;
  float* ws = part + 256;
  for (int i = tid; i < p.C * p.k; i += 256) ws[i] = p.w[i];
  const int f = *p.ctr - 1, base = ring_base(p.in, f);
  for (int i0 = tid; i0 < n; i0 += 256 * 12) {
    float v[12];
#pragma unroll
    for (int u = 0; u < 12; ++u) {
      const int i = i0 + 256 * u;
      v[u] = i < n ? *ring_ptr(p.in, base, i / W, t0 + i % W) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 12; ++u) { const int i = i0 + 256 * u; if (i < n) xs[i] = v[u]; }
  }
  __syncthreads();
  float a = 0.f;
  const int c0 = (p.C * qd) / 16, c1 = (p.C * (qd + 1)) / 16;
  for (int c = c0; c < c1; ++c)
    for (int k = 0; k < p.k; ++k) a = fmaf(ws[c * p.k + k], xs[c * W + l + k], a);
  part[qd * FIN_TW + l] = a;
  __syncthreads();
  const int t = t0 + l;
  if (qd == 0 && t < p.T) {
    float y = 0.f;
#pragma unroll
    for (int q = 0; q < 16; ++q) y += part[q * FIN_TW + l];  // group order: a fixed order of the sum
    y += p.b[0];
    p.audio[t] = fminf(1.0f, fmaxf(-1.0f, y));
  }
}

// ---- one-time repacking ----
__global__ void cv_pack_conv_kernel(const float* w, float* wp, int Cout, int Cin, int K) {  // (Cout,Cin,K) -> (K,Cout,Cin)
  const size_t n = (size_t)Cout * Cin * K;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const int ci = (int)(i % Cin);
    const int co = (int)((i / Cin) % Cout);
    const int k = (int)(i / ((size_t)Cin * Cout));
    wp[i] = w[((size_t)co * Cin + ci) * K + k];
  }
}
// ConvTranspose1d (Cin, Cout, K = taps*s) -> (taps, Cout*s, Cin); tap `taps-1` multiplies the current column
__global__ void cv_pack_tconv_kernel(const float* w, float* wp, int Cin, int Cout, int s, int taps) {
  const size_t n = (size_t)taps * Cout * s * Cin;
  const int K = taps * s;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const int ci = (int)(i % Cin);
    const int m = (int)((i / Cin) % ((size_t)Cout * s));
    const int tap = (int)(i / ((size_t)Cin * Cout * s));
    const int co = m / s, r = m % s;
    wp[i] = w[((size_t)ci * Cout + co) * K + r + (taps - 1 - tap) * s];
  }
}
// rows of src (M, K) into dst (M, ld) at column offset off
__global__ void cv_copy_rows_kernel(const float* src, float* dst, int M, int K, int ld, int off) {
  const size_t n = (size_t)M * K;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    dst[(i / K) * ld + off + (i % K)] = src[i];
}
// W (M, K) *= w (K) along every row
__global__ void cv_scale_cols_kernel(float* W, const float* w, int M, int K) {
  const size_t n = (size_t)M * K;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) W[i] *= w[i % K];
}
__global__ void cv_snake_tab_kernel(const float* alpha, const float* beta, float* ea, float* ib, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) { ea[i] = expf(alpha[i]); ib[i] = 1.0f / (expf(beta[i]) + 1e-9f); }
}
__global__ void cv_fill_kernel(float* p, size_t n, float v) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}
__global__ void cv_set_int_kernel(int* p, int v0, int v1) { p[0] = v0; p[1] = v1; }

// =================================== host side ===================================
struct Step {
  int kind;  // 0 gemm, 1 attn, 2 dwln
  CvGemm g;
  CvAttn a;
  CvDwLn d;
};

struct vui_codec {
  vui_codec_config cfg;
  int hop;
  char* ws;
  int64_t ws_bytes;
  float* state0;  // start of the zeroed-on-reset region (rings)
  size_t state_floats;
  int* ctr;  // [0] frames started since reset, [1] error flag
  int* cnt;  // arrival counters of split tiles
  size_t part_floats = 0, cnt_ints = 0;
  CvVq vq;
  std::vector<Step> steps;
  CvFinal fin;
  // the persistent form of the one-column steps (0: the kernel sequence runs them)
  CvTrunk trunk;
  int trunk_steps = 0;  // leading entries of `steps` the trunk kernel replaces (the codebook kernel as well)
  int trunk_wgs = 0;
  int w_nt = 0;          // GEMM weights with non-temporal loads: set when the vocoder is given part of the GPU
  int trunk_narrow = 0;  // the row plan of the kernel instantiation that trunk_wgs workgroups take
  int trunk_cap = 0;     // workgroups that can be resident at once on the whole GPU (at most 256 are used)
  size_t trunk_lds = 0;
  int use_trunk = 1;
};

static int ipow2(int n) { int r = 1; while (r < n) r <<= 1; return r; }

// Whether nwg workgroups can take the one-column steps with the row plan TrPlan<narrow>: every phase's rows per wave
// within the plan, every vector within the kernel's LDS areas.
template <bool NARROW> static bool trunk_fits_t(const vui_codec_config& k, int nwg) {
  typedef TrPlan<NARROW> P;
  const int A = k.n_heads * k.head_dim;
  auto fits = [&](int M, int K, int maxr, int maxc, int n) { return n > 0 && ((M + n - 1) / n + 3) / 4 <= maxr && K <= 256 * maxc && K % 4 == 0; };
  const int nq = nwg >= 4 * k.n_heads ? nwg - k.n_heads : nwg;  // the head-owning workgroups stay out of the q/k/v rows
  return nwg >= k.n_heads && fits(k.vq_dim, 2 * k.codebook_dim, P::VQ, 2, nwg) && fits(k.latent_dim, 3 * k.vq_dim, P::PRE, TR_MAXC, nwg) &&
         fits(k.d_model, k.latent_dim, P::IN, 4, nwg) && fits(3 * A, k.d_model, P::QKV, 2, nq) && fits(k.d_model, A, P::O, 4, nwg) &&
         2 * ((k.mlp_dim + nwg - 1) / nwg) <= 4 * P::GU && fits(k.d_model, k.mlp_dim, P::DN, 4, nwg) &&
         fits(k.latent_dim, k.d_model, P::OUT, 2, nwg) && (k.n_up == 0 || fits(k.latent_dim * k.up_ratios[0], k.latent_dim, P::UP, 4, nwg)) &&
         k.head_dim <= 64 && k.max_seq <= 256 && k.d_model <= 1536 && A <= 1536 && k.mlp_dim <= 1536 && k.latent_dim <= 1536 &&
         3 * k.vq_dim <= 1536;
}
static bool trunk_fits(const vui_codec_config& k, int nwg, bool narrow) {
  return narrow ? trunk_fits_t<true>(k, nwg) : trunk_fits_t<false>(k, nwg);
}

static int cv_check(const vui_codec_config* c) {
  if (!c) { vui_set_error("NULL codec config"); return VUI_EINVAL; }
  if (c->n_up < 0 || c->n_up > 4 || c->n_rates < 1 || c->n_rates > 8) { vui_set_error("codec: n_up=%d / n_rates=%d outside the supported range", c->n_up, c->n_rates); return VUI_EINVAL; }
  if (c->n_codebooks < 1 || c->n_semantic < 1 || c->n_semantic > c->n_codebooks || c->codebook_size < 1) { vui_set_error("codec: bad codebook layout"); return VUI_EINVAL; }
  const int A = c->n_heads * c->head_dim;
  int dims32[] = {2 * c->codebook_dim, c->vq_dim, c->latent_dim, c->d_model, A, c->mlp_dim, 4 * c->latent_dim, c->decoder_dim};
  for (int v : dims32)
    if (v < 32 || (v % 32)) { vui_set_error("codec: every layer width must be a multiple of 32 (got %d)", v); return VUI_EINVAL; }
  if (c->head_dim > 64 || (c->head_dim & 15) || c->n_heads < 1) { vui_set_error("codec: head_dim=%d unsupported (a multiple of 16, <= 64)", c->head_dim); return VUI_EINVAL; }
  if ((c->decoder_dim >> c->n_rates) * (FIN_TW + 6 + 7) * 4 > 60000) { vui_set_error("codec: last stage too wide"); return VUI_EINVAL; }
  if (c->max_seq < 1 || c->max_seq > 4096) { vui_set_error("codec: max_seq=%d outside [1,4096]", c->max_seq); return VUI_EINVAL; }
  if (c->latent_dim > 256 * DW_MAXC) { vui_set_error("codec: latent_dim=%d above %d", c->latent_dim, 256 * DW_MAXC); return VUI_EINVAL; }
  int dim = c->decoder_dim;
  for (int i = 0; i < c->n_rates; ++i) {
    if (c->rates[i] < 1 || (dim % 64)) { vui_set_error("codec: decoder stage %d: width %d must be a multiple of 64, rate >= 1", i, dim); return VUI_EINVAL; }
    dim /= 2;
  }
  for (int i = 0; i < c->n_up; ++i)
    if (c->up_ratios[i] < 1) { vui_set_error("codec: bad upsample ratio"); return VUI_EINVAL; }
  return VUI_OK;
}

int32_t vui_codec_hop(const vui_codec_config* c) {
  if (cv_check(c)) return VUI_EINVAL;
  int h = 1;
  for (int i = 0; i < c->n_up; ++i) h *= c->up_ratios[i];
  for (int i = 0; i < c->n_rates; ++i) h *= c->rates[i];
  return h;
}

int32_t vui_codec_n_tensors(const vui_codec_config* c) {
  if (cv_check(c)) return VUI_EINVAL;
  return 2 * 2 + c->n_codebooks + 2 + 2 + 11 * c->n_layers + 3 + 11 * c->n_up + 2 + c->n_rates * (4 + 3 * 8) + 2 + 2;
}

// Bump allocator over the workspace; with base == nullptr it only measures.
struct Arena {
  char* base;
  size_t off = 0;
  float* take(size_t floats) {
    float* p = base ? (float*)(base + off) : nullptr;
    off += (floats * 4 + 255) & ~(size_t)255;
    return p;
  }
};

static Ring mk_ring(Arena& ar, int C, int pad, int T, bool stream) {
  Ring r;
  r.rs = ipow2(pad + T);
  r.mask = r.rs - 1;
  r.pad = pad;
  r.tstep = stream ? T : 0;
  r.p = ar.take((size_t)C * r.rs);
  return r;
}
static Ring no_ring() { Ring r; r.p = nullptr; r.rs = 1; r.mask = 0; r.pad = 0; r.tstep = 0; return r; }

static void grid_for(size_t n, dim3& g) { size_t b = (n + 255) / 256; g = dim3((unsigned)(b > 4096 ? 4096 : (b ? b : 1))); }

// Lays out the workspace and (when tensors != nullptr) packs weights and records the launch plan.
static int cv_build(vui_codec* cc, const vui_codec_config* c, const void* const* tensors, char* ws, hipStream_t st, int64_t* need,
                    size_t part_cap, size_t cnt_cap, size_t* part_need, size_t* cnt_need) {
  Arena ar{ws};
  const bool real = ws != nullptr && tensors != nullptr;
  int ti = 0;
  auto next = [&]() -> const float* { return real ? (const float*)tensors[ti++] : (ti++, nullptr); };
  auto pack_copy = [&](const float* src, float* dst, int M, int K, int ld, int off) {
    if (!real) return;
    dim3 g; grid_for((size_t)M * K, g);
    hipLaunchKernelGGL(cv_copy_rows_kernel, g, dim3(256), 0, st, src, dst, M, K, ld, off);
  };
  auto pack_conv = [&](const float* src, int Cout, int Cin, int K) -> float* {
    float* dst = ar.take((size_t)Cout * Cin * K);
    if (real) { dim3 g; grid_for((size_t)Cout * Cin * K, g); hipLaunchKernelGGL(cv_pack_conv_kernel, g, dim3(256), 0, st, src, dst, Cout, Cin, K); }
    return dst;
  };
  auto pack_tconv = [&](const float* src, int Cin, int Cout, int s, int taps) -> float* {
    float* dst = ar.take((size_t)taps * Cout * s * Cin);
    if (real) { dim3 g; grid_for((size_t)taps * Cout * s * Cin, g); hipLaunchKernelGGL(cv_pack_tconv_kernel, g, dim3(256), 0, st, src, dst, Cin, Cout, s, taps); }
    return dst;
  };
  auto fold_norm = [&](float* W, const float* w, int M, int K) {
    if (!real) return;
    dim3 g; grid_for((size_t)M * K, g);
    hipLaunchKernelGGL(cv_scale_cols_kernel, g, dim3(256), 0, st, W, w, M, K);
  };
  auto vec = [&](const float* src, int n) -> float* { float* dst = ar.take(n); pack_copy(src, dst, 1, n, n, 0); return dst; };
  struct Snake { float* ea; float* ib; };
  auto snake = [&](int n) -> Snake {
    const float* al = next(); const float* be = next();
    Snake s{ar.take(n), ar.take(n)};
    if (real) hipLaunchKernelGGL(cv_snake_tab_kernel, dim3((n + 255) / 256), dim3(256), 0, st, al, be, s.ea, s.ib, n);
    return s;
  };
  int* ctr = (int*)ar.take(64);
  // launch-shape targets: workgroups in flight for weight-streaming (one column block) and for wider tiles
  const int wg_target = 512, wg_target2 = 200;
  // meeting place of split tiles: sized by a first pass (the sizes do not depend on the pointers)
  size_t part_floats = 0, cnt_ints = 0;
  float* part = ar.take(part_cap);
  int* cnt = (int*)ar.take(cnt_cap);
  auto gemm = [&](const float* W, const float* bias, int M, int Cin, int taps, int dil, int T, const Ring& in) -> CvGemm {
    CvGemm g;
    memset(&g, 0, sizeof(g));
    g.W = W; g.bias = bias; g.M = M; g.Cin = Cin; g.taps = taps; g.dil = dil; g.T = T; g.bias_div = 1;
    g.in = in; g.in_mode = IN_PLAIN; g.eps = 1e-6f; g.epi = EPI_NONE;
    g.res = no_ring(); g.out_raw = no_ring(); g.out_act = no_ring(); g.ctr = ctr;
    // Tile width: the one that pads the columns least, the wider one on a tie (a wave reuses its weight
    // registers for every 16-column block).  Then workgroups share a tile's units until about 512 (one
    // column block: the layer streams weights) or 200 (wider: the layer computes) are in flight, each wave
    // keeping at least four units.  Measured per layer shape on MI355X.
    const int U = taps * (Cin / 32);
    auto tiles = [&](int tt) { return (M / 16) * ((T + 16 * tt - 1) / (16 * tt)); };
    g.tt = 1;
    for (int tt : {2, 4})
      if (T > 8 * tt && tiles(tt) * tt <= tiles(g.tt) * g.tt) g.tt = tt;
    int sp = 1;
    if (U >= 64) {
      const int target = g.tt == 1 ? wg_target : wg_target2;
      sp = (2 * target + tiles(g.tt)) / (2 * tiles(g.tt));  // rounded
      if (sp > U / 16) sp = U / 16;
      if (sp > 8) sp = 8;
      if (sp < 1) sp = 1;
    }
    g.splits = sp; g.part = part; g.cnt = cnt;
    if ((size_t)tiles(g.tt) * sp * g.tt * 256 > part_floats) part_floats = (size_t)tiles(g.tt) * sp * g.tt * 256;
    if ((size_t)tiles(g.tt) > cnt_ints) cnt_ints = tiles(g.tt);
    return g;
  };
  auto push_gemm = [&](const CvGemm& g) { if (real) { Step s; memset((void*)&s, 0, sizeof(s)); s.kind = 0; s.g = g; cc->steps.push_back(s); } };

  const int cd = c->codebook_dim, CS = c->codebook_size, L = c->latent_dim, D = c->d_model, A = c->n_heads * c->head_dim;
  // ---- quantizer: [semantic | acoustic] rows times [W_sem | W_ac] ----
  float* embed = ar.take((size_t)c->n_codebooks * CS * cd);
  float* Wvq = ar.take((size_t)c->vq_dim * 2 * cd);
  {
    int cb = 0;
    for (int grp = 0; grp < 2; ++grp) {
      const int n = grp == 0 ? c->n_semantic : c->n_codebooks - c->n_semantic;
      next();  // input_proj: encoder side only
      const float* op = next();
      pack_copy(op, Wvq, c->vq_dim, cd, 2 * cd, grp * cd);
      for (int i = 0; i < n; ++i, ++cb) pack_copy(next(), embed + (size_t)cb * CS * cd, CS, cd, cd, 0);
    }
  }
  // ---- state region (zeroed by reset) starts here: all rings ----
  const size_t state_begin = ar.off;
  Ring pre_in = mk_ring(ar, c->vq_dim, 2, 1, true);
  std::vector<Ring> dw_in, tc_in, ru_in;
  int T = 1;
  for (int i = 0; i < c->n_up; ++i) { T *= c->up_ratios[i]; dw_in.push_back(mk_ring(ar, L, 6, T, true)); }
  const int T_lat = T;
  Ring dec0_in = mk_ring(ar, L, 6, T_lat, true);
  {
    int dim = c->decoder_dim, t = T_lat;
    for (int i = 0; i < c->n_rates; ++i) {
      tc_in.push_back(mk_ring(ar, dim, 1, t, true));
      t *= c->rates[i];
      dim /= 2;
      for (int j = 0; j < 3; ++j) { const int dil = j == 0 ? 1 : (j == 1 ? 3 : 9); ru_in.push_back(mk_ring(ar, dim, 6 * dil, t, true)); }
    }
  }
  int fin_dim = c->decoder_dim >> c->n_rates;
  const int hop = vui_codec_hop(c);
  Ring fin_in = mk_ring(ar, fin_dim, 6, hop, true);
  const size_t state_end = ar.off;
  // ---- plain activation buffers ----
  Ring vqx = mk_ring(ar, 2 * cd, 0, 1, false);
  Ring pre_out = mk_ring(ar, L, 0, 1, false);
  Ring xres = mk_ring(ar, D, 0, 1, false);
  Ring qkv = mk_ring(ar, 3 * A, 0, 1, false);
  Ring att = mk_ring(ar, A, 0, 1, false);
  Ring gu = mk_ring(ar, c->mlp_dim, 0, 1, false);
  float* kc = ar.take((size_t)c->n_layers * A * c->max_seq);
  float* vc = ar.take((size_t)c->n_layers * A * c->max_seq);
  float* inv_freq = ar.take(c->head_dim / 2);
  // persistent trunk: exchange words (never reused inside a launch), layer table, epoch / arrival / error words
  const size_t ll_words = (size_t)c->vq_dim + L + D + (size_t)c->n_layers * (3 * A + A + D + c->mlp_dim + D) + L;
  uint64_t* ll = (uint64_t*)ar.take(ll_words * 2);
  TrunkLayer* tl_dev = (TrunkLayer*)ar.take((sizeof(TrunkLayer) * c->n_layers + 3) / 4);
  uint32_t* tctl = (uint32_t*)ar.take(64);
  if (real) {
    std::vector<float> h(c->head_dim / 2);
    // 1 / theta^(2i/dim) in fp32, as torch evaluates it (qwen_codec.py:164)
    for (int i = 0; i < c->head_dim / 2; ++i) h[i] = 1.0f / powf(c->rope_theta, (float)(2 * i) / (float)c->head_dim);
    HIP_TRY(hipMemcpyAsync(inv_freq, h.data(), h.size() * 4, hipMemcpyHostToDevice, st));
    HIP_TRY(hipStreamSynchronize(st));  // h goes out of scope
  }

  // ---- pre_conv, pre_transformer ----
  CvTrunk tk;
  memset((void*)&tk, 0, sizeof(tk));
  std::vector<TrunkLayer> tl(c->n_layers);
  {
    CvGemm g = gemm(Wvq, nullptr, c->vq_dim, 2 * cd, 1, 1, 1, vqx);
    g.out_raw = pre_in;
    push_gemm(g);
    const float* w = next(); const float* b = next();
    g = gemm(pack_conv(w, L, c->vq_dim, 3), vec(b, L), L, c->vq_dim, 3, 1, 1, pre_in);
    g.out_raw = pre_out;
    push_gemm(g);
    tk.Wvq = Wvq; tk.vq_dim = c->vq_dim; tk.Wpre = g.W; tk.bpre = g.bias; tk.L = L; tk.pre_in = pre_in;
    w = next(); b = next();
    float* Wi = ar.take((size_t)D * L);
    pack_copy(w, Wi, D, L, L, 0);
    g = gemm(Wi, vec(b, D), D, L, 1, 1, 1, pre_out);
    g.out_raw = xres;
    push_gemm(g);
    tk.Win = g.W; tk.bin = g.bias; tk.D = D;
  }
  for (int l = 0; l < c->n_layers; ++l) {
    const float* ln1 = next();
    float* Wqkv = ar.take((size_t)3 * A * D);
    for (int i = 0; i < 3; ++i) pack_copy(next(), Wqkv + (size_t)i * A * D, A, D, D, 0);
    fold_norm(Wqkv, ln1, 3 * A, D);
    float* Wo = ar.take((size_t)D * A);
    pack_copy(next(), Wo, D, A, A, 0);
    const float* asc = next();
    const float* ln2 = next();
    float* Wgu = ar.take((size_t)2 * c->mlp_dim * D);  // rows interleaved: gate_0, up_0, gate_1, up_1, ...
    for (int i = 0; i < 2; ++i) pack_copy(next(), Wgu, c->mlp_dim, D, 2 * D, i * D);
    fold_norm(Wgu, ln2, 2 * c->mlp_dim, D);
    float* Wd = ar.take((size_t)D * c->mlp_dim);
    pack_copy(next(), Wd, D, c->mlp_dim, c->mlp_dim, 0);
    const float* msc = next();
    CvGemm g = gemm(Wqkv, nullptr, 3 * A, D, 1, 1, 1, xres);
    g.in_mode = IN_RMS; g.out_raw = qkv;
    push_gemm(g);
    if (real) {
      Step s; memset((void*)&s, 0, sizeof(s)); s.kind = 1;
      s.a.qkv = qkv.p; s.a.kc = kc + (size_t)l * A * c->max_seq; s.a.vc = vc + (size_t)l * A * c->max_seq;
      s.a.out = att.p; s.a.inv_freq = inv_freq; s.a.H = c->n_heads; s.a.hd = c->head_dim; s.a.max_seq = c->max_seq; s.a.ctr = ctr;
      cc->steps.push_back(s);
    }
    g = gemm(Wo, nullptr, D, A, 1, 1, 1, att);
    g.epi = EPI_SCALE_RES; g.scale = vec(asc, D); g.res = xres; g.out_raw = xres;
    push_gemm(g);
    tl[l].Wqkv = Wqkv; tl[l].Wo = Wo; tl[l].asc = g.scale; tl[l].Wgu = Wgu; tl[l].Wd = Wd;
    tl[l].kc = kc + (size_t)l * A * c->max_seq; tl[l].vc = vc + (size_t)l * A * c->max_seq;
    g = gemm(Wgu, nullptr, 2 * c->mlp_dim, D, 1, 1, 1, xres);
    g.in_mode = IN_RMS; g.epi = EPI_SILU_PAIR; g.out_raw = gu;
    push_gemm(g);
    g = gemm(Wd, nullptr, D, c->mlp_dim, 1, 1, 1, gu);
    g.epi = EPI_SCALE_RES; g.scale = vec(msc, D); g.res = xres; g.out_raw = xres;
    push_gemm(g);
    tl[l].msc = g.scale;
  }
  Ring cur = mk_ring(ar, L, 0, 1, false);  // output of the transformer = input of the first upsample stage
  {
    const float* nw = next(); const float* w = next(); const float* b = next();
    float* Wout = ar.take((size_t)L * D);
    pack_copy(w, Wout, L, D, D, 0);
    fold_norm(Wout, nw, L, D);
    CvGemm g = gemm(Wout, vec(b, L), L, D, 1, 1, 1, xres);
    g.in_mode = IN_RMS;
    g.out_raw = c->n_up ? cur : dec0_in;
    push_gemm(g);
    tk.Wout = g.W; tk.bout = g.bias; tk.out = dec0_in;
  }
  int trunk_steps = real ? (int)cc->steps.size() : 0;
  // ---- upsample stages: transposed conv (kernel = stride) + ConvNeXt block ----
  T = 1;
  for (int i = 0; i < c->n_up; ++i) {
    const int r = c->up_ratios[i], Tin = T;
    T *= r;
    const float* w = next(); const float* b = next();
    CvGemm g = gemm(pack_tconv(w, L, L, r, 1), vec(b, L), L * r, L, 1, 1, Tin, cur);
    g.bias_div = r; g.tc_stride = r; g.out_raw = dw_in[i];
    push_gemm(g);
    if (i == 0) { tk.Wt0 = g.W; tk.bt0 = g.bias; tk.r0 = r; tk.out = dw_in[0]; if (real) trunk_steps = (int)cc->steps.size(); }
    const float* dww = next(); const float* dwb = next(); const float* lnw = next(); const float* lnb = next();
    Ring ln = mk_ring(ar, L, 0, T, false);
    float* dwwp = vec(dww, L * 7); float* dwbp = vec(dwb, L); float* lnwp = vec(lnw, L); float* lnbp = vec(lnb, L);
    if (real) {
      Step s; memset((void*)&s, 0, sizeof(s)); s.kind = 2;
      s.d.in = dw_in[i]; s.d.w = dwwp; s.d.b = dwbp; s.d.lnw = lnwp; s.d.lnb = lnbp;
      s.d.out = ln.p; s.d.rs_out = ln.rs; s.d.C = L; s.d.k = 7; s.d.eps = 1e-6f; s.d.ctr = ctr;
      s.g.T = T;  // grid
      cc->steps.push_back(s);
    }
    const float* w1 = next(); const float* b1 = next(); const float* w2 = next(); const float* b2 = next(); const float* gam = next();
    Ring pw = mk_ring(ar, 4 * L, 0, T, false);
    float* W1 = ar.take((size_t)4 * L * L);
    pack_copy(w1, W1, 4 * L, L, L, 0);
    g = gemm(W1, vec(b1, 4 * L), 4 * L, L, 1, 1, T, ln);
    g.epi = EPI_GELU; g.out_raw = pw;
    push_gemm(g);
    float* W2 = ar.take((size_t)L * 4 * L);
    pack_copy(w2, W2, L, 4 * L, 4 * L, 0);
    g = gemm(W2, vec(b2, L), L, 4 * L, 1, 1, T, pw);
    g.epi = EPI_SCALE_RES; g.scale = vec(gam, L); g.res = dw_in[i];
    if (i + 1 < c->n_up) { cur = mk_ring(ar, L, 0, T, false); g.out_raw = cur; } else g.out_raw = dec0_in;
    push_gemm(g);
  }
  // ---- BigVGAN-style decoder ----
  {
    int dim = c->decoder_dim;
    const float* w = next(); const float* b = next();
    CvGemm g0 = gemm(pack_conv(w, dim, L, 7), vec(b, dim), dim, L, 7, 1, T_lat, dec0_in);
    int t = T_lat;
    CvGemm pending = g0;  // its out_act is the first block's snake, known once the block's tensors are read
    for (int i = 0; i < c->n_rates; ++i) {
      const int rate = c->rates[i], out = dim / 2, tin = t;
      t *= rate;
      Snake s0 = snake(dim);
      pending.out_act = tc_in[i]; pending.ea = s0.ea; pending.ib = s0.ib;
      push_gemm(pending);
      const float* tw = next(); const float* tb = next();
      CvGemm tg = gemm(pack_tconv(tw, dim, out, rate, 2), vec(tb, out), out * rate, dim, 2, 1, tin, tc_in[i]);
      tg.bias_div = rate; tg.tc_stride = rate;
      Ring R = mk_ring(ar, out, 0, t, false);
      Ring hbuf = mk_ring(ar, out, 0, t, false);
      tg.out_raw = R;
      pending = tg;
      for (int j = 0; j < 3; ++j) {
        const int dil = j == 0 ? 1 : (j == 1 ? 3 : 9);
        const Ring& rin = ru_in[i * 3 + j];
        Snake a1 = snake(out);
        pending.out_act = rin; pending.ea = a1.ea; pending.ib = a1.ib;
        push_gemm(pending);
        const float* w1 = next(); const float* b1 = next();
        Snake a2 = snake(out);
        const float* w2 = next(); const float* b2 = next();
        CvGemm c1 = gemm(pack_conv(w1, out, out, 7), vec(b1, out), out, out, 7, dil, t, rin);
        c1.out_act = hbuf; c1.ea = a2.ea; c1.ib = a2.ib;
        push_gemm(c1);
        float* W2 = ar.take((size_t)out * out);
        pack_copy(w2, W2, out, out, out, 0);
        CvGemm c2 = gemm(W2, vec(b2, out), out, out, 1, 1, t, hbuf);
        c2.epi = EPI_RES; c2.res = R;
        if (j < 2) c2.out_raw = R;
        pending = c2;
      }
      dim = out;
    }
    Snake sf = snake(dim);
    pending.out_act = fin_in; pending.ea = sf.ea; pending.ib = sf.ib;
    push_gemm(pending);
    const float* fw = next(); const float* fb = next();
    float* fwp = vec(fw, dim * 7); float* fbp = vec(fb, 1);
    if (real) {
      cc->fin.in = fin_in; cc->fin.w = fwp; cc->fin.b = fbp; cc->fin.audio = nullptr; cc->fin.C = dim; cc->fin.k = 7; cc->fin.T = hop; cc->fin.ctr = ctr;
    }
  }
  if (need) *need = (int64_t)ar.off;
  if (part_need) *part_need = part_floats;
  if (cnt_need) *cnt_need = cnt_ints;
  if (real) {
    tk.codes = nullptr; tk.n_q = 0; tk.n_sem = c->n_semantic; tk.CS = CS; tk.cd = cd; tk.embed = embed;
    tk.ctr = ctr; tk.err = ctr + 1; tk.max_seq = c->max_seq;
    tk.n_layers = c->n_layers; tk.H = c->n_heads; tk.hd = c->head_dim; tk.mlp = c->mlp_dim;
    tk.layers = tl_dev; tk.inv_freq = inv_freq; tk.ll = ll; tk.epoch = tctl; tk.arrive = tctl + 1; tk.lerr = tctl + 2;
    tk.eps = 1e-6f;
    HIP_TRY(hipMemcpyAsync(tl_dev, tl.data(), sizeof(TrunkLayer) * c->n_layers, hipMemcpyHostToDevice, st));
    {
      dim3 g; grid_for(ll_words * 2, g);
      hipLaunchKernelGGL(cv_fill_kernel, g, dim3(256), 0, st, (float*)ll, ll_words * 2, 0.0f);
      hipLaunchKernelGGL(cv_fill_kernel, dim3(1), dim3(64), 0, st, (float*)tctl, (size_t)16, 0.0f);
    }
    HIP_TRY(hipStreamSynchronize(st));  // tl goes out of scope
    cc->trunk = tk;
    cc->trunk_steps = trunk_steps;
    if (part_floats > part_cap || cnt_ints > cnt_cap) { vui_set_error("codec: internal scratch sizing"); return VUI_EINVAL; }
    cc->ctr = ctr; cc->cnt = cnt; cc->cnt_ints = cnt_cap;
    cc->state0 = (float*)(ws + state_begin);
    cc->state_floats = (state_end - state_begin) / 4;
    cc->vq.codes = nullptr; cc->vq.n_q = 0; cc->vq.n_sem = c->n_semantic; cc->vq.CS = CS; cc->vq.cd = cd;
    cc->vq.embed = embed; cc->vq.x = vqx.p; cc->vq.ctr = ctr; cc->vq.err = ctr + 1; cc->vq.max_seq = c->max_seq;
    if (ti != vui_codec_n_tensors(c)) { vui_set_error("codec: internal tensor count %d != %d", ti, vui_codec_n_tensors(c)); return VUI_EINVAL; }
    HIP_TRY(hipGetLastError());
  }
  return VUI_OK;
}

int64_t vui_codec_workspace_bytes(const vui_codec_config* c) {
  if (cv_check(c)) return VUI_EINVAL;
  int64_t need = 0;
  size_t pf = 0, ci = 0;
  if (cv_build(nullptr, c, nullptr, nullptr, nullptr, nullptr, 0, 0, &pf, &ci)) return VUI_EINVAL;
  if (cv_build(nullptr, c, nullptr, nullptr, nullptr, &need, pf, ci, nullptr, nullptr)) return VUI_EINVAL;
  return need;
}

int vui_codec_reset(vui_codec* c, vui_stream_t stream) {
  if (!c) { vui_set_error("NULL codec"); return VUI_EINVAL; }
  hipStream_t st = (hipStream_t)stream;
  dim3 g; grid_for(c->state_floats, g);
  hipLaunchKernelGGL(cv_fill_kernel, g, dim3(256), 0, st, c->state0, c->state_floats, 0.0f);
  hipLaunchKernelGGL(cv_set_int_kernel, dim3(1), dim3(1), 0, st, c->ctr, 0, 0);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

int vui_codec_init(const vui_codec_config* cfg, const void* const* tensors, int32_t n_tensors, void* workspace,
                   int64_t workspace_bytes, vui_stream_t stream, vui_codec** out) {
  if (!out) { vui_set_error("NULL out"); return VUI_EINVAL; }
  *out = nullptr;
  int rc = cv_check(cfg);
  if (rc) return rc;
  if (!tensors || !workspace) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  if (n_tensors != vui_codec_n_tensors(cfg)) { vui_set_error("codec: %d tensors given, %d expected", n_tensors, vui_codec_n_tensors(cfg)); return VUI_EINVAL; }
  for (int i = 0; i < n_tensors; ++i)
    if (!tensors[i]) { vui_set_error("codec: tensor %d is NULL", i); return VUI_EINVAL; }
  const int64_t need = vui_codec_workspace_bytes(cfg);
  if (need < 0) return (int)need;
  if (workspace_bytes < need) { vui_set_error("workspace too small: %lld < %lld", (long long)workspace_bytes, (long long)need); return VUI_ENOMEM; }
  if (((uintptr_t)workspace) & 255) { vui_set_error("workspace must be 256-byte aligned"); return VUI_EINVAL; }
  vui_codec* c = new (std::nothrow) vui_codec();
  if (!c) { vui_set_error("out of host memory"); return VUI_ENOMEM; }
  c->cfg = *cfg; c->hop = vui_codec_hop(cfg); c->ws = (char*)workspace; c->ws_bytes = workspace_bytes;
  size_t pf = 0, ci = 0;
  rc = cv_build(nullptr, cfg, nullptr, nullptr, nullptr, nullptr, 0, 0, &pf, &ci);
  if (!rc) rc = cv_build(c, cfg, tensors, (char*)workspace, (hipStream_t)stream, nullptr, pf, ci, nullptr, nullptr);
  if (!rc) {
    dim3 g; grid_for(ci, g);
    hipLaunchKernelGGL(cv_fill_kernel, g, dim3(256), 0, (hipStream_t)stream, (float*)c->cnt, ci, 0.0f);
  }
  if (!rc) rc = vui_codec_reset(c, stream);
  if (rc) { delete c; return rc; }
  // the persistent trunk needs all its workgroups resident at once and the per-wave row counts it was built for
  {
    const vui_codec_config& k = c->cfg;
    c->trunk_lds = (size_t)(1536 + k.d_model + 64 + k.max_seq + 192 + 256 + 16) * 4;
    int dev = 0, cus = 0, per_cu = 0;
    HIP_TRY(hipGetDevice(&dev));
    HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)cv_trunk_kernel<true>, FR_THREADS, c->trunk_lds));
    c->trunk_cap = cus * per_cu < 256 ? cus * per_cu : 256;
    c->trunk_wgs = 0;
    for (int narrow = 0; narrow < 2 && !c->trunk_wgs; ++narrow)
      if (trunk_fits(k, c->trunk_cap, narrow != 0)) { c->trunk_wgs = c->trunk_cap; c->trunk_narrow = narrow; }
    c->use_trunk = 1;
  }
  *out = c;
  return VUI_OK;
}

void vui_codec_destroy(vui_codec* c) { delete c; }

int vui_codec_workgroups(vui_codec* c, int nwg) {
  if (!c) { vui_set_error("NULL codec"); return VUI_EINVAL; }
  if (nwg < 1 || nwg > c->trunk_cap) { vui_set_error("codec: %d workgroups outside [1, %d]", nwg, c->trunk_cap); return VUI_EINVAL; }
  for (int narrow = 0; narrow < 2; ++narrow)
    if (trunk_fits(c->cfg, nwg, narrow != 0)) {
      c->trunk_wgs = nwg; c->trunk_narrow = narrow;
      c->w_nt = nwg < c->trunk_cap ? 1 : 0;
      return VUI_OK;
    }
  vui_set_error("codec: the persistent form of the one-column steps does not run on %d workgroups (too many rows per wave)", nwg);
  return VUI_EINVAL;
}

int vui_codec_persistent(vui_codec* c, int enable) {
  if (!c) { vui_set_error("NULL codec"); return 0; }
  if (enable >= 0) c->use_trunk = enable ? 1 : 0;
  return c->use_trunk && c->trunk_wgs > 0;
}

static int launch_cv_gemm(const CvGemm& g, bool w_nt, hipStream_t st) {
  if (g.M % 16 || g.Cin % 32 || g.T < 1) { vui_set_error("codec gemm: bad shape M=%d Cin=%d T=%d", g.M, g.Cin, g.T); return VUI_EINVAL; }
  const dim3 grid(g.M / 16, (g.T + 16 * g.tt - 1) / (16 * g.tt), g.splits);
  const dim3 block(64 * CV_NW);
  // units a wave of one part works through; one single-buffered round holds 8 / 6 / 3 of them
  const int U = g.taps * (g.Cin / 32), per_wave = ((U + g.splits - 1) / g.splits + CV_NW - 1) / CV_NW;
  const bool one_round = per_wave <= (g.tt == 1 ? 8 : (g.tt == 2 ? 6 : 3));
#define CV_LAUNCH(K, TT_)                                                                         \
  do {                                                                                            \
    if (w_nt) hipLaunchKernelGGL((K<TT_, true>), grid, block, 0, st, g);                          \
    else hipLaunchKernelGGL((K<TT_, false>), grid, block, 0, st, g);                              \
  } while (0)
  if (one_round) {
    if (g.tt == 1) CV_LAUNCH(cv_gemm1_kernel, 1);
    else if (g.tt == 2) CV_LAUNCH(cv_gemm1_kernel, 2);
    else CV_LAUNCH(cv_gemm1_kernel, 4);
  } else {
    if (g.tt == 1) CV_LAUNCH(cv_gemm_kernel, 1);
    else if (g.tt == 2) CV_LAUNCH(cv_gemm_kernel, 2);
    else CV_LAUNCH(cv_gemm_kernel, 4);
  }
#undef CV_LAUNCH
  return VUI_OK;
}

int vui_codec_decode_frame(vui_codec* c, const int64_t* codes, int32_t n_q, float* audio_out, vui_stream_t stream) {
  if (!c) { vui_set_error("NULL codec"); return VUI_EINVAL; }
  if (!codes || !audio_out) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  if (n_q < 1 || n_q > c->cfg.n_codebooks) { vui_set_error("n_q=%d outside [1,%d]", n_q, c->cfg.n_codebooks); return VUI_EINVAL; }
  hipStream_t st = (hipStream_t)stream;
  size_t first = 0;
  if (c->use_trunk && c->trunk_wgs > 0) {
    CvTrunk tk = c->trunk;
    tk.codes = codes; tk.n_q = n_q;
    if (c->trunk_narrow) hipLaunchKernelGGL(cv_trunk_kernel<true>, dim3(c->trunk_wgs), dim3(FR_THREADS), c->trunk_lds, st, tk);
    else hipLaunchKernelGGL(cv_trunk_kernel<false>, dim3(c->trunk_wgs), dim3(FR_THREADS), c->trunk_lds, st, tk);
    first = (size_t)c->trunk_steps;
  } else {
    CvVq vq = c->vq;
    vq.codes = codes; vq.n_q = n_q;
    hipLaunchKernelGGL(cv_vq_kernel, dim3(1), dim3(256), 0, st, vq);
  }
  for (size_t si = first; si < c->steps.size(); ++si) {
    const Step& s = c->steps[si];
    if (s.kind == 0) {
      int rc = launch_cv_gemm(s.g, c->w_nt != 0, st);
      if (rc) return rc;
    } else if (s.kind == 1) {
      const size_t lds = (size_t)(s.a.hd + s.a.max_seq + 4 * s.a.hd + 8) * 4;
      hipLaunchKernelGGL(cv_attn_kernel, dim3(s.a.H), dim3(256), lds, st, s.a);
    } else {
      hipLaunchKernelGGL(cv_dwln_kernel, dim3(s.g.T), dim3(256), 0, st, s.d);
    }
  }
  CvFinal fin = c->fin;
  fin.audio = audio_out;
  hipLaunchKernelGGL(cv_final_kernel, dim3((fin.T + FIN_TW - 1) / FIN_TW), dim3(256), (size_t)(fin.C * (FIN_TW + fin.k - 1) + 256 + fin.C * fin.k) * 4, st, fin);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

int64_t vui_codec_status(vui_codec* c, vui_stream_t stream) {
  if (!c) { vui_set_error("NULL codec"); return VUI_EINVAL; }
  int h[2] = {0, 0};
  uint32_t lerr = 0;
  HIP_TRY(hipMemcpyAsync(h, c->ctr, sizeof(h), hipMemcpyDeviceToHost, (hipStream_t)stream));
  if (c->trunk.lerr) HIP_TRY(hipMemcpyAsync(&lerr, c->trunk.lerr, sizeof(lerr), hipMemcpyDeviceToHost, (hipStream_t)stream));
  HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  if (lerr) {
    vui_set_error(lerr == 2 ? "codec: the persistent kernel's launch count wrapped; create the decoder again"
                            : "codec: an exchange wait of the persistent kernel timed out (is another kernel running on the device?)");
    return VUI_EHIP;
  }
  if (h[1] == 1) { vui_set_error("codec: a code outside [0, %d) was clamped", c->cfg.codebook_size); return VUI_EINVAL; }
  if (h[1] == 2) { vui_set_error("codec: more than max_seq=%d frames since the last reset", c->cfg.max_seq); return VUI_EINVAL; }
  return h[0];
}
