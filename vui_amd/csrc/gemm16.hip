// Skinny GEMM for 2..16 activation rows on the matrix cores: y (B, N) = x (B, K) W^T (N, K).
//
// One workgroup owns 16 consecutive output features; its four waves split K in steps of 64 and
// each issues v_mfma_f32_16x16x32_bf16 with A = a 16 x 32 weight tile (lane i: feature i % 16,
// eight consecutive k) and B = the activations (lane i: row i % 16, the same k), so the 16 x 16
// fp32 accumulator holds all rows of 16 features.  Each lane reads 32 contiguous weight bytes per
// step (two MFMAs), i.e. a full 128-byte line per feature; the k order inside a step is permuted the
// same way for A and B, which a dot product does not see.  int8 weights are widened to bf16 in
// registers (exact) and scaled per feature in the epilogue.  Activations are staged in LDS as bf16
// after the two-rounding RMSNorm (src/vui/model.py:286-297); row stride K + 8 keeps the 16 rows of a
// B-operand read on distinct banks.
#include "common.h"
#include "gemv_epi.h"
#include "internal.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define G16_THREADS 256
#define G16_MAXS 8  // K steps (of 64) per wave held in registers: K <= 2048
// from two rows on the matrix-core form wins over one wave per row pair (measured, bf16 and int8 weights:
// a 4-row int8 backbone step 1.6 ms -> see the benchmark); a single row stays on the GEMV
#define G16_MIN_ROWS 2

union U128 { uint4 u; bf16x8 v; };

__device__ __forceinline__ void cvt8u(const uint4& r, float* o) {
  o[0] = __uint_as_float(r.x << 16); o[1] = __uint_as_float(r.x & 0xffff0000u);
  o[2] = __uint_as_float(r.y << 16); o[3] = __uint_as_float(r.y & 0xffff0000u);
  o[4] = __uint_as_float(r.z << 16); o[5] = __uint_as_float(r.z & 0xffff0000u);
  o[6] = __uint_as_float(r.w << 16); o[7] = __uint_as_float(r.w & 0xffff0000u);
}

__device__ __forceinline__ bf16x8 as_bf16x8(const uint4& x) { U128 t; t.u = x; return t.v; }

// 8 int8 (two dwords) -> 8 bf16, exact
__device__ __forceinline__ uint4 i8x8_to_bf16(uint32_t lo, uint32_t hi) {
  auto cv = [](uint32_t w, int sh) -> uint32_t {
    const float f = (float)(int8_t)((w >> sh) & 0xff);
    return __float_as_uint(f) >> 16;
  };
  uint4 r;
  r.x = cv(lo, 0) | (cv(lo, 8) << 16);
  r.y = cv(lo, 16) | (cv(lo, 24) << 16);
  r.z = cv(hi, 0) | (cv(hi, 8) << 16);
  r.w = cv(hi, 16) | (cv(hi, 24) << 16);
  return r;
}

template <typename WT> struct W16;
template <> struct W16<bf16_t> {
  struct Raw { uint4 lo, hi; };
  static __device__ __forceinline__ Raw load(const bf16_t* p) {
    Raw r; r.lo = *reinterpret_cast<const uint4*>(p); r.hi = *reinterpret_cast<const uint4*>(p + 8); return r;
  }
  static __device__ __forceinline__ Raw zero() { Raw r; r.lo = make_uint4(0, 0, 0, 0); r.hi = r.lo; return r; }
  static __device__ __forceinline__ void split(const Raw& r, uint4& a, uint4& b) { a = r.lo; b = r.hi; }
};
template <> struct W16<int8_t> {
  typedef uint4 Raw;  // 16 int8
  static __device__ __forceinline__ Raw load(const int8_t* p) { return *reinterpret_cast<const uint4*>(p); }
  static __device__ __forceinline__ Raw zero() { return make_uint4(0, 0, 0, 0); }
  static __device__ __forceinline__ void split(const Raw& r, uint4& a, uint4& b) {
    a = i8x8_to_bf16(r.x, r.y); b = i8x8_to_bf16(r.z, r.w);
  }
};

// ---- epilogue of four consecutive features of one row (the lane's share of the 16 x 16 tile) ----
// Same arithmetic and rounding points as epilogue() of gemv_epi.h, for the forms the batch step uses, with what it
// reads fetched ahead (epi_prefetch) and one 8-byte store instead of four 2-byte ones.
struct EpiPre {
  uint2 sc, sc2, res;  // four bf16 each: scales of the two matrices, residual values
  float4 f0, f1;       // (cos, sin) of dims dd, dd + 1 and dd + 2, dd + 3
  int slot, pos;
};
__device__ __forceinline__ bool epi_fast(const GemvArgs& p) {
  if ((p.N & 3) || (p.ldy & 3)) return false;
  if (p.epi == EPI_STORE || p.epi == EPI_RESID || p.epi == EPI_SWIGLU) return true;
  return p.epi == EPI_QKV && !((p.nq | p.nkv | p.hd | p.rope_dim) & 3) && p.rope_dim >= 4;  // a group of four rotates as a whole or not at all
}
// region of feature n of the fused projection: 0 q, 1 k, 2 v; m = index inside the region
__device__ __forceinline__ int qkv_region(const GemvArgs& p, int n, int& m) {
  if (n < p.nq) { m = n; return 0; }
  if (n < p.nq + p.nkv) { m = n - p.nq; return 1; }
  m = n - p.nq - p.nkv;
  return 2;
}
template <bool DUAL>
__device__ __forceinline__ void epi_prefetch(const GemvArgs& p, bool fast, int eb, int en, EpiPre& e) {
  e.sc = e.sc2 = e.res = make_uint2(0, 0);
  e.f0 = e.f1 = make_float4(1.f, 0.f, 1.f, 0.f);
  e.slot = eb; e.pos = 0;
  if (!fast) return;  // uniform
  if (p.w_int8) {
    e.sc = *reinterpret_cast<const uint2*>((const bf16_t*)p.sc + en);
    if (DUAL) e.sc2 = *reinterpret_cast<const uint2*>((const bf16_t*)p.sc2 + en);
  }
  if (p.epi == EPI_RESID) e.res = *reinterpret_cast<const uint2*>((const bf16_t*)p.resid + (size_t)eb * p.ldy + en);
  if (p.epi == EPI_QKV) {
    // slot and position of every row through uniform addresses (the scalar unit fetches them, beside the queue of
    // vector loads and in no order with it), then this lane's pair by selection
    int sl[16], ps[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) sl[i] = min(i, p.B - 1);
    if (p.slot_idx) {
#pragma unroll
      for (int i = 0; i < 16; ++i) sl[i] = p.slot_idx[sl[i]];
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) ps[i] = p.seq_lens[sl[i]];
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (eb == i) { e.slot = sl[i]; e.pos = ps[i]; }
    int m;
    qkv_region(p, en, m);
    const int dd = min(m % p.hd, p.rope_dim - 4);           // clamped: unused where the dims are not rotated
    const int pc = min(max(e.pos, 0), p.S - 1);
    const float* f = p.rope + ((size_t)pc * p.rope_dim + dd) * 2;
    e.f0 = *reinterpret_cast<const float4*>(f);
    e.f1 = *reinterpret_cast<const float4*>(f + 4);
  }
}
template <bool DUAL>
__device__ __forceinline__ void epi_fast4(const GemvArgs& p, const EpiPre& e, int b, int n, const float* v, const float* v2) {
  float a[4], a2[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) { a[r] = v[r]; a2[r] = DUAL ? v2[r] : 0.f; }
  if (p.w_int8) {
    a[0] *= bf_lo(e.sc.x); a[1] *= bf_hi(e.sc.x); a[2] *= bf_lo(e.sc.y); a[3] *= bf_hi(e.sc.y);
    if (DUAL) { a2[0] *= bf_lo(e.sc2.x); a2[1] *= bf_hi(e.sc2.x); a2[2] *= bf_lo(e.sc2.y); a2[3] *= bf_hi(e.sc2.y); }
  }
  bf16_t* y = (bf16_t*)p.y;
  float o[4];
  bf16_t* dst = y + (size_t)b * p.ldy + n;
  if (p.epi == EPI_STORE) {
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] = a[r];
  } else if (p.epi == EPI_RESID) {
    const float rs[4] = {bf_lo(e.res.x), bf_hi(e.res.x), bf_lo(e.res.y), bf_hi(e.res.y)};
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] = rs[r] + El<bf16_t>::rnd(a[r]);
  } else if (p.epi == EPI_SWIGLU) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float g = El<bf16_t>::rnd(a[r]), c = El<bf16_t>::rnd(a2[r]);
      o[r] = El<bf16_t>::rnd(g / (1.0f + expf(-g))) * c;
    }
  } else {  // EPI_QKV
    int m;
    const int region = qkv_region(p, n, m);
    const int dd = m % p.hd;
    const bool in_cache = e.pos >= 0 && e.pos < p.S;
    const float cs[4] = {e.f0.x, e.f0.z, e.f1.x, e.f1.z}, sn[4] = {e.f0.y, e.f0.w, e.f1.y, e.f1.w};
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float val = El<bf16_t>::rnd(a[r]);
      if (region != 2 && dd + r < p.rope_dim && in_cache) {
        const float partner = El<bf16_t>::rnd(a[r ^ 1]);
        val = rope_mix(val, cs[r], (r & 1) ? partner : -partner, sn[r]);
      }
      o[r] = val;
    }
    if (region == 0) dst = y + (size_t)b * p.ldy + m;
    else {
      if (!in_cache) return;
      dst = (bf16_t*)(region == 1 ? p.kc : p.vc) + ((size_t)e.slot * p.S + e.pos) * p.nkv + m;
    }
  }
  *reinterpret_cast<uint2*>(dst) = make_uint2(f2bf2(o[0], o[1]), f2bf2(o[2], o[3]));
}

template <typename WT, bool DUAL>
__global__ __launch_bounds__(G16_THREADS) void gemm16_kernel(const GemvArgs p) {
  extern __shared__ __align__(16) unsigned char smem16[];
  const int K = p.K, KP = K + 8;
  bf16_t* xs = (bf16_t*)smem16;                       // 16 x KP
  float* red = (float*)(smem16 + (size_t)16 * KP * 2);  // 4 waves x 64 lanes x (4 | 8)
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int f16 = lane & 15, kg = lane >> 4;
  const int n0 = (int)blockIdx.x * 16;
  const int row = min(n0 + f16, p.N - 1);
  const int nsteps = (K + 63) >> 6;

  // this wave's weight tiles: steps wave, wave + 4, ...
  typename W16<WT>::Raw wr[G16_MAXS], wr2[DUAL ? G16_MAXS : 1];
  const WT* wrow = (const WT*)p.W + (size_t)row * K;
  const WT* wrow2 = DUAL ? (const WT*)p.W2 + (size_t)row * K : nullptr;
#pragma unroll
  for (int i = 0; i < G16_MAXS; ++i) {
    const int k = (wave + 4 * i) * 64 + kg * 16;
    const bool on = (wave + 4 * i) < nsteps && k < K;  // K is a multiple of 16 here
    wr[i] = on ? W16<WT>::load(wrow + k) : W16<WT>::zero();
    if (DUAL) wr2[i] = on ? W16<WT>::load(wrow2 + k) : W16<WT>::zero();
  }

  // What the epilogue of this lane will need (row f16, features n0 + 4 kg ... + 3) is requested now, behind the
  // weights: scales, the residual values, the row's position and its rotation factors.  Written as part of the
  // epilogue they were a chain of small dependent loads, each waited for in turn, after everything else was done.
  // Every wave runs this (only wave 0 uses it): no branch, so the loads go out together with the rest (the call
  // sits below, between the requests for the activations and their use).
  const bool fast = epi_fast(p);
  const int eb = min(f16, p.B - 1), en = fast ? min(n0 + 4 * kg, p.N - 4) : 0;
  EpiPre pre;

  // activations -> LDS (bf16), rows >= B are zero.  A wave stages rows wave, wave+4, ...: all their
  // 16-byte chunks (and the norm weights) are requested first, then normalised and written.
  {
    const bf16_t* x = (const bf16_t*)p.x;
    const bf16_t* nw = (const bf16_t*)p.norm_w;
    const int nch = K >> 3;  // 8-element chunks per row (K is a multiple of 16)
    uint4 xr[4][4], wn[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = lane + WAVE * i;
      wn[i] = (nw && c < nch) ? *reinterpret_cast<const uint4*>(nw + c * 8) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int b = wave + 4 * j;
        xr[j][i] = (b < p.B && c < nch) ? *reinterpret_cast<const uint4*>(x + (size_t)b * K + c * 8) : make_uint4(0, 0, 0, 0);
      }
    }
    epi_prefetch<DUAL>(p, fast, eb, en, pre);  // behind the weights and activations in the queue
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int b = wave + 4 * j;
      bf16_t* dst = xs + (size_t)b * KP;
      float r = 1.f;
      if (nw) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v8[8];
          cvt8u(xr[j][i], v8);
#pragma unroll
          for (int e = 0; e < 8; ++e) ss = fmaf(v8[e], v8[e], ss);
        }
        ss = wave_sum(ss);
        r = 1.0f / sqrtf(ss / (float)K + p.eps);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + WAVE * i;
        if (c < nch) {
          uint4 o = xr[j][i];
          if (nw) {
            float v8[8], w8[8], y8[8];
            cvt8u(xr[j][i], v8);
            cvt8u(wn[i], w8);
#pragma unroll
            for (int e = 0; e < 8; ++e) y8[e] = bf2f(f2bf(v8[e] * r)) * w8[e];
            o.x = (uint32_t)f2bf(y8[0]) | ((uint32_t)f2bf(y8[1]) << 16);
            o.y = (uint32_t)f2bf(y8[2]) | ((uint32_t)f2bf(y8[3]) << 16);
            o.z = (uint32_t)f2bf(y8[4]) | ((uint32_t)f2bf(y8[5]) << 16);
            o.w = (uint32_t)f2bf(y8[6]) | ((uint32_t)f2bf(y8[7]) << 16);
          }
          *reinterpret_cast<uint4*>(dst + c * 8) = o;
        }
      }
    }
  }
  __syncthreads();

  floatx4 acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < G16_MAXS; ++i) {
    const int step = wave + 4 * i;
    if (step < nsteps) {  // uniform over the wave
      // The matrix instructions run for all 64 lanes whatever the lanes' own conditions say, so nothing here may sit
      // behind a per-lane branch: a lane whose 16 columns lie beyond K (the last step of a K that is no multiple of 64)
      // holds zero weights (set when they were requested) and reads a staged chunk that exists.
      const int k = min(step * 64 + kg * 16, K - 16);
      const bf16_t* xp = xs + (size_t)f16 * KP + k;
      const uint4 b_lo = *reinterpret_cast<const uint4*>(xp);
      const uint4 b_hi = *reinterpret_cast<const uint4*>(xp + 8);
      uint4 a_lo, a_hi;
      W16<WT>::split(wr[i], a_lo, a_hi);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a_lo), as_bf16x8(b_lo), acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a_hi), as_bf16x8(b_hi), acc, 0, 0, 0);
      if (DUAL) {
        W16<WT>::split(wr2[i], a_lo, a_hi);
        acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a_lo), as_bf16x8(b_lo), acc2, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a_hi), as_bf16x8(b_hi), acc2, 0, 0, 0);
      }
    }
  }
  // add the four K parts in a fixed order
  const int per = DUAL ? 8 : 4;
  float* mine = red + ((size_t)wave * 64 + lane) * per;
#pragma unroll
  for (int r = 0; r < 4; ++r) { mine[r] = acc[r]; if (DUAL) mine[4 + r] = acc2[r]; }
  __syncthreads();
  if (wave != 0) return;
  float v[4], v2[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    v[r] = 0.f; v2[r] = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      v[r] += red[((size_t)w * 64 + lane) * per + r];
      if (DUAL) v2[r] += red[((size_t)w * 64 + lane) * per + 4 + r];
    }
  }
  // lane holds features n0 + 4 * kg + r (r = 0..3) of activation row f16
  const int b = f16;
  if (b >= p.B) return;
  if (fast) {
    if (n0 + 4 * kg < p.N) epi_fast4<DUAL>(p, pre, b, n0 + 4 * kg, v, v2);
    return;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int n = n0 + 4 * kg + r;
    if (n < p.N) {
      float a = v[r], ap = v[r ^ 1], a2 = v2[r];
      if (p.w_int8) {
        a *= bf2f(((const bf16_t*)p.sc)[n]);
        ap *= bf2f(((const bf16_t*)p.sc)[min(n ^ 1, p.N - 1)]);
        if (DUAL) a2 *= bf2f(((const bf16_t*)p.sc2)[n]);
      }
      epilogue<bf16_t>(p, n, b, a, ap, a2);
    }
  }
}

static size_t g16_lds(int K, bool dual) { return (size_t)16 * (K + 8) * 2 + (size_t)4 * 64 * (dual ? 8 : 4) * 4; }

template <typename WT, bool DUAL>
static int launch_g16(const GemvArgs& a, hipStream_t st) {
  static size_t attr = 0;
  const size_t lds = g16_lds(a.K, DUAL);
  if (lds > 64 * 1024 && lds > attr) {
    HIP_TRY(hipFuncSetAttribute((const void*)gemm16_kernel<WT, DUAL>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr = lds;
  }
  hipLaunchKernelGGL((gemm16_kernel<WT, DUAL>), dim3((a.N + 15) / 16), dim3(G16_THREADS), lds, st, a);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

bool gemm16_supported(const GemvArgs& a) {
  return a.dtype == VUI_DTYPE_BF16 && a.B >= G16_MIN_ROWS && a.B <= 16 && (a.K % 16) == 0 && a.K <= G16_MAXS * 4 * 64 &&
         g16_lds(a.K, a.epi == EPI_SWIGLU) <= 150 * 1024;
}

int launch_gemm16(const GemvArgs& a, hipStream_t st) {
  const bool dual = a.epi == EPI_SWIGLU;
  if (a.w_int8) return dual ? launch_g16<int8_t, true>(a, st) : launch_g16<int8_t, false>(a, st);
  return dual ? launch_g16<bf16_t, true>(a, st) : launch_g16<bf16_t, false>(a, st);
}
