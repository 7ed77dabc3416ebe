// Fused [RMSNorm ->] GEMV [-> epilogue] for a handful of activation rows (decode: B = 1..16).
//
// y[b, n] = sum_k W[n, k] * xn[b, k]: the weight matrix is streamed once from HBM with
// 16-byte loads per lane, the normalised activations sit in LDS as fp32, the accumulation is
// fp32.  One wave owns two adjacent output rows (an interleaved-RoPE pair); all weight
// loads of a wave are issued before the normalisation prologue so the HBM latency overlaps it.
//
// Reference arithmetic (rounding points): RMSNorm.forward src/vui/model.py:286-297,
// nn.Linear at :158/:220/:258/:282-283, apply_rotary_emb src/vui/rope.py:23-57,
// KV append of flash_attn_with_kvcache model.py:247-257.
#include "common.h"
#include "internal.h"
#include "gemv_epi.h"

#define RPW 2            // output rows per wave
#define GEMV_THREADS 128 // two waves per workgroup -> 4 rows per workgroup

template <typename WT> struct WL;
template <> struct WL<bf16_t> {
  typedef uint4 Raw;
  static __device__ __forceinline__ Raw load(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
  static __device__ __forceinline__ Raw zero() { return make_uint4(0, 0, 0, 0); }
  static __device__ __forceinline__ void cvt(const Raw& r, float* o) {
    o[0] = __uint_as_float(r.x << 16); o[1] = __uint_as_float(r.x & 0xffff0000u);
    o[2] = __uint_as_float(r.y << 16); o[3] = __uint_as_float(r.y & 0xffff0000u);
    o[4] = __uint_as_float(r.z << 16); o[5] = __uint_as_float(r.z & 0xffff0000u);
    o[6] = __uint_as_float(r.w << 16); o[7] = __uint_as_float(r.w & 0xffff0000u);
  }
};
template <> struct WL<float> {
  struct Raw { float4 a, b; };
  static __device__ __forceinline__ Raw load(const float* p) {
    Raw r; r.a = *reinterpret_cast<const float4*>(p); r.b = *reinterpret_cast<const float4*>(p + 4); return r;
  }
  static __device__ __forceinline__ Raw zero() { Raw r; r.a = make_float4(0, 0, 0, 0); r.b = r.a; return r; }
  static __device__ __forceinline__ void cvt(const Raw& r, float* o) {
    o[0] = r.a.x; o[1] = r.a.y; o[2] = r.a.z; o[3] = r.a.w; o[4] = r.b.x; o[5] = r.b.y; o[6] = r.b.z; o[7] = r.b.w;
  }
};
template <> struct WL<int8_t> {
  typedef uint2 Raw;
  static __device__ __forceinline__ Raw load(const int8_t* p) { return *reinterpret_cast<const uint2*>(p); }
  static __device__ __forceinline__ Raw zero() { return make_uint2(0, 0); }
  static __device__ __forceinline__ void cvt(const Raw& r, float* o) {
    o[0] = (float)(int8_t)(r.x & 0xff); o[1] = (float)(int8_t)((r.x >> 8) & 0xff);
    o[2] = (float)(int8_t)((r.x >> 16) & 0xff); o[3] = (float)(int8_t)(r.x >> 24);
    o[4] = (float)(int8_t)(r.y & 0xff); o[5] = (float)(int8_t)((r.y >> 8) & 0xff);
    o[6] = (float)(int8_t)((r.y >> 16) & 0xff); o[7] = (float)(int8_t)(r.y >> 24);
  }
};

// activations (B, K) -> LDS fp32, with the two-rounding RMSNorm when norm_w is given
template <typename T>
__device__ __forceinline__ void stage_x(const GemvArgs& p, float* xs, int nb) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const T* x = (const T*)p.x;
  const T* nw_ = (const T*)p.norm_w;
  for (int b = wave; b < nb; b += nw) {
    const T* xr = x + (size_t)b * p.K;
    if (nw_) {
      float ss = 0.f;
      for (int k = lane; k < p.K; k += WAVE) { float v = El<T>::ld(xr + k); ss += v * v; }
      ss = wave_sum(ss);
      const float r = 1.0f / sqrtf(ss / (float)p.K + p.eps);
      for (int k = lane; k < p.K; k += WAVE) {
        float v = El<T>::rnd(El<T>::ld(xr + k) * r);
        xs[b * p.K + k] = El<T>::rnd(v * El<T>::ld(nw_ + k));
      }
    } else {
      for (int k = lane; k < p.K; k += WAVE) xs[b * p.K + k] = El<T>::ld(xr + k);
    }
  }
}

template <typename T, typename WT, int NB, int MAXC, bool DUAL>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_kernel(const GemvArgs p, const int b0_in, const int nb_in) {
  extern __shared__ float xs[];
  // N == 0: only the extra outputs are wanted (the matrix cores did the rest); one row per workgroup then,
  // instead of one workgroup walking through eight rows
  const int b0 = p.N == 0 ? (int)blockIdx.x : b0_in, nb_rt = p.N == 0 ? 1 : nb_in;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int nch = p.K >> 3;
  const int nmain = (p.N + 2 * RPW - 1) / (2 * RPW);
  GemvArgs q = p;  // batch tile view
  q.x = (const T*)p.x + (size_t)b0 * p.K;
  const bool extra = (int)blockIdx.x >= nmain;

  typename WL<WT>::Raw wr[RPW][MAXC];
  typename WL<WT>::Raw wr2[DUAL ? RPW : 1][DUAL ? MAXC : 1];
  const int r0 = ((int)blockIdx.x * 2 + wave) * RPW;
  if (!extra) {
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      const int row = min(r0 + r, p.N - 1);
      const WT* wrow = (const WT*)p.W + (size_t)row * p.K;
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = lane + WAVE * i;
        wr[r][i] = (c < nch) ? WL<WT>::load(wrow + c * 8) : WL<WT>::zero();
      }
      if (DUAL) {
        const WT* wrow2 = (const WT*)p.W2 + (size_t)row * p.K;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
          const int c = lane + WAVE * i;
          wr2[r][i] = (c < nch) ? WL<WT>::load(wrow2 + c * 8) : WL<WT>::zero();
        }
      }
    }
  }

  stage_x<T>(q, xs, nb_rt);
  __syncthreads();

  if (extra) {
    // the single extra output row (eos head) and the position update
    if (p.hid_out)
      for (int i = threadIdx.x; i < nb_rt * p.K; i += blockDim.x)
        El<T>::st((T*)p.hid_out + (size_t)b0 * p.K + i, xs[i]);
    if (wave == 0) {
      const T* wx = (const T*)p.Wx;
      for (int b = 0; b < nb_rt; ++b) {
        float a = 0.f;
        for (int k = lane; k < p.K; k += WAVE) a += xs[b * p.K + k] * El<T>::ld(wx + k);
        a = wave_sum(a);
        if (lane == 0) El<T>::st((T*)p.yx + b0 + b, a + El<T>::ld((const T*)p.bx));
      }
    } else if (p.upd_seq_lens && b0 == 0) {
      if (p.upd_seq_inc) {
        for (int s = lane; s < p.n_slots; s += WAVE) p.upd_seq_lens[s] += p.upd_seq_inc[s];
      } else {
        for (int b = lane; b < p.B; b += WAVE) atomicAdd(&p.upd_seq_lens[p.slot_idx ? p.slot_idx[b] : b], 1);
      }
    }
    return;
  }

  float acc[RPW][NB], acc2[DUAL ? RPW : 1][DUAL ? NB : 1];
#pragma unroll
  for (int r = 0; r < RPW; ++r)
#pragma unroll
    for (int b = 0; b < NB; ++b) { acc[r][b] = 0.f; if (DUAL) acc2[r][b] = 0.f; }

#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int c = lane + WAVE * i;
    if (c < nch) {
      float w[RPW][8], w2[DUAL ? RPW : 1][8];
#pragma unroll
      for (int r = 0; r < RPW; ++r) { WL<WT>::cvt(wr[r][i], w[r]); if (DUAL) WL<WT>::cvt(wr2[r][i], w2[r]); }
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        if (b < nb_rt) {
          const float4 xa = *reinterpret_cast<const float4*>(xs + b * p.K + c * 8);
          const float4 xb = *reinterpret_cast<const float4*>(xs + b * p.K + c * 8 + 4);
          const float xv[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
          for (int r = 0; r < RPW; ++r) {
            float s = acc[r][b];
#pragma unroll
            for (int e = 0; e < 8; ++e) s = fmaf(w[r][e], xv[e], s);
            acc[r][b] = s;
            if (DUAL) {
              float s2 = acc2[r][b];
#pragma unroll
              for (int e = 0; e < 8; ++e) s2 = fmaf(w2[r][e], xv[e], s2);
              acc2[r][b] = s2;
            }
          }
        }
      }
    }
  }

  float v = 0.f, vp = 0.f, v2 = 0.f;
#pragma unroll
  for (int r = 0; r < RPW; ++r)
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const float s = wave_sum(acc[r][b]);
      float s2 = 0.f;
      if (DUAL) s2 = wave_sum(acc2[r][b]);
      if (lane == r * NB + b) { v = s; v2 = s2; }
      if (lane == (r ^ 1) * NB + b) vp = s;
    }
  if (lane < RPW * NB) {
    const int r = lane / NB, b = lane % NB;
    const int n = r0 + r;
    if (b < nb_rt && n < p.N) {
      if (p.w_int8) {
        v *= El<T>::ld((const T*)p.sc + n);
        vp *= El<T>::ld((const T*)p.sc + min(n ^ 1, p.N - 1));
        if (DUAL) v2 *= El<T>::ld((const T*)p.sc2 + n);
      }
      epilogue<T>(p, n, b0 + b, v, vp, v2);
    }
  }
}

template <typename T, typename WT, int NB, int MAXC, bool DUAL>
static int launch_one(const GemvArgs& a, int b0, int nb, hipStream_t st) {
  const int nmain = (a.N + 2 * RPW - 1) / (2 * RPW);
  const int grid = a.N == 0 ? a.B : nmain + ((a.Wx && b0 >= 0) ? 1 : 0);
  const size_t lds = (size_t)nb * a.K * sizeof(float);
  hipLaunchKernelGGL((gemv_kernel<T, WT, NB, MAXC, DUAL>), dim3(grid), dim3(GEMV_THREADS), lds, st, a, b0, nb);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

template <typename T, typename WT, int NB, bool DUAL>
static int pick_c(const GemvArgs& a, int b0, int nb, hipStream_t st) {
  const int per_lane = ((a.K >> 3) + WAVE - 1) / WAVE;
  if (per_lane <= 2) return launch_one<T, WT, NB, 2, DUAL>(a, b0, nb, st);
  if (per_lane <= 4) return launch_one<T, WT, NB, 4, DUAL>(a, b0, nb, st);
  if (!DUAL && per_lane <= 8) return launch_one<T, WT, NB, DUAL ? 4 : 8, DUAL>(a, b0, nb, st);
  vui_set_error("gemv: K=%d too large (max %d)", a.K, DUAL ? 2048 : 4096);
  return VUI_EINVAL;
}

template <typename T, typename WT, bool DUAL>
static int pick_nb(const GemvArgs& a, int b0, int nb, hipStream_t st) {
  if (nb <= 1) return pick_c<T, WT, 1, DUAL>(a, b0, nb, st);
  if (nb <= 2) return pick_c<T, WT, 2, DUAL>(a, b0, nb, st);
  if (nb <= 4) return pick_c<T, WT, 4, DUAL>(a, b0, nb, st);
  return pick_c<T, WT, 8, DUAL>(a, b0, nb, st);
}

int launch_gemv(const GemvArgs& a, hipStream_t st) {
  if (a.B < 1 || a.N < 1 || a.K < 8 || (a.K & 7)) {
    vui_set_error("gemv: bad shape B=%d N=%d K=%d (K must be a multiple of 8)", a.B, a.N, a.K);
    return VUI_EINVAL;
  }
  if ((a.epi == EPI_QKV) && ((a.hd & 1) || (a.rope_dim & 1) || (a.N & 1))) {
    vui_set_error("gemv: rotary pairs need even head_dim/rope_dim");
    return VUI_EINVAL;
  }
  const bool dual = a.epi == EPI_SWIGLU;
  if (gemm16_supported(a)) {
    // 2..16 rows: the matrix-core form computes the N outputs; the extra row and the position
    // update, if any, go through this kernel's extra block alone (N = 0 main blocks)
    int rc = launch_gemm16(a, st);
    if (rc || !a.Wx) return rc;
    GemvArgs x = a;
    x.N = 0;
    return pick_nb<bf16_t, bf16_t, false>(x, 0, 1, st);
  }
  // batch tile: at most 8 rows and at most 64 KiB of LDS
  int tile = 8;
  while (tile > 1 && (size_t)tile * a.K * sizeof(float) > 65536) tile >>= 1;
  for (int b0 = 0; b0 < a.B; b0 += tile) {
    const int nb = (a.B - b0 < tile) ? a.B - b0 : tile;
    int rc;
    if (a.dtype == VUI_DTYPE_F32) {
      if (a.w_int8) { vui_set_error("gemv: int8 weights need bf16 activations"); return VUI_EINVAL; }
      rc = dual ? pick_nb<float, float, true>(a, b0, nb, st) : pick_nb<float, float, false>(a, b0, nb, st);
    } else if (a.w_int8) {
      rc = dual ? pick_nb<bf16_t, int8_t, true>(a, b0, nb, st) : pick_nb<bf16_t, int8_t, false>(a, b0, nb, st);
    } else {
      rc = dual ? pick_nb<bf16_t, bf16_t, true>(a, b0, nb, st) : pick_nb<bf16_t, bf16_t, false>(a, b0, nb, st);
    }
    if (rc) return rc;
  }
  return VUI_OK;
}
