// Decode attention over the backbone KV cache (one new query per row) and the tiny
// attention of the depth head.
//
// Backbone: caches are (slots, S, KV, hd); the key range [start, len) of a (row, head) is cut
// into n_splits contiguous pieces, one workgroup each.  A group of 16 lanes owns one key
// (8 features per lane, 16-byte loads), so a 256-thread workgroup works on 16 keys at a time.
// Scores of the piece go to LDS, the piece maximum is taken over the workgroup, then
// exp-weights multiply V.  Each piece writes (max, sum, acc[hd]); a second small kernel merges the
// pieces of each (row, head) (a kernel boundary is cheaper here than device-scope fences in 256
// workgroups, which cost ~40 us per launch on the eight non-coherent L2s).
//
// Reference: flash_attn_with_kvcache call in MHA.forward_flash, src/vui/model.py:242-258
// (causal, one query at position seq_len; window (w, 0)); F.scaled_dot_product_attention in
// RQTransformer._gkv_step, model.py:899-902.
#include "common.h"
#include "internal.h"

#define ATT_THREADS 256
#define ATT_KEYS_PER_ITER 16  // 4 waves x 4 lane-groups

template <typename T>
__global__ __launch_bounds__(ATT_THREADS) void decode_attn_kernel(const AttnArgs p, const int max_chunk) {
  extern __shared__ float sc[];  // max_chunk scores
  __shared__ float red[ATT_KEYS_PER_ITER];
  __shared__ float accs[4][4][128];
  __shared__ float lsum[ATT_KEYS_PER_ITER];

  const int b = blockIdx.z, h = blockIdx.y, sp = blockIdx.x;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, grp = lane >> 4, l16 = lane & 15;
  const int g = wave * 4 + grp;  // 0..15 key lane-group inside the workgroup
  const int hd = p.hd;
  const int slot = p.slot_idx ? p.slot_idx[b] : b;
  int len = p.seq_lens[slot] + 1;
  len = max(1, min(len, p.S));
  const int start = (p.window > 0) ? max(0, len - 1 - p.window) : 0;
  const int n = len - start;
  int chunk = (n + p.n_splits - 1) / p.n_splits;
  chunk = (chunk + ATT_KEYS_PER_ITER - 1) / ATT_KEYS_PER_ITER * ATT_KEYS_PER_ITER;
  chunk = min(chunk, max_chunk);
  const int lo = start + sp * chunk;
  const int hi = min(lo + chunk, len);
  const int kvh = h / (p.H / p.KV);
  const bool act = l16 * 8 < hd;
  const float scale = 1.0f / sqrtf((float)hd);

  float q8[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) q8[e] = 0.f;
  if (act) El<T>::ld8((const T*)p.q + (size_t)b * p.H * hd + h * hd + l16 * 8, q8);

  const size_t rowstride = (size_t)p.KV * hd;
  const T* kbase = (const T*)p.kc + ((size_t)slot * p.S) * rowstride + kvh * hd + l16 * 8;
  const T* vbase = (const T*)p.vc + ((size_t)slot * p.S) * rowstride + kvh * hd + l16 * 8;

  // pass 1: scores (four keys per lane group in flight)
  float mloc = -INFINITY;
  for (int j0 = lo + g; j0 < hi; j0 += 4 * ATT_KEYS_PER_ITER) {
    float k8[4][8];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u * ATT_KEYS_PER_ITER;
      if (act && j < hi) El<T>::ld8(kbase + (size_t)j * rowstride, k8[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u * ATT_KEYS_PER_ITER;
      if (j < hi) {
        float d = 0.f;
        if (act) {
#pragma unroll
          for (int e = 0; e < 8; ++e) d = fmaf(q8[e], k8[u][e], d);
        }
        d = group16_sum(d) * scale;
        if (l16 == 0) sc[j - lo] = d;
        mloc = fmaxf(mloc, d);
      }
    }
  }
  if (l16 == 0) red[g] = mloc;
  __syncthreads();
  float M = -INFINITY;
#pragma unroll
  for (int i = 0; i < ATT_KEYS_PER_ITER; ++i) M = fmaxf(M, red[i]);

  // pass 2: weights and P.V
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  float l = 0.f;
  for (int j0 = lo + g; j0 < hi; j0 += 4 * ATT_KEYS_PER_ITER) {
    float v8[4][8];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u * ATT_KEYS_PER_ITER;
      if (act && j < hi) El<T>::ld8(vbase + (size_t)j * rowstride, v8[u]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u * ATT_KEYS_PER_ITER;
      if (j < hi) {
        const float pw = expf(sc[j - lo] - M);
        l += pw;
        if (act) {
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] = fmaf(pw, v8[u][e], acc[e]);
        }
      }
    }
  }
  if (act) {
#pragma unroll
    for (int e = 0; e < 8; ++e) accs[wave][grp][l16 * 8 + e] = acc[e];
  }
  if (l16 == 0) lsum[g] = l;
  __syncthreads();

  float* part = p.part + (((size_t)b * p.H + h) * p.n_splits + sp) * (hd + 2);
  if (tid < hd) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int gg = 0; gg < 4; ++gg) s += accs[w][gg][tid];
    part[2 + tid] = s;
  }
  if (tid == 0) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < ATT_KEYS_PER_ITER; ++i) s += lsum[i];
    part[0] = M;
    part[1] = s;
  }

}

// merge of the pieces of one (row, head): out = sum_s w_s acc_s / sum_s w_s l_s, w_s = exp(m_s - max m)
template <typename T>
__global__ __launch_bounds__(128) void attn_merge_kernel(const AttnArgs p) {
  const int b = blockIdx.y, h = blockIdx.x, tid = threadIdx.x;
  const int hd = p.hd;
  const float* pb = p.part + (((size_t)b * p.H + h) * p.n_splits) * (hd + 2);
  if (tid < hd) {
    float Mx = -INFINITY;
    for (int s = 0; s < p.n_splits; ++s) Mx = fmaxf(Mx, pb[(size_t)s * (hd + 2)]);
    float L = 0.f, o = 0.f;
    for (int s = 0; s < p.n_splits; ++s) {
      const float* ps = pb + (size_t)s * (hd + 2);
      const float ms = ps[0];
      const float w = (ms == -INFINITY) ? 0.f : expf(ms - Mx);
      L = fmaf(w, ps[1], L);
      o = fmaf(w, ps[2 + tid], o);
    }
    El<T>::st((T*)p.out + (size_t)b * p.H * hd + h * hd + tid, o / L);
  }
}

int launch_decode_attn(const AttnArgs& a, hipStream_t st) {
  if (a.hd > 128 || (a.hd & 7) || a.H % a.KV || a.n_splits < 1 || a.B < 1) {
    vui_set_error("decode_attn: unsupported shape hd=%d H=%d KV=%d splits=%d", a.hd, a.H, a.KV, a.n_splits);
    return VUI_EINVAL;
  }
  int max_chunk = (a.S + a.n_splits - 1) / a.n_splits;
  max_chunk = (max_chunk + ATT_KEYS_PER_ITER - 1) / ATT_KEYS_PER_ITER * ATT_KEYS_PER_ITER;
  if ((size_t)max_chunk * 4 > 60000) {
    vui_set_error("decode_attn: S=%d needs more than %d key splits", a.S, a.n_splits);
    return VUI_EINVAL;
  }
  dim3 grid(a.n_splits, a.H, a.B);
  dim3 mgrid(a.H, a.B);
  if (a.dtype == VUI_DTYPE_F32) {
    hipLaunchKernelGGL(decode_attn_kernel<float>, grid, dim3(ATT_THREADS), max_chunk * 4, st, a, max_chunk);
    hipLaunchKernelGGL(attn_merge_kernel<float>, mgrid, dim3(128), 0, st, a);
  } else {
    hipLaunchKernelGGL(decode_attn_kernel<bf16_t>, grid, dim3(ATT_THREADS), max_chunk * 4, st, a, max_chunk);
    hipLaunchKernelGGL(attn_merge_kernel<bf16_t>, mgrid, dim3(128), 0, st, a);
  }
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

// ---- append one K/V row per batch row (used by the stand-alone attention entry point) ----
template <typename T>
__global__ void kv_append_kernel(const T* k_new, const T* v_new, T* kc, T* vc, const int32_t* seq_lens,
                                 const int32_t* slot_idx, int KVhd, int S) {
  const int b = blockIdx.x;
  const int slot = slot_idx ? slot_idx[b] : b;
  const int pos = seq_lens[slot];
  if (pos < 0 || pos >= S) return;
  for (int i = threadIdx.x; i < KVhd; i += blockDim.x) {
    kc[((size_t)slot * S + pos) * KVhd + i] = k_new[(size_t)b * KVhd + i];
    vc[((size_t)slot * S + pos) * KVhd + i] = v_new[(size_t)b * KVhd + i];
  }
}

int launch_kv_append(int dtype, const void* k_new, const void* v_new, void* kc, void* vc, const int32_t* seq_lens,
                     const int32_t* slot_idx, int B, int KV, int hd, int S, hipStream_t st) {
  if (dtype == VUI_DTYPE_F32)
    hipLaunchKernelGGL(kv_append_kernel<float>, dim3(B), dim3(256), 0, st, (const float*)k_new, (const float*)v_new,
                       (float*)kc, (float*)vc, seq_lens, slot_idx, KV * hd, S);
  else
    hipLaunchKernelGGL(kv_append_kernel<bf16_t>, dim3(B), dim3(256), 0, st, (const bf16_t*)k_new,
                       (const bf16_t*)v_new, (bf16_t*)kc, (bf16_t*)vc, seq_lens, slot_idx, KV * hd, S);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

// ---- depth-head attention: one wave per (row, head), at most Q (<= 64) keys ----
template <typename T>
__global__ __launch_bounds__(WAVE) void rq_attn_kernel(const RqAttnArgs p) {
  const int b = blockIdx.x / p.heads, h = blockIdx.x % p.heads;
  const int lane = threadIdx.x;
  const int R = p.heads * p.hd;
  const int nk = p.pos + 1;
  const float scale = 1.0f / sqrtf((float)p.hd);
  const T* q = (const T*)p.q + (size_t)b * R + h * p.hd;
  const T* kc = (const T*)p.kc + (size_t)b * p.Q * R + h * p.hd;
  const T* vc = (const T*)p.vc + (size_t)b * p.Q * R + h * p.hd;
  // lanes over features (hd <= 128: two features per lane at most)
  float q0 = (lane < p.hd) ? El<T>::ld(q + lane) : 0.f;
  float q1 = (lane + WAVE < p.hd) ? El<T>::ld(q + lane + WAVE) : 0.f;
  float myscore = -INFINITY;  // lane j keeps the score of key j
  for (int j = 0; j < nk; ++j) {
    float d = 0.f;
    if (lane < p.hd) d = q0 * El<T>::ld(kc + (size_t)j * R + lane);
    if (lane + WAVE < p.hd) d = fmaf(q1, El<T>::ld(kc + (size_t)j * R + lane + WAVE), d);
    d = wave_sum(d) * scale;
    if (lane == j) myscore = d;
  }
  const float M = wave_max(myscore);
  const float pw = (lane < nk) ? expf(myscore - M) : 0.f;
  const float L = wave_sum(pw);
  float o0 = 0.f, o1 = 0.f;
  for (int j = 0; j < nk; ++j) {
    const float pj = __shfl(pw, j, WAVE);
    if (lane < p.hd) o0 = fmaf(pj, El<T>::ld(vc + (size_t)j * R + lane), o0);
    if (lane + WAVE < p.hd) o1 = fmaf(pj, El<T>::ld(vc + (size_t)j * R + lane + WAVE), o1);
  }
  T* out = (T*)p.out + (size_t)b * R + h * p.hd;
  if (lane < p.hd) El<T>::st(out + lane, o0 / L);
  if (lane + WAVE < p.hd) El<T>::st(out + lane + WAVE, o1 / L);
}

int launch_rq_attn(const RqAttnArgs& a, hipStream_t st) {
  if (a.hd > 128 || a.pos < 0 || a.pos >= a.Q || a.Q > WAVE) {
    vui_set_error("rq_attn: unsupported shape hd=%d pos=%d Q=%d", a.hd, a.pos, a.Q);
    return VUI_EINVAL;
  }
  if (a.dtype == VUI_DTYPE_F32)
    hipLaunchKernelGGL(rq_attn_kernel<float>, dim3(a.B * a.heads), dim3(WAVE), 0, st, a);
  else
    hipLaunchKernelGGL(rq_attn_kernel<bf16_t>, dim3(a.B * a.heads), dim3(WAVE), 0, st, a);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}
