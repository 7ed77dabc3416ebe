// Decode attention over the backbone KV cache (one new query per row) and the tiny
// attention of the depth head.
//
// Backbone: caches are (slots, S, KV, hd); the key range [start, len) of a (row, head) is cut
// into n_splits contiguous pieces, one workgroup each.  A group of 16 lanes owns one key
// (8 features per lane, 16-byte loads), so a 256-thread workgroup works on 16 keys at a time, and
// every group has four keys AND their values in flight per step: one pass with a running maximum
// (scores never go to memory).  The 16 groups are merged through LDS into the piece's
// (max, sum, acc[hd]).  Pieces of a (row, head) meet in memory: each workgroup writes its piece with
// device-scope write-through stores, waits for them to complete and bumps an arrival counter; the
// last arriver merges all pieces in piece order and writes the output (and zeroes the counter for
// the next launch).  No second kernel, no cache flush.
//
// Reference: flash_attn_with_kvcache call in MHA.forward_flash, src/vui/model.py:242-258
// (causal, one query at position seq_len; window (w, 0)); F.scaled_dot_product_attention in
// RQTransformer._gkv_step, model.py:899-902.
#include "common.h"
#include "internal.h"

#define ATT_THREADS 256
#define ATT_KEYS_PER_ITER 16  // 4 waves x 4 lane-groups

template <typename T>
__global__ __launch_bounds__(ATT_THREADS) void decode_attn_kernel(const AttnArgs p) {
  __shared__ float gm[ATT_KEYS_PER_ITER], gl[ATT_KEYS_PER_ITER], gw[ATT_KEYS_PER_ITER];
  __shared__ float gacc[ATT_KEYS_PER_ITER][128];
  __shared__ __align__(8) float fin[130];  // max, sum, acc[hd]
  __shared__ int s_last;

  const int b = blockIdx.z, h = blockIdx.y, sp = blockIdx.x;
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, grp = lane >> 4, l16 = lane & 15;
  const int g = wave * 4 + grp;  // 0..15 key lane-group inside the workgroup
  const int hd = p.hd;
  const int slot = p.slot_idx ? p.slot_idx[b] : b;
  int len = p.seq_lens[slot] + 1;
  len = max(1, min(len, p.S));
  const int start = (p.window > 0) ? max(0, len - 1 - p.window) : 0;
  const int n = len - start;
  int chunk = (n + p.n_splits - 1) / p.n_splits;
  chunk = (chunk + ATT_KEYS_PER_ITER - 1) / ATT_KEYS_PER_ITER * ATT_KEYS_PER_ITER;
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
  // lanes beyond head_dim read the head's first elements instead (their q is zero and their sums are dropped)
  const T* kbase = (const T*)p.kc + ((size_t)slot * p.S) * rowstride + kvh * hd + (act ? l16 * 8 : 0);
  const T* vbase = (const T*)p.vc + ((size_t)slot * p.S) * rowstride + kvh * hd + (act ? l16 * 8 : 0);

  float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  for (int j0 = lo + g; j0 < hi; j0 += 4 * ATT_KEYS_PER_ITER) {
    // Eight loads in flight per lane, none behind a branch (a guarded load is waited for inside its branch, one
    // at a time): a key beyond the piece reads the piece's last key instead and gets weight exp(-inf) = 0 below.
    float k8[4][8], v8[4][8];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = min(j0 + u * ATT_KEYS_PER_ITER, hi - 1);
      El<T>::ld8(kbase + (size_t)j * rowstride, k8[u]);
      El<T>::ld8(vbase + (size_t)j * rowstride, v8[u]);
    }
    float s[4];
    float mn = m;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float d = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) d = fmaf(q8[e], k8[u][e], d);
      d = group16_sum(d) * scale;
      s[u] = (j0 + u * ATT_KEYS_PER_ITER < hi) ? d : -INFINITY;
      mn = fmaxf(mn, s[u]);
    }
    // j0 < hi: at least one of the four keys is real, so mn is finite
    const float r = expf(m - mn);  // 0 on the first step (m = -inf)
    l *= r;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= r;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float pw = expf(s[u] - mn);  // 0 for a key beyond the piece
      l += pw;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = fmaf(pw, v8[u][e], acc[e]);
    }
    m = mn;
  }
  // the 16 groups of the workgroup -> one piece
  if (l16 == 0) { gm[g] = m; gl[g] = l; }
  if (act) {
#pragma unroll
    for (int e = 0; e < 8; ++e) gacc[g][l16 * 8 + e] = acc[e];
  }
  __syncthreads();
  if (tid < ATT_KEYS_PER_ITER) {
    float M = -INFINITY;
#pragma unroll
    for (int i = 0; i < ATT_KEYS_PER_ITER; ++i) M = fmaxf(M, gm[i]);
    gw[tid] = (gm[tid] == -INFINITY) ? 0.f : expf(gm[tid] - M);
    if (tid == 0) fin[0] = M;
  }
  __syncthreads();
  if (tid < hd) {
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < ATT_KEYS_PER_ITER; ++i) o = fmaf(gw[i], gacc[i][tid], o);
    fin[2 + tid] = o;
  }
  if (tid == 128) {
    float L = 0.f;
#pragma unroll
    for (int i = 0; i < ATT_KEYS_PER_ITER; ++i) L = fmaf(gw[i], gl[i], L);
    fin[1] = L;
  }
  __syncthreads();

  const int pw_ = hd + 2;  // floats per piece (even: hd is a multiple of 8)
  float* pbase = p.part + (((size_t)b * p.H + h) * p.n_splits) * pw_;
  if (p.n_splits > 1) {
    if (tid < pw_ / 2) st_dev(pbase + (size_t)sp * pw_ + 2 * tid, fin[2 * tid], fin[2 * tid + 1]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the write-through stores have completed
    __syncthreads();
    if (tid == 0) {
      uint32_t* cnt = p.counter + (size_t)b * p.H + h;
      const uint32_t old = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = old == (uint32_t)p.n_splits - 1u;
      if (s_last) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
  }
  // merge of the pieces: out = sum_s w_s acc_s / sum_s w_s l_s, w_s = exp(m_s - max m), in piece order.
  // All pieces are fetched into LDS with one round of loads (a chain of dependent device-scope loads
  // would cost a memory round trip each).
  extern __shared__ __align__(8) float pieces[];  // n_splits x (hd + 2)
  if (p.n_splits > 1) {
    const int np = p.n_splits * pw_ / 2;
    for (int i0 = tid; i0 < np; i0 += ATT_THREADS * 8) {
      uint64_t v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) { const int i = i0 + ATT_THREADS * u; v[u] = i < np ? ld_dev(pbase + 2 * i) : 0; }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + ATT_THREADS * u;
        if (i < np) { pieces[2 * i] = lo_f(v[u]); pieces[2 * i + 1] = hi_f(v[u]); }
      }
    }
    __syncthreads();
  }
  if (tid < hd) {
    float o, L;
    if (p.n_splits > 1) {
      float Mx = -INFINITY;
      for (int s0 = 0; s0 < p.n_splits; ++s0) Mx = fmaxf(Mx, pieces[s0 * pw_]);
      o = 0.f; L = 0.f;
      for (int s0 = 0; s0 < p.n_splits; ++s0) {
        const float ms = pieces[s0 * pw_];
        const float w = (ms == -INFINITY) ? 0.f : expf(ms - Mx);
        L = fmaf(w, pieces[s0 * pw_ + 1], L);
        o = fmaf(w, pieces[s0 * pw_ + 2 + tid], o);
      }
    } else {
      o = fin[2 + tid]; L = fin[1];
    }
    El<T>::st((T*)p.out + (size_t)b * p.H * hd + h * hd + tid, o / L);
  }
}

int launch_decode_attn(const AttnArgs& a, hipStream_t st) {
  if (a.hd > 128 || (a.hd & 7) || a.H % a.KV || a.n_splits < 1 || a.B < 1) {
    vui_set_error("decode_attn: unsupported shape hd=%d H=%d KV=%d splits=%d", a.hd, a.H, a.KV, a.n_splits);
    return VUI_EINVAL;
  }
  if (a.n_splits > 1 && (!a.part || !a.counter)) { vui_set_error("decode_attn: split pieces need scratch"); return VUI_EINVAL; }
  dim3 grid(a.n_splits, a.H, a.B);
  const size_t lds = a.n_splits > 1 ? (size_t)a.n_splits * (a.hd + 2) * 4 : 0;  // the pieces, for the last arriver
  if (a.dtype == VUI_DTYPE_F32) hipLaunchKernelGGL(decode_attn_kernel<float>, grid, dim3(ATT_THREADS), lds, st, a);
  else hipLaunchKernelGGL(decode_attn_kernel<bf16_t>, grid, dim3(ATT_THREADS), lds, st, a);
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
