// Small kernels around the GEMVs: embedding gather-sum, stand-alone RoPE, the fused
// temperature / top-k / repetition-penalty sampler with a counter-based generator, the depth
// head's token builder and the per-frame bookkeeping.
#include "common.h"
#include "internal.h"
#include "sample.h"

// ---- audio embedding: x[b] = rnd(sum_q table[codes[b,q] + q*CS])   (model.py:559-563) ----
template <typename T>
__global__ void embed_kernel(const int64_t* codes, const T* table, T* x, int Q, int CS, int d) {
  const int b = blockIdx.y;
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= d) return;
  float s = 0.f;
  for (int q0 = 0; q0 < Q; q0 += 16) {  // 16 codes, then their 16 rows, are requested together; summed in codebook order
    int64_t c[16];
    float v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) c[u] = codes[(size_t)b * Q + min(q0 + u, Q - 1)];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int64_t cc = c[u] < 0 ? 0 : (c[u] >= CS ? CS - 1 : c[u]);
      v[u] = El<T>::ld(table + ((size_t)(cc + (int64_t)min(q0 + u, Q - 1) * CS)) * d + k);
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) if (q0 + u < Q) s += v[u];
  }
  El<T>::st(x + (size_t)b * d + k, s);
}

int launch_embed(int dtype, const int64_t* codes, const void* table, void* x, int B, int Q, int CS, int d,
                 hipStream_t st) {
  dim3 grid((d + 255) / 256, B);
  if (dtype == VUI_DTYPE_F32)
    hipLaunchKernelGGL(embed_kernel<float>, grid, dim3(256), 0, st, codes, (const float*)table, (float*)x, Q, CS, d);
  else
    hipLaunchKernelGGL(embed_kernel<bf16_t>, grid, dim3(256), 0, st, codes, (const bf16_t*)table, (bf16_t*)x, Q, CS, d);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

__global__ void copy_bytes_kernel(const uint8_t* src, uint8_t* dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}
int launch_copy_rows(int dtype, const void* src, void* dst, int64_t n, hipStream_t st) {
  const int64_t bytes = n * (dtype == VUI_DTYPE_F32 ? 4 : 2);
  hipLaunchKernelGGL(copy_bytes_kernel, dim3((unsigned)((bytes + 255) / 256)), dim3(256), 0, st, (const uint8_t*)src,
                     (uint8_t*)dst, bytes);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}
int launch_fill_u32(uint32_t* p, uint32_t v, int64_t n, hipStream_t st) {
  hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p, v, n);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

// ---- stand-alone interleaved RoPE (rope.py:16-57), in place on (B, nh, hd) ----
template <typename T>
__global__ void rope_kernel(T* x, const float* table, const int32_t* pos, int nh, int hd, int rope_dim) {
  const int b = blockIdx.x;
  const int p = pos[b];
  for (int i = threadIdx.x; i < nh * (rope_dim / 2); i += blockDim.x) {
    const int h = i / (rope_dim / 2), j = i % (rope_dim / 2);
    T* px = x + ((size_t)b * nh + h) * hd + 2 * j;
    const float x0 = El<T>::ld(px), x1 = El<T>::ld(px + 1);
    const float* f0 = table + ((size_t)p * rope_dim + 2 * j) * 2;
    const float* f1 = f0 + 2;
    El<T>::st(px, rope_mix(x0, f0[0], -x1, f0[1]));
    El<T>::st(px + 1, rope_mix(x1, f1[0], x0, f1[1]));
  }
}
int launch_rope(int dtype, void* x, const float* table, const int32_t* pos, int B, int nh, int hd, int rope_dim,
                hipStream_t st) {
  if ((rope_dim & 1) || rope_dim > hd) { vui_set_error("rope: bad rope_dim %d", rope_dim); return VUI_EINVAL; }
  if (dtype == VUI_DTYPE_F32)
    hipLaunchKernelGGL(rope_kernel<float>, dim3(B), dim3(256), 0, st, (float*)x, table, pos, nh, hd, rope_dim);
  else
    hipLaunchKernelGGL(rope_kernel<bf16_t>, dim3(B), dim3(256), 0, st, (bf16_t*)x, table, pos, nh, hd, rope_dim);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

// ---- sampler: one 256-thread workgroup per row (see sample.h) ----
template <typename T, int EMAX>
__global__ __launch_bounds__(SAMP_THREADS) void sample_kernel(const SampleArgs p) {
  __shared__ SampleShared sh;
  __shared__ __align__(16) int hist[HIST_WORDS];
  __shared__ NucleusShared nuc;
  const int b = blockIdx.x, tid = threadIdx.x;
  const int CS = p.CS;
  const int E = (CS + SAMP_THREADS - 1) / SAMP_THREADS;  // contiguous elements per thread
  const T* lg = (const T*)p.logits + (size_t)b * CS;
  const float s_temp = p.dev ? p.dev->temperature : p.temperature;
  const int s_topk = p.dev ? p.dev->top_k : p.top_k;
  const uint64_t s_seed = p.dev ? p.dev->seed : p.seed;
  const bool greedy = (s_topk == 1) || !(s_temp > 0.f);
  const float div = greedy ? 1.0f : s_temp;
  const int sb = p.state_rows ? p.state_rows[b] : b;  // row of the repetition state and of the random stream
  const float* counts = (p.rep_counts && p.penalty > 1.0f) ? p.rep_counts + (size_t)sb * CS : nullptr;

  // untouched bf16 logits order the elements with 16-bit keys; bias or penalty need all 32 bits
  const bool raw_keys = sizeof(T) == 2 && !p.bias && !counts;
  float l[EMAX];
  uint32_t key[EMAX];
#pragma unroll
  for (int e = 0; e < EMAX; ++e) {
    l[e] = -INFINITY;
    key[e] = 0u;
    const int j = tid * E + e;
    if (e < E && j < CS) {
      const float raw = El<T>::ld(lg + j);
      l[e] = sample_value(raw, p.bias, j, counts, p.penalty, div);
      key[e] = float_key(raw_keys ? raw : l[e]);
    }
  }
  const uint32_t frame = p.frame_ctr ? (uint32_t)p.frame_ctr[0] : 0u;
  const uint32_t rnd = philox_u32(s_seed, frame, (uint32_t)sb, (uint32_t)p.codebook, 0u);
  if (p.top_p > 0.f && !greedy) nucleus_cut<EMAX>(l, key, raw_keys ? 16 : 0, CS, E, p.top_p, nuc);  // uniform over the block
  const int pick = block_sample<EMAX>(l, key, raw_keys ? 16 : 0, CS, E, greedy, s_topk, rnd, (uint32_t)p.codebook, sh, hist, p.exact_k != 0);

  if (tid == 0) {
    p.out[(size_t)b * p.out_stride + p.out_col] = (int64_t)pick;
    if (counts)
      rep_push(p.rep_counts + (size_t)sb * CS, p.rep_hist ? p.rep_hist + (size_t)sb * p.window : nullptr,
               p.rep_pos ? p.rep_pos + sb * 2 : nullptr, p.window, pick);
    if (p.eos_prob) {
      const float z = El<T>::ld((const T*)p.eos_logit + b);
      p.eos_prob[b] = 1.0f / (1.0f + expf(-z));
    }
  }
  for (int j = p.pad_from + tid; j < p.pad_to; j += SAMP_THREADS) p.out[(size_t)b * p.out_stride + j] = 0;
  if (p.tok_out) {
    const T* e = (const T*)p.tok_emb + ((size_t)pick + p.tok_emb_off) * p.R;
    for (int k = tid; k < p.R; k += SAMP_THREADS)
      El<T>::st((T*)p.tok_out + (size_t)b * p.R + k, El<T>::ld(e + k) + El<T>::ld((const T*)p.tok_pos + k));
  }
}

int launch_sample(const SampleArgs& a, hipStream_t st) {
  if (a.CS < 1 || a.CS > SAMP_THREADS * SAMP_MAX_E) {
    vui_set_error("sample: codebook_size %d out of range (max %d)", a.CS, SAMP_THREADS * SAMP_MAX_E);
    return VUI_EINVAL;
  }
  const bool small = a.CS <= SAMP_THREADS * 8;
  if (a.dtype == VUI_DTYPE_F32) {
    if (small) hipLaunchKernelGGL((sample_kernel<float, 8>), dim3(a.B), dim3(SAMP_THREADS), 0, st, a);
    else hipLaunchKernelGGL((sample_kernel<float, SAMP_MAX_E>), dim3(a.B), dim3(SAMP_THREADS), 0, st, a);
  } else {
    if (small) hipLaunchKernelGGL((sample_kernel<bf16_t, 8>), dim3(a.B), dim3(SAMP_THREADS), 0, st, a);
    else hipLaunchKernelGGL((sample_kernel<bf16_t, SAMP_MAX_E>), dim3(a.B), dim3(SAMP_THREADS), 0, st, a);
  }
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

// ---- depth head token from a code: x[b] = rnd(emb[code + off] + pos_vec)   (model.py:922-925, 967-970) ----
template <typename T>
__global__ void rq_token_kernel(const int64_t* code, int64_t off, const T* emb, const T* pos_vec, T* x, int R,
                                int64_t* codes_out, int stride, int CS) {
  const int b = blockIdx.x;
  int64_t c = code[b];
  c = c < 0 ? 0 : (c >= CS ? CS - 1 : c);
  const T* e = emb + (size_t)(c + off) * R;
  for (int k = threadIdx.x; k < R; k += blockDim.x)
    El<T>::st(x + (size_t)b * R + k, El<T>::ld(e + k) + El<T>::ld(pos_vec + k));
  if (codes_out && threadIdx.x == 0) codes_out[(size_t)b * stride] = c;
}
int launch_rq_token(int dtype, const int64_t* code, int64_t off, const void* emb, const void* pos_vec, void* x,
                    int B, int R, int64_t* codes_out, int stride, int CS, hipStream_t st) {
  if (dtype == VUI_DTYPE_F32)
    hipLaunchKernelGGL(rq_token_kernel<float>, dim3(B), dim3(256), 0, st, code, off, (const float*)emb,
                       (const float*)pos_vec, (float*)x, R, codes_out, stride, CS);
  else
    hipLaunchKernelGGL(rq_token_kernel<bf16_t>, dim3(B), dim3(256), 0, st, code, off, (const bf16_t*)emb,
                       (const bf16_t*)pos_vec, (bf16_t*)x, R, codes_out, stride, CS);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

// out[b] = rnd(rnd(a[b]) + vec)   (depth head token 0 when backbone_proj is the identity)
template <typename T>
__global__ void add_rows_kernel(const T* a, const T* vec, T* out, int R) {
  const int b = blockIdx.x;
  for (int k = threadIdx.x; k < R; k += blockDim.x)
    El<T>::st(out + (size_t)b * R + k, El<T>::ld(a + (size_t)b * R + k) + El<T>::ld(vec + k));
}
int launch_add_rows(int dtype, const void* a, const void* vec, void* out, int B, int R, hipStream_t st) {
  if (dtype == VUI_DTYPE_F32)
    hipLaunchKernelGGL(add_rows_kernel<float>, dim3(B), dim3(256), 0, st, (const float*)a, (const float*)vec, (float*)out, R);
  else
    hipLaunchKernelGGL(add_rows_kernel<bf16_t>, dim3(B), dim3(256), 0, st, (const bf16_t*)a, (const bf16_t*)vec, (bf16_t*)out, R);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}

__global__ void frame_finish_kernel(const int64_t* codes, int64_t* frames_out, int n, int max_frames, int32_t* ctr,
                                    const float* eos_in, float* eos_out, int B, int32_t* stop_state, float stop_thr,
                                    int stop_min) {
  const int f = ctr[0];
  if (stop_state && threadIdx.x == 0) {  // end-of-turn test on the device (row 0; the caller passes B == 1)
    const int step = stop_state[1];
    if (step >= stop_min && eos_in[0] > stop_thr) stop_state[0] = 1;
    stop_state[1] = step + 1;
  }
  const bool in_range = f >= 0 && f < max_frames;
  if (frames_out && in_range)
    for (int i = threadIdx.x; i < n; i += blockDim.x) frames_out[(size_t)f * n + i] = codes[i];
  if (eos_out && (in_range || !frames_out))
    for (int b = threadIdx.x; b < B; b += blockDim.x) eos_out[(frames_out ? (size_t)f * B : 0) + b] = eos_in[b];
  __syncthreads();
  if (threadIdx.x == 0) ctr[0] = f + 1;
}
int launch_frame_finish(const int64_t* codes, int64_t* frames_out, int n, int max_frames, int32_t* ctr,
                        const float* eos_in, float* eos_out, int B, int32_t* stop_state, float stop_thr, int stop_min,
                        hipStream_t st) {
  hipLaunchKernelGGL(frame_finish_kernel, dim3(1), dim3(256), 0, st, codes, frames_out, n, max_frames, ctr, eos_in,
                     eos_out, B, stop_state, stop_thr, stop_min);
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}
