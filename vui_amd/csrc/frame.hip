// The whole per-frame step of one stream as ONE persistent kernel (batch 1, bf16).
//
// On this GPU a dependent kernel boundary costs 4-5 us (every boundary writes back and
// invalidates the eight per-XCD L2s) and a frame is a chain of ~400 dependent small GEMVs, so
// the chain is run inside one resident grid instead: one workgroup per CU, every workgroup
// walks the same phase list, owns a fixed slice of each weight matrix and keeps the residual
// stream redundantly in LDS.  Between phases the workgroups exchange the small activation
// vectors through "flag-in-data" words: an 8-byte word = 4 bytes of payload (two bf16 or one
// fp32) + the 4-byte launch epoch, written and polled with device-scope relaxed atomics, which
// bypass the non-coherent L2s.  A consumer that sees the current epoch has the data: no barrier,
// no cache flush.  Weight loads of a phase are issued before its poll, so HBM latency overlaps
// the wait.  Every phase has its own word buffer, so nothing is reused within a launch.
//
// Arithmetic and rounding points are those of the per-kernel path (gemv.hip / attn.hip /
// sample.h), i.e. of the reference: src/vui/model.py:204-258, 282-297, 359-375 (backbone block),
// :908-986 (depth head), src/vui/engine.py:434-449, 571-590, 855-863, 1450-1485 (frame loop).
#include "common.h"
#include "internal.h"
#include "sample.h"
#include <stdio.h>

#include "ll.h"

// ---- per-workgroup slice of a GEMV: adjacent row pairs, dealt round-robin over workgroups ----
struct Plan {
  int np;      // row pairs of this workgroup
  int KS;      // waves sharing one pair along K (1, 2 or 4)
  int kpart;   // this wave's K part
  int nslots;  // pairs this wave works on (<= 2)
  int gp[2];   // their global pair indices
  int c0, c1;  // this wave's 8-element chunk range of K
};

// row pairs of workgroup wg when pairs are dealt round-robin (the one division per phase type)
__device__ __forceinline__ int pairs_of(int npairs, int wg, int nwg) {
  return (npairs > wg) ? (npairs - wg + nwg - 1) / nwg : 0;
}
// the rest of the plan costs a few shifts, so it is rebuilt at each use instead of being kept live
__device__ __forceinline__ Plan plan_of(int np, int K, int wg, int nwg, int wave) {
  Plan p;
  p.np = np;
  p.KS = np >= 3 ? 1 : (np == 2 ? 2 : (np == 1 ? 4 : 1));
  const int nch = K >> 3;
  if (p.KS == 1) {
    p.kpart = 0;
    p.nslots = (wave < np ? 1 : 0) + (wave + 4 < np ? 1 : 0);
    p.gp[0] = wg + wave * nwg;
    p.gp[1] = wg + (wave + 4) * nwg;
    p.c0 = 0; p.c1 = nch;
  } else {
    const int sh = p.KS == 2 ? 1 : 2;
    const int li = wave >> sh;
    p.kpart = wave & (p.KS - 1);
    p.nslots = 1;
    p.gp[0] = wg + li * nwg;
    p.gp[1] = p.gp[0];
    const int per = (nch + p.KS - 1) >> sh;
    p.c0 = p.kpart * per;
    p.c1 = min(nch, p.c0 + per);
  }
  return p;
}
__device__ __forceinline__ Plan make_plan(int npairs, int K, int wg, int nwg, int wave) {
  return plan_of(pairs_of(npairs, wg, nwg), K, wg, nwg, wave);
}

// I8: the matrix is int8 with one bf16 scale per row (weight-only quantisation): a chunk of eight weights is eight
// bytes, widened to packed bf16 pairs in registers at the point of use (exact: every int8 is a bf16), and the row's
// scale multiplies the finished sum.
template <bool I8> struct WVec { typedef uint4 T; };
template <> struct WVec<true> { typedef uint2 T; };
template <int MAXC, bool DUAL, bool I8 = false>
struct WRegs {
  typename WVec<I8>::T a[2][2][MAXC];
  typename WVec<I8>::T b[DUAL ? 2 : 1][DUAL ? 2 : 1][DUAL ? MAXC : 1];
  uint32_t sa[I8 ? 2 : 1], sb[(I8 && DUAL) ? 2 : 1];  // int8: the bf16 scales of a slot's two rows, packed
};

__device__ __forceinline__ void cvt8(const uint4& r, float* o) {
  o[0] = __uint_as_float(r.x << 16); o[1] = __uint_as_float(r.x & 0xffff0000u);
  o[2] = __uint_as_float(r.y << 16); o[3] = __uint_as_float(r.y & 0xffff0000u);
  o[4] = __uint_as_float(r.z << 16); o[5] = __uint_as_float(r.z & 0xffff0000u);
  o[6] = __uint_as_float(r.w << 16); o[7] = __uint_as_float(r.w & 0xffff0000u);
}
// eight int8 -> four packed bf16 pairs (a sign-extending byte conversion per weight, a packing conversion per pair)
__device__ __forceinline__ uint4 widen8(const uint2& w) {
  uint4 r;
  r.x = f2bf2((float)(int8_t)(w.x & 0xff), (float)(int8_t)((w.x >> 8) & 0xff));
  r.y = f2bf2((float)(int8_t)((w.x >> 16) & 0xff), (float)(int8_t)(w.x >> 24));
  r.z = f2bf2((float)(int8_t)(w.y & 0xff), (float)(int8_t)((w.y >> 8) & 0xff));
  r.w = f2bf2((float)(int8_t)((w.y >> 16) & 0xff), (float)(int8_t)(w.y >> 24));
  return r;
}

// W, W2: (N, K) row-major bf16, or int8 with the per-row bf16 scales S, S2
// NT: the matrix is read once per launch (the backbone's matrices, the codec head, the depth head's projection and
// per-codebook heads): its loads carry the non-temporal hint, so that 311 MB of such reads per frame do not push out of
// the caches what is read again and again (the depth head's layer matrices, 16 passes per frame; the keys and values,
// every frame).  Measured: 1.033 -> 0.992 ms per frame (int8 weights 1.023 -> 1.005); the same hint on the key / value
// loads made it slower (0.997 / 1.019): they are what the caches should keep from frame to frame.
typedef unsigned int fr_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int fr_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 ld_nt16(const void* p) {
  const fr_u32x4 v = __builtin_nontemporal_load((const __attribute__((address_space(1))) fr_u32x4*)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 ld_nt8(const void* p) {
  const fr_u32x2 v = __builtin_nontemporal_load((const __attribute__((address_space(1))) fr_u32x2*)p);
  return make_uint2(v.x, v.y);
}
template <int MAXC, bool DUAL, bool I8, bool NT = false>
__device__ __forceinline__ void gemv_prefetch(const void* Wv, const void* W2v, int K, const Plan& p,
                                              WRegs<MAXC, DUAL, I8>& r, const bf16_t* S = nullptr, const bf16_t* S2 = nullptr) {
  const int lane = threadIdx.x & 63;
  if constexpr (!I8) {
    const bf16_t* W = (const bf16_t*)Wv;
    const bf16_t* W2 = (const bf16_t*)W2v;
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int rr = 0; rr < 2; ++rr)
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
          const int c = p.c0 + lane + WAVE * i;
          const bool on = s < p.nslots && c < p.c1;
          const size_t off = ((size_t)(2 * p.gp[s] + rr)) * K + (size_t)c * 8;
          if constexpr (NT) {
            r.a[s][rr][i] = on ? ld_nt16(W + off) : make_uint4(0, 0, 0, 0);
            if (DUAL) r.b[s][rr][i] = on ? ld_nt16(W2 + off) : make_uint4(0, 0, 0, 0);
          } else {
            r.a[s][rr][i] = on ? *reinterpret_cast<const uint4*>(W + off) : make_uint4(0, 0, 0, 0);
            if (DUAL) r.b[s][rr][i] = on ? *reinterpret_cast<const uint4*>(W2 + off) : make_uint4(0, 0, 0, 0);
          }
        }
  } else {
    const int8_t* W = (const int8_t*)Wv;
    const int8_t* W2 = (const int8_t*)W2v;
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int rr = 0; rr < 2; ++rr)
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
          const int c = p.c0 + lane + WAVE * i;
          const bool on = s < p.nslots && c < p.c1;
          const size_t off = ((size_t)(2 * p.gp[s] + rr)) * K + (size_t)c * 8;
          if constexpr (NT) {
            r.a[s][rr][i] = on ? ld_nt8(W + off) : make_uint2(0, 0);
            if (DUAL) r.b[s][rr][i] = on ? ld_nt8(W2 + off) : make_uint2(0, 0);
          } else {
            r.a[s][rr][i] = on ? *reinterpret_cast<const uint2*>(W + off) : make_uint2(0, 0);
            if (DUAL) r.b[s][rr][i] = on ? *reinterpret_cast<const uint2*>(W2 + off) : make_uint2(0, 0);
          }
        }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      r.sa[s] = s < p.nslots ? *reinterpret_cast<const uint32_t*>(S + 2 * p.gp[s]) : 0u;
      if (DUAL) r.sb[s] = s < p.nslots ? *reinterpret_cast<const uint32_t*>(S2 + 2 * p.gp[s]) : 0u;
    }
  }
}

// xp: K staged activations in LDS as packed bf16 pairs (K/2 words; every activation this kernel
// multiplies is a bf16 value, so nothing is lost).  red: 4 x 4 floats of LDS.  epi(gp, v0, v1, u0, u1)
// is called by every lane of the finishing wave (same arguments in all lanes) with the fp32 dot products of
// rows 2gp, 2gp+1 (u*: second matrix), times the rows' scales for int8 weights.
template <int MAXC, bool DUAL, bool I8, typename Epi>
__device__ __forceinline__ void gemv_compute(const uint32_t* xp, const Plan& p, const WRegs<MAXC, DUAL, I8>& r, float* red,
                                             Epi&& epi) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;  // the wave index as a scalar
  float res[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  uint4 x[MAXC];
  if (p.nslots > 0) {
    // lanes beyond the K range hold zero weights; their reads are clamped to a staged chunk
#pragma unroll
    for (int i = 0; i < MAXC; ++i) x[i] = *reinterpret_cast<const uint4*>(xp + 4 * min(p.c0 + lane + WAVE * i, p.c1 - 1));
  }
  float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    if (s < p.nslots) {
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
          if constexpr (I8) {
            acc[s][rr] = dot8_bf(widen8(r.a[s][rr][i]), x[i], acc[s][rr]);
            if (DUAL) acc[s][2 + rr] = dot8_bf(widen8(r.b[s][rr][i]), x[i], acc[s][2 + rr]);
          } else {
            acc[s][rr] = dot8_bf(r.a[s][rr][i], x[i], acc[s][rr]);
            if (DUAL) acc[s][2 + rr] = dot8_bf(r.b[s][rr][i], x[i], acc[s][2 + rr]);
          }
        }
      }
    }
  }
  // several full-wave sums per butterfly; the totals are then spread to every lane of their quad
  if (DUAL) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
      if (s < p.nslots) {
        const float z = wave_sum4(acc[s][0], acc[s][1], acc[s][2], acc[s][3]);
        res[s][0] = dpp_f<0x00>(z); res[s][1] = dpp_f<0x55>(z); res[s][2] = dpp_f<0xAA>(z); res[s][3] = dpp_f<0xFF>(z);
      }
  } else if (p.nslots > 1) {
    const float z = wave_sum4(acc[0][0], acc[0][1], acc[1][0], acc[1][1]);
    res[0][0] = dpp_f<0x00>(z); res[0][1] = dpp_f<0x55>(z); res[1][0] = dpp_f<0xAA>(z); res[1][1] = dpp_f<0xFF>(z);
  } else if (p.nslots > 0) {
    const float z = wave_sum2(acc[0][0], acc[0][1]);
    res[0][0] = dpp_f<0x00>(z); res[0][1] = dpp_f<0x55>(z);
  }
  // int8: y[n] = scale[n] * sum_k q[n, k] x[k], the scale applied once to the finished sum
#define FR_SCALED(s, v0, v1, u0, u1)                                      \
  do {                                                                    \
    if constexpr (I8) {                                                   \
      v0 *= bf_lo(r.sa[s]); v1 *= bf_hi(r.sa[s]);                         \
      if (DUAL) { u0 *= bf_lo(r.sb[s]); u1 *= bf_hi(r.sb[s]); }           \
    }                                                                     \
  } while (0)
  if (p.KS > 1) {  // uniform over the workgroup
    if (lane == 0) { red[wave * 4 + 0] = res[0][0]; red[wave * 4 + 1] = res[0][1]; red[wave * 4 + 2] = res[0][2]; red[wave * 4 + 3] = res[0][3]; }
    __syncthreads();
    if (p.kpart == 0) {
      float t[4] = {0.f, 0.f, 0.f, 0.f};
      for (int k = 0; k < p.KS; ++k)
#pragma unroll
        for (int j = 0; j < 4; ++j) t[j] += red[(wave + k) * 4 + j];
      FR_SCALED(0, t[0], t[1], t[2], t[3]);
      epi(p.gp[0], t[0], t[1], t[2], t[3]);
    }
  } else {
    if (p.nslots > 0) { FR_SCALED(0, res[0][0], res[0][1], res[0][2], res[0][3]); epi(p.gp[0], res[0][0], res[0][1], res[0][2], res[0][3]); }
    if (p.nslots > 1) { FR_SCALED(1, res[1][0], res[1][1], res[1][2], res[1][3]); epi(p.gp[1], res[1][0], res[1][1], res[1][2], res[1][3]); }
  }
#undef FR_SCALED
}

// norm weights of a thread's feature pairs (pairs tid and tid + 256), fetched ahead of the wait
struct NormW { uint32_t w[2]; };
__device__ __forceinline__ NormW load_normw(const bf16_t* nw, int K) {
  NormW r;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int j = (int)threadIdx.x + FR_THREADS * i;
    r.w[i] = 2 * j < K ? reinterpret_cast<const uint32_t*>(nw)[j] : 0u;
  }
  return r;
}
// two-rounding RMSNorm of src[0..K) (LDS, 1024 floats, K <= 1024, K % 4 == 0) into packed bf16 pairs
// dst[0..K/2); every wave derives the same scale.  Straight-line: all LDS reads are issued before any use.
__device__ __forceinline__ void stage_norm(const float* src, const NormW& nw, float eps, int K, uint32_t* dst) {
  const int lane = threadIdx.x & 63;
  float4 q[4];
  float2 own[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) q[i] = *reinterpret_cast<const float4*>(src + 4 * lane + 256 * i);
#pragma unroll
  for (int i = 0; i < 2; ++i) own[i] = *reinterpret_cast<const float2*>(src + 2 * ((int)threadIdx.x + FR_THREADS * i));
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float t = (q[i].x * q[i].x + q[i].y * q[i].y) + (q[i].z * q[i].z + q[i].w * q[i].w);
    ss += (4 * lane + 256 * i < K) ? t : 0.f;
  }
  ss = wave_sum(ss);
  const float r = __builtin_amdgcn_rsqf(ss * (1.0f / (float)K) + eps);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int j = (int)threadIdx.x + FR_THREADS * i;
    const uint32_t v = f2bf2(own[i].x * r, own[i].y * r);
    const uint32_t o = f2bf2(bf_lo(v) * bf_lo(nw.w[i]), bf_hi(v) * bf_hi(nw.w[i]));
    if (2 * j < K) dst[j] = o;
  }
}

// Exchange helpers: wait for a vector of bf16 pairs and put it into LDS.  Both carry the
// workgroup barriers that separate them from earlier readers and later users of dst.
__device__ __forceinline__ void poll_words(uint32_t* dst, const uint64_t* buf, int nwords, Ctl& c) {
  __syncthreads();
  ll_poll_auto(buf, nwords, c, [&](int i, uint32_t v) { dst[i] = v; });
  __syncthreads();
}
__device__ __forceinline__ void poll_set(float* dst, const uint64_t* buf, int nwords, Ctl& c) {
  __syncthreads();
  ll_poll_auto(buf, nwords, c, [&](int i, uint32_t v) {
    *reinterpret_cast<float2*>(dst + 2 * i) = make_float2(bf_lo(v), bf_hi(v)); });
  __syncthreads();
}
// dst = rnd(dst + incoming): the residual add (src/vui/model.py:367, 374)
__device__ __forceinline__ void poll_add(float* dst, const uint64_t* buf, int nwords, Ctl& c) {
  __syncthreads();
  ll_poll_auto(buf, nwords, c, [&](int i, uint32_t v) {
    const float2 o = *reinterpret_cast<const float2*>(dst + 2 * i);
    const uint32_t pk = f2bf2(o.x + bf_lo(v), o.y + bf_hi(v));
    *reinterpret_cast<float2*>(dst + 2 * i) = make_float2(bf_lo(pk), bf_hi(pk)); });
  __syncthreads();
}

// fixed LDS carve-up (bytes)
#define LDS_XRES 0                       // 1024 floats: residual stream
#define LDS_XN (LDS_XRES + 4096)         // 2048 floats: staged GEMV input / attention scratch
#define LDS_LG (LDS_XN + 8192)           // 2048 floats: logits
#define LDS_SC (LDS_LG + 8192)           // 1024 floats: attention scores of one split
#define LDS_QKV (LDS_SC + 4096)          // 3 x 128 floats: q, new k, new v of one head
#define LDS_RED (LDS_QKV + 1536)         // 64 floats
#define LDS_MISC (LDS_RED + 256)         // 64 ints: sampled codes of the frame
#define LDS_SAMP (LDS_MISC + 256)        // SampleShared
#define LDS_PTAB (LDS_SAMP + 1280)       // 64 floats: penalty^count, count = 0..63 (SampleShared with its optional stamps before it)
#define LDS_FIXED (LDS_PTAB + 256)

// optional per-phase timestamps (100 MHz wall clock) of four workgroups, for profiling: kept in LDS
// as 16-bit deltas + 8-bit tags while the frame runs (a global store per stamp would sit in the
// in-order memory queue in front of the weight loads) and written out at the end
#define PROF_EVENTS 1000
#ifdef VUI_SAMPLE_CLOCK
#define PROF_KEEP(id) ((id) == 0 || (id) >= 40)  // room for the sampler's own stamps
#else
#define PROF_KEEP(id) true
#endif
#define PROF_LDS_BYTES (PROF_EVENTS * 3 + 8)
#define TS(id)                                                                      \
  do {                                                                              \
    if (prof_on && tid == 0 && nts < PROF_EVENTS && PROF_KEEP(id)) {                                 \
      const uint64_t now_ = wall_clock64();                                         \
      const uint64_t dl_ = now_ - ts_prev;                                          \
      prof_dt[nts] = (uint16_t)(dl_ > 65535 ? 65535 : dl_);                         \
      prof_id[nts] = (uint8_t)(id);                                                 \
      ts_prev = now_;                                                               \
      ++nts;                                                                        \
    }                                                                               \
  } while (0)

// a thread's E consecutive logits (elements tid*E ...) from the packed staging area
__device__ __forceinline__ void load_logits8(const uint32_t* lgw, int E, int CS, float (&raw)[8]) {
  const int tid = threadIdx.x;
  if (E == 8 && !(CS & 7)) {
    uint4 r = make_uint4(0, 0, 0, 0);
    if (tid * 8 < CS) r = reinterpret_cast<const uint4*>(lgw)[tid];
    raw[0] = bf_lo(r.x); raw[1] = bf_hi(r.x); raw[2] = bf_lo(r.y); raw[3] = bf_hi(r.y);
    raw[4] = bf_lo(r.z); raw[5] = bf_hi(r.z); raw[6] = bf_lo(r.w); raw[7] = bf_hi(r.w);
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = tid * E + e;
      raw[e] = (e < E && j < CS) ? bf2f(reinterpret_cast<const bf16_t*>(lgw)[j]) : 0.f;
    }
  }
}

struct LayerP { const bf16_t *attn_norm, *wqkv, *wo, *mlp_norm, *w1, *w3, *w2; };  // the backbone's matrices: bf16 or int8
// row scales of a backbone layer's int8 matrices: fetched from the weight table one layer ahead (uniform addresses,
// so the scalar unit does it) and kept in registers - the LDS pointer table has no room to spare
struct LayerS { const bf16_t *s_qkv, *s_o, *s_1, *s_3, *s_2; };
__device__ __forceinline__ LayerS load_scales(const vui_weights& W, int l) {
  const vui_layer_weights& g = W.layers[l];
  LayerS r = {(const bf16_t*)g.s_qkv, (const bf16_t*)g.s_o, (const bf16_t*)g.s_1, (const bf16_t*)g.s_3, (const bf16_t*)g.s_2};
  return r;
}

// KG: the depth head's keys live in a per-workgroup global scratch area instead of LDS (see below); a compile-time
// switch, so that the common form pays nothing for it.
// I8: the backbone's five matrices per layer are int8 with per-row scales (the heads and the depth head stay bf16).
template <bool KG, bool I8>
__global__ __launch_bounds__(FR_THREADS, 1) void frame_kernel(const FrameArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  float* xres = (float*)(smem + LDS_XRES);
  float* xn = (float*)(smem + LDS_XN);
  uint32_t* xp = (uint32_t*)(smem + LDS_XN);  // the same bytes as packed bf16 pairs
  float* lg = (float*)(smem + LDS_LG);
  float* sc = (float*)(smem + LDS_SC);
  float* qh = (float*)(smem + LDS_QKV);
  float* red = (float*)(smem + LDS_RED);
  int* codes_l = (int*)(smem + LDS_MISC);
  SampleShared& ssh = *(SampleShared*)(smem + LDS_SAMP);
  float* ptab = (float*)(smem + LDS_PTAB);
  LayerP* lp = (LayerP*)(smem + LDS_FIXED);          // backbone layers, then depth-head layers
  bf16_t* rqkv = (bf16_t*)(smem + a.lds_kv_off);

  // the wave index as a scalar: what depends on it alone (row plans, roles) is then scalar work and scalar branches
  const int wg = blockIdx.x, nwg = gridDim.x, tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  // a streamed turn that has met its end-of-turn test: steps enqueued ahead of the host's knowledge do nothing
  // (the flag was written by an earlier launch or by the host, so every workgroup reads the same value)
  if (a.stop_state && a.stop_state[0] != 0) return;
  Ctl c;
  ctl_begin(c, a.epoch, a.err);
  const uint32_t ep = c.epoch;
  uint64_t* llp = a.ll;
  const vui_weights& W = *a.w;
  const int d = a.d;
  int code0 = 0;
  float eos_logit = 0.f;
  const uint32_t frame0 = a.frame_ctr0 ? (uint32_t)a.frame_ctr0[0] : 0u;
  const uint32_t frame1 = a.frame_ctr1 ? (uint32_t)a.frame_ctr1[0] : 0u;
  int slot = 0, pos = 0;
  int nts = 0;
  // four workgroups record: prof_wg, the next one (next XCD), +8 (same XCD), +131
  const int prof_k = wg == a.prof_wg ? 0 : (wg == a.prof_wg + 1 ? 1 : (wg == a.prof_wg + 8 ? 2 : (wg == a.prof_wg + 131 ? 3 : -1)));
  const bool prof_on = a.prof != nullptr && prof_k >= 0;
  uint16_t* prof_dt = (uint16_t*)(smem + a.lds_prof_off);
  uint8_t* prof_id = (uint8_t*)(smem + a.lds_prof_off + 2 * PROF_EVENTS);
  const uint64_t ts_first = prof_on ? wall_clock64() : 0;
  const uint64_t cyc_first = prof_on ? (uint64_t)clock64() : 0;
  uint64_t ts_prev = ts_first;
  TS(0);

  // weight pointer tables into LDS (one pass, so no phase waits on a pointer load later)
  for (int i = tid; i < a.L + a.rqL; i += FR_THREADS) {
    LayerP t;
    if (i < a.L) {
      const vui_layer_weights& s = W.layers[i];
      t.attn_norm = (const bf16_t*)s.attn_norm; t.wqkv = (const bf16_t*)s.wqkv; t.wo = (const bf16_t*)s.wo;
      t.mlp_norm = (const bf16_t*)s.mlp_norm; t.w1 = (const bf16_t*)s.w1; t.w3 = (const bf16_t*)s.w3; t.w2 = (const bf16_t*)s.w2;
    } else {
      const vui_rq_layer_weights& s = W.rq_layers[i - a.L];
      t.attn_norm = (const bf16_t*)s.attn_norm; t.wqkv = (const bf16_t*)s.wqkv; t.wo = (const bf16_t*)s.wo;
      t.mlp_norm = (const bf16_t*)s.mlp_norm; t.w1 = (const bf16_t*)s.w1; t.w3 = (const bf16_t*)s.w3; t.w2 = (const bf16_t*)s.w2;
    }
    lp[i] = t;
  }
  // repetition penalty factors by count; counts stay below the window, the rest falls back to powf
  if ((a.mode & FR_CB0) && a.rep_counts && a.penalty > 1.0f && tid < 64) ptab[tid] = powf(a.penalty, (float)tid);
  const bf16_t* g_final_norm = (const bf16_t*)W.final_norm;
  const bf16_t* g_codec_head = (const bf16_t*)W.codec_head;
  const bf16_t* g_eos_w = (const bf16_t*)W.eos_w;
  const bf16_t* g_eos_b = (const bf16_t*)W.eos_b;
  const float* g_rope = W.rope_table;
  const float* g_rope_global = W.rope_table_global;
  const bf16_t* g_rq_proj = (const bf16_t*)W.rq_backbone_proj;
  const bf16_t* g_rq_emb = (const bf16_t*)W.rq_code_emb;
  const bf16_t* pos_emb = (const bf16_t*)W.rq_pos_emb;
  const bf16_t* g_rq_head = (const bf16_t*)W.rq_head_w;
  const bf16_t* g_rq_norm = (const bf16_t*)W.rq_norm;
  // the epoch has been read (the fence waits for it) before this workgroup reports its arrival
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  if (tid == 0) __hip_atomic_fetch_add(a.arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  if (a.mode & FR_BACKBONE) {
    slot = a.slot_idx ? a.slot_idx[0] : 0;
    pos = a.seq_lens[slot];
    if (pos < 0) pos = 0;
    if (pos >= a.S) pos = a.S - 1;
    // input embedding, redundantly in every workgroup: the clamped table rows go through LDS once, then
    // each thread sums feature pairs tid and tid + 256 with all row loads of both in flight together
    if (a.codes_in) {
      const uint32_t* table = (const uint32_t*)W.audio_emb;
      int* rows = codes_l;  // free until the depth head
      for (int q = tid; q < a.Q; q += FR_THREADS) {
        int64_t cc = a.codes_in[q];
        cc = cc < 0 ? 0 : (cc >= a.CS ? a.CS - 1 : cc);
        rows[q] = (int)(cc + (int64_t)q * a.CS);
      }
      __syncthreads();
      float s0[2] = {0.f, 0.f}, s1[2] = {0.f, 0.f};
      for (int q0 = 0; q0 < a.Q; q0 += 16) {
        uint32_t r[2][16];
#pragma unroll
        for (int q = 0; q < 16; ++q) {
          const int row = rows[min(q0 + q, a.Q - 1)];
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const int j = tid + FR_THREADS * i;
            r[i][q] = (q0 + q < a.Q && 2 * j < d) ? table[((size_t)row * d) / 2 + j] : 0u;
          }
        }
#pragma unroll
        for (int q = 0; q < 16; ++q)
#pragma unroll
          for (int i = 0; i < 2; ++i) { s0[i] += bf_lo(r[i][q]); s1[i] += bf_hi(r[i][q]); }
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int j = tid + FR_THREADS * i;
        if (2 * j < d) { const uint32_t pk = f2bf2(s0[i], s1[i]); xres[2 * j] = bf_lo(pk); xres[2 * j + 1] = bf_hi(pk); }
      }
    } else {
      for (int k = tid; k < d; k += FR_THREADS) xres[k] = bf2f(a.emb_in[k]);
    }
    __syncthreads();

    const int nq = a.H * a.hd, nkv = a.KV * a.hd, hd = a.hd;
    const int np_qkv = (nq + 2 * nkv) / 2;
    const int n_qkv = pairs_of(np_qkv, wg, nwg), n_o = pairs_of(d / 2, wg, nwg), n_sw = pairs_of(a.F / 2, wg, nwg);
    const Plan P_qkv = plan_of(n_qkv, d, wg, nwg, wave);
    // QKV epilogue constants of this wave's pairs: region, index in region, rotation factors (the layers' common
    // table; a global-attention layer with a table of its own fetches its factors at the top of the layer)
    int q_region[2], q_m[2];
    float4 q_rot[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int n = 2 * P_qkv.gp[s];
      int region, m;
      if (n < nq) { region = 0; m = n; }
      else if (n < nq + nkv) { region = 1; m = n - nq; }
      else { region = 2; m = n - nq - nkv; }
      const int dd = m % hd;
      q_region[s] = region; q_m[s] = m;
      q_rot[s] = make_float4(1.f, 0.f, 1.f, 0.f);
      if (s < P_qkv.nslots && region != 2 && dd < a.rope_dim)
        q_rot[s] = *reinterpret_cast<const float4*>(g_rope + ((size_t)pos * a.rope_dim + dd) * 2);
      else q_region[s] |= 4;  // no rotation
    }
    const uint64_t* ybuf = nullptr;  // previous layer's MLP output, still to be added to xres
    const int len = pos + 1;
    const int NS = a.ns;
    const size_t slab = (size_t)a.n_slots * a.S * nkv;
    const int att_h = wg % a.H, att_s = wg / a.H;
    const int kvh = att_h / (a.H / a.KV);
    const int cpd = (hd + 15) / 16;
    const bool mrg_on = wg < a.H * cpd;

    LayerS Ls = {nullptr, nullptr, nullptr, nullptr, nullptr}, Ls_next = Ls;
    if constexpr (I8) Ls_next = load_scales(W, 0);
    for (int l = 0; l < a.L; ++l) {
      const LayerP Lw = lp[l];
      if constexpr (I8) {
        Ls = Ls_next;
        if (l + 1 < a.L) Ls_next = load_scales(W, l + 1);
      }
      bf16_t* kcl = a.kc + slab * l;
      bf16_t* vcl = a.vc + slab * l;
      // this layer's window and rotation (src/vui/model.py:406-418, 504-509): a global layer sees the whole cache
      const bool glob = (a.global_layers >> l) & 1ull;
      const int win_l = glob ? 0 : a.window;
      int l_region[2] = {q_region[0], q_region[1]};
      float4 l_rot[2] = {q_rot[0], q_rot[1]};
      if (glob && g_rope_global) {  // uniform over the grid
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const int region = q_region[s] & 3, dd = q_m[s] % hd;
          l_region[s] = region | 4;
          l_rot[s] = make_float4(1.f, 0.f, 1.f, 0.f);
          if (s < P_qkv.nslots && region != 2 && dd < a.global_rope_dim) {
            l_rot[s] = *reinterpret_cast<const float4*>(g_rope_global + ((size_t)pos * a.global_rope_dim + dd) * 2);
            l_region[s] = region;
          }
        }
      }
      // attention split geometry of the layer (identical in every workgroup)
      const int start = (win_l > 0) ? max(0, len - 1 - win_l) : 0;
      const int nkeys = len - start;
      int ns_eff = (nkeys + 31) / 32;
      ns_eff = max(1, min(ns_eff, NS));
      int chunk = (nkeys + ns_eff - 1) / ns_eff;
      chunk = (chunk + 15) / 16 * 16;
      const bool att_on = att_s < ns_eff && wg < a.H * NS;
      const int att_lo = start + att_s * chunk, att_hi = min(att_lo + chunk, len);
      // ---- QKV + RoPE + cache append ----
      WRegs<2, false, I8> wr;
      const Plan P_qkv = plan_of(n_qkv, d, wg, nwg, wave);
      gemv_prefetch<2, false, I8, true>(Lw.wqkv, nullptr, d, P_qkv, wr, Ls.s_qkv);
      const NormW nw1 = load_normw(Lw.attn_norm, d);
      TS(1);
      if (ybuf) poll_add(xres, ybuf, d / 2, c);
      TS(2);
      stage_norm(xres, nw1, a.eps, d, xp);
      __syncthreads();
      TS(3);
      uint64_t* qkvbuf = llp;
      llp += np_qkv;
      gemv_compute<2, false, I8>(xp, P_qkv, wr, red, [&](int gp, float v0, float v1, float, float) {
        const bool s0 = (gp == P_qkv.gp[0]);
        float o0 = bf2f(f2bf(v0)), o1 = bf2f(f2bf(v1));
        const int rg = s0 ? l_region[0] : l_region[1];
        const int region = rg & 3, m = s0 ? q_m[0] : q_m[1];
        if (!(rg & 4)) {
          const float4 f = s0 ? l_rot[0] : l_rot[1];
          const float r0 = rope_mix(o0, f.x, -o1, f.y);
          const float r1 = rope_mix(o1, f.z, o0, f.w);
          o0 = r0; o1 = r1;
        }
        const uint32_t pk = pack2(o0, o1);
        if (lane != 0) return;
        ll_st(qkvbuf + gp, pk, ep);
        if (region == 1) *reinterpret_cast<uint32_t*>(kcl + ((size_t)slot * a.S + pos) * nkv + m) = pk;
        if (region == 2) *reinterpret_cast<uint32_t*>(vcl + ((size_t)slot * a.S + pos) * nkv + m) = pk;
      });
      TS(4);

      // ---- attention: workgroup (h, s) handles keys [lo, hi) of head h ----
      uint64_t* part = llp;
      llp += (size_t)a.H * NS * (hd + 2);
      if (att_on) {
        const int h = att_h, lo = att_lo, hi = att_hi;
        const bool has_new = (pos >= lo && pos < hi);
        const int grp = lane >> 4, l16 = lane & 15, g = wave * 4 + grp;
        const bool act = l16 * 8 < hd;
        const size_t rowstride = (size_t)nkv;
        const bf16_t* kbase = kcl + ((size_t)slot * a.S) * rowstride + kvh * hd + l16 * 8;
        const bf16_t* vbase = vcl + ((size_t)slot * a.S) * rowstride + kvh * hd + l16 * 8;
        // the first four keys/values of this lane group are fetched before q is waited for
        uint4 kreg[4], vreg[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = lo + g + 16 * i;
          const bool on = act && j < hi && j != pos;
          kreg[i] = on ? *reinterpret_cast<const uint4*>(kbase + (size_t)j * rowstride) : make_uint4(0, 0, 0, 0);
          vreg[i] = on ? *reinterpret_cast<const uint4*>(vbase + (size_t)j * rowstride) : make_uint4(0, 0, 0, 0);
        }
        const int hw = hd / 2;
        __syncthreads();
        {
          const uint64_t* p0 = (tid < hw) ? qkvbuf + (att_h * hd) / 2 + tid : nullptr;
          const uint64_t* p1 = (has_new && tid < hw) ? qkvbuf + (nq + kvh * hd) / 2 + tid : nullptr;
          const uint64_t* p2 = (has_new && tid < hw) ? qkvbuf + (nq + nkv + kvh * hd) / 2 + tid : nullptr;
          uint32_t r0, r1, r2;
          poll3(p0, p1, p2, c, r0, r1, r2);
          if (tid < hw) {
            qh[2 * tid] = bf2f((bf16_t)(r0 & 0xffff)); qh[2 * tid + 1] = bf2f((bf16_t)(r0 >> 16));
            if (has_new) {
              qh[128 + 2 * tid] = bf2f((bf16_t)(r1 & 0xffff)); qh[128 + 2 * tid + 1] = bf2f((bf16_t)(r1 >> 16));
              qh[256 + 2 * tid] = bf2f((bf16_t)(r2 & 0xffff)); qh[256 + 2 * tid + 1] = bf2f((bf16_t)(r2 >> 16));
            }
          }
        }
        __syncthreads();
        const float scale = 1.0f / sqrtf((float)hd);
        float q8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) q8[e] = act ? qh[l16 * 8 + e] : 0.f;
        float mloc = -INFINITY;
        {
          int i = 0;
          for (int j = lo + g; j < hi; j += 16, ++i) {
            float k8[8];
            float dsum = 0.f;
            if (act) {
              if (j == pos) {
#pragma unroll
                for (int e = 0; e < 8; ++e) k8[e] = qh[128 + l16 * 8 + e];
              } else if (i < 4) {
                cvt8(i == 0 ? kreg[0] : (i == 1 ? kreg[1] : (i == 2 ? kreg[2] : kreg[3])), k8);
              } else {
                El<bf16_t>::ld8(kbase + (size_t)j * rowstride, k8);
              }
#pragma unroll
              for (int e = 0; e < 8; ++e) dsum = fmaf(q8[e], k8[e], dsum);
            }
            dsum = group16_sum(dsum) * scale;
            if (l16 == 0) sc[j - lo] = dsum;
            mloc = fmaxf(mloc, dsum);
          }
        }
        if (l16 == 0) red[g] = mloc;
        __syncthreads();
        float M = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) M = fmaxf(M, red[i]);
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = 0.f;
        float lsum = 0.f;
        {
          int i = 0;
          for (int j = lo + g; j < hi; j += 16, ++i) {
            const float pw = expf(sc[j - lo] - M);
            lsum += pw;
            if (act) {
              float v8[8];
              if (j == pos) {
#pragma unroll
                for (int e = 0; e < 8; ++e) v8[e] = qh[256 + l16 * 8 + e];
              } else if (i < 4) {
                cvt8(i == 0 ? vreg[0] : (i == 1 ? vreg[1] : (i == 2 ? vreg[2] : vreg[3])), v8);
              } else {
                El<bf16_t>::ld8(vbase + (size_t)j * rowstride, v8);
              }
#pragma unroll
              for (int e = 0; e < 8; ++e) acc[e] = fmaf(pw, v8[e], acc[e]);
            }
          }
        }
        __syncthreads();  // maxima in red and QKV's xn fully read before they are reused
        float* accs = xn;  // 16 x 128 floats
        if (act) {
#pragma unroll
          for (int e = 0; e < 8; ++e) accs[g * 128 + l16 * 8 + e] = acc[e];
        }
        if (l16 == 0) red[16 + g] = lsum;
        __syncthreads();
        uint64_t* po = part + ((size_t)h * NS + att_s) * (hd + 2);
        if (tid < hd) {
          float t = 0.f;
#pragma unroll
          for (int gg = 0; gg < 16; ++gg) t += accs[gg * 128 + tid];
          ll_st(po + 2 + tid, __float_as_uint(t), ep);
        }
        if (tid == 0) {
          float t = 0.f;
#pragma unroll
          for (int i = 0; i < 16; ++i) t += red[16 + i];
          ll_st(po, __float_as_uint(M), ep);
          ll_st(po + 1, __float_as_uint(t), ep);
        }
      }
      TS(5);
      // ---- merge the splits: workgroup (h, 16-feature chunk); one wait for everything ----
      const RepBuf attbuf = rep_alloc(llp, d / 2);
      if (mrg_on) {
        const int h = wg / cpd, cc = wg % cpd;
        const uint64_t* pb = part + (size_t)h * NS * (hd + 2);
        float* ml = sc;         // 2 * ns_eff floats
        float* part_lds = lg;   // ns_eff x 16 raw accumulators
        __syncthreads();
        {
          // thread items: it = tid and tid + 256 -> (split, feature); threads < 2*ns_eff also fetch max/sum
          const int it0 = tid, it1 = tid + FR_THREADS;
          const int nitem = ns_eff * 16;
          const int dim0 = cc * 16 + (it0 & 15), dim1 = cc * 16 + (it1 & 15);
          const uint64_t* p0 = (it0 < nitem && dim0 < hd) ? pb + (size_t)(it0 >> 4) * (hd + 2) + 2 + dim0 : nullptr;
          const uint64_t* p1 = (it1 < nitem && dim1 < hd) ? pb + (size_t)(it1 >> 4) * (hd + 2) + 2 + dim1 : nullptr;
          const uint64_t* p2 = (tid < 2 * ns_eff) ? pb + (size_t)(tid >> 1) * (hd + 2) + (tid & 1) : nullptr;
          uint32_t r0, r1, r2;
          poll3(p0, p1, p2, c, r0, r1, r2);
          if (it0 < nitem) part_lds[it0] = p0 ? __uint_as_float(r0) : 0.f;
          if (it1 < nitem) part_lds[it1] = p1 ? __uint_as_float(r1) : 0.f;
          if (tid < 2 * ns_eff) ml[tid] = __uint_as_float(r2);
        }
        __syncthreads();
        if (tid < 16 * LL_REP) {  // eight groups of 16 lanes compute the same 16 features, one copy each
          const int f16 = tid & 15, rep = tid >> 4;
          float Mx = -INFINITY;
          for (int s = 0; s < ns_eff; ++s) Mx = fmaxf(Mx, ml[2 * s]);
          float Lt = 0.f, o = 0.f;
          for (int s = 0; s < ns_eff; ++s) {
            const float w = expf(ml[2 * s] - Mx);
            Lt = fmaf(w, ml[2 * s + 1], Lt);
            o = fmaf(w, part_lds[s * 16 + f16], o);
          }
          const float val = o / Lt;
          const float nb = dpp_f<DPP_QUAD_XOR1>(val);  // neighbour feature
          const int d0 = cc * 16 + f16;
          if (!(f16 & 1) && d0 < hd) ll_st(attbuf.base + (size_t)rep * attbuf.n + (h * hd + d0) / 2, pack2(val, nb), ep);
        }
      }
      TS(6);
      // ---- out_proj ----
      const RepBuf obuf = rep_alloc(llp, d / 2);
      {
        WRegs<2, false, I8> w2;
        const Plan P_o = plan_of(n_o, d, wg, nwg, wave);
        gemv_prefetch<2, false, I8, true>(Lw.wo, nullptr, d, P_o, w2, Ls.s_o);
        poll_words(xp, rep_rd(attbuf), d / 2, c);
        TS(7);
        gemv_compute<2, false, I8>(xp, P_o, w2, red, [&](int gp, float v0, float v1, float, float) {
          rep_st(obuf, gp, pack2(v0, v1), ep); });
      }
      TS(8);
      // ---- SwiGLU ----
      const RepBuf hbuf = rep_alloc(llp, a.F / 2);
      {
        WRegs<2, true, I8> w3;
        const Plan P_sw = plan_of(n_sw, d, wg, nwg, wave);
        gemv_prefetch<2, true, I8, true>(Lw.w1, Lw.w3, d, P_sw, w3, Ls.s_1, Ls.s_3);
        const NormW nw2 = load_normw(Lw.mlp_norm, d);
        poll_add(xres, rep_rd(obuf), d / 2, c);
        TS(9);
        stage_norm(xres, nw2, a.eps, d, xp);
        __syncthreads();
        TS(10);
        gemv_compute<2, true, I8>(xp, P_sw, w3, red, [&](int gp, float v0, float v1, float u0, float u1) {
          const float a0 = bf2f(f2bf(v0)), a1 = bf2f(f2bf(v1)), c0 = bf2f(f2bf(u0)), c1 = bf2f(f2bf(u1));
          const float s0 = bf2f(f2bf(a0 * __builtin_amdgcn_rcpf(1.0f + __expf(-a0)))), s1 = bf2f(f2bf(a1 * __builtin_amdgcn_rcpf(1.0f + __expf(-a1))));
          rep_st(hbuf, gp, pack2(s0 * c0, s1 * c1), ep);
        });
      }
      TS(11);
      // ---- W2 ----
      const RepBuf yb = rep_alloc(llp, d / 2);
      {
        WRegs<4, false, I8> w4;
        const Plan P_w2 = plan_of(n_o, a.F, wg, nwg, wave);
        gemv_prefetch<4, false, I8, true>(Lw.w2, nullptr, a.F, P_w2, w4, Ls.s_2);
        poll_words(xp, rep_rd(hbuf), a.F / 2, c);
        TS(12);
        gemv_compute<4, false, I8>(xp, P_w2, w4, red, [&](int gp, float v0, float v1, float, float) {
          rep_st(yb, gp, pack2(v0, v1), ep); });
      }
      ybuf = rep_rd(yb);
      TS(13);
    }
    // ---- final norm, codec head, eos head ----
    {
      const Plan p = make_plan(a.CS / 2, d, wg, nwg, wave);
      WRegs<2, false> wr;
      gemv_prefetch<2, false, false, true>(g_codec_head, nullptr, d, p, wr);
      const NormW nwf = load_normw(g_final_norm, d);
      uint32_t eosw[8];  // this lane's eos-head weight pairs (pair = lane, lane+64, ...), d <= 1024
#pragma unroll
      for (int i = 0; i < 8; ++i) { const int j = lane + WAVE * i; eosw[i] = 2 * j < d ? reinterpret_cast<const uint32_t*>(g_eos_w)[j] : 0u; }
      const float eosb = bf2f(*g_eos_b);
      poll_add(xres, ybuf, d / 2, c);
      stage_norm(xres, nwf, a.eps, d, xp);
      __syncthreads();
      const RepBuf lgbuf = rep_alloc(llp, a.CS / 2);
      gemv_compute<2, false, false>(xp, p, wr, red, [&](int gp, float v0, float v1, float, float) {
        const uint32_t pk = pack2(v0, v1);
        rep_st(lgbuf, gp, pk, ep);
        if (a.cb0_out && lane == 0) *reinterpret_cast<uint32_t*>(a.cb0_out + 2 * gp) = pk;
      });
      // eos logit: every workgroup (it is a 1 x d dot product), outputs by workgroup 0
      {
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) { const int j = lane + WAVE * i; t = dot2_bf(eosw[i], xp[min(j, d / 2 - 1)], t); }
        t = wave_sum(t);
        eos_logit = bf2f(f2bf(t + eosb));
      }
      if (wg == 0) {
        if (a.hidden_out) for (int j = tid; j < d / 2; j += FR_THREADS) reinterpret_cast<uint32_t*>(a.hidden_out)[j] = xp[j];
        if (a.eos_out && tid == 0) a.eos_out[0] = f2bf(eos_logit);
      }
      if (a.mode & FR_CB0) {
        const int E = (a.CS + FR_THREADS - 1) / FR_THREADS;
        // sampling settings: from the launch arguments, or from the device block a captured step reads anew at each
        // replay (fetched where they are used: kept live from the top of the kernel they cost scalar registers)
        const float temp0 = a.sdev0 ? a.sdev0->temperature : a.temp0;
        const int topk0 = a.sdev0 ? a.sdev0->top_k : a.topk0;
        const uint64_t seed0 = a.sdev0 ? a.sdev0->seed : a.seed0;
        const bool greedy = (topk0 == 1) || !(temp0 > 0.f);
        const float div = greedy ? 1.0f : temp0;
        const float* counts = (a.rep_counts && a.penalty > 1.0f) ? a.rep_counts : nullptr;
        // this thread's repetition counts, fetched ahead of the wait for the logits
        float cn[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (counts) {
          if (E == 8 && !(a.CS & 7)) {
            if (tid * 8 < a.CS) {
              const float4 c0 = *reinterpret_cast<const float4*>(counts + tid * 8), c1 = *reinterpret_cast<const float4*>(counts + tid * 8 + 4);
              cn[0] = c0.x; cn[1] = c0.y; cn[2] = c0.z; cn[3] = c0.w; cn[4] = c1.x; cn[5] = c1.y; cn[6] = c1.z; cn[7] = c1.w;
            }
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) { const int j = tid * E + e; if (e < E && j < a.CS) cn[e] = counts[j]; }
          }
        }
        const uint32_t rnd0 = philox_u32(seed0, frame0, 0u, 0u, 0u);  // ahead of the wait
        poll_words((uint32_t*)lg, rep_rd(lgbuf), a.CS / 2, c);
        float lv[8], raw[8];
        uint32_t key[8];
        load_logits8((const uint32_t*)lg, E, a.CS, raw);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          lv[e] = -INFINITY;
          key[e] = 0u;
          const int j = tid * E + e;
          if (e < E && j < a.CS) {
            float v = raw[e];
            if (counts) {  // src/vui/engine.py:571-576
              const float f = (cn[e] >= 0.f && cn[e] < 64.f) ? ptab[(int)cn[e]] : powf(a.penalty, cn[e]);
              v = (v > 0.f) ? v / f : v * f;
            }
            lv[e] = v / div;
            key[e] = float_key(counts ? lv[e] : raw[e]);
          }
        }
        TS(20);
        code0 = block_sample<8>(lv, key, counts ? 0 : 16, a.CS, E, greedy, topk0, rnd0, 0u, ssh, (int*)sc, a.exact0 != 0);
        TS(21);
      }
    }
  }

  // ------------------------------------------------------------------ depth head
  if (a.mode & FR_RQ) {
    const int R = a.R, CS = a.CS, Q = a.Q;
    const int rhd = R / a.rqH;
    if (!(a.mode & FR_BACKBONE)) {
      for (int j = tid; j < d / 2; j += FR_THREADS) xp[j] = reinterpret_cast<const uint32_t*>(a.rq_hidden)[j];
      __syncthreads();
    }
    if (!(a.mode & FR_CB0)) {
      int64_t cc = a.rq_code0[0];
      code0 = (int)(cc < 0 ? 0 : (cc >= CS ? CS - 1 : cc));
    }
    if (tid == 0) codes_l[0] = code0;
    const int m_qkv = pairs_of(3 * R / 2, wg, nwg), m_o = pairs_of(R / 2, wg, nwg), m_sw = pairs_of(a.rqF / 2, wg, nwg),
              m_hd = pairs_of(CS / 2, wg, nwg);
    const NormW nw_rq = load_normw(g_rq_norm, R);
    // attention lane layout: QP key slots x PP feature parts per wave
    const int QP8 = (Q + 7) & ~7;
    // values of positions not yet written this frame are multiplied by weight zero: they must be finite
    // Keys in global memory (kg): a depth head whose keys AND values do not fit beside the rest in LDS keeps the
    // values there (they are read once per position and feature by every lane) and the keys of earlier positions in
    // a global scratch area of this workgroup alone (written and read by the same CU, so plain stores and loads);
    // the key of the running position stays in a small LDS buffer.
    constexpr bool kg = KG;
    const int lds_cache_elems = kg ? a.rqL * R * QP8 + R : a.rqL * 2 * R * QP8;
    for (int i = tid; i < lds_cache_elems / 8; i += FR_THREADS) reinterpret_cast<uint4*>(rqkv)[i] = make_uint4(0, 0, 0, 0);
    bf16_t* knew = rqkv + (size_t)a.rqL * R * QP8;  // kg only: the running position's key, chunk-major [R/8][8]
    bf16_t* kglob = a.rq_kscratch + (size_t)wg * a.rqL * R * QP8;
    int PP = Q <= 16 ? 4 : (Q <= 32 ? 2 : 1);
    while (PP > 1 && ((rhd % PP) || ((rhd / PP) & 1))) PP >>= 1;
    const int fpp = rhd / PP;  // features per part, even
    // token 0: projected hidden + pos_emb[0]
    if (g_rq_proj) {
      const Plan p = make_plan(R / 2, d, wg, nwg, wave);
      WRegs<2, false> wr;
      gemv_prefetch<2, false, false, true>(g_rq_proj, nullptr, d, p, wr);
      // only pairs this wave really owns are inside pos_emb[0, R)
      const uint32_t pe0 = p.nslots > 0 ? *reinterpret_cast<const uint32_t*>(pos_emb + 2 * p.gp[0]) : 0u;
      const uint32_t pe1 = p.nslots > 1 ? *reinterpret_cast<const uint32_t*>(pos_emb + 2 * p.gp[1]) : 0u;
      const RepBuf tb = rep_alloc(llp, R / 2);
      gemv_compute<2, false, false>(xp, p, wr, red, [&](int gp, float v0, float v1, float, float) {
        const uint32_t pe = (gp == p.gp[0]) ? pe0 : pe1;
        const float o0 = bf2f(f2bf(v0)) + __uint_as_float(pe << 16), o1 = bf2f(f2bf(v1)) + __uint_as_float(pe & 0xffff0000u);
        rep_st(tb, gp, pack2(o0, o1), ep);
      });
      poll_set(xres, rep_rd(tb), R / 2, c);
    } else {
      __syncthreads();
      for (int j = tid; j < R / 2; j += FR_THREADS) {
        const uint32_t h2 = xp[j], p2 = reinterpret_cast<const uint32_t*>(pos_emb)[j];
        const uint32_t pk = f2bf2(bf_lo(h2) + bf_lo(p2), bf_hi(h2) + bf_hi(p2));
        xres[2 * j] = bf_lo(pk); xres[2 * j + 1] = bf_hi(pk);
      }
      __syncthreads();
    }

    int prev_code = code0;
    for (int t = 0; t < a.n_q; ++t) {
      if (t >= 1) {
        const bf16_t* e = g_rq_emb + ((size_t)prev_code + (size_t)(t - 1) * CS) * R;
        __syncthreads();
        for (int k = tid; k < R; k += FR_THREADS) xres[k] = bf2f(f2bf(bf2f(e[k]) + bf2f(pos_emb[(size_t)t * R + k])));
        __syncthreads();
      }
      const uint64_t* ybuf = nullptr;
      for (int l = 0; l < a.rqL; ++l) {
        const LayerP Lw = lp[a.L + l];
        // depth-head cache of this layer in LDS, QP8 = Q rounded up to 8 positions:
        //   keys    [R/8 chunks][QP8 positions][8 features]   (a lane group reads one position per lane: no bank conflicts)
        //   values  [R features][QP8 positions]               (one feature's values over the positions are contiguous)
        bf16_t* kcache = rqkv + (size_t)l * 2 * R * QP8;  // LDS form
        bf16_t* vcache = kg ? rqkv + (size_t)l * R * QP8 : kcache + (size_t)R * QP8;
        bf16_t* kcache_g = kglob + (size_t)l * R * QP8;   // global form, same [R/8][QP8][8] layout
        // ---- A: QKV ----
        const RepBuf qkvb = rep_alloc(llp, 3 * R / 2);
        {
          TS(30);
          WRegs<2, false> wr;
          const Plan R_qkv = plan_of(m_qkv, R, wg, nwg, wave);
          gemv_prefetch<2, false, false>(Lw.wqkv, nullptr, R, R_qkv, wr);
          const NormW nw1 = load_normw(Lw.attn_norm, R);
          if (ybuf) poll_add(xres, ybuf, R / 2, c);
          TS(31);
          stage_norm(xres, nw1, a.rq_eps, R, xp);
          __syncthreads();
          gemv_compute<2, false, false>(xp, R_qkv, wr, red, [&](int gp, float v0, float v1, float, float) {
            rep_st(qkvb, gp, pack2(v0, v1), ep); });
        }
        const bool kv_only = (t == 0 && l == a.rqL - 1);  // position 0 only feeds later keys/values
        // ---- B: attention (redundantly in every workgroup) + out_proj ----
        RepBuf ob = {llp, R / 2};
        if (!kv_only) ob = rep_alloc(llp, R / 2);
        {
          WRegs<2, false> wr;
          const Plan R_o = plan_of(m_o, R, wg, nwg, wave);
          if (!kv_only) gemv_prefetch<2, false, false>(Lw.wo, nullptr, R, R_o, wr);
          __syncthreads();  // xn (A's input) fully consumed before q overwrites it
          ll_poll_auto(rep_rd(qkvb), 3 * R / 2, c, [&](int i, uint32_t v) {
            const int n = 2 * i;
            if (n < R) xp[i] = v;  // q, packed
            else if (n < 2 * R) {   // new key: features n-R, n-R+1 of position t
              const int f = n - R;
              if (kg) {
                *reinterpret_cast<uint32_t*>(knew + f) = v;  // [f >> 3][f & 7] = f
                *reinterpret_cast<uint32_t*>(kcache_g + ((size_t)(f >> 3) * QP8 + t) * 8 + (f & 7)) = v;
              } else {
                *reinterpret_cast<uint32_t*>(kcache + ((size_t)(f >> 3) * QP8 + t) * 8 + (f & 7)) = v;
              }
            } else {                // new value
              const int f = n - 2 * R;
              vcache[(size_t)f * QP8 + t] = (bf16_t)(v & 0xffff);
              vcache[(size_t)(f + 1) * QP8 + t] = (bf16_t)(v >> 16);
            }
          });
          __syncthreads();
          if (kv_only) break;
          TS(32);
          const int nk = t + 1;
          const int kj = lane / PP, part = lane % PP;
          const float scale = 1.0f / sqrtf((float)rhd);
          // this wave's softmax weights of two heads as bf16 hi + lo parts: [head][hi 64 | lo 64]
          bf16_t* pw_hi = reinterpret_cast<bf16_t*>(sc) + wave * 256;
          bf16_t* pw_lo = pw_hi + 64;
          // two heads per pass, written side by side so that their LDS round trips and reductions overlap
          for (int hb0 = wave; hb0 < a.rqH; hb0 += 8) {
            int hs[2];
            hs[0] = hb0;
            hs[1] = min(hb0 + 4, a.rqH - 1);  // a missing second head repeats a valid one and is not written
            const bool second = hb0 + 4 < a.rqH;
            const int kk = min(kj, nk - 1);
            float dsum[2] = {0.f, 0.f};
            if (!(fpp & 7)) {
              for (int i = 0; i < fpp / 8; ++i) {
                uint4 kr[2], qr[2];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                  const int f0 = hs[h] * rhd + part * fpp + 8 * i;
                  if (!kg) kr[h] = *reinterpret_cast<const uint4*>(kcache + ((size_t)(f0 >> 3) * QP8 + kk) * 8);
                  else if (kk == t) kr[h] = *reinterpret_cast<const uint4*>(knew + f0);
                  else kr[h] = *reinterpret_cast<const uint4*>(kcache_g + ((size_t)(f0 >> 3) * QP8 + kk) * 8);
                  qr[h] = *reinterpret_cast<const uint4*>(xp + f0 / 2);
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) dsum[h] = dot8_bf(kr[h], qr[h], dsum[h]);
              }
            } else {
              for (int i = 0; i < fpp / 2; ++i)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                  const int f = hs[h] * rhd + part * fpp + 2 * i;
                  const uint32_t kw = !kg ? *reinterpret_cast<const uint32_t*>(kcache + ((size_t)(f >> 3) * QP8 + kk) * 8 + (f & 7))
                                      : (kk == t ? *reinterpret_cast<const uint32_t*>(knew + f)
                                                 : *reinterpret_cast<const uint32_t*>(kcache_g + ((size_t)(f >> 3) * QP8 + kk) * 8 + (f & 7)));
                  dsum[h] = dot2_bf(kw, xp[f / 2], dsum[h]);
                }
            }
            float pw[2], Ls[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              if (PP >= 2) dsum[h] += dpp_f<DPP_QUAD_XOR1>(dsum[h]);
              if (PP >= 4) dsum[h] += dpp_f<DPP_QUAD_XOR2>(dsum[h]);
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              const float sco = (kj < nk) ? dsum[h] * scale : -INFINITY;
              const float M = rows_max(group16_max(sco));
              pw[h] = (kj < nk) ? __expf(sco - M) : 0.f;
              Ls[h] = wave_sum_v(part == 0 ? pw[h] : 0.f);
            }
            // the weights go through LDS as bf16 pairs: p = hi + lo keeps 16 mantissa bits
            if (part == 0) {
#pragma unroll
              for (int h = 0; h < 2; ++h) {
                const bf16_t hi = f2bf(pw[h]);
                pw_hi[h * 128 + kj] = hi;
                pw_lo[h * 128 + kj] = f2bf(pw[h] - bf2f(hi));
              }
            }
            // lane = feature: dot product of the feature's values over the positions with the weights
            float o0[2] = {0.f, 0.f}, o1[2] = {0.f, 0.f};
            for (int j0 = 0; j0 < nk; j0 += 8) {
              uint4 ph[2], pl[2], va[2], vb[2];
#pragma unroll
              for (int h = 0; h < 2; ++h) {
                ph[h] = *reinterpret_cast<const uint4*>(pw_hi + h * 128 + j0);
                pl[h] = *reinterpret_cast<const uint4*>(pw_lo + h * 128 + j0);
                va[h] = *reinterpret_cast<const uint4*>(vcache + (size_t)(hs[h] * rhd + min(lane, rhd - 1)) * QP8 + j0);
                if (rhd > WAVE) vb[h] = *reinterpret_cast<const uint4*>(vcache + (size_t)(hs[h] * rhd + min(lane + WAVE, rhd - 1)) * QP8 + j0);
              }
#pragma unroll
              for (int h = 0; h < 2; ++h) {
                o0[h] = dot8_bf(va[h], ph[h], o0[h]);
                o0[h] = dot8_bf(va[h], pl[h], o0[h]);
                if (rhd > WAVE) { o1[h] = dot8_bf(vb[h], ph[h], o1[h]); o1[h] = dot8_bf(vb[h], pl[h], o1[h]); }
              }
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              const float inv = __builtin_amdgcn_rcpf(Ls[h]);
              const float a0 = o0[h] * inv, a1 = o1[h] * inv;
              const float n0 = dpp_f<DPP_QUAD_XOR1>(a0), n1 = dpp_f<DPP_QUAD_XOR1>(a1);  // neighbour features
              if (!(lane & 1) && (h == 0 || second)) {
                if (lane < rhd) xp[(R + hs[h] * rhd + lane) / 2] = f2bf2(a0, n0);
                if (lane + WAVE < rhd) xp[(R + hs[h] * rhd + lane + WAVE) / 2] = f2bf2(a1, n1);
              }
            }
          }
          __syncthreads();
          TS(33);
          gemv_compute<2, false, false>(xp + R / 2, R_o, wr, red, [&](int gp, float v0, float v1, float, float) {
            rep_st(ob, gp, pack2(v0, v1), ep); });
        }
        TS(34);
        // ---- C: SwiGLU ----
        const RepBuf hb = rep_alloc(llp, a.rqF / 2);
        {
          WRegs<2, true> wr;
          const Plan R_sw = plan_of(m_sw, R, wg, nwg, wave);
          gemv_prefetch<2, true, false>(Lw.w1, Lw.w3, R, R_sw, wr);
          const NormW nw2 = load_normw(Lw.mlp_norm, R);
          poll_add(xres, rep_rd(ob), R / 2, c);
          TS(35);
          stage_norm(xres, nw2, a.rq_eps, R, xp);
          __syncthreads();
          gemv_compute<2, true, false>(xp, R_sw, wr, red, [&](int gp, float v0, float v1, float u0, float u1) {
            const float a0 = bf2f(f2bf(v0)), a1 = bf2f(f2bf(v1)), c0 = bf2f(f2bf(u0)), c1 = bf2f(f2bf(u1));
            const float s0 = bf2f(f2bf(a0 * __builtin_amdgcn_rcpf(1.0f + __expf(-a0)))), s1 = bf2f(f2bf(a1 * __builtin_amdgcn_rcpf(1.0f + __expf(-a1))));
            rep_st(hb, gp, pack2(s0 * c0, s1 * c1), ep);
          });
        }
        TS(36);
        // ---- D: W2 ----
        const RepBuf yb = rep_alloc(llp, R / 2);
        {
          WRegs<4, false> wr;
          const Plan R_w2 = plan_of(m_o, a.rqF, wg, nwg, wave);
          gemv_prefetch<4, false, false>(Lw.w2, nullptr, a.rqF, R_w2, wr);
          poll_words(xp, rep_rd(hb), a.rqF / 2, c);
          TS(37);
          gemv_compute<4, false, false>(xp, R_w2, wr, red, [&](int gp, float v0, float v1, float, float) {
            rep_st(yb, gp, pack2(v0, v1), ep); });
        }
        ybuf = rep_rd(yb);
      }
      if (t >= 1) {
        // ---- head t-1: logits of codebook t, then the draw in every workgroup ----
        WRegs<2, false> wr;
        const Plan R_hd = plan_of(m_hd, R, wg, nwg, wave);
        gemv_prefetch<2, false, false, true>(g_rq_head + (size_t)(t - 1) * CS * R, nullptr, R, R_hd, wr);
        TS(40);
        poll_add(xres, ybuf, R / 2, c);
        TS(41);
        stage_norm(xres, nw_rq, a.rq_eps, R, xp);
        __syncthreads();
        const RepBuf lgbuf = rep_alloc(llp, CS / 2);
        gemv_compute<2, false, false>(xp, R_hd, wr, red, [&](int gp, float v0, float v1, float, float) {
          rep_st(lgbuf, gp, pack2(v0, v1), ep); });
        TS(42);
        const float temp1 = a.sdev1 ? a.sdev1->temperature : a.temp1;
        const int topk1 = a.sdev1 ? a.sdev1->top_k : a.topk1;
        const uint64_t seed1 = a.sdev1 ? a.sdev1->seed : a.seed1;
        const uint32_t rnd = philox_u32(seed1, frame1, 0u, (uint32_t)t, 0u);  // ahead of the wait
        poll_words((uint32_t*)lg, rep_rd(lgbuf), CS / 2, c);
        TS(43);
        const int E = (CS + FR_THREADS - 1) / FR_THREADS;
        const bool greedy = (topk1 == 1) || !(temp1 > 0.f);
        const float div = greedy ? 1.0f : temp1;
        const float* bias = a.logit_bias ? a.logit_bias + (size_t)(t - 1) * CS : nullptr;
        float lv[8], raw[8];
        uint32_t key[8];
        load_logits8((const uint32_t*)lg, E, CS, raw);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          lv[e] = -INFINITY;
          key[e] = 0u;
          const int j = tid * E + e;
          if (e < E && j < CS) {
            lv[e] = sample_value(raw[e], bias, j, nullptr, 1.0f, div);
            key[e] = float_key(bias ? lv[e] : raw[e]);
          }
        }
        prev_code = block_sample<8>(lv, key, bias ? 0 : 16, CS, E, greedy, topk1, rnd, (uint32_t)t, ssh, (int*)sc);
        TS(44);
#ifdef VUI_SAMPLE_CLOCK
        if (prof_on && tid == 0) {
          nts -= 1;  // replace stamp 44 by the sampler's own
          ts_prev -= prof_dt[nts];
          for (int k = 0; k < 8; ++k)
            if (nts < PROF_EVENTS) { prof_dt[nts] = (uint16_t)(ssh.ts[k] - ts_prev); prof_id[nts] = (uint8_t)(60 + k); ts_prev = ssh.ts[k]; ++nts; }
        }
#endif
        if (tid == 0) codes_l[t] = prev_code;
      }
    }
  }

  // ------------------------------------------------------------------ bookkeeping by workgroup 0
  __syncthreads();
  TS(50);
  if (prof_on && tid == 0) {
    uint64_t t = ts_first;
    const int n = min(nts, a.prof_cap);
    uint64_t* out = a.prof + (size_t)prof_k * (a.prof_cap + 1);
    for (int i = 0; i < n; ++i) { t += prof_dt[i]; out[i] = (t << 8) | (uint64_t)prof_id[i]; }
    out[a.prof_cap] = (uint64_t)n | (((uint64_t)clock64() - cyc_first) << 32);  // count | shader cycles of the launch
  }
  if (wg == 0) {
    // Nothing is committed (positions, repetition state, codes, frame log) by a launch in which this workgroup gave
    // up a wait, or on a context whose error word is already raised: the caller sees the failure through
    // vui_ctx_status instead of consuming unwritten words as if they were results.
    // (the flag goes through a word of the dynamic LDS: a block-wide vote would add static LDS to a kernel whose
    // dynamic part already fills the CU's)
    int* bad = (int*)(red + 48);
    if (tid == 0) *bad = ctl_failed(c) ? 1 : 0;
    __syncthreads();
    if (c.dead) *bad = 1;
    __syncthreads();
    if (!*bad) {
    if ((a.mode & FR_CB0) && tid == 0) {
      if (a.code0_out) a.code0_out[0] = code0;
      if (a.rep_counts && a.penalty > 1.0f) rep_push(a.rep_counts, a.rep_hist, a.rep_pos, a.rep_window, code0);
    }
    if (a.mode & FR_RQ) {
      for (int t = tid; t < a.codes_stride; t += FR_THREADS) {
        if (t < a.n_q) a.codes_out[t] = codes_l[t];
        else if (a.zero_pad) a.codes_out[t] = 0;
      }
    }
    if (a.mode & FR_BACKBONE) {
      if (a.seq_inc) { for (int s = tid; s < a.n_slots; s += FR_THREADS) a.seq_lens[s] += a.seq_inc[s]; }
      else if (tid == 0) a.seq_lens[slot] += 1;
    }
    if (a.mode & FR_FINISH) {
      const int f = a.frame_ctr[0];
      const bool in_range = f >= 0 && f < a.max_frames;
      if (a.frames_out && in_range)
        for (int t = tid; t < a.Q; t += FR_THREADS) a.frames_out[(size_t)f * a.Q + t] = (t < a.n_q) ? codes_l[t] : 0;
      const float p_eos = 1.0f / (1.0f + expf(-eos_logit));
      if (a.eos_prob_out && tid == 0 && (in_range || !a.frames_out)) a.eos_prob_out[a.frames_out ? f : 0] = p_eos;
      __syncthreads();
      if (tid == 0) {
        a.frame_ctr[0] = f + 1;
        if (a.stop_state) {  // src/vui/engine.py:1468-1471, decided here instead of on the host
          const int step = a.stop_state[1];
          if (step >= a.stop_min && p_eos > a.stop_thr) a.stop_state[0] = 1;
          a.stop_state[1] = step + 1;
        }
      }
    }
    } else if ((a.mode & FR_FINISH) && tid == 0) {
      // a failed step marks its EOS probability with -1 and the end-of-turn flag with 2, so a caller that reads
      // one of them every frame learns of the failure from the same read (and steps enqueued behind it do nothing)
      const int f = a.frame_ctr[0];
      if (a.eos_prob_out) {
        if (!a.frames_out) a.eos_prob_out[0] = -1.0f;
        else if (f >= 0 && f < a.max_frames) a.eos_prob_out[f] = -1.0f;
      }
      if (a.stop_state) a.stop_state[0] = 2;
    }
    if (tid == 0) ctl_finish(c, a.epoch, a.arrive, (uint32_t)nwg);
  }
}

// ---------------------------------------------------------------------------------------------
// host side
size_t frame_ll_words(const vui_config& c, int ns) {
  const size_t d = c.d_model, hd = c.head_dim, rep = LL_REP;
  // per backbone layer: q/k/v and the attention partials once; attention output, out_proj, SwiGLU and W2 outputs in copies
  size_t per_layer = (size_t)(c.n_heads + 2 * c.n_kv_heads) * hd / 2 + (size_t)c.n_heads * ns * (hd + 2) +
                     rep * (d / 2 + d / 2 + c.ffn / 2 + d / 2);
  size_t total = per_layer * c.n_layers + rep * (c.codebook_size / 2);
  const size_t R = c.rq_dim;
  size_t rq_layer = 3 * R / 2 + R / 2 + c.rq_ffn / 2 + R / 2;
  total += rep * (R / 2 + (size_t)c.n_quantizers * (rq_layer * c.rq_layers + c.codebook_size / 2));
  return total + 64;
}

size_t frame_prof_lds_bytes();
static size_t frame_ptr_bytes(const vui_config& c) {
  return (((size_t)(c.n_layers + c.rq_layers) * sizeof(LayerP)) + 15) & ~(size_t)15;
}
// depth-head keys and values of every layer, positions rounded up to 8
size_t frame_rq_cache_bytes(const vui_config& c) {
  return (size_t)c.rq_layers * ((c.n_quantizers + 7) & ~7) * 2 * c.rq_dim * 2;
}
// 1 when the keys of the depth head live in a per-workgroup global scratch area (its keys and values together do not
// fit in LDS beside the rest, the values and one position's key do)
int frame_rq_keys_global(const vui_config& c) {
  return (size_t)LDS_FIXED + frame_ptr_bytes(c) + frame_rq_cache_bytes(c) + frame_prof_lds_bytes() > 160 * 1024 ? 1 : 0;
}
// the part of the depth-head cache kept in LDS
size_t frame_rq_lds_cache_bytes(const vui_config& c) {
  if (!frame_rq_keys_global(c)) return frame_rq_cache_bytes(c);
  return (frame_rq_cache_bytes(c) / 2 + (size_t)c.rq_dim * 2 + 15) & ~(size_t)15;
}
size_t frame_rq_key_scratch_bytes(const vui_config& c, int nwg) {
  if (c.dtype != VUI_DTYPE_BF16 || c.rq_layers < 1 || !frame_rq_keys_global(c)) return 0;
  return (size_t)nwg * frame_rq_cache_bytes(c) / 2;
}
size_t frame_lds_bytes(const vui_config& c) {
  return (size_t)LDS_FIXED + frame_ptr_bytes(c) + frame_rq_lds_cache_bytes(c);
}
// launches that stop after the backbone step need no room for the depth head's keys and values
size_t frame_lds_bytes_backbone(const vui_config& c) { return (size_t)LDS_FIXED + frame_ptr_bytes(c); }

// with_rq false: only what a backbone-step launch (mode FR_BACKBONE alone) needs
bool frame_supported(const vui_config& c, int nwg, int ns, bool with_rq, char* why, size_t why_len) {
  const char* r = nullptr;
  if (c.dtype != VUI_DTYPE_BF16) r = "bf16 only";
  else if (c.d_model > 1024 || c.ffn > 2048 || c.rq_dim > 1024 || c.rq_ffn > 2048) r = "vector longer than the LDS staging area";
  else if (c.codebook_size > 2048 || (c.codebook_size & 1)) r = "codebook_size > 2048";
  else if (c.n_quantizers > 64) r = "too many codebooks";
  else if ((c.head_dim & 7) || c.head_dim > 128) r = "head_dim";
  else if (c.rq_layers < 1 || c.rq_heads < 1) r = "no depth head";
  else if ((c.rq_dim / c.rq_heads) % 2 || c.rq_dim / c.rq_heads > 128) r = "depth-head head_dim must be even, at most 128";
  else if ((c.d_model | c.ffn | c.rq_dim | c.rq_ffn) & 7) r = "vector lengths must be multiples of 8";
  else if (with_rq && frame_lds_bytes(c) > 160 * 1024) r = "depth-head values do not fit in LDS";
  else {
    const int np_max = (c.n_heads + 2 * c.n_kv_heads) * c.head_dim / 2;
    int m = np_max;
    if (c.ffn / 2 > m) m = c.ffn / 2;
    if (c.codebook_size / 2 > m) m = c.codebook_size / 2;
    if (3 * c.rq_dim / 2 > m) m = 3 * c.rq_dim / 2;
    if (c.rq_ffn / 2 > m) m = c.rq_ffn / 2;
    if (m > 8 * nwg) r = "too few workgroups for the widest matrix";
    if ((c.max_seqlen + ns - 1) / ns + 16 > 1024) r = "key split longer than the LDS score buffer";
    if (nwg < c.n_heads * ns || nwg < c.n_heads * ((c.head_dim + 15) / 16)) r = "too few workgroups for the attention split";
  }
  if (r && why) snprintf(why, why_len, "%s", r);
  return r == nullptr;
}

size_t frame_prof_lds_bytes() { return (PROF_LDS_BYTES + 15) & ~(size_t)15; }

int frame_max_resident(size_t lds_bytes, int* n_cu) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, dev));
  // the attribute is per kernel, not per context: never lower it for another, larger context
  static size_t lds_attr = 0;
  if (lds_bytes > lds_attr) {
    // room for the optional phase-clock buffer where it fits
    const size_t want = lds_bytes + frame_prof_lds_bytes() <= 160 * 1024 ? lds_bytes + frame_prof_lds_bytes() : lds_bytes;
    HIP_TRY(hipFuncSetAttribute((const void*)frame_kernel<false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)want));
    HIP_TRY(hipFuncSetAttribute((const void*)frame_kernel<true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)want));
    HIP_TRY(hipFuncSetAttribute((const void*)frame_kernel<false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)want));
    HIP_TRY(hipFuncSetAttribute((const void*)frame_kernel<true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)want));
    lds_attr = lds_bytes;
  }
  int occ = 0, occ8 = 0;
  HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, frame_kernel<true, false>, FR_THREADS, lds_bytes));
  HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ8, frame_kernel<true, true>, FR_THREADS, lds_bytes));
  if (occ8 < occ) occ = occ8;
  if (n_cu) *n_cu = prop.multiProcessorCount;
  return occ * prop.multiProcessorCount;
}

int launch_frame(const FrameArgs& a_in, int nwg, size_t lds_bytes, hipStream_t st) {
  FrameArgs a = a_in;
  a.lds_prof_off = (int)lds_bytes;
  if (a.prof) {
    if (lds_bytes + frame_prof_lds_bytes() > 160 * 1024) { vui_set_error("no LDS left for the phase clock"); return VUI_EINVAL; }
    lds_bytes += frame_prof_lds_bytes();
  }
  if (a.w_int8) {
    if (a.rq_kg) hipLaunchKernelGGL((frame_kernel<true, true>), dim3(nwg), dim3(FR_THREADS), lds_bytes, st, a);
    else hipLaunchKernelGGL((frame_kernel<false, true>), dim3(nwg), dim3(FR_THREADS), lds_bytes, st, a);
  } else {
    if (a.rq_kg) hipLaunchKernelGGL((frame_kernel<true, false>), dim3(nwg), dim3(FR_THREADS), lds_bytes, st, a);
    else hipLaunchKernelGGL((frame_kernel<false, false>), dim3(nwg), dim3(FR_THREADS), lds_bytes, st, a);
  }
  HIP_TRY(hipGetLastError());
  return VUI_OK;
}
