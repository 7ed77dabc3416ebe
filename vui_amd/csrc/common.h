// Device helpers shared by the gfx950 kernels: element types, 16-byte loads, wave64 reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define WAVE 64

typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf2f(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// round-to-nearest-even, NaN kept quiet (same result as torch's float -> bfloat16): gfx950 converts in
// hardware (v_cvt_pk_bf16_f32), bit-identical to the integer formula on every fp32 input
__device__ __forceinline__ bf16_t f2bf(float f) { return __builtin_bit_cast(bf16_t, (__bf16)f); }
// two values -> one packed word (low half = a)
__device__ __forceinline__ uint32_t f2bf2(float a, float b) {
  typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
  typedef float f2_t __attribute__((ext_vector_type(2)));
  const f2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2_t));
}

// acc + w.lo*x.lo + w.hi*x.hi on packed bf16 pairs, fp32 accumulate (v_dot2c_f32_bf16)
__device__ __forceinline__ float dot2_bf(uint32_t w, uint32_t x, float acc) {
  typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2_t, w), __builtin_bit_cast(bf2_t, x), acc, false);
}
__device__ __forceinline__ float dot8_bf(const uint4& w, const uint4& x, float acc) {
  acc = dot2_bf(w.x, x.x, acc);
  acc = dot2_bf(w.y, x.y, acc);
  acc = dot2_bf(w.z, x.z, acc);
  return dot2_bf(w.w, x.w, acc);
}
__device__ __forceinline__ float bf_lo(uint32_t v) { return __uint_as_float(v << 16); }
__device__ __forceinline__ float bf_hi(uint32_t v) { return __uint_as_float(v & 0xffff0000u); }

template <typename T> struct El;
template <> struct El<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return bf2f(*p); }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = f2bf(v); }
  static __device__ __forceinline__ float rnd(float v) { return bf2f(f2bf(v)); }
  // 8 consecutive elements (16 bytes) -> fp32
  static __device__ __forceinline__ void ld8(const bf16_t* p, float* o) {
    uint4 r = *reinterpret_cast<const uint4*>(p);
    o[0] = __uint_as_float(r.x << 16); o[1] = __uint_as_float(r.x & 0xffff0000u);
    o[2] = __uint_as_float(r.y << 16); o[3] = __uint_as_float(r.y & 0xffff0000u);
    o[4] = __uint_as_float(r.z << 16); o[5] = __uint_as_float(r.z & 0xffff0000u);
    o[6] = __uint_as_float(r.w << 16); o[7] = __uint_as_float(r.w & 0xffff0000u);
  }
  static __device__ __forceinline__ void st8(bf16_t* p, const float* v) {
    uint4 r;
    r.x = f2bf2(v[0], v[1]);
    r.y = f2bf2(v[2], v[3]);
    r.z = f2bf2(v[4], v[5]);
    r.w = f2bf2(v[6], v[7]);
    *reinterpret_cast<uint4*>(p) = r;
  }
};
template <> struct El<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float rnd(float v) { return v; }
  static __device__ __forceinline__ void ld8(const float* p, float* o) {
    float4 a = *reinterpret_cast<const float4*>(p);
    float4 b = *reinterpret_cast<const float4*>(p + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
  static __device__ __forceinline__ void st8(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
};

// 8 consecutive int8 weights (8 bytes) -> fp32
__device__ __forceinline__ void ld8_i8(const int8_t* p, float* o) {
  uint2 r = *reinterpret_cast<const uint2*>(p);
  o[0] = (float)(int8_t)(r.x & 0xff); o[1] = (float)(int8_t)((r.x >> 8) & 0xff);
  o[2] = (float)(int8_t)((r.x >> 16) & 0xff); o[3] = (float)(int8_t)(r.x >> 24);
  o[4] = (float)(int8_t)(r.y & 0xff); o[5] = (float)(int8_t)((r.y >> 8) & 0xff);
  o[6] = (float)(int8_t)((r.y >> 16) & 0xff); o[7] = (float)(int8_t)(r.y >> 24);
}

// ---- wave64 reductions on the DPP data path (no LDS crossbar traffic) ----
// Within a row of 16 lanes: quad xor-1, quad xor-2, half-row mirror, row mirror leave the row
// total in every lane of the row; the four row totals are then read as scalars and added.
#define DPP_QUAD_XOR1 0xB1   // quad_perm [1,0,3,2]
#define DPP_QUAD_XOR2 0x4E   // quad_perm [2,3,0,1]
#define DPP_ROW_HALF_MIRROR 0x141
#define DPP_ROW_MIRROR 0x140

template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL> __device__ __forceinline__ int dpp_i(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
__device__ __forceinline__ float lane_f(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }

// sum within aligned groups of 16 lanes (every lane of the group gets it)
__device__ __forceinline__ float group16_sum(float v) {
  v += dpp_f<DPP_QUAD_XOR1>(v);
  v += dpp_f<DPP_QUAD_XOR2>(v);
  v += dpp_f<DPP_ROW_HALF_MIRROR>(v);
  v += dpp_f<DPP_ROW_MIRROR>(v);
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  v = group16_sum(v);
  return (lane_f(v, 0) + lane_f(v, 16)) + (lane_f(v, 32) + lane_f(v, 48));
}
// ---- reductions that stay in vector registers (gfx950 lane-swap instructions) ----
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its
// second, v_permlane32_swap the upper half of the first with the lower half of the second; applied to
// two copies of one value and added, they fold rows 0+1 / 2+3 and then the two halves.
__device__ __forceinline__ float rows_sum(float v) {  // in: per-row values; out: sum of the four rows, every lane
  const uint32_t u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float s = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const uint32_t w = __float_as_uint(s);
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}
__device__ __forceinline__ float rows_max(float v) {
  const uint32_t u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float s = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const uint32_t w = __float_as_uint(s);
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
// full-wave sum left in every lane, no scalar round trip
__device__ __forceinline__ float wave_sum_v(float v) { return rows_sum(group16_sum(v)); }
#define DPP_ROW_ROR4 0x124
#define DPP_ROW_ROR8 0x128
// Sums of four values at once: lane l returns the full-wave sum of value (l & 3).  Each step halves
// the number of live values by pairing a select with a quad exchange.
__device__ __forceinline__ float wave_sum4(float a, float b, float c, float d) {
  const int lane = threadIdx.x & 63;
  const bool o1 = lane & 1, o2 = lane & 2;
  const float u = (o1 ? b : a) + dpp_f<DPP_QUAD_XOR1>(o1 ? a : b);  // lanes (l&1): partial of a / b over the lane pair
  const float w = (o1 ? d : c) + dpp_f<DPP_QUAD_XOR1>(o1 ? c : d);
  float z = (o2 ? w : u) + dpp_f<DPP_QUAD_XOR2>(o2 ? u : w);        // lane (l&3): partial of value l&3 over the quad
  z += dpp_f<DPP_ROW_ROR4>(z);
  z += dpp_f<DPP_ROW_ROR8>(z);
  return rows_sum(z);
}
// two values: lane l returns the full-wave sum of value (l & 1)
__device__ __forceinline__ float wave_sum2(float a, float b) {
  const int lane = threadIdx.x & 63;
  const bool o1 = lane & 1;
  float z = (o1 ? b : a) + dpp_f<DPP_QUAD_XOR1>(o1 ? a : b);
  z += dpp_f<DPP_QUAD_XOR2>(z);
  z += dpp_f<DPP_ROW_ROR4>(z);
  z += dpp_f<DPP_ROW_ROR8>(z);
  return rows_sum(z);
}

__device__ __forceinline__ float group16_max(float v) {
  v = fmaxf(v, dpp_f<DPP_QUAD_XOR1>(v));
  v = fmaxf(v, dpp_f<DPP_QUAD_XOR2>(v));
  v = fmaxf(v, dpp_f<DPP_ROW_HALF_MIRROR>(v));
  v = fmaxf(v, dpp_f<DPP_ROW_MIRROR>(v));
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  v = group16_max(v);
  return fmaxf(fmaxf(lane_f(v, 0), lane_f(v, 16)), fmaxf(lane_f(v, 32), lane_f(v, 48)));
}
__device__ __forceinline__ int wave_sum_i(int v) {
  v += dpp_i<DPP_QUAD_XOR1>(v);
  v += dpp_i<DPP_QUAD_XOR2>(v);
  v += dpp_i<DPP_ROW_HALF_MIRROR>(v);
  v += dpp_i<DPP_ROW_MIRROR>(v);
  return (__builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16)) +
         (__builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48));
}
__device__ __forceinline__ int wave_min_i(int v) {
  v = min(v, dpp_i<DPP_QUAD_XOR1>(v));
  v = min(v, dpp_i<DPP_QUAD_XOR2>(v));
  v = min(v, dpp_i<DPP_ROW_HALF_MIRROR>(v));
  v = min(v, dpp_i<DPP_ROW_MIRROR>(v));
  return min(min(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
             min(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

// a*c + b*s with both products rounded before the add (the reference multiplies and adds as
// separate tensor ops, src/vui/rope.py:50); contraction into an fma is switched off here.
__device__ __forceinline__ float rope_mix(float a, float c, float b, float s) {
#pragma clang fp contract(off)
  const float p0 = a * c;
  const float p1 = b * s;
  return p0 + p1;
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + __expf(-x)); }

// ---- values that workgroups of one launch hand to each other ----
// Device-scope relaxed accesses bypass the per-XCD L2s (write-through stores, loads served from memory), so
// another workgroup's value is seen without a cache flush.  After such stores `s_waitcnt vmcnt(0)` means
// they have completed; a counter incremented afterwards tells the last arriver that everything is there.
__device__ __forceinline__ void st_dev(float* p, float a, float b) {
  __hip_atomic_store(reinterpret_cast<uint64_t*>(p), ((uint64_t)__float_as_uint(b) << 32) | __float_as_uint(a),
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t ld_dev(const float* p) {
  return __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float lo_f(uint64_t v) { return __uint_as_float((uint32_t)v); }
__device__ __forceinline__ float hi_f(uint64_t v) { return __uint_as_float((uint32_t)(v >> 32)); }
