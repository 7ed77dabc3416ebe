// Epilogues shared by the row-per-wave GEMV (gemv.hip) and the 16-row MFMA GEMM (gemm16.hip).
#pragma once
#include "common.h"
#include "internal.h"

// n: output feature, b: activation row, v: fp32 dot product, vp: dot product of the rotary partner
// row (n ^ 1), v2: dot product with the second matrix (SwiGLU).
template <typename T>
__device__ __forceinline__ void epilogue(const GemvArgs& p, int n, int b, float v, float vp, float v2) {
  if (n >= p.N) return;
  T* y = (T*)p.y;
  switch (p.epi) {
    case EPI_STORE:
      El<T>::st(y + (size_t)b * p.ldy + n, v);
      break;
    case EPI_RESID: {
      float r = El<T>::ld((const T*)p.resid + (size_t)b * p.ldy + n);
      El<T>::st(y + (size_t)b * p.ldy + n, r + El<T>::rnd(v));
    } break;
    case EPI_ADDVEC:
      El<T>::st(y + (size_t)b * p.ldy + n, El<T>::rnd(v) + El<T>::ld((const T*)p.vec + n));
      break;
    case EPI_SWIGLU: {
      float a = El<T>::rnd(v), c = El<T>::rnd(v2);
      float s = El<T>::rnd(a / (1.0f + expf(-a)));
      El<T>::st(y + (size_t)b * p.ldy + n, s * c);
    } break;
    case EPI_QKV: {
      const int slot = p.slot_idx ? p.slot_idx[b] : b;
      const int pos = p.seq_lens[slot];
      float val = El<T>::rnd(v);
      int region, m;  // 0 q, 1 k, 2 v ; m = index inside the region
      if (n < p.nq) { region = 0; m = n; }
      else if (n < p.nq + p.nkv) { region = 1; m = n - p.nq; }
      else { region = 2; m = n - p.nq - p.nkv; }
      const int dd = m % p.hd;
      if (region != 2 && dd < p.rope_dim && pos >= 0 && pos < p.S) {
        const float* f = p.rope + ((size_t)pos * p.rope_dim + dd) * 2;
        const float partner = El<T>::rnd(vp);
        const float rot = (dd & 1) ? partner : -partner;
        val = rope_mix(val, f[0], rot, f[1]);
      }
      if (region == 0) {
        El<T>::st(y + (size_t)b * p.ldy + m, val);
      } else if (pos >= 0 && pos < p.S) {
        T* c = (T*)(region == 1 ? p.kc : p.vc);
        El<T>::st(c + ((size_t)slot * p.S + pos) * p.nkv + m, val);
      }
    } break;
    case EPI_RQ_QKV: {
      const int R = p.nq;
      if (n < R) El<T>::st(y + (size_t)b * p.ldy + n, v);
      else if (n < 2 * R) El<T>::st((T*)p.kc + ((size_t)b * p.S + p.rq_pos) * R + (n - R), v);
      else El<T>::st((T*)p.vc + ((size_t)b * p.S + p.rq_pos) * R + (n - 2 * R), v);
    } break;
  }
}

