// Flag-in-data exchange between the resident workgroups of a persistent kernel: an 8-byte word =
// 4 bytes of payload + the 4-byte launch epoch, written and polled with device-scope relaxed
// atomics (which bypass the per-XCD L2s).  A word that shows the current epoch is the data.
#pragma once
#include "common.h"

#define FR_THREADS 256
#define SPIN_LIMIT (1 << 21)
#ifndef POLL_SLEEP
#define POLL_SLEEP 0
#endif
#ifndef POLL_DELAY
#define POLL_DELAY 0
#endif

__device__ __forceinline__ uint64_t ll_ld(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void ll_st(uint64_t* p, uint32_t payload, uint32_t epoch) {
  __hip_atomic_store(p, ((uint64_t)epoch << 32) | payload, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Vectors that every workgroup reads can be kept in LL_REP copies, copy r read by the workgroups with
// index % LL_REP == r (those share an XCD); writers store all copies with one instruction (lanes
// 0..LL_REP-1).  Measured: 8 copies shorten a bare exchange of <= 512 words between 256 workgroups by
// 0.4-0.8 us in isolation but not inside this kernel, so one copy is used.
#define LL_REP 1
struct RepBuf { uint64_t* base; int n; };
__device__ __forceinline__ RepBuf rep_alloc(uint64_t*& llp, int n) { RepBuf b = {llp, n}; llp += (size_t)LL_REP * n; return b; }
__device__ __forceinline__ const uint64_t* rep_rd(const RepBuf& b) { return b.base + (size_t)(blockIdx.x & (LL_REP - 1)) * b.n; }
// every lane of the wave calls this with the same (i, payload)
__device__ __forceinline__ void rep_st(const RepBuf& b, int i, uint32_t payload, uint32_t epoch) {
  const int lane = threadIdx.x & 63;
  if (lane < LL_REP) ll_st(b.base + (size_t)lane * b.n + i, payload, epoch);
}
__device__ __forceinline__ uint32_t pack2(float a, float b) { return f2bf2(a, b); }

struct Ctl {
  uint32_t epoch;
  uint32_t* err;
  int dead;
};

// Launch handshake of a persistent kernel over three control words: the epoch of the last finished launch, the
// number of workgroups of the running launch that have read it, and a sticky error word.
// A launch uses epoch + 1.  Epoch 0 means "never written" in every exchange word, so when the 32-bit count
// wraps the launch raises the error word (value 2) instead of running: the host re-initialises the context
// (which zeroes the words) and goes on.
__device__ __forceinline__ void ctl_begin(Ctl& c, const uint32_t* epoch, uint32_t* err) {
  c.epoch = __hip_atomic_load(epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
  c.err = err;
  c.dead = 0;
  if (c.epoch == 0u) {
    c.dead = 1;
    if (threadIdx.x == 0) __hip_atomic_store(err, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}
// A non-zero error word (this launch or an earlier one): results must not be committed.
__device__ __forceinline__ bool ctl_failed(const Ctl& c) {
  return __hip_atomic_load(c.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
}
// One thread of workgroup 0, last thing in the launch: every workgroup has read the epoch before it may change.
// If some workgroup never arrives the error word is raised and the words are left as they are; the context is
// then unusable until it is re-initialised (a late arrival would otherwise be counted into the next launch).
__device__ __forceinline__ void ctl_finish(const Ctl& c, uint32_t* epoch, uint32_t* arrive, uint32_t nwg) {
  int spins = 0;
  while (__hip_atomic_load(arrive, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < nwg) {
    if (++spins >= SPIN_LIMIT) {
      __hip_atomic_store(c.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    if (POLL_SLEEP) __builtin_amdgcn_s_sleep(POLL_SLEEP);
  }
  if (ctl_failed(c)) return;
  __hip_atomic_store(arrive, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(epoch, c.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Wait until words [0, n) of buf carry the current epoch; sink(i, payload) once per word.
// Threads take words tid, tid+256, ...  A thread that exceeds the spin limit raises the error
// word and stops waiting for the rest of the launch, so every wave always reaches the end.
template <typename F>
__device__ __forceinline__ void ll_poll(const uint64_t* buf, int n, Ctl& c, F&& sink) {
  if (POLL_DELAY) __builtin_amdgcn_s_sleep(POLL_DELAY);
  for (int base = 0; base < n; base += FR_THREADS * 4) {
    int idx[4];
    bool ok[4];
    uint64_t v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { idx[i] = base + (int)threadIdx.x + FR_THREADS * i; ok[i] = idx[i] >= n; }
    int spins = 0;
    while (true) {
#pragma unroll
      for (int i = 0; i < 4; ++i) if (!ok[i]) v[i] = ll_ld(buf + idx[i]);
      bool all = true;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (!ok[i]) {
          if ((uint32_t)(v[i] >> 32) == c.epoch || c.dead) { ok[i] = true; sink(idx[i], (uint32_t)v[i]); }
          else all = false;
        }
      if (all) break;
      if (++spins > SPIN_LIMIT) {
        c.dead = 1;
        __hip_atomic_store(c.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      if (POLL_SLEEP) __builtin_amdgcn_s_sleep(POLL_SLEEP);
    }
  }
}

// Straight-line form of the same wait: every thread has exactly NW words in flight (word tid + 256 * i, clamped to the
// last word: threads past the end wait for that one too and drop it) and re-reads all of them until all carry the
// epoch.  One loop, one exit test per round, no per-word branches: a third of the instructions of ll_poll.
// NW * 256 >= n.
template <int NW, typename F>
__device__ __forceinline__ void ll_poll_n(const uint64_t* buf, int n, Ctl& c, F&& sink) {
  const uint64_t* p[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i) p[i] = buf + min((int)threadIdx.x + FR_THREADS * i, n - 1);
  uint64_t v[NW];
  int spins = 0;
  while (true) {
#pragma unroll
    for (int i = 0; i < NW; ++i) v[i] = ll_ld(p[i]);
    uint32_t bad = 0;
#pragma unroll
    for (int i = 0; i < NW; ++i) bad |= (uint32_t)(v[i] >> 32) ^ c.epoch;
    if (bad == 0u || c.dead) break;
    if (++spins > SPIN_LIMIT) {
      c.dead = 1;
      __hip_atomic_store(c.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (POLL_SLEEP) __builtin_amdgcn_s_sleep(POLL_SLEEP);
  }
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int idx = (int)threadIdx.x + FR_THREADS * i;
    if (idx < n) sink(idx, (uint32_t)v[i]);
  }
}
// picks the round count from the vector length (uniform over the workgroup).  Precondition: n >= 1 - the clamped
// addresses of ll_poll_n would point in front of an empty vector.  Every caller waits for a vector whose length is a
// model dimension (or a row count that it has tested to be positive), and the host refuses configurations with a
// zero dimension (check_cfg, rq_batch_supported, the codec's init), so the waits carry no test of their own.
template <typename F>
__device__ __forceinline__ void ll_poll_auto(const uint64_t* buf, int n, Ctl& c, F&& sink) {
  if (n <= FR_THREADS) ll_poll_n<1>(buf, n, c, sink);
  else if (n <= 2 * FR_THREADS) ll_poll_n<2>(buf, n, c, sink);
  else if (n <= 3 * FR_THREADS) ll_poll_n<3>(buf, n, c, sink);
  else if (n <= 4 * FR_THREADS) ll_poll_n<4>(buf, n, c, sink);
  else if (n <= 6 * FR_THREADS) ll_poll_n<6>(buf, n, c, sink);
  else ll_poll(buf, n, c, sink);
}

// The same for long vectors: every thread has NW words in flight at once (one round trip for 256 * NW
// words when the data is there), stragglers are re-read one by one.
template <int NW, typename F>
__device__ __forceinline__ void ll_poll_wide(const uint64_t* buf, int n, Ctl& c, F&& sink) {
  for (int base = 0; base < n; base += FR_THREADS * NW) {
    uint64_t v[NW];
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int idx = base + (int)threadIdx.x + FR_THREADS * i;
      v[i] = idx < n ? ll_ld(buf + idx) : 0;
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int idx = base + (int)threadIdx.x + FR_THREADS * i;
      if (idx < n) {
        int spins = 0;
        while ((uint32_t)(v[i] >> 32) != c.epoch && !c.dead) {
          v[i] = ll_ld(buf + idx);
          if (++spins > SPIN_LIMIT) {
            c.dead = 1;
            __hip_atomic_store(c.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
        sink(idx, (uint32_t)v[i]);
      }
    }
  }
}

// wait for up to 3 scattered words per thread (nullptr = none); returns payloads
__device__ __forceinline__ void poll3(const uint64_t* p0, const uint64_t* p1, const uint64_t* p2, Ctl& c, uint32_t& r0,
                                      uint32_t& r1, uint32_t& r2) {
  bool k0 = p0 == nullptr, k1 = p1 == nullptr, k2 = p2 == nullptr;
  uint64_t v0 = 0, v1 = 0, v2 = 0;
  int spins = 0;
  while (true) {
    if (!k0) v0 = ll_ld(p0);
    if (!k1) v1 = ll_ld(p1);
    if (!k2) v2 = ll_ld(p2);
    if (!k0 && ((uint32_t)(v0 >> 32) == c.epoch || c.dead)) k0 = true;
    if (!k1 && ((uint32_t)(v1 >> 32) == c.epoch || c.dead)) k1 = true;
    if (!k2 && ((uint32_t)(v2 >> 32) == c.epoch || c.dead)) k2 = true;
    if (k0 && k1 && k2) break;
    if (++spins > SPIN_LIMIT) { c.dead = 1; __hip_atomic_store(c.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    if (POLL_SLEEP) __builtin_amdgcn_s_sleep(POLL_SLEEP);
  }
  r0 = (uint32_t)v0; r1 = (uint32_t)v1; r2 = (uint32_t)v2;
}

