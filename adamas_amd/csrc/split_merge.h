// Split results that are merged inside the launch that produced them (gfx950).
//
// Several workgroups each hold a partial softmax state (m, l, o[128]) of one head; the last one to
// arrive folds them.  The partials cross workgroups inside one launch, so they are written and read
// with agent-scope relaxed atomics (write-through stores, cache-bypassing loads) instead of plain
// accesses fenced by __threadfence(): an agent-scope fence on this multi-die part writes back and
// invalidates a whole L2, once per workgroup.  The ordering that takes the place of the fence is
// kept in ONE function, split_arrive_is_last():
//   1. every wave that stored a partial waits until the memory system has acknowledged its own
//      write-through stores (s_waitcnt vmcnt(0): a workgroup barrier alone waits for LDS traffic only);
//   2. a workgroup barrier orders all those waits ahead of
//   3. one relaxed agent-scope add on the arrival counter (thread 0);
//   4. the workgroup that reads n_split - 1 from the counter knows that every other workgroup passed
//      step 1 for all of its stores before its add, so the cache-bypassing loads of merge_partials()
//      find every partial in memory.
// This is an argument about the hardware (acknowledged write-through stores are visible to
// cache-bypassing loads of any CU), not about the HIP memory model; it is covered by tests that run
// many launches and compare their bits.  Where there are many splits the kernels write plain
// partials instead and leave the merge to a launch of its own, which needs none of this.
#pragma once

#include "attend.h"
#include "workspace.h"

namespace adamas {

// Called by every thread of the workgroup after it has issued its agent-scope stores of the partial.
// Returns true in every thread of the workgroup that arrived last for this counter (false in all
// others); is_last_lds is a word of LDS.  The caller of the last workgroup merges and then puts the
// counter back to zero for the next launch on the stream.
__device__ __forceinline__ bool split_arrive_is_last(uint32_t* counter, uint32_t n_split,
                                                     uint32_t& is_last_lds, uint32_t tid) {
  wait_own_stores();
  __syncthreads();
  if (tid == 0) {
    const uint32_t prev = atomicAdd(counter, 1u);
    is_last_lds = (prev == n_split - 1) ? 1u : 0u;
  }
  __syncthreads();
  return is_last_lds != 0;
}

// Merge of the n_split partial states (m, l, o[128]) of one head, read with agent-scope loads: the
// values of `kVec` channels starting at channel `ch` for this thread.  kBatch splits are fetched
// per round (all loads of a round are independent) and folded into a running (M, L, A) with the
// usual rescaling, so 128 splits cost 128 / kBatch memory round trips instead of 128.
template <int kVec, int kBatch = 16>
__device__ __forceinline__ void merge_partials(const float* base, uint32_t n_split, uint32_t ch,
                                               float& L, float (&A)[kVec]) {
  float M = kNegBig;
  L = 0.f;
#pragma unroll
  for (int e = 0; e < kVec; ++e) A[e] = 0.f;
  for (uint32_t s0 = 0; s0 < n_split; s0 += kBatch) {
    float m[kBatch], l[kBatch], a[kBatch][kVec];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const uint32_t s2 = min(s0 + u, n_split - 1);  // past the end: a duplicate, weighted zero below
      const float* p = base + static_cast<size_t>(s2) * kPartialFloats;
      m[u] = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      l[u] = __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int e = 0; e < kVec; ++e)
        a[u][e] = __hip_atomic_load(p + 2 + ch + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    float m_new = M;
#pragma unroll
    for (int u = 0; u < kBatch; ++u) m_new = fmaxf(m_new, s0 + u < n_split ? m[u] : kNegBig);
    const float keep = exp2_raw(M - m_new);
    L *= keep;
#pragma unroll
    for (int e = 0; e < kVec; ++e) A[e] *= keep;
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const float w = s0 + u < n_split ? exp2_raw(m[u] - m_new) : 0.f;
      L += l[u] * w;
#pragma unroll
      for (int e = 0; e < kVec; ++e) A[e] += a[u][e] * w;
    }
    M = m_new;
  }
}

// The same for two adjacent channels (ch even) with 64-bit accesses: (m, l) and the channel pair of a
// partial are each one load, and a thread publishes its pair with one store.
__device__ __forceinline__ void store_partial_pair(float* p, float a, float b) {
  const uint64_t v = static_cast<uint64_t>(__float_as_uint(a)) |
                     (static_cast<uint64_t>(__float_as_uint(b)) << 32);
  __hip_atomic_store(reinterpret_cast<uint64_t*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int kBatch>
__device__ __forceinline__ void merge_partial_pairs(const float* base, uint32_t n_split, uint32_t ch,
                                                    float& L, float (&A)[2]) {
  float M = kNegBig;
  L = 0.f;
  A[0] = A[1] = 0.f;
  for (uint32_t s0 = 0; s0 < n_split; s0 += kBatch) {
    uint64_t ml[kBatch], aa[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const uint32_t s2 = min(s0 + u, n_split - 1);  // past the end: a duplicate, weighted zero below
      const uint64_t* p =
          reinterpret_cast<const uint64_t*>(base + static_cast<size_t>(s2) * kPartialFloats);
      ml[u] = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      aa[u] = __hip_atomic_load(p + 1 + ch / 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    float m_new = M;
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
      m_new = fmaxf(m_new, s0 + u < n_split ? __uint_as_float(static_cast<uint32_t>(ml[u])) : kNegBig);
    const float keep = exp2_raw(M - m_new);
    L *= keep;
    A[0] *= keep;
    A[1] *= keep;
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const float w = s0 + u < n_split
                          ? exp2_raw(__uint_as_float(static_cast<uint32_t>(ml[u])) - m_new)
                          : 0.f;
      L += __uint_as_float(static_cast<uint32_t>(ml[u] >> 32)) * w;
      A[0] += __uint_as_float(static_cast<uint32_t>(aa[u])) * w;
      A[1] += __uint_as_float(static_cast<uint32_t>(aa[u] >> 32)) * w;
    }
    M = m_new;
  }
}

}  // namespace adamas
