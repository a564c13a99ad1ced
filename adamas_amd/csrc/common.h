// Shared device helpers for the gfx950 kernels of libadamas_hip.so.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/adamas_hip.h"

namespace adamas {

constexpr int kHeadDim = ADAMAS_HEAD_DIM;      // channels per head
constexpr int kCodeWords = ADAMAS_CODE_WORDS;  // u16 words of code per (token, head)
constexpr int kWave = 64;                      // CDNA wavefront width

// Launch-error check used by every host launcher: returns the hipError_t as a positive int.
#define ADAMAS_RETURN_IF_LAUNCH_FAILED()            \
  do {                                              \
    hipError_t e_ = hipGetLastError();              \
    if (e_ != hipSuccess) return static_cast<int>(e_); \
  } while (0)

__device__ __forceinline__ int wave_id_uniform() {
  // threadIdx.x / 64 is the same for all lanes of a wave; tell the compiler so that everything
  // derived from it lives in scalar registers.
  return __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
}

// Waits until every global store this wave has issued is acknowledged by the memory system.  A
// workgroup barrier does not: it waits for LDS traffic only, so a wave that publishes data with
// write-through stores for another workgroup calls this before the barrier that precedes the flag.
__device__ __forceinline__ void wait_own_stores() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

__device__ __forceinline__ int lane_id() { return static_cast<int>(threadIdx.x) & 63; }

// 4-level bucket of a Hadamard output value: (v > -10) + (v > 0) + (v > 10).
__device__ __forceinline__ uint32_t bucket4(float v) {
  return static_cast<uint32_t>(v > -10.0f) + static_cast<uint32_t>(v > 0.0f) +
         static_cast<uint32_t>(v > 10.0f);
}

// ---- the two 16-bit float formats of q, K, V and the outputs -------------------------------------
// Kernels that read or write float data take `bool kBf16`: false = IEEE fp16 (the reference's only
// dtype), true = bfloat16.  Pointers to such data are typed __half* in both cases and only used for
// 2-byte address arithmetic.

// bits of the bfloat16 nearest to x (ties to even; NaN stays a quiet NaN)
__device__ __forceinline__ uint32_t bf16_bits(float x) {
  const uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x0040u;
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

template <bool kBf16>
__device__ __forceinline__ uint32_t elem_bits(float x) {
  if (kBf16) return bf16_bits(x);
  return static_cast<uint32_t>(__half_as_ushort(__float2half_rn(x)));
}

// x rounded to the 16-bit format and back: what a tensor of that dtype would hold
template <bool kBf16>
__device__ __forceinline__ float round_elem(float x) {
  if (kBf16) return __uint_as_float(bf16_bits(x) << 16);
  return __half2float(__float2half_rn(x));
}

// two adjacent elements of one 32-bit word (low half = lower address)
template <bool kBf16>
__device__ __forceinline__ void unpack2(uint32_t w, float& lo, float& hi) {
  if (kBf16) {
    lo = __uint_as_float(w << 16);
    hi = __uint_as_float(w & 0xffff0000u);
  } else {
    const __half2 hv = *reinterpret_cast<const __half2*>(&w);
    lo = __low2float(hv);
    hi = __high2float(hv);
  }
}

template <bool kBf16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  return elem_bits<kBf16>(lo) | (elem_bits<kBf16>(hi) << 16);
}

template <bool kBf16>
__device__ __forceinline__ void store_elem(__half* p, float x) {
  *reinterpret_cast<uint16_t*>(p) = static_cast<uint16_t>(elem_bits<kBf16>(x));
}

// Key/value head of a query head, head / group with group = num_heads / num_kv_heads, without a
// division in the kernel: the host passes the 16-bit reciprocal of the group size.  Exact while
// head * group < 65536 (the host checks num_heads * group).
inline uint32_t group_inv16(uint32_t group) { return (65536u + group - 1u) / group; }
__device__ __forceinline__ uint32_t kv_head_of(uint32_t head, uint32_t inv16) {
  return (head * inv16) >> 16;
}

// Physical location of logical token t of a sequence whose page table starts at `table`.
template <typename T>
__device__ __forceinline__ T token_slot(const int32_t* __restrict__ table, uint32_t t,
                                        uint32_t page_size) {
  uint32_t lp = t / page_size;
  uint32_t slot = t - lp * page_size;
  return static_cast<T>(table[lp]) * page_size + slot;
}

}  // namespace adamas
