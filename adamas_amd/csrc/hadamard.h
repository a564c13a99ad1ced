// Hadamard transform, 4-level bucketize, 2-bit packing and rotary-embedding helpers shared by the
// append kernels (hadamard.hip) and the decode-step kernels that take the fused projection directly.
//
// The numeric contract is "one IEEE fp32 operation per butterfly step, one fp32 multiply by the
// scale, one rounding to the 16-bit format": every function that does arithmetic switches fp
// contraction off for its own body, so that including this header leaves the rest of a translation
// unit alone.
#pragma once

#include "common.h"

namespace adamas {

// x0, x1: channels 2*lane and 2*lane+1 of the row.  On return they hold the transformed channels.
__device__ __forceinline__ void wave_hadamard128(float& x0, float& x1, int lane) {
#pragma clang fp contract(off)
  float a = x0, b = x1;
  x0 = a + b;  // stride 1
  x1 = a - b;
#pragma unroll
  for (int m = 1; m < kWave; m <<= 1) {  // lane distance m == channel stride 2m
    float p0 = __shfl_xor(x0, m);
    float p1 = __shfl_xor(x1, m);
    bool upper = (lane & m) != 0;
    // lower lane holds a, partner b -> a + b ; upper lane holds b, partner a -> a - b
    x0 = upper ? (p0 - x0) : (x0 + p0);
    x1 = upper ? (p1 - x1) : (x1 + p1);
  }
}

// Codes of the two channels of this lane -> the 16 packed words of the row.  After the call the
// lanes with (lane & 3) == 0 hold word lane/4 in the low 16 bits of the return value.
__device__ __forceinline__ uint32_t wave_pack_codes(float v0, float v1, int lane) {
  uint32_t nib = bucket4(v0) | (bucket4(v1) << 2);
  uint32_t part = nib << (4 * (lane & 3));
  part |= __shfl_xor(part, 1);
  part |= __shfl_xor(part, 2);
  return part & 0xffffu;
}

template <bool kBf16 = false>
__device__ __forceinline__ void load_pair(const __half* row, int lane, float& x0, float& x1) {
  unpack2<kBf16>(reinterpret_cast<const uint32_t*>(row)[lane], x0, x1);
}

// fp32 product with its own rounding: the empty asm keeps the compiler from merging the multiply
// and a following fp16 conversion into one mixed-precision instruction (v_fma_mixlo_f16).
__device__ __forceinline__ float scaled_f32(float x, float scale) {
#pragma clang fp contract(off)
  float y = x * scale;
  asm volatile("" : "+v"(y));
  return y;
}

// Transform + scale + (optionally) rounding to the 16-bit format of the data, exactly as the code
// generation defines it.
template <bool kBf16 = false>
__device__ __forceinline__ void transform_row(float& x0, float& x1, int lane, float scale,
                                              bool keep_fp32) {
  wave_hadamard128(x0, x1, lane);
  x0 = scaled_f32(x0, scale);
  x1 = scaled_f32(x1, scale);
  if (!keep_fp32) {
    x0 = round_elem<kBf16>(x0);
    x1 = round_elem<kBf16>(x1);
  }
}

// ------------------------------------------------------------------------------------------------
// The same transform with a row spread over 16 lanes (8 adjacent channels = one 128-bit access per
// lane, four rows per wave): the layout of the kernels that stream many rows.
// ------------------------------------------------------------------------------------------------
// value of lane (l ^ kMask) of the 16-lane row, kMask in {1, 2, 4, 8}
template <int kMask>
__device__ __forceinline__ float row_xor(float v) {
  const int x = __float_as_int(v);
  int r;
  if (kMask == 1) {
    r = __builtin_amdgcn_update_dpp(x, x, 0xB1, 0xF, 0xF, false);  // quad_perm [1,0,3,2]
  } else if (kMask == 2) {
    r = __builtin_amdgcn_update_dpp(x, x, 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
  } else if (kMask == 4) {
    r = __builtin_amdgcn_update_dpp(x, x, 0x104, 0xF, 0x5, false);  // row_shl:4 into banks 0, 2
    r = __builtin_amdgcn_update_dpp(r, x, 0x114, 0xF, 0xA, false);  // row_shr:4 into banks 1, 3
  } else {
    r = __builtin_amdgcn_update_dpp(x, x, 0x128, 0xF, 0xF, false);  // row_ror:8
  }
  return __int_as_float(r);
}

template <int kMask>
__device__ __forceinline__ void row_butterfly_stage(float (&x)[8], uint32_t c) {
#pragma clang fp contract(off)
  const bool upper = (c & kMask) != 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float p = row_xor<kMask>(x[e]);
    x[e] = upper ? (p - x[e]) : (x[e] + p);  // lower lane: a + b, upper lane: a - b
  }
}

// x: channels 8c .. 8c+7 of a row spread over 16 lanes; transformed in place (unscaled)
__device__ __forceinline__ void row_hadamard128(float (&x)[8], uint32_t c) {
#pragma clang fp contract(off)
#pragma unroll
  for (int s = 1; s < 8; s <<= 1) {
#pragma unroll
    for (int lo = 0; lo < 8; ++lo) {
      if (lo & s) continue;
      const float a = x[lo], b = x[lo | s];
      x[lo] = a + b;
      x[lo | s] = a - b;
    }
  }
  row_butterfly_stage<1>(x, c);
  row_butterfly_stage<2>(x, c);
  row_butterfly_stage<4>(x, c);
  row_butterfly_stage<8>(x, c);
}

template <bool kBf16>
__device__ __forceinline__ void unpack_elem8(const uint4& raw, float (&x)[8]) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) unpack2<kBf16>(w[i], x[2 * i], x[2 * i + 1]);
}


// element offset of the K (kv = 0) or V (kv = 1) row of (page, slot, head) in a KV page pool:
// pages are [2][page_size][heads][128], or [2][heads][page_size][128] with ADAMAS_F_HND
__device__ __forceinline__ size_t kv_row_offset(size_t page, uint32_t kv, uint32_t slot, uint32_t hd,
                                                uint32_t page_size, uint32_t num_heads,
                                                uint32_t flags) {
  if (flags & ADAMAS_F_HND) return (((page * 2 + kv) * num_heads + hd) * page_size + slot) * kHeadDim;
  return (((page * 2 + kv) * page_size + slot) * num_heads + hd) * kHeadDim;
}

// Rotary embedding of one channel pair (c, c + 64) in rotate-half pairing: `x` is this lane's
// value, `partner` the value of the paired channel, `upper` whether this lane holds the channel
// c + 64.  lower: x*cos - partner*sin, upper: x*cos + partner*sin; two products and one sum, each
// rounded on its own.
__device__ __forceinline__ float rope_channel(float x, float partner, float c, float s, bool upper) {
#pragma clang fp contract(off)
  return upper ? x * c + partner * s : x * c - partner * s;
}

}  // namespace adamas
