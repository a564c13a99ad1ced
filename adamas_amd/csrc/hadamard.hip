// Hadamard transform, 4-level bucketize, 2-bit packing and the KV/code append kernels (gfx950).
//
// One wave64 owns one row of 128 channels: lane l holds channels 2l and 2l+1.  The butterfly runs
// stride 1 inside the lane and strides 2..64 across lanes; every stage is a plain fp32 add or
// subtract of the same operand pairs a sequential radix-2 butterfly would form, so the result is
// bit-identical to a CPU restatement that uses the same stage order.
#include "hadamard.h"

// The numeric contract of this file is "one IEEE fp32 operation per butterfly step, one fp32
// multiply by the scale, one rounding to fp16".  Contraction would let the compiler merge the
// multiply and the fp16 rounding into a single mixed-precision instruction with one rounding.
#pragma clang fp contract(off)

namespace adamas {
// ------------------------------------------------------------------------------------------------
// Standalone transform: out = fp16 or bf16 of (x . H_128 * scale); a wave owns four adjacent rows
// ------------------------------------------------------------------------------------------------
template <bool kBf16>
__global__ __launch_bounds__(256) void hadamard_rows_kernel(const __half* x, __half* out,
                                                            uint64_t n_rows, float scale) {
  const uint32_t lane = static_cast<uint32_t>(lane_id());
  const uint32_t c = lane & 15u;
  const uint64_t r = (static_cast<uint64_t>(blockIdx.x) * 4 + wave_id_uniform()) * 4 + (lane >> 4);
  if (r >= n_rows) return;  // whole 16-lane rows drop out together
  float f[8];
  unpack_elem8<kBf16>(*reinterpret_cast<const uint4*>(x + r * kHeadDim + 8u * c), f);
  row_hadamard128(f, c);
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = pack2<kBf16>(scaled_f32(f[2 * i], scale), scaled_f32(f[2 * i + 1], scale));
  *reinterpret_cast<uint4*>(out + r * kHeadDim + 8u * c) = make_uint4(w[0], w[1], w[2], w[3]);
}

// ------------------------------------------------------------------------------------------------
// pack_2bit of integer-valued fp16 (or bf16) input: word = sum (uint16(v) & 3) << 2i
// ------------------------------------------------------------------------------------------------
template <bool kBf16>
__global__ __launch_bounds__(256) void pack_2bit_kernel(const __half* __restrict__ h,
                                                        uint16_t* __restrict__ o,
                                                        uint64_t n_words) {
  uint64_t w = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (; w < n_words; w += stride) {
    const uint4 raw = *reinterpret_cast<const uint4*>(h + w * 8);
    float v[8];
    unpack_elem8<kBf16>(raw, v);
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t c = static_cast<uint32_t>(static_cast<int>(v[i])) & 3u;
      packed |= c << (2 * i);
    }
    o[w] = static_cast<uint16_t>(packed);
  }
}

// ------------------------------------------------------------------------------------------------
// Decode append: rows [0, batch*Hq) are query rows, rows [batch*Hq, batch*(Hq+Hkv)) are key rows.
// ------------------------------------------------------------------------------------------------
template <bool kBf16>
__global__ __launch_bounds__(256) void append_decode_kernel(
    const __half* __restrict__ q, const __half* __restrict__ k, const __half* __restrict__ v,
    const __half* __restrict__ h, uint16_t* __restrict__ q_code_out, __half* __restrict__ kv_data,
    uint16_t* __restrict__ code_data, const int32_t* __restrict__ page_indices,
    const int32_t* __restrict__ page_indptr, const int32_t* __restrict__ seq_lens, uint32_t batch,
    uint32_t num_q_heads, uint32_t num_heads, uint32_t page_size, float scale, uint32_t flags) {
  // num_heads: key/value heads (the caches), num_q_heads: query heads
  const int lane = lane_id();
  const uint32_t q_rows = batch * num_q_heads;
  const uint32_t r = blockIdx.x * 4 + wave_id_uniform();
  if (r >= q_rows + batch * num_heads) return;
  const uint32_t kind = r < q_rows ? 0u : 1u;  // 0 = query, 1 = key
  const uint32_t bh = r - kind * q_rows;        // row inside q, or inside k and v
  const uint32_t b = bh / num_heads;            // only used for key rows
  const uint32_t hd = bh - b * num_heads;

  float x0, x1;
  if (h != nullptr) {
    load_pair<kBf16>(h + static_cast<size_t>(r) * kHeadDim, lane, x0, x1);
  } else {
    const __half* src = (kind == 0 ? q : k) + static_cast<size_t>(bh) * kHeadDim;
    load_pair<kBf16>(src, lane, x0, x1);
    transform_row<kBf16>(x0, x1, lane, scale, (flags & ADAMAS_F_CODE_FROM_FP32) != 0);
  }
  const uint32_t word = wave_pack_codes(x0, x1, lane);

  if (kind == 0) {
    if ((lane & 3) == 0) q_code_out[static_cast<size_t>(bh) * kCodeWords + (lane >> 2)] =
        static_cast<uint16_t>(word);
    return;
  }
  const uint32_t pos = static_cast<uint32_t>(seq_lens[b]) - 1u;
  const int32_t* table = page_indices + page_indptr[b];
  const uint32_t lp = pos / page_size;
  const uint32_t slot = pos - lp * page_size;
  const size_t page = static_cast<size_t>(table[lp]);
  if ((lane & 3) == 0)
    code_data[((page * page_size + slot) * num_heads + hd) * kCodeWords + (lane >> 2)] =
        static_cast<uint16_t>(word);
  // copy the raw key and value rows into the KV page
  const size_t k_off = kv_row_offset(page, 0, slot, hd, page_size, num_heads, flags);
  const size_t v_off = kv_row_offset(page, 1, slot, hd, page_size, num_heads, flags);
  const uint32_t* ks = reinterpret_cast<const uint32_t*>(k + static_cast<size_t>(bh) * kHeadDim);
  const uint32_t* vs = reinterpret_cast<const uint32_t*>(v + static_cast<size_t>(bh) * kHeadDim);
  reinterpret_cast<uint32_t*>(kv_data + k_off)[lane] = ks[lane];
  reinterpret_cast<uint32_t*>(kv_data + v_off)[lane] = vs[lane];
}

// ------------------------------------------------------------------------------------------------
// Decode append straight from the fused q/k/v projection: rotary embedding, KV append and both codes
// in one launch.  qkv [batch][Hq + 2*Hkv][128]; wave r = (sequence b, query head): lane l holds channels 2l, 2l+1,
// whose rotary partners (channel +-64) sit in lane l ^ 32.  q (rotated) goes to q_out for the
// attention kernels, k (rotated) and v into the KV page of position seq_lens[b] - 1, the codes of
// Hadamard(q) and Hadamard(k) to q_code_out and the code page.  The rotated values are rounded to fp16
// before the transform, exactly as if they had been stored and appended separately.
// ------------------------------------------------------------------------------------------------
template <bool kBf16>
__global__ __launch_bounds__(256) void rope_append_decode_kernel(
    const __half* __restrict__ qkv, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, __half* __restrict__ q_out,
    uint16_t* __restrict__ q_code_out, __half* __restrict__ kv_data,
    uint16_t* __restrict__ code_data, const int32_t* __restrict__ page_indices,
    const int32_t* __restrict__ page_indptr, const int32_t* __restrict__ seq_lens, uint32_t batch,
    uint32_t num_q_heads, uint32_t num_heads, uint32_t page_size, float scale, uint32_t flags) {
  // one wave per (sequence, query head); the waves of the first num_heads (key/value) heads also
  // carry the key and value row of that head
  const int lane = lane_id();
  const uint32_t bh = blockIdx.x * 4 + wave_id_uniform();
  if (bh >= batch * num_q_heads) return;
  const uint32_t b = bh / num_q_heads;
  const uint32_t hd = bh - b * num_q_heads;
  const bool has_kv = hd < num_heads;
  const uint32_t pos = static_cast<uint32_t>(seq_lens[b]) - 1u;

  const size_t row_len = static_cast<size_t>(num_q_heads + 2 * num_heads) * kHeadDim;
  const __half* row = qkv + static_cast<size_t>(b) * row_len;
  float q0, q1, k0 = 0.f, k1 = 0.f;
  load_pair<kBf16>(row + static_cast<size_t>(hd) * kHeadDim, lane, q0, q1);
  if (has_kv) load_pair<kBf16>(row + static_cast<size_t>(num_q_heads + hd) * kHeadDim, lane, k0, k1);

  // channel c pairs with c + 64 (lanes l and l + 32): out_lo = lo*cos - hi*sin, out_hi = hi*cos + lo*sin
  const uint32_t c0 = (2u * static_cast<uint32_t>(lane)) & 63u;  // table column of channel 2l
  const float2 cs = *reinterpret_cast<const float2*>(cos_table + static_cast<size_t>(pos) * 64 + c0);
  const float2 sn = *reinterpret_cast<const float2*>(sin_table + static_cast<size_t>(pos) * 64 + c0);
  const bool upper = lane >= 32;
  const float pq0 = __shfl_xor(q0, 32), pq1 = __shfl_xor(q1, 32);
  const float pk0 = __shfl_xor(k0, 32), pk1 = __shfl_xor(k1, 32);
  // the rotated values as a stored tensor of the data's format holds them
  float x0 = round_elem<kBf16>(rope_channel(q0, pq0, cs.x, sn.x, upper));
  float x1 = round_elem<kBf16>(rope_channel(q1, pq1, cs.y, sn.y, upper));
  const float kr0 = round_elem<kBf16>(rope_channel(k0, pk0, cs.x, sn.x, upper));
  const float kr1 = round_elem<kBf16>(rope_channel(k1, pk1, cs.y, sn.y, upper));
  reinterpret_cast<uint32_t*>(q_out + static_cast<size_t>(bh) * kHeadDim)[lane] = pack2<kBf16>(x0, x1);

  const bool keep_fp32 = (flags & ADAMAS_F_CODE_FROM_FP32) != 0;
  transform_row<kBf16>(x0, x1, lane, scale, keep_fp32);
  const uint32_t qword = wave_pack_codes(x0, x1, lane);
  if ((lane & 3) == 0)
    q_code_out[static_cast<size_t>(bh) * kCodeWords + (lane >> 2)] = static_cast<uint16_t>(qword);
  if (!has_kv) return;  // whole waves leave: nothing below synchronises

  const int32_t* table = page_indices + page_indptr[b];
  const uint32_t lp = pos / page_size;
  const uint32_t slot = pos - lp * page_size;
  const size_t page = static_cast<size_t>(table[lp]);
  const uint32_t vraw =
      reinterpret_cast<const uint32_t*>(row + static_cast<size_t>(num_q_heads + num_heads + hd) * kHeadDim)[lane];
  const size_t k_off = kv_row_offset(page, 0, slot, hd, page_size, num_heads, flags);
  const size_t v_off = kv_row_offset(page, 1, slot, hd, page_size, num_heads, flags);
  reinterpret_cast<uint32_t*>(kv_data + k_off)[lane] = pack2<kBf16>(kr0, kr1);
  reinterpret_cast<uint32_t*>(kv_data + v_off)[lane] = vraw;
  x0 = kr0;
  x1 = kr1;
  transform_row<kBf16>(x0, x1, lane, scale, keep_fp32);
  const uint32_t kword = wave_pack_codes(x0, x1, lane);
  if ((lane & 3) == 0)
    code_data[((page * page_size + slot) * num_heads + hd) * kCodeWords + (lane >> 2)] =
        static_cast<uint16_t>(kword);
}

// ------------------------------------------------------------------------------------------------
// Prefill append of one sequence.  A row = (token, head) = 256 bytes; a 16-lane group owns a row and a
// lane 8 adjacent channels (one 128-bit load of k, one of v), so a wave moves four adjacent rows =
// 1 KB contiguous per instruction, and the lane's eight codes are exactly one packed word.  The
// butterfly runs strides 1, 2, 4 inside the lane and 8..64 across the 16 lanes with DPP; operand
// pairs and order are those of wave_hadamard128, so both give the same bits.  kPrefillUnroll groups
// of four rows are loaded before the first one is transformed; measured at 32768 tokens x 32 heads:
// 205 us with 1, 218 with 2, 231 with 4, 267 with 8 (occupancy already keeps enough loads in flight).
// ------------------------------------------------------------------------------------------------
constexpr int kPrefillUnroll = 1;
constexpr int kPrefillRowsPerWave = 4 * kPrefillUnroll;

template <bool kBf16>
__global__ __launch_bounds__(256) void append_prefill_kernel(
    const __half* __restrict__ k, const __half* __restrict__ v, const __half* __restrict__ h,
    uint32_t n_rows, uint32_t start_pos, __half* __restrict__ kv_data,
    uint16_t* __restrict__ code_data, const int32_t* __restrict__ table, uint32_t num_heads,
    uint32_t page_size, float scale, uint32_t flags) {
  const uint32_t lane = static_cast<uint32_t>(lane_id());
  const uint32_t c = lane & 15u;   // channels [8c, 8c+8)
  const uint32_t sub = lane >> 4;  // row inside a group of four
  const uint32_t wave_global = blockIdx.x * 4u + static_cast<uint32_t>(wave_id_uniform());
  const uint32_t row0 = wave_global * kPrefillRowsPerWave + sub;

  uint4 kr[kPrefillUnroll], vr[kPrefillUnroll], hr[kPrefillUnroll];
#pragma unroll
  for (int u = 0; u < kPrefillUnroll; ++u) {
    const uint32_t r = row0 + 4u * u;
    if (r < n_rows) {
      const size_t off = static_cast<size_t>(r) * kHeadDim + 8u * c;
      kr[u] = *reinterpret_cast<const uint4*>(k + off);
      vr[u] = *reinterpret_cast<const uint4*>(v + off);
      if (h != nullptr) hr[u] = *reinterpret_cast<const uint4*>(h + off);
    }
  }
#pragma unroll
  for (int u = 0; u < kPrefillUnroll; ++u) {
    const uint32_t r = row0 + 4u * u;
    if (r >= n_rows) continue;  // whole 16-lane rows drop out together: the DPP partners stay in step
    const uint32_t tok = r / num_heads;
    const uint32_t hd = r - tok * num_heads;
    const uint32_t pos = start_pos + tok;
    const uint32_t lp = pos / page_size;
    const uint32_t slot = pos - lp * page_size;
    const size_t page = static_cast<size_t>(table[lp]);

    float x[8];
    if (h != nullptr) {
      unpack_elem8<kBf16>(hr[u], x);
    } else {
      unpack_elem8<kBf16>(kr[u], x);
      row_hadamard128(x, c);
      const bool keep_fp32 = (flags & ADAMAS_F_CODE_FROM_FP32) != 0;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        x[e] = scaled_f32(x[e], scale);
        if (!keep_fp32) x[e] = round_elem<kBf16>(x[e]);
      }
    }
    uint32_t word = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) word |= bucket4(x[e]) << (2 * e);
    code_data[((page * page_size + slot) * num_heads + hd) * kCodeWords + c] =
        static_cast<uint16_t>(word);
    const size_t k_off = kv_row_offset(page, 0, slot, hd, page_size, num_heads, flags) + 8u * c;
    const size_t v_off = kv_row_offset(page, 1, slot, hd, page_size, num_heads, flags) + 8u * c;
    *reinterpret_cast<uint4*>(kv_data + k_off) = kr[u];
    *reinterpret_cast<uint4*>(kv_data + v_off) = vr[u];
  }
}

}  // namespace adamas

using namespace adamas;

extern "C" int adamas_hadamard_f(const void* x, void* out, uint64_t n_rows, float scale,
                                 uint32_t flags, adamas_stream_t stream) {
  if (flags & ~ADAMAS_F_BF16) return ADAMAS_E_BADARG;
  const bool bf16 = (flags & ADAMAS_F_BF16) != 0;
  if (n_rows == 0) return 0;
  if (!x || !out) return ADAMAS_E_BADARG;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15) return ADAMAS_E_ALIGN;
  const uint64_t blocks = (n_rows + 15) / 16;
  if (blocks > 0x7fffffffull) return ADAMAS_E_UNSUPPORTED;
  if (bf16)
    hipLaunchKernelGGL(hadamard_rows_kernel<true>, dim3(static_cast<uint32_t>(blocks)), dim3(256),
                       0, static_cast<hipStream_t>(stream), static_cast<const __half*>(x),
                       static_cast<__half*>(out), n_rows, scale);
  else
    hipLaunchKernelGGL(hadamard_rows_kernel<false>, dim3(static_cast<uint32_t>(blocks)), dim3(256),
                       0, static_cast<hipStream_t>(stream), static_cast<const __half*>(x),
                       static_cast<__half*>(out), n_rows, scale);
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int adamas_hadamard(const void* x, void* out, uint64_t n_rows, float scale,
                               adamas_stream_t stream) {
  return adamas_hadamard_f(x, out, n_rows, scale, 0u, stream);
}

extern "C" int adamas_pack_2bit_f(const void* h, void* o, uint64_t n_rows, uint32_t flags,
                                  adamas_stream_t stream) {
  if (flags & ~ADAMAS_F_BF16) return ADAMAS_E_BADARG;
  const bool bf16 = (flags & ADAMAS_F_BF16) != 0;
  if (n_rows == 0) return 0;
  if (!h || !o) return ADAMAS_E_BADARG;
  if (reinterpret_cast<uintptr_t>(h) & 15) return ADAMAS_E_ALIGN;
  const uint64_t n_words = n_rows * kCodeWords;
  uint64_t blocks = (n_words + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (bf16)
    hipLaunchKernelGGL(pack_2bit_kernel<true>, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const __half*>(h),
                       static_cast<uint16_t*>(o), n_words);
  else
    hipLaunchKernelGGL(pack_2bit_kernel<false>, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const __half*>(h),
                       static_cast<uint16_t*>(o), n_words);
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int adamas_pack_2bit(const void* h, void* o, uint64_t n_rows, adamas_stream_t stream) {
  return adamas_pack_2bit_f(h, o, n_rows, 0u, stream);
}

extern "C" int adamas_append_decode(const void* q, const void* k, const void* v, const void* h,
                                    void* q_code_out, void* kv_data, void* code_data,
                                    const int32_t* page_indices, const int32_t* page_indptr,
                                    const int32_t* seq_lens, uint32_t batch, uint32_t num_heads,
                                    uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size,
                                    float scale, uint32_t flags, adamas_stream_t stream) {
  if (!k || !v || !q_code_out || !kv_data || !code_data || !page_indices || !page_indptr ||
      !seq_lens || batch == 0 || num_heads == 0 || num_kv_heads == 0 || page_size == 0)
    return ADAMAS_E_BADARG;
  if (h == nullptr && q == nullptr) return ADAMAS_E_BADARG;
  if (head_dim != kHeadDim || num_heads % num_kv_heads != 0) return ADAMAS_E_UNSUPPORTED;
  const uint32_t rows = batch * (num_heads + num_kv_heads);
#define ADAMAS_LAUNCH_APPEND(BF)                                                                 \
  hipLaunchKernelGGL(append_decode_kernel<BF>, dim3((rows + 3) / 4), dim3(256), 0,               \
                     static_cast<hipStream_t>(stream), static_cast<const __half*>(q),            \
                     static_cast<const __half*>(k), static_cast<const __half*>(v),               \
                     static_cast<const __half*>(h), static_cast<uint16_t*>(q_code_out),          \
                     static_cast<__half*>(kv_data), static_cast<uint16_t*>(code_data),           \
                     page_indices, page_indptr, seq_lens, batch, num_heads, num_kv_heads,        \
                     page_size, scale, flags)
  if (flags & ADAMAS_F_BF16) ADAMAS_LAUNCH_APPEND(true);
  else ADAMAS_LAUNCH_APPEND(false);
#undef ADAMAS_LAUNCH_APPEND
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int adamas_rope_append_decode(const void* qkv, const float* cos_table,
                                         const float* sin_table, void* q_out, void* q_code_out,
                                         void* kv_data, void* code_data,
                                         const int32_t* page_indices, const int32_t* page_indptr,
                                         const int32_t* seq_lens, uint32_t batch, uint32_t num_heads,
                                         uint32_t num_kv_heads, uint32_t head_dim,
                                         uint32_t page_size, float scale, uint32_t flags,
                                         adamas_stream_t stream) {
  if (!qkv || !cos_table || !sin_table || !q_out || !q_code_out || !kv_data || !code_data ||
      !page_indices || !page_indptr || !seq_lens || batch == 0 || num_heads == 0 ||
      num_kv_heads == 0 || page_size == 0)
    return ADAMAS_E_BADARG;
  if (head_dim != kHeadDim || num_heads % num_kv_heads != 0) return ADAMAS_E_UNSUPPORTED;
  if (flags & ~(ADAMAS_F_BF16 | ADAMAS_F_HND | ADAMAS_F_CODE_FROM_FP32)) return ADAMAS_E_BADARG;
  if ((reinterpret_cast<uintptr_t>(cos_table) | reinterpret_cast<uintptr_t>(sin_table)) & 7)
    return ADAMAS_E_ALIGN;
  const uint32_t rows = batch * num_heads;
#define ADAMAS_LAUNCH_ROPE_APPEND(BF)                                                              \
  hipLaunchKernelGGL(rope_append_decode_kernel<BF>, dim3((rows + 3) / 4), dim3(256), 0,            \
                     static_cast<hipStream_t>(stream), static_cast<const __half*>(qkv), cos_table, \
                     sin_table, static_cast<__half*>(q_out), static_cast<uint16_t*>(q_code_out),   \
                     static_cast<__half*>(kv_data), static_cast<uint16_t*>(code_data),             \
                     page_indices, page_indptr, seq_lens, batch, num_heads, num_kv_heads,          \
                     page_size, scale, flags)
  if (flags & ADAMAS_F_BF16) ADAMAS_LAUNCH_ROPE_APPEND(true);
  else ADAMAS_LAUNCH_ROPE_APPEND(false);
#undef ADAMAS_LAUNCH_ROPE_APPEND
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int adamas_append_prefill(const void* k, const void* v, const void* h,
                                     uint32_t n_tokens, uint32_t start_pos, void* kv_data,
                                     void* code_data, const int32_t* page_table,
                                     uint32_t n_table_entries, uint32_t num_heads,
                                     uint32_t head_dim, uint32_t page_size, float scale,
                                     uint32_t flags, adamas_stream_t stream) {
  if (n_tokens == 0) return 0;
  if (!k || !v || !kv_data || !code_data || !page_table || num_heads == 0 || page_size == 0)
    return ADAMAS_E_BADARG;
  if (head_dim != kHeadDim) return ADAMAS_E_UNSUPPORTED;
  // every token must land inside the page table handed in
  const uint64_t last_page = (static_cast<uint64_t>(start_pos) + n_tokens - 1) / page_size;
  if (last_page >= n_table_entries) return ADAMAS_E_BADARG;
  if ((reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) |
       reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(kv_data)) & 15)
    return ADAMAS_E_ALIGN;
  // rows are indexed with 32 bits inside a launch: long inputs go in slices of whole tokens
  const uint32_t tokens_per_launch = (0x80000000u / num_heads) & ~15u;
  if (tokens_per_launch == 0) return ADAMAS_E_UNSUPPORTED;
  for (uint64_t t0 = 0; t0 < n_tokens; t0 += tokens_per_launch) {
    const uint64_t left = n_tokens - t0;
    const uint32_t nt = left < tokens_per_launch ? static_cast<uint32_t>(left) : tokens_per_launch;
    const uint32_t n_rows = nt * num_heads;
    const size_t in_off = static_cast<size_t>(t0) * num_heads * kHeadDim;
    const uint32_t rows_per_block = 4 * kPrefillRowsPerWave;
    const uint32_t blocks = (n_rows + rows_per_block - 1) / rows_per_block;
#define ADAMAS_LAUNCH_PREFILL(BF)                                                                \
  hipLaunchKernelGGL(append_prefill_kernel<BF>, dim3(blocks), dim3(256), 0,                      \
                     static_cast<hipStream_t>(stream), static_cast<const __half*>(k) + in_off,   \
                     static_cast<const __half*>(v) + in_off,                                     \
                     h ? static_cast<const __half*>(h) + in_off : nullptr, n_rows,               \
                     start_pos + static_cast<uint32_t>(t0), static_cast<__half*>(kv_data),       \
                     static_cast<uint16_t*>(code_data), page_table, num_heads, page_size, scale, \
                     flags)
    if (flags & ADAMAS_F_BF16) ADAMAS_LAUNCH_PREFILL(true);
    else ADAMAS_LAUNCH_PREFILL(false);
#undef ADAMAS_LAUNCH_PREFILL
  }
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  return 0;
}
