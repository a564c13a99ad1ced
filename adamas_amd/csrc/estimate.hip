// Distance estimator (gfx950): integer L1 distance between the 2-bit code of the query and the
// 2-bit code of every cached key, streamed from the paged code cache.
//
// Layout facts the kernel is built on.  The codes of one token are num_kv_heads * 32 bytes, contiguous
// (code page = [page_size][num_kv_heads][16] u16).  For 32 heads that is 1 KiB = 64 lanes x 16 bytes:
// one wave reads one token with a single 128-bit load per lane, lane l owning (head l/2, half l%2),
// so every lane keeps the bit planes of "its" 64 query channels in registers for the whole kernel.
// A wave takes 16 consecutive tokens (16 loads in flight), adds the two halves of a head with one
// DPP lane swap, and stores 8 distances per lane as one 128-bit store into out[head][t..t+8).
// The distance arithmetic on the packed codes is in codes.h.
#include "codes.h"

namespace adamas {

// two integer distances (low/high 16 bits) -> two fp16 values in the same positions
__device__ __forceinline__ uint32_t pair_to_fp16(uint32_t p) {
  __half lo = __ushort2half_rn(static_cast<unsigned short>(p & 0xffffu));
  __half hi = __ushort2half_rn(static_cast<unsigned short>(p >> 16));
  return static_cast<uint32_t>(__half_as_ushort(lo)) |
         (static_cast<uint32_t>(__half_as_ushort(hi)) << 16);
}

constexpr int kTokPerWave = 16;
constexpr int kTokPerBlock = 64;  // 4 waves

// kPage: compile-time page size (16 or 1), 0 = run-time page size.
template <int kPage>
__global__ __launch_bounds__(256) void estimate_kernel(
    const uint16_t* __restrict__ q_code, const unsigned char* __restrict__ code_data,
    const int32_t* __restrict__ page_indices, const int32_t* __restrict__ page_indptr,
    const int32_t* __restrict__ seq_lens, uint16_t* __restrict__ out, int64_t out_bs,
    int64_t out_hs, uint32_t out_format, uint32_t num_heads, uint32_t num_kv_heads,
    uint32_t kv_inv16, uint32_t page_size_rt, uint32_t vec_ok) {
  const uint32_t page_size = kPage ? static_cast<uint32_t>(kPage) : page_size_rt;
  const uint32_t b = blockIdx.y;
  const uint32_t seg = blockIdx.z;  // group of 32 heads
  const int lane = lane_id();
  const int32_t n = seq_lens[b] - 1;  // past tokens to score
  const uint32_t t0 = (blockIdx.x * 4u + static_cast<uint32_t>(wave_id_uniform())) * kTokPerWave;
  if (n <= 0 || t0 >= static_cast<uint32_t>(n)) return;

  // (a head count that is no multiple of 32 leaves lanes of the last group without a head: they
  // compute the last head's distances again and store nothing)
  const uint32_t head_lane = seg * 32u + (static_cast<uint32_t>(lane) >> 1);
  const bool head_ok = head_lane < num_heads;
  const uint32_t head = head_ok ? head_lane : num_heads - 1u;
  const uint32_t half = static_cast<uint32_t>(lane) & 1u;
  const uint4 qraw = *reinterpret_cast<const uint4*>(
      q_code + (static_cast<size_t>(b) * num_heads + head) * kCodeWords + half * 8u);
  const QueryPlanes qp = make_query_planes(qraw);

  const int32_t* table = page_indices + page_indptr[b];
  // grouped-query attention: query head h reads the codes of key head h / (num_heads / num_kv_heads);
  // lanes of one group then load the same bytes (merged by the memory pipeline)
  // (from the reciprocal of the group size; 32-bit strides: one multiply-add per load address)
  const uint32_t kv_head = kv_head_of(head, kv_inv16);
  const uint32_t row_bytes = num_kv_heads * 32u;
  const unsigned char* lane_base = code_data + kv_head * 32u + half * 16u;

  uint4 kw[kTokPerWave];
  const uint32_t last = static_cast<uint32_t>(n) - 1u;
  if (kPage == 16) {
    // t0 is a multiple of 16: all 16 tokens sit in one page
    const uint32_t slot0 = static_cast<uint32_t>(table[t0 >> 4]) * 16u;
#pragma unroll
    for (int j = 0; j < kTokPerWave; ++j) {
      uint32_t s = min(t0 + j, last) - t0;
      kw[j] = *reinterpret_cast<const uint4*>(lane_base + static_cast<size_t>(slot0 + s) * row_bytes);
    }
  } else {
#pragma unroll
    for (int j = 0; j < kTokPerWave; ++j) {
      uint32_t t = min(t0 + j, last);
      const uint32_t slot = token_slot<uint32_t>(table, t, page_size);
      kw[j] = *reinterpret_cast<const uint4*>(lane_base + static_cast<size_t>(slot) * row_bytes);
    }
  }

  // pair (2i, 2i+1) packed in one register, halves of the head added with one lane swap
  uint32_t p[kTokPerWave / 2];
#pragma unroll
  for (int i = 0; i < kTokPerWave / 2; ++i) {
    uint32_t v = l1_64(kw[2 * i], qp) | (l1_64(kw[2 * i + 1], qp) << 16);
    p[i] = v + swap_adjacent(v);
  }

  // even lane stores tokens t0..t0+7, odd lane t0+8..t0+15
  uint32_t w0 = half ? p[4] : p[0];
  uint32_t w1 = half ? p[5] : p[1];
  uint32_t w2 = half ? p[6] : p[2];
  uint32_t w3 = half ? p[7] : p[3];
  if (out_format == ADAMAS_DIST_FP16) {
    w0 = pair_to_fp16(w0);
    w1 = pair_to_fp16(w1);
    w2 = pair_to_fp16(w2);
    w3 = pair_to_fp16(w3);
  }
  const uint32_t ts = t0 + half * 8u;
  uint16_t* dst = out + static_cast<int64_t>(b) * out_bs + static_cast<int64_t>(head) * out_hs + ts;
  if (!head_ok) return;
  if (vec_ok && ts + 8u <= static_cast<uint32_t>(n)) {
    *reinterpret_cast<uint4*>(dst) = make_uint4(w0, w1, w2, w3);
  } else {
    const uint32_t w[4] = {w0, w1, w2, w3};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (ts + i < static_cast<uint32_t>(n))
        dst[i] = static_cast<uint16_t>((w[i >> 1] >> (16 * (i & 1))) & 0xffffu);
    }
  }
}

// Measurement aid: reads `n_vec` 128-bit words and does nothing else (the words are folded into one
// value that is only stored if it matches a pattern no data holds).  256 workgroups x 512 threads,
// 16 independent loads in flight per lane, a wave reads 1 KB contiguous per instruction: what the
// memory system gives a kernel that streams a code cache once, without any of the estimator's work.
__global__ __launch_bounds__(512) void read_probe_kernel(const uint4* __restrict__ p, uint64_t n_vec,
                                                         uint32_t* __restrict__ sink) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 512u;
  uint32_t acc = 0;
  for (uint64_t i0 = static_cast<uint64_t>(blockIdx.x) * 512u + threadIdx.x; i0 < n_vec;
       i0 += 16 * stride) {
    uint4 v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const uint64_t i = i0 + j * stride;
      v[j] = i < n_vec ? p[i] : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) acc ^= v[j].x + v[j].y + v[j].z + v[j].w;
  }
  if (acc == 0x9e3779b9u && sink) *sink = acc;
}

}  // namespace adamas

using namespace adamas;

extern "C" int adamas_read_probe(const void* data, size_t bytes, void* sink,
                                 adamas_stream_t stream) {
  if (!data || bytes == 0) return ADAMAS_E_BADARG;
  if ((reinterpret_cast<uintptr_t>(data) & 15) || (bytes & 15)) return ADAMAS_E_ALIGN;
  hipLaunchKernelGGL(read_probe_kernel, dim3(256), dim3(512), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(data), static_cast<uint64_t>(bytes / 16),
                     static_cast<uint32_t*>(sink));
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int adamas_estimate(const void* q_code, const void* code_data,
                               const int32_t* page_indices, const int32_t* page_indptr,
                               const int32_t* seq_lens, void* out, int64_t out_batch_stride,
                               int64_t out_head_stride, uint32_t out_format, uint32_t batch,
                               uint32_t num_heads, uint32_t num_kv_heads, uint32_t page_size,
                               uint32_t max_seq_len, adamas_stream_t stream) {
  if (!q_code || !code_data || !page_indices || !page_indptr || !seq_lens || !out || batch == 0 ||
      page_size == 0)
    return ADAMAS_E_BADARG;
  if (num_heads == 0) return ADAMAS_E_UNSUPPORTED;
  if (num_kv_heads == 0 || num_heads % num_kv_heads != 0) return ADAMAS_E_UNSUPPORTED;
  // the kernel takes head / group from a 16-bit reciprocal (kv_head_of)
  if (static_cast<uint64_t>(num_heads) * (num_heads / num_kv_heads) >= 65536u) return ADAMAS_E_UNSUPPORTED;
  if (out_format != ADAMAS_DIST_FP16 && out_format != ADAMAS_DIST_U16) return ADAMAS_E_BADARG;
  if ((reinterpret_cast<uintptr_t>(q_code) | reinterpret_cast<uintptr_t>(code_data)) & 15)
    return ADAMAS_E_ALIGN;
  if (reinterpret_cast<uintptr_t>(out) & 1) return ADAMAS_E_ALIGN;
  if (max_seq_len <= 1) return 0;  // nothing to score
  if (batch > 65535) return ADAMAS_E_UNSUPPORTED;
  const uint32_t n_max = max_seq_len - 1;
  const uint32_t vec_ok = ((reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
                           out_head_stride % 8 == 0 && out_batch_stride % 8 == 0)
                              ? 1u
                              : 0u;
  dim3 grid((n_max + kTokPerBlock - 1) / kTokPerBlock, batch, (num_heads + 31) / 32);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define ADAMAS_LAUNCH_ESTIMATE(PG)                                                              \
  hipLaunchKernelGGL(estimate_kernel<PG>, grid, dim3(256), 0, s,                                \
                     static_cast<const uint16_t*>(q_code),                                     \
                     static_cast<const unsigned char*>(code_data), page_indices, page_indptr,  \
                     seq_lens, static_cast<uint16_t*>(out), out_batch_stride, out_head_stride, \
                     out_format, num_heads, num_kv_heads,                                       \
                     group_inv16(num_heads / num_kv_heads), page_size, vec_ok)
  if (page_size == 16) {
    ADAMAS_LAUNCH_ESTIMATE(16);
  } else if (page_size == 1) {
    ADAMAS_LAUNCH_ESTIMATE(1);
  } else {
    ADAMAS_LAUNCH_ESTIMATE(0);
  }
#undef ADAMAS_LAUNCH_ESTIMATE
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  return 0;
}
