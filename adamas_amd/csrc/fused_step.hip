// The whole sparse decode step in two launches (gfx950):
//
//   estimate_select_kernel  grid (token chunks, head groups of 8 or 4, batch), one wave per head.
//       A sequence is cut into chunks whose lengths differ by at most 16 tokens (StepPlan in
//       workspace.h: 64 chunks x 4 head groups = one workgroup per CU for a single sequence of 32
//       heads), so the cost of the launch grows smoothly with the sequence.  Per pass of 512 tokens
//       the workgroup streams the 2-bit codes of 512 tokens x 8 heads (256 contiguous bytes per
//       token, one 128-bit load per lane, 16 loads in flight per wave; the loads of the next pass are
//       issued before the distances of the current one are computed; 16-token units go to the waves
//       round robin, and in the last pass a wave skips the units its chunk does not have), computes
//       the integer L1 distances to the query code and keeps them in LDS only.  Then one wave per
//       head selects the kc nearest tokens of the chunk, exactly, ties to the lowest index, and
//       writes them as candidates (distance, token offset, K row index).  kc is the budget where the
//       lists of all chunks fit 1024 slots per head and 16 otherwise.  The distance matrix never
//       reaches HBM.
//   select_attend_kernel    grid (heads, batch), 512 threads.
//       Two candidate slots per thread.  A 512-bin histogram of the candidates' distances in LDS
//       gives the threshold and the tie quota without any search; lists keep the (below threshold,
//       tied) x ascending-index order and chunks are concatenated in index order, so "ties to the
//       lowest index" carries over: ranks come from DPP prefix scans, no atomic decides a position.
//       A list of kc entries is a prefix of its chunk in (distance, index) order: if its last entry
//       is not selected, nothing the chunk left out can be.  If it is (a chunk that holds more than
//       kc of the selection: clustered neighbours, or long runs of equal distances), the workgroup
//       scores that chunk again from its codes and selects among all of its tokens: the result is
//       exact for any input.  The attention then runs over the selected rows plus the current
//       token: groups of 16 lanes, fp32 online softmax.  Candidates carry their K row index, so no
//       page-table access sits between the selection and the K/V gather.
#include "attend.h"
#include "codes.h"
#include "hadamard.h"
#include <atomic>

#include "chunk_select.h"
#include "split_merge.h"
#include "workspace.h"

namespace adamas {

// The estimator's workgroup covers a chunk of tokens for kHeads heads with kHeads waves: 8 heads =
// 512 threads reading 256 contiguous bytes per token, or 4 heads = 256 threads reading 128.  One wave
// per head in the selection phase.
constexpr int kFusedHeads = 8;                      // the wide workgroup
constexpr int kAttThreads = 512;
constexpr int kAttWaves = kAttThreads / kWave;      // 8

// A wave stores the distances of eight heads in one instruction; with rows a multiple of 128 bytes
// apart those stores would all fall into the same LDS banks, so every row is padded by 16 bytes
// (eight rows x four words then cover the 32 banks once).
constexpr uint32_t kDistRowPad = 8;  // u16 elements

template <int kPasses, int kHeads>
struct EstimateSelectShared {
  alignas(16) uint16_t dist[kHeads][kFusedBlock * kPasses + kDistRowPad];  // 0xFFFF = no token
  uint32_t krow[kFusedBlock * kPasses];       // K row index (page * rows per page + slot) of every token
  // tokens per distance value of one head: one word per value, read off for the chunk's threshold
  // (selection), or two 16-bit bins per word in the first 256 words, written out as they are
  // (histogram mode); rows are read with 128-bit accesses
  alignas(16) uint32_t hist[kHeads][kChunkHistWords];
  alignas(16) uint16_t qcode[kHeads][kCodeWords];  // query codes made in the kernel (kFromQkv)
};

// Where the query comes from when a kernel of the step takes the fused q/k/v projection of the
// decoder instead of a rotated query and its code: qkv [batch][Hq + 2*Hkv][128] fp16 or bf16
// (ADAMAS_F_BF16 in code_flags), rotary tables [positions][64] fp32 (rotate-half pairing), and the
// parameters of the code generation.
struct QkvSource {
  const __half* qkv = nullptr;
  const float* cos_table = nullptr;
  const float* sin_table = nullptr;
  float scale = 1.0f;
  uint32_t code_flags = 0;
};

// The chunks of the step (StepPlan): chunk c starts at 16-token unit c*units_q + min(c, units_r) and
// has units_q + (c < units_r) units; kc candidate slots per (head, chunk).
struct StepGeom {
  uint32_t units_q, units_r;
  uint32_t kc, kc_log2;
};

__device__ __forceinline__ uint32_t chunk_first_unit(const StepGeom& g, uint32_t c) {
  return c * g.units_q + min(c, g.units_r);
}
__device__ __forceinline__ uint32_t chunk_units(const StepGeom& g, uint32_t c) {
  return g.units_q + (c < g.units_r ? 1u : 0u);
}

// Rotary embedding of a row of 128 fp16 held by a wave (lane l = channels 2l and 2l+1) at position
// pos, in two parts so that a kernel can put other loads between the loads and their first use.
struct WaveRopeLoads {
  uint32_t raw;    // the two channels of the lane
  float2 cs, sn;   // their rotary factors
};

__device__ __forceinline__ WaveRopeLoads wave_rope_load(const __half* row, const QkvSource& src,
                                                        uint32_t pos, int lane) {
  WaveRopeLoads r;
  r.raw = reinterpret_cast<const uint32_t*>(row)[lane];
  const uint32_t c0 = (2u * static_cast<uint32_t>(lane)) & 63u;  // table column of channel 2l
  r.cs = *reinterpret_cast<const float2*>(src.cos_table + static_cast<size_t>(pos) * 64 + c0);
  r.sn = *reinterpret_cast<const float2*>(src.sin_table + static_cast<size_t>(pos) * 64 + c0);
  return r;
}

// x0, x1: the rotated channels rounded to the 16-bit format, as a stored tensor would hold them
template <bool kBf16>
__device__ __forceinline__ void wave_rope_apply(const WaveRopeLoads& r, int lane, float& x0,
                                                float& x1) {
  float q0, q1;
  unpack2<kBf16>(r.raw, q0, q1);
  const bool upper = lane >= 32;  // channels 64 .. 127 pair with the lane 32 below
  const float p0 = __shfl_xor(q0, 32), p1 = __shfl_xor(q1, 32);
  x0 = round_elem<kBf16>(rope_channel(q0, p0, r.cs.x, r.sn.x, upper));
  x1 = round_elem<kBf16>(rope_channel(q1, p1, r.cs.y, r.sn.y, upper));
}

// The query code of a row of the fused projection (rotary embedding, transform, buckets) with the
// format known at run time only (uniform over the launch): the estimator is not instantiated twice
// for something a wave does once.
__device__ __forceinline__ uint32_t wave_query_code(const WaveRopeLoads& r, int lane, float scale,
                                                    uint32_t code_flags) {
  float x0, x1;
  const bool keep = (code_flags & ADAMAS_F_CODE_FROM_FP32) != 0;
  if (code_flags & ADAMAS_F_BF16) {
    wave_rope_apply<true>(r, lane, x0, x1);
    transform_row<true>(x0, x1, lane, scale, keep);
  } else {
    wave_rope_apply<false>(r, lane, x0, x1);
    transform_row<false>(x0, x1, lane, scale, keep);
  }
  return wave_pack_codes(x0, x1, lane);
}

// kPartial: chunks may be shorter than kPasses * 512 tokens by whole 16-token units (balanced chunks
// of a sequence whose length is no multiple of the chunk count): the units of the last pass are
// tested one by one (uniform over the wave).  Without it every chunk has exactly kPasses * 512 tokens
// and only the end of the sequence is masked.
// kHist (budgets beyond the candidate lists, chunks of 512 tokens): instead of selecting, every wave
// writes the distances of its head (dist_out [sequence*heads][dist_stride] u16) and a 512-bin
// histogram of them (16-bit counts, hist_out [sequence*heads][chunks][512]); threshold and positions
// are then read off the histograms by hist_select_attend_kernel below.  The first head group also
// writes the K row index of every token (rowmap_out [sequence][dist_stride]), so that the attention
// of that kernel reads no page table.
// kFromQkv: q_code is not read; wave w makes the code of query head w of the group from the fused
// projection (rotary embedding, Hadamard transform, buckets) while the code loads are in flight.
// qcode_out (selection mode) [sequence*heads][16]: the query codes this launch worked with, written by
// the workgroups of chunk 0 for the second launch, which scores truncated chunks again.
template <int kPage, int kPasses, bool kPartial, bool kHist = false, int kHeads = kFusedHeads,
          bool kFromQkv = false>
__global__ __launch_bounds__(kHeads * kWave) void estimate_select_kernel(
    const uint16_t* __restrict__ q_code, const unsigned char* __restrict__ code_data,
    const int32_t* __restrict__ page_indices, const int32_t* __restrict__ page_indptr,
    const int32_t* __restrict__ seq_lens, uint64_t* __restrict__ cand, StepGeom geom,
    uint16_t* __restrict__ qcode_out, uint32_t num_heads, uint32_t num_kv_heads, uint32_t kv_inv16,
    uint32_t page_size_rt, uint32_t table_stride, uint32_t rows_per_page,
    unsigned char* __restrict__ hist_out = nullptr, uint32_t hist_stride = 0,
    uint16_t* __restrict__ dist_out = nullptr, int64_t dist_stride = 0,
    uint32_t* __restrict__ rowmap_out = nullptr, QkvSource src = QkvSource()) {
  static_assert(!kHist || (kPasses == 1 && !kPartial), "the histogram mode works on 512-token chunks");
  constexpr int kItems = 8 * kPasses;                 // tokens per lane in the selection phase
  static_assert(kHeads == 8 || kHeads == 4, "a token's codes are read by 2 * kHeads lanes");
  constexpr uint32_t kLoadTokens = 32 / kHeads;       // tokens per load instruction: 4 or 8
  constexpr uint32_t kUnitLoads = kStepUnit / kLoadTokens;  // loads per 16-token unit: 4 or 2
  constexpr uint32_t kWaveUnits = 16 / kUnitLoads;    // units per wave and pass: 4 or 8
  constexpr uint32_t kPassUnits = kFusedBlock / kStepUnit;  // 32
  static_assert(kWaveUnits * kHeads == kPassUnits, "the waves of a workgroup cover a pass");
  __shared__ EstimateSelectShared<kPasses, kHeads> sh;
  const uint32_t page_size = kPage ? static_cast<uint32_t>(kPage) : page_size_rt;
  const uint32_t chunk = blockIdx.x, n_chunks = gridDim.x;
  const uint32_t hg = blockIdx.y;
  const uint32_t b = blockIdx.z;
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t unit0 = chunk_first_unit(geom, chunk);
  const uint32_t n_units = kPartial ? chunk_units(geom, chunk) : kPassUnits * kPasses;
  const uint32_t chunk_base = unit0 * kStepUnit;
  uint64_t* dst =
      cand + ((static_cast<size_t>(b) * num_heads + hg * kHeads + wave) * n_chunks + chunk) *
                 geom.kc;

  constexpr uint32_t kTokLanes = 2 * kHeads;                        // lanes per token
  const uint32_t sub = static_cast<uint32_t>(lane) / kTokLanes;    // token within a load
  const uint32_t hl = (static_cast<uint32_t>(lane) % kTokLanes) >> 1;  // head within the group
  const uint32_t half = static_cast<uint32_t>(lane) & 1u;        // which 64 channels

  // Unit u (of kWaveUnits) of this wave in pass `pass`, counted from the start of the chunk: the
  // units of a pass go to the waves round robin, so that a short last pass is spread over all waves.
  auto unit_of = [&](int pass, uint32_t u) __attribute__((always_inline)) -> uint32_t {
    return static_cast<uint32_t>(pass) * kPassUnits + u * kHeads + static_cast<uint32_t>(wave);
  };
  // whether the chunk has that unit (always true except in the last pass of a kPartial launch)
  auto has_unit = [&](int pass, uint32_t u) __attribute__((always_inline)) -> bool {
    return !kPartial || pass + 1 < kPasses || unit_of(pass, u) < n_units;
  };

  // Memory round trips before the first code load: with a fixed table stride the sequence length and
  // the page ids are fetched side by side (two dependent levels: table, codes); with an indptr array
  // the table address itself has to be loaded first (three levels).
  // page ids per pass: one per unit (kPage == 16: a unit is a page, uniform over the wave) or one per load
  constexpr int kPageRegs = kPage == 16 ? static_cast<int>(kWaveUnits) : 16;
  uint32_t pages[kPasses][kPageRegs];
  const int32_t* table;
  uint32_t lp_max;
  auto lookup_all = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int pass = 0; pass < kPasses; ++pass) {
#pragma unroll
      for (int j = 0; j < kPageRegs; ++j) {
        uint32_t lp;
        if (kPage == 16) {
          lp = unit0 + unit_of(pass, j);
        } else {
          const uint32_t u = static_cast<uint32_t>(j) / kUnitLoads, i = static_cast<uint32_t>(j) % kUnitLoads;
          lp = (chunk_base + unit_of(pass, u) * kStepUnit + i * kLoadTokens + sub) / page_size;
        }
        pages[pass][j] = static_cast<uint32_t>(table[min(lp, lp_max)]);
      }
    }
  };
  const int32_t seq_len = seq_lens[b];
  if (table_stride) {
    table = page_indices + static_cast<size_t>(b) * table_stride;
    lp_max = table_stride - 1u;
    lookup_all();
  }
  const uint32_t n = seq_len > 1 ? static_cast<uint32_t>(seq_len) - 1u : 0u;  // past tokens
  // histogram mode: the 1 KB row of 16-bit counts of this (head, chunk), 16 bytes per lane
  uint4* hrow16 = reinterpret_cast<uint4*>(
                      hist_out + ((static_cast<size_t>(b) * num_heads + hg * kHeads + wave) *
                                      hist_stride + chunk) * (2 * kHistBins)) + lane;
  if (chunk_base >= n) {  // no token of this sequence in the chunk: an empty candidate list
    if (kHist) {
      *hrow16 = make_uint4(0u, 0u, 0u, 0u);
      return;
    }
    for (uint32_t i = lane; i < geom.kc; i += kWave) dst[i] = kEmptyCand64;
    return;
  }
  if (!table_stride) {
    table = page_indices + page_indptr[b];
    lp_max = (n - 1u) / page_size;
    lookup_all();
  }

  // ---- distances: per pass, 16 loads per lane = 64 (or 128) tokens x kHeads heads per wave --------
  {
    const uint32_t head = hg * kHeads + hl;
    QueryPlanes qp;
    uint4 qraw_copy = make_uint4(0u, 0u, 0u, 0u);
    WaveRopeLoads qload;  // kFromQkv: the query row of head hg*kHeads + wave and its rotary factors
    if (kFromQkv) {
      // issued ahead of the code loads, used after them: the wait for these leaves the code loads in flight
      const size_t row_len = static_cast<size_t>(num_heads + 2 * num_kv_heads) * kHeadDim;
      qload = wave_rope_load(src.qkv + static_cast<size_t>(b) * row_len +
                                 static_cast<size_t>(hg * kHeads + wave) * kHeadDim,
                             src, static_cast<uint32_t>(seq_len) - 1u, lane);
    } else {
      const uint4 qraw = *reinterpret_cast<const uint4*>(
          q_code + (static_cast<size_t>(b) * num_heads + head) * kCodeWords + half * 8u);
      qp = make_query_planes(qraw);
      qraw_copy = qraw;
    }

    // grouped-query attention: query head h scores the codes of key head h / group; the lanes of a
    // group load the same bytes, and the workgroups of a group read the same rows through L2
    // (32-bit operands: the byte offset of a token is then one 32 x 32 -> 64 bit multiply-add per
    // load, and the key/value head comes from the reciprocal of the group size, not a division)
    const uint32_t row_bytes = num_kv_heads * 32u;
    const unsigned char* lane_base = code_data + kv_head_of(head, kv_inv16) * 32u + half * 16u;

    // issues the 16 loads of pass `pass`; tokens past the end of the sequence read some valid slot and
    // are masked when the distances are stored
    auto issue = [&](int pass, uint4 (&kw)[16]) __attribute__((always_inline)) {
#pragma unroll
      for (uint32_t u = 0; u < kWaveUnits; ++u) {
        if (!has_unit(pass, u)) continue;
        const uint32_t tok_u = unit_of(pass, u) * kStepUnit;  // first token of the unit, in the chunk
#pragma unroll
        for (uint32_t i = 0; i < kUnitLoads; ++i) {
          const int j = static_cast<int>(u * kUnitLoads + i);
          uint32_t page, in_page;
          if (kPage == 16) {
            page = pages[pass][u];
            in_page = i * kLoadTokens + sub;
          } else {
            page = pages[pass][j];
            in_page = (chunk_base + tok_u + i * kLoadTokens + sub) % page_size;
          }
          kw[j] = *reinterpret_cast<const uint4*>(
              lane_base + static_cast<size_t>(page * page_size + in_page) * row_bytes);
          // (written between the loads on purpose: with the 16 loads of a wave back to back the
          // launch is 0.1 us slower from HBM, although 0.2 us faster from the Infinity Cache)
          if ((static_cast<uint32_t>(lane) % kTokLanes) == 0)
            sh.krow[tok_u + i * kLoadTokens + sub] = page * rows_per_page + in_page;
        }
      }
    };
    auto consume = [&](int pass, const uint4 (&kw)[16]) __attribute__((always_inline)) {
#pragma unroll
      for (uint32_t u = 0; u < kWaveUnits; ++u) {
        const uint32_t tok_u = unit_of(pass, u) * kStepUnit;
        if (!has_unit(pass, u)) {  // a unit the chunk does not have: no tokens
#pragma unroll
          for (uint32_t i2 = 0; i2 < kUnitLoads / 2; ++i2)
            sh.dist[hl][tok_u + (2 * i2 + half) * kLoadTokens + sub] = 0xffffu;
          continue;
        }
#pragma unroll
        for (uint32_t i2 = 0; i2 < kUnitLoads / 2; ++i2) {
          const int j = static_cast<int>(u * kUnitLoads + 2 * i2);
          uint32_t v = l1_64(kw[j], qp) | (l1_64(kw[j + 1], qp) << 16);
          v += swap_adjacent(v);  // both lanes of a head now hold the distances of loads j, j+1
          // the even lane keeps load j, the odd lane load j+1
          const uint32_t tok = tok_u + (2 * i2 + half) * kLoadTokens + sub;
          const uint32_t d = half ? (v >> 16) : (v & 0xffffu);
          sh.dist[hl][tok] = (chunk_base + tok < n) ? static_cast<uint16_t>(d) : 0xffffu;
        }
      }
    };
    uint4 buf0[16], buf1[16];
    issue(0, buf0);
    // the query codes for the second launch (behind the code loads: the store waits for the query
    // code, which must not hold the code loads back)
    if (!kFromQkv && !kHist && chunk == 0 && sub == 0)
      *reinterpret_cast<uint4*>(qcode_out + (static_cast<size_t>(b) * num_heads + head) * kCodeWords +
                                half * 8u) = qraw_copy;
    if (kFromQkv) {
      const uint32_t word = wave_query_code(qload, lane, src.scale, src.code_flags);
      if ((lane & 3) == 0) {
        sh.qcode[wave][lane >> 2] = static_cast<uint16_t>(word);
        if (chunk == 0)
          qcode_out[(static_cast<size_t>(b) * num_heads + hg * kHeads + wave) * kCodeWords +
                    (lane >> 2)] = static_cast<uint16_t>(word);
      }
      // a barrier that waits for the LDS writes only: __syncthreads() would also wait for the 16
      // code loads of every wave before any of them is used
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      qp = make_query_planes(*reinterpret_cast<const uint4*>(&sh.qcode[hl][half * 8u]));
    }
#pragma unroll
    for (int pass = 0; pass < kPasses; ++pass) {
      if (pass + 1 < kPasses) {
        if (pass & 1) issue(pass + 1, buf0);
        else issue(pass + 1, buf1);
      }
      if (pass & 1) consume(pass, buf1);
      else consume(pass, buf0);
    }
  }
  __syncthreads();

  if (kHist) {
    // ---- wave w = head w of the group: its 512 distances go out (1 KB contiguous) and are counted
    const uint32_t tok0 = static_cast<uint32_t>(lane) * 8u;
    const uint4 v = *reinterpret_cast<const uint4*>(&sh.dist[wave][tok0]);
    uint32_t* hw = sh.hist[wave];
    *reinterpret_cast<uint4*>(&hw[4 * lane]) = make_uint4(0u, 0u, 0u, 0u);
    uint16_t* drow = dist_out +
                     (static_cast<size_t>(b) * num_heads + hg * kHeads + wave) * dist_stride +
                     chunk_base + tok0;
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    if (chunk_base + tok0 + 8u <= n) {
      *reinterpret_cast<uint4*>(drow) = v;  // rows and chunks are 16-byte aligned
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (chunk_base + tok0 + i < n)
          drow[i] = static_cast<uint16_t>((w[i >> 1] >> (16 * (i & 1))) & 0xffffu);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {  // tokens past the end carry 0xffff; a bin holds at most 512
      const uint32_t d = (w[i >> 1] >> (16 * (i & 1))) & 0xffffu;
      if (d != 0xffffu) atomicAdd(&hw[d >> 1], 1u << (16 * (d & 1u)));
    }
    // the LDS operations of one wave are carried out in order: the counts are complete here
    *hrow16 = *reinterpret_cast<const uint4*>(&hw[4 * lane]);
    if (hg == 0 && rowmap_out) {
      for (uint32_t tok = static_cast<uint32_t>(wave) * 64u + static_cast<uint32_t>(lane);
           tok < kFusedBlock; tok += kHeads * 64u)
        if (chunk_base + tok < n)
          rowmap_out[static_cast<size_t>(b) * dist_stride + chunk_base + tok] = sh.krow[tok];
    }
    return;
  }

  // ---- wave w = head w of the group: the kc nearest tokens of the chunk ---------------------------
  // lane l holds tokens kItems*l .. kItems*l + kItems-1 (item order = token order)
  uint32_t keys[kItems];
#pragma unroll
  for (int p8 = 0; p8 < kPasses; ++p8) {
    const uint4 v = *reinterpret_cast<const uint4*>(&sh.dist[wave][lane * kItems + p8 * 8]);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // 0xffff (no token) stays as it is: above every threshold
      keys[p8 * 8 + 2 * i] = w[i] & 0xffffu;
      keys[p8 * 8 + 2 * i + 1] = w[i] >> 16;
    }
  }
  // the K row of a listed token is read when it is written out (a handful per wave)
  chunk_select_capped<kItems, kPartial>(
      keys, geom.kc, dst, sh.hist[wave],
      [&](uint32_t tok) __attribute__((always_inline)) -> uint32_t { return sh.dist[wave][tok]; },
      [&](uint32_t tok) __attribute__((always_inline)) -> uint32_t { return sh.krow[tok]; });
}

// Up to 128 rows (one round of loads) the attention of launch 2 runs on the first four waves only (16
// groups of 16 lanes, 8 rows in flight per group instead of 32 groups with 4 each).  The other four
// waves leave once the row list is closed: the kernel is bound by instruction issue, and the folding
// and merging of the group states is paid per wave, so half the waves with twice the rows each cost
// less (budget 128: 0.05 - 0.2 us).  With more rows all eight waves are faster (budget 256: 0.35 us),
// again with eight rows per group.
constexpr int kAttendWaves = 4;
constexpr int kAttendGroups = 4 * kAttendWaves;

struct SelectAttendShared {
  MergeShared<32> merge;
  MergeShared<kAttendGroups> merge_few;
  int32_t rows[kFusedMaxSel + 1];     // K row index of every selected token, then the current one
  int32_t sel_pos[kFusedMaxSel + 1];  // position of every selected token
  alignas(16) uint32_t hist[kHistBins];  // candidates per distance value
  alignas(16) uint32_t wclass[kAttWaves];  // per-wave class totals of the rank scan: below | tied << 16
  // chunks whose list is exhausted by the selection and that hold more tokens (scored again):
  uint32_t flag[kStepMaxChunks];
  uint32_t any_flag;
  uint32_t fb[kStepMaxChunks], ft[kStepMaxChunks];  // their tokens below / equal to the threshold
  uint32_t tbase[kStepMaxChunks];                   // tied list entries of all chunks before them
  // kFromQkv: the rotated query (scaled for the softmax), the rotated new key and the new value
  alignas(16) float qkv_now[3][kHeadDim];
};

// kSlots (2 or 4) candidate slots per thread: slots kSlots*tid .. of the head's n_chunks * kc slots
// (at most kSlots * 512; they belong to one chunk since kc is a multiple of 8).
// q_code [sequence*heads][16], code_data: the query codes and the code cache the first launch worked
// with, read only when a chunk has to be scored again; dist_scratch [sequence*heads][dist_stride]
// u16 then holds that chunk's distances (rows are private to a workgroup).
// kFromQkv: q is not read; the kernel takes the fused projection of the decoder, applies the rotary
// embedding to the query and to the new key itself, appends the new key, its code and the new value
// (the workgroup of the first query head of a key/value head), and attends the current token from
// registers instead of reading it back: the decode append needs no launch of its own.
template <int kSlots, bool kBf16, bool kHnd, bool kFromQkv = false>
__global__ __launch_bounds__(kAttThreads) void select_attend_kernel(
    const __half* __restrict__ q, const __half* __restrict__ kv_data,
    const int32_t* __restrict__ page_indices, const int32_t* __restrict__ page_indptr,
    const int32_t* __restrict__ seq_lens, const uint64_t* __restrict__ cand, StepGeom geom,
    uint32_t n_chunks, uint32_t k, __half* __restrict__ out, int32_t* __restrict__ sel_out,
    uint32_t num_heads, uint32_t num_kv_heads, uint32_t kv_group, uint32_t kv_inv16,
    uint32_t page_size, float scale_log2, uint32_t table_stride,
    const uint16_t* __restrict__ q_code, const unsigned char* code_data,
    uint16_t* __restrict__ dist_scratch, int64_t dist_stride, QkvSource src = QkvSource(),
    __half* kv_append = nullptr, uint16_t* code_append = nullptr) {
  static_assert(kAttThreads == kHistBins, "one thread per distance value");
  static_assert(kSlots == 2 || kSlots == 4, "one or two 128-bit loads of candidates per thread");
  static_assert(kStepMaxSlots == 4 * kAttThreads, "at most four candidate slots per thread");
  static_assert(kStepMaxChunks == kWave, "the flags of all chunks fit one ballot");
  __shared__ SelectAttendShared sh;
  const uint32_t head = blockIdx.x;
  const uint32_t b = blockIdx.y;
  const uint32_t bh = b * num_heads + head;
  const uint32_t tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t n_slots = n_chunks << geom.kc_log2;
  const uint64_t* crow = cand + static_cast<size_t>(bh) * n_slots;

  // ---- the candidates of this head: two slots per thread --------------------------------------------
  // (asked for ahead of everything that waits for the sequence length: the list of a sequence
  // without tokens is valid memory, if meaningless)
  const uint32_t slot0 = static_cast<uint32_t>(kSlots) * tid;
  const bool have = slot0 < n_slots;
  uint4 raw[kSlots / 2];
#pragma unroll
  for (int j = 0; j < kSlots / 2; ++j) {
    raw[j] = make_uint4(~0u, ~0u, ~0u, ~0u);  // an unused slot is all ones
    if (have) raw[j] = *reinterpret_cast<const uint4*>(crow + slot0 + 2 * j);  // lists are 64-byte aligned
  }

  // K row of the current token: a chain of three dependent scalar loads, started early so that it
  // has long finished when the row list is closed
  const int32_t seq_len = seq_lens[b];
  if (seq_len <= 0) {  // a sequence without tokens: zeros and an empty selection (whole workgroup leaves)
    if (tid < kHeadDim) store_elem<kBf16>(out + static_cast<size_t>(bh) * kHeadDim + tid, 0.f);
    if (sel_out)
      for (uint32_t i = tid; i < k; i += kAttThreads) sel_out[static_cast<size_t>(bh) * k + i] = -1;
    return;
  }
  const uint32_t n = static_cast<uint32_t>(seq_len) - 1u;  // past tokens
  const int32_t* table = page_indices + (table_stride ? static_cast<size_t>(b) * table_stride
                                                      : static_cast<size_t>(page_indptr[b]));
  const uint32_t rows_per_page = kHnd ? 2u * page_size * num_kv_heads : 2u * page_size;
  int32_t cur_row;
  uint32_t cur_page, cur_slot;
  {
    const uint32_t lp = n / page_size;
    cur_page = static_cast<uint32_t>(table[lp]);
    cur_slot = n - lp * page_size;
    cur_row = static_cast<int32_t>(cur_page * rows_per_page + cur_slot);
  }

  sh.hist[tid] = 0u;
  if (tid < kStepMaxChunks) sh.flag[tid] = 0u;
  if (tid == 0) sh.any_flag = 0u;

  const uint32_t g = tid >> 4;    // group of 16 lanes (32 groups)
  const uint32_t c16 = tid & 15;  // channels [8*c16, 8*c16 + 8)
  float qf[8];
  float kcur[8], vcur[8];  // kFromQkv: the new key (rotated) and value, channels 8*c16 .. +7
  // kFromQkv: wave 0 takes the query row of the projection, wave 1 the new key row, wave 2 the new
  // value row (lane l = channels 2l and 2l+1).  The loads are issued here and used once the
  // candidates have been counted; the results go to the other waves through LDS.
  WaveRopeLoads row_now = {};
  const uint32_t kv_head_now = kv_head_of(head, kv_inv16);  // kv_group = num_heads / num_kv_heads
  // the waves that append the new token of this head's key/value head (one workgroup per key/value head)
  const bool appends = kFromQkv && kv_head_now * kv_group == head;
  uint32_t kcode_word = 0, kpacked = 0;  // wave 1: code word and fp16 pair of the rotated new key
  if (kFromQkv) {
    if (wave < 3) {
      const __half* row = src.qkv + static_cast<size_t>(b) * (num_heads + 2 * num_kv_heads) * kHeadDim;
      const uint32_t sel_row = wave == 0 ? head
                               : wave == 1 ? num_heads + kv_head_now
                                           : num_heads + num_kv_heads + kv_head_now;
      row_now = wave_rope_load(row + static_cast<size_t>(sel_row) * kHeadDim, src, n, lane);
    }
  } else {
    load_query<kBf16>(q + static_cast<size_t>(bh) * kHeadDim, c16, scale_log2, qf);
  }

  // a candidate is (distance << 48) | (token offset in its chunk << 32) | K row index
  uint32_t key[kSlots], off[kSlots], krow[kSlots];
#pragma unroll
  for (int j = 0; j < kSlots / 2; ++j) {
    key[2 * j] = raw[j].y >> 16;  // an unused slot reads 0xffff: above every threshold
    key[2 * j + 1] = raw[j].w >> 16;
    off[2 * j] = raw[j].y & 0xffffu;
    off[2 * j + 1] = raw[j].w & 0xffffu;
    krow[2 * j] = raw[j].x;
    krow[2 * j + 1] = raw[j].z;
  }
  const uint32_t chunk_mine = slot0 >> geom.kc_log2;
  const uint32_t chunk_tok0 = chunk_first_unit(geom, chunk_mine) * kStepUnit;
  __syncthreads();  // the histogram is cleared
#pragma unroll
  for (int i = 0; i < kSlots; ++i)
    if (key[i] < static_cast<uint32_t>(kHistBins)) atomicAdd(&sh.hist[key[i]], 1u);
  if (kFromQkv && wave < 3) {
    float x0, x1;
    if (wave == 2) {  // the value row is taken as it is
      unpack2<kBf16>(row_now.raw, x0, x1);
    } else {
      wave_rope_apply<kBf16>(row_now, lane, x0, x1);
    }
    const float f = wave == 0 ? scale_log2 : 1.0f;
    *reinterpret_cast<float2*>(&sh.qkv_now[wave][2 * lane]) = make_float2(x0 * f, x1 * f);
    if (wave == 1) {
      kpacked = pack2<kBf16>(x0, x1);
      transform_row<kBf16>(x0, x1, lane, src.scale, (src.code_flags & ADAMAS_F_CODE_FROM_FP32) != 0);
      kcode_word = wave_pack_codes(x0, x1, lane);
    }
  }
  __syncthreads();  // the histogram is complete

  // ---- selection among the listed candidates ----------------------------------------------------------
  // every wave reads the threshold off the histogram for itself (no exchange)
  WavePlan plan = wave_plan_from_hist(sh.hist, k);
  // Ranks of this thread's two slots: `rb` listed candidates below the threshold and `re` tied ones
  // come before them in slot order (wave prefix scan + the totals of the earlier waves).
  uint32_t rb, re, list_below;
  auto rank_slots = [&]() __attribute__((always_inline)) {
    uint32_t mine = 0;
#pragma unroll
    for (int i = 0; i < kSlots; ++i)
      mine += (key[i] < plan.thr ? 1u : 0u) + ((key[i] == plan.thr ? 1u : 0u) << 16);
    const uint32_t incl = wave_inclusive_scan_dpp(mine);
    if (lane == kWave - 1) sh.wclass[wave] = incl;
    __syncthreads();
    static_assert(kAttWaves == 8, "two 128-bit reads cover the wave totals");
    const uint4 lo = *reinterpret_cast<const uint4*>(&sh.wclass[0]);
    const uint4 hi = *reinterpret_cast<const uint4*>(&sh.wclass[4]);
    const uint32_t t[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    uint32_t before = 0, all = 0;  // the 16-bit fields cannot carry: at most 2048 slots
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      before += w < wave ? t[w] : 0u;
      all += t[w];
    }
    const uint32_t excl = before + incl - mine;
    rb = excl & 0xffffu;
    re = excl >> 16;
    list_below = all & 0xffffu;
  };
  const bool want_pos = sel_out != nullptr;
  // writes the selected ones of this thread's slots into the row list; `tie_shift` tied tokens of
  // re-scored chunks come before this thread's chunk.  Returns whether the last slot was selected.
  auto emit_slots = [&](uint32_t tie_shift) __attribute__((always_inline)) -> bool {
    uint32_t pb = rb, pe = re + tie_shift;
    bool last_selected = false;
#pragma unroll
    for (int i = 0; i < kSlots; ++i) {
      const bool is_b = key[i] < plan.thr, is_e = key[i] == plan.thr;
      const bool take = is_b || (is_e && pe < plan.quota);
      if (take) {
        const uint32_t pos = is_b ? pb : plan.n_below + pe;
        sh.rows[pos] = static_cast<int32_t>(krow[i]);
        if (want_pos) sh.sel_pos[pos] = static_cast<int32_t>(chunk_tok0 + off[i]);
      }
      pb += is_b ? 1u : 0u;
      pe += is_e ? 1u : 0u;
      last_selected = take;
    }
    return last_selected;
  };
  rank_slots();
  {
    const bool last_selected = emit_slots(0u);
    // The list of a chunk is a prefix of the chunk in (distance, index) order.  If its last entry is
    // selected and the chunk holds more tokens than the list, tokens outside the list may belong to
    // the selection too: the chunk is scored again below.
    if (last_selected && ((slot0 + kSlots - 1u) & (geom.kc - 1u)) == geom.kc - 1u) {
      const uint32_t chunk_len = min(chunk_units(geom, chunk_mine) * kStepUnit, n - chunk_tok0);
      if (chunk_len > geom.kc) {
        sh.flag[chunk_mine] = 1u;
        sh.any_flag = 1u;
      }
    }
  }
  if (!kFromQkv && tid == 0) sh.rows[plan.n_take] = cur_row;  // the current token closes the list
  __syncthreads();  // the row list is complete, or some chunk is flagged

  if (sh.any_flag) {
    // ---- some lists were too short: score those chunks again and select among all their tokens -------
    // (at most (budget-1) / kc chunks: every one of them has kc selected entries)
    const uint64_t fmask = __ballot(sh.flag[lane] != 0u);  // the same in every wave
    const bool mine_flagged = have && ((fmask >> chunk_mine) & 1ull) != 0;
    if (mine_flagged) {  // the listed entries of such a chunk leave the count: its tokens come back below
#pragma unroll
      for (int i = 0; i < kSlots; ++i) {
        if (key[i] < static_cast<uint32_t>(kHistBins)) atomicSub(&sh.hist[key[i]], 1u);
        key[i] = 0xffffu;
      }
    }
    const uint16_t* qc = q_code + static_cast<size_t>(bh) * kCodeWords;
    const QueryPlanes qp_lo = make_query_planes(*reinterpret_cast<const uint4*>(qc));
    const QueryPlanes qp_hi = make_query_planes(*reinterpret_cast<const uint4*>(qc + 8));
    uint16_t* drow = dist_scratch + static_cast<size_t>(bh) * dist_stride;
    const uint32_t code_row_bytes = num_kv_heads * 32u;
    for (uint64_t m = fmask; m; m &= m - 1) {
      const uint32_t c = static_cast<uint32_t>(__ffsll(static_cast<long long>(m)) - 1);
      const uint32_t t0 = chunk_first_unit(geom, c) * kStepUnit;
      const uint32_t len = min(chunk_units(geom, c) * kStepUnit, n - t0);
      for (uint32_t t = tid; t < len; t += kAttThreads) {
        const uint32_t pos = t0 + t;
        const uint32_t lp = pos / page_size;
        const uint32_t tslot = static_cast<uint32_t>(table[lp]) * page_size + (pos - lp * page_size);
        const unsigned char* cp =
            code_data + static_cast<size_t>(tslot) * code_row_bytes + kv_head_now * 32u;
        const uint32_t d = l1_64(*reinterpret_cast<const uint4*>(cp), qp_lo) +
                           l1_64(*reinterpret_cast<const uint4*>(cp + 16), qp_hi);
        drow[pos] = static_cast<uint16_t>(d);
        atomicAdd(&sh.hist[d], 1u);
      }
    }
    __syncthreads();  // counts complete; the distances written above are visible to the workgroup
    plan = wave_plan_from_hist(sh.hist, k);
    // wave w counts the tokens below / equal to the new threshold in the flagged chunks w, w+8, ...
    {
      uint32_t f = 0;
      for (uint64_t m = fmask; m; m &= m - 1, ++f) {
        if ((f & (kAttWaves - 1)) != static_cast<uint32_t>(wave)) continue;
        const uint32_t c = static_cast<uint32_t>(__ffsll(static_cast<long long>(m)) - 1);
        const uint32_t t0 = chunk_first_unit(geom, c) * kStepUnit;
        const uint32_t len = min(chunk_units(geom, c) * kStepUnit, n - t0);
        uint32_t cb = 0, ce = 0;
        for (uint32_t t = 0; t < len; t += kWave) {
          const uint32_t d = t + lane < len ? static_cast<uint32_t>(drow[t0 + t + lane]) : 0xffffu;
          cb += __popcll(__ballot(d < plan.thr));
          ce += __popcll(__ballot(d == plan.thr));
        }
        if (lane == 0) {
          sh.fb[c] = cb;
          sh.ft[c] = ce;
        }
      }
    }
    rank_slots();  // (its barrier also publishes fb and ft)
    // listed ties of all chunks in front of a flagged chunk: what its first slot's thread counted
    if (mine_flagged && (slot0 & (geom.kc - 1u)) == 0u) sh.tbase[chunk_mine] = re;
    uint32_t tie_shift = 0;  // tied tokens of flagged chunks in front of this thread's chunk
    for (uint64_t m = have ? fmask & ((1ull << chunk_mine) - 1ull) : 0ull; m; m &= m - 1)
      tie_shift += sh.ft[__ffsll(static_cast<long long>(m)) - 1];
    __syncthreads();
    emit_slots(tie_shift);
    // the flagged chunks, walked in token order by their waves: tokens below the threshold go behind
    // the listed ones, tied tokens take the rank their index gives them among all ties
    {
      uint32_t f = 0, bb = list_below, tb = 0;
      for (uint64_t m = fmask; m; m &= m - 1, ++f) {
        const uint32_t c = static_cast<uint32_t>(__ffsll(static_cast<long long>(m)) - 1);
        if ((f & (kAttWaves - 1)) == static_cast<uint32_t>(wave)) {
          const uint32_t t0 = chunk_first_unit(geom, c) * kStepUnit;
          const uint32_t len = min(chunk_units(geom, c) * kStepUnit, n - t0);
          uint32_t pb = bb, pe = sh.tbase[c] + tb;
          for (uint32_t t = 0; t < len; t += kWave) {
            const uint32_t pos = t0 + t + lane;
            const uint32_t d = t + lane < len ? static_cast<uint32_t>(drow[pos]) : 0xffffu;
            const uint64_t mb = __ballot(d < plan.thr), me = __ballot(d == plan.thr);
            const uint32_t r_e = pe + lanes_below(me);
            const bool is_b = d < plan.thr;
            if (is_b || (d == plan.thr && r_e < plan.quota)) {
              const uint32_t dst_pos = is_b ? pb + lanes_below(mb) : plan.n_below + r_e;
              const uint32_t lp = pos / page_size;
              sh.rows[dst_pos] = static_cast<int32_t>(static_cast<uint32_t>(table[lp]) * rows_per_page +
                                                      (pos - lp * page_size));
              if (want_pos) sh.sel_pos[dst_pos] = static_cast<int32_t>(pos);
            }
            pb += __popcll(mb);
            pe += __popcll(me);
          }
        }
        bb += sh.fb[c];
        tb += sh.ft[c];
      }
    }
    if (!kFromQkv && tid == 0) sh.rows[plan.n_take] = cur_row;
    __syncthreads();  // the row list is complete
  }
  const uint32_t n_take = plan.n_take;
  if (want_pos) {
    int32_t* sdst = sel_out + static_cast<size_t>(bh) * k;
    for (uint32_t i = tid; i < k; i += kAttThreads) sdst[i] = i < n_take ? sh.sel_pos[i] : -1;
  }
  if (kFromQkv) {
    // the query for every group, the new key and value for the group that attends them
    const float4 a0 = *reinterpret_cast<const float4*>(&sh.qkv_now[0][8 * c16]);
    const float4 a1 = *reinterpret_cast<const float4*>(&sh.qkv_now[0][8 * c16 + 4]);
    qf[0] = a0.x; qf[1] = a0.y; qf[2] = a0.z; qf[3] = a0.w;
    qf[4] = a1.x; qf[5] = a1.y; qf[6] = a1.z; qf[7] = a1.w;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      kcur[j] = sh.qkv_now[1][8 * c16 + j];
      vcur[j] = sh.qkv_now[2][8 * c16 + j];
    }
    if (appends && (wave == 1 || wave == 2)) {
      // the new token goes into the caches after every read of them: wave 1 writes K (rotated) and
      // its code, wave 2 writes V
      const uint32_t lay = kHnd ? ADAMAS_F_HND : 0u;
      if (wave == 1) {
        reinterpret_cast<uint32_t*>(kv_append + kv_row_offset(cur_page, 0, cur_slot, kv_head_now,
                                                              page_size, num_kv_heads, lay))[lane] =
            kpacked;
        if ((lane & 3) == 0)
          code_append[((static_cast<size_t>(cur_page) * page_size + cur_slot) * num_kv_heads +
                       kv_head_now) * kCodeWords + (lane >> 2)] = static_cast<uint16_t>(kcode_word);
      } else {
        reinterpret_cast<uint32_t*>(kv_append + kv_row_offset(cur_page, 1, cur_slot, kv_head_now,
                                                              page_size, num_kv_heads, lay))[lane] =
            row_now.raw;
      }
    }
  }

  // ---- attention over the selected tokens and the current one ------------------------------------
  const uint32_t n_rows = kFromQkv ? n_take : n_take + 1u;
  const bool few = n_rows <= kAttendGroups * 8u;  // uniform
  if (few && wave >= kAttendWaves) return;  // (the barriers below count the waves that are still here)
  HeadKV kv;
  kv.kv_data = kv_data;
  kv.table = nullptr;  // rows are K row indices already
  set_kv_layout_static<kHnd>(kv, kv_head_now, c16, num_kv_heads, page_size);
  kv.seq_len = seq_len;
  SoftmaxState st;
  auto row_of = [&](uint32_t r) __attribute__((always_inline)) -> int32_t { return sh.rows[r]; };
  if (few)
    attend_rows<kAttendGroups, 8, true, kBf16, true>(kv, qf, g, 0u, n_rows, row_of, st);
  else  // (129 .. 256 rows in one round of 8 per group: 0.2 us less than two rounds of 4)
    attend_rows<32, 8, true, kBf16, true>(kv, qf, g, 0u, n_rows, row_of, st);
  if (kFromQkv) {
    // the current token, from registers: one more row for group 0
    float d = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) d += qf[j] * kcur[j];
    d = group16_sum(d);
    const bool mine = g == 0;
    const float m_new = mine ? fmaxf(st.m, d) : st.m;
    const float alpha = exp2_raw(st.m - m_new);
    const float pw = mine ? exp2_raw(d - m_new) : 0.f;
    st.l = st.l * alpha + pw;
#pragma unroll
    for (int j = 0; j < 8; ++j) st.o[j] = st.o[j] * alpha + pw * vcur[j];
    st.m = m_new;
  }
  float M, L, O;
  if (few)
    merge_groups<kAttendGroups>(st, g, c16, tid, sh.merge_few, M, L, O);
  else
    merge_groups<32>(st, g, c16, tid, sh.merge, M, L, O);
  if (tid < kHeadDim) store_elem<kBf16>(out + static_cast<size_t>(bh) * kHeadDim + tid, O / L);
}

// ---- budgets beyond the candidate lists: selection from the histograms and attention in one launch --
// The estimator in histogram mode leaves, per head, the distances of all tokens, a 512-bin histogram
// per chunk of 512 tokens and, per sequence, the K row index of every token.  grid (sequence*heads,
// slabs of 4096 tokens), 256 threads.  Every workgroup works the threshold out for itself from the
// chunk rows (they are small and sit in L2; rows of one head are the fast grid dimension so that its
// slabs share a die), adding up on the side the rows of the chunks BEFORE its slab: those give the
// number of selected tokens that precede the slab, i.e. the tie quota left for it and where its
// positions go.  Then it selects among its own 4096 distances (class masks and DPP prefix scans),
// keeps the K rows of the selected tokens in LDS and attends them: 16 groups of 16 lanes, tiles of
// 8 rows.  The slabs of a head are merged inside the launch (split_merge.h).  Against a launch that
// writes the selection followed by the attention operator, this saves a launch, the list's trip
// through memory and the wait for it.
constexpr int kHsaThreads = 256;
constexpr int kHsaWaves = kHsaThreads / kWave;
constexpr int kHsaMaxItems = 16;                                 // distances per thread, at most
constexpr uint32_t kHsaMaxSlab = kHsaThreads * kHsaMaxItems;     // 4096 tokens per workgroup, at most
constexpr int kHsaGroups = kHsaThreads / 16;
constexpr uint32_t kHsaMaxTokens = kHsaMaxSlab * 32;             // 32 slabs per head at most

// Tokens per thread of hist_select_attend_kernel (4, 8 or 16: slabs of 1024, 2048 or 4096 tokens).
// One CU gathers scattered rows slowly, so the slab is halved while that leaves at most
// max(slabs of 4096 tokens, min(16, budget / 64)) slabs per head: about 64 selected rows per
// workgroup where the length allows it, and never more than 16 slabs for the sake of the rows
// (beyond that the merge inside the launch costs more than the shorter gather saves).  Measured
// against slabs of 4096 tokens throughout: 8192 tokens, budget 4096: 41.0 -> 24.8 us; 16384 / 1024:
// 20.1 -> 18.4; 32768 / 1024: 23.3 -> 22.7; a target of 32 rows or a cap of 32 slabs is slower.
inline int hsa_items(uint32_t max_seq_len, uint32_t budget) {
  const uint32_t n = max_seq_len > 1 ? max_seq_len - 1 : 1;
  const uint32_t most =
      std::max((n + kHsaMaxSlab - 1) / kHsaMaxSlab, std::min(16u, (budget + 63u) / 64u));
  int items = kHsaMaxItems;
  while (items > 4 && (n + kHsaThreads * (items / 2) - 1) / (kHsaThreads * (items / 2)) <= most)
    items /= 2;
  return items;
}

template <int kItems>
struct HistSelectAttendShared {
  alignas(16) uint32_t all[kHsaWaves][kHistBins];  // partial sums over all chunk rows
  alignas(16) uint32_t pre[kHsaWaves][kHistBins];  // partial sums over the chunk rows before the slab
  uint32_t wtot[kHsaWaves], wpre[kHsaWaves], wclass[kHsaWaves];
  uint32_t pre_tied;   // tokens at the threshold distance in the chunks before the slab
  SelectPlan plan;
  int32_t rows[kHsaThreads * kItems + 1];  // K rows of the slab's selected tokens (slab 0: then the current token)
  MergeShared<kHsaGroups> merge;
  uint32_t is_last;
};

template <bool kBf16, bool kHnd, int kItems>
__global__ __launch_bounds__(kHsaThreads) void hist_select_attend_kernel(
    const __half* __restrict__ q, const __half* __restrict__ kv_data,
    const int32_t* __restrict__ page_indices, const int32_t* __restrict__ page_indptr,
    const int32_t* __restrict__ seq_lens, const uint16_t* __restrict__ dist, int64_t dist_stride,
    const uint16_t* __restrict__ hist, uint32_t n_chunks, const uint32_t* __restrict__ rowmap,
    uint32_t k, __half* __restrict__ out, int32_t* __restrict__ sel_out, float* partial,
    uint32_t* __restrict__ counters, uint32_t num_heads, uint32_t num_kv_heads, uint32_t kv_inv16,
    uint32_t page_size, float scale_log2) {
  static_assert(kHsaThreads * 2 == kHistBins, "two bins per thread in the prefix sum");
  static_assert(kItems == 4 || kItems == 8 || kItems == 16, "whole histogram rows per slab");
  constexpr uint32_t kSlab = kHsaThreads * kItems;         // tokens per workgroup
  constexpr uint32_t kSlabChunks = kSlab / kFusedBlock;    // histogram rows per slab
  __shared__ HistSelectAttendShared<kItems> sh;
  const uint32_t bh = blockIdx.x, slab = blockIdx.y;
  const uint32_t b = bh / num_heads, head = bh - b * num_heads;
  const uint32_t tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t g = tid >> 4, c16 = tid & 15;
  int32_t* sdst = sel_out ? sel_out + static_cast<size_t>(bh) * k : nullptr;
  const int32_t seq_len = seq_lens[b];
  if (seq_len <= 0) {  // a sequence without tokens: zeros and an empty selection
    if (slab == 0) {
      if (tid < kHeadDim) store_elem<kBf16>(out + static_cast<size_t>(bh) * kHeadDim + tid, 0.f);
      if (sdst)
        for (uint32_t i = tid; i < k; i += kHsaThreads) sdst[i] = -1;
    }
    return;
  }
  const uint32_t n = static_cast<uint32_t>(seq_len) - 1u;                 // past tokens
  const uint32_t n_split = n ? (n + kSlab - 1) / kSlab : 1u;              // slabs that hold tokens
  if (slab >= n_split) return;
  const uint32_t slab_base = slab * kSlab;
  // thread t holds the kItems consecutive tokens t*kItems .. of the slab: distances and K rows,
  // asked for first
  const uint32_t e0 = slab_base + tid * kItems;
  uint32_t keys[kItems], trow[kItems];
  {
    const uint16_t* vrow = dist + static_cast<int64_t>(bh) * dist_stride + e0;  // 2*kItems-byte aligned
    const uint32_t* rm = rowmap + static_cast<int64_t>(b) * dist_stride + e0;
    uint32_t kw[kItems / 2];  // two distances per word
    uint4 rraw[kItems / 4];
    if (kItems == 4) {
      const uint2 v = e0 < n ? *reinterpret_cast<const uint2*>(vrow) : make_uint2(~0u, ~0u);
      kw[0] = v.x;
      kw[1] = v.y;
    } else {
#pragma unroll
      for (int j = 0; j < kItems / 8; ++j) {
        const uint4 v = e0 + 8 * j < n ? *reinterpret_cast<const uint4*>(vrow + 8 * j)
                                       : make_uint4(~0u, ~0u, ~0u, ~0u);
        kw[4 * j] = v.x;
        kw[4 * j + 1] = v.y;
        kw[4 * j + 2] = v.z;
        kw[4 * j + 3] = v.w;
      }
    }
#pragma unroll
    for (int j = 0; j < kItems / 4; ++j)
      rraw[j] = e0 + 4 * j < n ? *reinterpret_cast<const uint4*>(rm + 4 * j)
                               : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
    for (int i = 0; i < kItems; ++i) {
      const uint32_t v = (kw[i >> 1] >> (16 * (i & 1))) & 0xffffu;
      keys[i] = e0 + i < n ? v : 0xffffu;  // past the end: above every threshold
    }
#pragma unroll
    for (int j = 0; j < kItems / 4; ++j) {
      trow[4 * j] = rraw[j].x;
      trow[4 * j + 1] = rraw[j].y;
      trow[4 * j + 2] = rraw[j].z;
      trow[4 * j + 3] = rraw[j].w;
    }
  }
  float qf[8];
  load_query<kBf16>(q + static_cast<size_t>(bh) * kHeadDim, c16, scale_log2, qf);
  const int32_t* table = page_indices + page_indptr[b];
  const uint32_t rows_per_page = kHnd ? 2u * page_size * num_kv_heads : 2u * page_size;
  int32_t cur_row = 0;
  if (slab == 0) {  // the current token is attended with the first slab
    const uint32_t lp = n / page_size;
    cur_row = static_cast<int32_t>(static_cast<uint32_t>(table[lp]) * rows_per_page + (n - lp * page_size));
  }

  // ---- chunk rows (16-bit counts): thread (part, seg) adds bins 8*seg .. 8*seg+7 of rows part, part+4, ...
  {
    const uint32_t part = tid >> 6, seg = tid & 63u;
    const uint32_t c_first = slab * kSlabChunks;  // chunks below it precede the slab
    const unsigned char* hb = reinterpret_cast<const unsigned char*>(hist) +
                              static_cast<size_t>(bh) * n_chunks * (2 * kHistBins) + seg * 16u;
    const uint32_t rows_used = min(n_chunks, (n + kFusedBlock - 1) / kFusedBlock);  // rows of this sequence
    uint32_t acc[8] = {0, 0, 0, 0, 0, 0, 0, 0}, pre[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (uint32_t c0 = part; c0 < rows_used; c0 += 16) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t c = c0 + 4u * u;
        v[u] = c < rows_used
                   ? *reinterpret_cast<const uint4*>(hb + static_cast<size_t>(c) * (2 * kHistBins))
                   : make_uint4(0u, 0u, 0u, 0u);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
        const uint32_t m = (c0 + 4u * u < c_first) ? 0xffffffffu : 0u;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[2 * j] += w[j] & 0xffffu;
          acc[2 * j + 1] += w[j] >> 16;
          pre[2 * j] += w[j] & 0xffffu & m;
          pre[2 * j + 1] += (w[j] >> 16) & m;
        }
      }
    }
    uint4* da = reinterpret_cast<uint4*>(&sh.all[part][seg * 8u]);
    da[0] = make_uint4(acc[0], acc[1], acc[2], acc[3]);
    da[1] = make_uint4(acc[4], acc[5], acc[6], acc[7]);
    uint4* dp = reinterpret_cast<uint4*>(&sh.pre[part][seg * 8u]);
    dp[0] = make_uint4(pre[0], pre[1], pre[2], pre[3]);
    dp[1] = make_uint4(pre[4], pre[5], pre[6], pre[7]);
  }
  __syncthreads();
  // ---- thread t owns bins 2t and 2t+1: prefix sum -> the plan
  uint32_t ca0 = 0, ca1 = 0, cp0 = 0, cp1 = 0;
#pragma unroll
  for (int p = 0; p < kHsaWaves; ++p) {
    const uint2 x = *reinterpret_cast<const uint2*>(&sh.all[p][2 * tid]);
    const uint2 y = *reinterpret_cast<const uint2*>(&sh.pre[p][2 * tid]);
    ca0 += x.x;
    ca1 += x.y;
    cp0 += y.x;
    cp1 += y.y;
  }
  const uint32_t incl = wave_inclusive_scan_dpp(ca0 + ca1);
  if (lane == kWave - 1) sh.wtot[wave] = incl;
  __syncthreads();
  uint32_t cum1 = incl;  // tokens with a distance <= bin 2t+1
  for (int w = 0; w < wave; ++w) cum1 += sh.wtot[w];
  const uint32_t cum0 = cum1 - ca1;  // <= bin 2t
  if (cum0 >= k && cum0 - ca0 < k) {  // exactly one bin holds the k-th smallest distance
    sh.plan.thr = 2 * tid;
    sh.plan.n_below = cum0 - ca0;
    sh.plan.quota = k - (cum0 - ca0);
    sh.plan.n_take = k;
    sh.pre_tied = cp0;
  }
  if (cum1 >= k && cum0 < k) {
    sh.plan.thr = 2 * tid + 1;
    sh.plan.n_below = cum0;
    sh.plan.quota = k - cum0;
    sh.plan.n_take = k;
    sh.pre_tied = cp1;
  }
  if (tid == kHsaThreads - 1 && cum1 < k) {  // fewer tokens than k: all of them are taken
    sh.plan.thr = kHistBins;
    sh.plan.n_below = cum1;
    sh.plan.quota = 0;
    sh.plan.n_take = cum1;
    sh.pre_tied = 0;
  }
  __syncthreads();
  const SelectPlan plan = sh.plan;
  const uint32_t pre_tied = sh.pre_tied;

  // ---- selected tokens before the slab, class masks and ranks inside it
  const uint32_t mine_pre = (2 * tid < plan.thr ? cp0 : 0u) + (2 * tid + 1 < plan.thr ? cp1 : 0u);
  const uint32_t wave_pre = wave_sum(mine_pre);
  uint32_t below[kItems / 4], equal[kItems / 4];
  raw_class_masks<kItems>(keys, plan.thr, below, equal);
  uint32_t total;
  const uint32_t excl = lane_scan<kItems / 4>(below, equal, total);  // below | tied << 16
  if (lane == 0) {
    sh.wpre[wave] = wave_pre;
    sh.wclass[wave] = total;
  }
  __syncthreads();
  uint32_t base_b = 0, before = 0, slab_all = 0;
#pragma unroll
  for (int w = 0; w < kHsaWaves; ++w) {
    base_b += sh.wpre[w];
    before += w < wave ? sh.wclass[w] : 0u;
    slab_all += sh.wclass[w];
  }
  const uint32_t slab_below = slab_all & 0xffffu, slab_tied = slab_all >> 16;
  // tied tokens of this slab that are inside the quota (ties go to the lowest index: the chunks
  // before the slab come first)
  const uint32_t tied_left = plan.quota > pre_tied ? plan.quota - pre_tied : 0u;
  const uint32_t slab_tied_taken = min(slab_tied, tied_left);
  // positions in the whole selection: the tokens below the threshold in index order, then the ties
  lane_emit<kItems / 4>(below, equal, plan.n_below, plan.quota,
                           base_b + (before & 0xffffu) + (excl & 0xffffu),
                           pre_tied + (before >> 16) + (excl >> 16),
                           [&](uint32_t pos, int i) __attribute__((always_inline)) {
                             const bool is_b = keys[i] < plan.thr;
                             const uint32_t local = is_b ? pos - base_b
                                                         : slab_below + (pos - plan.n_below - pre_tied);
                             sh.rows[local] = static_cast<int32_t>(trow[i]);
                             if (sdst) sdst[pos] = static_cast<int32_t>(e0 + i);
                           });
  uint32_t n_rows = slab_below + slab_tied_taken;
  if (slab == 0) {
    if (tid == 0) sh.rows[n_rows] = cur_row;
    ++n_rows;
    if (sdst)
      for (uint32_t i = plan.n_take + tid; i < k; i += kHsaThreads) sdst[i] = -1;
  }
  __syncthreads();

  // ---- attention over the rows of the slab -------------------------------------------------------------
  HeadKV kv;
  kv.kv_data = kv_data;
  kv.table = nullptr;  // rows are K row indices already
  set_kv_layout_static<kHnd>(kv, kv_head_of(head, kv_inv16), c16, num_kv_heads, page_size);
  kv.seq_len = seq_len;
  SoftmaxState st;
  // (a group asks for 2, 4 or 8 rows at a time: slots past the end load the last row again, so the
  // round is no larger than the slab's rows need)
  auto row_of = [&](uint32_t r) __attribute__((always_inline)) -> int32_t { return sh.rows[r]; };
  if (n_rows <= kHsaGroups * 2u)
    attend_rows<kHsaGroups, 2, true, kBf16, true>(kv, qf, g, 0u, n_rows, row_of, st);
  else if (n_rows <= kHsaGroups * 4u)
    attend_rows<kHsaGroups, 4, true, kBf16, true>(kv, qf, g, 0u, n_rows, row_of, st);
  else
    attend_rows<kHsaGroups, 8, true, kBf16, true>(kv, qf, g, 0u, n_rows, row_of, st);
  float M, L, O;
  merge_groups<kHsaGroups>(st, g, c16, tid, sh.merge, M, L, O);
  if (n_split == 1) {
    if (tid < kHeadDim)
      store_elem<kBf16>(out + static_cast<size_t>(bh) * kHeadDim + tid, L > 0.f ? O / L : 0.f);
    return;
  }
  // several slabs: publish the partial, the last arrival merges (protocol: split_merge.h)
  float* mine = partial + (static_cast<size_t>(bh) * kMaxSplits + slab) * kPartialFloats;
  if (tid < kHeadDim) {
    if (tid == 0) {
      __hip_atomic_store(mine + 0, M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(mine + 1, L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __hip_atomic_store(mine + 2 + tid, O, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (!split_arrive_is_last(&counters[bh], n_split, sh.is_last, tid)) return;
  if (tid < kHeadDim) {
    float LL, OO[1];
    merge_partials<1>(partial + static_cast<size_t>(bh) * kMaxSplits * kPartialFloats, n_split, tid,
                      LL, OO);
    store_elem<kBf16>(out + static_cast<size_t>(bh) * kHeadDim + tid, LL > 0.f ? OO[0] / LL : 0.f);
  }
  if (tid == 0) counters[bh] = 0;  // ready for the next launch on this stream
}

}  // namespace adamas

using namespace adamas;

// the two-launch path serves budgets up to 256 and sequences the plan of workspace.h covers
static bool fused_eligible(const WorkspaceLayout& w) { return w.plan.ok != 0; }

extern "C" int adamas_step_fused_supported(uint32_t batch, uint32_t num_heads,
                                           uint32_t max_seq_len, uint32_t budget) {
  if (batch == 0 || num_heads == 0 || num_heads % 8 != 0 || budget == 0 || max_seq_len == 0)
    return 0;
  return fused_eligible(workspace_layout(batch, num_heads, max_seq_len, budget)) ? 1 : 0;
}

extern "C" int adamas_step_plan(uint32_t batch, uint32_t num_heads, uint32_t max_seq_len,
                                uint32_t budget, uint32_t* plan_out) {
  if (!plan_out) return ADAMAS_E_BADARG;
  const StepPlan p = (batch && num_heads && num_heads % 8 == 0)
                         ? step_plan(batch, num_heads, max_seq_len, budget)
                         : StepPlan{};
  const uint32_t v[8] = {p.ok, p.heads, p.chunks, p.units_q, p.units_r, p.passes, p.partial, p.kc};
  for (int i = 0; i < 8; ++i) plan_out[i] = v[i];
  return 0;
}

// rows per page of the KV layout the K row indices are meant for
static uint32_t rows_per_page_of(uint32_t flags, uint32_t page_size, uint32_t num_kv_heads) {
  return make_kv_layout((flags & ADAMAS_F_HND) != 0, page_size, num_kv_heads).rows_per_page;
}

static StepGeom geom_of(const StepPlan& p) {
  StepGeom g;
  g.units_q = p.units_q;
  g.units_r = p.units_r;
  g.kc = p.kc;
  g.kc_log2 = p.kc_log2;
  return g;
}

// qsrc != nullptr: the query codes are made in the kernel from the fused projection (q_code unused)
static int step_candidates_impl(const void* q_code, const void* code_data,
                                const int32_t* page_indices, const int32_t* page_indptr,
                                const int32_t* seq_lens, uint32_t budget, void* workspace,
                                size_t workspace_bytes, uint32_t batch, uint32_t num_heads,
                                uint32_t num_kv_heads, uint32_t page_size, uint32_t max_seq_len,
                                uint32_t page_table_stride, uint32_t flags,
                                adamas_stream_t stream, const QkvSource* qsrc) {
  if (flags & ~(ADAMAS_F_BF16 | ADAMAS_F_HND)) return ADAMAS_E_BADARG;
  if (qsrc) q_code = qsrc->qkv;  // any valid, aligned pointer: the kernel does not read it
  if (!q_code || !code_data || !page_indices || (!page_indptr && !page_table_stride) ||
      !seq_lens || !workspace ||
      budget == 0 || max_seq_len == 0 || batch == 0 || page_size == 0)
    return ADAMAS_E_BADARG;
  if (num_heads == 0 || num_heads % 8 != 0 || batch > 65535) return ADAMAS_E_UNSUPPORTED;
  if (num_kv_heads == 0 || num_heads % num_kv_heads != 0) return ADAMAS_E_UNSUPPORTED;
  // the kernels take head / group from a 16-bit reciprocal (kv_head_of)
  if (static_cast<uint64_t>(num_heads) * (num_heads / num_kv_heads) >= 65536u) return ADAMAS_E_UNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(workspace) & 255) return ADAMAS_E_ALIGN;
  if ((reinterpret_cast<uintptr_t>(q_code) | reinterpret_cast<uintptr_t>(code_data)) & 15)
    return ADAMAS_E_ALIGN;
  const WorkspaceLayout w = workspace_layout(batch, num_heads, max_seq_len, budget);
  if (workspace_bytes < w.total) return ADAMAS_E_WORKSPACE;
  if (!fused_eligible(w)) return ADAMAS_E_UNSUPPORTED;
  char* ws = static_cast<char*>(workspace);
  uint64_t* cand = reinterpret_cast<uint64_t*>(ws + w.cand_off);
  uint16_t* qcode_ws = reinterpret_cast<uint16_t*>(ws + w.qcode_off);
  const StepPlan& plan = w.plan;
  const int est_heads = static_cast<int>(plan.heads);
  const dim3 grid(plan.chunks, num_heads / est_heads, batch);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define ADAMAS_LAUNCH_ESTSEL_Q(PG, PASSES, PARTIAL, HEADS, FROMQKV)                             \
  hipLaunchKernelGGL((estimate_select_kernel<PG, PASSES, PARTIAL, false, HEADS, FROMQKV>), grid, \
                     dim3(HEADS * kWave), 0, s,                                                 \
                     static_cast<const uint16_t*>(q_code),                                    \
                     static_cast<const unsigned char*>(code_data), page_indices, page_indptr, \
                     seq_lens, cand, geom_of(plan), qcode_ws,                                 \
                     num_heads, num_kv_heads, group_inv16(num_heads / num_kv_heads),         \
                     page_size, page_table_stride,                                            \
                     rows_per_page_of(flags, page_size, num_kv_heads),                        \
                     static_cast<unsigned char*>(nullptr), 0u,                                \
                     static_cast<uint16_t*>(nullptr), static_cast<int64_t>(0),                \
                     static_cast<uint32_t*>(nullptr), qsrc ? *qsrc : QkvSource())
#define ADAMAS_LAUNCH_ESTSEL_H(PG, PASSES, PARTIAL, HEADS)        \
  if (qsrc) {                                                     \
    ADAMAS_LAUNCH_ESTSEL_Q(PG, PASSES, PARTIAL, HEADS, true);     \
  } else {                                                        \
    ADAMAS_LAUNCH_ESTSEL_Q(PG, PASSES, PARTIAL, HEADS, false);    \
  }
#define ADAMAS_LAUNCH_ESTSEL(PG, PASSES, PARTIAL)       \
  if (est_heads == 4) {                                 \
    ADAMAS_LAUNCH_ESTSEL_H(PG, PASSES, PARTIAL, 4)      \
  } else {                                              \
    ADAMAS_LAUNCH_ESTSEL_H(PG, PASSES, PARTIAL, 8)      \
  }
#define ADAMAS_LAUNCH_ESTSEL_PAGE(PASSES, PARTIAL)   \
  if (page_size == 16) {                             \
    ADAMAS_LAUNCH_ESTSEL(16, PASSES, PARTIAL)        \
  } else {                                           \
    ADAMAS_LAUNCH_ESTSEL(0, PASSES, PARTIAL)         \
  }
  // chunks of exactly 512, 1024 or 2048 tokens have instances without the per-unit tests
  if (!plan.partial && plan.passes == 1) {
    ADAMAS_LAUNCH_ESTSEL_PAGE(1, false)
  } else if (!plan.partial && plan.passes == 2) {
    ADAMAS_LAUNCH_ESTSEL_PAGE(2, false)
  } else if (!plan.partial && plan.passes == 4) {
    ADAMAS_LAUNCH_ESTSEL_PAGE(4, false)
  } else if (plan.passes == 1) {
    return ADAMAS_E_UNSUPPORTED;  // (no plan has a partial single pass: its chunks are 512 tokens)
  } else if (plan.passes == 2) {
    ADAMAS_LAUNCH_ESTSEL_PAGE(2, true)
  } else if (plan.passes == 3) {
    ADAMAS_LAUNCH_ESTSEL_PAGE(3, true)
  } else {
    ADAMAS_LAUNCH_ESTSEL_PAGE(4, true)
  }
#undef ADAMAS_LAUNCH_ESTSEL_PAGE
#undef ADAMAS_LAUNCH_ESTSEL
#undef ADAMAS_LAUNCH_ESTSEL_H
#undef ADAMAS_LAUNCH_ESTSEL_Q
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int adamas_step_candidates_f(const void* q_code, const void* code_data,
                                        const int32_t* page_indices, const int32_t* page_indptr,
                                        const int32_t* seq_lens, uint32_t budget, void* workspace,
                                        size_t workspace_bytes, uint32_t batch, uint32_t num_heads,
                                        uint32_t num_kv_heads, uint32_t page_size,
                                        uint32_t max_seq_len, uint32_t page_table_stride,
                                        uint32_t flags, adamas_stream_t stream) {
  return step_candidates_impl(q_code, code_data, page_indices, page_indptr, seq_lens, budget,
                              workspace, workspace_bytes, batch, num_heads, num_kv_heads,
                              page_size, max_seq_len, page_table_stride, flags, stream, nullptr);
}

extern "C" int adamas_step_candidates(const void* q_code, const void* code_data,
                                      const int32_t* page_indices, const int32_t* page_indptr,
                                      const int32_t* seq_lens, uint32_t budget, void* workspace,
                                      size_t workspace_bytes, uint32_t batch, uint32_t num_heads,
                                      uint32_t num_kv_heads, uint32_t page_size,
                                      uint32_t max_seq_len, uint32_t page_table_stride,
                                      adamas_stream_t stream) {
  return adamas_step_candidates_f(q_code, code_data, page_indices, page_indptr, seq_lens, budget,
                                  workspace, workspace_bytes, batch, num_heads, num_kv_heads,
                                  page_size, max_seq_len, page_table_stride, 0u, stream);
}

// qsrc != nullptr: q is made in the kernel from the fused projection, the new token is
// appended by it (kv_data and code_data are written)
static int step_attend_impl(const void* q, void* kv_data, void* code_data,
                            const int32_t* page_indices,
                            const int32_t* page_indptr, const int32_t* seq_lens, uint32_t budget,
                            void* out, int32_t* sel_out, void* workspace, size_t workspace_bytes,
                            uint32_t batch, uint32_t num_heads, uint32_t num_kv_heads,
                            uint32_t head_dim, uint32_t page_size, float sm_scale,
                            uint32_t max_seq_len, uint32_t page_table_stride, uint32_t flags,
                            adamas_stream_t stream, const QkvSource* qsrc) {
  if (flags & ~(ADAMAS_F_BF16 | ADAMAS_F_HND)) return ADAMAS_E_BADARG;
  if (qsrc) q = qsrc->qkv;
  const bool bf16 = (flags & ADAMAS_F_BF16) != 0;
  const bool hnd = (flags & ADAMAS_F_HND) != 0;
  if (!q || !kv_data || !code_data || !page_indices || (!page_indptr && !page_table_stride) ||
      !seq_lens || !out || !workspace ||
      budget == 0 || max_seq_len == 0 || batch == 0 || page_size == 0)
    return ADAMAS_E_BADARG;
  if (head_dim != kHeadDim || num_heads == 0 || num_heads % 8 != 0 || batch > 65535)
    return ADAMAS_E_UNSUPPORTED;
  if (num_kv_heads == 0 || num_heads % num_kv_heads != 0) return ADAMAS_E_UNSUPPORTED;
  // the kernels take head / group from a 16-bit reciprocal (kv_head_of)
  if (static_cast<uint64_t>(num_heads) * (num_heads / num_kv_heads) >= 65536u) return ADAMAS_E_UNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(workspace) & 255) return ADAMAS_E_ALIGN;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(kv_data) |
       reinterpret_cast<uintptr_t>(code_data)) & 15)
    return ADAMAS_E_ALIGN;
  const WorkspaceLayout w = workspace_layout(batch, num_heads, max_seq_len, budget);
  if (workspace_bytes < w.total) return ADAMAS_E_WORKSPACE;
  if (!fused_eligible(w)) return ADAMAS_E_UNSUPPORTED;
  char* ws = static_cast<char*>(workspace);
  const StepPlan& plan = w.plan;
#define ADAMAS_LAUNCH_SELATT_S(SLOTS, BF, HND, FROMQKV)                                          \
  hipLaunchKernelGGL((select_attend_kernel<SLOTS, BF, HND, FROMQKV>), dim3(num_heads, batch),    \
                     dim3(kAttThreads), 0,                                                       \
                     static_cast<hipStream_t>(stream), static_cast<const __half*>(q),           \
                     static_cast<const __half*>(kv_data), page_indices, page_indptr, seq_lens,  \
                     reinterpret_cast<const uint64_t*>(ws + w.cand_off), geom_of(plan),         \
                     plan.chunks, budget - 1, static_cast<__half*>(out), sel_out, num_heads,    \
                     num_kv_heads, num_heads / num_kv_heads,                                    \
                     group_inv16(num_heads / num_kv_heads), page_size,                          \
                     sm_scale * 1.4426950408889634f, page_table_stride,                         \
                     reinterpret_cast<const uint16_t*>(ws + w.qcode_off),                       \
                     static_cast<const unsigned char*>(code_data),                              \
                     reinterpret_cast<uint16_t*>(ws + w.dist_off), w.dist_stride,               \
                     qsrc ? *qsrc : QkvSource(), static_cast<__half*>(kv_data),                 \
                     static_cast<uint16_t*>(code_data))
#define ADAMAS_LAUNCH_SELATT_BF(BF, HND, FROMQKV)     \
  if (plan.chunks * plan.kc > 2 * kAttThreads) {      \
    ADAMAS_LAUNCH_SELATT_S(4, BF, HND, FROMQKV);      \
  } else {                                            \
    ADAMAS_LAUNCH_SELATT_S(2, BF, HND, FROMQKV);      \
  }
#define ADAMAS_LAUNCH_SELATT(FROMQKV)                 \
  if (bf16 && hnd) {                                  \
    ADAMAS_LAUNCH_SELATT_BF(true, true, FROMQKV);     \
  } else if (bf16) {                                  \
    ADAMAS_LAUNCH_SELATT_BF(true, false, FROMQKV);    \
  } else if (hnd) {                                   \
    ADAMAS_LAUNCH_SELATT_BF(false, true, FROMQKV);    \
  } else {                                            \
    ADAMAS_LAUNCH_SELATT_BF(false, false, FROMQKV);   \
  }
  if (qsrc) {
    ADAMAS_LAUNCH_SELATT(true)
  } else {
    ADAMAS_LAUNCH_SELATT(false)
  }
#undef ADAMAS_LAUNCH_SELATT
#undef ADAMAS_LAUNCH_SELATT_BF
#undef ADAMAS_LAUNCH_SELATT_S
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int adamas_step_attend_f(const void* q, const void* kv_data, const void* code_data,
                                    const int32_t* page_indices, const int32_t* page_indptr,
                                    const int32_t* seq_lens, uint32_t budget, void* out,
                                    int32_t* sel_out, void* workspace, size_t workspace_bytes,
                                    uint32_t batch, uint32_t num_heads, uint32_t num_kv_heads,
                                    uint32_t head_dim, uint32_t page_size, float sm_scale,
                                    uint32_t max_seq_len, uint32_t page_table_stride,
                                    uint32_t flags, adamas_stream_t stream) {
  return step_attend_impl(q, const_cast<void*>(kv_data), const_cast<void*>(code_data), page_indices,
                          page_indptr, seq_lens, budget, out, sel_out, workspace, workspace_bytes,
                          batch, num_heads, num_kv_heads, head_dim, page_size, sm_scale, max_seq_len,
                          page_table_stride, flags, stream, nullptr);
}

extern "C" int adamas_step_attend(const void* q, const void* kv_data, const void* code_data,
                                  const int32_t* page_indices,
                                  const int32_t* page_indptr, const int32_t* seq_lens,
                                  uint32_t budget, void* out, int32_t* sel_out, void* workspace,
                                  size_t workspace_bytes, uint32_t batch, uint32_t num_heads,
                                  uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size,
                                  float sm_scale, uint32_t max_seq_len, uint32_t page_table_stride,
                                  adamas_stream_t stream) {
  return adamas_step_attend_f(q, kv_data, code_data, page_indices, page_indptr, seq_lens, budget,
                              out, sel_out, workspace, workspace_bytes, batch, num_heads,
                              num_kv_heads, head_dim, page_size, sm_scale, max_seq_len,
                              page_table_stride, 0u, stream);
}

extern "C" int adamas_decode_step_f(const void* q, const void* q_code, const void* kv_data,
                                    const void* code_data, const int32_t* page_indices,
                                    const int32_t* page_indptr, const int32_t* seq_lens,
                                    uint32_t budget, void* out, int32_t* sel_out, void* workspace,
                                    size_t workspace_bytes, uint32_t batch, uint32_t num_heads,
                                    uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size,
                                    float sm_scale, uint32_t max_seq_len,
                                    uint32_t page_table_stride, uint32_t flags,
                                    adamas_stream_t stream) {
  if (flags & ~(ADAMAS_F_BF16 | ADAMAS_F_HND)) return ADAMAS_E_BADARG;
  if (!q || !q_code || !kv_data || !code_data || !page_indices || !page_indptr || !seq_lens ||
      !out || !workspace || budget == 0 || max_seq_len == 0 || batch == 0 || page_size == 0)
    return ADAMAS_E_BADARG;
  if (head_dim != kHeadDim || num_heads == 0 || num_heads % 8 != 0) return ADAMAS_E_UNSUPPORTED;
  if (num_kv_heads == 0 || num_heads % num_kv_heads != 0) return ADAMAS_E_UNSUPPORTED;
  // the kernels take head / group from a 16-bit reciprocal (kv_head_of)
  if (static_cast<uint64_t>(num_heads) * (num_heads / num_kv_heads) >= 65536u) return ADAMAS_E_UNSUPPORTED;
  if (batch > 65535) return ADAMAS_E_UNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(workspace) & 255) return ADAMAS_E_ALIGN;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(q_code) |
       reinterpret_cast<uintptr_t>(kv_data) | reinterpret_cast<uintptr_t>(code_data)) & 15)
    return ADAMAS_E_ALIGN;
  const WorkspaceLayout w = workspace_layout(batch, num_heads, max_seq_len, budget);
  if (workspace_bytes < w.total) return ADAMAS_E_WORKSPACE;
  char* ws = static_cast<char*>(workspace);
  const uint32_t n_sel = budget - 1;

  if (fused_eligible(w)) {
    int rc = adamas_step_candidates_f(q_code, code_data, page_indices, page_indptr, seq_lens,
                                      budget, workspace, workspace_bytes, batch, num_heads,
                                      num_kv_heads, page_size, max_seq_len, page_table_stride,
                                      flags, stream);
    if (rc != 0) return rc;
    return adamas_step_attend_f(q, kv_data, code_data, page_indices, page_indptr, seq_lens, budget,
                                out, sel_out, workspace, workspace_bytes, batch, num_heads,
                                num_kv_heads, head_dim, page_size, sm_scale, max_seq_len,
                                page_table_stride, flags, stream);
  }

  uint16_t* dist = reinterpret_cast<uint16_t*>(ws + w.dist_off);
  int32_t* sel = sel_out ? sel_out : reinterpret_cast<int32_t*>(ws + w.sel_off);
  // budgets beyond the candidate lists, rows of moderate length: the estimator writes the distances
  // and a histogram per 512-token chunk; the second launch reads threshold and positions off the
  // histograms and attends the selected tokens (also two launches)
  if (n_sel > 0 && max_seq_len > 1 && max_seq_len - 1 <= 131072 && w.hist_stride > 0 &&
      batch <= 65535) {
    // workgroups of 4 heads wherever the 8-head ones would leave CUs idle or unevenly loaded
    const uint64_t wide = static_cast<uint64_t>(w.hist_stride) * (num_heads / kFusedHeads) * batch;
    const int est_heads =
        (batch > 1 || (2 * wide + kStepWorkgroups - 1) / kStepWorkgroups <
                          2 * ((wide + kStepWorkgroups - 1) / kStepWorkgroups))
            ? 4
            : kFusedHeads;
    const dim3 grid(w.hist_stride, num_heads / est_heads, batch);
    StepGeom hist_geom;  // chunks of 512 tokens
    hist_geom.units_q = kFusedBlock / kStepUnit;
    hist_geom.units_r = 0;
    hist_geom.kc = 0;
    hist_geom.kc_log2 = 0;
    unsigned char* hist = reinterpret_cast<unsigned char*>(ws + w.hist_off);
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint32_t* rowmap = reinterpret_cast<uint32_t*>(ws + w.rowmap_off);
#define ADAMAS_LAUNCH_ESTHIST_H(PG, HEADS)                                                       \
  hipLaunchKernelGGL((estimate_select_kernel<PG, 1, false, true, HEADS>), grid,                  \
                     dim3(HEADS * kWave), 0, s,                                                  \
                     static_cast<const uint16_t*>(q_code),                                      \
                     static_cast<const unsigned char*>(code_data), page_indices, page_indptr,   \
                     seq_lens, static_cast<uint64_t*>(nullptr), hist_geom,                      \
                     static_cast<uint16_t*>(nullptr),                                           \
                     num_heads, num_kv_heads, group_inv16(num_heads / num_kv_heads),           \
                     page_size, page_table_stride,                                              \
                     rows_per_page_of(flags, page_size, num_kv_heads), hist, w.hist_stride,     \
                     dist, static_cast<int64_t>(w.dist_stride), rowmap)
#define ADAMAS_LAUNCH_ESTHIST(PG)        \
  if (est_heads == 4) {                  \
    ADAMAS_LAUNCH_ESTHIST_H(PG, 4);      \
  } else {                               \
    ADAMAS_LAUNCH_ESTHIST_H(PG, 8);      \
  }
    if (page_size == 16) {
      ADAMAS_LAUNCH_ESTHIST(16)
    } else {
      ADAMAS_LAUNCH_ESTHIST(0)
    }
#undef ADAMAS_LAUNCH_ESTHIST
#undef ADAMAS_LAUNCH_ESTHIST_H
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    // selection from the histograms and attention over the selected rows, one launch
    const bool bf16 = (flags & ADAMAS_F_BF16) != 0, hnd = (flags & ADAMAS_F_HND) != 0;
    const int items = hsa_items(max_seq_len, budget);
    const uint32_t slab_tokens = kHsaThreads * static_cast<uint32_t>(items);
    const dim3 hgrid(batch * num_heads, (max_seq_len - 1 + slab_tokens - 1) / slab_tokens);
#define ADAMAS_LAUNCH_HSA_I(BF, HND, ITEMS)                                                        \
  hipLaunchKernelGGL((hist_select_attend_kernel<BF, HND, ITEMS>), hgrid, dim3(kHsaThreads), 0, s,  \
                     static_cast<const __half*>(q), static_cast<const __half*>(kv_data),           \
                     page_indices, page_indptr, seq_lens, dist, w.dist_stride,                     \
                     reinterpret_cast<const uint16_t*>(hist), w.hist_stride, rowmap, n_sel,        \
                     static_cast<__half*>(out), sel_out,                                           \
                     reinterpret_cast<float*>(ws + w.partial_off),                                 \
                     reinterpret_cast<uint32_t*>(ws + w.counters_off), num_heads, num_kv_heads,    \
                     group_inv16(num_heads / num_kv_heads), page_size,                             \
                     sm_scale * 1.4426950408889634f)
#define ADAMAS_LAUNCH_HSA(BF, HND)          \
  if (items == 4) {                         \
    ADAMAS_LAUNCH_HSA_I(BF, HND, 4);        \
  } else if (items == 8) {                  \
    ADAMAS_LAUNCH_HSA_I(BF, HND, 8);        \
  } else {                                  \
    ADAMAS_LAUNCH_HSA_I(BF, HND, 16);       \
  }
    if (bf16 && hnd) {
      ADAMAS_LAUNCH_HSA(true, true);
    } else if (bf16) {
      ADAMAS_LAUNCH_HSA(true, false);
    } else if (hnd) {
      ADAMAS_LAUNCH_HSA(false, true);
    } else {
      ADAMAS_LAUNCH_HSA(false, false);
    }
#undef ADAMAS_LAUNCH_HSA
#undef ADAMAS_LAUNCH_HSA_I
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  // general path: the stand-alone entry points one after the other
  if (n_sel > 0 && max_seq_len > 1) {
    int rc = adamas_estimate(q_code, code_data, page_indices, page_indptr, seq_lens, dist,
                             static_cast<int64_t>(num_heads) * w.dist_stride, w.dist_stride,
                             ADAMAS_DIST_U16, batch, num_heads, num_kv_heads, page_size, max_seq_len,
                             stream);
    if (rc != 0) return rc;
    rc = adamas_topk(dist, w.dist_stride, max_seq_len - 1, seq_lens, num_heads, -1, nullptr, 0,
                     batch * num_heads, n_sel, sel, nullptr, static_cast<int64_t>(n_sel),
                     ADAMAS_KEY_U16_INT, ws + w.topk_off, w.topk_bytes, stream);
    if (rc != 0) return rc;
  }
  // with n_sel == 0 the list is empty and only the current token is attended
  return adamas_sparse_decode_f(q, kv_data, page_indices, page_indptr, seq_lens, sel,
                                static_cast<int64_t>(n_sel), (max_seq_len > 1) ? n_sel : 0u, out,
                                workspace, workspace_bytes, batch, num_heads, num_kv_heads,
                                head_dim, page_size, sm_scale, max_seq_len, flags, stream);
}

extern "C" int adamas_decode_step(const void* q, const void* q_code, const void* kv_data,
                                  const void* code_data, const int32_t* page_indices,
                                  const int32_t* page_indptr, const int32_t* seq_lens,
                                  uint32_t budget, void* out, int32_t* sel_out, void* workspace,
                                  size_t workspace_bytes, uint32_t batch, uint32_t num_heads,
                                  uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size,
                                  float sm_scale, uint32_t max_seq_len, uint32_t page_table_stride,
                                  adamas_stream_t stream) {
  return adamas_decode_step_f(q, q_code, kv_data, code_data, page_indices, page_indptr, seq_lens,
                              budget, out, sel_out, workspace, workspace_bytes, batch, num_heads,
                              num_kv_heads, head_dim, page_size, sm_scale, max_seq_len,
                              page_table_stride, 0u, stream);
}

extern "C" int adamas_decode_layer_step(const void* qkv, const float* cos_table,
                                        const float* sin_table, void* kv_data, void* code_data,
                                        const int32_t* page_indices, const int32_t* page_indptr,
                                        const int32_t* seq_lens, uint32_t budget, void* out,
                                        int32_t* sel_out, void* workspace, size_t workspace_bytes,
                                        uint32_t batch, uint32_t num_heads, uint32_t num_kv_heads,
                                        uint32_t head_dim, uint32_t page_size, float sm_scale,
                                        uint32_t max_seq_len, uint32_t page_table_stride,
                                        float hadamard_scale, uint32_t flags,
                                        adamas_stream_t stream) {
  if (!qkv || !cos_table || !sin_table || !kv_data || !code_data) return ADAMAS_E_BADARG;
  if (flags & ~(ADAMAS_F_CODE_FROM_FP32 | ADAMAS_F_BF16 | ADAMAS_F_HND)) return ADAMAS_E_BADARG;
  if ((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(cos_table) |
       reinterpret_cast<uintptr_t>(sin_table)) & 15)
    return ADAMAS_E_ALIGN;
  QkvSource src;
  src.qkv = static_cast<const __half*>(qkv);
  src.cos_table = cos_table;
  src.sin_table = sin_table;
  src.scale = hadamard_scale;
  src.code_flags = flags;
  const uint32_t kv_flags = flags & (ADAMAS_F_BF16 | ADAMAS_F_HND);  // format and layout of the caches
  int rc = step_candidates_impl(nullptr, code_data, page_indices, page_indptr, seq_lens, budget,
                                workspace, workspace_bytes, batch, num_heads, num_kv_heads,
                                page_size, max_seq_len, page_table_stride, kv_flags, stream, &src);
  if (rc != 0) return rc;
  return step_attend_impl(nullptr, kv_data, code_data, page_indices, page_indptr, seq_lens, budget,
                          out, sel_out, workspace, workspace_bytes, batch, num_heads, num_kv_heads,
                          head_dim, page_size, sm_scale, max_seq_len, page_table_stride, kv_flags,
                          stream, &src);
}

// ---- the decode step for callers that cannot allocate ----------------------------------------------
// The workspace of adamas_decode_step_f lives in a file-scope device array instead of caller memory:
// every GPU the library runs on holds one copy of it (ADAMAS_STATIC_SCRATCH_BYTES) until the process
// ends.  In host code the array's name is only a handle: its device address is asked for once per
// device (hipGetSymbolAddress, with that device current) and kept; kernels receive that address as
// the workspace pointer, exactly as they receive a caller's buffer.  The array is zero at load, which
// is the state the split-merge arrival counters need; every kernel that uses a counter puts it back
// to zero, and candidates, histograms and partial sums are written before they are read within one
// call, so a call finds what it needs whatever the previous call (of any size) left behind.  Calls
// that overlap on one GPU (two streams, two threads) share the array and race.
static __device__ __align__(256) unsigned char scratch[ADAMAS_STATIC_SCRATCH_BYTES];

static int static_scratch_address(void** out) {
  static std::atomic<void*> per_device[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= 64) return ADAMAS_E_UNSUPPORTED;
  void* p = per_device[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    if (!p) return ADAMAS_E_SCRATCH;
    per_device[dev].store(p, std::memory_order_release);  // every thread finds the same address
  }
  *out = p;
  return 0;
}

extern "C" int adamas_decode_step_noalloc(const void* q, const void* q_code, const void* kv_data,
                                          const void* code_data, const int32_t* page_indices,
                                          const int32_t* page_indptr, const int32_t* seq_lens,
                                          uint32_t budget, void* out, int32_t* sel_out,
                                          uint32_t batch, uint32_t num_heads, uint32_t num_kv_heads,
                                          uint32_t head_dim, uint32_t page_size, float sm_scale,
                                          uint32_t max_seq_len, uint32_t page_table_stride,
                                          uint32_t flags, adamas_stream_t stream) {
  if (budget == 0 || max_seq_len == 0 || batch == 0 || num_heads == 0) return ADAMAS_E_BADARG;
  // sizes first: the product below must not wrap before it is compared with the limit
  if (batch > 65535 || num_heads > 65535 || max_seq_len > (1u << 24) || budget > (1u << 24))
    return ADAMAS_E_SCRATCH;
  const WorkspaceLayout w = workspace_layout(batch, num_heads, max_seq_len, budget);
  if (w.total > ADAMAS_STATIC_SCRATCH_BYTES) return ADAMAS_E_SCRATCH;
  void* ws = nullptr;
  const int rc = static_scratch_address(&ws);
  if (rc != 0) return rc;
  return adamas_decode_step_f(q, q_code, kv_data, code_data, page_indices, page_indptr, seq_lens,
                              budget, out, sel_out, ws, ADAMAS_STATIC_SCRATCH_BYTES, batch, num_heads,
                              num_kv_heads, head_dim, page_size, sm_scale, max_seq_len,
                              page_table_stride, flags, stream);
}
