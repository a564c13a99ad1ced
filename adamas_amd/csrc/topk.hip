// Row-wise selection of the k smallest 16-bit keys, ties to the lowest index (gfx950).
//
// The block-level algorithm lives in select.h (bisection on the key range with wave ballots, ranks
// from ballots; deterministic output order: items below the threshold by ascending index, then the
// tied items by ascending index).  This file wraps it into launches:
//
//   k <= 1024  rows of up to 32768 items are selected by one workgroup of 1024 threads (32 items per
//              lane, in registers).  Longer rows first go through one or more reduction levels:
//              grid (chunks, rows) of 256 threads, every workgroup selects the k smallest of its
//              chunk of 4096 items into a candidate list (the k smallest of a row are always among the
//              per-chunk winners; candidate lists keep the (below, tied) x ascending-index order per
//              chunk and chunks are concatenated in index order, so later levels see every class in
//              ascending index order as well).  Levels are separate launches: the kernel boundary
//              makes the candidates visible, no atomics or fences are involved.
//   k > 1024   one workgroup of 1024 threads per row streams the row once per bisection round.
//
// Integer keys (the distances of the estimator, ADAMAS_KEY_*_INT) with k <= 255 take the two-level
// scheme the fused decode step uses, given a workspace: a launch of one WAVE per chunk of 512-2048
// keys (threshold of the chunk from a histogram in LDS, 2048 waves for 32 rows of 32768) that writes
// a short list of the chunk's smallest keys, then one workgroup per row that reads the threshold off
// a histogram of the listed keys and goes back to the input for the rare chunk whose list ran out.
// Two short launches: 6.1 us for 32 rows of 32768 keys at k = 127, against 9.6 us with lists of the
// full k and 21 us for the bisection kernels; also faster than the single launch for short rows
// (4096 keys: 5.9 against 9.5 us).  Rows beyond 131072 keys keep lists of the full k and a histogram
// row per chunk (select_chunks_int_kernel, select_final_int_kernel).  Integer keys with a larger k
// take the histogram scheme at the end of this file: the same two launches, with plain 512-bin
// counts per chunk instead of candidate lists.
#include "chunk_select.h"
#include "select.h"
#include "workspace.h"

namespace adamas {

constexpr uint32_t kChunkedMaxK = 1024;
constexpr uint32_t kChunkItems = 4096;     // 256 threads x 16 items
constexpr uint32_t kFinalItems = 32768;    // 1024 threads x 32 items
constexpr uint32_t kMaxRowLen = 1u << 21;  // 2,097,152 elements
constexpr uint64_t kEmptyCand = ~0ull;     // candidate = (key << 48) | (raw << 32) | payload

struct SelectArgs {
  // source: a row of 16-bit values ...
  const uint16_t* values;
  int64_t row_stride;
  uint32_t n_max;
  const int32_t* seq_lens;
  uint32_t rows_per_seq;
  int32_t len_delta;
  const int32_t* in_idx;
  int64_t in_idx_stride;
  uint32_t vec_ok;
  // ... or the candidate slots of a row
  const uint64_t* cand_in;
  uint32_t n_in_slots;
  // selection
  uint32_t k;
  uint32_t key_mode;
  // destination: candidate lists [row][chunk][k] or the final outputs
  uint64_t* cand_out;
  int32_t* out_idx;
  uint16_t* out_vals;
  int64_t out_stride;
};

__device__ __forceinline__ uint32_t row_length(const SelectArgs& a, uint32_t row) {
  if (a.seq_lens == nullptr) return a.n_max;
  int32_t len = a.seq_lens[row / a.rows_per_seq] + a.len_delta;
  len = len < 0 ? 0 : len;
  return static_cast<uint32_t>(len) < a.n_max ? static_cast<uint32_t>(len) : a.n_max;
}

// keys of items e0..e0+7 of a row of values (n = row length)
__device__ __forceinline__ void load_value_keys(const uint16_t* vrow, uint32_t e0, uint32_t n,
                                                bool vec_ok, uint32_t key_mode, uint32_t* keys) {
  if (vec_ok && e0 + 8 <= n) {
    const uint4 v = *reinterpret_cast<const uint4*>(vrow + e0);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      keys[2 * i] = make_key(w[i] & 0xffffu, key_mode);
      keys[2 * i + 1] = make_key(w[i] >> 16, key_mode);
    }
  } else {
#pragma unroll
    for (int r = 0; r < 8; ++r)
      keys[r] = (e0 + r < n) ? make_key(vrow[e0 + r], key_mode) : kInvalidKey;
  }
}

__device__ __forceinline__ void load_cand_keys(const uint64_t* crow, uint32_t e0, uint32_t n,
                                               uint32_t* keys) {
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const uint64_t c = (e0 + r < n) ? crow[e0 + r] : kEmptyCand;
    keys[r] = (c == kEmptyCand) ? kInvalidKey : static_cast<uint32_t>(c >> 48);
  }
}

// grid (chunks, rows); every workgroup selects the k smallest of its chunk of kThreads*kItems items.
template <int kThreads, int kItems, bool kSrcCand, bool kDstCand>
__global__ __launch_bounds__(kThreads) void select_kernel(SelectArgs a) {
  constexpr int kWaves = kThreads / kWave;
  constexpr int kGroups = kItems / 8;
  __shared__ SelectScratch<kWaves> sh;
  const uint32_t chunk = blockIdx.x, n_chunks = gridDim.x, row = blockIdx.y;
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t chunk_base = chunk * (kThreads * kItems);

  const uint32_t n = kSrcCand ? a.n_in_slots : row_length(a, row);
  const uint16_t* vrow = kSrcCand ? nullptr : a.values + static_cast<int64_t>(row) * a.row_stride;
  const uint64_t* crow = kSrcCand ? a.cand_in + static_cast<size_t>(row) * a.n_in_slots : nullptr;

  uint32_t keys[kItems];
#pragma unroll
  for (int j = 0; j < kGroups; ++j) {
    const uint32_t e0 = chunk_base + block_item_index<kItems>(wave, lane, j, 0);
    if (kSrcCand) load_cand_keys(crow, e0, n, &keys[j * 8]);
    else load_value_keys(vrow, e0, n, a.vec_ok != 0, a.key_mode, &keys[j * 8]);
  }

  const SelectPlan plan =
      block_select_plan<kWaves, kItems>(keys, a.k, key_max_of(a.key_mode), sh);

  uint64_t* cdst =
      kDstCand ? a.cand_out + (static_cast<size_t>(row) * n_chunks + chunk) * a.k : nullptr;
  int32_t* idst = kDstCand ? nullptr : a.out_idx + static_cast<int64_t>(row) * a.out_stride;
  uint16_t* vdst = (kDstCand || !a.out_vals)
                       ? nullptr
                       : a.out_vals + static_cast<int64_t>(row) * a.out_stride;
  const int32_t* grow =
      (!kSrcCand && a.in_idx) ? a.in_idx + static_cast<int64_t>(row) * a.in_idx_stride : nullptr;

  block_select_emit<kWaves, kItems>(
      keys, plan, sh, [&](uint32_t pos, int j, int r) __attribute__((always_inline)) {
        const uint32_t e = chunk_base + block_item_index<kItems>(wave, lane, j, r);
        uint32_t raw, payload;
        if (kSrcCand) {
          const uint64_t c = crow[e];
          raw = static_cast<uint32_t>(c >> 32) & 0xffffu;
          payload = static_cast<uint32_t>(c);
        } else {
          raw = raw_of_key(keys[j * 8 + r], a.key_mode);  // no reload inside the emission loop
          payload = grow ? static_cast<uint32_t>(grow[e]) : e;
        }
        if (kDstCand) {
          cdst[pos] = (static_cast<uint64_t>((keys[j * 8 + r] << 16) | raw) << 32) | payload;
        } else {
          idst[pos] = static_cast<int32_t>(payload);
          if (vdst) vdst[pos] = static_cast<uint16_t>(raw);
        }
      });
  for (uint32_t i = plan.n_take + threadIdx.x; i < a.k; i += kThreads) {  // pad
    if (kDstCand) {
      cdst[i] = kEmptyCand;
    } else {
      idst[i] = -1;
      if (vdst) vdst[i] = 0;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// k > 1024: one workgroup per row, the row is streamed once per bisection round.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void select_stream_kernel(SelectArgs a) {
  constexpr int kWaves = 16;
  constexpr uint32_t kSlab = 1024 * 8;
  __shared__ SelectScratch<kWaves> sh;
  const uint32_t row = blockIdx.x;
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t n = row_length(a, row);
  const uint16_t* vrow = a.values + static_cast<int64_t>(row) * a.row_stride;
  const int32_t* grow = a.in_idx ? a.in_idx + static_cast<int64_t>(row) * a.in_idx_stride : nullptr;
  int32_t* idst = a.out_idx + static_cast<int64_t>(row) * a.out_stride;
  uint16_t* vdst = a.out_vals ? a.out_vals + static_cast<int64_t>(row) * a.out_stride : nullptr;
  const uint32_t n_slabs = (n + kSlab - 1) / kSlab;
  const uint32_t key_max = key_max_of(a.key_mode);
  const uint32_t k = a.k;
  uint32_t round = 0;

  auto count_le = [&](uint32_t bound) __attribute__((always_inline)) {
    uint32_t c = 0;
    for (uint32_t s = 0; s < n_slabs; ++s) {
      uint32_t keys[8];
      load_value_keys(vrow, s * kSlab + block_item_index<8>(wave, lane, 0, 0), n, a.vec_ok != 0,
                      a.key_mode, keys);
#pragma unroll
      for (int r = 0; r < 8; ++r) c += __popcll(__ballot(keys[r] <= bound));
    }
    const uint32_t slot = round & 1u;
    ++round;
    if (lane == 0) sh.cnt[slot][wave] = c;
    __syncthreads();
    uint32_t total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) total += sh.cnt[slot][w];
    return total;
  };

  SelectPlan plan;
  const uint32_t n_valid = count_le(key_max);
  if (n_valid <= k) {
    plan.thr = key_max + 1;
    plan.n_below = n_valid;
    plan.quota = 0;
    plan.n_take = n_valid;
  } else {
    uint32_t lo = 0, hi = key_max;
    while (lo < hi) {
      const uint32_t mid = (lo + hi) >> 1;
      if (count_le(mid) >= k) hi = mid;
      else lo = mid + 1;
    }
    plan.thr = lo;
    plan.n_below = lo == 0 ? 0u : count_le(lo - 1);
    plan.quota = k - plan.n_below;
    plan.n_take = k;
  }

  // Emission slab by slab.  block_select_emit numbers the below-class items of one slab from 0 and
  // the tied ones from n_below; the class counts of the earlier slabs shift both.
  uint32_t base_b = 0, base_e = 0;
  for (uint32_t s = 0; s < n_slabs; ++s) {
    uint32_t keys[8];
    const uint32_t slab_base = s * kSlab;
    load_value_keys(vrow, slab_base + block_item_index<8>(wave, lane, 0, 0), n, a.vec_ok != 0,
                    a.key_mode, keys);
    SelectPlan shifted = plan;
    shifted.n_below = plan.n_below + base_e;
    shifted.quota = plan.quota > base_e ? plan.quota - base_e : 0u;
    block_select_emit<kWaves, 8>(
        keys, shifted, sh, [&](uint32_t pos, int j, int r) __attribute__((always_inline)) {
          const uint32_t e = slab_base + block_item_index<8>(wave, lane, j, r);
          const uint32_t out_pos = (keys[r] == plan.thr) ? pos : pos + base_b;
          idst[out_pos] = grow ? grow[e] : static_cast<int32_t>(e);
          if (vdst) vdst[out_pos] = static_cast<uint16_t>(raw_of_key(keys[r], a.key_mode));
        });
    uint32_t tb = 0, te = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      tb += sh.below[w];
      te += sh.equal[w];
    }
    base_b += tb;
    base_e += te;
    __syncthreads();  // sh.below / sh.equal are rewritten by the next slab
  }
  for (uint32_t i = plan.n_take + threadIdx.x; i < k; i += 1024) {
    idst[i] = -1;
    if (vdst) vdst[i] = 0;
  }
}

inline uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

// ---- integer keys, two levels (chunk_select.h) ----------------------------------------------------
constexpr uint32_t kHistSchemeMaxRowLen = 131072;  // rows the chip-wide histogram emission serves
constexpr int kIntWaves = 8;            // chunks per workgroup of level 1
constexpr uint32_t kIntMaxK = 255;
constexpr uint32_t kIntMaxSlots = 16384;  // candidate slots per row level 2 can hold

struct IntLayout {
  uint32_t ok;            // 1: the two-level path serves these sizes
  uint32_t items;         // keys per lane at level 1: 8, 16 or 32
  uint32_t chunk;         // keys per chunk = 64 * items
  uint32_t n_chunks;
  uint32_t cand_stride;   // k rounded up to a multiple of 8
  size_t cand_bytes, hist_bytes;
};

static IntLayout int_layout(uint32_t num_rows, uint32_t n_max, uint32_t k) {
  IntLayout L{};
  L.cand_stride = (k + 7) / 8 * 8;
  if (k == 0 || k > kIntMaxK || n_max <= kChunkItems) return L;
  for (uint32_t items = 8; items <= 32; items *= 2) {
    L.items = items;
    L.chunk = 64 * items;
    L.n_chunks = ceil_div(n_max, L.chunk);
    if (static_cast<uint64_t>(L.n_chunks) * L.cand_stride <= kIntMaxSlots) {
      L.ok = 1;
      break;
    }
  }
  // more than 8192 candidate slots per row make the final pass slower than the histogram scheme
  // (15.6 against 12 us at 32768 keys and k = 255): those sizes go there, as long as it serves them
  if (L.ok && n_max <= kHistSchemeMaxRowLen &&
      static_cast<uint64_t>(L.n_chunks) * L.cand_stride > 8192)
    L.ok = 0;
  if (!L.ok) return L;
  L.cand_bytes = (static_cast<size_t>(num_rows) * L.n_chunks * L.cand_stride * 8 + 255) / 256 * 256;
  L.hist_bytes = (static_cast<size_t>(num_rows) * L.n_chunks * kHistBins + 255) / 256 * 256;
  return L;
}

// level 1: grid (ceil(n_chunks / 8), rows), 512 threads; wave w takes chunk blockIdx.x * 8 + w
// kKeyMode: as for select_hist_emit_kernel (>= 0: format fixed at compile time, aligned rows)
template <int kItems, int kKeyMode>
__global__ __launch_bounds__(kIntWaves* kWave) void select_chunks_int_kernel(
    SelectArgs a, uint64_t* __restrict__ cand, unsigned char* __restrict__ hist, uint32_t n_chunks,
    uint32_t cand_stride) {
  const uint32_t key_mode = kKeyMode >= 0 ? static_cast<uint32_t>(kKeyMode) : a.key_mode;
  const bool vec_ok = kKeyMode >= 0 || a.vec_ok != 0;
  __shared__ alignas(16) uint32_t hist_lds[kIntWaves][kChunkHistWords];
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t row = blockIdx.y;
  const uint32_t chunk = blockIdx.x * kIntWaves + static_cast<uint32_t>(wave);
  if (chunk >= n_chunks) return;  // whole waves leave; nothing below synchronises the workgroup
  constexpr uint32_t kChunk = kWave * kItems;
  const uint32_t chunk_base = chunk * kChunk;
  const uint32_t n = row_length(a, row);
  uint64_t* dst = cand + (static_cast<size_t>(row) * n_chunks + chunk) * cand_stride;
  uint2* hrow =
      reinterpret_cast<uint2*>(hist + (static_cast<size_t>(row) * n_chunks + chunk) * kHistBins) + lane;
  if (chunk_base >= n) {
    for (uint32_t i = lane; i < cand_stride; i += kWave) dst[i] = kEmptyCand64;
    *hrow = make_uint2(0u, 0u);
    return;
  }
  const uint16_t* vrow = a.values + static_cast<int64_t>(row) * a.row_stride;
  uint32_t keys[kItems];
#pragma unroll
  for (int j = 0; j < kItems / 8; ++j)
    load_value_keys(vrow, chunk_base + static_cast<uint32_t>(lane) * kItems + j * 8, n,
                    vec_ok, key_mode, &keys[j * 8]);
  const int32_t* irow =
      a.in_idx ? a.in_idx + static_cast<int64_t>(row) * a.in_idx_stride : nullptr;
  chunk_select_emit<kItems>(keys, min(kChunk, n - chunk_base), a.k, cand_stride, dst, hrow,
                            hist_lds[wave], [&](uint32_t item, int) __attribute__((always_inline)) {
                              const uint32_t e = chunk_base + item;
                              return irow ? static_cast<uint32_t>(irow[e]) : e;
                            });
}

struct IntFinalShared {
  FinalSelectShared sel;
  int32_t idx[kIntMaxK + 1];
  uint16_t val[kIntMaxK + 1];
};

// level 2: grid (rows), 512 threads
template <int kGroups>
__global__ __launch_bounds__(kFinalThreads) void select_final_int_kernel(
    SelectArgs a, const uint64_t* __restrict__ cand, const unsigned char* __restrict__ hist,
    uint32_t n_chunks, uint32_t cand_stride) {
  __shared__ IntFinalShared sh;
  const uint32_t row = blockIdx.x;
  const uint32_t n_slots = n_chunks * cand_stride;
  const bool as_half = a.key_mode == ADAMAS_KEY_FP16_INT;
  const uint32_t n_take = final_select<kGroups>(
      cand + static_cast<size_t>(row) * n_slots, n_slots,
      hist + static_cast<size_t>(row) * n_chunks * kHistBins, n_chunks, a.k, cand_stride, sh.sel,
      [&](uint32_t pos, uint32_t, uint32_t, uint32_t key, uint32_t payload)
          __attribute__((always_inline)) {
            sh.idx[pos] = static_cast<int32_t>(payload);
            // the key in the format of the input: integer keys are their own value
            sh.val[pos] = as_half ? __half_as_ushort(__float2half_rn(static_cast<float>(key)))
                                  : static_cast<uint16_t>(key);
          },
      []() {});
  __syncthreads();
  int32_t* oi = a.out_idx + static_cast<int64_t>(row) * a.out_stride;
  uint16_t* ov = a.out_vals ? a.out_vals + static_cast<int64_t>(row) * a.out_stride : nullptr;
  for (uint32_t i = threadIdx.x; i < a.k; i += kFinalThreads) {
    oi[i] = i < n_take ? sh.idx[i] : -1;
    if (ov) ov[i] = i < n_take ? sh.val[i] : static_cast<uint16_t>(0);
  }
}

// ---- integer keys, k <= 255, rows of up to 131072 keys: short candidate lists ------------------------
// The scheme of the fused decode step (fused_step.hip).  Level 1: one wave per chunk of 512 - 2048
// keys (at most 64 chunks per row) writes the kc = 16 .. 256 smallest keys of its chunk, ties to the
// lowest index: a chunk holds k / chunks of the selection on average, so lists of the full k would be
// mostly padding (64 x 128 slots for 127 winners).  Level 2: one workgroup per row builds a histogram
// of the listed keys in LDS, reads threshold and tie quota off it and ranks the listed candidates
// with prefix scans.  A list is a prefix of its chunk in (key, index) order: if its last entry is not
// selected, nothing the chunk left out can be.  If it is, and the chunk holds more keys than the
// list, the workgroup takes that chunk's keys from the input row again and selects among all of them,
// so the result is exact for any input (at most k / kc chunks can need that).
constexpr uint32_t kCapMaxChunks = 64;       // the flags of all chunks fit one ballot
constexpr uint32_t kCapMaxRowLen = kCapMaxChunks * 2048;
constexpr uint32_t kCapSlots = 2 * kFinalThreads;  // candidate slots per row: two per thread of level 2

struct CapLayout {
  uint32_t ok;
  uint32_t items;      // keys per lane at level 1: 8, 16 or 32
  uint32_t n_chunks;   // <= kCapMaxChunks
  uint32_t kc, kc_log2;
  size_t cand_bytes;
};

static CapLayout cap_layout(uint32_t num_rows, uint32_t n_max, uint32_t k) {
  CapLayout L{};
  if (k == 0 || k > kIntMaxK || n_max == 0 || n_max > kCapMaxRowLen) return L;
  L.items = 8;
  while (ceil_div(n_max, kWave * L.items) > kCapMaxChunks) L.items *= 2;
  L.n_chunks = ceil_div(n_max, kWave * L.items);
  L.kc = std::max(8u, std::min(pow2_floor(kCapSlots / L.n_chunks), pow2_ceil(k)));
  while ((1u << L.kc_log2) < L.kc) ++L.kc_log2;
  L.cand_bytes = (static_cast<size_t>(num_rows) * L.n_chunks * L.kc * 8 + 255) / 256 * 256;
  L.ok = 1;
  return L;
}

// level 1: grid (ceil(n_chunks / 8), rows), 512 threads; wave w takes chunk blockIdx.x * 8 + w
template <int kItems, int kKeyMode>
__global__ __launch_bounds__(kIntWaves* kWave) void select_chunks_capped_kernel(
    SelectArgs a, uint64_t* __restrict__ cand, uint32_t n_chunks, uint32_t kc) {
  const uint32_t key_mode = kKeyMode >= 0 ? static_cast<uint32_t>(kKeyMode) : a.key_mode;
  const bool vec_ok = kKeyMode >= 0 || a.vec_ok != 0;
  __shared__ alignas(16) uint32_t hist_lds[kIntWaves][kChunkHistWords];
  __shared__ alignas(16) uint32_t key_lds[kIntWaves][kWave * kItems / 2];  // two keys per word
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t row = blockIdx.y;
  const uint32_t chunk = blockIdx.x * kIntWaves + static_cast<uint32_t>(wave);
  if (chunk >= n_chunks) return;  // whole waves leave; nothing below synchronises the workgroup
  constexpr uint32_t kChunk = kWave * kItems;
  const uint32_t chunk_base = chunk * kChunk;
  const uint32_t n = row_length(a, row);
  uint64_t* dst = cand + (static_cast<size_t>(row) * n_chunks + chunk) * kc;
  if (chunk_base >= n) {
    for (uint32_t i = lane; i < kc; i += kWave) dst[i] = kEmptyCand64;
    return;
  }
  const uint16_t* vrow = a.values + static_cast<int64_t>(row) * a.row_stride;
  uint32_t keys[kItems];
#pragma unroll
  for (int j = 0; j < kItems / 8; ++j)
    load_value_keys(vrow, chunk_base + static_cast<uint32_t>(lane) * kItems + j * 8, n,
                    vec_ok, key_mode, &keys[j * 8]);
  // a listed key is picked by a run-time index: the keys of the chunk go to LDS, item order
  // (the LDS operations of one wave are carried out in order, so the wave reads them back below
  // without a barrier)
  uint32_t* kl = key_lds[wave] + lane * (kItems / 2);
#pragma unroll
  for (int j = 0; j < kItems / 8; ++j)
    *reinterpret_cast<uint4*>(kl + 4 * j) =
        make_uint4((keys[8 * j] & 0xffffu) | (keys[8 * j + 1] << 16),
                   (keys[8 * j + 2] & 0xffffu) | (keys[8 * j + 3] << 16),
                   (keys[8 * j + 4] & 0xffffu) | (keys[8 * j + 5] << 16),
                   (keys[8 * j + 6] & 0xffffu) | (keys[8 * j + 7] << 16));
  const int32_t* irow =
      a.in_idx ? a.in_idx + static_cast<int64_t>(row) * a.in_idx_stride : nullptr;
  const uint16_t* kl16 = reinterpret_cast<const uint16_t*>(key_lds[wave]);
  chunk_select_capped<kItems, true>(
      keys, kc, dst, hist_lds[wave],
      [&](uint32_t item) __attribute__((always_inline)) -> uint32_t { return kl16[item]; },
      [&](uint32_t item) __attribute__((always_inline)) -> uint32_t {
        const uint32_t e = chunk_base + item;
        return irow ? static_cast<uint32_t>(irow[e]) : e;
      });
}

struct CapFinalShared {
  alignas(16) uint32_t hist[kHistBins];      // listed candidates per key value
  alignas(16) uint32_t wclass[kFinalWaves];  // per-wave class totals of the rank scan: below | tied << 16
  uint32_t flag[kCapMaxChunks];              // chunks whose list ran out (taken from the row again)
  uint32_t any_flag;
  uint32_t fb[kCapMaxChunks], ft[kCapMaxChunks];  // their keys below / equal to the threshold
  uint32_t tbase[kCapMaxChunks];             // tied list entries of all chunks before them
  uint32_t bbase[kCapMaxChunks];             // list entries below the threshold of all chunks before them
  int32_t idx[kIntMaxK + 1];
  uint16_t val[kIntMaxK + 1];
};

// level 2: grid (rows), 512 threads, two candidate slots per thread
__global__ __launch_bounds__(kFinalThreads) void select_final_capped_kernel(
    SelectArgs a, const uint64_t* __restrict__ cand, uint32_t n_chunks, uint32_t kc_log2,
    uint32_t chunk_keys) {
  static_assert(kFinalThreads == kHistBins, "one thread per key value");
  static_assert(kFinalWaves == 8, "two 128-bit reads cover the wave totals");
  static_assert(kCapMaxChunks == kWave, "the flags of all chunks fit one ballot");
  __shared__ CapFinalShared sh;
  const uint32_t row = blockIdx.x;
  const uint32_t tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t kc = 1u << kc_log2;
  const uint32_t n_slots = n_chunks << kc_log2;
  const uint64_t* crow = cand + static_cast<size_t>(row) * n_slots;
  const uint32_t slot0 = 2u * tid;
  const bool have = slot0 < n_slots;
  uint4 raw = make_uint4(~0u, ~0u, ~0u, ~0u);  // an unused slot is all ones
  if (have) raw = *reinterpret_cast<const uint4*>(crow + slot0);
  const uint32_t n = row_length(a, row);
  const uint32_t k = a.k;
  sh.hist[tid] = 0u;
  if (tid < kCapMaxChunks) sh.flag[tid] = 0u;
  if (tid == 0) sh.any_flag = 0u;
  // a candidate is (key << 48) | (item index in its chunk << 32) | payload
  uint32_t key[2] = {raw.y >> 16, raw.w >> 16};  // an unused slot reads 0xffff: above every threshold
  const uint32_t pay[2] = {raw.x, raw.z};
  const uint32_t chunk_mine = slot0 >> kc_log2;
  __syncthreads();  // the histogram is cleared
#pragma unroll
  for (int i = 0; i < 2; ++i)
    if (key[i] < static_cast<uint32_t>(kHistBins)) atomicAdd(&sh.hist[key[i]], 1u);
  __syncthreads();  // the histogram is complete
  WavePlan plan = wave_plan_from_hist(sh.hist, k);  // every wave for itself
  uint32_t rb, re;
  auto rank_slots = [&]() __attribute__((always_inline)) {
    uint32_t mine = 0;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      mine += (key[i] < plan.thr ? 1u : 0u) + ((key[i] == plan.thr ? 1u : 0u) << 16);
    const uint32_t incl = wave_inclusive_scan_dpp(mine);
    if (lane == kWave - 1) sh.wclass[wave] = incl;
    __syncthreads();
    const uint4 lo = *reinterpret_cast<const uint4*>(&sh.wclass[0]);
    const uint4 hi = *reinterpret_cast<const uint4*>(&sh.wclass[4]);
    const uint32_t t[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    uint32_t before = 0;  // the 16-bit fields cannot carry: at most 1024 slots
#pragma unroll
    for (int w = 0; w < 8; ++w) before += w < wave ? t[w] : 0u;
    const uint32_t excl = before + incl - mine;
    rb = excl & 0xffffu;
    re = excl >> 16;
  };
  const bool as_half = a.key_mode == ADAMAS_KEY_FP16_INT;
  auto put = [&](uint32_t pos, uint32_t kv, uint32_t payload) __attribute__((always_inline)) {
    sh.idx[pos] = static_cast<int32_t>(payload);
    // the key in the format of the input: integer keys are their own value
    sh.val[pos] = as_half ? __half_as_ushort(__float2half_rn(static_cast<float>(kv)))
                          : static_cast<uint16_t>(kv);
  };
  auto emit_slots = [&](uint32_t below_shift, uint32_t tie_shift) __attribute__((always_inline)) -> bool {
    uint32_t pb = rb + below_shift, pe = re + tie_shift;
    bool last_selected = false;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const bool is_b = key[i] < plan.thr, is_e = key[i] == plan.thr;
      const bool take = is_b || (is_e && pe < plan.quota);
      if (take) put(is_b ? pb : plan.n_below + pe, key[i], pay[i]);
      pb += is_b ? 1u : 0u;
      pe += is_e ? 1u : 0u;
      last_selected = take;
    }
    return last_selected;
  };
  auto chunk_len = [&](uint32_t c) __attribute__((always_inline)) -> uint32_t {
    const uint32_t t0 = c * chunk_keys;
    return t0 < n ? min(chunk_keys, n - t0) : 0u;
  };
  rank_slots();
  {
    const bool last_selected = emit_slots(0u, 0u);
    if (last_selected && ((slot0 + 1u) & (kc - 1u)) == kc - 1u && chunk_len(chunk_mine) > kc) {
      sh.flag[chunk_mine] = 1u;
      sh.any_flag = 1u;
    }
  }
  __syncthreads();  // the output list is complete, or some chunk is flagged

  if (sh.any_flag) {
    const uint16_t* vrow = a.values + static_cast<int64_t>(row) * a.row_stride;
    const int32_t* irow =
        a.in_idx ? a.in_idx + static_cast<int64_t>(row) * a.in_idx_stride : nullptr;
    const uint32_t key_mode = a.key_mode;
    const uint64_t fmask = __ballot(sh.flag[lane] != 0u);  // the same in every wave
    const bool mine_flagged = have && ((fmask >> chunk_mine) & 1ull) != 0;
    if (mine_flagged) {  // the listed entries of such a chunk leave the count: its keys come back below
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (key[i] < static_cast<uint32_t>(kHistBins)) atomicSub(&sh.hist[key[i]], 1u);
        key[i] = 0xffffu;
      }
    }
    for (uint64_t m = fmask; m; m &= m - 1) {
      const uint32_t c = static_cast<uint32_t>(__ffsll(static_cast<long long>(m)) - 1);
      const uint32_t t0 = c * chunk_keys, len = chunk_len(c);
      for (uint32_t t = tid; t < len; t += kFinalThreads)
        atomicAdd(&sh.hist[make_key(vrow[t0 + t], key_mode)], 1u);
    }
    __syncthreads();  // counts complete
    plan = wave_plan_from_hist(sh.hist, k);
    // wave w counts the keys below / equal to the new threshold in the flagged chunks w, w+8, ...
    {
      uint32_t f = 0;
      for (uint64_t m = fmask; m; m &= m - 1, ++f) {
        if ((f & (kFinalWaves - 1)) != static_cast<uint32_t>(wave)) continue;
        const uint32_t c = static_cast<uint32_t>(__ffsll(static_cast<long long>(m)) - 1);
        const uint32_t t0 = c * chunk_keys, len = chunk_len(c);
        uint32_t cb = 0, ce = 0;
        for (uint32_t t = 0; t < len; t += kWave) {
          const uint32_t d = t + lane < len ? make_key(vrow[t0 + t + lane], key_mode) : 0xffffu;
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
    // listed entries of all chunks in front of a flagged chunk: what its first slot's thread counted
    if (mine_flagged && (slot0 & (kc - 1u)) == 0u) {
      sh.tbase[chunk_mine] = re;
      sh.bbase[chunk_mine] = rb;
    }
    // keys of flagged chunks in front of this thread's chunk, by class
    uint32_t tie_shift = 0, below_shift = 0;
    for (uint64_t m = have ? fmask & ((1ull << chunk_mine) - 1ull) : 0ull; m; m &= m - 1) {
      const int fc = __ffsll(static_cast<long long>(m)) - 1;
      tie_shift += sh.ft[fc];
      below_shift += sh.fb[fc];
    }
    __syncthreads();
    emit_slots(below_shift, tie_shift);
    // the flagged chunks, walked in index order by their waves: every key takes the rank its index
    // gives it within its class, among listed entries and keys of flagged chunks alike
    {
      uint32_t f = 0, bb = 0, tb = 0;
      for (uint64_t m = fmask; m; m &= m - 1, ++f) {
        const uint32_t c = static_cast<uint32_t>(__ffsll(static_cast<long long>(m)) - 1);
        if ((f & (kFinalWaves - 1)) == static_cast<uint32_t>(wave)) {
          const uint32_t t0 = c * chunk_keys, len = chunk_len(c);
          uint32_t pb = sh.bbase[c] + bb, pe = sh.tbase[c] + tb;
          for (uint32_t t = 0; t < len; t += kWave) {
            const uint32_t e = t0 + t + lane;
            const uint32_t d = t + lane < len ? make_key(vrow[e], key_mode) : 0xffffu;
            const uint64_t mb = __ballot(d < plan.thr), me = __ballot(d == plan.thr);
            const uint32_t r_e = pe + lanes_below(me);
            const bool is_b = d < plan.thr;
            if (is_b || (d == plan.thr && r_e < plan.quota))
              put(is_b ? pb + lanes_below(mb) : plan.n_below + r_e, d,
                  irow ? static_cast<uint32_t>(irow[e]) : e);
            pb += __popcll(mb);
            pe += __popcll(me);
          }
        }
        bb += sh.fb[c];
        tb += sh.ft[c];
      }
    }
    __syncthreads();  // the output list is complete
  }
  const uint32_t n_take = plan.n_take;
  int32_t* oi = a.out_idx + static_cast<int64_t>(row) * a.out_stride;
  uint16_t* ov = a.out_vals ? a.out_vals + static_cast<int64_t>(row) * a.out_stride : nullptr;
  for (uint32_t i = tid; i < k; i += kFinalThreads) {
    oi[i] = i < n_take ? sh.idx[i] : -1;
    if (ov) ov[i] = i < n_take ? sh.val[i] : static_cast<uint16_t>(0);
  }
}

// ---- integer keys, any k: chunk histograms, then threshold and emission ------------------------------
// Integer keys take 512 values, so the k-th smallest key of a row can be read off a histogram instead
// of being searched for.  Level 1 (one wave per chunk of 1024 keys, the row spread over many CUs)
// counts the keys of its chunk with LDS atomics - 1024 per wave, which is cheap, unlike a whole row in
// one workgroup - and writes a 512-bin row of 16-bit counts.  Level 2 (one workgroup of 1024 threads
// per row) sums the chunk rows, takes the threshold and the tie quota from the prefix sum and walks
// over the row once to emit: items below the threshold by ascending index, then the tied ones.
constexpr int kHistWaves = 8;                         // chunks per workgroup of level 1
constexpr int kHistItems = 16;                        // keys per lane
constexpr uint32_t kHistChunk = kWave * kHistItems;   // 1024 keys per chunk
constexpr uint32_t kHistRowBytes = kHistBins * 2;     // one chunk's counts

// kKeyMode: as for select_hist_emit_kernel (>= 0: format fixed at compile time, aligned rows)
template <int kKeyMode>
__global__ __launch_bounds__(kHistWaves* kWave) void hist_chunks_int_kernel(
    SelectArgs a, uint16_t* __restrict__ hist, uint32_t n_chunks) {
  const uint32_t key_mode = kKeyMode >= 0 ? static_cast<uint32_t>(kKeyMode) : a.key_mode;
  const bool vec_ok = kKeyMode >= 0 || a.vec_ok != 0;
  __shared__ uint32_t h[kHistWaves][kHistBins / 2];  // two 16-bit bins per word
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t row = blockIdx.y;
  const uint32_t chunk = blockIdx.x * kHistWaves + static_cast<uint32_t>(wave);
  if (chunk >= n_chunks) return;  // whole waves leave; nothing below synchronises the workgroup
  uint32_t* hw = h[wave];
  *reinterpret_cast<uint4*>(&hw[4 * lane]) = make_uint4(0u, 0u, 0u, 0u);
  const uint32_t chunk_base = chunk * kHistChunk;
  const uint32_t n = row_length(a, row);
  if (chunk_base < n) {
    const uint16_t* vrow = a.values + static_cast<int64_t>(row) * a.row_stride;
    uint32_t keys[kHistItems];
#pragma unroll
    for (int j = 0; j < kHistItems / 8; ++j)
      load_value_keys(vrow, chunk_base + static_cast<uint32_t>(lane) * kHistItems + j * 8, n,
                      vec_ok, key_mode, &keys[j * 8]);
#pragma unroll
    for (int i = 0; i < kHistItems; ++i)  // a bin holds at most 1024 entries: no carry into its neighbour
      if (keys[i] != kInvalidKey) atomicAdd(&hw[keys[i] >> 1], 1u << (16 * (keys[i] & 1u)));
  }
  // the LDS operations of one wave are carried out in order: the counts are complete here
  uint4* dst = reinterpret_cast<uint4*>(
      reinterpret_cast<unsigned char*>(hist) +
      (static_cast<size_t>(row) * n_chunks + chunk) * kHistRowBytes);
  dst[lane] = *reinterpret_cast<const uint4*>(&hw[4 * lane]);
}

struct HistFinalShared {
  uint32_t part[16][kHistBins];  // partial sums of the chunk rows (32 KB)
  uint32_t wtot[8];
  uint32_t wclass[16];  // per-wave class totals of a slab: below | tied << 16
  SelectPlan plan;
};

__global__ __launch_bounds__(1024) void select_hist_final_kernel(SelectArgs a,
                                                                 const uint16_t* __restrict__ hist,
                                                                 uint32_t n_chunks) {
  constexpr int kWaves = 16;
  constexpr int kItems = 32;
  constexpr uint32_t kSlab = 1024 * kItems;
  __shared__ HistFinalShared sh;
  const uint32_t row = blockIdx.x;
  const uint32_t tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t n = row_length(a, row);
  const uint32_t k = a.k;
  const uint16_t* vrow = a.values + static_cast<int64_t>(row) * a.row_stride;
  const int32_t* grow = a.in_idx ? a.in_idx + static_cast<int64_t>(row) * a.in_idx_stride : nullptr;
  int32_t* idst = a.out_idx + static_cast<int64_t>(row) * a.out_stride;
  uint16_t* vdst = a.out_vals ? a.out_vals + static_cast<int64_t>(row) * a.out_stride : nullptr;

  // the keys of the first slab are asked for before anything else: they arrive while the threshold
  // is worked out (thread t holds the 32 consecutive keys t*32 .. t*32+31 of a slab)
  uint32_t keys[kItems];
#pragma unroll
  for (int j = 0; j < kItems / 8; ++j)
    load_value_keys(vrow, tid * kItems + j * 8, n, a.vec_ok != 0, a.key_mode, &keys[j * 8]);

  // ---- count[v] over the chunks: thread (part, seg) adds bins 8*seg .. 8*seg+7 of the chunk rows
  // part, part + 16, ... (one 128-bit load per row), then the 16 parts are folded through LDS
  {
    const uint32_t part = tid >> 6, seg = tid & 63u;
    const unsigned char* hb = reinterpret_cast<const unsigned char*>(hist) +
                              static_cast<size_t>(row) * n_chunks * kHistRowBytes + seg * 16u;
    uint32_t acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (uint32_t c0 = part; c0 < n_chunks; c0 += 64) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t c = c0 + 16u * u;
        v[u] = c < n_chunks
                   ? *reinterpret_cast<const uint4*>(hb + static_cast<size_t>(c) * kHistRowBytes)
                   : make_uint4(0u, 0u, 0u, 0u);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[2 * j] += w[j] & 0xffffu;
          acc[2 * j + 1] += w[j] >> 16;
        }
      }
    }
    uint4* dstp = reinterpret_cast<uint4*>(&sh.part[part][seg * 8u]);
    dstp[0] = make_uint4(acc[0], acc[1], acc[2], acc[3]);
    dstp[1] = make_uint4(acc[4], acc[5], acc[6], acc[7]);
  }
  __syncthreads();
  // ---- prefix sum over the 512 bins (the first eight waves, one thread per bin) -> the plan
  uint32_t count = 0, incl = 0;
  if (tid < kHistBins) {
#pragma unroll
    for (int p = 0; p < 16; ++p) count += sh.part[p][tid];
    incl = wave_inclusive_scan_dpp(count);
    if (lane == kWave - 1) sh.wtot[wave] = incl;
  }
  __syncthreads();
  if (tid < kHistBins) {
    uint32_t cum = incl;
    for (int w = 0; w < wave; ++w) cum += sh.wtot[w];
    if (cum >= k && cum - count < k) {  // exactly one bin holds the k-th smallest key
      sh.plan.thr = tid;
      sh.plan.n_below = cum - count;
      sh.plan.quota = k - (cum - count);
      sh.plan.n_take = k;
    }
    if (tid == kHistBins - 1 && cum < k) {  // fewer valid keys than k: all of them are taken
      sh.plan.thr = kHistBins;
      sh.plan.n_below = cum;
      sh.plan.quota = 0;
      sh.plan.n_take = cum;
    }
  }
  __syncthreads();
  const SelectPlan plan = sh.plan;

  // ---- emission, slab by slab: ranks come from class masks and DPP prefix scans (chunk_select.h), the class counts of the
  // earlier waves and slabs shift the positions
  uint32_t base_b = 0, base_e = 0;
  for (uint32_t slab_base = 0; slab_base < n; slab_base += kSlab) {
    const uint32_t e0 = slab_base + tid * kItems;
    if (slab_base != 0) {
#pragma unroll
      for (int j = 0; j < kItems / 8; ++j)
        load_value_keys(vrow, e0 + j * 8, n, a.vec_ok != 0, a.key_mode, &keys[j * 8]);
    }
    uint32_t below[kItems / 4], equal[kItems / 4];
    raw_class_masks<kItems>(keys, plan.thr, below, equal);
    uint32_t total;
    const uint32_t excl = lane_scan<kItems / 4>(below, equal, total);  // below | tied << 16
    if (lane == 0) sh.wclass[wave] = total;
    __syncthreads();
    uint32_t before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      before += w < wave ? sh.wclass[w] : 0u;
      all += sh.wclass[w];
    }
    lane_emit<kItems / 4>(below, equal, plan.n_below, plan.quota,
                          base_b + (before & 0xffffu) + (excl & 0xffffu),
                          base_e + (before >> 16) + (excl >> 16),
                          [&](uint32_t pos, int i) __attribute__((always_inline)) {
                            const uint32_t e = e0 + i;
                            idst[pos] = grow ? grow[e] : static_cast<int32_t>(e);
                            // the value comes from the key: no reload inside the emission loop
                            if (vdst)
                              vdst[pos] = static_cast<uint16_t>(raw_of_key(keys[i], a.key_mode));
                          });
    base_b += all & 0xffffu;
    base_e += all >> 16;
    if (slab_base + kSlab < n) __syncthreads();  // sh.wclass is rewritten by the next slab
  }
  for (uint32_t i = plan.n_take + tid; i < k; i += 1024) {
    idst[i] = -1;
    if (vdst) vdst[i] = 0;
  }
}

// Level 2 for rows of moderate length, spread over the chip: grid (rows, slabs of 4096 keys), 256
// threads.  Rows are the fast grid dimension: workgroups are dealt to the eight dies by their linear
// id, so with 8 | rows all slabs of a row run on one die and its chunk rows are fetched into that
// die's L2 once instead of once per die (32 rows x 32768 keys: 1.0 us less than slabs first).  Every workgroup works the threshold out for itself from the chunk rows (they are small
// and sit in L2), adding up on the side the rows of the chunks BEFORE its slab: those give the number
// of selected items that precede the slab, i.e. where its own items go.  Then it emits the selected
// ones among its 4096 keys.  The same output order as select_hist_final_kernel.
constexpr int kEmitThreads = 256;
constexpr int kEmitItems = 16;
constexpr uint32_t kEmitSlab = kEmitThreads * kEmitItems;             // 4096 keys
constexpr uint32_t kEmitMaxRowLen = kHistSchemeMaxRowLen;  // longer rows: one workgroup per row

struct HistEmitShared {
  uint32_t all[4][kHistBins];  // partial sums over all chunks
  uint32_t pre[4][kHistBins];  // partial sums over the chunks before the slab
  uint32_t wtot[4], wpre[4], wclass[4];
  uint32_t pre_tied;
  SelectPlan plan;
};

// chunks_per_slab: histogram rows per 4096 keys (4 for chunks of 1024 keys, 8 for chunks of 512).
// kKeyMode >= 0: the key format is known at compile time and the rows are read with 128-bit loads
// (the caller has checked their alignment); -1: both are taken from the arguments.  The instances
// with a fixed format leave out the element-wise loads and the other formats' conversions, which
// are most of the code of the general one.
template <int kKeyMode>
__global__ __launch_bounds__(kEmitThreads) void select_hist_emit_kernel(
    SelectArgs a, const uint16_t* __restrict__ hist, uint32_t n_chunks, uint32_t chunks_per_slab) {
  const uint32_t key_mode = kKeyMode >= 0 ? static_cast<uint32_t>(kKeyMode) : a.key_mode;
  const bool vec_ok = kKeyMode >= 0 || a.vec_ok != 0;
  constexpr int kWaves = kEmitThreads / kWave;
  __shared__ HistEmitShared sh;
  const uint32_t row = blockIdx.x, slab = blockIdx.y;
  const uint32_t tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t n = row_length(a, row);
  const uint32_t k = a.k;
  const uint32_t slab_base = slab * kEmitSlab;
  if (slab_base >= n && slab != 0) return;  // nothing of this row here (slab 0 writes the padding)
  const uint16_t* vrow = a.values + static_cast<int64_t>(row) * a.row_stride;
  const int32_t* grow = a.in_idx ? a.in_idx + static_cast<int64_t>(row) * a.in_idx_stride : nullptr;
  int32_t* idst = a.out_idx + static_cast<int64_t>(row) * a.out_stride;
  uint16_t* vdst = a.out_vals ? a.out_vals + static_cast<int64_t>(row) * a.out_stride : nullptr;

  // thread t holds the 16 consecutive keys t*16 .. t*16+15 of the slab; asked for first
  const uint32_t e0 = slab_base + tid * kEmitItems;
  uint32_t keys[kEmitItems];
#pragma unroll
  for (int j = 0; j < kEmitItems / 8; ++j)
    load_value_keys(vrow, e0 + j * 8, n, vec_ok, key_mode, &keys[j * 8]);

  // ---- chunk rows: thread (part, seg) adds bins 8*seg .. 8*seg+7 of rows part, part + 4, ...
  {
    const uint32_t part = tid >> 6, seg = tid & 63u;
    const uint32_t c_first = slab * chunks_per_slab;  // chunks below it precede the slab
    const unsigned char* hb = reinterpret_cast<const unsigned char*>(hist) +
                              static_cast<size_t>(row) * n_chunks * kHistRowBytes + seg * 16u;
    uint32_t acc[8] = {0, 0, 0, 0, 0, 0, 0, 0}, pre[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (uint32_t c0 = part; c0 < n_chunks; c0 += 16) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t c = c0 + 4u * u;
        v[u] = c < n_chunks
                   ? *reinterpret_cast<const uint4*>(hb + static_cast<size_t>(c) * kHistRowBytes)
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
  for (int p = 0; p < 4; ++p) {
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
  uint32_t cum1 = incl;  // keys <= bin 2t+1
  for (int w = 0; w < wave; ++w) cum1 += sh.wtot[w];
  const uint32_t cum0 = cum1 - ca1;  // keys <= bin 2t
  if (cum0 >= k && cum0 - ca0 < k) {  // exactly one bin holds the k-th smallest key
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
  if (tid == kEmitThreads - 1 && cum1 < k) {  // fewer valid keys than k: all of them are taken
    sh.plan.thr = kHistBins;
    sh.plan.n_below = cum1;
    sh.plan.quota = 0;
    sh.plan.n_take = cum1;
    sh.pre_tied = 0;
  }
  __syncthreads();
  const SelectPlan plan = sh.plan;

  // ---- selected items before the slab, class masks and ranks inside it
  const uint32_t mine_pre = (2 * tid < plan.thr ? cp0 : 0u) + (2 * tid + 1 < plan.thr ? cp1 : 0u);
  const uint32_t wave_pre = wave_sum(mine_pre);
  uint32_t below[kEmitItems / 4], equal[kEmitItems / 4];
  raw_class_masks<kEmitItems>(keys, plan.thr, below, equal);
  uint32_t total;
  const uint32_t excl = lane_scan<kEmitItems / 4>(below, equal, total);  // below | tied << 16
  if (lane == 0) {
    sh.wpre[wave] = wave_pre;
    sh.wclass[wave] = total;
  }
  __syncthreads();
  uint32_t base_b = 0, before = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    base_b += sh.wpre[w];
    before += w < wave ? sh.wclass[w] : 0u;
  }
  lane_emit<kEmitItems / 4>(below, equal, plan.n_below, plan.quota,
                            base_b + (before & 0xffffu) + (excl & 0xffffu),
                            sh.pre_tied + (before >> 16) + (excl >> 16),
                            [&](uint32_t pos, int i) __attribute__((always_inline)) {
                              const uint32_t e = e0 + i;
                              idst[pos] = grow ? grow[e] : static_cast<int32_t>(e);
                              if (vdst)
                                vdst[pos] =
                                    static_cast<uint16_t>(raw_of_key(keys[i], key_mode));
                            });
  if (slab == 0) {
    for (uint32_t i = plan.n_take + tid; i < k; i += kEmitThreads) {
      idst[i] = -1;
      if (vdst) vdst[i] = 0;
    }
  }
}

static size_t hist_path_bytes(uint32_t num_rows, uint32_t n_max) {
  return (static_cast<size_t>(num_rows) * ceil_div(n_max, kHistChunk) * kHistRowBytes + 255) / 256 *
         256;
}

}  // namespace adamas

using namespace adamas;

extern "C" size_t adamas_topk_workspace_bytes(uint32_t num_rows, uint32_t n_max, uint32_t k) {
  const IntLayout il = int_layout(num_rows, n_max, k);
  size_t int_bytes = il.ok ? il.cand_bytes + il.hist_bytes : 0;  // two-level integer path
  const CapLayout cl = cap_layout(num_rows, n_max, k);
  // integer keys outside its reach (k above 255, very long rows): chunk histograms
  if (!il.ok && n_max > kChunkItems) int_bytes = hist_path_bytes(num_rows, n_max);
  if (cl.ok && cl.cand_bytes > int_bytes) int_bytes = cl.cand_bytes;
  if (k > kChunkedMaxK || n_max <= kFinalItems) return int_bytes > 256 ? int_bytes : 256;
  size_t slots = 0;
  uint32_t n = n_max;
  while (n > kFinalItems) {  // one candidate buffer per reduction level
    const uint32_t chunks = ceil_div(n, kChunkItems);
    slots += static_cast<size_t>(chunks) * k;
    n = chunks * k;
  }
  const size_t level_bytes = (static_cast<size_t>(num_rows) * slots * sizeof(uint64_t) + 255) / 256 * 256;
  return level_bytes > int_bytes ? level_bytes : int_bytes;
}

extern "C" int adamas_topk(const void* values, int64_t row_stride, uint32_t n_max,
                           const int32_t* seq_lens, uint32_t rows_per_seq, int32_t len_delta,
                           const int32_t* in_idx, int64_t in_idx_stride, uint32_t num_rows,
                           uint32_t k, int32_t* out_idx, void* out_vals, int64_t out_stride,
                           uint32_t key_mode, void* workspace, size_t workspace_bytes,
                           adamas_stream_t stream) {
  if (num_rows == 0 || k == 0) return 0;
  if (!values || !out_idx) return ADAMAS_E_BADARG;
  if (seq_lens != nullptr && rows_per_seq == 0) return ADAMAS_E_BADARG;
  if (key_mode > ADAMAS_KEY_U16_INT) return ADAMAS_E_BADARG;
  if (out_stride < static_cast<int64_t>(k)) return ADAMAS_E_BADARG;
  if (n_max > kMaxRowLen || num_rows > 65535) return ADAMAS_E_UNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(values) & 1) return ADAMAS_E_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);

  SelectArgs a{};
  a.values = static_cast<const uint16_t*>(values);
  a.row_stride = row_stride;
  a.n_max = n_max;
  a.seq_lens = seq_lens;
  a.rows_per_seq = rows_per_seq == 0 ? 1u : rows_per_seq;
  a.len_delta = len_delta;
  a.in_idx = in_idx;
  a.in_idx_stride = in_idx_stride;
  a.vec_ok = ((reinterpret_cast<uintptr_t>(values) & 15) == 0 && row_stride % 8 == 0) ? 1u : 0u;
  a.k = k;
  a.key_mode = key_mode;
  a.out_idx = out_idx;
  a.out_vals = static_cast<uint16_t*>(out_vals);
  a.out_stride = out_stride;

  // integer keys, k <= 255, rows up to 131072 keys: short candidate lists per chunk, then one
  // workgroup per row (two short launches), when the caller's workspace holds the lists
  const CapLayout cl = cap_layout(num_rows, n_max, k);
  if (cl.ok && key_mode != ADAMAS_KEY_FP16_GENERIC && workspace &&
      workspace_bytes >= cl.cand_bytes && (reinterpret_cast<uintptr_t>(workspace) & 255) == 0) {
    uint64_t* cand = static_cast<uint64_t*>(workspace);
    const dim3 grid1(ceil_div(cl.n_chunks, kIntWaves), num_rows);
#define ADAMAS_LAUNCH_CHUNKS_CAP(ITEMS, MODE)                                                       \
  hipLaunchKernelGGL((select_chunks_capped_kernel<ITEMS, MODE>), grid1, dim3(kIntWaves * kWave), 0, \
                     s, a, cand, cl.n_chunks, cl.kc)
#define ADAMAS_LAUNCH_CHUNKS_CAP_MODE(ITEMS)                                \
  if (a.vec_ok && key_mode == ADAMAS_KEY_FP16_INT) {                        \
    ADAMAS_LAUNCH_CHUNKS_CAP(ITEMS, static_cast<int>(ADAMAS_KEY_FP16_INT)); \
  } else if (a.vec_ok && key_mode == ADAMAS_KEY_U16_INT) {                  \
    ADAMAS_LAUNCH_CHUNKS_CAP(ITEMS, static_cast<int>(ADAMAS_KEY_U16_INT));  \
  } else {                                                                  \
    ADAMAS_LAUNCH_CHUNKS_CAP(ITEMS, -1);                                    \
  }
    if (cl.items == 8) {
      ADAMAS_LAUNCH_CHUNKS_CAP_MODE(8)
    } else if (cl.items == 16) {
      ADAMAS_LAUNCH_CHUNKS_CAP_MODE(16)
    } else {
      ADAMAS_LAUNCH_CHUNKS_CAP_MODE(32)
    }
#undef ADAMAS_LAUNCH_CHUNKS_CAP_MODE
#undef ADAMAS_LAUNCH_CHUNKS_CAP
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    hipLaunchKernelGGL(select_final_capped_kernel, dim3(num_rows), dim3(kFinalThreads), 0, s, a, cand,
                       cl.n_chunks, cl.kc_log2, kWave * cl.items);
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  // the same with lists of the full k and a histogram row per chunk (rows beyond 131072 keys): when
  // the caller's workspace holds them; otherwise the general paths below
  const IntLayout il = int_layout(num_rows, n_max, k);
  if (il.ok && key_mode != ADAMAS_KEY_FP16_GENERIC && workspace &&
      workspace_bytes >= il.cand_bytes + il.hist_bytes &&
      (reinterpret_cast<uintptr_t>(workspace) & 255) == 0) {
    uint64_t* cand = static_cast<uint64_t*>(workspace);
    unsigned char* hist = static_cast<unsigned char*>(workspace) + il.cand_bytes;
    const dim3 grid1(ceil_div(il.n_chunks, kIntWaves), num_rows);
    // the instance with the key format compiled in, where the rows allow 128-bit loads
#define ADAMAS_LAUNCH_CHUNKS_INT(ITEMS, MODE)                                                    \
  hipLaunchKernelGGL((select_chunks_int_kernel<ITEMS, MODE>), grid1, dim3(kIntWaves * kWave), 0, \
                     s, a, cand, hist, il.n_chunks, il.cand_stride)
#define ADAMAS_LAUNCH_CHUNKS_INT_MODE(ITEMS)                          \
  if (a.vec_ok && key_mode == ADAMAS_KEY_FP16_INT) {                  \
    ADAMAS_LAUNCH_CHUNKS_INT(ITEMS, static_cast<int>(ADAMAS_KEY_FP16_INT)); \
  } else if (a.vec_ok && key_mode == ADAMAS_KEY_U16_INT) {            \
    ADAMAS_LAUNCH_CHUNKS_INT(ITEMS, static_cast<int>(ADAMAS_KEY_U16_INT));  \
  } else {                                                            \
    ADAMAS_LAUNCH_CHUNKS_INT(ITEMS, -1);                              \
  }
    if (il.items == 8) {
      ADAMAS_LAUNCH_CHUNKS_INT_MODE(8)
    } else if (il.items == 16) {
      ADAMAS_LAUNCH_CHUNKS_INT_MODE(16)
    } else {
      ADAMAS_LAUNCH_CHUNKS_INT_MODE(32)
    }
#undef ADAMAS_LAUNCH_CHUNKS_INT_MODE
#undef ADAMAS_LAUNCH_CHUNKS_INT
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    const uint64_t slots = static_cast<uint64_t>(il.n_chunks) * il.cand_stride;
#define ADAMAS_LAUNCH_FINAL(G)                                                                      \
  hipLaunchKernelGGL(select_final_int_kernel<G>, dim3(num_rows), dim3(kFinalThreads), 0, s, a, cand, \
                     hist, il.n_chunks, il.cand_stride)
    if (slots <= 4096) {
      ADAMAS_LAUNCH_FINAL(1);
    } else if (slots <= 8192) {
      ADAMAS_LAUNCH_FINAL(2);
    } else if (slots <= 12288) {
      ADAMAS_LAUNCH_FINAL(3);
    } else {
      ADAMAS_LAUNCH_FINAL(4);
    }
#undef ADAMAS_LAUNCH_FINAL
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  // integer keys beyond the two-level scheme: histogram per chunk, then threshold and emission
  if (!il.ok && key_mode != ADAMAS_KEY_FP16_GENERIC && n_max > kChunkItems && workspace &&
      workspace_bytes >= hist_path_bytes(num_rows, n_max) &&
      (reinterpret_cast<uintptr_t>(workspace) & 255) == 0) {
    const uint32_t n_chunks = ceil_div(n_max, kHistChunk);
    uint16_t* hist = static_cast<uint16_t*>(workspace);
    const dim3 hgrid(ceil_div(n_chunks, kHistWaves), num_rows);
    if (a.vec_ok && key_mode == ADAMAS_KEY_FP16_INT)
      hipLaunchKernelGGL(hist_chunks_int_kernel<static_cast<int>(ADAMAS_KEY_FP16_INT)>, hgrid,
                         dim3(kHistWaves * kWave), 0, s, a, hist, n_chunks);
    else if (a.vec_ok && key_mode == ADAMAS_KEY_U16_INT)
      hipLaunchKernelGGL(hist_chunks_int_kernel<static_cast<int>(ADAMAS_KEY_U16_INT)>, hgrid,
                         dim3(kHistWaves * kWave), 0, s, a, hist, n_chunks);
    else
      hipLaunchKernelGGL(hist_chunks_int_kernel<-1>, hgrid, dim3(kHistWaves * kWave), 0, s, a, hist,
                         n_chunks);
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    if (n_max <= kEmitMaxRowLen) {
      const dim3 egrid(num_rows, ceil_div(n_max, kEmitSlab));
      if (a.vec_ok && key_mode == ADAMAS_KEY_FP16_INT)
        hipLaunchKernelGGL(select_hist_emit_kernel<ADAMAS_KEY_FP16_INT>, egrid, dim3(kEmitThreads),
                           0, s, a, hist, n_chunks, kEmitSlab / kHistChunk);
      else if (a.vec_ok && key_mode == ADAMAS_KEY_U16_INT)
        hipLaunchKernelGGL(select_hist_emit_kernel<ADAMAS_KEY_U16_INT>, egrid, dim3(kEmitThreads),
                           0, s, a, hist, n_chunks, kEmitSlab / kHistChunk);
      else
        hipLaunchKernelGGL(select_hist_emit_kernel<-1>, egrid, dim3(kEmitThreads), 0, s, a, hist,
                           n_chunks, kEmitSlab / kHistChunk);
    } else {
      hipLaunchKernelGGL(select_hist_final_kernel, dim3(num_rows), dim3(1024), 0, s, a, hist,
                         n_chunks);
    }
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  if (k > kChunkedMaxK) {
    hipLaunchKernelGGL(select_stream_kernel, dim3(num_rows), dim3(1024), 0, s, a);
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  if (n_max <= kChunkItems) {
    hipLaunchKernelGGL((select_kernel<256, 16, false, false>), dim3(1, num_rows), dim3(256), 0, s,
                       a);
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  if (n_max <= kFinalItems) {
    hipLaunchKernelGGL((select_kernel<1024, 32, false, false>), dim3(1, num_rows), dim3(1024), 0,
                       s, a);
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  // reduction levels, then the final selection among the candidates
  if (!workspace || workspace_bytes < adamas_topk_workspace_bytes(num_rows, n_max, k))
    return ADAMAS_E_WORKSPACE;
  if (reinterpret_cast<uintptr_t>(workspace) & 255) return ADAMAS_E_ALIGN;
  uint64_t* level_out = static_cast<uint64_t*>(workspace);
  uint32_t n = n_max;
  bool from_values = true;
  while (n > kFinalItems) {
    const uint32_t chunks = ceil_div(n, kChunkItems);
    a.cand_out = level_out;
    if (from_values) {
      hipLaunchKernelGGL((select_kernel<256, 16, false, true>), dim3(chunks, num_rows), dim3(256),
                         0, s, a);
    } else {
      hipLaunchKernelGGL((select_kernel<256, 16, true, true>), dim3(chunks, num_rows), dim3(256), 0,
                         s, a);
    }
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    a.cand_in = level_out;
    a.n_in_slots = chunks * k;
    level_out += static_cast<size_t>(num_rows) * chunks * k;
    n = chunks * k;
    from_values = false;
  }
  if (n <= kChunkItems) {
    hipLaunchKernelGGL((select_kernel<256, 16, true, false>), dim3(1, num_rows), dim3(256), 0, s,
                       a);
  } else {
    hipLaunchKernelGGL((select_kernel<1024, 32, true, false>), dim3(1, num_rows), dim3(1024), 0, s,
                       a);
  }
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  return 0;
}
