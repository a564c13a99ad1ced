// Two-level exact selection of the k smallest integer keys (0..511), shared by the fused decode step
// and the stand-alone top-k (gfx950).
//
// Level 1, one wave per chunk of 64 x kItems keys: the smallest keys of the chunk, exactly (threshold
// from a per-chunk histogram in LDS), ties to the lowest index, written as candidates
//     (key << 48) | (offset inside the chunk << 32) | 32-bit payload
// in (below threshold, tied) x ascending-index order.  Two forms:
//   chunk_select_capped  a short list of kc entries (16 for a long row): a chunk holds k / chunks of
//                        the selection on average.  The list is a prefix of the chunk in (key, index)
//                        order, so the second level can tell from its last entry whether the chunk
//                        may hold more of the selection than the list, and then goes back to the
//                        chunk's keys (fused_step.hip: select_attend_kernel; topk.hip:
//                        select_final_capped_kernel).  wave_plan_from_hist reads threshold and tie
//                        quota off a 512-bin histogram, for both levels.
//   chunk_select_emit    a list of the full k plus a 512-bin byte histogram of its keys; the second
//                        level (final_select, one workgroup of 512 threads per row) sums the chunk
//                        histograms and needs no way back to the keys (topk.hip, rows beyond 131072
//                        keys).
// Chunks are concatenated in index order and every list keeps its order, so "ties to the lowest
// index" carries over: the selected candidates are ranked by DPP prefix scans, no atomics.
#pragma once

#include "select.h"

namespace adamas {

constexpr int kHistBins = 512;                  // key values 0..511
// LDS words of chunk_select_emit's histogram, per wave: one 32-bit counter per key value and, behind
// them, a counter that takes the items that are no keys (padded to a multiple of 16 bytes)
constexpr int kChunkHistWords = kHistBins + 4;
constexpr uint64_t kEmptyCand64 = ~0ull;        // an unused candidate slot
constexpr int kFinalThreads = 512;              // workgroup of final_select: one thread per bin
constexpr int kFinalWaves = kFinalThreads / kWave;

// inclusive prefix sum over the lanes of the wave
__device__ __forceinline__ uint32_t wave_inclusive_scan_dpp(uint32_t v) {
  int x = static_cast<int>(v);
  x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, false);  // row_shr:1
  x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, false);  // row_shr:2
  x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, false);  // row_shr:4
  x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, false);  // row_shr:8
  x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1, 3
  x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2, 3
  return static_cast<uint32_t>(x);
}

// Per-lane exclusive prefix (below | tied << 16) over the lower lanes of the wave, for class masks
// spread over kRegs registers per lane (4 items each, item order = register order); `total` gets the
// wave totals.
template <int kRegs>
__device__ __forceinline__ uint32_t lane_scan(const uint32_t (&below)[kRegs],
                                              const uint32_t (&equal)[kRegs], uint32_t& total) {
  uint32_t cb = 0, ce = 0;
#pragma unroll
  for (int j = 0; j < kRegs; ++j) {
    cb += __builtin_popcount(below[j]);
    ce += __builtin_popcount(equal[j]);
  }
  const uint32_t mine = cb | (ce << 16);
  const uint32_t incl = wave_inclusive_scan_dpp(mine);
  total = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(incl), 63));
  return incl - mine;
}

// Emits the selected items of this lane: item i (compile-time at every call site) goes to position
// pb (below class) or n_below + pe (tied class, while the quota lasts).
template <int kRegs, typename Emit>
__device__ __forceinline__ void lane_emit(const uint32_t (&below)[kRegs],
                                          const uint32_t (&equal)[kRegs], uint32_t n_below,
                                          uint32_t quota, uint32_t pb, uint32_t pe, Emit&& emit) {
#pragma unroll
  for (int i = 0; i < 4 * kRegs; ++i) {
    const uint32_t bit = 0x80u << (8 * (i & 3));
    const bool is_b = (below[i >> 2] & bit) != 0;
    const bool is_e = (equal[i >> 2] & bit) != 0;
    if (is_b || (is_e && pe < quota)) emit(is_b ? pb : n_below + pe, i);
    pb += is_b ? 1u : 0u;
    pe += is_e ? 1u : 0u;
  }
}

// The same without branches: emit is called for EVERY item, with position `dump` for the ones that
// are not selected (the caller points that at a spare slot of its own for this lane).  Where emit is
// a pair of LDS writes this costs fewer instructions than the compare-and-branch around each item.
template <int kRegs, typename Emit>
__device__ __forceinline__ void lane_emit_all(const uint32_t (&below)[kRegs],
                                              const uint32_t (&equal)[kRegs], uint32_t n_below,
                                              uint32_t quota, uint32_t pb, uint32_t pe,
                                              uint32_t dump, Emit&& emit) {
  pe += n_below;  // tied items go behind the ones below the threshold
  const uint32_t pe_end = n_below + quota;
#pragma unroll
  for (int i = 0; i < 4 * kRegs; ++i) {
    const uint32_t bit = 0x80u << (8 * (i & 3));
    const bool is_b = (below[i >> 2] & bit) != 0;
    const bool is_e = (equal[i >> 2] & bit) != 0;
    const uint32_t pos = is_b ? pb : ((is_e && pe < pe_end) ? pe : dump);
    emit(pos, i);
    pb += is_b ? 1u : 0u;
    pe += is_e ? 1u : 0u;
  }
}

// class masks of kItems keys against a full-width threshold (bit 8r+7 of word j = item 4j+r)
template <int kItems>
__device__ __forceinline__ void raw_class_masks(const uint32_t (&keys)[kItems], uint32_t thr,
                                                uint32_t (&below)[kItems / 4],
                                                uint32_t (&equal)[kItems / 4]) {
#pragma unroll
  for (int j = 0; j < kItems / 4; ++j) {
    below[j] = 0;
    equal[j] = 0;
  }
#pragma unroll
  for (int i = 0; i < kItems; ++i) {
    const uint32_t bit = 0x80u << (8 * (i & 3));
    below[i >> 2] |= keys[i] < thr ? bit : 0u;  // an empty item compares above everything
    equal[i >> 2] |= keys[i] == thr ? bit : 0u;
  }
}

// One wave: the k smallest of its 64 x kItems keys (lane l holds items kItems*l .. kItems*l + kItems-1,
// any value above 511, e.g. kInvalidKey, = no item; n_valid = number of items).  dst: the chunk's
// candidate list (cand_stride slots, unused ones are filled with kEmptyCand64); hrow: this lane's 8
// bytes of the chunk's histogram row; hist_lds: kChunkHistWords words of LDS owned by this wave,
// 16-byte aligned; payload(item, i) -> 32 bits stored with the candidate (evaluated for selected
// items only; i = item - kItems * lane is a constant at every call, so a caller can keep its
// payloads in registers).
// The threshold is read off a histogram instead of being searched for: every lane counts its keys
// into 512 counters in LDS, a prefix sum over the bins (8 bins per lane, DPP scan
// across the lanes) finds the bin that holds the k-th smallest key, and the histogram of the
// candidates follows from the same counts (bins below the threshold whole, the threshold bin up to
// the tie quota).  Measured against a 7-round bisection on byte-packed keys (one add + and + popcount
// per four keys and round), which this replaced: 1.5 us less per launch of the fused estimator at
// 32768 tokens, 1.6 us less for the stand-alone top-k, +0.7 % on a batch of 16 sequences.
template <int kItems, typename Payload>
__device__ __forceinline__ void chunk_select_emit(const uint32_t (&keys)[kItems],
                                                       uint32_t n_valid, uint32_t k,
                                                       uint32_t cand_stride, uint64_t* dst,
                                                       uint2* hrow, uint32_t* hist_lds,
                                                       Payload&& payload) {
  const int lane = lane_id();
  *reinterpret_cast<uint4*>(&hist_lds[8 * lane]) = make_uint4(0u, 0u, 0u, 0u);
  *reinterpret_cast<uint4*>(&hist_lds[8 * lane + 4]) = make_uint4(0u, 0u, 0u, 0u);
  // One 32-bit counter per key value, and no branch: an item that is no key (any value above 511) counts
  // into the word behind the last bin, which nobody reads.  (Packing two 16-bit bins into a word
  // and skipping the invalid items cost seven more instructions per item.)
#pragma unroll
  for (int i = 0; i < kItems; ++i)
    atomicAdd(&hist_lds[min(keys[i], static_cast<uint32_t>(kHistBins))], 1u);
  // the LDS operations of one wave are carried out in order: the counts are complete here
  const uint4 hv0 = *reinterpret_cast<const uint4*>(&hist_lds[8 * lane]);
  const uint4 hv1 = *reinterpret_cast<const uint4*>(&hist_lds[8 * lane + 4]);
  const uint32_t c[8] = {hv0.x, hv0.y, hv0.z, hv0.w, hv1.x, hv1.y, hv1.z, hv1.w};
  uint32_t lane_sum = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) lane_sum += c[j];
  const uint32_t incl = wave_inclusive_scan_dpp(lane_sum);
  uint32_t thr, n_below, quota, n_take;
  if (n_valid <= k) {  // fewer keys than asked for: all of them are taken
    thr = static_cast<uint32_t>(kHistBins);
    n_below = n_valid;
    quota = 0;
    n_take = n_valid;
  } else {
    // exactly one bin holds the k-th smallest key; its lane finds it among its 8 bins
    uint32_t run = incl - lane_sum, t_l = 0, nb_l = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool here = run < k && run + c[j] >= k;
      t_l = here ? 8u * static_cast<uint32_t>(lane) + j : t_l;
      nb_l = here ? run : nb_l;
      run += c[j];
    }
    const uint64_t cross = __ballot(incl - lane_sum < k && incl >= k);
    const int src = __builtin_amdgcn_readfirstlane(__ffsll(static_cast<long long>(cross)) - 1);
    thr = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(t_l), src));
    n_below = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(nb_l), src));
    quota = k - n_below;
    n_take = k;
  }
  // the histogram of this chunk's candidates, one byte per distance value (at most k <= 255 each)
  {
    uint32_t w[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t bin = 8u * static_cast<uint32_t>(lane) + j;
      const uint32_t cnt = bin < thr ? c[j] : (bin == thr ? quota : 0u);
      w[j >> 2] |= cnt << (8 * (j & 3));
    }
    *hrow = make_uint2(w[0], w[1]);
  }
  uint32_t below[kItems / 4], equal[kItems / 4];
  raw_class_masks<kItems>(keys, thr, below, equal);
  uint32_t total;
  const uint32_t excl = lane_scan<kItems / 4>(below, equal, total);
  lane_emit<kItems / 4>(below, equal, n_below, quota, excl & 0xffffu, excl >> 16,
                        [&](uint32_t pos, int i) __attribute__((always_inline)) {
                          const uint32_t tok = static_cast<uint32_t>(lane) * kItems + i;
                          dst[pos] =
                              (static_cast<uint64_t>((keys[i] << 16) | tok) << 32) | payload(tok, i);
                        });
  for (uint32_t i = n_take + lane; i < cand_stride; i += kWave) dst[i] = kEmptyCand64;
}

// Threshold of the k smallest keys from a 512-bin histogram in LDS (one 32-bit counter per key
// value, 16-byte aligned), computed by one wave; every lane returns the same plan.  Lane l reads
// bins 8l .. 8l+7 (two 128-bit reads), a DPP prefix sum over the lanes finds the bin that holds the
// k-th smallest key.  Any number of waves may call this on the same histogram side by side: they
// only read.
struct WavePlan {
  uint32_t thr;      // threshold key (kHistBins when there are at most k keys: all of them are taken)
  uint32_t n_below;  // keys below the threshold
  uint32_t quota;    // keys equal to the threshold to take, lowest index first
  uint32_t n_take;   // k, or the number of keys if that is smaller
};

__device__ __forceinline__ WavePlan wave_plan_from_hist(const uint32_t* hist_lds, uint32_t k) {
  const int lane = lane_id();
  const uint4 hv0 = *reinterpret_cast<const uint4*>(&hist_lds[8 * lane]);
  const uint4 hv1 = *reinterpret_cast<const uint4*>(&hist_lds[8 * lane + 4]);
  const uint32_t c[8] = {hv0.x, hv0.y, hv0.z, hv0.w, hv1.x, hv1.y, hv1.z, hv1.w};
  uint32_t lane_sum = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) lane_sum += c[j];
  const uint32_t incl = wave_inclusive_scan_dpp(lane_sum);
  const uint32_t total = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(incl), 63));
  WavePlan p;
  if (total <= k) {
    p.thr = static_cast<uint32_t>(kHistBins);
    p.n_below = total;
    p.quota = 0;
    p.n_take = total;
    return p;
  }
  // exactly one bin holds the k-th smallest key; its lane finds it among its 8 bins
  uint32_t run = incl - lane_sum, t_l = 0, nb_l = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const bool here = run < k && run + c[j] >= k;
    t_l = here ? 8u * static_cast<uint32_t>(lane) + j : t_l;
    nb_l = here ? run : nb_l;
    run += c[j];
  }
  const uint64_t cross = __ballot(incl - lane_sum < k && incl >= k);
  const int src = __builtin_amdgcn_readfirstlane(__ffsll(static_cast<long long>(cross)) - 1);
  p.thr = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(t_l), src));
  p.n_below = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(nb_l), src));
  p.quota = k - p.n_below;
  p.n_take = k;
  return p;
}

// One wave: the kc smallest of its 64 x kItems keys (lane l holds items kItems*l .. kItems*l +
// kItems-1 in index order, kItems <= 32; any value above 511 = no item), ties to the lowest index,
// written to the chunk's candidate list dst[kc] as (key << 48) | (item index << 32) | payload, first
// the keys below the chunk's threshold, then the tied ones, each class in ascending index order;
// unused slots are filled with kEmptyCand64.  A list is a prefix of the chunk in (key, index) order:
// when its last entry is not among the keys a caller finally selects, no key of the chunk outside the
// list can be.
// hist_lds: kChunkHistWords words of LDS owned by this wave, 16-byte aligned.  key_of(item) -> the
// key of an item (the caller's LDS copy: a listed item is picked by a run-time index), payload(item)
// -> 32 bits stored with the candidate; both are evaluated for listed items only.
// A list has a handful of entries among hundreds of items, so the items are not tested one by one
// when the list is written: every lane walks the set bits of its own class masks, and the wave makes
// as many rounds as its busiest lane has listed items (one or two, against kItems tests of a dozen
// instructions each).
// kSkipInvalid: items that are no keys are left out of the counting by a branch (worth it where many
// lanes hold none: they would all add to one spare word); otherwise they count into a spare word
// without a branch.
template <int kItems, bool kSkipInvalid, typename KeyOf, typename Payload>
__device__ __forceinline__ void chunk_select_capped(const uint32_t (&keys)[kItems], uint32_t kc,
                                                    uint64_t* dst, uint32_t* hist_lds,
                                                    KeyOf&& key_of, Payload&& payload) {
  static_assert(kItems <= 32, "one class bit per item");
  const int lane = lane_id();
  *reinterpret_cast<uint4*>(&hist_lds[8 * lane]) = make_uint4(0u, 0u, 0u, 0u);
  *reinterpret_cast<uint4*>(&hist_lds[8 * lane + 4]) = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
  for (int i = 0; i < kItems; ++i) {
    if (kSkipInvalid) {
      if (keys[i] < static_cast<uint32_t>(kHistBins)) atomicAdd(&hist_lds[keys[i]], 1u);
    } else {
      atomicAdd(&hist_lds[min(keys[i], static_cast<uint32_t>(kHistBins))], 1u);
    }
  }
  // the LDS operations of one wave are carried out in order: the counts are complete here
  const WavePlan p = wave_plan_from_hist(hist_lds, kc);
  uint32_t below = 0, equal = 0;  // bit i: item i is below / equal to the threshold
#pragma unroll
  for (int i = 0; i < kItems; ++i) {
    below |= keys[i] < p.thr ? (1u << i) : 0u;  // an empty item compares above everything
    equal |= keys[i] == p.thr ? (1u << i) : 0u;
  }
  const uint32_t mine = static_cast<uint32_t>(__builtin_popcount(below)) |
                        (static_cast<uint32_t>(__builtin_popcount(equal)) << 16);
  const uint32_t excl = wave_inclusive_scan_dpp(mine) - mine;
  uint32_t pb = excl & 0xffffu, pe = excl >> 16;  // items of each class in the lower lanes
  uint32_t todo = below | (pe < p.quota ? equal : 0u);
  while (todo) {
    const uint32_t i = static_cast<uint32_t>(__builtin_ctz(todo));
    todo &= todo - 1u;
    const bool is_b = ((below >> i) & 1u) != 0;
    const uint32_t item = static_cast<uint32_t>(lane) * kItems + i;
    uint32_t pos, key;
    if (is_b) {
      pos = pb++;
      key = key_of(item);
    } else {  // a tied item inside the quota
      pos = p.n_below + pe++;
      key = p.thr;
      if (pe >= p.quota) todo &= below;  // the quota is used up: the lane's further ties stay out
    }
    dst[pos] = (static_cast<uint64_t>((key << 16) | item) << 32) | payload(item);
  }
  for (uint32_t i = p.n_take + lane; i < kc; i += kWave) dst[i] = kEmptyCand64;
}

struct FinalSelectShared {
  uint16_t hpart[kFinalThreads / 32][kHistBins];  // partial histogram sums (16 KB)
  alignas(16) uint32_t wtot[kFinalWaves];         // per-wave totals of the histogram scan
  alignas(16) uint32_t wclass[kFinalWaves];       // per-wave class totals: below | tied << 16
  uint32_t thr, n_below, total;                   // the selection plan
};

// Level 2 for one row, called by all 512 threads of the workgroup.  crow: the row's n_slots =
// n_chunks * cand_stride candidate slots (n_slots <= 512 * 8 * kGroups, cand_stride a multiple of 8);
// hist_rows: its n_chunks histogram rows of 512 bytes.  emit(pos, slot0, offset, key, payload) is
// called once per selected candidate, pos in [0, n_take), in the lane that holds it; slot0 is the
// first slot of the candidate's group of 8 (its chunk is slot0 / cand_stride), offset its token
// offset inside the chunk.  Returns n_take
// (k, or the number of candidates if smaller).  Ends without a barrier: the caller synchronises
// before it reads what emit() wrote.
// while_loading() is called once by every thread after the loads of the histogram rows and of the
// candidates have been consumed and before the first barrier: work of the caller that depends on
// loads it issued earlier costs no wait of its own there.
// kEmitAll: emit is called for every candidate slot, unselected ones with position dump_base + lane
// (see lane_emit_all); the caller's arrays have 64 spare entries there.
template <int kGroups, bool kEmitAll = false, typename Emit, typename WhileLoading>
__device__ __forceinline__ uint32_t final_select(const uint64_t* __restrict__ crow, uint32_t n_slots,
                                                 const unsigned char* __restrict__ hist_rows,
                                                 uint32_t n_chunks, uint32_t k,
                                                 uint32_t cand_stride, FinalSelectShared& sh,
                                                 Emit&& emit, WhileLoading&& while_loading,
                                                 uint32_t dump_base = 0) {
  static_assert(kFinalThreads == kHistBins, "one thread per key value");
  constexpr int kItems = 8 * kGroups;
  constexpr int kAttThreads = kFinalThreads;
  const uint32_t tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  // ---- threshold from the per-chunk histograms ------------------------------------------------------
  // count[v] = candidates of this head with distance v, summed over the chunks (one byte per chunk);
  // a partial sum stays below 2^16 as long as a thread adds at most 257 chunks of <= 255 each
  // Step 1: thread t sums 16 adjacent bins (one 128-bit load per chunk row) over the chunks
  // t/32, t/32 + 16, ...; all loads are independent.  Bytes are widened to 16-bit pairs (SWAR).
  {
    const uint32_t part = tid >> 5;   // 16 partial sums per bin
    const uint32_t seg = tid & 31u;   // bins 16*seg .. 16*seg + 15
    const unsigned char* hbase = hist_rows + seg * 16u;
    uint32_t ev[4] = {0, 0, 0, 0}, od[4] = {0, 0, 0, 0};
    constexpr uint32_t kParts = kAttThreads / 32;
    for (uint32_t c0 = part; c0 < n_chunks; c0 += 4 * kParts) {
      uint4 v[4];  // four rows in flight per thread
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t c = c0 + u * kParts;
        v[u] = c < n_chunks
                   ? *reinterpret_cast<const uint4*>(hbase + static_cast<size_t>(c) * kHistBins)
                   : make_uint4(0u, 0u, 0u, 0u);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          ev[j] += w[j] & 0x00ff00ffu;         // bins 4j, 4j+2
          od[j] += (w[j] >> 8) & 0x00ff00ffu;  // bins 4j+1, 4j+3
        }
      }
    }
    uint32_t o[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      o[2 * j] = (ev[j] & 0xffffu) | (od[j] << 16);          // bins 4j, 4j+1
      o[2 * j + 1] = (ev[j] >> 16) | (od[j] & 0xffff0000u);  // bins 4j+2, 4j+3
    }
    uint4* dstp = reinterpret_cast<uint4*>(&sh.hpart[part][seg * 16u]);
    dstp[0] = make_uint4(o[0], o[1], o[2], o[3]);
    dstp[1] = make_uint4(o[4], o[5], o[6], o[7]);
  }

  // ---- stage: kItems candidate slots per thread, as groups of 8 consecutive slots -----------------
  // group j of this thread = slots ((wave*kGroups + j)*64 + lane)*8 .. +7
  uint32_t keys[kItems];      // distance of each candidate
  uint32_t krow[kItems];      // its payload
  uint32_t toks[kItems / 2];  // its token offset inside the chunk, two per register
#pragma unroll
  for (int j = 0; j < kGroups; ++j) {
    const uint32_t e0 = block_item_index<kItems>(wave, lane, j, 0);
    uint64_t c[8];
    if (e0 < n_slots) {  // rows are 64-byte aligned
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const uint4 a = *reinterpret_cast<const uint4*>(crow + e0 + 2 * r);
        c[2 * r] = static_cast<uint64_t>(a.x) | (static_cast<uint64_t>(a.y) << 32);
        c[2 * r + 1] = static_cast<uint64_t>(a.z) | (static_cast<uint64_t>(a.w) << 32);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 8; ++r) c[r] = kEmptyCand64;
    }
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      // an unused slot is all ones: its key field reads 0xffff, above every threshold (<= 512), so it
      // needs no test of its own
      keys[j * 8 + r] = static_cast<uint32_t>(c[r] >> 48);
      krow[j * 8 + r] = static_cast<uint32_t>(c[r]);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
      toks[j * 4 + r] = (static_cast<uint32_t>(c[2 * r] >> 32) & 0xffffu) |
                        (static_cast<uint32_t>(c[2 * r + 1] >> 32) << 16);
  }

  while_loading();
  // Step 2: thread v folds the 16 partial sums of its bin
  __syncthreads();
  uint32_t count = 0;
#pragma unroll
  for (int p = 0; p < kAttThreads / 32; ++p) count += sh.hpart[p][tid];

  // block prefix sum of count[]: cum[v] = candidates with distance <= v
  const uint32_t incl = wave_inclusive_scan_dpp(count);
  if (lane == kWave - 1) sh.wtot[wave] = incl;
  __syncthreads();
  uint32_t cum = incl;
  {  // totals of the earlier waves: all eight read at once, the later ones masked out
    static_assert(kFinalWaves == 8, "two 128-bit reads cover the wave totals");
    const uint4 lo = *reinterpret_cast<const uint4*>(&sh.wtot[0]);
    const uint4 hi = *reinterpret_cast<const uint4*>(&sh.wtot[4]);
    const uint32_t t[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
    for (int w = 0; w < 8; ++w) cum += w < wave ? t[w] : 0u;
  }
  // exactly one thread sees the k-th smallest candidate inside its bin
  if (cum >= k && cum - count < k) {
    sh.thr = tid;
    sh.n_below = cum - count;
  }
  if (tid == kAttThreads - 1) sh.total = cum;
  __syncthreads();
  const uint32_t total = sh.total;
  uint32_t thr, n_below, quota, n_take;
  if (total <= k) {  // fewer candidates than the budget: all of them are taken
    thr = kHistBins;
    n_below = total;
    quota = 0;
    n_take = total;
  } else {
    thr = sh.thr;
    n_below = sh.n_below;
    quota = k - n_below;
    n_take = k;
  }

  // ---- every wave emits its own selected slots, group by group (the item order of select.h) ------
  uint32_t below[kItems / 4], equal[kItems / 4];
  raw_class_masks<kItems>(keys, thr, below, equal);
  uint32_t ex[kGroups], tot[kGroups];
  uint32_t wave_total = 0;
#pragma unroll
  for (int j = 0; j < kGroups; ++j) {
    const uint32_t bj[2] = {below[2 * j], below[2 * j + 1]}, ej[2] = {equal[2 * j], equal[2 * j + 1]};
    ex[j] = lane_scan<2>(bj, ej, tot[j]);
    wave_total += tot[j];  // fields stay below 2^16
  }
  if (lane == 0) sh.wclass[wave] = wave_total;
  __syncthreads();
  uint32_t base_b = 0, base_e = 0;  // class counts of all earlier waves
  {
    const uint4 lo = *reinterpret_cast<const uint4*>(&sh.wclass[0]);
    const uint4 hi = *reinterpret_cast<const uint4*>(&sh.wclass[4]);
    const uint32_t t[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    uint32_t both = 0;  // the two 16-bit fields cannot carry into each other: at most 16384 slots
#pragma unroll
    for (int w = 0; w < 8; ++w) both += w < wave ? t[w] : 0u;
    base_b = both & 0xffffu;
    base_e = both >> 16;
  }
#pragma unroll
  for (int j = 0; j < kGroups; ++j) {
    const uint32_t bj[2] = {below[2 * j], below[2 * j + 1]}, ej[2] = {equal[2 * j], equal[2 * j + 1]};
    // cand_stride is a multiple of 8: the 8 slots of a group belong to one chunk, slot0 / cand_stride
    // (left to the caller: a division per lane that only a caller who wants positions has to pay)
    const uint32_t slot0 = block_item_index<kItems>(wave, lane, j, 0);
    auto emit_item = [&](uint32_t pos, int i) __attribute__((always_inline)) {
      const uint32_t tk = toks[j * 4 + (i >> 1)];
      emit(pos, slot0, (i & 1) ? (tk >> 16) : (tk & 0xffffu), keys[j * 8 + i], krow[j * 8 + i]);
    };
    if (kEmitAll)
      lane_emit_all<2>(bj, ej, n_below, quota, base_b + (ex[j] & 0xffffu),
                       base_e + (ex[j] >> 16), dump_base + static_cast<uint32_t>(lane), emit_item);
    else
      lane_emit<2>(bj, ej, n_below, quota, base_b + (ex[j] & 0xffffu), base_e + (ex[j] >> 16),
                   emit_item);
    base_b += tot[j] & 0xffffu;
    base_e += tot[j] >> 16;
  }
  return n_take;
}

}  // namespace adamas
