// Layout of the caller-allocated workspace shared by adamas_sparse_decode and adamas_decode_step.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <algorithm>

#include "../../include/adamas_hip.h"

namespace adamas {

constexpr uint32_t kMaxSplits = 128;                 // KV splits per (sequence, head)
constexpr uint32_t kPartialFloats = 2 + 128;         // m, l, o[128]
constexpr uint32_t kFusedBlock = 512;                // tokens per pass of the fused estimator
constexpr uint32_t kFusedMaxPasses = 4;              // a workgroup covers at most 2048 tokens
constexpr uint32_t kFusedMaxSel = 255;               // largest budget-1 of the two-launch path
constexpr uint32_t kStepUnit = 16;                   // chunk boundaries are multiples of 16 tokens
constexpr uint32_t kStepMaxChunks = 64;              // token chunks per sequence of the two-launch step
constexpr uint32_t kStepMaxSlots = 2048;             // candidate slots per head: chunks x slots per chunk
constexpr uint32_t kStepWorkgroups = 256;            // the estimator aims at one workgroup per CU of an MI355X

// Geometry of the two-launch step (estimate_select_kernel, select_attend_kernel), fixed on the host
// from the sizes of the call.  A sequence is cut into `chunks` token chunks; chunk c covers the
// 16-token units [c*units_q + min(c, units_r), ...) and has units_q + (c < units_r) of them, so the
// chunks differ by at most 16 tokens and their number does not change while the sequence grows: the
// cost of the step is a smooth function of the length.  Every chunk hands its `kc` nearest tokens per
// head to the second launch.
struct StepPlan {
  uint32_t ok;        // 1 when the two-launch path serves these sizes
  uint32_t heads;     // heads per workgroup of the estimator: 8 (512 threads) or 4 (256 threads)
  uint32_t chunks;    // token chunks per sequence (grid.x of the estimator), <= kStepMaxChunks
  uint32_t units_q, units_r;
  uint32_t passes;    // passes of 512 tokens a workgroup makes over its chunk (1 .. 4)
  uint32_t partial;   // 1 when a chunk can be shorter than passes * 512 tokens by whole units
  uint32_t kc;        // candidate slots per (head, chunk): a power of two, 8 .. 256
  uint32_t kc_log2;
};

inline uint32_t pow2_floor(uint32_t v) {
  uint32_t p = 1;
  while (p * 2 <= v) p *= 2;
  return p;
}
inline uint32_t pow2_ceil(uint32_t v) {
  uint32_t p = 1;
  while (p < v) p *= 2;
  return p;
}

inline StepPlan step_plan(uint32_t batch, uint32_t num_heads, uint32_t max_seq_len,
                          uint32_t budget) {
  StepPlan p = {};
  if (batch == 0 || num_heads == 0 || num_heads % 8 != 0 || max_seq_len < 2 || budget < 2 ||
      budget - 1 > kFusedMaxSel)
    return p;
  const uint32_t n = max_seq_len - 1;                       // past tokens, at most
  const uint32_t units = (n + kStepUnit - 1) / kStepUnit;
  const uint32_t pass_units = kFusedBlock / kStepUnit;      // 32
  const uint32_t max_chunk_units = pass_units * kFusedMaxPasses;
  if (batch == 1) {
    // one workgroup per CU where the sequence is long enough: the wide workgroup (8 heads, 256
    // contiguous bytes per token) from 512 tokens per chunk on, else the narrow one (4 heads), else
    // chunks of 512 tokens that do not fill the chip
    const uint32_t c_wide = std::max(1u, kStepWorkgroups / (num_heads / 8));
    const uint32_t c_narrow = std::max(1u, kStepWorkgroups / (num_heads / 4));
    uint32_t chunks;
    if (units >= pass_units * std::min(c_wide, kStepMaxChunks)) {
      p.heads = 8;
      chunks = std::min(c_wide, kStepMaxChunks);
    } else if (units >= pass_units * std::min(c_narrow, kStepMaxChunks)) {
      p.heads = 4;
      chunks = std::min(c_narrow, kStepMaxChunks);
    } else {
      p.heads = 4;
      chunks = 0;  // fixed chunks of 512 tokens, below
    }
    if (chunks) {
      // more chunks than CUs / head groups only where a chunk would exceed the workgroup's capacity
      const uint32_t need = (units + max_chunk_units - 1) / max_chunk_units;
      chunks = std::max(chunks, need);
      if (chunks > kStepMaxChunks) return p;
      p.chunks = chunks;
      p.units_q = units / chunks;
      p.units_r = units % chunks;
    } else {
      p.chunks = (units + pass_units - 1) / pass_units;
      p.units_q = pass_units;
      p.units_r = 0;
    }
  } else {
    // several sequences: their lengths differ and only the device knows them; chunks of a fixed
    // size (the smallest of 512, 1024, 2048 tokens that keeps the chunk count), narrow workgroups
    p.heads = 4;
    uint32_t passes = 1;
    while (passes <= kFusedMaxPasses &&
           (units + pass_units * passes - 1) / (pass_units * passes) > kStepMaxChunks)
      passes *= 2;
    if (passes > kFusedMaxPasses) return p;
    p.chunks = (units + pass_units * passes - 1) / (pass_units * passes);
    p.units_q = pass_units * passes;
    p.units_r = 0;
  }
  const uint32_t longest = p.units_q + (p.units_r ? 1u : 0u);
  p.passes = (longest + pass_units - 1) / pass_units;
  if (p.passes == 0 || p.passes > kFusedMaxPasses) return p;
  p.partial = (p.units_r != 0 || p.units_q % pass_units != 0) ? 1u : 0u;
  // slots per chunk: the whole budget where the lists of all chunks fit, else what fits (at least
  // 16: the second launch re-scores the rare chunk that holds more of the selection than its list).
  // One sequence: 1024 slots per head (two per thread of the second launch; a chunk holds
  // budget / chunks of the selection on average, a small fraction of its list).  Several sequences:
  // the chunks are sized for the longest one, a short sequence spreads its selection over few of
  // them, and twice the slots keep those lists from running out.
  const uint32_t fit = pow2_floor((batch == 1 ? kStepMaxSlots / 2 : kStepMaxSlots) / p.chunks);
  p.kc = std::max(8u, std::min(fit, pow2_ceil(budget - 1)));
  p.kc_log2 = 0;
  while ((1u << p.kc_log2) < p.kc) ++p.kc_log2;
  p.ok = 1;
  return p;
}

struct WorkspaceLayout {
  size_t counters_off;  // uint32 [batch*heads], arrival counters of the split merge (kept at zero)
  size_t partial_off;   // float  [batch*heads][kMaxSplits][kPartialFloats]
  size_t dist_off;      // uint16 [batch*heads][dist_stride]: distances of the step for large budgets;
                        // in the two-launch step, the re-scored distances of truncated chunks
  size_t sel_off;       // int32  [batch*heads][budget], selection of the fused step
  size_t rowmap_off;    // uint32 [batch][dist_stride], K row index of every past token (same step)
  size_t topk_off;      // workspace of adamas_topk inside the fused step
  size_t topk_bytes;
  size_t cand_off;      // uint64 [batch*heads][plan.chunks][plan.kc], candidates of the two-launch step
  size_t qcode_off;     // uint16 [batch*heads][16], the query codes the first launch worked with
  StepPlan plan;        // geometry of the two-launch step (plan.ok: it serves these sizes)
  size_t hist_off;      // uint16 [batch*heads][hist_stride][512], tokens per distance in chunks of 512
                        // (the step for large budgets only)
  uint32_t hist_stride; // chunk rows per head
  size_t total;
  int64_t dist_stride;  // elements, multiple of 8
};

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

inline WorkspaceLayout workspace_layout(uint32_t batch, uint32_t num_heads, uint32_t max_seq_len,
                                        uint32_t budget) {
  WorkspaceLayout w;
  const size_t rows = static_cast<size_t>(batch) * num_heads;
  size_t off = 0;
  w.counters_off = off;
  off = align_up(off + rows * sizeof(uint32_t), 256);
  w.partial_off = off;
  off = align_up(off + rows * kMaxSplits * kPartialFloats * sizeof(float), 256);
  w.dist_stride = static_cast<int64_t>(align_up(max_seq_len, 8));
  w.dist_off = off;
  off = align_up(off + rows * static_cast<size_t>(w.dist_stride) * sizeof(uint16_t), 256);
  w.sel_off = off;
  off = align_up(off + rows * static_cast<size_t>(budget ? budget : 1) * sizeof(int32_t), 256);
  w.rowmap_off = off;
  off = align_up(off + static_cast<size_t>(batch) * static_cast<size_t>(w.dist_stride) * sizeof(uint32_t), 256);
  w.topk_off = off;
  w.topk_bytes = (budget > 1 && max_seq_len > 1)
                     ? adamas_topk_workspace_bytes(static_cast<uint32_t>(rows), max_seq_len - 1,
                                                   budget - 1)
                     : 0;
  off = align_up(off + w.topk_bytes, 256);
  w.plan = step_plan(batch, num_heads, max_seq_len, budget);
  w.cand_off = off;
  w.qcode_off = off;
  w.hist_off = off;
  w.hist_stride = 0;
  if (w.plan.ok) {
    off = align_up(off + rows * w.plan.chunks * static_cast<size_t>(w.plan.kc) * sizeof(uint64_t), 256);
    w.qcode_off = off;
    off = align_up(off + rows * 16 * sizeof(uint16_t), 256);
  } else if (max_seq_len > 1 && budget > 1) {
    w.hist_off = off;
    w.hist_stride = (max_seq_len - 1 + kFusedBlock - 1) / kFusedBlock;
    off = align_up(off + rows * 1024 * static_cast<size_t>(w.hist_stride), 256);
  }
  w.total = off;
  return w;
}

}  // namespace adamas
