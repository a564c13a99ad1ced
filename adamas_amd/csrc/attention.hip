// Paged decode attention over a per-head list of token positions (gfx950).
//
// grid = (splits, heads, batch), 256 - 1024 threads = 16 - 64 groups of 16 lanes.  A K or V row of one
// head is 128 fp16 = 256 bytes = 16 lanes x 128-bit, so a group owns a row and a lane owns 8 channels.
// Each group asks for its 2 or 4 K rows and V rows before any of them is used, the dot products are
// reduced over the 16 lanes, and an fp32 online softmax (base 2) keeps (m, l, o[8]) per lane.  Groups
// are merged through LDS; when a head is cut into several splits the partial (m, l, o[128]) go to
// the workspace and the last workgroup to arrive for that head merges them, so there is no second
// launch (from 24 splits on the merge is a short launch of its own).
#include "attend.h"
#include "split_merge.h"
#include "workspace.h"

namespace adamas {

constexpr int kTile = 8;             // rows per group per tile, at most
// A workgroup has 256, 512 or 1024 threads = 16, 32 or 64 groups of 16 lanes; a group has 2 or 4
// rows in flight, and a split is one such round of loads.  One CU gathers scattered rows slowly (a
// single workgroup per head takes 25 us for 1024 rows), a group finishes sooner the fewer rows it
// has to ask for, and publishing a partial result costs about a microsecond.  Hence: up to 64 rows
// 16 groups of 4, up to 128 rows 32 groups of 4 (one split, no merge, no workspace); up to 512 rows
// splits of 64 rows (32 groups of 2, at most 8 splits); up to 2048 rows splits of 128 (64 groups of
// 2, at most 16); beyond that splits of 256 (64 groups of 4).  Measured at 32 heads, rows = 128 /
// 256 / 512 / 1024 / 2048 / 4096, in us: 5.8 / 6.5 / 7.4 / 9.3 / 13.5 / 18.8 (with 16 groups of 8
// rows and splits of 128 rows up to 1024 rows, 32 groups of 8 beyond: 7.5 / 9.5 / 10.1 / 12.4 / 15.8
// / 20.6).
constexpr uint32_t kDeferredMergeSplits = 24;  // splits from which the partials get a merge launch
// (measured at 32768 tokens, 32 heads: 16 splits 14.7 us merged inside the launch, 15.8 us with a merge
// launch; 32 splits 26.6 against 22.5 us)

template <int kGroups>
struct AttnShared {
  MergeShared<kGroups> merge;
  uint32_t is_last;
};

template <bool kBf16, bool kHnd, int kThreads = 256, int kTileRows = kTile>
__global__ __launch_bounds__(kThreads) void sparse_decode_kernel(
    const __half* __restrict__ q, const __half* __restrict__ kv_data,
    const int32_t* __restrict__ page_indices, const int32_t* __restrict__ page_indptr,
    const int32_t* __restrict__ seq_lens, const int32_t* __restrict__ sel_idx, int64_t sel_stride,
    uint32_t n_sel, __half* __restrict__ out, float* partial,
    uint32_t* __restrict__ counters, uint32_t num_heads, uint32_t num_kv_heads, uint32_t page_size,
    float scale_log2, uint32_t rows_per_split, uint32_t deferred_merge) {
  constexpr int kGroups = kThreads / 16;  // rows in flight per load instruction of the workgroup
  __shared__ AttnShared<kGroups> sh;
  const uint32_t split = blockIdx.x, n_split = gridDim.x;
  const uint32_t head = blockIdx.y;
  const uint32_t b = blockIdx.z;
  const uint32_t tid = threadIdx.x;
  const uint32_t g = tid >> 4;   // group
  const uint32_t c = tid & 15;   // lane in group: channels [8c, 8c+8)
  const uint32_t bh = b * num_heads + head;

  const int32_t seq_len = seq_lens[b];
  const bool dense = sel_idx == nullptr;
  const uint32_t n_rows = dense ? static_cast<uint32_t>(seq_len) : n_sel + 1u;
  const int32_t* sel = dense ? nullptr : sel_idx + static_cast<int64_t>(bh) * sel_stride;
  const uint32_t row_begin = split * rows_per_split;
  const uint32_t row_end = min(n_rows, row_begin + rows_per_split);

  float qf[8];
  load_query<kBf16>(q + static_cast<size_t>(bh) * kHeadDim, c, scale_log2, qf);
  HeadKV kv;
  kv.kv_data = kv_data;
  kv.table = page_indices + page_indptr[b];
  // grouped-query attention: query head h reads the K/V rows of key head h / group
  set_kv_layout_static<kHnd>(kv, head / (num_heads / num_kv_heads), c, num_kv_heads, page_size);
  kv.seq_len = seq_len;

  SoftmaxState st;
  // (token positions through the page table: branching around unused entries measured faster
  // here than loading always, 7.9 against 8.0 us at 128 rows)
  attend_rows<kGroups, kTileRows, false, kBf16>(kv, qf, g, row_begin, row_end,
                              [&](uint32_t r) __attribute__((always_inline)) -> int32_t {
                                if (dense) return static_cast<int32_t>(r);
                                return (r < n_sel) ? sel[r] : seq_len - 1;
                              },
                              st);

  float M, L, O;
  merge_groups<kGroups>(st, g, c, tid, sh.merge, M, L, O);
  if (n_split == 1) {
    // an empty row list (a sequence without tokens) gives zeros, not 0/0
    if (tid < kHeadDim)
      store_elem<kBf16>(out + static_cast<size_t>(bh) * kHeadDim + tid, L > 0.f ? O / L : 0.f);
    return;
  }

  float* mine = partial + (static_cast<size_t>(bh) * kMaxSplits + split) * kPartialFloats;
  if (deferred_merge) {
    // many splits: the partials are merged by a launch of their own (merge_splits_kernel).  Plain
    // stores and a kernel boundary cost less than publishing inside the launch, whose critical path
    // holds the acknowledgement of the write-through stores, the arrival counter and the merge.
    if (tid < kHeadDim) {
      if (tid == 0) {
        mine[0] = M;
        mine[1] = L;
      }
      mine[2 + tid] = O;
    }
    return;
  }
  // ---- several splits: publish the partial, the last arrival merges (protocol: split_merge.h) ------
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

// Merge of the split partials as a launch of its own: grid (heads, batch), 512 threads = four groups
// of one thread per channel; group g folds the splits g, g + 4, ... (plain loads, sixteen in flight
// per round, so up to 64 splits cost one memory round trip), the four running states meet in LDS.
constexpr int kMergeGroups = 4;

template <bool kBf16>
__global__ __launch_bounds__(kMergeGroups* kHeadDim) void merge_splits_kernel(
    const float* __restrict__ partial, __half* __restrict__ out, uint32_t num_heads,
    uint32_t n_split) {
  __shared__ float sm[kMergeGroups][kHeadDim], sl[kMergeGroups][kHeadDim], sa[kMergeGroups][kHeadDim];
  const uint32_t bh = blockIdx.y * num_heads + blockIdx.x;
  const uint32_t ch = threadIdx.x & (kHeadDim - 1);
  const uint32_t grp = threadIdx.x / kHeadDim;
  const float* base = partial + static_cast<size_t>(bh) * kMaxSplits * kPartialFloats;
  float M = kNegBig, L = 0.f, A = 0.f;
  for (uint32_t s0 = grp; s0 < n_split; s0 += 16 * kMergeGroups) {
    float m[16], l[16], a[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      // past the end: a duplicate of the last split, weighted zero below
      const uint32_t s2 = min(s0 + u * kMergeGroups, n_split - 1);
      const float* p = base + static_cast<size_t>(s2) * kPartialFloats;
      m[u] = p[0];
      l[u] = p[1];
      a[u] = p[2 + ch];
    }
    float m_new = M;
#pragma unroll
    for (int u = 0; u < 16; ++u)
      m_new = fmaxf(m_new, s0 + u * kMergeGroups < n_split ? m[u] : kNegBig);
    const float keep = exp2_raw(M - m_new);
    L *= keep;
    A *= keep;
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const float w = s0 + u * kMergeGroups < n_split ? exp2_raw(m[u] - m_new) : 0.f;
      L += l[u] * w;
      A += a[u] * w;
    }
    M = m_new;
  }
  sm[grp][ch] = M;
  sl[grp][ch] = L;
  sa[grp][ch] = A;
  __syncthreads();
  if (grp != 0) return;
  float Mt = kNegBig;
#pragma unroll
  for (int g = 0; g < kMergeGroups; ++g) Mt = fmaxf(Mt, sm[g][ch]);
  float Lt = 0.f, At = 0.f;
#pragma unroll
  for (int g = 0; g < kMergeGroups; ++g) {
    const float w = exp2_raw(sm[g][ch] - Mt);  // a group without splits holds (kNegBig, 0, 0): weight 0 or 1 on zeros
    Lt += sl[g][ch] * w;
    At += sa[g][ch] * w;
  }
  store_elem<kBf16>(out + static_cast<size_t>(bh) * kHeadDim + ch, Lt > 0.f ? At / Lt : 0.f);
}

// ---- dense decode attention: every token of the sequence -----------------------------------------
// grid = (splits, heads / 8, batch), 512 threads = 8 heads x 4 token slices x 16 lanes.  In the
// [page][K|V][slot][head][128] layout the rows of adjacent heads of one token are adjacent in memory:
// a wave covers four heads of one token (1 KB contiguous per load instruction) and a workgroup eight
// heads (2 KB), instead of 256-byte pieces 8 KB apart as in the per-head walk above.  Each lane keeps
// 8 K and 8 V loads in flight (128 KB per workgroup).  The four token slices are merged through LDS,
// splits through the workspace exactly as above (one arrival counter per group of eight heads).
constexpr int kDenseThreads = 512;
constexpr int kDenseHeads = 8;
constexpr int kDenseSlices = 4;
constexpr int kDenseTile = 8;
constexpr uint32_t kDenseRowsPerIter = kDenseSlices * kDenseTile;  // 32 tokens
// Workgroups per launch.  Measured at 32K tokens x 32 heads with the merge of the splits in a launch
// of its own: 192 workgroups stream at 5.37 TB/s, 128 at 5.12, 256 at 5.31, 384 at 4.79, 512 at 5.12
// (beyond ~24 MB in flight the memory system loses more to queueing than it gains in parallelism).
// The grouped-query kernels read a fraction of the bytes per unit of work and want every CU busy.
constexpr uint32_t kDenseTargetBlocks = 192;
constexpr uint32_t kDenseGqaTargetBlocks = 256;
// Splits from which the dense kernels leave the merge of their partials to a launch of its own.
// Publishing partials inside the launch (write-through stores, their acknowledgement, the arrival
// counter, the last workgroup's merge) sits at the end of every workgroup's critical path: with the
// 64 splits of the grouped-query kernels it cost 10 us of 38, the extra launch costs 4.4.
constexpr uint32_t kDenseDeferredSplits = 24;

struct DenseShared {
  float m[kDenseSlices][kDenseHeads];
  float l[kDenseSlices][kDenseHeads];
  alignas(16) float o[kDenseSlices][kDenseHeads][kHeadDim];
  uint32_t is_last;
};

template <bool kBf16>
__global__ __launch_bounds__(kDenseThreads) void dense_decode_kernel(
    const __half* __restrict__ q, const __half* __restrict__ kv_data,
    const int32_t* __restrict__ page_indices, const int32_t* __restrict__ page_indptr,
    const int32_t* __restrict__ seq_lens, __half* __restrict__ out, float* partial,
    uint32_t* __restrict__ counters, uint32_t num_heads, uint32_t num_kv_heads, uint32_t page_size,
    float scale_log2, uint32_t rows_per_split, KvLayout lay, uint32_t deferred_merge) {
  __shared__ DenseShared sh;
  const uint32_t split = blockIdx.x, n_split = gridDim.x;
  const uint32_t hg = blockIdx.y;
  const uint32_t b = blockIdx.z;
  const uint32_t tid = threadIdx.x;
  const int wave = wave_id_uniform();
  const int lane = lane_id();
  const uint32_t slice = static_cast<uint32_t>(wave) >> 1;  // uniform over the wave
  const uint32_t hl = ((static_cast<uint32_t>(wave) & 1u) << 2) | (static_cast<uint32_t>(lane) >> 4);
  const uint32_t c = static_cast<uint32_t>(lane) & 15u;     // channels [8c, 8c+8)
  const uint32_t head = hg * kDenseHeads + hl;

  const int32_t seq_len = seq_lens[b];
  const uint32_t row_begin = split * rows_per_split;
  const uint32_t row_end = min(static_cast<uint32_t>(seq_len), row_begin + rows_per_split);

  float qf[8];
  load_query<kBf16>(q + (static_cast<size_t>(b) * num_heads + head) * kHeadDim, c, scale_log2, qf);
  HeadKV kv;
  kv.kv_data = kv_data;
  kv.table = page_indices + page_indptr[b];
  set_kv_layout(kv, lay, head / (num_heads / num_kv_heads), c, page_size);
  kv.seq_len = seq_len;

  SoftmaxState st;
  attend_rows<kDenseSlices, kDenseTile, false, kBf16, true>(kv, qf, slice, row_begin, row_end,
                                        [&](uint32_t r) __attribute__((always_inline)) -> int32_t {
                                          return static_cast<int32_t>(r);
                                        },
                                        st);
  if (c == 0) {
    sh.m[slice][hl] = st.m;
    sh.l[slice][hl] = st.l;
  }
#pragma unroll
  for (int j = 0; j < 2; ++j)  // two 128-bit stores: 512 contiguous bytes per lane group
    *reinterpret_cast<float4*>(&sh.o[slice][hl][8 * c + 4 * j]) =
        make_float4(st.o[4 * j], st.o[4 * j + 1], st.o[4 * j + 2], st.o[4 * j + 3]);
  __syncthreads();

  // thread -> (head hh of the octet, channels 2cp and 2cp+1)
  const uint32_t hh = tid >> 6, cp = tid & 63u;
  float M = kNegBig;
#pragma unroll
  for (int s2 = 0; s2 < kDenseSlices; ++s2) M = fmaxf(M, sh.m[s2][hh]);
  float L = 0.f, O0 = 0.f, O1 = 0.f;
#pragma unroll
  for (int s2 = 0; s2 < kDenseSlices; ++s2) {
    const float wgt = exp2_raw(sh.m[s2][hh] - M);
    L += sh.l[s2][hh] * wgt;
    O0 += sh.o[s2][hh][2 * cp] * wgt;
    O1 += sh.o[s2][hh][2 * cp + 1] * wgt;
  }
  const size_t bh = static_cast<size_t>(b) * num_heads + hg * kDenseHeads + hh;
  uint32_t* orow = reinterpret_cast<uint32_t*>(out + bh * kHeadDim) + cp;
  if (n_split == 1) {
    const float inv = L > 0.f ? 1.f / L : 0.f;  // no tokens: zeros
    *orow = pack2<kBf16>(O0 * inv, O1 * inv);
    return;
  }

  // several splits: publish the partial, the last workgroup of this head octet merges (same
  // agent-scope protocol as sparse_decode_kernel)
  float* mine = partial + (bh * kMaxSplits + split) * kPartialFloats;
  if (deferred_merge) {  // many splits: plain stores, merged by merge_splits_kernel
    if (cp == 0) *reinterpret_cast<float2*>(mine) = make_float2(M, L);
    *reinterpret_cast<float2*>(mine + 2 + 2 * cp) = make_float2(O0, O1);
    return;
  }
  if (cp == 0) store_partial_pair(mine, M, L);
  store_partial_pair(mine + 2 + 2 * cp, O0, O1);
  uint32_t* counter = counters + static_cast<size_t>(b) * num_heads + hg * kDenseHeads;
  if (!split_arrive_is_last(counter, n_split, sh.is_last, tid)) return;
  {
    float LL, A[2];
    merge_partial_pairs<32>(partial + bh * kMaxSplits * kPartialFloats, n_split, 2 * cp, LL, A);
    const float inv = LL > 0.f ? 1.f / LL : 0.f;
    *orow = pack2<kBf16>(A[0] * inv, A[1] * inv);
  }
  if (tid == 0) *counter = 0;  // ready for the next launch on this stream
}

// ---- dense decode attention with grouped queries -------------------------------------------------
// The same walk, but a 16-lane group owns a KEY/VALUE head and serves the kG query heads of its group
// from every K and V row it loads: the rows are read once instead of once per query head.  A
// workgroup still owns eight query heads (8 / kG key/value heads), so the split merge is the one of
// dense_decode_kernel; the lane groups left over become more token slices (32 * kG / 8).
// grid = (splits, kv heads * kG / 8, batch).
// sum of the eight products of two 128-bit operands (8 fp16 or 8 bf16 each), accumulated in fp32
template <bool kBf16>
__device__ __forceinline__ float dot8(const uint4& a, const uint4& b) {
  float acc = 0.f;
  if (kBf16) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const bf16x2_t* ah = reinterpret_cast<const bf16x2_t*>(&a);
    const bf16x2_t* bh = reinterpret_cast<const bf16x2_t*>(&b);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2_f32_bf16(ah[i], bh[i], acc, false);
  } else {
    typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
    const half2_t* ah = reinterpret_cast<const half2_t*>(&a);
    const half2_t* bh = reinterpret_cast<const half2_t*>(&b);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2(ah[i], bh[i], acc, false);
  }
  return acc;
}

template <int kG>
struct DenseGqaShared {
  static constexpr int kKv = kDenseHeads / kG;      // key/value heads per workgroup
  static constexpr int kSlices = 32 / kKv;          // token slices per workgroup
  float m[kSlices][kDenseHeads];
  float l[kSlices][kDenseHeads];
  alignas(16) float o[kSlices][kDenseHeads][kHeadDim];
  uint32_t is_last;
};

template <int kG, int kTile, bool kBf16>
__global__ __launch_bounds__(kDenseThreads) void dense_decode_gqa_kernel(
    const __half* __restrict__ q, const __half* __restrict__ kv_data,
    const int32_t* __restrict__ page_indices, const int32_t* __restrict__ page_indptr,
    const int32_t* __restrict__ seq_lens, __half* __restrict__ out, float* partial,
    uint32_t* __restrict__ counters, uint32_t num_heads, uint32_t num_kv_heads, uint32_t page_size,
    float scale_log2, uint32_t rows_per_split, KvLayout kvl, uint32_t deferred_merge) {
  constexpr int kKv = DenseGqaShared<kG>::kKv;
  constexpr int kSlices = DenseGqaShared<kG>::kSlices;
  __shared__ DenseGqaShared<kG> sh;
  const uint32_t split = blockIdx.x, n_split = gridDim.x;
  const uint32_t b = blockIdx.z;
  const uint32_t tid = threadIdx.x;
  const uint32_t gi = tid >> 4;            // lane group 0..31
  const uint32_t kl = gi % kKv;            // key/value head inside the workgroup
  const uint32_t slice = gi / kKv;         // token slice
  const uint32_t c = tid & 15u;            // channels [8c, 8c+8)
  const uint32_t kv_head = blockIdx.y * kKv + kl;
  const uint32_t head0 = blockIdx.y * kDenseHeads;  // first query head of the workgroup

  const int32_t seq_len = seq_lens[b];
  const uint32_t row_begin = split * rows_per_split;
  const uint32_t row_end = min(static_cast<uint32_t>(seq_len), row_begin + rows_per_split);
  const int32_t* table = page_indices + page_indptr[b];
  HeadKV lay;  // strides of the page layout
  set_kv_layout(lay, kvl, kv_head, c, page_size);
  const size_t tok_stride = lay.tok_stride;
  const size_t v_delta = lay.v_delta;
  const uint32_t row_mult = lay.row_mult;
  const __half* kv_lane = kv_data + lay.head_off;

  // the query stays in its 16-bit format: q.k is formed with the two-element dot instruction (exact products,
  // fp32 accumulation) and scaled after the sum over the 16 lanes
  uint4 qraw[kG];
  SoftmaxState st[kG];
#pragma unroll
  for (int j = 0; j < kG; ++j)
    qraw[j] = *reinterpret_cast<const uint4*>(
        q + (static_cast<size_t>(b) * num_heads + head0 + kl * kG + j) * kHeadDim + 8 * c);

  for (uint32_t base = row_begin; base < row_end; base += kSlices * kTile) {
    uint4 kr[kTile], vr[kTile];
    bool valid[kTile];
#pragma unroll
    for (int i = 0; i < kTile; ++i) {
      const uint32_t r = base + i * kSlices + slice;
      valid[i] = r < row_end;
      kr[i] = make_uint4(0, 0, 0, 0);
      vr[i] = make_uint4(0, 0, 0, 0);
      if (valid[i]) {
        const uint32_t lp = r / page_size;
        const uint32_t slot = r - lp * page_size;
        const size_t row = static_cast<size_t>(table[lp]) * row_mult + slot;
        const __half* kp = kv_lane + row * tok_stride;
        kr[i] = *reinterpret_cast<const uint4*>(kp);
        vr[i] = *reinterpret_cast<const uint4*>(kp + v_delta);
      }
    }
#pragma unroll
    for (int j = 0; j < kG; ++j) {
      float sc[kTile];
      float m_new = st[j].m;
#pragma unroll
      for (int i = 0; i < kTile; ++i) {
        const float d = group16_sum(dot8<kBf16>(qraw[j], kr[i])) * scale_log2;
        sc[i] = valid[i] ? d : kNegBig;
        m_new = fmaxf(m_new, sc[i]);
      }
      const float alpha = exp2_raw(st[j].m - m_new);
      st[j].l *= alpha;
#pragma unroll
      for (int e = 0; e < 8; ++e) st[j].o[e] *= alpha;
#pragma unroll
      for (int i = 0; i < kTile; ++i) {
        const float pw = valid[i] ? exp2_raw(sc[i] - m_new) : 0.f;
        st[j].l += pw;
        float vf[8];
        unpack8<kBf16>(vr[i], vf);
#pragma unroll
        for (int e = 0; e < 8; ++e) st[j].o[e] += pw * vf[e];
      }
      st[j].m = m_new;
    }
  }
#pragma unroll
  for (int j = 0; j < kG; ++j) {
    const uint32_t hl = kl * kG + j;  // query head inside the workgroup
    if (c == 0) {
      sh.m[slice][hl] = st[j].m;
      sh.l[slice][hl] = st[j].l;
    }
#pragma unroll
    for (int e = 0; e < 2; ++e)  // two 128-bit stores: 512 contiguous bytes per lane group
      *reinterpret_cast<float4*>(&sh.o[slice][hl][8 * c + 4 * e]) =
          make_float4(st[j].o[4 * e], st[j].o[4 * e + 1], st[j].o[4 * e + 2], st[j].o[4 * e + 3]);
  }
  __syncthreads();

  // from here on as in dense_decode_kernel: thread -> (query head hh, channels 2cp and 2cp+1)
  const uint32_t hh = tid >> 6, cp = tid & 63u;
  float M = kNegBig;
#pragma unroll
  for (int s2 = 0; s2 < kSlices; ++s2) M = fmaxf(M, sh.m[s2][hh]);
  float L = 0.f, O0 = 0.f, O1 = 0.f;
#pragma unroll
  for (int s2 = 0; s2 < kSlices; ++s2) {
    const float wgt = exp2_raw(sh.m[s2][hh] - M);
    L += sh.l[s2][hh] * wgt;
    O0 += sh.o[s2][hh][2 * cp] * wgt;
    O1 += sh.o[s2][hh][2 * cp + 1] * wgt;
  }
  const size_t bh = static_cast<size_t>(b) * num_heads + head0 + hh;
  uint32_t* orow = reinterpret_cast<uint32_t*>(out + bh * kHeadDim) + cp;
  if (n_split == 1) {
    const float inv = L > 0.f ? 1.f / L : 0.f;
    *orow = pack2<kBf16>(O0 * inv, O1 * inv);
    return;
  }
  float* mine = partial + (bh * kMaxSplits + split) * kPartialFloats;
  if (deferred_merge) {  // many splits: plain stores, merged by merge_splits_kernel
    if (cp == 0) *reinterpret_cast<float2*>(mine) = make_float2(M, L);
    *reinterpret_cast<float2*>(mine + 2 + 2 * cp) = make_float2(O0, O1);
    return;
  }
  if (cp == 0) store_partial_pair(mine, M, L);
  store_partial_pair(mine + 2 + 2 * cp, O0, O1);
  uint32_t* counter = counters + static_cast<size_t>(b) * num_heads + head0;
  if (!split_arrive_is_last(counter, n_split, sh.is_last, tid)) return;
  {
    float LL, A[2];
    merge_partial_pairs<32>(partial + bh * kMaxSplits * kPartialFloats, n_split, 2 * cp, LL, A);
    const float inv = LL > 0.f ? 1.f / LL : 0.f;
    *orow = pack2<kBf16>(A[0] * inv, A[1] * inv);
  }
  if (tid == 0) *counter = 0;  // ready for the next launch on this stream
}


// ---- dense decode attention with grouped queries on the matrix cores -------------------------------
// The one GEMM-shaped piece of the path: a key/value head serves kG query heads, so the scores of a
// tile of 16 tokens are a [16 tokens x 128] x [128 x kG] product and the weighted values a
// [128 channels x 16 tokens] x [16 tokens x kG] product.  Both run as 16x16 MFMA tiles with the query
// heads in the N dimension (kG of the 16 columns are used: the matrix cores have throughput to spare,
// what matters is that the products leave the vector ALU, which the scalar kernel above keeps busy
// with ~125 instructions per row and lane).
//
//   scores   S^T[token][head] = sum over four k-steps of v_mfma_f32_16x16x32: lane (t = lane % 16,
//            qt = lane / 16) supplies the eight K channels 32j + 8qt .. +7 of token t for step j -
//            exactly one 128-bit load of that token's row - and the same channels of query head
//            lane % 16 (zero for the unused columns).  The order of the k index is the same on both
//            sides, which is all the product needs.
//   softmax  lane (head = lane % 16, qt) then holds the scores of tokens 4qt .. 4qt+3 of its head:
//            fp32 online softmax, base 2; the running maximum is shared by the four lanes of a head,
//            the denominator is kept per lane and summed at the end.
//   values   O^T[channel][head] += V^T[channel][token] x P[token][head] as eight v_mfma_f32_16x16x16
//            tiles.  P in the lane layout the score product left it in IS the B operand (tokens
//            4qt .. 4qt+3 of head lane % 16).  The A operand wants four TOKENS of one channel per lane,
//            memory has eight channels of one token per lane: the V tile goes through LDS (rows of
//            264 bytes, so that the four token groups of a read fall into different banks).
//
// Workgroup = 8 waves = 8 query heads = 8 / kG key/value heads x kG token slices (wave w: key/value
// head w % (8 / kG), slice w / (8 / kG)), so the merge of the slices and of the splits is the one of
// the kernels above.  A wave walks over its tiles with the loads of the next tile and the page id of
// the one after in flight.  grid = (splits, query heads / 8, batch).
typedef _Float16 mfma_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 mfma_half4 __attribute__((ext_vector_type(4)));
typedef __bf16 mfma_bf8 __attribute__((ext_vector_type(8)));
typedef short mfma_short4 __attribute__((ext_vector_type(4)));
typedef float mfma_float4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kVtRowBytes = 264;                 // one token's 128 channels + 8 bytes
constexpr uint32_t kVtWaveBytes = 16 * kVtRowBytes;   // a tile of 16 tokens

template <bool kBf16>
__device__ __forceinline__ mfma_float4 mfma_qk(const uint4& a, const uint4& b, mfma_float4 c) {
  if (kBf16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const mfma_bf8*>(&a),
                                                   *reinterpret_cast<const mfma_bf8*>(&b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(*reinterpret_cast<const mfma_half8*>(&a),
                                                *reinterpret_cast<const mfma_half8*>(&b), c, 0, 0, 0);
}

// a, b: four 16-bit values each, packed in two words
template <bool kBf16>
__device__ __forceinline__ mfma_float4 mfma_pv(const uint2& a, const uint2& b, mfma_float4 c) {
  if (kBf16)
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(*reinterpret_cast<const mfma_short4*>(&a),
                                                     *reinterpret_cast<const mfma_short4*>(&b), c, 0,
                                                     0, 0);
  return __builtin_amdgcn_mfma_f32_16x16x16f16(*reinterpret_cast<const mfma_half4*>(&a),
                                               *reinterpret_cast<const mfma_half4*>(&b), c, 0, 0, 0);
}

template <int kG>
struct DenseGqaMfmaShared {
  // the V tiles of the eight waves while they walk, the slice states once they are done
  union {
    alignas(16) unsigned char vt[8][kVtWaveBytes];
    alignas(16) float o[kG][kDenseHeads][kHeadDim];
  };
  float m[kG][kDenseHeads];
  float l[kG][kDenseHeads];
  uint32_t is_last;
};

template <int kG, bool kBf16>
__global__ __launch_bounds__(kDenseThreads) void dense_decode_gqa_mfma_kernel(
    const __half* __restrict__ q, const __half* __restrict__ kv_data,
    const int32_t* __restrict__ page_indices, const int32_t* __restrict__ page_indptr,
    const int32_t* __restrict__ seq_lens, __half* __restrict__ out, float* partial,
    uint32_t* __restrict__ counters, uint32_t num_heads, uint32_t num_kv_heads, uint32_t page_size,
    float scale_log2, uint32_t rows_per_split, KvLayout kvl, uint32_t deferred_merge) {
  static_assert(kG == 2 || kG == 4 || kG == 8, "2, 4 or 8 query heads per key/value head");
  constexpr int kKv = kDenseHeads / kG;   // key/value heads per workgroup
  constexpr uint32_t kStep = 16u * kG;    // tokens between two tiles of a wave
  __shared__ DenseGqaMfmaShared<kG> sh;
  const uint32_t split = blockIdx.x, n_split = gridDim.x;
  const uint32_t b = blockIdx.z;
  const uint32_t tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = wave_id_uniform();
  const uint32_t kl = static_cast<uint32_t>(wave) % kKv;     // key/value head inside the workgroup
  const uint32_t slice = static_cast<uint32_t>(wave) / kKv;  // token slice
  const uint32_t t16 = static_cast<uint32_t>(lane) & 15u;    // token of the tile (loads), head (scores)
  const uint32_t qt = static_cast<uint32_t>(lane) >> 4;      // channel quarter (loads), token group (scores)
  const uint32_t kv_head = blockIdx.y * kKv + kl;
  const uint32_t head0 = blockIdx.y * kDenseHeads;           // first query head of the workgroup

  const int32_t seq_len = seq_lens[b];
  const uint32_t row_begin = split * rows_per_split;
  const uint32_t row_end = min(static_cast<uint32_t>(seq_len), row_begin + rows_per_split);
  const int32_t* table = page_indices + page_indptr[b];
  const uint32_t lp_last = seq_len > 0 ? (static_cast<uint32_t>(seq_len) - 1u) / page_size : 0u;
  const __half* kv_lane = kv_data + static_cast<size_t>(kv_head) * kvl.head_stride + 8u * qt;

  // B operand of the score product: channels 32j + 8qt .. +7 of query head t16 (columns >= kG: zero)
  uint4 qb[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    qb[j] = make_uint4(0u, 0u, 0u, 0u);
    if (t16 < kG)
      qb[j] = *reinterpret_cast<const uint4*>(
          q + (static_cast<size_t>(b) * num_heads + head0 + kl * kG + t16) * kHeadDim + 32 * j + 8 * qt);
  }

  mfma_float4 acc[8];  // acc[ct][i] = O[head t16][channel 16ct + 4qt + i]
#pragma unroll
  for (int ct = 0; ct < 8; ++ct) acc[ct] = mfma_float4{0.f, 0.f, 0.f, 0.f};
  float m_run = kNegBig, l_run = 0.f;

  unsigned char* vt = sh.vt[wave];
  // page of the tile that starts at token `base` for this lane's token (clamped to the sequence)
  auto page_of = [&](uint32_t base) __attribute__((always_inline)) -> uint32_t {
    const uint32_t lp = min((base + t16) / page_size, lp_last);
    return static_cast<uint32_t>(table[lp]);
  };
  // the eight loads of a tile: K and V channels 32j + 8qt .. +7 of token base + t16
  auto issue = [&](uint32_t base, uint32_t page, uint4 (&kr)[4], uint4 (&vr)[4])
                   __attribute__((always_inline)) {
    const uint32_t r = min(base + t16, static_cast<uint32_t>(max(seq_len, 1)) - 1u);
    const uint32_t lp = r / page_size;
    const size_t row = static_cast<size_t>(page) * kvl.rows_per_page + (r - lp * page_size);
    const __half* kp = kv_lane + row * kvl.tok_stride;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      kr[j] = *reinterpret_cast<const uint4*>(kp + 32 * j);
      vr[j] = *reinterpret_cast<const uint4*>(kp + kvl.v_delta + 32 * j);
    }
  };
  auto compute = [&](uint32_t base, const uint4 (&kr)[4], const uint4 (&vr)[4])
                     __attribute__((always_inline)) {
    mfma_float4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) sc = mfma_qk<kBf16>(kr[j], qb[j], sc);
    // the V tile on its way to the layout the second product wants (64-bit stores: rows are 8-byte
    // aligned); the wave's LDS operations are carried out in order, no barrier needed
    {
      unsigned char* dst = vt + t16 * kVtRowBytes + 16u * qt;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        *reinterpret_cast<uint2*>(dst + 64 * j) = make_uint2(vr[j].x, vr[j].y);
        *reinterpret_cast<uint2*>(dst + 64 * j + 8) = make_uint2(vr[j].z, vr[j].w);
      }
    }
    float s[4];
    bool ok[4];
    float tmax = kNegBig;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ok[i] = base + 4u * qt + i < row_end;
      s[i] = ok[i] ? sc[i] * scale_log2 : kNegBig;
      tmax = fmaxf(tmax, s[i]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
    const float m_new = fmaxf(m_run, tmax);
    const float alpha = exp2_raw(m_run - m_new);
    float p[4], psum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = ok[i] ? exp2_raw(s[i] - m_new) : 0.f;
      psum += p[i];
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
#pragma unroll
    for (int ct = 0; ct < 8; ++ct) {
      acc[ct][0] *= alpha;
      acc[ct][1] *= alpha;
      acc[ct][2] *= alpha;
      acc[ct][3] *= alpha;
    }
    const uint2 pb = make_uint2(pack2<kBf16>(p[0], p[1]), pack2<kBf16>(p[2], p[3]));
    // A operand of tile ct: channel 16ct + t16 of tokens 4qt .. 4qt+3
    const unsigned char* src = vt + 4u * qt * kVtRowBytes + 2u * t16;
#pragma unroll
    for (int ct = 0; ct < 8; ++ct) {
      uint32_t e[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        e[i] = *reinterpret_cast<const uint16_t*>(src + i * kVtRowBytes + 32 * ct);
      const uint2 va = make_uint2(e[0] | (e[1] << 16), e[2] | (e[3] << 16));
      acc[ct] = mfma_pv<kBf16>(va, pb, acc[ct]);
    }
  };

  // ---- the walk: compute tile t with the loads of the next kAhead tiles and the page id of the one
  // after them in flight (a ring of kAhead + 1 register buffers, indexed at compile time) ----------
  constexpr int kAhead = 1;  // two tiles ahead measure the same, three slower (registers)
  constexpr int kBuf = kAhead + 1;
  const uint32_t first = row_begin + slice * 16u;
  if (first < row_end) {
    const uint32_t n_tiles = (row_end - first + kStep - 1) / kStep;  // tiles of this wave
    uint4 kr[kBuf][4], vr[kBuf][4];
#pragma unroll
    for (int j = 0; j < kAhead; ++j)
      if (static_cast<uint32_t>(j) < n_tiles)
        issue(first + j * kStep, page_of(first + j * kStep), kr[j], vr[j]);
    uint32_t page_next = page_of(first + kAhead * kStep);  // of the tile the first round issues
    for (uint32_t t0 = 0; t0 < n_tiles; t0 += kBuf) {
#pragma unroll
      for (int sl = 0; sl < kBuf; ++sl) {
        const uint32_t t = t0 + sl;
        if (t >= n_tiles) break;
        const uint32_t page_after = page_of(first + (t + kAhead + 1) * kStep);
        if (t + kAhead < n_tiles)
          issue(first + (t + kAhead) * kStep, page_next, kr[(sl + kAhead) % kBuf],
                vr[(sl + kAhead) % kBuf]);
        compute(first + t * kStep, kr[sl], vr[sl]);
        page_next = page_after;
      }
    }
  }

  // ---- the slices of the workgroup, then the splits: as in dense_decode_gqa_kernel ------------------
  __syncthreads();  // every wave is done with its V tile: the same LDS now takes the slice states
  float l_tot = l_run;  // the four lanes of a head hold the denominators of their own tokens
  l_tot += __shfl_xor(l_tot, 16);
  l_tot += __shfl_xor(l_tot, 32);
  if (t16 < kG) {
    const uint32_t hl = kl * kG + t16;  // query head inside the workgroup
    if (qt == 0) {
      sh.m[slice][hl] = m_run;
      sh.l[slice][hl] = l_tot;
    }
#pragma unroll
    for (int ct = 0; ct < 8; ++ct)
      *reinterpret_cast<float4*>(&sh.o[slice][hl][16 * ct + 4 * qt]) =
          make_float4(acc[ct][0], acc[ct][1], acc[ct][2], acc[ct][3]);
  }
  __syncthreads();

  const uint32_t hh = tid >> 6, cp = tid & 63u;  // thread -> (query head hh, channels 2cp and 2cp+1)
  float M = kNegBig;
#pragma unroll
  for (int s2 = 0; s2 < kG; ++s2) M = fmaxf(M, sh.m[s2][hh]);
  float L = 0.f, O0 = 0.f, O1 = 0.f;
#pragma unroll
  for (int s2 = 0; s2 < kG; ++s2) {
    const float wgt = exp2_raw(sh.m[s2][hh] - M);
    L += sh.l[s2][hh] * wgt;
    O0 += sh.o[s2][hh][2 * cp] * wgt;
    O1 += sh.o[s2][hh][2 * cp + 1] * wgt;
  }
  const size_t bh = static_cast<size_t>(b) * num_heads + head0 + hh;
  uint32_t* orow = reinterpret_cast<uint32_t*>(out + bh * kHeadDim) + cp;
  if (n_split == 1) {
    const float inv = L > 0.f ? 1.f / L : 0.f;
    *orow = pack2<kBf16>(O0 * inv, O1 * inv);
    return;
  }
  float* mine = partial + (bh * kMaxSplits + split) * kPartialFloats;
  if (deferred_merge) {
    // many splits: plain stores, the partials are merged by a launch of their own
    // (merge_splits_kernel); publishing them inside the launch - write-through stores, their
    // acknowledgement, the arrival counter, the last workgroup's merge - sat at the end of every
    // workgroup's critical path and cost 10 us of 38 at 64 splits
    if (cp == 0) *reinterpret_cast<float2*>(mine) = make_float2(M, L);
    *reinterpret_cast<float2*>(mine + 2 + 2 * cp) = make_float2(O0, O1);
    return;
  }
  if (cp == 0) store_partial_pair(mine, M, L);
  store_partial_pair(mine + 2 + 2 * cp, O0, O1);
  uint32_t* counter = counters + static_cast<size_t>(b) * num_heads + head0;
  if (!split_arrive_is_last(counter, n_split, sh.is_last, tid)) return;
  {
    float LL, A[2];
    merge_partial_pairs<32>(partial + bh * kMaxSplits * kPartialFloats, n_split, 2 * cp, LL, A);
    const float inv = LL > 0.f ? 1.f / LL : 0.f;
    *orow = pack2<kBf16>(A[0] * inv, A[1] * inv);
  }
  if (tid == 0) *counter = 0;  // ready for the next launch on this stream
}

}  // namespace adamas

using namespace adamas;

extern "C" size_t adamas_workspace_bytes(uint32_t batch, uint32_t num_heads, uint32_t max_seq_len,
                                         uint32_t budget) {
  return workspace_layout(batch, num_heads, max_seq_len, budget).total;
}

static int sparse_decode_impl(const void* q, const void* kv_data, const int32_t* page_indices,
                              const int32_t* page_indptr, const int32_t* seq_lens,
                              const int32_t* sel_idx, int64_t sel_stride, uint32_t n_sel, void* out,
                              void* workspace, size_t workspace_bytes, uint32_t batch,
                              uint32_t num_heads, uint32_t num_kv_heads, uint32_t head_dim,
                              uint32_t page_size, float sm_scale, uint32_t max_seq_len,
                              adamas_stream_t stream, uint32_t flags) {
  if (flags & ~(ADAMAS_F_BF16 | ADAMAS_F_HND | ADAMAS_F_NO_MFMA)) return ADAMAS_E_BADARG;
  const bool bf16 = (flags & ADAMAS_F_BF16) != 0;
  const KvLayout lay = make_kv_layout((flags & ADAMAS_F_HND) != 0, page_size, num_kv_heads);
  if (!q || !kv_data || !page_indices || !page_indptr || !seq_lens || !out || batch == 0 ||
      num_heads == 0 || page_size == 0 || max_seq_len == 0)
    return ADAMAS_E_BADARG;
  if (head_dim != kHeadDim) return ADAMAS_E_UNSUPPORTED;
  if (batch > 65535 || num_heads > 65535) return ADAMAS_E_UNSUPPORTED;
  if (num_kv_heads == 0 || num_heads % num_kv_heads != 0) return ADAMAS_E_UNSUPPORTED;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(kv_data)) & 15)
    return ADAMAS_E_ALIGN;
  if (sel_idx != nullptr && sel_stride < static_cast<int64_t>(n_sel)) return ADAMAS_E_BADARG;

  const float scale_log2 = sm_scale * 1.4426950408889634f;
  const uint32_t gq = num_heads / num_kv_heads;  // query heads per key/value head
  // 2, 4 or 8 query heads per key/value head: the kernel that loads every row once (a workgroup owns
  // 8 query heads = 8 / gq key/value heads); other group sizes run the per-query-head kernels, whose
  // lanes of one group load the same rows (correct, merged by the memory pipeline, but slower)
  const bool gqa_kernel = (gq == 2 || gq == 4 || gq == 8) && num_heads % kDenseHeads == 0;
  // Short sequences attend all their tokens through the kernel for row lists below (sel_idx ==
  // nullptr: the rows are the positions 0 .. seq_len - 1): the dense kernels cut a sequence into
  // splits of at least 128 tokens for eight heads at once, which leaves most CUs idle when the
  // sequence is short (1024 tokens: 17.5 us against 9.4; 130 tokens: 16.4 against 7.1; equal at
  // 4096 tokens; with four query heads per key/value head, whose rows the row kernel reads four
  // times, 14.3 against 8.6 us at 1024 tokens and 11.8 at 2048).
  const uint32_t dense_rows_limit = gq == 1 ? 4096u : 2048u;
  if (!sel_idx && num_heads % kDenseHeads == 0 && max_seq_len > dense_rows_limit) {
    // dense: kDenseTargetBlocks workgroups, at least 128 tokens per split
    const uint32_t groups = batch * (num_heads / kDenseHeads);
    // grouped queries read 1/gq of the bytes per unit of arithmetic: there the kernel is bound by
    // instruction issue, not by the memory system, and wants every CU busy
    const uint32_t target_blocks = gqa_kernel ? kDenseGqaTargetBlocks : kDenseTargetBlocks;
    uint32_t n_split = (target_blocks + groups - 1) / groups;
    n_split = n_split > kMaxSplits ? kMaxSplits : n_split;
    uint32_t rows_per_split = (max_seq_len + n_split - 1) / n_split;
    rows_per_split = rows_per_split < 128 ? 128 : rows_per_split;
    // whole tiles: 32 tokens per round of the vector kernels, 16 * group tokens (at most 128) per
    // round of a workgroup of the matrix-core kernel
    const bool gqa_mfma = gqa_kernel && !(flags & ADAMAS_F_NO_MFMA);
    const uint32_t round_rows = gqa_mfma ? 128u : kDenseRowsPerIter;
    rows_per_split = (rows_per_split + round_rows - 1) / round_rows * round_rows;
    n_split = (max_seq_len + rows_per_split - 1) / rows_per_split;
    float* partial = nullptr;
    uint32_t* counters = nullptr;
    if (n_split > 1) {
      const WorkspaceLayout w = workspace_layout(batch, num_heads, 0, 0);
      if (!workspace || workspace_bytes < w.dist_off) return ADAMAS_E_WORKSPACE;
      if (reinterpret_cast<uintptr_t>(workspace) & 255) return ADAMAS_E_ALIGN;
      counters = reinterpret_cast<uint32_t*>(static_cast<char*>(workspace) + w.counters_off);
      partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + w.partial_off);
    }
    // from kDenseDeferredSplits splits on, the merge of the splits is a second short launch
    const uint32_t deferred = n_split >= kDenseDeferredSplits ? 1u : 0u;
    auto merge_launch = [&]() -> int {
      if (!deferred) return 0;
      if (bf16)
        hipLaunchKernelGGL(merge_splits_kernel<true>, dim3(num_heads, batch),
                           dim3(kMergeGroups * kHeadDim), 0, static_cast<hipStream_t>(stream),
                           partial, static_cast<__half*>(out), num_heads, n_split);
      else
        hipLaunchKernelGGL(merge_splits_kernel<false>, dim3(num_heads, batch),
                           dim3(kMergeGroups * kHeadDim), 0, static_cast<hipStream_t>(stream),
                           partial, static_cast<__half*>(out), num_heads, n_split);
      ADAMAS_RETURN_IF_LAUNCH_FAILED();
      return 0;
    };
    if (gqa_mfma) {
#define ADAMAS_LAUNCH_DENSE_GQA_MFMA(G, BF)                                                      \
  hipLaunchKernelGGL((dense_decode_gqa_mfma_kernel<G, BF>),                                      \
                     dim3(n_split, num_heads / kDenseHeads, batch), dim3(kDenseThreads), 0,      \
                     static_cast<hipStream_t>(stream), static_cast<const __half*>(q),            \
                     static_cast<const __half*>(kv_data), page_indices, page_indptr, seq_lens,   \
                     static_cast<__half*>(out), partial, counters, num_heads, num_kv_heads,      \
                     page_size, scale_log2, rows_per_split, lay, deferred)
      if (gq == 2) {
        if (bf16) ADAMAS_LAUNCH_DENSE_GQA_MFMA(2, true);
        else ADAMAS_LAUNCH_DENSE_GQA_MFMA(2, false);
      } else if (gq == 4) {
        if (bf16) ADAMAS_LAUNCH_DENSE_GQA_MFMA(4, true);
        else ADAMAS_LAUNCH_DENSE_GQA_MFMA(4, false);
      } else {
        if (bf16) ADAMAS_LAUNCH_DENSE_GQA_MFMA(8, true);
        else ADAMAS_LAUNCH_DENSE_GQA_MFMA(8, false);
      }
#undef ADAMAS_LAUNCH_DENSE_GQA_MFMA
      ADAMAS_RETURN_IF_LAUNCH_FAILED();
      return merge_launch();
    }
    if (gqa_kernel) {
#define ADAMAS_LAUNCH_DENSE_GQA(G, TILE, BF)                                                     \
  hipLaunchKernelGGL((dense_decode_gqa_kernel<G, TILE, BF>),                                     \
                     dim3(n_split, num_heads / kDenseHeads, batch), dim3(kDenseThreads), 0,      \
                     static_cast<hipStream_t>(stream), static_cast<const __half*>(q),            \
                     static_cast<const __half*>(kv_data), page_indices, page_indptr, seq_lens,   \
                     static_cast<__half*>(out), partial, counters, num_heads, num_kv_heads,      \
                     page_size, scale_log2, rows_per_split, lay, deferred)
      if (gq == 2) {
        if (bf16) ADAMAS_LAUNCH_DENSE_GQA(2, 8, true);
        else ADAMAS_LAUNCH_DENSE_GQA(2, 8, false);
      } else if (gq == 4) {
        if (bf16) ADAMAS_LAUNCH_DENSE_GQA(4, 8, true);
        else ADAMAS_LAUNCH_DENSE_GQA(4, 8, false);
      } else {
        if (bf16) ADAMAS_LAUNCH_DENSE_GQA(8, 4, true);
        else ADAMAS_LAUNCH_DENSE_GQA(8, 4, false);
      }
#undef ADAMAS_LAUNCH_DENSE_GQA
      ADAMAS_RETURN_IF_LAUNCH_FAILED();
      return merge_launch();
    }
#define ADAMAS_LAUNCH_DENSE(BF)                                                                  \
  hipLaunchKernelGGL(dense_decode_kernel<BF>, dim3(n_split, num_heads / kDenseHeads, batch),     \
                     dim3(kDenseThreads), 0, static_cast<hipStream_t>(stream),                   \
                     static_cast<const __half*>(q), static_cast<const __half*>(kv_data),         \
                     page_indices, page_indptr, seq_lens, static_cast<__half*>(out), partial,    \
                     counters, num_heads, num_kv_heads, page_size, scale_log2, rows_per_split,   \
                     lay, deferred)
    if (bf16) ADAMAS_LAUNCH_DENSE(true);
    else ADAMAS_LAUNCH_DENSE(false);
#undef ADAMAS_LAUNCH_DENSE
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
    return merge_launch();
  }
  const uint32_t n_rows = sel_idx ? n_sel + 1u : max_seq_len;
  // one round of loads per split (see the rule at kTile; up to 128 rows that is a single
  // split, which needs no workspace), more where that would take more than kMaxSplits splits
  const uint32_t threads = n_rows <= 64 ? 256u : n_rows <= 512 ? 512u : 1024u;
  const uint32_t tile = n_rows <= 128 ? 4u : n_rows <= 2048 ? 2u : 4u;
  const uint32_t rows_per_iter = threads / 16u * tile;
  uint32_t rows_per_split = rows_per_iter;
  uint32_t n_split = (n_rows + rows_per_split - 1) / rows_per_split;
  if (n_split > kMaxSplits) {
    rows_per_split = ((n_rows + kMaxSplits - 1) / kMaxSplits + rows_per_iter - 1) / rows_per_iter *
                     rows_per_iter;
    n_split = (n_rows + rows_per_split - 1) / rows_per_split;
  }
  float* partial = nullptr;
  uint32_t* counters = nullptr;
  if (n_split > 1) {
    const WorkspaceLayout w = workspace_layout(batch, num_heads, 0, 0);
    if (!workspace || workspace_bytes < w.dist_off) return ADAMAS_E_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return ADAMAS_E_ALIGN;
    counters = reinterpret_cast<uint32_t*>(static_cast<char*>(workspace) + w.counters_off);
    partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + w.partial_off);
  }
  // from kDeferredMergeSplits splits on, the merge is a second short launch
  const uint32_t deferred = n_split >= kDeferredMergeSplits ? 1u : 0u;
#define ADAMAS_LAUNCH_SPARSE_T(BF, HND, T, TILE)                                                 \
  hipLaunchKernelGGL((sparse_decode_kernel<BF, HND, T, TILE>), dim3(n_split, num_heads, batch),  \
                     dim3(T), 0, static_cast<hipStream_t>(stream),                               \
                     static_cast<const __half*>(q), static_cast<const __half*>(kv_data),         \
                     page_indices, page_indptr, seq_lens, sel_idx, sel_stride, n_sel,            \
                     static_cast<__half*>(out), partial, counters, num_heads, num_kv_heads,      \
                     page_size, scale_log2, rows_per_split, deferred)
#define ADAMAS_LAUNCH_SPARSE_L(BF, HND)          \
  if (threads == 256) {                          \
    ADAMAS_LAUNCH_SPARSE_T(BF, HND, 256, 4);     \
  } else if (threads == 512 && tile == 4) {      \
    ADAMAS_LAUNCH_SPARSE_T(BF, HND, 512, 4);     \
  } else if (threads == 512) {                   \
    ADAMAS_LAUNCH_SPARSE_T(BF, HND, 512, 2);     \
  } else if (tile == 2) {                        \
    ADAMAS_LAUNCH_SPARSE_T(BF, HND, 1024, 2);    \
  } else {                                       \
    ADAMAS_LAUNCH_SPARSE_T(BF, HND, 1024, 4);    \
  }
#define ADAMAS_LAUNCH_SPARSE(BF)        \
  if (flags & ADAMAS_F_HND) {           \
    ADAMAS_LAUNCH_SPARSE_L(BF, true)    \
  } else {                              \
    ADAMAS_LAUNCH_SPARSE_L(BF, false)   \
  }
  if (bf16) {
    ADAMAS_LAUNCH_SPARSE(true)
  } else {
    ADAMAS_LAUNCH_SPARSE(false)
  }
#undef ADAMAS_LAUNCH_SPARSE
#undef ADAMAS_LAUNCH_SPARSE_L
#undef ADAMAS_LAUNCH_SPARSE_T
  ADAMAS_RETURN_IF_LAUNCH_FAILED();
  if (deferred) {
    if (bf16)
      hipLaunchKernelGGL(merge_splits_kernel<true>, dim3(num_heads, batch), dim3(kMergeGroups * kHeadDim), 0,
                         static_cast<hipStream_t>(stream), partial, static_cast<__half*>(out),
                         num_heads, n_split);
    else
      hipLaunchKernelGGL(merge_splits_kernel<false>, dim3(num_heads, batch), dim3(kMergeGroups * kHeadDim), 0,
                         static_cast<hipStream_t>(stream), partial, static_cast<__half*>(out),
                         num_heads, n_split);
    ADAMAS_RETURN_IF_LAUNCH_FAILED();
  }
  return 0;
}

extern "C" int adamas_sparse_decode_f(const void* q, const void* kv_data,
                                      const int32_t* page_indices, const int32_t* page_indptr,
                                      const int32_t* seq_lens, const int32_t* sel_idx,
                                      int64_t sel_stride, uint32_t n_sel, void* out,
                                      void* workspace, size_t workspace_bytes, uint32_t batch,
                                      uint32_t num_heads, uint32_t num_kv_heads, uint32_t head_dim,
                                      uint32_t page_size, float sm_scale, uint32_t max_seq_len,
                                      uint32_t flags, adamas_stream_t stream) {
  return sparse_decode_impl(q, kv_data, page_indices, page_indptr, seq_lens, sel_idx, sel_stride,
                            n_sel, out, workspace, workspace_bytes, batch, num_heads, num_kv_heads,
                            head_dim, page_size, sm_scale, max_seq_len, stream, flags);
}

extern "C" int adamas_sparse_decode(const void* q, const void* kv_data,
                                    const int32_t* page_indices, const int32_t* page_indptr,
                                    const int32_t* seq_lens, const int32_t* sel_idx,
                                    int64_t sel_stride, uint32_t n_sel, void* out, void* workspace,
                                    size_t workspace_bytes, uint32_t batch, uint32_t num_heads,
                                    uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size,
                                    float sm_scale, uint32_t max_seq_len, adamas_stream_t stream) {
  return sparse_decode_impl(q, kv_data, page_indices, page_indptr, seq_lens, sel_idx, sel_stride,
                            n_sel, out, workspace, workspace_bytes, batch, num_heads, num_kv_heads,
                            head_dim, page_size, sm_scale, max_seq_len, stream, 0u);
}

extern "C" int adamas_version(void) { return 100; }

extern "C" const char* adamas_error_string(int code) {
  switch (code) {
    case 0: return "success";
    case ADAMAS_E_BADARG: return "adamas: bad argument (null pointer, zero or inconsistent size)";
    case ADAMAS_E_UNSUPPORTED: return "adamas: unsupported shape (head_dim must be 128, num_heads a multiple of 32)";
    case ADAMAS_E_WORKSPACE: return "adamas: workspace missing or too small";
    case ADAMAS_E_ALIGN: return "adamas: pointer or stride not aligned as documented";
    case ADAMAS_E_SCRATCH: return "adamas: sizes beyond the static scratch (ADAMAS_STATIC_SCRATCH_BYTES) of adamas_decode_step_noalloc";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "adamas: unknown error code";
}
