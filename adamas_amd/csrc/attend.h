// Shared pieces of the paged decode-attention kernels (gfx950).
//
// A K or V row of one head is 128 fp16 (or bf16) = 256 bytes = 16 lanes x 128-bit: a group of 16 lanes owns a
// row and a lane owns 8 channels.  Each group walks its rows in tiles: all K and V loads of a tile
// are issued before any of them is used, the dot products are reduced over the 16 lanes, and an
// fp32 online softmax (base 2) keeps (m, l, o[8]) per lane.  Groups are merged through LDS.
#pragma once

#include "common.h"

namespace adamas {

constexpr float kNegBig = -1.0e30f;

// 2^x as the bare hardware instruction.  The library routine exp2f() wraps it in five more
// instructions that only matter for results below 2^-126, which are weights of zero here; for every
// other argument the bits are the same.  The attention kernels are bound by instruction issue, and a
// softmax has many of these.
__device__ __forceinline__ float exp2_raw(float x) { return __builtin_amdgcn_exp2f(x); }

template <bool kBf16 = false>
__device__ __forceinline__ void unpack8(uint4 r, float f[8]) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) unpack2<kBf16>(w[i], f[2 * i], f[2 * i + 1]);
}

// sum over the 16 lanes of a group (a DPP row), result in every lane; no LDS crossbar involved
template <int kCtrl>
__device__ __forceinline__ float dpp_add_step(float v) {
  const int o = __builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xF, 0xF, false);
  return v + __int_as_float(o);
}

__device__ __forceinline__ float group16_sum(float v) {
  v = dpp_add_step<0xB1>(v);   // quad_perm [1,0,3,2]: pairs
  v = dpp_add_step<0x4E>(v);   // quad_perm [2,3,0,1]: quads
  v = dpp_add_step<0x141>(v);  // row_half_mirror: lane i + lane 7-i of each half row
  v = dpp_add_step<0x140>(v);  // row_mirror: lane i + lane 15-i
  return v;
}

// Where one head's rows live: everything needed to turn a token position into K and V addresses.
// A K row is addressed as kv_data + row * tok_stride + head_off with row = page * row_mult + slot:
//   pages [2][page_size][heads][128] (NHD): tok_stride = heads*128, head_off = head*128,
//                                           row_mult = 2*page_size
//   pages [2][heads][page_size][128] (HND): tok_stride = 128, head_off = head*page_size*128,
//                                           row_mult = 2*page_size*heads
// and the V row of the same token lies v_delta = page_size*heads*128 elements further in both.
struct HeadKV {
  const __half* kv_data;   // page pool of the layer
  const int32_t* table;    // page table of the sequence
  size_t head_off;         // offset of the head (see above) + 8 * lane_in_group
  uint32_t tok_stride;     // elements between adjacent slots of a page (32 bits: row * tok_stride
                           // is then one 32 x 32 -> 64 bit multiply-add per row address)
  size_t v_delta;          // K -> V inside a page
  uint32_t row_mult;       // rows per page
  uint32_t page_size;
  int32_t seq_len;
};

// The constants of a page layout, worked out on the host and passed to the kernels by value.
struct KvLayout {
  uint32_t tok_stride;     // elements between adjacent slots
  uint32_t head_stride;    // elements between adjacent heads
  uint32_t rows_per_page;  // row_mult
  uint32_t v_delta;        // K -> V inside a page: page_size * heads * 128
};

inline KvLayout make_kv_layout(bool hnd, uint32_t page_size, uint32_t num_kv_heads) {
  KvLayout l;
  l.tok_stride = hnd ? kHeadDim : num_kv_heads * kHeadDim;
  l.head_stride = hnd ? page_size * kHeadDim : kHeadDim;
  l.rows_per_page = hnd ? 2u * page_size * num_kv_heads : 2u * page_size;
  l.v_delta = page_size * num_kv_heads * kHeadDim;
  return l;
}

// the same with the layout known at compile time (the kernels of the decode step: the NHD instance
// keeps its strides as shifts of num_kv_heads instead of multiplications by launch arguments)
template <bool kHnd>
__device__ __forceinline__ void set_kv_layout_static(HeadKV& kv, uint32_t kv_head, uint32_t c,
                                                     uint32_t num_kv_heads, uint32_t page_size) {
  if (kHnd) {
    kv.tok_stride = kHeadDim;
    kv.head_off = static_cast<size_t>(kv_head) * page_size * kHeadDim + 8 * c;
    kv.row_mult = 2u * page_size * num_kv_heads;
    kv.v_delta = static_cast<size_t>(page_size) * num_kv_heads * kHeadDim;
  } else {
    kv.tok_stride = num_kv_heads * kHeadDim;
    kv.head_off = static_cast<size_t>(kv_head) * kHeadDim + 8 * c;
    kv.row_mult = 2u * page_size;
    kv.v_delta = static_cast<size_t>(page_size) * kv.tok_stride;
  }
  kv.page_size = page_size;
}

__device__ __forceinline__ void set_kv_layout(HeadKV& kv, const KvLayout& lay, uint32_t kv_head,
                                              uint32_t c, uint32_t page_size) {
  kv.tok_stride = lay.tok_stride;
  kv.head_off = static_cast<size_t>(kv_head) * lay.head_stride + 8 * c;
  kv.row_mult = lay.rows_per_page;
  kv.v_delta = lay.v_delta;
  kv.page_size = page_size;
}

// Online-softmax state of one lane: running max, running denominator, 8 output channels.
struct SoftmaxState {
  float m = kNegBig;
  float l = 0.f;
  float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
};

// Processes rows [row_begin, row_end) of the list described by pos_of(row).  Group g of kGroups
// takes rows row_begin + g, + kGroups, ...
//   kRowIndex == false: pos_of gives a token position (negative or >= seq_len = skip) that is
//                       translated through the page table;
//   kRowIndex == true : pos_of gives the K row index page*row_mult + slot directly (negative =
//                       skip), no table access.
//   kLoadAlways: no branch around the loads.  A slot past row_end reads the last list entry again
//                       and an unused entry reads row 0 of the pool (kRowIndex) or token 0 of the
//                       sequence, all with weight zero: the loads cost less than the branches and
//                       the zeroed registers they replace.  A sequence without tokens is left
//                       before the first load.
template <int kGroups, int kTile, bool kRowIndex = false, bool kBf16 = false, bool kLoadAlways = false,
          typename PosFn>
__device__ __forceinline__ void attend_rows(const HeadKV& kv, const float (&qf)[8], uint32_t g,
                                            uint32_t row_begin, uint32_t row_end, PosFn&& pos_of,
                                            SoftmaxState& st) {
  if (kLoadAlways && !kRowIndex && kv.seq_len <= 0) return;  // no token a clamped position could name
  for (uint32_t base = row_begin; base < row_end; base += kGroups * kTile) {
    uint4 kr[kTile], vr[kTile];
    bool valid[kTile];
#pragma unroll
    for (int i = 0; i < kTile; ++i) {
      const uint32_t r = base + i * kGroups + g;
      if (kLoadAlways) {
        const int32_t pos = pos_of(min(r, row_end - 1u));
        uint32_t row;
        if (kRowIndex) {
          valid[i] = r < row_end && pos >= 0;
          row = static_cast<uint32_t>(max(pos, 0));
        } else {
          valid[i] = r < row_end && pos >= 0 && pos < kv.seq_len;
          const uint32_t pc = static_cast<uint32_t>(min(max(pos, 0), kv.seq_len - 1));
          const uint32_t lp = pc / kv.page_size;
          row = static_cast<uint32_t>(kv.table[lp]) * kv.row_mult + (pc - lp * kv.page_size);
        }
        const __half* kp = kv.kv_data + static_cast<size_t>(row) * kv.tok_stride + kv.head_off;
        kr[i] = *reinterpret_cast<const uint4*>(kp);
        vr[i] = *reinterpret_cast<const uint4*>(kp + kv.v_delta);
        continue;
      }
      const int32_t pos = (r < row_end) ? pos_of(r) : -1;
      valid[i] = pos >= 0 && (kRowIndex || pos < kv.seq_len);
      kr[i] = make_uint4(0, 0, 0, 0);
      vr[i] = make_uint4(0, 0, 0, 0);
      if (valid[i]) {
        uint32_t row;  // K row indices are below 2^31 everywhere (the row lists are int32)
        if (kRowIndex) {
          row = static_cast<uint32_t>(pos);
        } else {
          const uint32_t lp = static_cast<uint32_t>(pos) / kv.page_size;
          const uint32_t slot = static_cast<uint32_t>(pos) - lp * kv.page_size;
          row = static_cast<uint32_t>(kv.table[lp]) * kv.row_mult + slot;
        }
        const __half* kp = kv.kv_data + static_cast<size_t>(row) * kv.tok_stride + kv.head_off;
        kr[i] = *reinterpret_cast<const uint4*>(kp);
        vr[i] = *reinterpret_cast<const uint4*>(kp + kv.v_delta);
      }
    }
    float s[kTile];
    float m_new = st.m;
#pragma unroll
    for (int i = 0; i < kTile; ++i) {
      float kf[8];
      unpack8<kBf16>(kr[i], kf);
      float d = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) d += qf[j] * kf[j];
      d = group16_sum(d);
      s[i] = valid[i] ? d : kNegBig;
      m_new = fmaxf(m_new, s[i]);
    }
    const float alpha = exp2_raw(st.m - m_new);
    st.l *= alpha;
#pragma unroll
    for (int j = 0; j < 8; ++j) st.o[j] *= alpha;
#pragma unroll
    for (int i = 0; i < kTile; ++i) {
      const float p = valid[i] ? exp2_raw(s[i] - m_new) : 0.f;
      st.l += p;
      float vf[8];
      unpack8<kBf16>(vr[i], vf);
#pragma unroll
      for (int j = 0; j < 8; ++j) st.o[j] += p * vf[j];
    }
    st.m = m_new;
  }
}

// LDS of the group merge: one partial state per WAVE (the four 16-lane groups of a wave are folded
// with lane shuffles first).
template <int kGroups>
struct MergeShared {
  static constexpr int kWavesM = kGroups / 4;
  float m[kWavesM];
  float l[kWavesM];
  float o[kWavesM][kHeadDim];
};

// Folds the state of the lane `delta` lanes away into this lane's state (both hold the same channels).
__device__ __forceinline__ void fold_state(SoftmaxState& st, int delta) {
  const float m_o = __shfl_xor(st.m, delta);
  const float l_o = __shfl_xor(st.l, delta);
  const float m_n = fmaxf(st.m, m_o);
  const float a = exp2_raw(st.m - m_n), b = exp2_raw(m_o - m_n);
  st.l = st.l * a + l_o * b;
#pragma unroll
  for (int j = 0; j < 8; ++j) st.o[j] = st.o[j] * a + __shfl_xor(st.o[j], delta) * b;
  st.m = m_n;
}

// Merges the kGroups group states of a workgroup (kGroups / 4 waves).  After the call the threads
// tid < 128 hold, for channel tid, the merged maximum M, denominator L and numerator O.
template <int kGroups>
__device__ __forceinline__ void merge_groups(SoftmaxState st, uint32_t g, uint32_t c,
                                             uint32_t tid, MergeShared<kGroups>& sh, float& M,
                                             float& L, float& O) {
  constexpr int kWavesM = kGroups / 4;
  fold_state(st, 16);
  fold_state(st, 32);  // every lane now holds the state of its wave for channels 8c .. 8c+7
  const uint32_t w = g >> 2;
  if ((g & 3u) == 0) {
    if (c == 0) {
      sh.m[w] = st.m;
      sh.l[w] = st.l;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) sh.o[w][8 * c + j] = st.o[j];
  }
  __syncthreads();
  M = kNegBig;
  L = 0.f;
  O = 0.f;
  if (tid < kHeadDim) {
#pragma unroll
    for (int i = 0; i < kWavesM; ++i) M = fmaxf(M, sh.m[i]);
#pragma unroll
    for (int i = 0; i < kWavesM; ++i) {
      const float wgt = exp2_raw(sh.m[i] - M);
      L += sh.l[i] * wgt;
      O += sh.o[i][tid] * wgt;
    }
  }
}

// query fragment of a lane: 8 channels, pre-multiplied by sm_scale * log2(e)
template <bool kBf16 = false>
__device__ __forceinline__ void load_query(const __half* q_row, uint32_t c, float scale_log2,
                                           float (&qf)[8]) {
  unpack8<kBf16>(*reinterpret_cast<const uint4*>(q_row + 8 * c), qf);
#pragma unroll
  for (int i = 0; i < 8; ++i) qf[i] *= scale_log2;
}

}  // namespace adamas
