/*
 * adamas_hip.h - C ABI of libadamas_hip.so: the MI355X (gfx950) implementation of the Adamas
 * decode-time sparse-attention path.
 *
 * Every entry point is a plain C function: device pointers, sizes and a HIP stream.  No torch types,
 * no hidden allocation, no hidden state: all inputs, outputs and workspaces are allocated by the
 * caller.  Every function enqueues its kernels on `stream` and returns without synchronising, so the
 * calls can be recorded into a HIP graph.  Return value: 0 on success, a positive hipError_t if the
 * HIP runtime reported an error, or one of the negative ADAMAS_E_* codes below for argument errors.
 *
 * Each declaration cites the interface of the reference (FibonaccciYan/Adamas) that it replaces.
 *
 * Data formats (all little endian, all device memory):
 *   KV page pool of one layer   fp16 [num_pages][2][page_size][num_kv_heads][128] (0 = K, 1 = V; "NHD")
 *   code page pool of one layer u16  [num_pages][page_size][num_kv_heads][16]
 *       word g of (token, head) = sum_{i<8} code(channel 8g+i) << (2i), code in {0,1,2,3}
 *       code(v) = (v > -10) + (v > 0) + (v > 10) applied to the Hadamard-transformed key
 *   page table                  int32 page_indices[], int32 page_indptr[batch+1]:
 *       logical page p of sequence b is physical page page_indices[page_indptr[b] + p] in BOTH pools
 *   seq_lens                    int32 [batch]: tokens held by each sequence, current token included
 *   token t of sequence b lives in physical page page_indices[page_indptr[b] + t / page_size],
 *   slot t % page_size.
 *
 * Grouped-query attention: num_heads query heads share num_kv_heads key/value heads (num_heads a
 * multiple of num_kv_heads; equal in the reference, which asserts it,
 * kernels/include/decode/decode_handler.cuh:83).  Query head h uses key/value head
 * h / (num_heads / num_kv_heads): its distances are taken against that head's codes, its selection is
 * its own, its attention reads that head's rows.  The estimator and the decode step want
 * num_heads * (num_heads / num_kv_heads) < 65536 (ADAMAS_E_UNSUPPORTED otherwise).
 */
#ifndef ADAMAS_HIP_H_
#define ADAMAS_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Opaque HIP stream handle (hipStream_t); NULL is the default stream. */
typedef void* adamas_stream_t;

#define ADAMAS_HEAD_DIM 128
#define ADAMAS_CODE_WORDS 16 /* uint16 words of packed code per (token, head) */

/* Negative error codes (positive values are hipError_t). */
#define ADAMAS_E_BADARG (-1)      /* null pointer, zero size, inconsistent sizes          */
#define ADAMAS_E_UNSUPPORTED (-2) /* head_dim != 128, num_heads not a multiple of 8, ... */
#define ADAMAS_E_WORKSPACE (-3)   /* workspace too small                                  */
#define ADAMAS_E_ALIGN (-4)       /* pointer or stride not aligned as documented          */
#define ADAMAS_E_SCRATCH (-5)     /* sizes beyond the static scratch of adamas_decode_step_noalloc */

/* Bytes of device memory adamas_decode_step_noalloc works in (held by every GPU the library runs on). */
#define ADAMAS_STATIC_SCRATCH_BYTES (24u << 20)

/* flags for the append / code-generation entry points */
#define ADAMAS_F_CODE_FROM_FP32 1u /* bucketize the fp32 butterfly output instead of its fp16 rounding */
#define ADAMAS_F_BF16 2u           /* q, k, v, h and the KV cache hold bfloat16 instead of fp16          */
#define ADAMAS_F_HND 4u            /* KV pages are [2][heads][page_size][128] instead of
                                      [2][page_size][heads][128]; the code cache keeps its layout      */
#define ADAMAS_F_NO_MFMA 8u        /* adamas_sparse_decode_f, dense mode with 2, 4 or 8 query heads per
                                      key/value head: the vector-ALU kernel instead of the matrix-core
                                      one (same results within tolerance; kept for measurement)       */

/* output formats of adamas_estimate / key modes of adamas_topk */
#define ADAMAS_DIST_FP16 0u /* integer distance stored as fp16 (the reference's output dtype) */
#define ADAMAS_DIST_U16 1u  /* integer distance stored as uint16                               */
#define ADAMAS_KEY_FP16_GENERIC 0u /* arbitrary finite fp16 values                              */
#define ADAMAS_KEY_FP16_INT 1u     /* fp16 holding integers in [0, 511]                         */
#define ADAMAS_KEY_U16_INT 2u      /* uint16 integers in [0, 511]                               */

/* Library version, major*10000 + minor*100 + patch. */
int adamas_version(void);

/* Text for a return code of this library (static storage). */
const char* adamas_error_string(int code);

/*
 * Hadamard transform over the last axis (length 128) of n_rows rows of fp16, fp32 butterfly with the
 * canonical stage order (strides 1,2,...,64; (a+b, a-b)), result * scale rounded to fp16.
 * `out` may alias `x` (in place).  x and out must be 16-byte aligned (ADAMAS_E_ALIGN otherwise).
 * Replaces: faster_hadamard_transform.hadamard_transform(x, inplace) as called at
 * adamas/models/Adamas.py:120 and :150 (third-party module, absent from the reference tree).
 */
int adamas_hadamard(const void* x, void* out, uint64_t n_rows, float scale, adamas_stream_t stream);

/*
 * Entry points with a `flags` argument (suffix _f): the entry point of the same name with
 *   ADAMAS_F_BF16 : bfloat16 in place of fp16 wherever it reads or writes float data (q, k, v, h,
 *                   the KV cache, the attention output); codes, distances, selections and all
 *                   arithmetic (fp32) are unchanged;
 *   ADAMAS_F_HND  : the other page layout of the KV cache (see the flag).
 * The un-suffixed entry points are flags = 0; the append entry points have taken flags all along;
 * estimate and top-k see neither float data nor KV pages.  Flags an entry point does not know give
 * ADAMAS_E_BADARG.  The reference dispatches fp16 only
 * (kernels/include/pytorch_extension_utils.h:25-37) and instantiates the NHD layout only
 * (adamas/ops/csrc/approx_attn.cu:107-123), so these have no counterpart there.
 */
int adamas_hadamard_f(const void* x, void* out, uint64_t n_rows, float scale, uint32_t flags,
                      adamas_stream_t stream);

/*
 * Pack integer-valued fp16 codes (values 0..3) into 2-bit words, LSB first.
 * h [n_rows][128] fp16 -> o [n_rows][16] u16.
 * Replaces: _kernels.pack_2bit, adamas/ops/csrc/bsk_ops.h:29-31 (kernel HPack2bitKernel,
 * kernels/include/decode/decode_page.cuh:751-772).
 */
int adamas_pack_2bit(const void* h, void* o, uint64_t n_rows, adamas_stream_t stream);
int adamas_pack_2bit_f(const void* h, void* o, uint64_t n_rows, uint32_t flags,
                       adamas_stream_t stream);

/*
 * Decode-step append for `batch` sequences: writes the new k and v row of every sequence at position
 * seq_lens[b]-1 of its paged KV cache, writes the 2-bit code of the new key into the code cache and
 * returns the 2-bit code of the query in q_code_out [batch][num_heads][16] u16.  q is
 * [batch][num_heads][128], k and v [batch][num_kv_heads][128].
 *   h != NULL : h is batch*num_heads rows of Hadamard(q) followed by batch*num_kv_heads rows of
 *               Hadamard(k), fp16, computed by the caller (the reference's calling convention,
 *               Hadamard(cat(q, k))); q may be NULL.
 *   h == NULL : q and k are transformed in the kernel (fused path), `scale` and `flags` apply.
 * Replaces: _kernels.append_kv_cache_decode, adamas/ops/csrc/bsk_ops.h:70-84
 * (kernel AppendPagedKVCacheDecodeKernel, kernels/include/decode/decode_page.cuh:421-469).
 */
int adamas_append_decode(const void* q, const void* k, const void* v, const void* h,
                         void* q_code_out, void* kv_data, void* code_data,
                         const int32_t* page_indices, const int32_t* page_indptr,
                         const int32_t* seq_lens, uint32_t batch, uint32_t num_heads,
                         uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size, float scale,
                         uint32_t flags, adamas_stream_t stream);

/*
 * Prefill append for ONE sequence: writes n_tokens rows of k and v at positions
 * [start_pos, start_pos + n_tokens) and the 2-bit code of every key.
 *   h != NULL : h [n_tokens][num_heads][128] fp16 = Hadamard(k) computed by the caller.
 *   h == NULL : k is transformed in the kernel.
 * num_heads here is the number of key/value heads (the rows of k, v and h).
 * page_table points at the first page-table entry of this sequence (n_table_entries of them).
 * k, v, h and kv_data must be 16-byte aligned (ADAMAS_E_ALIGN otherwise).
 * Replaces: _kernels.append_kv_cache_prefill, adamas/ops/csrc/bsk_ops.h:55-68
 * (kernel AppendPagedKVCachePrefillKernel, kernels/include/decode/decode_page.cuh:492-548).
 */
int adamas_append_prefill(const void* k, const void* v, const void* h, uint32_t n_tokens,
                          uint32_t start_pos, void* kv_data, void* code_data,
                          const int32_t* page_table, uint32_t n_table_entries, uint32_t num_heads,
                          uint32_t head_dim, uint32_t page_size, float scale, uint32_t flags,
                          adamas_stream_t stream);

/*
 * Distance estimator: out[b][h][t] = sum_{j<128} |code_q[b][h][j] - code_k[b][t][h][j]| (true integer
 * L1, 0..384) for every past token t < seq_lens[b]-1 (the current token is excluded).
 * q_code [batch][num_heads][16] u16.  out element (b,h,t) is at out + b*out_batch_stride +
 * h*out_head_stride + t (strides in elements, 2 bytes each); a head stride that is a multiple of 8
 * with a 16-byte aligned `out` enables vector stores.  out_format: ADAMAS_DIST_FP16 or ADAMAS_DIST_U16.
 * max_seq_len >= max_b seq_lens[b] sizes the grid (host-side hint, seq_lens stays on the device).
 * Replaces: _kernels.estimate_attn_score, adamas/ops/csrc/bsk_ops.h:46-53 (kernel
 * MaxPossibleSampleWithPagedKVCacheKernel, kernels/include/decode/decode_attn.cuh:300-443, distance
 * loop :172-223 - whose live XOR-weighted metric is replaced by the true L1 of the reference's
 * PyTorch path, evaluation/adamas_attention.py:222, adamas/tests/test_estimate.py:57-61).
 */
int adamas_estimate(const void* q_code, const void* code_data, const int32_t* page_indices,
                    const int32_t* page_indptr, const int32_t* seq_lens, void* out,
                    int64_t out_batch_stride, int64_t out_head_stride, uint32_t out_format,
                    uint32_t batch, uint32_t num_heads, uint32_t num_kv_heads, uint32_t page_size,
                    uint32_t max_seq_len, adamas_stream_t stream);

/*
 * Row-wise selection of the k smallest values, ties broken by the lowest index (deterministic).
 * values: num_rows rows of 2-byte keys, row r starts at values + r*row_stride (elements).
 * Row length: n_max for every row when seq_lens == NULL, else seq_lens[r / rows_per_seq] + len_delta
 * (must be <= n_max).  A row shorter than k selects all of its elements and pads with -1.
 * in_idx (optional, same row layout with in_idx_stride): values written to out_idx are
 * in_idx[r][e] instead of the position e.  out_idx [num_rows][out_stride] int32 receives k entries per
 * row: first the elements strictly below the threshold value in index order, then the tied ones in
 * index order.  out_vals (optional, 2-byte elements, same layout as out_idx) receives the keys.
 * key_mode: one of ADAMAS_KEY_*.  in_idx entries must be non-negative.
 * workspace: adamas_topk_workspace_bytes(num_rows, n_max, k) bytes, 256-byte aligned, zero-filled
 * once after allocation (the library leaves it reusable).  With the integer key modes it holds, for
 * k <= 255, the candidate lists of a two-level selection (one wave per chunk of 512-2048 keys writes
 * a short list of the chunk's smallest keys, then one workgroup per row selects among the listed
 * keys and goes back to the row for a chunk whose list ran out) and, for larger k and rows longer
 * than 4096, one 512-bin histogram per chunk of 1024 keys (threshold and positions are then read off
 * the histograms).  out_vals holds the key
 * in the format of the input (integer keys are clamped to 511).  It may be NULL for rows of at most
 * 32768 elements or k > 1024: those are served by one launch with one workgroup per row, which is
 * several times slower for long rows.  The reference passes a scratch buffer too (`buf`).
 * Replaces: _kernels.topk_filtering, adamas/ops/csrc/bsk_ops.h:39-44 (decode_select_k,
 * kernels/include/topk/decode_select_k.cuh:26-61, RAFT radix select with greater=false).
 */
int adamas_topk(const void* values, int64_t row_stride, uint32_t n_max, const int32_t* seq_lens,
                uint32_t rows_per_seq, int32_t len_delta, const int32_t* in_idx,
                int64_t in_idx_stride, uint32_t num_rows, uint32_t k, int32_t* out_idx,
                void* out_vals, int64_t out_stride, uint32_t key_mode, void* workspace,
                size_t workspace_bytes, adamas_stream_t stream);

/*
 * Measurement aid, no counterpart in the reference: one launch that reads `bytes` bytes at `data`
 * (16-byte aligned, a multiple of 16) with 128-bit loads, 256 workgroups, 16 loads in flight per
 * lane, and computes nothing.  Its duration over a code cache is the rate the memory system gives a
 * kernel that streams those bytes once: the practical ceiling the estimator is compared with.
 * sink (optional, 4 bytes) is never written for ordinary data.
 */
int adamas_read_probe(const void* data, size_t bytes, void* sink, adamas_stream_t stream);

/* Bytes of workspace adamas_topk needs for these sizes (see adamas_topk). */
size_t adamas_topk_workspace_bytes(uint32_t num_rows, uint32_t n_max, uint32_t k);

/*
 * Bytes of workspace adamas_sparse_decode / adamas_decode_step need for these sizes.  The workspace
 * must be zero-filled once after allocation; the library leaves it in a reusable state.  Calls that
 * share a workspace must be ordered (same stream, or events between streams): it holds arrival
 * counters, split partials and the candidate lists that travel from adamas_step_candidates to
 * adamas_step_attend, which therefore must be called with the same sizes.
 */
size_t adamas_workspace_bytes(uint32_t batch, uint32_t num_heads, uint32_t max_seq_len,
                              uint32_t budget);

/*
 * Paged decode attention over selected tokens, fp32 online softmax, fp16 output:
 *   o[b][h] = softmax_{t in S(b,h)} (q[b][h] . K[t][h] * sm_scale) . V[t][h]
 *   sel_idx != NULL : S(b,h) = { sel_idx[(b*num_heads+h)*sel_stride + i], i < n_sel, entry >= 0 }
 *                     united with the current token seq_lens[b]-1 (logical token positions).
 *   sel_idx == NULL : S(b,h) = all tokens 0 .. seq_lens[b]-1 (dense decode attention).
 * q, out [batch][num_heads][128] fp16.
 * Replaces: BatchDecodeWithPagedKVCachePyTorchWrapper::Forward, adamas/ops/csrc/bsk_ops.h:95-124
 * (kernel BatchDecodeWithPagedKVCacheKernel, kernels/include/decode/decode_attn.cuh:482-702, and the
 * BeginForward/EndForward planning of kernels/include/decode/decode_handler.cuh:73-136, which has no
 * counterpart here: there is nothing to plan or free).
 */
int adamas_sparse_decode(const void* q, const void* kv_data, const int32_t* page_indices,
                         const int32_t* page_indptr, const int32_t* seq_lens,
                         const int32_t* sel_idx, int64_t sel_stride, uint32_t n_sel, void* out,
                         void* workspace, size_t workspace_bytes, uint32_t batch,
                         uint32_t num_heads, uint32_t num_kv_heads, uint32_t head_dim,
                         uint32_t page_size, float sm_scale, uint32_t max_seq_len,
                         adamas_stream_t stream);
int adamas_sparse_decode_f(const void* q, const void* kv_data, const int32_t* page_indices,
                           const int32_t* page_indptr, const int32_t* seq_lens,
                           const int32_t* sel_idx, int64_t sel_stride, uint32_t n_sel, void* out,
                           void* workspace, size_t workspace_bytes, uint32_t batch,
                           uint32_t num_heads, uint32_t num_kv_heads, uint32_t head_dim,
                           uint32_t page_size, float sm_scale, uint32_t max_seq_len,
                           uint32_t flags, adamas_stream_t stream);

/*
 * One whole decode step of the sparse path for every sequence of the batch:
 * estimate -> select (budget-1 nearest past tokens, ties to the lowest index) -> attention over the
 * selection plus the current token.  Sequences with seq_lens[b] <= budget attend to everything.
 * q_code comes from adamas_append_decode.  sel_out (optional) [batch*num_heads][budget-1] int32
 * receives the selected logical positions (a set: the order within a row is deterministic but not
 * specified; unused entries are -1).
 * page_table_stride: 0 = sequence b's page list starts at page_indices[page_indptr[b]]; otherwise it
 * starts at page_indices[b * page_table_stride] (fixed-stride tables), every entry of a row must be
 * a valid page id, and the kernels fetch page ids and sequence length side by side instead of one
 * after the other (one memory round trip less per launch).  page_indptr is still required here
 * (the paths for larger budgets use it); the two functions below accept NULL with a non-zero stride.
 * Replaces the call sequence decode_estimate / decode_topk / decode_sparse_attn of
 * adamas/models/Adamas.py:176-201 (adamas/utils/__init__.py:203-308).
 */
int adamas_decode_step(const void* q, const void* q_code, const void* kv_data,
                       const void* code_data, const int32_t* page_indices,
                       const int32_t* page_indptr, const int32_t* seq_lens, uint32_t budget,
                       void* out, int32_t* sel_out, void* workspace, size_t workspace_bytes,
                       uint32_t batch, uint32_t num_heads, uint32_t num_kv_heads, uint32_t head_dim,
                       uint32_t page_size, float sm_scale, uint32_t max_seq_len,
                       uint32_t page_table_stride, adamas_stream_t stream);
int adamas_decode_step_f(const void* q, const void* q_code, const void* kv_data,
                         const void* code_data, const int32_t* page_indices,
                         const int32_t* page_indptr, const int32_t* seq_lens, uint32_t budget,
                         void* out, int32_t* sel_out, void* workspace, size_t workspace_bytes,
                         uint32_t batch, uint32_t num_heads, uint32_t num_kv_heads,
                         uint32_t head_dim, uint32_t page_size, float sm_scale,
                         uint32_t max_seq_len, uint32_t page_table_stride, uint32_t flags,
                         adamas_stream_t stream);

/*
 * adamas_decode_step_f without the workspace arguments, for callers that cannot allocate device
 * memory (code under HIP graph capture, serving loops and harnesses that forbid it): the library
 * works in a static device array of ADAMAS_STATIC_SCRATCH_BYTES per GPU instead and calls no
 * allocating routine.  Sizes whose workspace (adamas_workspace_bytes) exceeds that give
 * ADAMAS_E_SCRATCH: at 32 heads the limit admits one sequence of up to 131072 tokens at budgets up
 * to 4096, or two sequences of 32768 tokens at budget 128; larger batches need the caller-workspace
 * entry point.  All calls on one GPU share the array: calls that overlap on one GPU (different streams
 * or threads) race; calls on one stream are ordered and fine.  The first call on a device looks up
 * the array's address (no allocation, but make it outside a stream capture).  Same results as
 * adamas_decode_step_f, bit for bit.  No counterpart in the reference, whose decode handler
 * allocates its buffers in every begin_forward (kernels/include/decode/decode_handler.cuh:105-117).
 */
int adamas_decode_step_noalloc(const void* q, const void* q_code, const void* kv_data,
                               const void* code_data, const int32_t* page_indices,
                               const int32_t* page_indptr, const int32_t* seq_lens, uint32_t budget,
                               void* out, int32_t* sel_out, uint32_t batch, uint32_t num_heads,
                               uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size,
                               float sm_scale, uint32_t max_seq_len, uint32_t page_table_stride,
                               uint32_t flags, adamas_stream_t stream);

/*
 * The two halves of adamas_decode_step, for callers that want to time or schedule them separately.
 * adamas_step_fused_supported returns 1 when these sizes are served by the two-launch path (budget
 * <= 256; one sequence of up to 131072 tokens, or several whose chunk lists fit: at most 64 chunks of
 * 512, 1024 or 2048 tokens each); otherwise adamas_decode_step takes another route (budgets above
 * 256 on rows of up to 131072 tokens: an estimator launch that leaves distances and per-chunk
 * histograms, and a launch that selects from the histograms and attends; anything else: the three
 * stand-alone operators one after the other) and the two functions below return
 * ADAMAS_E_UNSUPPORTED.
 *   adamas_step_candidates : distance estimate over the code cache fused with the selection of the
 *                            nearest tokens of every chunk (chunks of a single sequence are balanced:
 *                            their lengths differ by at most 16 tokens and their number does not
 *                            change with the length).  Every chunk leaves a list of its nearest
 *                            tokens per head, and the query codes, in the workspace.
 *   adamas_step_attend     : final selection among the listed tokens (same tie rule) and attention
 *                            over the selected tokens plus the current one.  A chunk whose list is
 *                            used up by the selection is scored again from code_data, so the
 *                            selection is exact for any input.
 * No counterpart in the reference: its three operators (adamas/utils/__init__.py:203-308) are one
 * launch each and exchange the full [heads, L-1] distance matrix through HBM.
 */
int adamas_step_fused_supported(uint32_t batch, uint32_t num_heads, uint32_t max_seq_len,
                                uint32_t budget);
/*
 * How the two-launch step cuts these sizes up (host arithmetic only, for tools and tests; no
 * counterpart in the reference).  plan_out receives 8 values: supported (0/1), heads per workgroup of
 * the first launch (8 or 4), chunks per sequence, 16-token units per chunk (quotient), chunks that
 * have one unit more (remainder), passes of 512 tokens per workgroup, whether the last pass can be
 * partial (0/1), candidate slots per head and chunk.
 */
int adamas_step_plan(uint32_t batch, uint32_t num_heads, uint32_t max_seq_len, uint32_t budget,
                     uint32_t* plan_out);
int adamas_step_candidates(const void* q_code, const void* code_data, const int32_t* page_indices,
                           const int32_t* page_indptr, const int32_t* seq_lens, uint32_t budget,
                           void* workspace, size_t workspace_bytes, uint32_t batch,
                           uint32_t num_heads, uint32_t num_kv_heads, uint32_t page_size,
                           uint32_t max_seq_len, uint32_t page_table_stride, adamas_stream_t stream);
int adamas_step_attend(const void* q, const void* kv_data, const void* code_data,
                       const int32_t* page_indices, const int32_t* page_indptr,
                       const int32_t* seq_lens, uint32_t budget, void* out, int32_t* sel_out,
                       void* workspace, size_t workspace_bytes, uint32_t batch, uint32_t num_heads,
                       uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size, float sm_scale,
                       uint32_t max_seq_len, uint32_t page_table_stride, adamas_stream_t stream);
int adamas_step_candidates_f(const void* q_code, const void* code_data,
                             const int32_t* page_indices, const int32_t* page_indptr,
                             const int32_t* seq_lens, uint32_t budget, void* workspace,
                             size_t workspace_bytes, uint32_t batch, uint32_t num_heads,
                             uint32_t num_kv_heads, uint32_t page_size, uint32_t max_seq_len,
                             uint32_t page_table_stride, uint32_t flags, adamas_stream_t stream);
int adamas_step_attend_f(const void* q, const void* kv_data, const void* code_data,
                         const int32_t* page_indices, const int32_t* page_indptr,
                         const int32_t* seq_lens, uint32_t budget, void* out, int32_t* sel_out,
                         void* workspace, size_t workspace_bytes, uint32_t batch,
                         uint32_t num_heads, uint32_t num_kv_heads, uint32_t head_dim,
                         uint32_t page_size, float sm_scale, uint32_t max_seq_len,
                         uint32_t page_table_stride, uint32_t flags, adamas_stream_t stream);

/*
 * Per-token operators of the decoder around the attention path, one launch each (fp16 in/out, fp32
 * arithmetic).  They exist so that a decode step recorded in a HIP graph is not dominated by chains
 * of elementwise launches.
 *   adamas_rmsnorm    : out[r] = fp16(s[r] * rsqrt(mean(s[r]^2) + eps)) * weight, rows of `hidden`
 *                       (multiple of 8), with s = x, or, when delta is given, s = fp16(x + delta),
 *                       also written to sum_out (the residual add of a decoder layer fused in;
 *                       sum_out may be x).  Replaces rms_norm_forward,
 *                       adamas/ops/csrc/bsk_ops.h:33-36 (adamas/utils/__init__.py:79-92).
 *   adamas_rope_split : qkv [rows][num_heads + 2*num_kv_heads][128] (query heads, key heads, value
 *                       heads of a fused projection) -> q [rows][num_heads][128] and k
 *                       [rows][num_kv_heads][128] with rotary embedding (rotate-half pairing
 *                       (i, i+64), cos/sin tables [positions][64] fp32) and v [rows][num_kv_heads][128].  Position of row r: seq_lens[r]-1 when seq_lens is
 *                       given (decode, read on the device), else start_pos + r (prefill).  Takes the
 *                       place of apply_rope_in_place, adamas/ops/csrc/bsk_ops.h:23-27
 *                       (adamas/utils/__init__.py:26-53), which takes the position from the host.
 *   adamas_silu_mul   : out[r][i] = fp16(silu(gate_up[r][i])) * gate_up[r][inter + i].  No
 *                       counterpart in the reference (it uses torch for the MLP activation).
 */
int adamas_rmsnorm(const void* x, const void* delta, const void* weight, void* sum_out, void* out,
                   uint32_t rows, uint32_t hidden, float eps, adamas_stream_t stream);
int adamas_rope_split(const void* qkv, const float* cos_table, const float* sin_table,
                      const int32_t* seq_lens, uint32_t start_pos, void* q, void* k, void* v,
                      uint32_t rows, uint32_t num_heads, uint32_t num_kv_heads, uint32_t head_dim,
                      adamas_stream_t stream);
int adamas_silu_mul(const void* gate_up, void* out, uint32_t rows, uint32_t inter,
                    adamas_stream_t stream);
/*
 * Rotary embedding of q [rows][num_heads][128] and k [rows][num_kv_heads][128] where they lie
 * (fp16, or bf16 with ADAMAS_F_BF16), row r at position past_kv_len + r, pairing (i, i+64), angle
 * = float(position) * fp32(rope_theta^(-2i/128) / rope_scale).  Replaces apply_rope_in_place,
 * adamas/ops/csrc/bsk_ops.h:23-27 (binding adamas/ops/csrc/page.cu:228-269, wrapper
 * adamas/utils/__init__.py:26-53); same argument meaning.  Positions must stay below 2^24.
 */
int adamas_rope_in_place(void* q, void* k, uint32_t rows, uint32_t num_heads, uint32_t num_kv_heads,
                         uint32_t head_dim, uint32_t past_kv_len, float rope_scale, float rope_theta,
                         uint32_t flags, adamas_stream_t stream);
/*
 * Decode append straight from the fused q/k/v projection qkv [batch][num_heads + 2*num_kv_heads][128]
 * (query heads, then key heads, then value heads): rotary
 * embedding at position seq_lens[b]-1 (tables as for adamas_rope_split), rotated q to q_out
 * [batch][num_heads][128], rotated k and v into the KV page, the codes of Hadamard(q) to q_code_out
 * and of Hadamard(k) into the code page.  Same results as adamas_rope_split followed by
 * adamas_append_decode (adamas/models/Adamas.py:113 and :145-155 in the reference), one launch.
 * flags: ADAMAS_F_BF16 (qkv, q_out and the KV pages hold bfloat16), ADAMAS_F_HND (page layout),
 * ADAMAS_F_CODE_FROM_FP32.
 */
int adamas_rope_append_decode(const void* qkv, const float* cos_table, const float* sin_table,
                              void* q_out, void* q_code_out, void* kv_data, void* code_data,
                              const int32_t* page_indices, const int32_t* page_indptr,
                              const int32_t* seq_lens, uint32_t batch, uint32_t num_heads,
                              uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size,
                              float scale, uint32_t flags, adamas_stream_t stream);
/*
 * One decode step of a sparse layer straight from the fused q/k/v projection of the decoder, in the
 * two launches of adamas_decode_step: what adamas_rope_append_decode followed by adamas_decode_step
 * compute, without the launch of the append.  qkv [batch][num_heads + 2*num_kv_heads][128] fp16 (query
 * heads, key heads, value heads), cos/sin tables [positions][64] fp32 (rotate-half pairing), position
 * of sequence b = seq_lens[b] - 1 (its page must exist).  Launch 1 makes the query codes itself
 * (rotary embedding, Hadamard transform, buckets) while it streams the code cache; launch 2 applies
 * the rotary embedding to the query and the new key, writes the new key, its code and the new value
 * into the caches and attends the selected tokens plus the new one (from registers).  Results are
 * those of the two-call sequence: identical codes, cache contents and selections, outputs equal up
 * to the order of the softmax accumulation.
 * flags: ADAMAS_F_BF16 (qkv, the KV pages and out hold bfloat16), ADAMAS_F_HND (page layout),
 * ADAMAS_F_CODE_FROM_FP32.  Returns ADAMAS_E_UNSUPPORTED where adamas_step_fused_supported() is 0
 * (the caller then uses the two-call sequence).
 * No counterpart in the reference (its decode step is apply_rope_in_place, append_kv_cache_decode,
 * estimate, top-k and attention as separate launches, adamas/models/Adamas.py:129-201).
 */
int adamas_decode_layer_step(const void* qkv, const float* cos_table, const float* sin_table,
                             void* kv_data, void* code_data, const int32_t* page_indices,
                             const int32_t* page_indptr, const int32_t* seq_lens, uint32_t budget,
                             void* out, int32_t* sel_out, void* workspace, size_t workspace_bytes,
                             uint32_t batch, uint32_t num_heads, uint32_t num_kv_heads,
                             uint32_t head_dim, uint32_t page_size, float sm_scale,
                             uint32_t max_seq_len, uint32_t page_table_stride,
                             float hadamard_scale, uint32_t flags, adamas_stream_t stream);

/*
 * y[n] = sum_k w[n][k] * x[k] for one row of activations: w [n_rows][k] fp16 row-major, x [k], y
 * [n_rows] fp16, fp32 accumulation; k a multiple of 8, at most 16384.  The projections of a one-token
 * decode step (torch.nn.Linear in the reference's model, adamas/models/llama.py) as a kernel that
 * only streams the weights.
 */
int adamas_gemv(const void* w, const void* x, void* y, uint32_t n_rows, uint32_t k,
                adamas_stream_t stream);
/* The same for the gated MLP: w_gate_up [2*inter][k] (gate rows, then up rows);
 * y[n] = fp16(silu(fp16(gate_n . x))) * fp16(up_n . x), n < inter: adamas_gemv followed by
 * adamas_silu_mul in one launch, same bits. */
int adamas_gemv_silu_gate(const void* w_gate_up, const void* x, void* y, uint32_t inter, uint32_t k,
                          adamas_stream_t stream);

/*
 * The residual add and the RMSNorm of a decoder layer folded into the projections around them (one
 * new token; no launch for the add or the norm):
 *   adamas_gemv_add     : resid[n] = fp16(resid[n] + fp16(w[n] . x)) in place, n < n_rows (a multiple
 *                         of 4), and partials[n / 4] = the sum of the squares of the four new values
 *                         resid[4i .. 4i+3] (fp32, fixed order): the output projection or the down
 *                         projection writing straight into the residual stream.
 *   adamas_gemv_normed  : y[n] = fp16(rs * (w[n] . x)), rs = rsqrt(sum(partials) / k + eps): the
 *                         projection of RMSNorm(x) for the residual stream x whose partial sums the
 *                         call above left behind.  A norm weight g is folded into w beforehand
 *                         (w[n][c] * g[c]).
 *   adamas_gemv_silu_gate_normed : the same for adamas_gemv_silu_gate.
 *   adamas_sumsq_partials : partials[i] = x[4i]^2 + .. + x[4i+3]^2 for a row no adamas_gemv_add
 *                         produced (the embedding of the new token).
 * Replace, together, the calls of rms_norm_forward (adamas/ops/csrc/bsk_ops.h:33-36) and the
 * residual adds of the reference's decoder layer (adamas/models/llama.py) at decode time.
 */
int adamas_gemv_add(const void* w, const void* x, void* resid, float* partials, uint32_t n_rows,
                    uint32_t k, adamas_stream_t stream);
int adamas_gemv_normed(const void* w, const void* x, const float* partials, uint32_t n_partials,
                       float eps, void* y, uint32_t n_rows, uint32_t k, adamas_stream_t stream);
int adamas_gemv_silu_gate_normed(const void* w_gate_up, const void* x, const float* partials,
                                 uint32_t n_partials, float eps, void* y, uint32_t inter, uint32_t k,
                                 adamas_stream_t stream);
int adamas_sumsq_partials(const void* x, float* partials, uint32_t hidden, adamas_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* ADAMAS_HIP_H_ */
