"""Operator API of the decode-time sparse-attention path on MI355X.

Same function names, argument order and return values as adamas/utils/__init__.py of the reference
(append_kvh :94-157, decode_estimate :203-237, decode_topk :239-269, decode_sparse_attn :271-308,
pack_2bit :55-76), apply_rope_in_place :26-53, prefill_forward :159-201, rms_norm_forward :79-92), so the reference's
attention module (adamas/models/Adamas.py:68-225) can drive it unchanged.  Every function allocates its output with torch, checks shapes and dtypes in Python
(RuntimeError on violation, like TORCH_CHECK in the reference bindings) and calls one entry point of
libadamas_hip.so on the current stream.  There is no fallback path: without the library the calls raise.

Additions that have no counterpart in the reference:
  hadamard_transform   the transform itself (the reference imports a third-party CUDA module);
  append_kvh(..., h=None, q=q)  fused Hadamard + code generation inside the append kernel;
  decode_step          estimate + top-k + attention behind one call.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .. import _lib
from .controller import ALL_PAST_TOKENS, ORTHONORMAL_SCALE, RAW_SCALE, InferenceController
from .paging import CODE_WORDS, KvCache, PagePool, PagedSequences, TensorLayout

__all__ = [
    "TensorLayout",
    "KvCache",
    "PagePool",
    "PagedSequences",
    "InferenceController",
    "BatchDecodeWithPagedKVCacheWrapper",
    "ALL_PAST_TOKENS",
    "ORTHONORMAL_SCALE",
    "RAW_SCALE",
    "hadamard_transform",
    "pack_2bit",
    "append_kvh",
    "decode_estimate",
    "decode_topk",
    "decode_sparse_attn",
    "decode_step",
    "apply_rope_in_place",
    "prefill_forward",
    "rms_norm_forward",
    "add_rms_norm",
    "rope_split",
    "silu_mul",
    "gemv",
    "rope_append_decode",
    "gemv_silu_gate",
    "decode_layer_step",
    "layer_step_supported",
    "gemv_add",
    "gemv_normed",
    "sumsq_partials",
]


_FLOAT_DTYPES = (torch.float16, torch.bfloat16)


def _check_cuda_contig(t: torch.Tensor, name: str, dtype=None, ndim=None):
    if not isinstance(t, torch.Tensor):
        raise RuntimeError(f"{name} must be a tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA (HIP) tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if dtype is not None and (t.dtype not in dtype if isinstance(dtype, tuple) else t.dtype != dtype):
        raise RuntimeError(f"{name} must have dtype {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise RuntimeError(f"{name} must have {ndim} dimensions, got {t.dim()}")


def hadamard_transform(x: torch.Tensor, inplace: bool = False,
                       scale: float = ORTHONORMAL_SCALE) -> torch.Tensor:
    """y = x . H_128 * scale over the last axis, fp32 butterfly, result in the dtype of x (fp16 or bf16).

    Stand-in for `faster_hadamard_transform.hadamard_transform(x, inplace)` as the reference calls it
    (adamas/models/Adamas.py:120, :150), which passes no scale: the default is the orthonormal
    transform (128**-0.5) that module's published source computes; `scale` 1.0 is the raw +-1
    butterfly.
    """
    _check_cuda_contig(x, "x", _FLOAT_DTYPES)
    if x.shape[-1] != 128:
        raise RuntimeError("hadamard_transform supports a last dimension of 128 only")
    out = x if inplace else torch.empty_like(x)
    n_rows = x.numel() // 128
    rc = _lib.load().adamas_hadamard_f(x.data_ptr(), out.data_ptr(), n_rows, scale,
                                       _lib.dtype_flags(x.dtype), _lib.current_stream())
    _lib.check(rc, "adamas_hadamard")
    return out


def pack_2bit(h: torch.Tensor, past_kv_len: int = 0, dtype: torch.dtype = torch.int16) -> torch.Tensor:
    """Pack integer-valued codes (0..3, stored as fp16 or bf16) into 2-bit words, LSB first.
    h [N, H, D] -> [N, H, D/8] (reference utils/__init__.py:55-76; `past_kv_len` is unused there too).
    `dtype` only re-labels the 16-bit words (int16 by default, float16 to mimic the reference)."""
    _check_cuda_contig(h, "h", _FLOAT_DTYPES, 3)
    n, nh, d = h.shape
    if d != 128:
        raise RuntimeError("pack_2bit supports head_dim 128 only")
    o = torch.empty((n, nh, d // 8), dtype=torch.int16, device=h.device)
    rc = _lib.load().adamas_pack_2bit_f(h.data_ptr(), o.data_ptr(), n * nh,
                                        _lib.dtype_flags(h.dtype), _lib.current_stream())
    _lib.check(rc, "adamas_pack_2bit")
    return o.view(dtype)


def append_kvh(k: torch.Tensor, v: torch.Tensor, h: Optional[torch.Tensor],
               iController: InferenceController, layer_idx: int, *,
               q: Optional[torch.Tensor] = None, seq_idx: int = 0):
    """Append new k/v rows to the paged KV cache and their 2-bit codes to the code cache.

    Prefill (k.shape[0] > 1 and the controller holds a single sequence, or `seq_idx` given):
        k, v [N, H, D]; h [N, H, D] = Hadamard(k), or None to transform inside the kernel.
        The tokens take the last N positions of sequence `seq_idx` (prepare_hadamard(N) comes first).
        Returns None.
    Decode (one new token per sequence):
        k, v [B, H, D] with B = batch size of the controller (1 in the reference);
        h [2B, H, D] = Hadamard(cat(q, k)), or None with `q=` [B, H, D] for the fused kernel.
        Returns the packed 2-bit code of the query, [B, H, D/8] int16.
    With grouped-query attention (controller built with num_kv_heads < num_heads) k, v and the
    prefill h hold num_kv_heads heads, q holds num_heads, and a decode h is the 2-D stack
    [B*num_heads + B*num_kv_heads, D] of Hadamard(q) rows followed by Hadamard(k) rows.
    Reference: adamas/utils/__init__.py:94-157.
    """
    lib = _lib.load()
    c = iController
    _check_cuda_contig(k, "k", c.dtype, 3)
    _check_cuda_contig(v, "v", c.dtype, 3)
    if k.shape != v.shape:
        raise RuntimeError("k and v must have the same shape")
    n, nh, d = k.shape
    if nh != c.num_kv_heads or d != c.head_dim:
        raise RuntimeError("k does not match the controller's num_kv_heads/head_dim")
    nq = c.num_heads   # query heads (= nh unless grouped-query attention)
    kv = c.pool.kv[layer_idx]
    codes = c.pool.codes[layer_idx]
    stream = _lib.current_stream()
    # decode: h stacks Hadamard(q) on Hadamard(k) (twice the rows of k), or q is given for the fused kernel
    is_decode = q is not None or (h is not None and (
        h.shape[0] == 2 * n if nq == nh else h.dim() == 2 and h.shape[0] == n * (nq + nh)))
    if is_decode and n != c.batch_size:
        raise RuntimeError("decode append expects one new token per sequence of the controller")
    if not is_decode:
        if h is not None:
            _check_cuda_contig(h, "h", c.dtype, 3)
            if h.shape != k.shape:
                raise RuntimeError("prefill h must have the shape of k")
        total = c.seqs.lengths[seq_idx]
        if n > total:
            raise RuntimeError("prepare_hadamard must reserve the tokens before append_kvh")
        rc = lib.adamas_append_prefill(k.data_ptr(), v.data_ptr(), _lib.ptr(h), n, total - n,
                                       kv.data_ptr(), codes.data_ptr(), c.seqs.table_ptr(seq_idx),
                                       c.seqs.max_pages, nh, d, c.page_size, c.hadamard_scale,
                                       c.code_flags, stream)
        _lib.check(rc, "adamas_append_prefill")
        return None
    if h is not None:
        _check_cuda_contig(h, "h", c.dtype, 3 if nq == nh else 2)
        if nq == nh:
            if h.shape != (2 * n, nh, d):
                raise RuntimeError("decode h must be [2*B, H, D] = Hadamard(cat(q, k))")
        elif h.shape != (n * (nq + nh), d):
            raise RuntimeError("decode h must be [B*(Hq + Hkv), D]: Hadamard(q) rows, then Hadamard(k) rows")
    else:
        _check_cuda_contig(q, "q", c.dtype, 3)
        if q.shape != (n, nq, d):
            raise RuntimeError("q must be [B, num_heads, D]")
    if c.min_len_now < 1:
        raise RuntimeError("prepare_hadamard must reserve the token before append_kvh")
    o = torch.empty((n, nq, d // 8), dtype=torch.int16, device=k.device)
    rc = lib.adamas_append_decode(_lib.ptr(q), k.data_ptr(), v.data_ptr(), _lib.ptr(h), o.data_ptr(),
                                  kv.data_ptr(), codes.data_ptr(), c.seqs.table_dev.data_ptr(),
                                  c.seqs.indptr_dev.data_ptr(), c.seqs.seq_lens_dev.data_ptr(), n,
                                  nq, nh, d, c.page_size, c.hadamard_scale, c.code_flags, stream)
    _lib.check(rc, "adamas_append_decode")
    return o


def decode_estimate(q: torch.Tensor, iController: InferenceController, layer_idx: int) -> torch.Tensor:
    """Integer L1 distance between the query code and the code of every past token.

    q: the packed query code returned by append_kvh, [B, H, D/8].  Returns [H, L-1] float16 for a
    single sequence (the reference's shape, utils/__init__.py:226) or [B, H, Lmax-1] for a batch;
    entries are exact integers in [0, 384].  The current token is excluded.
    Reference: adamas/utils/__init__.py:203-237.
    """
    c = iController
    _check_cuda_contig(q, "q", None, 3)
    if q.element_size() != 2 or q.shape != (c.batch_size, c.num_heads, CODE_WORDS):
        raise RuntimeError("q must be the packed query code [B, H, 16] of 16-bit words")
    lmax = c.max_len_now
    if lmax < 2:
        raise RuntimeError("decode_estimate needs at least one past token")
    stride = (lmax - 1 + 7) // 8 * 8
    buf = torch.empty((c.batch_size, c.num_heads, stride), dtype=torch.float16, device=q.device)
    rc = _lib.load().adamas_estimate(q.data_ptr(), c.pool.codes[layer_idx].data_ptr(),
                                     c.seqs.table_dev.data_ptr(), c.seqs.indptr_dev.data_ptr(),
                                     c.seqs.seq_lens_dev.data_ptr(), buf.data_ptr(),
                                     c.num_heads * stride, stride, _lib.DIST_FP16, c.batch_size,
                                     c.num_heads, c.num_kv_heads, c.page_size, lmax,
                                     _lib.current_stream())
    _lib.check(rc, "adamas_estimate")
    out = buf[:, :, :lmax - 1]
    if c.batch_size == 1:
        out = out[0]
    # The controller keeps the buffer it handed out (until the next estimate): decode_topk takes the
    # single-pass integer selection for any view of it (slices, reshapes).  Holding the tensor keeps
    # its address from being handed to another tensor by the allocator, and its version counter
    # tells an in-place edit by the caller (est.mul_(...)) from the values the kernel wrote.
    c._estimate_buf = buf
    c._estimate_version = buf._version
    return out


def decode_topk(estimated_attn_score: torch.Tensor, iController: InferenceController,
                integer_keys: Optional[bool] = None):
    """Select the budget-1 past tokens with the SMALLEST estimate per head, ties to the lowest index.
    Fills iController.topk_dindices_buffer (logical token positions, int32) and topk_dout_buffer
    (their estimates).  Reference: adamas/utils/__init__.py:239-269.

    integer_keys: True promises that every estimate is an integer in [0, 511] (what decode_estimate
    produces) and selects with one histogram pass; False takes the selection for arbitrary fp16
    keys.  None (the reference's two-argument call) decides by whether the tensor is a view of the
    buffer the controller's last decode_estimate filled and that buffer has not been edited in
    place since (the controller holds the buffer, so its memory cannot be reused by another tensor
    meanwhile); a copy of it, or any other tensor, is treated as arbitrary keys.
    """
    c = iController
    est = estimated_attn_score
    if est.dtype != torch.float16 or not est.is_cuda or est.stride(-1) != 1:
        raise RuntimeError("estimated_attn_score must be a float16 CUDA tensor with unit inner stride")
    rows = c.batch_size * c.num_heads
    if est.dim() == 3:  # [B, H, n] view of a padded buffer: fold (B, H) into rows
        if est.shape[0] * est.shape[1] != rows or est.stride(0) != est.stride(1) * est.shape[1]:
            raise RuntimeError("batched estimate must be [B, H, n] with a uniform row stride")
        est2 = est.as_strided((rows, est.shape[-1]), (est.stride(1), 1))
    else:
        est2 = est
    if est2.shape[0] != rows:
        raise RuntimeError("estimated_attn_score must have one row per (sequence, head)")
    if c.topk_dindices_buffer is None:
        raise RuntimeError("begin_forward must be called before decode_topk")
    k = c.inference_page_budget - 1
    n = est2.shape[1]
    if n < k and c.batch_size == 1:
        # reference check CHECK_GE(num_pages, page_budget) in adamas/ops/csrc/topk.cu:26
        raise RuntimeError("fewer candidates than the budget")
    if integer_keys is None:
        buf = getattr(c, "_estimate_buf", None)
        integer_keys = False
        if buf is not None and buf._version == c._estimate_version:
            base, nbytes = buf.untyped_storage().data_ptr(), buf.untyped_storage().nbytes()
            integer_keys = base <= est.data_ptr() < base + nbytes
    mode = _lib.KEY_FP16_INT if integer_keys else _lib.KEY_FP16_GENERIC
    ragged = c.batch_size > 1
    buf = c.topk_workspace(n, k)
    rc = _lib.load().adamas_topk(est2.data_ptr(), est2.stride(0), n,
                                 c.seqs.seq_lens_dev.data_ptr() if ragged else None,
                                 c.num_heads, -1, None, 0, rows, k,
                                 c.topk_dindices_buffer.data_ptr(), c.topk_dout_buffer.data_ptr(), k,
                                 mode, buf.data_ptr(), buf.numel(), _lib.current_stream())
    _lib.check(rc, "adamas_topk")


def decode_sparse_attn(q: torch.Tensor, iController: InferenceController, layer_idx: int,
                       topk_indices, rope_scale: Optional[float] = None,
                       rope_theta: Optional[float] = None) -> torch.Tensor:
    """Attention over the selected tokens plus the current one.

    q [B, H, D]; topk_indices [B*H, budget-1] int32 logical token positions (negative = unused), or
    iController.kv_indices_without_last (= ALL_PAST_TOKENS) for dense attention over the whole cache,
    which is how the reference serves the non-estimated layers (Adamas.py:165-173).
    rope_scale / rope_theta are accepted and ignored, as in the reference (RotaryMode::kNone,
    adamas/ops/csrc/approx_attn.cu:135).  Reference: adamas/utils/__init__.py:271-308.
    """
    c = iController
    _check_cuda_contig(q, "q", c.dtype, 3)
    if q.shape != (c.batch_size, c.num_heads, c.head_dim):
        raise RuntimeError("q must be [B, H, D]")
    o = torch.empty_like(q)
    if topk_indices is ALL_PAST_TOKENS or topk_indices is None:
        sel_ptr, stride, n_sel = None, 0, 0
    else:
        _check_cuda_contig(topk_indices, "topk_indices", torch.int32, 2)
        if topk_indices.shape[0] != c.batch_size * c.num_heads:
            raise RuntimeError("topk_indices must have one row per (sequence, head)")
        sel_ptr, stride, n_sel = topk_indices.data_ptr(), topk_indices.stride(0), topk_indices.shape[1]
    ws = c.workspace(c.inference_page_budget or 1)
    rc = _lib.load().adamas_sparse_decode_f(
        q.data_ptr(), c.pool.kv[layer_idx].data_ptr(), c.seqs.table_dev.data_ptr(),
        c.seqs.indptr_dev.data_ptr(), c.seqs.seq_lens_dev.data_ptr(), sel_ptr, stride, n_sel,
        o.data_ptr(), ws.data_ptr(), ws.numel(), c.batch_size, c.num_heads, c.num_kv_heads,
        c.head_dim, c.page_size, 1.0 / math.sqrt(c.head_dim), c.max_len_now, c.kv_flags,
        _lib.current_stream())
    _lib.check(rc, "adamas_sparse_decode")
    return o


class BatchDecodeWithPagedKVCacheWrapper:
    """Counterpart of the reference's decode wrapper (adamas/utils/decode_wrapper.py:11-82; exported by
    adamas/utils/__init__.py:9,15): attention of one new token over a per-head list of physical
    pages plus the (partly filled) last page, with the reference's method names and argument lists.

    The reference plans split-KV work and allocates temporary buffers in begin_forward
    (decode_handler.cuh:73-136); the HIP kernel splits and merges on its own, so begin_forward only
    records the sizes and end_forward has nothing to free.  forward() maps the page list onto
    adamas_sparse_decode: the pool's pages in identity order form a virtual sequence whose one extra
    page is `paged_kv_last_page_idx`, every slot of a listed page becomes a token position of that
    sequence, and the newest token is the last valid slot of the extra page.  One sequence, as in
    the reference (batch_size 1, approx_attn.cu:78).  decode_sparse_attn is the path the model
    takes; this class serves callers that hold page lists of their own."""

    def __init__(self, kv_layout: str = "NHD"):
        if not hasattr(TensorLayout, kv_layout) or kv_layout not in ("NHD", "HND"):
            raise KeyError("Invalide kv_layout {}".format(kv_layout))  # (sic) the reference's message
        self.kv_layout = kv_layout
        self._plan = None
        self._table = None
        self._workspace = None

    def begin_forward(self, indptr: torch.Tensor, num_qo_heads: int, num_kv_heads: int,
                      head_dim: int, page_size: int, data_type):
        """indptr = [0, pages listed per head] (one sequence).  Reads indptr once, here."""
        if head_dim != 128:
            raise RuntimeError("BatchDecodeWithPagedKVCacheWrapper supports head_dim 128 only")
        if num_qo_heads % num_kv_heads != 0:
            raise RuntimeError("num_qo_heads must be a multiple of num_kv_heads")
        if data_type not in _FLOAT_DTYPES:
            raise RuntimeError("BatchDecodeWithPagedKVCacheWrapper failed to dispatch with dtype %s"
                               % data_type)
        if indptr.numel() != 2:
            raise RuntimeError("indptr must be [0, n_pages] of one sequence")
        n_listed = int(indptr.reshape(-1)[1].item()) - int(indptr.reshape(-1)[0].item())
        if n_listed < 0:
            raise RuntimeError("indptr must not decrease")
        self._plan = (n_listed, num_qo_heads, num_kv_heads, page_size, data_type)

    def end_forward(self):
        self._plan = None

    def forward(self, q: torch.Tensor, o: torch.Tensor, paged_kv_data: torch.Tensor,
                paged_kv_indices: torch.Tensor, paged_kv_indptr: torch.Tensor,
                paged_kv_last_page_len: int, paged_kv_last_page_idx: int,
                rope_scale: Optional[float] = None, rope_theta: Optional[float] = None):
        """q, o [1, Hq, 128]; paged_kv_data [pages, 2, P, Hkv, 128] (NHD) or [pages, 2, Hkv, P, 128];
        paged_kv_indices [Hq, row stride] int32 physical page ids, the first indptr[1] of every row
        are attended in full; the first paged_kv_last_page_len slots of page paged_kv_last_page_idx
        are attended too (its last valid slot is the newest token).  rope_* are accepted and unused
        (RotaryMode::kNone in the reference, approx_attn.cu:135).  Writes o."""
        if self._plan is None:
            # the reference's handler throws when forward comes before begin_forward
            # (decode_handler.cuh:226-231)
            raise RuntimeError("BatchDecodeWithPagedKVCacheWrapper: begin_forward must come first")
        n_listed, nq, nkv, page, dtype = self._plan
        # the reference's kernel reads the page count from the indptr given here; begin_forward has
        # fixed it, so a different one is an error rather than a silently stale page count (a device
        # tensor is not read back: that would stall the stream)
        if (isinstance(paged_kv_indptr, torch.Tensor) and not paged_kv_indptr.is_cuda
                and paged_kv_indptr.numel() == 2):
            now = int(paged_kv_indptr.reshape(-1)[1]) - int(paged_kv_indptr.reshape(-1)[0])
            if now != n_listed:
                raise RuntimeError("paged_kv_indptr lists %d pages, begin_forward was given %d"
                                   % (now, n_listed))
        _check_cuda_contig(q, "q", dtype, 3)
        _check_cuda_contig(o, "o", dtype, 3)
        _check_cuda_contig(paged_kv_data, "paged_kv_data", dtype, 5)
        _check_cuda_contig(paged_kv_indices, "paged_kv_indices", torch.int32, 2)
        hnd = self.kv_layout == "HND"
        want = (2, nkv, page, 128) if hnd else (2, page, nkv, 128)
        if tuple(paged_kv_data.shape[1:]) != want:
            raise RuntimeError("paged_kv_data must be [pages, %s]" % ", ".join(map(str, want)))
        if q.shape != (1, nq, 128) or o.shape != q.shape:
            raise RuntimeError("q and o must be [1, num_qo_heads, 128]")
        if paged_kv_indices.shape[0] != nq or paged_kv_indices.shape[1] < n_listed:
            raise RuntimeError("paged_kv_indices must be [num_qo_heads, >= indptr[1]]")
        n_pool = paged_kv_data.shape[0]
        last_len, last_idx = int(paged_kv_last_page_len), int(paged_kv_last_page_idx)
        if not (1 <= last_len <= page and 0 <= last_idx < n_pool):
            raise RuntimeError("last page: 1 <= len <= page_size and a valid page id expected")
        dev = q.device
        if self._table is None or self._table.numel() != n_pool + 1 or self._table.device != dev:
            self._table = torch.arange(n_pool + 1, dtype=torch.int32, device=dev)
            self._indptr = torch.tensor([0, n_pool + 1], dtype=torch.int32, device=dev)
            self._len = torch.zeros(1, dtype=torch.int32, device=dev)
        self._table[n_pool] = last_idx
        seq_len = n_pool * page + last_len
        self._len.fill_(seq_len)
        slots = torch.arange(page, dtype=torch.int32, device=dev)
        pos = (paged_kv_indices[:, :n_listed, None] * page + slots).reshape(nq, n_listed * page)
        tail = (n_pool * page + slots[:last_len - 1]).expand(nq, last_len - 1)
        sel = torch.cat((pos, tail), dim=1).contiguous()
        if sel.shape[1] == 0:   # only the newest token: one unused entry (a null list means "dense")
            sel = torch.full((nq, 1), -1, dtype=torch.int32, device=dev)
        n_sel = sel.shape[1]
        lib = _lib.load()
        need = lib.adamas_workspace_bytes(1, nq, 1, 1)
        if self._workspace is None or self._workspace.numel() < need or self._workspace.device != dev:
            self._workspace = torch.zeros(need, dtype=torch.uint8, device=dev)
        flags = _lib.dtype_flags(dtype) | (_lib.F_HND if hnd else 0)
        rc = lib.adamas_sparse_decode_f(
            q.data_ptr(), paged_kv_data.data_ptr(), self._table.data_ptr(), self._indptr.data_ptr(),
            self._len.data_ptr(), sel.data_ptr(), max(n_sel, 1), n_sel, o.data_ptr(),
            self._workspace.data_ptr(), self._workspace.numel(), 1, nq, nkv, 128, page,
            1.0 / math.sqrt(128), seq_len, flags, _lib.current_stream())
        _lib.check(rc, "adamas_sparse_decode")


def decode_step(q: torch.Tensor, q_code: torch.Tensor, iController: InferenceController,
                layer_idx: int, return_indices: bool = False):
    """estimate -> top-k -> sparse attention for one layer behind a single call (the sequence
    Adamas.py:176-201 of the reference).  Returns o [B, H, D] and, on request, the selected
    positions [B*H, budget-1]."""
    c = iController
    _check_cuda_contig(q, "q", c.dtype, 3)
    _check_cuda_contig(q_code, "q_code", None, 3)
    if c.inference_page_budget is None:
        raise RuntimeError("begin_forward must be called before decode_step")
    budget = c.inference_page_budget
    o = torch.empty_like(q)
    ws = c.workspace(budget)
    sel = c.topk_dindices_buffer if return_indices else None
    rc = _lib.load().adamas_decode_step_f(
        q.data_ptr(), q_code.data_ptr(), c.pool.kv[layer_idx].data_ptr(),
        c.pool.codes[layer_idx].data_ptr(), c.seqs.table_dev.data_ptr(),
        c.seqs.indptr_dev.data_ptr(), c.seqs.seq_lens_dev.data_ptr(), budget, o.data_ptr(),
        _lib.ptr(sel), ws.data_ptr(), ws.numel(), c.batch_size, c.num_heads, c.num_kv_heads,
        c.head_dim, c.page_size, 1.0 / math.sqrt(c.head_dim), c.max_len_now, c.seqs.max_pages,
        c.kv_flags, _lib.current_stream())
    _lib.check(rc, "adamas_decode_step")
    return (o, sel) if return_indices else o


# --- per-token operators of the decoder around the attention path -----------------------------------
def apply_rope_in_place(q: torch.Tensor, k: torch.Tensor, past_kv_len: int,
                        rope_scale: Optional[float] = None, rope_theta: Optional[float] = None) -> None:
    """Rotary embedding of q [N, Hq, 128] and k [N, Hkv, 128] where they lie, row r at position
    past_kv_len + r (adamas/utils/__init__.py:26-53; defaults rope_scale 1.0, rope_theta 1e4 as
    there).  The pairing is (i, i + 64), the convention of the Llama implementation the reference
    tests against (adamas/tests/test_rope.py:17-31).  The reference requires equal head counts
    (page.cu:241-243); here k may hold fewer (key/value) heads."""
    if rope_scale is None:
        rope_scale = 1.0
    if rope_theta is None:
        rope_theta = 1e4
    _check_cuda_contig(q, "q", ndim=3)
    _check_cuda_contig(k, "k", q.dtype, 3)
    if q.dtype not in _FLOAT_DTYPES:
        raise RuntimeError("apply_rope_in_place failed to dispatch with dtype %s" % q.dtype)
    if q.shape[0] != k.shape[0] or q.shape[2] != 128 or k.shape[2] != 128:
        raise RuntimeError("q and k must be [N, heads, 128] with the same N")
    if past_kv_len < 0:
        raise RuntimeError("past_kv_len must not be negative")
    rc = _lib.load().adamas_rope_in_place(q.data_ptr(), k.data_ptr(), q.shape[0], q.shape[1],
                                          k.shape[1], 128, int(past_kv_len), float(rope_scale),
                                          float(rope_theta), _lib.dtype_flags(q.dtype),
                                          _lib.current_stream())
    _lib.check(rc, "adamas_rope_in_place")


def prefill_forward(q: torch.Tensor, iController: InferenceController, layer_idx: int,
                    rope_scale: Optional[float] = None, rope_theta: Optional[float] = None) -> torch.Tensor:
    """Causal attention of the last N tokens of the sequence, q [N, Hq, 128], over the K/V already in
    the paged cache of `layer_idx` (adamas/utils/__init__.py:159-201); returns [N, Hq, 128].  The
    reference's prefill kernel is FlashInfer's tensor-core kernel, which is not part of the decode
    path this library implements: this operator collects the sequence's pages with torch indexing and
    calls torch.nn.functional.scaled_dot_product_attention (query blocks of 4096 rows when N is
    shorter than the sequence).  rope_scale and rope_theta are accepted and unused, as in the
    reference, whose q and cached k are already rotated.  Single sequence, like the reference."""
    c = iController
    _check_cuda_contig(q, "q", c.dtype, 3)
    if c.batch_size != 1:
        raise RuntimeError("prefill_forward serves one sequence")
    n, length = q.shape[0], c.kv_cache.seqlen
    if q.shape[1] != c.num_heads or q.shape[2] != c.head_dim:
        raise RuntimeError("q must be [N, num_heads, head_dim]")
    if n == 0 or n > length:
        raise RuntimeError("q holds %d tokens, the cache %d" % (n, length))
    p = c.page_size
    n_pages = (length + p - 1) // p
    pages = c.seqs.table_dev[:n_pages].long()
    kv = c.kv_cache.buf_layer(layer_idx).index_select(0, pages)  # [pages, 2, ...]
    if c.layout == TensorLayout.NHD:  # [pages, 2, P, H, D] -> [H, pages*P, D]
        kv = kv.permute(1, 3, 0, 2, 4)
    else:                             # [pages, 2, H, P, D]
        kv = kv.permute(1, 2, 0, 3, 4)
    kv = kv.reshape(2, c.num_kv_heads, n_pages * p, c.head_dim)[:, :, :length]
    keys, values = kv[0][None], kv[1][None]
    qh = q.transpose(0, 1)[None]  # [1, Hq, N, D]
    gqa = c.num_kv_heads != c.num_heads
    sdpa = torch.nn.functional.scaled_dot_product_attention
    if n == length:
        o = sdpa(qh, keys, values, is_causal=True, enable_gqa=gqa)
    else:
        o = torch.empty_like(qh)
        past = length - n
        cols = torch.arange(length, device=q.device)
        for r0 in range(0, n, 4096):
            r1 = min(n, r0 + 4096)
            # query row r sees tokens 0 .. past + r
            visible = past + r1
            mask = cols[None, :visible] <= (past + torch.arange(r0, r1, device=q.device))[:, None]
            o[:, :, r0:r1] = sdpa(qh[:, :, r0:r1], keys[:, :, :visible], values[:, :, :visible],
                                  attn_mask=mask, enable_gqa=gqa)
    return o[0].transpose(0, 1).contiguous()


def rms_norm_forward(input: torch.Tensor, weight: torch.Tensor, epsilon: float) -> torch.Tensor:
    """RMSNorm over the last axis: fp16(x * rsqrt(mean(x^2) + eps)) * weight, one launch.
    Same name, arguments and result as the reference's op (adamas/utils/__init__.py:79-92)."""
    _check_cuda_contig(input, "input", torch.float16)
    _check_cuda_contig(weight, "weight", torch.float16, 1)
    hidden = input.shape[-1]
    if weight.shape[0] != hidden:
        raise RuntimeError("weight must have the size of the last axis of input")
    o = torch.empty_like(input)
    rc = _lib.load().adamas_rmsnorm(input.data_ptr(), None, weight.data_ptr(), None, o.data_ptr(),
                                    input.numel() // hidden, hidden, float(epsilon),
                                    _lib.current_stream())
    _lib.check(rc, "adamas_rmsnorm")
    return o


def add_rms_norm(x: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, epsilon: float):
    """Residual add fused with RMSNorm: x += delta in place (fp16 add), returns RMSNorm(x) * weight.
    One launch instead of an add (or a GEMM epilogue with its copy) plus a norm."""
    _check_cuda_contig(x, "x", torch.float16)
    _check_cuda_contig(delta, "delta", torch.float16)
    _check_cuda_contig(weight, "weight", torch.float16, 1)
    hidden = x.shape[-1]
    if delta.shape != x.shape or weight.shape[0] != hidden:
        raise RuntimeError("delta must have the shape of x and weight the size of its last axis")
    o = torch.empty_like(x)
    rc = _lib.load().adamas_rmsnorm(x.data_ptr(), delta.data_ptr(), weight.data_ptr(), x.data_ptr(),
                                    o.data_ptr(), x.numel() // hidden, hidden, float(epsilon),
                                    _lib.current_stream())
    _lib.check(rc, "adamas_rmsnorm")
    return o


def _qkv_heads(qkv: torch.Tensor, num_kv_heads: Optional[int]):
    """(rows, query heads, key/value heads) of a fused projection output: [N, 3, H, 128] for equal
    head counts, or [N, Hq + 2*Hkv, 128] (query heads, key heads, value heads) with Hkv given."""
    if qkv.dim() == 4:
        n, three, nh, d = qkv.shape
        if three != 3 or d != 128 or (num_kv_heads not in (None, nh)):
            raise RuntimeError("a 4-D qkv must be [N, 3, H, 128] with equal head counts")
        return n, nh, nh
    if qkv.dim() != 3 or qkv.shape[2] != 128 or not num_kv_heads:
        raise RuntimeError("qkv must be [N, 3, H, 128], or [N, Hq + 2*Hkv, 128] with num_kv_heads")
    n, all_heads, _ = qkv.shape
    nq = all_heads - 2 * num_kv_heads
    if nq <= 0 or nq % num_kv_heads != 0:
        raise RuntimeError("qkv holds Hq + 2*Hkv heads with Hq a multiple of Hkv")
    return n, nq, num_kv_heads


def rope_split(qkv: torch.Tensor, cos_table: torch.Tensor, sin_table: torch.Tensor, *,
               seq_lens: Optional[torch.Tensor] = None, start_pos: int = 0,
               num_kv_heads: Optional[int] = None):
    """qkv (the output of a fused q/k/v projection: [N, 3, H, 128], or [N, Hq + 2*Hkv, 128] with
    `num_kv_heads` for grouped-query attention) -> q [N, Hq, 128] and k [N, Hkv, 128] with rotary
    embedding, v [N, Hkv, 128], in one launch.  Decode: pass the device-side `seq_lens` [N] int32, row r
    takes position seq_lens[r] - 1 (no host value involved, so the call can sit in a HIP graph).
    Prefill: row r takes position start_pos + r.  Takes the place of the reference's
    apply_rope_in_place (adamas/utils/__init__.py:26-53), whose position is a host integer."""
    _check_cuda_contig(qkv, "qkv", torch.float16)
    _check_cuda_contig(cos_table, "cos_table", torch.float32, 2)
    _check_cuda_contig(sin_table, "sin_table", torch.float32, 2)
    n, nq, nkv = _qkv_heads(qkv, num_kv_heads)
    if cos_table.shape[1] != 64 or sin_table.shape != cos_table.shape:
        raise RuntimeError("rotary tables must be [positions, 64]")
    if seq_lens is not None:
        _check_cuda_contig(seq_lens, "seq_lens", torch.int32, 1)
        if seq_lens.shape[0] != n:
            raise RuntimeError("one length per row expected")
    elif start_pos + n > cos_table.shape[0]:
        raise RuntimeError("positions run past the rotary tables")
    q = torch.empty((n, nq, 128), dtype=torch.float16, device=qkv.device)
    k = torch.empty((n, nkv, 128), dtype=torch.float16, device=qkv.device)
    v = torch.empty_like(k)
    rc = _lib.load().adamas_rope_split(qkv.data_ptr(), cos_table.data_ptr(), sin_table.data_ptr(),
                                       _lib.ptr(seq_lens), start_pos, q.data_ptr(), k.data_ptr(),
                                       v.data_ptr(), n, nq, nkv, 128, _lib.current_stream())
    _lib.check(rc, "adamas_rope_split")
    return q, k, v


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """gate_up [N, 2*I] fp16 -> fp16(silu(gate_up[:, :I])) * gate_up[:, I:], one launch."""
    _check_cuda_contig(gate_up, "gate_up", torch.float16, 2)
    n, two_i = gate_up.shape
    if two_i % 4 != 0:
        raise RuntimeError("the inner size must be a multiple of 4")
    o = torch.empty((n, two_i // 2), dtype=torch.float16, device=gate_up.device)
    rc = _lib.load().adamas_silu_mul(gate_up.data_ptr(), o.data_ptr(), n, two_i // 2,
                                     _lib.current_stream())
    _lib.check(rc, "adamas_silu_mul")
    return o


def gemv(w: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """w [N, K] fp16 (row-major weights of a linear layer) times one row of activations x [K] or
    [1, K] -> [1, N] fp16, fp32 accumulation: the projection of a one-token decode step as a kernel
    that only streams the weights."""
    _check_cuda_contig(w, "w", torch.float16, 2)
    _check_cuda_contig(x, "x", torch.float16)
    n, k = w.shape
    if x.numel() != k:
        raise RuntimeError("x must hold one row of w.shape[1] values")
    y = torch.empty((1, n), dtype=torch.float16, device=w.device)
    rc = _lib.load().adamas_gemv(w.data_ptr(), x.data_ptr(), y.data_ptr(), n, k, _lib.current_stream())
    _lib.check(rc, "adamas_gemv")
    return y


def rope_append_decode(qkv: torch.Tensor, cos_table: torch.Tensor, sin_table: torch.Tensor,
                       iController: InferenceController, layer_idx: int):
    """Decode append straight from the fused projection (qkv [B, 3, H, 128], or [B, Hq + 2*Hkv, 128]
    for a controller with grouped-query attention): rotary embedding at the position of the new token
    (device-side length - 1), KV append and code generation in one launch.  Returns (q [B, Hq, 128]
    rotated, q_code [B, Hq, 16]): the same tensors rope_split followed by
    append_kvh(k, v, None, ..., q=q) produce (Adamas.py:113 and :145-155 in the reference)."""
    c = iController
    _check_cuda_contig(qkv, "qkv", c.dtype)
    _check_cuda_contig(cos_table, "cos_table", torch.float32, 2)
    _check_cuda_contig(sin_table, "sin_table", torch.float32, 2)
    n, nq, nkv = _qkv_heads(qkv, c.num_kv_heads)
    if n != c.batch_size or nq != c.num_heads or nkv != c.num_kv_heads:
        raise RuntimeError("qkv must hold one new token per sequence and the controller's head counts")
    if cos_table.shape[1] != 64 or sin_table.shape != cos_table.shape or cos_table.shape[0] < c.max_len_now:
        raise RuntimeError("rotary tables must be [positions >= sequence length, 64]")
    if c.min_len_now < 1:
        raise RuntimeError("prepare_hadamard must reserve the token before the append")
    q = torch.empty((n, nq, 128), dtype=c.dtype, device=qkv.device)
    q_code = torch.empty((n, nq, 16), dtype=torch.int16, device=qkv.device)
    rc = _lib.load().adamas_rope_append_decode(
        qkv.data_ptr(), cos_table.data_ptr(), sin_table.data_ptr(), q.data_ptr(), q_code.data_ptr(),
        c.pool.kv[layer_idx].data_ptr(), c.pool.codes[layer_idx].data_ptr(),
        c.seqs.table_dev.data_ptr(), c.seqs.indptr_dev.data_ptr(), c.seqs.seq_lens_dev.data_ptr(), n,
        nq, nkv, 128, c.page_size, c.hadamard_scale, c.code_flags, _lib.current_stream())
    _lib.check(rc, "adamas_rope_append_decode")
    return q, q_code


def gemv_add(w: torch.Tensor, x: torch.Tensor, resid: torch.Tensor, partials: torch.Tensor) -> None:
    """resid [1, N] += w [N, K] . x (fp16 sum, in place) and partials [N/4] fp32 = sums of squares of
    the new values, four at a time: a projection that writes straight into the residual stream and
    prepares the RMSNorm that gemv_normed applies."""
    _check_cuda_contig(w, "w", torch.float16, 2)
    _check_cuda_contig(x, "x", torch.float16)
    _check_cuda_contig(resid, "resid", torch.float16)
    _check_cuda_contig(partials, "partials", torch.float32, 1)
    n, k = w.shape
    if x.numel() != k or resid.numel() != n or n % 4 != 0 or partials.numel() != n // 4:
        raise RuntimeError("gemv_add: x needs K values, resid N (a multiple of 4), partials N/4")
    rc = _lib.load().adamas_gemv_add(w.data_ptr(), x.data_ptr(), resid.data_ptr(), partials.data_ptr(),
                                     n, k, _lib.current_stream())
    _lib.check(rc, "adamas_gemv_add")


def gemv_normed(w: torch.Tensor, x: torch.Tensor, partials: torch.Tensor, epsilon: float,
                gated: bool = False) -> torch.Tensor:
    """w . RMSNorm(x) for one row x whose partial sums of squares are in `partials` (gemv_add or
    sumsq_partials); the norm weight is folded into w.  gated: w holds gate rows then up rows and
    the result is silu(gate) * up, as gemv_silu_gate."""
    _check_cuda_contig(w, "w", torch.float16, 2)
    _check_cuda_contig(x, "x", torch.float16)
    _check_cuda_contig(partials, "partials", torch.float32, 1)
    n, k = w.shape
    if x.numel() != k or (gated and n % 2 != 0):
        raise RuntimeError("gemv_normed handles one row of K values (and 2*I rows of weights when gated)")
    lib = _lib.load()
    if gated:
        y = torch.empty((1, n // 2), dtype=torch.float16, device=w.device)
        rc = lib.adamas_gemv_silu_gate_normed(w.data_ptr(), x.data_ptr(), partials.data_ptr(),
                                              partials.numel(), float(epsilon), y.data_ptr(), n // 2,
                                              k, _lib.current_stream())
    else:
        y = torch.empty((1, n), dtype=torch.float16, device=w.device)
        rc = lib.adamas_gemv_normed(w.data_ptr(), x.data_ptr(), partials.data_ptr(), partials.numel(),
                                    float(epsilon), y.data_ptr(), n, k, _lib.current_stream())
    _lib.check(rc, "adamas_gemv_normed")
    return y


def sumsq_partials(x: torch.Tensor, partials: torch.Tensor) -> None:
    """partials [K/4] fp32 = sums of squares of x [1, K], four values at a time."""
    _check_cuda_contig(x, "x", torch.float16)
    _check_cuda_contig(partials, "partials", torch.float32, 1)
    if x.numel() % 4 != 0 or partials.numel() != x.numel() // 4:
        raise RuntimeError("sumsq_partials: partials needs one value per four of x")
    rc = _lib.load().adamas_sumsq_partials(x.data_ptr(), partials.data_ptr(), x.numel(),
                                           _lib.current_stream())
    _lib.check(rc, "adamas_sumsq_partials")


def layer_step_supported(iController: InferenceController) -> bool:
    """Whether decode_layer_step serves the controller's current sizes (a budget and lengths the
    two-launch step covers); otherwise use rope_append_decode + decode_step."""
    c = iController
    if c.inference_page_budget is None:
        return False
    return bool(_lib.load().adamas_step_fused_supported(c.batch_size, c.num_heads, c.max_len_now,
                                                        c.inference_page_budget))


def decode_layer_step(qkv: torch.Tensor, cos_table: torch.Tensor, sin_table: torch.Tensor,
                      iController: InferenceController, layer_idx: int,
                      return_indices: bool = False):
    """rope_append_decode followed by decode_step in the two launches of the latter: the rotary
    embedding, the query code, the append of the new token and the step itself.  qkv
    [B, Hq + 2*Hkv, 128] (the fused projection of the new token of every sequence).  Returns
    o [B, Hq, 128] and, on request, the selected positions.  The controller must have reserved the
    token (prepare_hadamard / begin_forward, or a graph decode)."""
    c = iController
    _check_cuda_contig(qkv, "qkv", c.dtype)
    _check_cuda_contig(cos_table, "cos_table", torch.float32, 2)
    _check_cuda_contig(sin_table, "sin_table", torch.float32, 2)
    nq, nkv = c.num_heads, c.num_kv_heads
    n = qkv.numel() // ((nq + 2 * nkv) * 128)
    if n != c.batch_size or qkv.numel() != n * (nq + 2 * nkv) * 128:
        raise RuntimeError("qkv must hold one row of (num_heads + 2*num_kv_heads) * 128 values per sequence")
    if cos_table.shape[1] != 64 or sin_table.shape != cos_table.shape or cos_table.shape[0] < c.max_len_now:
        raise RuntimeError("rotary tables must be [positions >= sequence length, 64]")
    if c.inference_page_budget is None:
        raise RuntimeError("begin_forward must be called before decode_layer_step")
    if c.min_len_now < 1:
        raise RuntimeError("prepare_hadamard must reserve the token before the step")
    budget = c.inference_page_budget
    o = torch.empty((n, nq, 128), dtype=c.dtype, device=qkv.device)
    ws = c.workspace(budget)
    sel = c.topk_dindices_buffer if return_indices else None
    rc = _lib.load().adamas_decode_layer_step(
        qkv.data_ptr(), cos_table.data_ptr(), sin_table.data_ptr(), c.pool.kv[layer_idx].data_ptr(),
        c.pool.codes[layer_idx].data_ptr(), c.seqs.table_dev.data_ptr(), c.seqs.indptr_dev.data_ptr(),
        c.seqs.seq_lens_dev.data_ptr(), budget, o.data_ptr(), _lib.ptr(sel), ws.data_ptr(), ws.numel(),
        n, nq, nkv, 128, c.page_size, 1.0 / math.sqrt(c.head_dim), c.max_len_now, c.seqs.max_pages,
        c.hadamard_scale, c.code_flags, _lib.current_stream())
    _lib.check(rc, "adamas_decode_layer_step")
    return (o, sel) if return_indices else o


def gemv_silu_gate(w_gate_up: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """w_gate_up [2*I, K] (gate rows, then up rows), x one row of K values -> [1, I] =
    silu(gate . x) * (up . x) with the roundings of gemv followed by silu_mul, in one launch."""
    _check_cuda_contig(w_gate_up, "w_gate_up", torch.float16, 2)
    _check_cuda_contig(x, "x", torch.float16)
    two_i, k = w_gate_up.shape
    if two_i % 2 != 0 or x.numel() != k:
        raise RuntimeError("w_gate_up must be [2*I, K] and x one row of K values")
    y = torch.empty((1, two_i // 2), dtype=torch.float16, device=x.device)
    rc = _lib.load().adamas_gemv_silu_gate(w_gate_up.data_ptr(), x.data_ptr(), y.data_ptr(),
                                           two_i // 2, k, _lib.current_stream())
    _lib.check(rc, "adamas_gemv_silu_gate")
    return y
