"""Step controller of the decode path: page bookkeeping, budget regime, selection buffers.

Counterpart of adamas/utils/controller.py (InferenceController :7-148) with the same constructor
arguments, methods and public fields, re-designed so that a decode step moves no page table and
plans nothing:

* page tables, indptr and sequence lengths stay on the device (paging.PagedSequences);
* the budget counts TOKENS (the reference counts pages, which is the same thing at its only working
  page size, 1): `budget - 1` past tokens are selected, the current token is always attended;
* there is no decode handler to begin/end: the HIP attention kernel splits and merges on its own, so
  begin_forward/end_forward only fix the budget regime and (re)use the selection buffers;
* `kv_indices_without_last`, which the reference materialises as an [H, L-1] int32 tensor every step
  (controller.py:108), is the marker ALL_PAST_TOKENS: decode_sparse_attn turns it into the dense
  kernel mode instead of reading 4 MB of indices.
"""
from __future__ import annotations

from typing import Optional, Sequence, Union

import torch

from .paging import CODE_WORDS, KvCache, PagePool, PagedSequences, TensorLayout
from .. import _lib


class _AllPastTokens:
    """Marker for "attend to every cached token" (dense decode attention)."""

    def __repr__(self):
        return "ALL_PAST_TOKENS"


ALL_PAST_TOKENS = _AllPastTokens()

# Scale of the Hadamard transform behind the 2-bit codes.  The reference calls a third-party transform
# without a scale argument (adamas/models/Adamas.py:120,150) and bucketizes the result against the
# absolute thresholds -10 / 0 / 10 (kernels/include/decode/decode_page.cuh:385); that module's published
# source is orthonormal (x . H_128 / sqrt(128)), so that is what a caller who passes nothing gets here.
# 1.0 is the raw +-1 butterfly.
ORTHONORMAL_SCALE = 128 ** -0.5
RAW_SCALE = 1.0


class InferenceController:
    def __init__(self, num_layers, num_heads, head_dim, page_size,
                 page_budget,   # token budget, current token included
                 max_seq_len,   # capacity of every sequence, in tokens
                 dtype, device, *, batch_size: int = 1, hadamard_scale: float = ORTHONORMAL_SCALE,
                 code_from_fp32: bool = False, page_order=None, num_kv_heads: Optional[int] = None,
                 layout: int = TensorLayout.NHD):
        if dtype not in (torch.float16, torch.bfloat16):
            # the reference dispatches fp16 only (adamas/ops/csrc/pytorch_extension_utils.h:25-37);
            # bfloat16 q/k/v and caches are served through ADAMAS_F_BF16 in the flags of the library entry points
            raise RuntimeError(
                f"Adamas HIP path supports torch.float16 and torch.bfloat16 only, got {dtype}")
        if head_dim != 128:
            raise RuntimeError("Adamas HIP path supports head_dim 128 only")
        if num_heads % 8 != 0:
            raise RuntimeError("Adamas HIP path needs num_heads to be a multiple of 8")
        self.device = torch.device(device)
        self.dtype = dtype
        self.num_layers = num_layers
        self.num_heads = num_heads
        # grouped-query attention (not in the reference, which asserts equal head counts,
        # decode_handler.cuh:83): the caches hold num_kv_heads heads, query head h uses head
        # h // (num_heads // num_kv_heads)
        self.num_kv_heads = num_heads if num_kv_heads is None else int(num_kv_heads)
        if self.num_kv_heads <= 0 or num_heads % self.num_kv_heads != 0:
            raise RuntimeError("num_heads must be a multiple of num_kv_heads")
        self.head_dim = head_dim
        self.page_size = page_size
        self.batch_size = batch_size
        self.max_seq_len = max_seq_len
        if layout not in (TensorLayout.NHD, TensorLayout.HND):
            raise RuntimeError("layout must be TensorLayout.NHD or TensorLayout.HND")
        self.layout = layout
        self.hadamard_scale = float(hadamard_scale)
        # flags of the C ABI: data format and page layout for every entry point that sees them,
        # plus the code-generation option for the append entry points
        self.kv_flags = _lib.dtype_flags(dtype) | (_lib.F_HND if layout == TensorLayout.HND else 0)
        self.code_flags = (_lib.F_CODE_FROM_FP32 if code_from_fp32 else 0) | self.kv_flags

        pages_per_seq = (max_seq_len + page_size - 1) // page_size
        self.pool = PagePool(num_layers, self.num_kv_heads, head_dim, page_size, pages_per_seq * batch_size,
                             dtype, self.device, page_order=page_order, layout=layout)
        self.seqs = PagedSequences(self.pool, batch_size, max_seq_len, self.device)
        self.kv_cache = KvCache(self.seqs, 0, codes=False)
        self.hadamard_cache = KvCache(self.seqs, 0, codes=True)

        self._page_budget = page_budget
        self.inference_page_budget: Optional[int] = None

        # selection buffers, allocated once per budget value
        self.topk_dout_buffer: Optional[torch.Tensor] = None
        self.topk_dindices_buffer: Optional[torch.Tensor] = None
        self._topk_cache = {}
        self.topk_buf: Optional[torch.Tensor] = None   # scratch of the top-k kernel (zeroed once)
        self.kv_indices_without_last = ALL_PAST_TOKENS

        # workspace of the attention kernel and of the fused step (zero-filled once)
        self._workspace: Optional[torch.Tensor] = None
        self._workspace_need = {}
        self._len_bound: Optional[int] = None

    # --- device-side views used by the operator functions -----------------------------------------
    @property
    def kv_indices_with_last(self) -> torch.Tensor:
        return self.seqs.table_dev

    @property
    def kv_indptr_for_append(self) -> torch.Tensor:
        return self.seqs.indptr_dev

    @property
    def seq_lens(self) -> torch.Tensor:
        return self.seqs.seq_lens_dev

    @property
    def max_len_now(self) -> int:
        """Longest sequence: sizes grids and workspaces.  While a decode graph is being captured or
        replayed it is the bound fixed by begin_graph_decode (lengths then grow on the device only)."""
        if self._len_bound is not None:
            return self._len_bound
        return max(self.seqs.lengths)

    @property
    def min_len_now(self) -> int:
        return min(self.seqs.lengths)

    def workspace(self, budget: int, max_len: Optional[int] = None) -> torch.Tensor:
        """Workspace of the attention kernel and of the step for this token budget and the length
        bound the library is called with (`max_len`, by default max_len_now, which is what the
        operator functions pass).  The size the library asks for is monotonic neither in the budget
        nor in the length (different sizes take different paths), so reuse is decided by bytes, for
        exactly the sizes of the call; a new buffer is sized with a quarter of slack and for the
        full capacity too, so that a sequence growing token by token (or a dense budget that grows
        with it) reallocates a bounded number of times."""
        budget = max(1, min(int(budget), self.max_seq_len))
        max_len = self.max_len_now if max_len is None else int(max_len)
        max_len = max(1, min(max_len, self.max_seq_len))
        key = (budget, max_len)
        need = self._workspace_need.get(key)
        if need is None:
            need = _lib.load().adamas_workspace_bytes(self.batch_size, self.num_heads, max_len, budget)
            if len(self._workspace_need) > 4096:
                self._workspace_need.clear()
            self._workspace_need[key] = need
        if self._workspace is None or need > self._workspace.numel():
            full = _lib.load().adamas_workspace_bytes(self.batch_size, self.num_heads,
                                                      self.max_seq_len, budget)
            size = (max(need, full) * 5 // 4 + 255) // 256 * 256
            self._workspace = torch.zeros(size, dtype=torch.uint8, device=self.device)
        return self._workspace

    def topk_workspace(self, n: int, k: int) -> torch.Tensor:
        """Scratch of adamas_topk for rows of up to n candidates (the reference's `topk_buf`,
        controller.py:122, there sized for 8192 candidates whatever the sequence length)."""
        rows = self.batch_size * self.num_heads
        need = _lib.load().adamas_topk_workspace_bytes(rows, max(n, self.max_seq_len), k)
        if self.topk_buf is None or self.topk_buf.numel() < need:
            self.topk_buf = torch.zeros(need, dtype=torch.uint8, device=self.device)
        return self.topk_buf

    # --- reference interface ----------------------------------------------------------------------
    def set_page_budget(self, page_budget: int):
        """Token budget of the following begin_forward (reference controller.py:70-71; the model
        sets 1 << 20 for the two dense layers, llama.py:428)."""
        self._page_budget = page_budget

    def prepare_hadamard(self, seq_len: Union[int, Sequence[int]]):
        """Reserve room for `seq_len` new tokens (per sequence if a list is given) in the KV pages
        and, implicitly, in the code pages that share them (reference controller.py:74-78)."""
        if isinstance(seq_len, int):
            seq_len = [seq_len] * self.batch_size
        self.seqs.reserve(list(seq_len))

    def begin_forward(self, seq_len: int, updateTensor: bool = True):
        """Fix the budget regime of the coming layers (reference controller.py:82-131).  Nothing is
        uploaded or planned here; `updateTensor` is accepted for compatibility."""
        if seq_len > 1:
            return  # prefill: nothing to prepare
        if self.min_len_now < 2:
            # the reference asserts "at least two pages for excluding last page" (controller.py:101)
            raise AssertionError("decode needs at least one cached token before the current one")
        # In a ragged batch the budget is clamped by the longest sequence; a shorter sequence simply
        # selects all of its tokens (the kernels pad its selection with -1).
        self.inference_page_budget = min(self._page_budget, self.max_len_now)
        n_sel = self.inference_page_budget - 1
        if n_sel not in self._topk_cache:
            rows = self.batch_size * self.num_heads
            self._topk_cache[n_sel] = (
                # distances are integers up to 384: fp16 holds them exactly (bfloat16 would not)
                torch.zeros((rows, n_sel), dtype=torch.float16, device=self.device),
                torch.zeros((rows, n_sel), dtype=torch.int32, device=self.device),
            )
        self.topk_dout_buffer, self.topk_dindices_buffer = self._topk_cache[n_sel]

    # --- decode steps recorded in a HIP graph --------------------------------------------------------
    # The reference re-plans every step on the host (controller.py:82-131).  Here a step needs no host
    # work at all once the pages exist: lengths live on the device and every kernel masks by them.
    def begin_graph_decode(self, max_new_tokens: int):
        """Reserve the pages of the next `max_new_tokens` tokens and freeze the sizes the kernels are
        launched with (grids, workspaces) at the final length, so that one captured step can be
        replayed for all of them.  Call advance_on_device() at the start of the captured step."""
        self.seqs.reserve_pages_ahead(max_new_tokens)
        self._len_bound = max(self.seqs.lengths) + max_new_tokens

    def advance_on_device(self):
        self.seqs.advance_on_device()

    def end_graph_decode(self, tokens_generated: int):
        self.seqs.note_advanced(tokens_generated)
        self._len_bound = None

    def end_forward(self):
        """Nothing to free: the kernels own no state (reference controller.py:136-137)."""

    def need_estimate(self) -> bool:
        """True when the cache holds more tokens than the budget (reference controller.py:139-144)."""
        if self.inference_page_budget is None:
            return False
        return self.max_len_now > self.inference_page_budget

    def clean_states(self):
        self.seqs.release()
        self.inference_page_budget = None
