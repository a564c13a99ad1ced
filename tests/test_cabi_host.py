"""CPU-side checks: the C-ABI library loads and exports what include/adamas_hip.h declares, argument
validation returns the documented codes before anything is launched, and the host-side paging and
controller logic behaves like the reference's controller."""
import ctypes
import os
import re

import pytest
import torch

import adamas_amd.utils as U
from adamas_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "adamas_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(adamas_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), n
    assert set(names) == set(_lib.EXPORTED_SYMBOLS)
    assert lib.adamas_version() >= 100


def _declared_prototypes():
    """name -> list of parameter declarations, parsed from the header."""
    text = open(os.path.join(ROOT, "include", "adamas_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    protos = {}
    for m in re.finditer(r"\b(adamas_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        params = [p.strip() for p in m.group(2).replace("\n", " ").split(",")]
        protos[m.group(1)] = [] if params == ["void"] else params
    return protos


def test_ctypes_signatures_match_the_header():
    """Every prototype of the header against the ctypes table: same number of arguments, pointers
    bound as pointers, 64-bit integers as 64-bit, floats as floats."""
    import ctypes as C
    protos = _declared_prototypes()
    assert set(protos) == set(_lib.EXPORTED_SYMBOLS)
    for name, params in protos.items():
        _, argtypes = _lib._SIGNATURES[name]
        assert len(argtypes) == len(params), (name, len(argtypes), len(params))
        for decl, ct in zip(params, argtypes):
            if "*" in decl or "adamas_stream_t" in decl:
                assert ct in (C.c_void_p, C.c_char_p), (name, decl, ct)
            elif decl.startswith("float"):
                assert ct is C.c_float, (name, decl, ct)
            elif decl.startswith(("int64_t", "uint64_t", "size_t")):
                assert C.sizeof(ct) == 8, (name, decl, ct)
            else:
                assert decl.startswith(("uint32_t", "int32_t", "int ")), (name, decl)
                assert C.sizeof(ct) == 4, (name, decl, ct)


def test_argument_errors_are_reported_before_any_launch():
    lib = _lib.load()
    assert lib.adamas_hadamard(None, None, 0, 1.0, None) == 0                       # empty: no-op
    assert lib.adamas_hadamard(None, None, 4, 1.0, None) == -1                      # BADARG
    assert lib.adamas_hadamard(2, 2, 4, 1.0, None) == -4                            # ALIGN
    assert lib.adamas_pack_2bit(None, None, 3, None) == -1
    assert lib.adamas_append_decode(*([None] * 10), 1, 32, 32, 128, 16, 1.0, 0, None) == -1
    assert lib.adamas_append_prefill(16, 16, None, 4, 0, 16, 16, 16, 1, 32, 64, 16, 1.0, 0, None) == -2
    assert lib.adamas_append_prefill(16, 16, None, 40, 0, 16, 16, 16, 1, 32, 128, 16, 1.0, 0, None) == -1
    assert lib.adamas_estimate(16, 16, 16, 16, 16, 16, 8, 8, 0, 1, 0, 24, 16, 100, None) == -2    # no heads
    assert lib.adamas_estimate(16, 16, 16, 16, 16, 16, 8, 8, 0, 1, 32, 5, 16, 100, None) == -2    # 32 % kv heads
    assert lib.adamas_estimate(16, 16, 16, 16, 16, 16, 8, 8, 7, 1, 32, 32, 16, 100, None) == -1   # format
    assert lib.adamas_estimate(16, 16, 16, 16, 16, 16, 8, 8, 0, 1, 32, 8, 16, 1, None) == 0      # nothing to do
    assert lib.adamas_topk(None, 8, 8, None, 1, 0, None, 0, 1, 4, None, None, 4, 0, None, 0, None) == -1
    assert lib.adamas_topk(16, 8, 8, None, 1, 0, None, 0, 1, 4, 16, None, 2, 0, None, 0, None) == -1   # stride < k
    assert lib.adamas_topk(16, 40000, 40000, None, 1, 0, None, 0, 1, 4, 16, None, 4, 0, None, 0, None) == -3  # reduction levels need a workspace
    assert lib.adamas_topk_workspace_bytes(32, 131071, 255) >= 32 * 32 * 255 * 8
    # two-level integer path: 64 chunks x (128 candidates x 8 B + 512 B of histogram) per row
    assert lib.adamas_topk_workspace_bytes(32, 32767, 127) == 32 * 64 * (128 * 8 + 512)
    # k above 255: one row of 512 16-bit counts per chunk of 1024 keys
    assert lib.adamas_topk_workspace_bytes(32, 32767, 300) == 32 * 32 * 1024
    # short rows, k <= 255: 8 chunks x 128 candidates x 8 B per row (short candidate lists)
    assert lib.adamas_topk_workspace_bytes(32, 4096, 127) == 32 * 8 * 128 * 8
    assert lib.adamas_topk_workspace_bytes(32, 4096, 300) == 256       # one launch, no workspace
    assert lib.adamas_sparse_decode(16, 16, 16, 16, 16, None, 0, 0, 16, None, 0, 1, 32, 32, 64, 16, 0.1, 10, None) == -2
    # several splits without a workspace
    assert lib.adamas_sparse_decode(16, 16, 16, 16, 16, None, 0, 0, 16, None, 0, 1, 32, 8, 128, 16, 0.1, 5000, None) == -3
    assert lib.adamas_decode_step(*([16] * 7), 128, 16, None, None, 0, 1, 32, 32, 128, 16, 0.1, 100, 0, None) == -1
    assert lib.adamas_step_fused_supported(1, 32, 32768, 128) == 1
    assert lib.adamas_step_fused_supported(1, 32, 131072, 256) == 1       # 64 chunks of 2048 tokens
    assert lib.adamas_step_fused_supported(1, 32, 262144, 256) == 0       # too many candidate slots
    assert lib.adamas_step_fused_supported(1, 32, 4096, 1024) == 0        # budget beyond 256
    assert lib.adamas_step_fused_supported(1, 40, 32768, 128) == 1        # any multiple of 8 heads
    assert lib.adamas_step_fused_supported(1, 36, 32768, 128) == 0
    assert lib.adamas_step_candidates(16, 16, 16, 16, 16, 1024, 256, 1 << 30, 1, 32, 32, 16, 4096, 0, None) == -2
    assert lib.adamas_step_candidates(16, 16, 16, None, 16, 128, 256, 1 << 30, 1, 32, 32, 16, 4096, 0, None) == -1
    assert lib.adamas_step_attend(16, 16, 16, 16, 16, 16, 128, 16, None, None, 0, 1, 32, 32, 128, 16, 0.1, 4096, 0, None) == -1
    assert "workspace" in _lib.error_string(-3)
    with pytest.raises(RuntimeError):
        _lib.check(-2, "x")


def test_workspace_bytes_grows_with_sizes():
    lib = _lib.load()
    a = lib.adamas_workspace_bytes(1, 32, 4096, 64)
    b = lib.adamas_workspace_bytes(1, 32, 32768, 128)
    c = lib.adamas_workspace_bytes(16, 32, 32768, 128)
    assert 0 < a < b < c
    assert a % 256 == 0


def test_controller_workspace_covers_every_size_it_is_asked_for():
    """The size the library asks for is monotonic neither in the budget nor in the length: a
    controller that has served one size must still hand out enough bytes for the next, whatever
    the order (budget 300 then 256; 32832 tokens then 32769), and a sequence or a dense budget that
    grows token by token must not reallocate at every token."""
    lib = _lib.load()
    assert lib.adamas_workspace_bytes(1, 32, 32769, 128) > lib.adamas_workspace_bytes(1, 32, 32832, 128)
    c = _ctrl(max_seq_len=32832, num_layers=1)
    c.prepare_hadamard(32769)
    for budget in (32769, 128, 300, 256, 200, 128, 4096, 129):
        ws = c.workspace(budget)
        assert ws.numel() >= lib.adamas_workspace_bytes(1, 32, 32769, budget), budget
    seen = set()
    for _ in range(40):
        c.prepare_hadamard(1)
        n = c.max_len_now
        for budget in (n, 128):       # the dense layers, then the sparse ones, as a model alternates
            ws = c.workspace(budget)
            assert ws.numel() >= lib.adamas_workspace_bytes(1, 32, n, budget)
            seen.add(ws.data_ptr())
    assert len(seen) <= 2


def _ctrl(**kw):
    args = dict(num_layers=2, num_heads=32, head_dim=128, page_size=16, page_budget=64,
                max_seq_len=256, dtype=torch.float16, device="cpu")
    args.update(kw)
    return U.InferenceController(**args)


def test_controller_paging_and_budget_regime():
    c = _ctrl()
    assert not c.need_estimate()                      # before any begin_forward
    c.prepare_hadamard(40)                            # prefill of 40 tokens -> 3 pages
    assert c.kv_cache.seqlen == 40 and len(c.kv_cache.indicies) == 3
    assert c.kv_cache.last_page_len == 8 and c.hadamard_cache.seqlen == 40
    assert c.seq_lens.tolist() == [40]
    assert c.kv_indices_with_last[:3].tolist() == c.kv_cache.indicies
    c.begin_forward(40)
    c.end_forward()
    c.prepare_hadamard(1)
    c.begin_forward(1)
    assert c.inference_page_budget == 41 and not c.need_estimate()   # 41 tokens <= budget 64
    for _ in range(30):
        c.prepare_hadamard(1)
    c.begin_forward(1)
    assert c.inference_page_budget == 64 and c.need_estimate()
    assert c.topk_dindices_buffer.shape == (32, 63) and c.topk_dindices_buffer.dtype == torch.int32
    c.set_page_budget(1 << 20)                        # the two dense layers of the model
    c.begin_forward(1, updateTensor=False)
    assert not c.need_estimate()
    assert c.kv_indices_without_last is U.ALL_PAST_TOKENS
    c.clean_states()
    assert c.kv_cache.seqlen == 0 and c.pool.num_free_pages == 16


def test_controller_errors():
    with pytest.raises(RuntimeError):
        _ctrl(dtype=torch.float32)                    # fp16 (as the reference) and bf16 only
    with pytest.raises(RuntimeError):
        _ctrl(head_dim=64)
    with pytest.raises(RuntimeError):
        _ctrl(num_heads=12)
    c = _ctrl(max_seq_len=32)
    with pytest.raises(ValueError):
        c.prepare_hadamard(33)                        # beyond max_seq_len
    c.prepare_hadamard(1)
    with pytest.raises(AssertionError):
        c.begin_forward(1)                            # decode needs a past token
    with pytest.raises(ValueError):
        _ctrl(page_order=[0, 0, 1])


def test_pool_exhaustion_raises_keyerror_and_pages_are_reused():
    pool = U.PagePool(1, 32, 128, 16, 2, torch.float16, "cpu", page_order=[1, 0])
    assert pool.take() == 1 and pool.take() == 0
    with pytest.raises(KeyError):
        pool.take()
    pool.give_back([0])
    assert pool.take() == 0
    with pytest.raises(ValueError):
        pool.give_back([5])


def test_batched_sequences_fixed_stride_tables():
    c = _ctrl(batch_size=3, max_seq_len=64, page_order=list(range(11, -1, -1)))
    c.prepare_hadamard([5, 20, 64])
    assert c.seq_lens.tolist() == [5, 20, 64]
    assert c.kv_indptr_for_append.tolist() == [0, 4, 8, 12]
    assert [len(p) for p in c.seqs.pages] == [1, 2, 4]
    t = c.kv_indices_with_last.tolist()
    assert t[0] == 11 and t[4:6] == [10, 9] and t[8:12] == [8, 7, 6, 5]
    assert c.max_len_now == 64 and c.min_len_now == 5


def test_graph_decode_reserves_pages_ahead_and_tracks_lengths():
    """The HIP-graph decode loop: pages of the coming tokens are reserved up front, the lengths then
    advance on the device only, and the host catches up afterwards."""
    c = _ctrl(batch_size=2, max_seq_len=64)
    c.prepare_hadamard([10, 33])                       # 1 and 3 pages of 16 tokens
    free0 = c.pool.num_free_pages
    c.begin_graph_decode(20)                           # up to 30 and 53 tokens: 2 and 4 pages
    assert [len(p) for p in c.seqs.pages] == [2, 4]
    assert c.pool.num_free_pages == free0 - 2
    t = c.kv_indices_with_last.tolist()
    assert t[0:2] == c.seqs.pages[0] and t[4:8] == c.seqs.pages[1]
    assert c.max_len_now == 33 + 20                    # the bound the launches are sized with
    for _ in range(7):
        c.advance_on_device()
    assert c.seq_lens.tolist() == [17, 40]             # device lengths moved, host lengths did not
    assert c.seqs.lengths == [10, 33]
    c.end_graph_decode(7)
    assert c.seqs.lengths == [17, 40] and c.max_len_now == 40
    c.prepare_hadamard(1)                              # the eager path continues from there
    assert c.seq_lens.tolist() == [18, 41] and [len(p) for p in c.seqs.pages] == [2, 4]
    with pytest.raises(ValueError):
        c.begin_graph_decode(64)                       # beyond max_seq_len
    c.clean_states()
    assert c.pool.num_free_pages == 8 and c.seq_lens.tolist() == [0, 0]
    c.prepare_hadamard([3, 3])
    c.begin_graph_decode(4)
    with pytest.raises(RuntimeError):
        c.end_graph_decode(40)                         # more tokens than pages were reserved for


def test_ops_reject_cpu_tensors():
    c = _ctrl()
    c.prepare_hadamard(4)
    x = torch.zeros(4, 32, 128, dtype=torch.float16)
    with pytest.raises(RuntimeError):
        U.append_kvh(x, x, x, c, 0)
    with pytest.raises(RuntimeError):
        U.hadamard_transform(x)


def test_step_plan_covers_every_sequence_with_balanced_chunks():
    """The geometry the two-launch step derives from the sizes of a call (adamas_step_plan): the
    chunks tile the past tokens of the longest sequence in 16-token units, differ by at most one
    unit for a single sequence, fit the workgroup (at most four passes of 512 tokens) and the
    second launch (at most 64 chunks, 1024 candidate slots per head for one sequence, 2048 for a
    batch; a power of two of 8 .. 256 slots per chunk, never more than the budget needs)."""
    lens = sorted(set([2, 3, 17, 18, 33, 511, 512, 513, 514, 1000, 4096, 4097, 8192, 8193, 16384, 16385,
                       16400, 20000, 32767, 32768, 32769, 32784, 32785, 33024, 36864, 40000, 65536, 65537,
                       100000, 131056, 131072] + list(range(2, 140000, 3571))))
    for batch in (1, 2, 16):
        for heads in (32, 40, 64):
            for budget in (2, 16, 64, 128, 200, 256):
                for L in lens:
                    p = _lib.step_plan(batch, heads, L, budget)
                    where = (batch, heads, L, budget, p)
                    if not p["ok"]:
                        assert L - 1 > 64 * 2048 or (batch > 1 and L - 1 > 64 * 2048), where
                        continue
                    units = (L - 1 + 15) // 16
                    assert 1 <= p["chunks"] <= 64, where
                    assert p["heads"] in (4, 8) and heads % p["heads"] == 0, where
                    # the chunks cover all units: a single sequence is tiled exactly, a batch is
                    # covered by fixed-size chunks
                    total = p["chunks"] * p["units_q"] + p["units_r"]
                    if batch == 1 and p["units_r"] == 0 and p["units_q"] % 32 == 0 and p["chunks"] * p["units_q"] > units:
                        assert total - units < p["units_q"], where      # fixed 512-token chunks
                    elif batch == 1:
                        assert total == units or total - units < p["units_q"], where
                    else:
                        assert total >= units and p["units_r"] == 0, where
                    assert p["units_r"] < p["chunks"], where
                    longest = p["units_q"] + (1 if p["units_r"] else 0)
                    assert 1 <= p["passes"] <= 4 and longest <= 32 * p["passes"], where
                    assert longest > 32 * (p["passes"] - 1), where
                    assert p["partial"] == int(p["units_r"] != 0 or p["units_q"] % 32 != 0), where
                    kc = p["kc"]
                    assert kc in (8, 16, 32, 64, 128, 256), where
                    assert p["chunks"] * kc <= (1024 if batch == 1 else 2048) or kc == 8, where
                    # never more slots than the budget can use (rounded up to a power of two, at least 8)
                    need = 8
                    while need < budget - 1:
                        need *= 2
                    assert kc <= need, where
    # what the headline workloads get
    assert _lib.step_plan(1, 32, 32768, 128) == {"ok": 1, "heads": 8, "chunks": 64, "units_q": 32, "units_r": 0,
                                                 "passes": 1, "partial": 0, "kc": 16}
    p = _lib.step_plan(1, 32, 33024, 128)
    assert (p["chunks"], p["units_q"], p["units_r"], p["passes"], p["partial"]) == (64, 32, 16, 2, 1)
    assert _lib.step_plan(1, 32, 131072, 256)["passes"] == 4
    assert _lib.step_plan(16, 32, 32768, 128)["kc"] == 32
    assert _lib.step_plan(1, 32, 32768, 1024)["ok"] == 0       # budgets above 256 take the histogram path
