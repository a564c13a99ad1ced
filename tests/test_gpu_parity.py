"""GPU parity tests: the HIP path (through adamas_amd.utils -> ctypes -> libadamas_hip.so) against
the CPU oracle on the same seeded inputs.

Bars: 2-bit codes, integer L1 distances and top-k index sets bit-exact; attention outputs within
2e-3 max-abs (fp16 output, fp32 accumulation), the tolerance the benchmark definition states.
"""
import math

import numpy as np
import pytest
import torch

import adamas_amd.utils as U
from adamas_amd import _lib, synth
from oracle import adamas_oracle as O
from tests import helpers as T

pytestmark = pytest.mark.gpu
ATTN_TOL = 2e-3


# ------------------------------------------------------------------------ Hadamard and packing --
@pytest.mark.parametrize("scale", [1.0, 128 ** -0.5])
@pytest.mark.parametrize("rows", [1, 2, 64, 1000])
def test_hadamard_bit_exact(gpu_device, scale, rows):
    g = torch.Generator().manual_seed(rows)
    x = (torch.randn(rows, 32, 128, generator=g) * 3).half()
    y = U.hadamard_transform(x.to(gpu_device), scale=scale)
    want = O.hadamard_fp16(T.np16(x), scale)
    got = T.np16(y)
    bad = np.argwhere(got.view(np.uint16) != want.view(np.uint16))
    assert len(bad) == 0, (len(bad), [(tuple(i), float(got[tuple(i)]), float(want[tuple(i)])) for i in bad[:5]])
    xi = x.to(gpu_device).clone()
    U.hadamard_transform(xi, inplace=True, scale=scale)
    assert torch.equal(xi, y)


def test_pack_2bit_bit_exact(gpu_device):
    g = torch.Generator().manual_seed(0)
    codes = torch.randint(0, 4, (77, 32, 128), generator=g)
    got = U.pack_2bit(codes.half().to(gpu_device), 0)
    assert np.array_equal(T.words_u16(got), O.pack_2bit(codes.numpy()))


# ------------------------------------------------------------------------------------ append ----
@pytest.mark.parametrize("page_size", [1, 16, 7])
@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("scale", [1.0, 128 ** -0.5])
def test_append_codes_and_kv(gpu_device, page_size, fused, scale):
    L = 203
    seq = synth.make_sequence(L, 4, torch.Generator().manual_seed(11))
    ctrl = T.make_controller(gpu_device, 256, 64, page_size, scale=scale, shuffle_seed=5)
    k, v, q = seq.k.to(gpu_device), seq.v.to(gpu_device), seq.q.to(gpu_device)
    T.fill_sequence(ctrl, k[:L - 1], v[:L - 1], fused=fused, chunk=64)
    q_code = T.decode_append(ctrl, q[None], k[L - 1:], v[L - 1:], fused=fused)
    kk, vv, cc = T.read_logical_cache(ctrl)
    assert np.array_equal(kk.view(np.uint16), T.np16(seq.k).view(np.uint16))
    assert np.array_equal(vv.view(np.uint16), T.np16(seq.v).view(np.uint16))
    assert np.array_equal(cc, O.codes_from_raw(T.np16(seq.k), scale))
    assert np.array_equal(T.words_u16(q_code)[0], O.codes_from_raw(T.np16(seq.q), scale))


@pytest.mark.parametrize("hkv,chunk", [(1, 1), (1, 7), (2, 5), (4, 3), (8, 37), (32, 1), (32, 33)])
@pytest.mark.parametrize("fused", [True, False])
def test_prefill_append_partial_row_groups(gpu_device, hkv, chunk, fused):
    """Prefill slices whose row count (tokens x key/value heads) is not a multiple of the rows a wave
    or a workgroup of the append kernel covers, starting at positions inside a page."""
    L = 83
    seq = synth.make_sequence(L, 2, torch.Generator().manual_seed(40 + hkv + chunk))
    k, v = seq.k[:, :hkv].contiguous(), seq.v[:, :hkv].contiguous()
    ctrl = T.make_controller(gpu_device, 96, 16, 7, shuffle_seed=2, num_kv_heads=hkv)
    T.fill_sequence(ctrl, k.to(gpu_device), v.to(gpu_device), fused=fused, chunk=chunk)
    kk, vv, cc = T.read_logical_cache(ctrl)
    assert np.array_equal(kk.view(np.uint16), T.np16(k).view(np.uint16))
    assert np.array_equal(vv.view(np.uint16), T.np16(v).view(np.uint16))
    assert np.array_equal(cc, O.codes_from_raw(T.np16(k), 1.0))


def test_append_codes_from_fp32_flag(gpu_device):
    L = 300
    seq = synth.make_sequence(L, 4, torch.Generator().manual_seed(12))
    ctrl = T.make_controller(gpu_device, 512, 64, 16, code_from_fp32=True)
    T.fill_sequence(ctrl, seq.k.to(gpu_device), seq.v.to(gpu_device))
    _, _, cc = T.read_logical_cache(ctrl)
    assert np.array_equal(cc, O.codes_from_raw(T.np16(seq.k), 1.0, round_fp16=False))


# ---------------------------------------------------------------------------------- estimate ----
# kv lengths of the reference's estimator test (adamas/tests/test_estimate.py:67)
@pytest.mark.parametrize("kv_len", [27, 61, 113, 482, 577, 1110, 1541, 2047, 3330])
@pytest.mark.parametrize("page_size", [1, 16, 3])
def test_estimate_bit_exact(gpu_device, kv_len, page_size):
    seq = synth.make_sequence(kv_len, 4, torch.Generator().manual_seed(kv_len))
    ctrl = T.make_controller(gpu_device, 4096, 1024, page_size, shuffle_seed=kv_len)
    k, v, q = seq.k.to(gpu_device), seq.v.to(gpu_device), seq.q.to(gpu_device)
    T.fill_sequence(ctrl, k[:kv_len - 1], v[:kv_len - 1])
    q_code = T.decode_append(ctrl, q[None], k[kv_len - 1:], v[kv_len - 1:])
    est = U.decode_estimate(q_code, ctrl, 0)
    assert est.shape == (32, kv_len - 1) and est.dtype == torch.float16
    ora = T.oracle_step(seq.q, seq.k, seq.v, 1024)
    assert np.array_equal(T.np16(est).astype(np.int32), ora["dist"])


def test_estimate_uniform_random_codes(gpu_device):
    """Codes drawn uniformly (not Hadamard-derived) so that every code pair, including (1,2) and
    (0,3), occurs; written straight into the code cache."""
    L, P = 1000, 16
    rng = np.random.default_rng(0)
    kc = rng.integers(0, 4, size=(L, 32, 128)).astype(np.uint8)
    qc = rng.integers(0, 4, size=(32, 128)).astype(np.uint8)
    ctrl = T.make_controller(gpu_device, 1024, 64, P, shuffle_seed=1)
    ctrl.prepare_hadamard(L)
    words = torch.from_numpy(O.pack_2bit(kc).view(np.int16)).to(gpu_device)      # [L, H, 16]
    pages = torch.tensor(ctrl.seqs.pages[0], dtype=torch.long, device=gpu_device)
    padded = torch.zeros((len(pages) * P, 32, 16), dtype=torch.int16, device=gpu_device)
    padded[:L] = words
    ctrl.pool.codes[0][pages] = padded.view(len(pages), P, 32, 16)
    q_code = torch.from_numpy(O.pack_2bit(qc).view(np.int16))[None].to(gpu_device)
    est = U.decode_estimate(q_code, ctrl, 0)
    want = O.l1_distance_codes(qc, kc[:L - 1])
    assert np.array_equal(T.np16(est).astype(np.int32), want)
    xor = O.xor_metric_packed(O.pack_2bit(qc), O.pack_2bit(kc[:L - 1]))
    assert not np.array_equal(want, xor)  # the reference CUDA metric would fail this test


# ------------------------------------------------------------------------------------- top-k ----
def _call_topk(values_fp16, k, mode, in_idx=None):
    rows, n = values_fp16.shape
    out_idx = torch.full((rows, k), -7, dtype=torch.int32, device=values_fp16.device)
    out_val = torch.zeros((rows, k), dtype=torch.float16, device=values_fp16.device)
    lib = _lib.load()
    ws = torch.zeros(lib.adamas_topk_workspace_bytes(rows, n, k), dtype=torch.uint8,
                     device=values_fp16.device)
    rc = lib.adamas_topk(values_fp16.data_ptr(), values_fp16.stride(0), n, None, 1, 0,
                         _lib.ptr(in_idx), in_idx.stride(0) if in_idx is not None else 0,
                         rows, k, out_idx.data_ptr(), out_val.data_ptr(), k, mode,
                         ws.data_ptr(), ws.numel(), _lib.current_stream())
    _lib.check(rc, "adamas_topk")
    # a second call on the same workspace must give the same answer (counters back at zero)
    out_idx2 = torch.full_like(out_idx, -9)
    rc = lib.adamas_topk(values_fp16.data_ptr(), values_fp16.stride(0), n, None, 1, 0,
                         _lib.ptr(in_idx), in_idx.stride(0) if in_idx is not None else 0,
                         rows, k, out_idx2.data_ptr(), None, k, mode,
                         ws.data_ptr(), ws.numel(), _lib.current_stream())
    assert torch.equal(out_idx, out_idx2)
    _lib.check(rc, "adamas_topk")
    return out_idx, out_val


# sizes of the reference's top-k test (adamas/tests/test_topk.py:23)
@pytest.mark.parametrize("kv_len", [13, 24, 51, 77, 244, 311, 502, 1110])
@pytest.mark.parametrize("k_budget", [2, 5, 7, 19, 31, 69, 111, 251])
def test_topk_generic_fp16(gpu_device, kv_len, k_budget):
    if k_budget > kv_len:
        pytest.skip("k should be less than kv_len")
    g = torch.Generator().manual_seed(kv_len * 1000 + k_budget)
    q = torch.randn(32, 1, 128, generator=g).half()
    k = torch.randn(32, kv_len, 128, generator=g).half()
    w = (torch.matmul(q.float(), k.float().transpose(1, 2)) / math.sqrt(128)).squeeze(1).half()
    idx, val = _call_topk(w.to(gpu_device).contiguous(), k_budget, _lib.KEY_FP16_GENERIC)
    want = O.topk_smallest(T.np16(w).astype(np.float32), k_budget)
    got = np.sort(T.np16(idx), axis=-1)
    assert np.array_equal(got, want)
    # the reference's own check: sum of the selected values (test_topk.py:42-64)
    ref_sum = torch.topk(w.float(), k_budget, dim=-1, largest=False).values.sum(-1)
    torch.testing.assert_close(val.float().sum(-1).cpu(), ref_sum, rtol=5e-3, atol=5e-3)
    # values travel with their indices
    assert torch.equal(val.cpu(), torch.gather(w, 1, idx.cpu().long()))


@pytest.mark.parametrize("n,k", [(100, 10), (5000, 127), (32767, 127), (40000, 255), (8193, 8192),
                                 (131071, 255), (300000, 1024), (4097, 1024), (9000, 1025),
                                 (32767, 512), (32767, 4096), (70000, 2000), (5000, 300),
                                 (32769, 256), (1000000, 64)])
def test_topk_integer_ties_lowest_index(gpu_device, n, k):
    rng = np.random.default_rng(n)
    v = rng.integers(100, 140, size=(32, n)).astype(np.float16)   # heavy ties
    vt = torch.from_numpy(v).to(gpu_device)
    idx, _ = _call_topk(vt, k, _lib.KEY_FP16_INT)
    want = O.topk_smallest(v.astype(np.int32), k)
    assert np.array_equal(np.sort(T.np16(idx), axis=-1), want)
    # generic mode must agree on the same data
    idx2, _ = _call_topk(vt, k, _lib.KEY_FP16_GENERIC)
    assert torch.equal(idx, idx2)
    # output order: below-threshold by index, then ties by index (deterministic)
    idx3, _ = _call_topk(vt, k, _lib.KEY_FP16_INT)
    assert torch.equal(idx, idx3)


def test_topk_all_equal_and_gather(gpu_device):
    v = torch.full((32, 3000), 7.0, dtype=torch.float16, device=gpu_device)
    idx, _ = _call_topk(v, 50, _lib.KEY_FP16_INT)
    assert torch.equal(idx.cpu(), torch.arange(50, dtype=torch.int32).repeat(32, 1))
    perm = torch.stack([torch.randperm(3000, generator=torch.Generator().manual_seed(i)) for i in range(32)])
    idx_g, _ = _call_topk(v, 50, _lib.KEY_FP16_INT, in_idx=perm.int().to(gpu_device))
    assert torch.equal(idx_g.cpu(), perm[:, :50].int())


@pytest.mark.parametrize("n,k,mode", [(20000, 100, "fp16"), (9001, 255, "fp16"), (70000, 31, "u16"),
                                      (20000, 700, "fp16"), (32768, 1024, "u16"),
                                      (70000, 3000, "u16")])
def test_topk_two_level_integer_path(gpu_device, n, k, mode):
    """Long rows of integer keys (k up to 255: candidates per chunk, then one workgroup per row;
    larger k: a histogram per chunk, then threshold and emission): gathered indices, returned values,
    unaligned rows, and the same answer as the general path without a workspace."""
    rng = np.random.default_rng(n + k)
    flat = rng.integers(0, 385, size=(32 * (n + 5) + 1,))
    if mode == "fp16":
        base = torch.from_numpy(flat.astype(np.float16)).to(gpu_device)
        key_mode = _lib.KEY_FP16_INT
    else:
        base = torch.from_numpy(flat.astype(np.uint16).view(np.int16)).to(gpu_device).view(torch.float16)
        key_mode = _lib.KEY_U16_INT
    v = base[1:].view(32, n + 5)[:, :n]      # odd offset, odd stride: the scalar load path
    ints = flat[1:].reshape(32, n + 5)[:, :n]
    perm = torch.stack([torch.randperm(n, generator=torch.Generator().manual_seed(i)) for i in range(32)])
    idx, val = _call_topk(v, k, key_mode, in_idx=perm.int().to(gpu_device))
    want = O.topk_smallest(ints.astype(np.int32), k)          # sorted positions
    got_pos = torch.argsort(perm, dim=1)[torch.arange(32)[:, None], idx.cpu().long()]  # undo the gather
    assert np.array_equal(np.sort(got_pos.numpy(), axis=-1), want)
    picked = np.take_along_axis(ints, got_pos.numpy(), axis=1)
    got_val = T.np16(val).astype(np.float32) if mode == "fp16" else T.np16(val).view(np.uint16)
    assert np.array_equal(got_val.astype(np.int64), picked)
    if n <= 32768:   # without a workspace the single-launch path answers, in the same order
        lib = _lib.load()
        out2 = torch.full_like(idx, -5)
        pi = perm.int().to(gpu_device)
        rc = lib.adamas_topk(v.data_ptr(), v.stride(0), n, None, 1, 0, pi.data_ptr(), pi.stride(0), 32,
                             k, out2.data_ptr(), None, k, key_mode, None, 0, _lib.current_stream())
        assert rc == 0
        assert torch.equal(idx, out2)


@pytest.mark.parametrize("mode", ["fp16", "u16"])
@pytest.mark.parametrize("kind", ["equal", "clustered", "runs", "short_rows"])
@pytest.mark.parametrize("n,k", [(32768, 127), (33000, 127), (131072, 255), (5000, 63), (70000, 255),
                                 (20000, 16), (600, 200)])
def test_topk_short_lists_fall_back_to_the_row(gpu_device, n, k, kind, mode):
    """The chunk lists of the two-level integer selection hold fewer entries than k.  Rows whose
    selection needs more keys of one chunk than its list holds (every key tied, the smallest keys
    clustered in one chunk, long runs of equal keys across chunk boundaries, rows that end inside
    the first chunk) are completed from the input row: positions, order, gathered indices and
    returned values must equal the general path's."""
    rng = np.random.default_rng(n * 7 + k)
    rows = 32
    if kind == "equal":
        ints = np.full((rows, n), 37, dtype=np.int64)
    elif kind == "clustered":
        ints = rng.integers(200, 385, size=(rows, n))
        for r in range(rows):
            start = int(rng.integers(0, max(1, n - 2 * k)))
            ints[r, start:start + 2 * k] = rng.integers(0, 50, size=min(2 * k, n - start))
    elif kind == "runs":
        run = np.repeat(rng.integers(90, 110, size=(rows, n // 300 + 1)), 300, axis=1)[:, :n]
        ints = run
    else:
        ints = rng.integers(0, 385, size=(rows, n))
    if mode == "fp16":
        v = torch.from_numpy(ints.astype(np.float16)).to(gpu_device)
        key_mode = _lib.KEY_FP16_INT
    else:
        v = torch.from_numpy(ints.astype(np.uint16).view(np.int16)).to(gpu_device).view(torch.float16)
        key_mode = _lib.KEY_U16_INT
    lens = None
    if kind == "short_rows":   # per-row lengths, some shorter than k, some ending inside chunk 0
        lens = rng.integers(1, n, size=rows).astype(np.int32)
        lens[:4] = [1, k - 1, k, k + 1]
        lens[4] = min(n, 300)
    perm = torch.stack([torch.randperm(n, generator=torch.Generator().manual_seed(i)) for i in range(rows)])
    pi = perm.int().to(gpu_device)
    lib = _lib.load()
    idx = torch.full((rows, k), -7, dtype=torch.int32, device=gpu_device)
    val = torch.zeros((rows, k), dtype=torch.float16, device=gpu_device)
    ws = torch.zeros(lib.adamas_topk_workspace_bytes(rows, n, k), dtype=torch.uint8, device=gpu_device)
    lens_d = torch.from_numpy(lens).to(gpu_device) if lens is not None else None
    for _ in range(2):   # twice on the same workspace
        rc = lib.adamas_topk(v.data_ptr(), v.stride(0), n, _lib.ptr(lens_d), 1, 0, pi.data_ptr(), pi.stride(0),
                             rows, k, idx.data_ptr(), val.data_ptr(), k, key_mode, ws.data_ptr(), ws.numel(),
                             _lib.current_stream())
        _lib.check(rc, "adamas_topk")
    got = idx.cpu().numpy()
    gval = T.np16(val).astype(np.float32) if mode == "fp16" else T.np16(val).view(np.uint16).astype(np.float32)
    inv = torch.argsort(perm, dim=1).numpy()
    for r in range(rows):
        nr = int(lens[r]) if lens is not None else n
        row = ints[r, :nr]
        take = min(k, nr)
        # ties to the lowest index; output order: keys below the threshold by index, then the ties
        order = np.lexsort((np.arange(nr), row))[:take]
        thr = row[order[-1]]
        want = np.concatenate([np.sort(order[row[order] < thr]), np.sort(order[row[order] == thr])])
        if nr <= k:   # a row no longer than k is taken whole, in index order
            want = np.arange(nr)
        assert (got[r, take:] == -1).all(), (r, nr)
        pos = inv[r][got[r, :take]]          # undo the gather
        assert np.array_equal(pos, want), (r, nr)
        assert np.array_equal(gval[r, :take], row[want].astype(np.float32)), (r, nr)


def test_topk_unaligned_rows_and_short_rows(gpu_device):
    rng = np.random.default_rng(3)
    base = torch.from_numpy(rng.integers(0, 385, size=(32 * 1001 + 3,)).astype(np.float16)).to(gpu_device)
    v = base[3:].view(32, 1001)[:, :999]   # odd offset and odd row stride: scalar load path
    idx, _ = _call_topk(v, 64, _lib.KEY_FP16_INT)
    want = O.topk_smallest(T.np16(v).astype(np.int32), 64)
    assert np.array_equal(np.sort(T.np16(idx), axis=-1), want)
    # a row shorter than k selects everything and pads with -1
    short = v[:, :10]
    idx_s, _ = _call_topk(short, 16, _lib.KEY_FP16_INT)
    exp = torch.cat([torch.arange(10), torch.full((6,), -1)]).int().repeat(32, 1)
    assert torch.equal(idx_s.cpu(), exp)


# --------------------------------------------------------------------------- sparse attention ---
# shapes of the reference's approximate-attention test (adamas/tests/test_approx_attention.py:100)
@pytest.mark.parametrize("kv_len", [27, 61, 113, 482, 577, 1011, 1541])
@pytest.mark.parametrize("token_budget", [64, 112, 240, 496, 880, 1136])
def test_sparse_attention_forced_indices(gpu_device, kv_len, token_budget):
    seq = synth.make_sequence(kv_len, 4, torch.Generator().manual_seed(kv_len + token_budget))
    ctrl = T.make_controller(gpu_device, 2048, token_budget, 16, shuffle_seed=2)
    k, v, q = seq.k.to(gpu_device), seq.v.to(gpu_device), seq.q.to(gpu_device)
    T.fill_sequence(ctrl, k[:kv_len - 1], v[:kv_len - 1])
    T.decode_append(ctrl, q[None], k[kv_len - 1:], v[kv_len - 1:])
    ora = T.oracle_step(seq.q, seq.k, seq.v, token_budget)
    if not ctrl.need_estimate():
        o = U.decode_sparse_attn(q[None], ctrl, 0, ctrl.kv_indices_without_last)
    else:
        sel = np.stack([s[:-1] for s in ora["sets"]]).astype(np.int32)   # indices forced from the oracle
        o = U.decode_sparse_attn(q[None], ctrl, 0, torch.from_numpy(sel).to(gpu_device))
    err = np.abs(T.np16(o)[0].astype(np.float64) - ora["out"]).max()
    assert err <= ATTN_TOL, err


# the sweep of the reference's kernel test (kernels/src/test/test_batch_decode.cu:238-257): sequence
# lengths 63 .. 28837, page sizes 1, 3, 7, 16, 32, budgets 16 .. 128; indices are random here (that
# test draws them at random too), the whole step is run on the same state as well
@pytest.mark.parametrize("page_size", [1, 3, 7, 16, 32])
@pytest.mark.parametrize("kv_len,budget", [(63, 16), (63, 128), (2111, 32), (28837, 64), (28837, 128)])
def test_sparse_attention_page_size_sweep(gpu_device, kv_len, budget, page_size):
    g = torch.Generator().manual_seed(kv_len * 37 + budget + page_size)
    q = torch.randn(32, 128, generator=g).half()
    k = torch.randn(kv_len, 32, 128, generator=g).half()
    v = torch.randn(kv_len, 32, 128, generator=g).half()
    ctrl = T.make_controller(gpu_device, kv_len, budget, page_size, shuffle_seed=page_size)
    kd, vd, qd = k.to(gpu_device), v.to(gpu_device), q.to(gpu_device)
    T.fill_sequence(ctrl, kd[:kv_len - 1], vd[:kv_len - 1])
    q_code = T.decode_append(ctrl, qd[None], kd[kv_len - 1:], vd[kv_len - 1:])
    n_sel = min(budget, kv_len) - 1
    sel = torch.stack([torch.randperm(kv_len - 1, generator=g)[:n_sel] for _ in range(32)]).int()
    o = U.decode_sparse_attn(qd[None], ctrl, 0, sel.to(gpu_device))
    sets = [np.append(sel[h].numpy(), kv_len - 1) for h in range(32)]
    want = O.sparse_attention(T.np16(q), T.np16(k), T.np16(v), sets)
    assert np.abs(T.np16(o)[0].astype(np.float64) - want).max() <= ATTN_TOL
    if ctrl.need_estimate():   # the fused step on the same caches: compare with the three operators
        est = U.decode_estimate(q_code, ctrl, 0)
        U.decode_topk(est, ctrl)
        o3 = U.decode_sparse_attn(qd[None], ctrl, 0, ctrl.topk_dindices_buffer)
        sel3 = np.sort(T.np16(ctrl.topk_dindices_buffer).astype(np.int64), axis=1)
        o_f, sel_f = U.decode_step(qd[None], q_code, ctrl, 0, return_indices=True)
        assert np.array_equal(np.sort(T.np16(sel_f).astype(np.int64), axis=1), sel3)
        assert np.abs(T.np16(o_f).astype(np.float64) - T.np16(o3).astype(np.float64)).max() <= ATTN_TOL


# the operator picks workgroup size, rows per lane group and rows per split from the row count: both
# sides of every boundary of that rule, random indices, twice in a row (arrival counters back at zero)
@pytest.mark.parametrize("budget", [64, 65, 128, 129, 512, 513, 1024, 2048, 2049, 3000])
def test_sparse_attention_row_count_boundaries(gpu_device, budget):
    kv_len = 4100
    g = torch.Generator().manual_seed(budget)
    q = torch.randn(32, 128, generator=g).half()
    k = torch.randn(kv_len, 32, 128, generator=g).half()
    v = torch.randn(kv_len, 32, 128, generator=g).half()
    ctrl = T.make_controller(gpu_device, kv_len, budget, 16, shuffle_seed=budget)
    kd, vd, qd = k.to(gpu_device), v.to(gpu_device), q.to(gpu_device)
    T.fill_sequence(ctrl, kd[:kv_len - 1], vd[:kv_len - 1])
    T.decode_append(ctrl, qd[None], kd[kv_len - 1:], vd[kv_len - 1:])
    sel = torch.stack([torch.randperm(kv_len - 1, generator=g)[:budget - 1] for _ in range(32)]).int()
    o = U.decode_sparse_attn(qd[None], ctrl, 0, sel.to(gpu_device))
    sets = [np.append(sel[h].numpy(), kv_len - 1) for h in range(32)]
    want = O.sparse_attention(T.np16(q), T.np16(k), T.np16(v), sets)
    assert np.abs(T.np16(o)[0].astype(np.float64) - want).max() <= ATTN_TOL
    o2 = U.decode_sparse_attn(qd[None], ctrl, 0, sel.to(gpu_device))
    assert torch.equal(o, o2)


@pytest.mark.parametrize("kv_len", [1, 2, 129, 4000, 9000])
def test_dense_mode_equals_dense_attention(gpu_device, kv_len):
    seq = synth.make_sequence(kv_len, 0, torch.Generator().manual_seed(kv_len))
    ctrl = T.make_controller(gpu_device, 9216, 1 << 20, 16, shuffle_seed=3)
    k, v, q = seq.k.to(gpu_device), seq.v.to(gpu_device), seq.q.to(gpu_device)
    T.fill_sequence(ctrl, k, v)
    ctrl.inference_page_budget = 1 << 20
    o = U.decode_sparse_attn(q[None], ctrl, 0, U.ALL_PAST_TOKENS)
    want = O.dense_attention(T.np16(seq.q), T.np16(seq.k), T.np16(seq.v))
    assert np.abs(T.np16(o)[0].astype(np.float64) - want).max() <= ATTN_TOL
    # twice in a row: the split-merge counters must be back at zero
    o2 = U.decode_sparse_attn(q[None], ctrl, 0, U.ALL_PAST_TOKENS)
    assert torch.equal(o, o2)


def test_sparse_attention_one_hot_v_and_padding(gpu_device):
    L = 500
    seq = synth.make_sequence(L, 0, torch.Generator().manual_seed(77))
    ctrl = T.make_controller(gpu_device, 512, 32, 16)
    T.fill_sequence(ctrl, seq.k.to(gpu_device), seq.v.to(gpu_device))
    ctrl.inference_page_budget = 32
    sel = torch.full((32, 31), -1, dtype=torch.int32)
    sel[:, 0] = 17   # one real entry, the rest padding; the current token is added by the kernel
    o = U.decode_sparse_attn(seq.q[None].to(gpu_device), ctrl, 0, sel.to(gpu_device))
    want = O.sparse_attention(T.np16(seq.q), T.np16(seq.k), T.np16(seq.v), [np.array([17, L - 1])] * 32)
    assert np.abs(T.np16(o)[0].astype(np.float64) - want).max() <= ATTN_TOL


# ------------------------------------------------------------------------------ whole step ------
SCALES = [1.0, 128 ** -0.5]   # raw butterfly (this build's default) and the orthonormal transform


def _run_step(gpu_device, seq, budget, page_size, shuffle_seed, fused_append=True, scale=1.0):
    L = seq.k.shape[0]
    ctrl = T.make_controller(gpu_device, L, budget, page_size, shuffle_seed=shuffle_seed, scale=scale)
    k, v, q = seq.k.to(gpu_device), seq.v.to(gpu_device), seq.q.to(gpu_device)
    T.fill_sequence(ctrl, k[:L - 1], v[:L - 1])
    q_code = T.decode_append(ctrl, q[None], k[L - 1:], v[L - 1:], fused=fused_append)
    assert ctrl.need_estimate()
    est = U.decode_estimate(q_code, ctrl, 0)
    U.decode_topk(est, ctrl)
    o = U.decode_sparse_attn(q[None], ctrl, 0, ctrl.topk_dindices_buffer)
    sel = ctrl.topk_dindices_buffer.clone()
    o_fused, sel_fused = U.decode_step(q[None], q_code, ctrl, 0, return_indices=True)
    return ctrl, q_code, est, sel, o, o_fused, sel_fused.clone()


def _check_step(seq, budget, q_code, est, sel, o, o_fused, sel_fused, scale=1.0):
    L = seq.k.shape[0]
    ora = T.oracle_step(seq.q, seq.k, seq.v, budget, scale=scale)
    assert np.array_equal(T.words_u16(q_code)[0], ora["q_words"])
    assert np.array_equal(T.np16(est).astype(np.int32), ora["dist"])
    ok, h = T.sets_equal(T.np16(sel), ora["sets"], L)
    assert ok, f"index set differs for head {h}"
    ok, h = T.sets_equal(T.np16(sel_fused), ora["sets"], L)
    assert ok, f"fused index set differs for head {h}"
    assert np.abs(T.np16(o)[0].astype(np.float64) - ora["out"]).max() <= ATTN_TOL
    assert np.abs(T.np16(o_fused)[0].astype(np.float64) - ora["out"]).max() <= ATTN_TOL
    return ora


# The scale of the reference's third-party Hadamard transform is not fixed by anything in its tree,
# so every configuration runs at both candidates.  With the orthonormal scale the synthetic inputs
# give codes 1 and 2 almost everywhere, distances fall into a few bins and most of a selection is
# decided by the lowest-index tie rule: the tie quota paths of both selection levels at full size.
@pytest.mark.parametrize("scale", SCALES)
def test_step_config1_4k_budget64(gpu_device, scale):
    w = synth.WORKLOADS["c1_4k_b64"]
    seq = synth.make_workload(w)[0]
    _, q_code, est, sel, o, o_f, sel_f = _run_step(gpu_device, seq, w.budget, w.page_size, 1,
                                                   scale=scale)
    ora = _check_step(seq, w.budget, q_code, est, sel, o, o_f, sel_f, scale=scale)
    if scale == 1.0:
        # the planted needles are among the selected tokens (with the orthonormal scale the codes
        # are too coarse to tell them apart from their many ties)
        for h in range(32):
            assert set(seq.needles[h].tolist()) <= set(int(x) for x in ora["sets"][h])


def test_step_config1_page_size_1_unfused(gpu_device):
    w = synth.WORKLOADS["c1_4k_b64"]
    seq = synth.make_workload(w)[0]
    _, q_code, est, sel, o, o_f, sel_f = _run_step(gpu_device, seq, w.budget, 1, 9, fused_append=False)
    _check_step(seq, w.budget, q_code, est, sel, o, o_f, sel_f)


@pytest.mark.timeout(600)
@pytest.mark.parametrize("scale", SCALES)
def test_step_config2_32k_budget128(gpu_device, scale):
    w = synth.WORKLOADS["c2_32k_b128"]
    T.heartbeat("config 2: generating inputs")
    seq = synth.make_workload(w)[0]
    T.heartbeat("config 2: running the HIP path")
    _, q_code, est, sel, o, o_f, sel_f = _run_step(gpu_device, seq, w.budget, w.page_size, 2,
                                                   scale=scale)
    _check_step(seq, w.budget, q_code, est, sel, o, o_f, sel_f, scale=scale)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("scale", SCALES)
def test_step_config4_128k_budget256(gpu_device, scale):
    w = synth.WORKLOADS["c4_128k_b256"]
    T.heartbeat("config 4: generating inputs")
    seq = synth.make_workload(w)[0]
    T.heartbeat("config 4: running the HIP path")
    _, q_code, est, sel, o, o_f, sel_f = _run_step(gpu_device, seq, w.budget, w.page_size, 4,
                                                   scale=scale)
    _check_step(seq, w.budget, q_code, est, sel, o, o_f, sel_f, scale=scale)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("kv_len,budget,page_size", [
    (20000, 200, 16),   # 512-token chunks, 8000 candidate slots
    (40000, 200, 16),   # 512-token chunks, 15800 slots
    (50000, 256, 16),   # 1024-token chunks
    (30000, 250, 3),    # page size other than 16
    (70000, 256, 1),    # 2048-token chunks, page size 1
    (60001, 9, 16),     # smallest candidate rows (8 slots), 118 chunks
])
def test_step_chunk_variants_match_three_launch_path(gpu_device, kv_len, budget, page_size):
    """Every chunk size / slot count of the two-launch step against the three stand-alone operators
    (which the other tests pin to the oracle): identical index sets, outputs within tolerance."""
    assert _lib.load().adamas_step_fused_supported(1, 32, kv_len, budget) == 1
    T.heartbeat(f"step variants: L={kv_len} budget={budget} page={page_size}")
    seq = synth.make_sequence(kv_len, 8, torch.Generator().manual_seed(kv_len + budget))
    _, q_code, est, sel, o, o_f, sel_f = _run_step(gpu_device, seq, budget, page_size, 5)
    a = np.sort(T.np16(sel).astype(np.int64), axis=1)
    b = np.sort(T.np16(sel_f).astype(np.int64), axis=1)
    assert np.array_equal(a, b)
    assert (a >= 0).all() and (np.diff(a, axis=1) > 0).all()
    assert np.abs(T.np16(o).astype(np.float64) - T.np16(o_f).astype(np.float64)).max() <= ATTN_TOL


def _random_step_cases():
    rng = np.random.default_rng(2024)
    cases = []
    for i in range(28):
        L = int(np.exp(rng.uniform(np.log(130), np.log(45000))))
        budget = int(rng.choice([2, 3, 8, 9, 16, 33, 64, 100, 128, 129, 200, 255, 256]))
        budget = min(budget, L - 1)
        page = int(rng.choice([1, 3, 16, 16, 32]))
        cases.append((L, budget, page, i % 3))
    return cases


@pytest.mark.timeout(900)
@pytest.mark.parametrize("kv_len,budget,page_size,kind", _random_step_cases())
def test_step_random_shapes_match_three_launch_path(gpu_device, kv_len, budget, page_size, kind):
    """Seeded random lengths, budgets and page sizes; kind 1 draws the keys from six distinct rows
    (most distances are tied, the selection is decided by the lowest-index rule), kind 2 from
    sixty.  The step against the three stand-alone operators: identical index sets."""
    g = torch.Generator().manual_seed(kv_len * 7 + budget)
    seq = synth.make_sequence(kv_len, 4, g)
    if kind:
        n_rows = 6 if kind == 1 else 60
        pick = torch.randint(0, n_rows, (kv_len,), generator=g)
        seq = synth.SequenceData(q=seq.q, k=seq.k[:n_rows][pick].contiguous(),
                                 v=seq.v, needles=seq.needles)
    _, q_code, est, sel, o, o_f, sel_f = _run_step(gpu_device, seq, budget, page_size, kv_len % 11)
    a = np.sort(T.np16(sel).astype(np.int64), axis=1)
    b = np.sort(T.np16(sel_f).astype(np.int64), axis=1)
    assert np.array_equal(a, b)
    assert (a >= 0).all() and (np.diff(a, axis=1) > 0).all()
    if kind == 1:   # with at most six distinct distances the lowest-index rule is easy to restate
        d = T.np16(est).astype(np.int64)
        d = d.reshape(-1, d.shape[-1])
        for h in (0, 13, 31):
            want = np.sort(np.argsort(d[h], kind="stable")[:budget - 1])
            assert np.array_equal(a[h], want), h
    assert np.abs(T.np16(o).astype(np.float64) - T.np16(o_f).astype(np.float64)).max() <= ATTN_TOL


def _device_sequence(gpu_device, kv_len, seed, kind="random"):
    """q [32, 128], k, v [L, 32, 128] fp16 drawn on the device (long sequences without the host
    generator's seconds per test); same distribution as synth.make_sequence, no needles.
    kind "equal": every key equals key 0 (all distances tied: the selection is the first tokens,
    which the stable argsort in _assert_step_equals_operators restates);
    kind "clustered": the last 700 tokens are noisy copies of the query (one chunk holds most of the
    selection, with distinct distances); kind "runs": keys repeat in runs of 300 tokens drawn from 5
    rows (long runs of equal distances across chunk boundaries)."""
    g = torch.Generator(device=gpu_device).manual_seed(seed)
    gain = torch.ones(32, 128, device=gpu_device)
    for h in range(32):
        gain[h, torch.randperm(128, generator=g, device=gpu_device)[:4]] = 8.0
    q = (torch.randn(32, 128, generator=g, device=gpu_device) * gain).half()
    k = (torch.randn(kv_len, 32, 128, generator=g, device=gpu_device) * gain).half()
    v = torch.randn(kv_len, 32, 128, generator=g, device=gpu_device).half()
    if kind == "equal":
        k = k[:1].expand(kv_len, 32, 128).contiguous()
    elif kind == "clustered":
        m = min(700, kv_len - 1)
        noise = torch.randn(m, 32, 128, generator=g, device=gpu_device) * gain
        mix = torch.rand(m, 1, 1, generator=g, device=gpu_device) * 0.6 + 0.2
        k[kv_len - 1 - m:kv_len - 1] = (q.float()[None] * mix + noise * (1 - mix)).half()
    elif kind == "runs":
        pick = (torch.arange(kv_len, device=gpu_device) // 300) % 5
        k = k[:5][pick].contiguous()
    return synth.SequenceData(q=q, k=k, v=v, needles=None)


def _assert_step_equals_operators(gpu_device, seq, budget, page_size, shuffle_seed=5, scale=1.0):
    """The two-launch step against the three stand-alone operators (pinned to the oracle by the
    tests above): identical index sets, every entry a distinct past token, outputs within tolerance;
    and the operators' own selection against a stable argsort of the distances they selected from."""
    _, q_code, est, sel, o, o_f, sel_f = _run_step(gpu_device, seq, budget, page_size, shuffle_seed,
                                                   scale=scale)
    a = np.sort(T.np16(sel).astype(np.int64), axis=1)
    b = np.sort(T.np16(sel_f).astype(np.int64), axis=1)
    d = T.np16(est).astype(np.int64)
    d = d.reshape(-1, d.shape[-1])
    for h in (0, 7, 31):
        want = np.sort(np.argsort(d[h], kind="stable")[:budget - 1])
        assert np.array_equal(a[h], want), h
    assert np.array_equal(a, b)
    assert (a >= 0).all() and (np.diff(a, axis=1) > 0).all()
    assert np.abs(T.np16(o).astype(np.float64) - T.np16(o_f).astype(np.float64)).max() <= ATTN_TOL


@pytest.mark.timeout(900)
@pytest.mark.parametrize("kv_len", [
    16384, 16385, 16400, 24000,          # narrow workgroups: 32 balanced chunks
    32768, 32769, 32770, 32784, 32785,   # 64 chunks of 512 tokens, then of 512 and 528
    33024, 33025, 36864, 40960, 40961,   # ... 576, 640 and 656 tokens
    49152, 49153, 65536, 65537, 65553,   # two whole passes, three partial ones
    98304, 98321, 131072,                # three and four passes
    513, 1025, 8191, 8192, 8193, 16383,  # chunks of 512 tokens that do not fill the chip
])
def test_step_balanced_chunks_at_length_boundaries(gpu_device, kv_len):
    """Lengths on both sides of every boundary of the chunk plan (the number of passes a workgroup
    makes, a partial last pass, the heads per workgroup, the last unit of a chunk)."""
    assert _lib.load().adamas_step_fused_supported(1, 32, kv_len, 128) == 1
    T.heartbeat(f"balanced chunks: L={kv_len}")
    seq = _device_sequence(gpu_device, kv_len, kv_len)
    _assert_step_equals_operators(gpu_device, seq, 128, 16)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("scale", SCALES)
@pytest.mark.parametrize("kind", ["equal", "clustered", "runs"])
@pytest.mark.parametrize("kv_len,budget,page_size", [
    (33000, 128, 16), (32768, 128, 16), (70000, 256, 16), (5000, 64, 3), (131072, 256, 16),
    (20000, 17, 16), (40000, 128, 1),
])
def test_step_truncated_chunk_lists_are_rescored(gpu_device, kv_len, budget, page_size, kind, scale):
    """Inputs whose selection needs more tokens of one chunk than the chunk's list holds: every
    distance tied, most of the selection inside one chunk, long runs of equal distances.  The second
    launch scores such chunks again, and the result stays exact."""
    T.heartbeat(f"truncated lists: L={kv_len} budget={budget} {kind}")
    seq = _device_sequence(gpu_device, kv_len, kv_len + budget, kind)
    _assert_step_equals_operators(gpu_device, seq, budget, page_size, scale=scale)


@pytest.mark.timeout(900)
@pytest.mark.parametrize("kv_len,budget,page_size", [
    (5000, 300, 16), (20000, 512, 16), (32768, 1024, 16), (9000, 4096, 3), (40000, 2048, 1),
    (2000, 257, 16), (131072, 700, 16), (16384, 2048, 16), (8192, 4096, 16),
])
def test_step_large_budgets(gpu_device, kv_len, budget, page_size):
    """Budgets above 256 (the reference's kernel benchmarks go up to 4096): the step runs as
    estimator-with-histograms, selection from the histograms, attention.  Against the three
    stand-alone operators, and against the oracle where it finishes quickly."""
    assert _lib.load().adamas_step_fused_supported(1, 32, kv_len, budget) == 0
    T.heartbeat(f"large budget: L={kv_len} budget={budget} page={page_size}")
    seq = synth.make_sequence(kv_len, 8, torch.Generator().manual_seed(kv_len + budget))
    _, q_code, est, sel, o, o_f, sel_f = _run_step(gpu_device, seq, budget, page_size, 6)
    a = np.sort(T.np16(sel).astype(np.int64), axis=1)
    b = np.sort(T.np16(sel_f).astype(np.int64), axis=1)
    assert np.array_equal(a, b)
    assert (a >= 0).all() and (np.diff(a, axis=1) > 0).all()
    assert np.abs(T.np16(o).astype(np.float64) - T.np16(o_f).astype(np.float64)).max() <= ATTN_TOL
    if kv_len <= 20000:
        _check_step(seq, budget, q_code, est, sel, o, o_f, sel_f)


def test_step_large_budget_ragged_batch(gpu_device):
    lens = [3000, 700, 5000, 301, 4097]
    budget = 600
    g = torch.Generator().manual_seed(77)
    seqs = [synth.make_sequence(L, 4, g) for L in lens]
    B = len(lens)
    ctrl = T.make_controller(gpu_device, 5008, budget, 16, batch_size=B, shuffle_seed=4)
    for b, s in enumerate(seqs):
        T.fill_sequence(ctrl, s.k[:-1].to(gpu_device), s.v[:-1].to(gpu_device), seq_idx=b)
    q = torch.stack([s.q for s in seqs]).to(gpu_device)
    kn = torch.stack([s.k[-1] for s in seqs]).to(gpu_device)
    vn = torch.stack([s.v[-1] for s in seqs]).to(gpu_device)
    q_code = T.decode_append(ctrl, q, kn, vn)
    o_f, sel_f = U.decode_step(q, q_code, ctrl, 0, return_indices=True)
    for b, s in enumerate(seqs):
        ora = T.oracle_step(s.q, s.k, s.v, budget)
        ok, h = T.sets_equal(T.np16(sel_f[b * 32:(b + 1) * 32]), ora["sets"], lens[b])
        assert ok, (b, h)
        assert np.abs(T.np16(o_f)[b].astype(np.float64) - ora["out"]).max() <= ATTN_TOL


@pytest.mark.parametrize("scale", SCALES)
def test_step_short_sequences_in_a_long_batch(gpu_device, scale):
    """A batch whose longest sequence fixes 64 chunks and lists of 32 entries, next to sequences
    shorter than the budget, shorter than a list, and between the two: a short sequence has all its
    tokens in chunk 0, whose list then runs out although the whole sequence is selected."""
    lens = [32000, 100, 40, 600, 33, 129, 8000, 2]
    budget = 128
    assert _lib.step_plan(len(lens), 32, max(lens), budget)["kc"] == 32
    g = torch.Generator().manual_seed(21)
    seqs = [synth.make_sequence(L, 4, g) for L in lens]
    B = len(lens)
    ctrl = T.make_controller(gpu_device, max(lens), budget, 16, batch_size=B, shuffle_seed=6, scale=scale)
    for b, s in enumerate(seqs):
        if lens[b] > 1:
            T.fill_sequence(ctrl, s.k[:-1].to(gpu_device), s.v[:-1].to(gpu_device), seq_idx=b)
    q = torch.stack([s.q for s in seqs]).to(gpu_device)
    kn = torch.stack([s.k[-1] for s in seqs]).to(gpu_device)
    vn = torch.stack([s.v[-1] for s in seqs]).to(gpu_device)
    q_code = T.decode_append(ctrl, q, kn, vn)
    est = U.decode_estimate(q_code, ctrl, 0)
    U.decode_topk(est, ctrl)
    sel = ctrl.topk_dindices_buffer.clone()
    o = U.decode_sparse_attn(q, ctrl, 0, sel)
    o_f, sel_f = U.decode_step(q, q_code, ctrl, 0, return_indices=True)
    a = np.sort(T.np16(sel).astype(np.int64), axis=1)
    b_ = np.sort(T.np16(sel_f).astype(np.int64), axis=1)
    assert np.array_equal(a, b_)
    assert np.abs(T.np16(o).astype(np.float64) - T.np16(o_f).astype(np.float64)).max() <= ATTN_TOL
    for b, s in enumerate(seqs):
        if lens[b] > 700:
            continue
        ora = T.oracle_step(s.q, s.k, s.v, budget, scale=scale)
        ok, h = T.sets_equal(T.np16(sel_f[b * 32:(b + 1) * 32]), ora["sets"], lens[b])
        assert ok, (b, h)
        assert np.abs(T.np16(o_f)[b].astype(np.float64) - ora["out"]).max() <= ATTN_TOL, b


def test_step_wide_distance_spread(gpu_device):
    """Two past tokens equal the query (distance 0) while every other token has saturated codes
    (distances around 190): the k-th nearest lies far above the minimum of its chunk, and the
    chunk histograms are empty between the two."""
    L, budget = 3000, 64
    g = torch.Generator().manual_seed(77)
    q = (torch.randn(32, 128, generator=g) * 100).half()
    k = (torch.randn(L, 32, 128, generator=g) * 100).half()
    v = torch.randn(L, 32, 128, generator=g).half()
    k[5] = q
    k[1777] = q
    seq = synth.SequenceData(q=q, k=k, v=v, needles=None)
    _, q_code, est, sel, o, o_f, sel_f = _run_step(gpu_device, seq, budget, 16, 6)
    ora = T.oracle_step(q, k, v, budget)
    d = ora["dist"]
    assert d.min() == 0 and np.sort(d, axis=1)[:, budget - 2].min() > 126
    ok, h = T.sets_equal(T.np16(sel_f), ora["sets"], L)
    assert ok, f"fused index set differs for head {h}"
    ok, h = T.sets_equal(T.np16(sel), ora["sets"], L)
    assert ok, f"index set differs for head {h}"
    # logits are huge here (|q.k| ~ 1e6 * scale): the softmax is one-hot, compare loosely
    assert np.abs(T.np16(o_f)[0].astype(np.float64) - ora["out"]).max() <= 2e-2


@pytest.mark.parametrize("scale", SCALES)
def test_step_ragged_batch(gpu_device, scale):
    """Batched ragged decode (no reference implementation: the oracle is the single-sequence oracle
    applied per sequence).  Lengths are scaled down so the oracle finishes in seconds; one sequence
    is shorter than the budget and must fall back to attending everything."""
    lens = [900, 2500, 77, 1601, 3000, 1024]
    budget = 128
    g = torch.Generator().manual_seed(3)
    seqs = [synth.make_sequence(L, 8, g) for L in lens]
    B = len(lens)
    ctrl = T.make_controller(gpu_device, 3072, budget, 16, batch_size=B, shuffle_seed=3, scale=scale)
    for b, s in enumerate(seqs):
        T.fill_sequence(ctrl, s.k[:-1].to(gpu_device), s.v[:-1].to(gpu_device), seq_idx=b)
    q = torch.stack([s.q for s in seqs]).to(gpu_device)
    kn = torch.stack([s.k[-1] for s in seqs]).to(gpu_device)
    vn = torch.stack([s.v[-1] for s in seqs]).to(gpu_device)
    q_code = T.decode_append(ctrl, q, kn, vn)
    est = U.decode_estimate(q_code, ctrl, 0)
    U.decode_topk(est, ctrl)
    sel = ctrl.topk_dindices_buffer.clone()
    o = U.decode_sparse_attn(q, ctrl, 0, sel)
    o_f, sel_f = U.decode_step(q, q_code, ctrl, 0, return_indices=True)
    for b, s in enumerate(seqs):
        L = lens[b]
        ora = T.oracle_step(s.q, s.k, s.v, budget, scale=scale)
        assert np.array_equal(T.words_u16(q_code)[b], ora["q_words"])
        assert np.array_equal(T.np16(est[b, :, :L - 1]).astype(np.int32), ora["dist"])
        for which in (sel, sel_f):
            ok, h = T.sets_equal(T.np16(which[b * 32:(b + 1) * 32]), ora["sets"], L)
            assert ok, (b, h)
        for out in (o, o_f):
            assert np.abs(T.np16(out)[b].astype(np.float64) - ora["out"]).max() <= ATTN_TOL


@pytest.mark.parametrize("page_size", [16, 5])
def test_step_many_work_items(gpu_device, page_size):
    """A batch with more than a thousand (sequence, head group, chunk) items: the first launch runs
    with workgroups that walk over several items and overlap them.  Checked against the three
    stand-alone operators for every sequence and against the oracle for some, with sequences that
    end inside a chunk, fit the budget, or hold a single past token."""
    lens = [6000, 5121, 4097, 3000, 513, 512, 100, 2, 5990, 2049, 777, 5633,
            4500, 1025, 6001, 3333, 2, 130, 4096, 5000, 600, 5555, 2500, 6000]
    budget = 128
    g = torch.Generator().manual_seed(31)
    seqs = [synth.make_sequence(L, 4, g) for L in lens]
    B = len(lens)
    ctrl = T.make_controller(gpu_device, 6016, budget, page_size, batch_size=B, shuffle_seed=9)
    for b, s in enumerate(seqs):
        T.fill_sequence(ctrl, s.k[:-1].to(gpu_device), s.v[:-1].to(gpu_device), seq_idx=b)
    q = torch.stack([s.q for s in seqs]).to(gpu_device)
    kn = torch.stack([s.k[-1] for s in seqs]).to(gpu_device)
    vn = torch.stack([s.v[-1] for s in seqs]).to(gpu_device)
    q_code = T.decode_append(ctrl, q, kn, vn)
    est = U.decode_estimate(q_code, ctrl, 0)
    U.decode_topk(est, ctrl)
    sel = ctrl.topk_dindices_buffer.clone()
    o = U.decode_sparse_attn(q, ctrl, 0, sel)
    for _ in range(2):   # twice: the second call finds the workspace as the first left it
        o_f, sel_f = U.decode_step(q, q_code, ctrl, 0, return_indices=True)
        for b in range(B):
            a_ = np.sort(T.np16(sel[b * 32:(b + 1) * 32]), axis=1)
            b_ = np.sort(T.np16(sel_f[b * 32:(b + 1) * 32]), axis=1)
            assert np.array_equal(a_, b_), b
        assert (o.float() - o_f.float()).abs().max().item() <= ATTN_TOL
    for b in (0, 4, 6, 7, 14):
        L, s = lens[b], seqs[b]
        ora = T.oracle_step(s.q, s.k, s.v, budget)
        ok, h = T.sets_equal(T.np16(sel_f[b * 32:(b + 1) * 32]), ora["sets"], L)
        assert ok, (b, h)
        assert np.abs(T.np16(o_f)[b].astype(np.float64) - ora["out"]).max() <= ATTN_TOL


def test_step_indptr_tables_match_fixed_stride(gpu_device):
    """The step takes page tables either with a fixed stride per sequence (what the controller keeps)
    or as concatenated lists with an indptr array (the reference's layout): same results."""
    lens = [900, 2500, 1601]
    budget = 96
    g = torch.Generator().manual_seed(31)
    seqs = [synth.make_sequence(L, 4, g) for L in lens]
    B = len(lens)
    ctrl = T.make_controller(gpu_device, 2560, budget, 16, batch_size=B, shuffle_seed=8)
    for b, s in enumerate(seqs):
        T.fill_sequence(ctrl, s.k[:-1].to(gpu_device), s.v[:-1].to(gpu_device), seq_idx=b)
    q = torch.stack([s.q for s in seqs]).to(gpu_device)
    kn = torch.stack([s.k[-1] for s in seqs]).to(gpu_device)
    vn = torch.stack([s.v[-1] for s in seqs]).to(gpu_device)
    q_code = T.decode_append(ctrl, q, kn, vn)
    o_ref, sel_ref = U.decode_step(q, q_code, ctrl, 0, return_indices=True)
    sel_ref = sel_ref.clone()

    pages = [p for b in range(B) for p in ctrl.seqs.pages[b]]
    table = torch.tensor(pages, dtype=torch.int32, device=gpu_device)
    indptr = torch.tensor(np.cumsum([0] + [len(ctrl.seqs.pages[b]) for b in range(B)]),
                          dtype=torch.int32, device=gpu_device)
    bud = ctrl.inference_page_budget
    o = torch.empty_like(q)
    sel = torch.full_like(sel_ref, -7)
    ws = ctrl.workspace(bud)
    rc = _lib.load().adamas_decode_step(
        q.data_ptr(), q_code.data_ptr(), ctrl.pool.kv[0].data_ptr(), ctrl.pool.codes[0].data_ptr(),
        table.data_ptr(), indptr.data_ptr(), ctrl.seqs.seq_lens_dev.data_ptr(), bud, o.data_ptr(),
        sel.data_ptr(), ws.data_ptr(), ws.numel(), B, 32, 32, 128, 16, 1.0 / math.sqrt(128),
        ctrl.max_len_now, 0, _lib.current_stream())
    assert rc == 0
    assert torch.equal(sel, sel_ref)
    assert torch.equal(o, o_ref)


def test_empty_and_single_token_sequences_through_the_c_abi(gpu_device):
    """A batch whose sequences hold 0, 1 and 700 tokens (the Python controller refuses to decode
    such a batch, the C ABI must still behave): zeros and an empty selection for the empty sequence,
    the value row of its only token for the second, the oracle's answer for the third."""
    budget, L = 64, 700
    seq = synth.make_sequence(L, 4, torch.Generator().manual_seed(44))
    ctrl = T.make_controller(gpu_device, 1024, budget, 16, batch_size=3, shuffle_seed=4)
    T.fill_sequence(ctrl, seq.k[:L - 1].to(gpu_device), seq.v[:L - 1].to(gpu_device), seq_idx=2)
    g = torch.Generator().manual_seed(45)
    q = torch.stack([torch.randn(32, 128, generator=g).half(), torch.randn(32, 128, generator=g).half(),
                     seq.q]).to(gpu_device)
    kn = torch.stack([torch.randn(32, 128, generator=g).half(), torch.randn(32, 128, generator=g).half(),
                      seq.k[-1]]).to(gpu_device)
    vn = torch.stack([torch.randn(32, 128, generator=g).half(), torch.randn(32, 128, generator=g).half(),
                      seq.v[-1]]).to(gpu_device)
    ctrl.prepare_hadamard(1)                       # lengths 1, 1, 700
    q_code = U.append_kvh(kn, vn, None, ctrl, 0, q=q)
    lens = torch.tensor([0, 1, L], dtype=torch.int32, device=gpu_device)   # pretend sequence 0 is empty
    lib = _lib.load()
    ws = ctrl.workspace(budget)
    ora = T.oracle_step(seq.q, seq.k, seq.v, budget)

    def check(o, sel=None):
        o = T.np16(o).astype(np.float64)
        assert np.all(o[0] == 0)
        assert np.abs(o[1] - T.np16(vn[1]).astype(np.float64)).max() <= 1e-3
        assert np.abs(o[2] - ora["out"]).max() <= ATTN_TOL
        if sel is not None:
            s3 = T.np16(sel).reshape(3, 32, budget - 1)
            assert (s3[0] == -1).all() and (s3[1] == -1).all()
            ok, h = T.sets_equal(s3[2], ora["sets"], L)
            assert ok, h

    tbl, indptr = ctrl.seqs.table_dev.data_ptr(), ctrl.seqs.indptr_dev.data_ptr()
    for stride in (ctrl.seqs.max_pages, 0):
        o = torch.full_like(q, 7.0)
        sel = torch.full((96, budget - 1), -5, dtype=torch.int32, device=gpu_device)
        rc = lib.adamas_decode_step(q.data_ptr(), q_code.data_ptr(), ctrl.pool.kv[0].data_ptr(),
                                    ctrl.pool.codes[0].data_ptr(), tbl, indptr, lens.data_ptr(), budget,
                                    o.data_ptr(), sel.data_ptr(), ws.data_ptr(), ws.numel(), 3, 32, 32,
                                    128, 16, 1.0 / math.sqrt(128), L, stride, _lib.current_stream())
        assert rc == 0
        check(o, sel)
    # dense attention over the same batch, then the sparse kernel with the selection just made
    o = torch.full_like(q, 7.0)
    rc = lib.adamas_sparse_decode(q.data_ptr(), ctrl.pool.kv[0].data_ptr(), tbl, indptr, lens.data_ptr(),
                                  None, 0, 0, o.data_ptr(), ws.data_ptr(), ws.numel(), 3, 32, 32, 128, 16,
                                  1.0 / math.sqrt(128), L, _lib.current_stream())
    assert rc == 0
    o = T.np16(o).astype(np.float64)
    assert np.all(o[0] == 0)
    assert np.abs(o[1] - T.np16(vn[1]).astype(np.float64)).max() <= 1e-3
    want = O.dense_attention(T.np16(seq.q), T.np16(seq.k), T.np16(seq.v))
    assert np.abs(o[2] - want).max() <= ATTN_TOL
    o = torch.full_like(q, 7.0)
    rc = lib.adamas_sparse_decode(q.data_ptr(), ctrl.pool.kv[0].data_ptr(), tbl, indptr, lens.data_ptr(),
                                  sel.data_ptr(), budget - 1, budget - 1, o.data_ptr(), ws.data_ptr(),
                                  ws.numel(), 3, 32, 32, 128, 16, 1.0 / math.sqrt(128), L,
                                  _lib.current_stream())
    assert rc == 0
    check(o)


@pytest.mark.parametrize("hq,hkv,page_size,budget", [
    (32, 8, 16, 96), (64, 16, 16, 96), (32, 32, 16, 96), (32, 4, 3, 96), (32, 16, 16, 96),
    (64, 8, 7, 96), (32, 8, 16, 400), (64, 16, 5, 1000),
    # head counts that are no multiple of 32 (40 heads: the 13B shape of the model family)
    (40, 40, 16, 96), (40, 8, 16, 96), (40, 10, 7, 400), (8, 8, 16, 64), (24, 8, 16, 96), (40, 40, 16, 1000)])
@pytest.mark.parametrize("fused_append", [True, False])
@pytest.mark.parametrize("scale", SCALES)
def test_grouped_query_attention_step(gpu_device, hq, hkv, page_size, budget, fused_append, scale):
    """Grouped-query attention (no counterpart in the reference): the oracle is the plain one on
    K and V with every key/value head repeated for the query heads of its group.  Budgets up to
    256 run as two launches, larger ones as three (histogram mode)."""
    L, g = 1500, hq // hkv
    gen = torch.Generator().manual_seed(hq * 100 + hkv + page_size)
    q = (torch.randn(hq, 128, generator=gen) * 2).half()
    k = (torch.randn(L, hkv, 128, generator=gen) * 2).half()
    v = torch.randn(L, hkv, 128, generator=gen).half()
    ctrl = T.make_controller(gpu_device, L, budget, page_size, shuffle_seed=5, num_heads=hq,
                             num_kv_heads=hkv, scale=scale)
    kd, vd, qd = k.to(gpu_device), v.to(gpu_device), q.to(gpu_device)
    T.fill_sequence(ctrl, kd[:L - 1], vd[:L - 1])
    ctrl.prepare_hadamard(1)
    ctrl.begin_forward(1)
    if fused_append:
        q_code = U.append_kvh(kd[L - 1:], vd[L - 1:], None, ctrl, 0, q=qd[None])
    else:
        h = U.hadamard_transform(torch.cat((qd, kd[L - 1])).contiguous(), scale=ctrl.hadamard_scale)     # [Hq + Hkv, D]
        if hq == hkv:
            h = h.view(2, hq, 128)    # the reference's shape for equal head counts
        q_code = U.append_kvh(kd[L - 1:], vd[L - 1:], h, ctrl, 0)
    k_back, v_back, codes_back = T.read_logical_cache(ctrl)
    assert np.array_equal(k_back.view(np.uint16), T.np16(k).view(np.uint16))
    assert np.array_equal(v_back.view(np.uint16), T.np16(v).view(np.uint16))
    assert np.array_equal(codes_back, O.codes_from_raw(T.np16(k), scale))

    k_full, v_full = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    ora = T.oracle_step(q, k_full, v_full, budget, scale=scale)
    assert np.array_equal(T.words_u16(q_code)[0], ora["q_words"])
    est = U.decode_estimate(q_code, ctrl, 0)
    assert np.array_equal(T.np16(est).astype(np.int32), ora["dist"])
    U.decode_topk(est, ctrl)
    ok, h_bad = T.sets_equal(T.np16(ctrl.topk_dindices_buffer), ora["sets"], L)
    assert ok, h_bad
    o3 = U.decode_sparse_attn(qd[None], ctrl, 0, ctrl.topk_dindices_buffer)
    o_f, sel_f = U.decode_step(qd[None], q_code, ctrl, 0, return_indices=True)
    ok, h_bad = T.sets_equal(T.np16(sel_f), ora["sets"], L)
    assert ok, h_bad
    for o in (o3, o_f):
        assert np.abs(T.np16(o)[0].astype(np.float64) - ora["out"]).max() <= ATTN_TOL
    od = U.decode_sparse_attn(qd[None], ctrl, 0, ctrl.kv_indices_without_last)
    want = O.dense_attention(T.np16(q), T.np16(k_full), T.np16(v_full))
    assert np.abs(T.np16(od)[0].astype(np.float64) - want).max() <= ATTN_TOL


def test_paging_identity_vs_shuffled(gpu_device):
    """Size-independent property: the physical placement of pages must not change any result."""
    seq = synth.make_sequence(5000, 8, torch.Generator().manual_seed(21))
    outs = []
    for shuffle in (None, 123):
        _, q_code, est, sel, o, o_f, sel_f = _run_step(gpu_device, seq, 128, 16, shuffle)
        outs.append((q_code.clone(), est.clone(), sel, o, o_f, sel_f))
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize("scale", SCALES)
def test_step_gives_the_same_bits_every_time(gpu_device, scale):
    """The two-launch step on changing queries, each repeated: outputs and selections must agree with
    themselves bit for bit (ranks come from prefix scans, nothing is decided by arrival order), also
    where chunks are scored again (the orthonormal scale gives long runs of equal distances)."""
    L, budget = 33000, 128
    seq = _device_sequence(gpu_device, L, 5)
    ctrl = T.make_controller(gpu_device, L, budget, 16, shuffle_seed=9, scale=scale)
    T.fill_sequence(ctrl, seq.k[:L - 1], seq.v[:L - 1])
    T.decode_append(ctrl, seq.q[None], seq.k[L - 1:], seq.v[L - 1:])
    g = torch.Generator(device=gpu_device).manual_seed(11)
    for it in range(100):
        q = (torch.randn(1, 32, 128, generator=g, device=gpu_device) * (1 + it % 4)).half()
        q_code = U.pack_2bit(U.hadamard_transform(q, scale=ctrl.hadamard_scale))
        a, sa = U.decode_step(q, q_code, ctrl, 0, return_indices=True)
        a, sa = a.clone(), sa.clone()
        b, sb = U.decode_step(q, q_code, ctrl, 0, return_indices=True)
        assert torch.equal(a, b) and torch.equal(sa, sb), it


def test_split_merge_inside_the_launch_gives_the_same_bits_every_time(gpu_device):
    """The attention over 1023 rows per head is cut into eight splits whose partial results are
    merged by the last workgroup to arrive, inside the launch (write-through stores, an arrival
    counter, cache-bypassing loads; csrc/split_merge.h).  A partial that is read before it has
    arrived shows up as different output bits: 300 launches on changing inputs, each repeated, must
    agree with themselves bit for bit, and the result must not depend on what the workspace held."""
    L, budget = 9000, 1024
    seq = _device_sequence(gpu_device, L, 99)
    ctrl = T.make_controller(gpu_device, L, budget, 16, shuffle_seed=5)
    T.fill_sequence(ctrl, seq.k[:L - 1], seq.v[:L - 1])
    q_code = T.decode_append(ctrl, seq.q[None], seq.k[L - 1:], seq.v[L - 1:])
    est = U.decode_estimate(q_code, ctrl, 0)
    U.decode_topk(est, ctrl)
    sel = ctrl.topk_dindices_buffer
    g = torch.Generator(device=gpu_device).manual_seed(7)
    for it in range(150):
        q = (torch.randn(1, 32, 128, generator=g, device=gpu_device) * (1 + it % 5)).half()
        a = U.decode_sparse_attn(q, ctrl, 0, sel).clone()
        b = U.decode_sparse_attn(q, ctrl, 0, sel)
        assert torch.equal(a, b), it
    # the large-budget step merges its slabs the same way
    for it in range(50):
        q = (torch.randn(1, 32, 128, generator=g, device=gpu_device) * (1 + it % 3)).half()
        a = U.decode_step(q, q_code, ctrl, 0).clone()
        b = U.decode_step(q, q_code, ctrl, 0)
        assert torch.equal(a, b), it
