"""GPU parity tests of the data formats beyond the reference's: bfloat16 (q, k, v, caches and
outputs) and the HND page layout of the KV cache.

The reference is fp16 only, so there is no reference behaviour to match here; the oracle is the same
CPU restatement fed with the bfloat16 values (exact in fp32) and rounding the transform's output to
bfloat16 where the fp16 path rounds to fp16.  Bars: codes, distances and index sets bit-exact; the
attention output within ATTN_TOL_ABS + |expected| * 2**-8 (a bfloat16 result carries 8 significant
bits, so the rounding of the output alone is up to |expected| * 2**-9).  HND pages must give exactly
what NHD pages give (the same kernels with other strides), so fp16 runs keep the 2e-3 bar.
"""
import numpy as np
import pytest
import torch

import adamas_amd.utils as U
from oracle import adamas_oracle as O
from tests import helpers as T

pytestmark = pytest.mark.gpu
ATTN_TOL_ABS = 2e-3
BF = torch.bfloat16
FP = torch.float16
NHD, HND = U.TensorLayout.NHD, U.TensorLayout.HND


def _close(got: torch.Tensor, want: np.ndarray) -> bool:
    g = T.np16(got).astype(np.float64)
    rel = 2.0 ** -8 if got.dtype == BF else 0.0
    return bool((np.abs(g - want) <= ATTN_TOL_ABS + np.abs(want) * rel).all())


@pytest.mark.parametrize("scale", [1.0, 128 ** -0.5])
@pytest.mark.parametrize("rows", [1, 3, 1000])
def test_hadamard_bf16_bit_exact(gpu_device, scale, rows):
    g = torch.Generator().manual_seed(rows)
    x = (torch.randn(rows, 32, 128, generator=g) * 3).to(BF)
    y = U.hadamard_transform(x.to(gpu_device), scale=scale)
    assert y.dtype == BF
    want = O.hadamard_bf16(T.np16(x), scale)
    assert np.array_equal(T.words_u16(y), T.bf16_words(want))
    xi = x.to(gpu_device).clone()
    U.hadamard_transform(xi, inplace=True, scale=scale)
    assert torch.equal(xi, y)


def test_pack_2bit_bf16(gpu_device):
    g = torch.Generator().manual_seed(0)
    codes = torch.randint(0, 4, (77, 32, 128), generator=g)
    got = U.pack_2bit(codes.to(BF).to(gpu_device), 0)
    assert np.array_equal(T.words_u16(got), O.pack_2bit(codes.numpy()))


def test_mixed_dtypes_are_rejected(gpu_device):
    ctrl = T.make_controller(gpu_device, 64, 16, 16, dtype=BF)
    k = torch.zeros(4, 32, 128, dtype=torch.float16, device=gpu_device)
    ctrl.prepare_hadamard(4)
    with pytest.raises(RuntimeError):
        U.append_kvh(k, k, None, ctrl, 0)
    with pytest.raises(RuntimeError):
        U.InferenceController(1, 32, 128, 16, 16, 64, torch.float32, gpu_device)


def _make(L, hq, hkv, seed, dtype=BF):
    gen = torch.Generator().manual_seed(seed)
    q = (torch.randn(hq, 128, generator=gen) * 2).to(dtype)
    k = (torch.randn(L, hkv, 128, generator=gen) * 2).to(dtype)
    v = torch.randn(L, hkv, 128, generator=gen).to(dtype)
    # a few tokens close to the query so that the selection matters for the output
    for t in range(5, L - 1, max(1, L // 9)):
        k[t] = (q.float().view(hkv, hq // hkv, 128)[:, 0] * 0.9 + k[t].float() * 0.1).to(dtype)
    return q, k, v


@pytest.mark.parametrize("L,hq,hkv,page_size,budget,fused_append,dtype,layout", [
    (203, 32, 32, 16, 64, True, BF, NHD),       # two launches
    (203, 32, 32, 7, 64, False, BF, NHD),       # caller-side transform, odd page size
    (1500, 32, 8, 16, 96, True, BF, NHD),       # grouped queries, two launches
    (1500, 64, 16, 5, 1000, False, BF, NHD),    # grouped queries, three launches (histograms)
    (9000, 32, 32, 16, 400, True, BF, NHD),     # three launches
    (40000, 32, 32, 16, 128, True, BF, NHD),    # two launches, long row
    (5000, 32, 32, 1, 5000, True, BF, NHD),     # budget >= length: everything is attended
    (203, 32, 32, 16, 64, True, FP, HND),
    (203, 32, 32, 7, 64, False, FP, HND),
    (1500, 32, 8, 16, 96, True, FP, HND),
    (1500, 64, 16, 5, 1000, False, BF, HND),
    (9000, 32, 32, 16, 400, True, FP, HND),
    (40000, 32, 4, 16, 128, True, BF, HND),
    (5000, 32, 32, 1, 5000, True, FP, HND),
    (3000, 32, 2, 3, 2000, True, FP, HND),      # 16 query heads per key/value head
])
@pytest.mark.parametrize("scale", [1.0, 128 ** -0.5])
def test_step_formats(gpu_device, L, hq, hkv, page_size, budget, fused_append, dtype, layout, scale):
    g = hq // hkv
    bf = dtype == BF
    q, k, v = _make(L, hq, hkv, L + hq + page_size, dtype)
    ctrl = T.make_controller(gpu_device, L, budget, page_size, shuffle_seed=3, num_heads=hq,
                             num_kv_heads=hkv, dtype=dtype, layout=layout, scale=scale)
    kd, vd, qd = k.to(gpu_device), v.to(gpu_device), q.to(gpu_device)
    T.fill_sequence(ctrl, kd[:L - 1], vd[:L - 1], fused=fused_append, chunk=4096)
    ctrl.prepare_hadamard(1)
    ctrl.begin_forward(1)
    if fused_append:
        q_code = U.append_kvh(kd[L - 1:], vd[L - 1:], None, ctrl, 0, q=qd[None])
    else:
        h = U.hadamard_transform(torch.cat((qd, kd[L - 1])).contiguous(), scale=ctrl.hadamard_scale)     # [Hq + Hkv, D]
        if hq == hkv:
            h = h.view(2, hq, 128)
        q_code = U.append_kvh(kd[L - 1:], vd[L - 1:], h, ctrl, 0)
    k_back, v_back, codes_back = T.read_logical_cache(ctrl)
    assert np.array_equal(k_back, T.np16(k)) and np.array_equal(v_back, T.np16(v))
    assert np.array_equal(codes_back, O.codes_from_raw(T.np16(k), scale, bf16=bf))

    k_full, v_full = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    want_dense = O.dense_attention(T.np16(q), T.np16(k_full), T.np16(v_full))
    od = U.decode_sparse_attn(qd[None], ctrl, 0, ctrl.kv_indices_without_last)
    assert od.dtype == dtype and _close(od[0], want_dense)
    if not ctrl.need_estimate():
        o_f = U.decode_step(qd[None], q_code, ctrl, 0)
        assert _close(o_f[0], want_dense)
        return

    ora = T.oracle_step(q, k_full, v_full, budget, scale=scale, bf16=bf)
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
    assert o_f.dtype == dtype
    assert _close(o3[0], ora["out"]) and _close(o_f[0], ora["out"])


@pytest.mark.parametrize("layout", [NHD, HND])
def test_step_bf16_ragged_batch(gpu_device, layout):
    lens = [1200, 37, 4000, 2]
    budget, page_size = 48, 16
    ctrl = T.make_controller(gpu_device, max(lens), budget, page_size, batch_size=len(lens),
                             shuffle_seed=8, dtype=BF, layout=layout)
    seqs = [_make(L, 32, 32, 100 + L) for L in lens]
    for i, (q, k, v) in enumerate(seqs):
        T.fill_sequence(ctrl, k[:-1].to(gpu_device), v[:-1].to(gpu_device), seq_idx=i)
    qd = torch.stack([s[0] for s in seqs]).to(gpu_device)
    kn = torch.stack([s[1][-1] for s in seqs]).to(gpu_device)
    vn = torch.stack([s[2][-1] for s in seqs]).to(gpu_device)
    q_code = T.decode_append(ctrl, qd, kn, vn)
    o, sel = U.decode_step(qd, q_code, ctrl, 0, return_indices=True)
    sel = T.np16(sel).reshape(len(lens), 32, -1)
    for i, (q, k, v) in enumerate(seqs):
        L = lens[i]
        if L <= budget:
            want = O.dense_attention(T.np16(q), T.np16(k), T.np16(v))
        else:
            ora = T.oracle_step(q, k, v, budget, bf16=True)
            ok, h_bad = T.sets_equal(sel[i], ora["sets"], L)
            assert ok, (i, h_bad)
            want = ora["out"]
        assert _close(o[i], want), i


@pytest.mark.parametrize("dtype,layout", [(FP, NHD), (BF, NHD), (FP, HND)])
@pytest.mark.parametrize("hq,hkv,page_size,kv_len", [
    (32, 8, 16, 1), (32, 8, 16, 17), (32, 8, 16, 2049), (32, 8, 5, 1000), (32, 8, 16, 20000),
    (32, 16, 16, 777), (32, 4, 16, 3001), (64, 8, 16, 513), (32, 4, 3, 130),
])
def test_dense_grouped_query_attention_on_matrix_cores(gpu_device, dtype, layout, hq, hkv, page_size,
                                                       kv_len):
    """Dense decode attention with 2, 4 or 8 query heads per key/value head: the matrix-core kernel
    against the oracle on repeated heads, and against the vector-ALU kernel it replaced (flag
    ADAMAS_F_NO_MFMA), on lengths that end inside a tile, inside a page and inside a split."""
    import math
    from adamas_amd import _lib
    g = torch.Generator().manual_seed(kv_len * 7 + hq + hkv)
    q = torch.randn(1, hq, 128, generator=g).to(dtype)
    k = (torch.randn(kv_len, hkv, 128, generator=g) * 1.5).to(dtype)
    v = torch.randn(kv_len, hkv, 128, generator=g).to(dtype)
    cap = (kv_len + page_size - 1) // page_size * page_size
    ctrl = T.make_controller(gpu_device, cap, 1 << 20, page_size, shuffle_seed=5, num_heads=hq,
                             num_kv_heads=hkv, dtype=dtype, layout=layout)
    T.fill_sequence(ctrl, k.to(gpu_device), v.to(gpu_device))
    ctrl.inference_page_budget = 1 << 20
    qd = q.to(gpu_device)
    o = U.decode_sparse_attn(qd, ctrl, 0, U.ALL_PAST_TOKENS)
    rep = hq // hkv
    want = O.dense_attention(T.np16(q)[0], np.repeat(T.np16(k), rep, axis=1),
                             np.repeat(T.np16(v), rep, axis=1))
    assert _close(o[0], want)
    assert torch.equal(o, U.decode_sparse_attn(qd, ctrl, 0, U.ALL_PAST_TOKENS))   # counters back at zero
    # the vector-ALU kernel through the C ABI
    lib = _lib.load()
    o2 = torch.empty_like(qd)
    ws = ctrl.workspace(1)
    rc = lib.adamas_sparse_decode_f(
        qd.data_ptr(), ctrl.pool.kv[0].data_ptr(), ctrl.seqs.table_dev.data_ptr(),
        ctrl.seqs.indptr_dev.data_ptr(), ctrl.seqs.seq_lens_dev.data_ptr(), None, 0, 0, o2.data_ptr(),
        ws.data_ptr(), ws.numel(), 1, hq, hkv, 128, page_size, 1.0 / math.sqrt(128), kv_len,
        ctrl.kv_flags | _lib.F_NO_MFMA, _lib.current_stream())
    assert rc == 0, _lib.error_string(rc)
    assert _close(o2[0], want)
    tol = 4e-3 if dtype == BF else 2e-3
    assert (o.float() - o2.float()).abs().max().item() <= tol + 2.0 ** -7 * float(np.abs(want).max()) * (dtype == BF)
