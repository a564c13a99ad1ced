"""The two benchmark configurations whose size the other parity tests scale down, at full size:

* batched ragged decode: 16 sequences with lengths uniform in [8192, 32768], one shared shuffled page
  pool, budget 128: the step's launches as the benchmark runs them (narrow estimator workgroups,
  64 chunks per sequence, several sequences per launch of the final selection) against the three
  stand-alone operators for every sequence, and against the oracle for the shortest and the longest;
* end-to-end decode on the Llama-2-7B shape (32 layers, hidden 4096, 32 heads, random weights): a
  32768-token prompt, the captured HIP graph against the eager loop, host and device lengths, and
  one sparse layer of that state against the oracle and against the unfused operators.

Plus the exported decode wrapper and the robustness of decode_topk's choice of selection kernel.
"""
import numpy as np
import pytest
import torch

import adamas_amd.utils as U
from adamas_amd import synth
from adamas_amd.decoder import DecoderConfig, LlamaShapedDecoder
from oracle import adamas_oracle as O

import helpers as T

pytestmark = pytest.mark.gpu

ATTN_TOL = 2e-3


def _device_sequence(L, gen, dev, n_needles=8, H=32, D=128):
    """One sequence of the benchmark's distribution drawn on the device (q, K with 4 outlier
    channels per head scaled by 8, V; needles planted like synth.make_sequence)."""
    gain = torch.ones(H, D, device=dev)
    for h in range(H):
        gain[h, torch.randperm(D, generator=gen, device=dev)[:4]] = 8.0
    q = torch.randn(H, D, generator=gen, device=dev) * gain
    k = torch.randn(L, H, D, generator=gen, device=dev) * gain
    v = torch.randn(L, H, D, generator=gen, device=dev)
    qhat = q / q.norm(dim=-1, keepdim=True) * D ** 0.5
    for h in range(H):
        pos = torch.randperm(L - 1, generator=gen, device=dev)[:n_needles]
        k[pos, h] = 0.9 * qhat[h] + 0.1 * torch.randn(n_needles, D, generator=gen, device=dev)
    return q.half(), k.half(), v.half()


@pytest.mark.timeout(900)
@pytest.mark.parametrize("scale", [1.0, 128 ** -0.5])
def test_ragged_batch_of_16_at_full_size(gpu_device, scale):
    w = synth.WORKLOADS["c3_ragged16_b128"]
    lens, budget, P = list(w.seq_lens), w.budget, w.page_size
    B = len(lens)
    assert B == 16 and min(lens) >= 8192 and max(lens) <= 32768
    cap = (max(lens) + P - 1) // P * P
    ctrl = T.make_controller(gpu_device, cap, budget, P, batch_size=B, shuffle_seed=w.seed,
                             scale=scale)
    gen = torch.Generator(device=gpu_device).manual_seed(w.seed)
    qs, kn, vn = [], [], []
    keep = {int(np.argmin(lens)), int(np.argmax(lens))}
    host = {}
    for b, L in enumerate(lens):
        T.heartbeat(f"ragged batch: sequence {b} of {L} tokens")
        q, k, v = _device_sequence(L, gen, gpu_device)
        T.fill_sequence(ctrl, k[:-1], v[:-1], seq_idx=b)
        qs.append(q)
        kn.append(k[-1])
        vn.append(v[-1])
        if b in keep:
            host[b] = (q.cpu(), k.cpu(), v.cpu())
        del k, v
    q = torch.stack(qs)
    q_code = T.decode_append(ctrl, q, torch.stack(kn), torch.stack(vn))
    assert ctrl.need_estimate()
    est = U.decode_estimate(q_code, ctrl, 0)
    U.decode_topk(est, ctrl)
    sel = ctrl.topk_dindices_buffer.clone()
    o = U.decode_sparse_attn(q, ctrl, 0, sel)
    o_f, sel_f = U.decode_step(q, q_code, ctrl, 0, return_indices=True)
    a = np.sort(T.np16(sel).astype(np.int64), axis=1)
    f = np.sort(T.np16(sel_f).astype(np.int64), axis=1)
    for b in range(B):
        rows = slice(b * 32, (b + 1) * 32)
        assert np.array_equal(a[rows], f[rows]), f"sequence {b}: step and operators select differently"
        assert (a[rows] >= 0).all() and (a[rows] < lens[b] - 1).all()
        assert (np.diff(a[rows], axis=1) > 0).all()
    assert np.abs(T.np16(o).astype(np.float64) - T.np16(o_f).astype(np.float64)).max() <= ATTN_TOL
    for b in sorted(keep):
        T.heartbeat(f"ragged batch: oracle for sequence {b}")
        qh, kh, vh = host[b]
        L = lens[b]
        ora = T.oracle_step(qh, kh, vh, budget, scale=scale)
        assert np.array_equal(T.words_u16(q_code)[b], ora["q_words"])
        assert np.array_equal(T.np16(est[b, :, :L - 1]).astype(np.int32), ora["dist"])
        ok, h = T.sets_equal(T.np16(sel_f[b * 32:(b + 1) * 32]), ora["sets"], L)
        assert ok, (b, h)
        assert np.abs(T.np16(o_f)[b].astype(np.float64) - ora["out"]).max() <= ATTN_TOL
        assert np.abs(T.np16(o)[b].astype(np.float64) - ora["out"]).max() <= ATTN_TOL


@pytest.mark.timeout(1200)
@pytest.mark.parametrize("scale", [128 ** -0.5, 1.0])
def test_llama2_7b_shape_32k_prompt_graph_eager_and_oracle(gpu_device, scale):
    cfg = DecoderConfig.llama2_7b()
    prompt, budget, steps = 32768, 128, 16
    T.heartbeat("7B shape: drawing weights")
    model = LlamaShapedDecoder(cfg, gpu_device, seed=11)
    ids = torch.randint(0, cfg.vocab, (prompt,), generator=torch.Generator().manual_seed(5)).to(gpu_device)
    outs = []
    for use_graph in (False, True):
        T.heartbeat(f"7B shape: prefill, graph={use_graph}")
        model.init_cache(page_size=16, max_seq_len=prompt + 64, token_budget=budget,
                         hadamard_scale=scale)
        first = model.prefill(ids).argmax(-1)
        T.heartbeat("7B shape: decoding")
        toks, _ = model.generate(first, steps, sparse=True, use_graph=use_graph)
        assert model.ctrl.seqs.lengths[0] == prompt + steps          # host-side length
        assert int(model.ctrl.seq_lens[0]) == prompt + steps         # device-side length
        outs.append(toks.numpy())
        if not use_graph:
            model.clear()
    assert np.array_equal(outs[0], outs[1]), "graph replay and eager loop generate different tokens"

    # one sparse layer of this state, one more token: the two launches that take the fused
    # projection against rotary+append followed by the step, and both against the oracle
    ctrl, layer = model.ctrl, 7
    g = torch.Generator(device=gpu_device).manual_seed(3)
    qkv = torch.randn(1, 3 * cfg.num_heads, 128, generator=g, device=gpu_device).half()
    ctrl.prepare_hadamard(1)
    ctrl.set_page_budget(budget)
    ctrl.begin_forward(1)
    assert ctrl.need_estimate() and U.layer_step_supported(ctrl)
    o_a, sel_a = U.decode_layer_step(qkv, model.rope_cos, model.rope_sin, ctrl, layer,
                                     return_indices=True)
    sel_a = sel_a.clone()
    q_rot, q_code = U.rope_append_decode(qkv, model.rope_cos, model.rope_sin, ctrl, layer)
    o_b, sel_b = U.decode_step(q_rot, q_code, ctrl, layer, return_indices=True)
    a = np.sort(T.np16(sel_a).astype(np.int64), axis=1)
    b = np.sort(T.np16(sel_b).astype(np.int64), axis=1)
    assert np.array_equal(a, b)
    assert np.abs(T.np16(o_a).astype(np.float64) - T.np16(o_b).astype(np.float64)).max() <= ATTN_TOL
    T.heartbeat("7B shape: oracle for one layer")
    k_log, v_log, words = T.read_logical_cache(ctrl, layer)
    L = k_log.shape[0]
    assert L == prompt + steps + 1
    ora = O.decode_step(T.np16(q_rot)[0], k_log, v_log, budget, scale=scale, k_words=words)
    assert np.array_equal(T.words_u16(q_code)[0], ora["q_words"])
    ok, h = T.sets_equal(T.np16(sel_a), ora["sets"], L)
    assert ok, h
    assert np.abs(T.np16(o_a)[0].astype(np.float64) - ora["out"]).max() <= ATTN_TOL
    # and the cached codes are the codes of the cached keys
    some = np.random.default_rng(0).choice(L, 512, replace=False)
    assert np.array_equal(words[some], O.codes_from_raw(k_log[some], scale))
    model.clear()


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("page_size,last_len", [(1, 1), (16, 16), (16, 5), (4, 1)])
def test_decode_wrapper_page_lists_against_oracle(gpu_device, layout, page_size, last_len):
    """BatchDecodeWithPagedKVCacheWrapper with the reference's call sequence (begin_forward,
    forward, end_forward): per-head lists of physical pages, attended in full, plus the first
    `last_len` slots of the last page."""
    H, D, n_pool, n_listed = 32, 128, 96, 9
    g = torch.Generator().manual_seed(page_size * 100 + last_len)
    shape = (n_pool, 2, page_size, H, D) if layout == "NHD" else (n_pool, 2, H, page_size, D)
    kv = torch.randn(shape, generator=g).half()
    q = torch.randn(1, H, D, generator=g).half()
    last_idx = 17
    idx = torch.stack([torch.randperm(n_pool - 1, generator=g)[:n_listed + 3] for _ in range(H)])
    idx = (idx + (idx >= last_idx)).to(torch.int32)            # any page but the last one
    wrapper = U.BatchDecodeWithPagedKVCacheWrapper(layout)
    o = torch.empty_like(q, device=gpu_device)
    with pytest.raises(RuntimeError):
        wrapper.forward(q.to(gpu_device), o, kv.to(gpu_device), idx.to(gpu_device),
                        torch.tensor([0, n_listed], dtype=torch.int32), last_len, last_idx)
    wrapper.begin_forward(torch.tensor([0, n_listed], dtype=torch.int32, device=gpu_device), H, H, D,
                          page_size, torch.float16)
    for _ in range(2):
        wrapper.forward(q.to(gpu_device), o, kv.to(gpu_device), idx.to(gpu_device),
                        torch.tensor([0, n_listed], dtype=torch.int32, device=gpu_device),
                        last_len, last_idx)
    with pytest.raises(RuntimeError):   # a host indptr that disagrees with the plan of begin_forward
        wrapper.forward(q.to(gpu_device), o, kv.to(gpu_device), idx.to(gpu_device),
                        torch.tensor([0, n_listed + 1], dtype=torch.int32), last_len, last_idx)
    wrapper.end_forward()
    kvn = kv.numpy() if layout == "NHD" else kv.permute(0, 1, 3, 2, 4).numpy()   # [pool, 2, P, H, D]
    k_flat = kvn[:, 0].reshape(n_pool * page_size, H, D)
    v_flat = kvn[:, 1].reshape(n_pool * page_size, H, D)
    sets = []
    for h in range(H):
        rows = [int(p) * page_size + s for p in idx[h, :n_listed].tolist() for s in range(page_size)]
        rows += [last_idx * page_size + s for s in range(last_len)]
        sets.append(np.array(rows))
    want = O.sparse_attention(q[0].numpy(), k_flat, v_flat, sets)
    assert np.abs(T.np16(o)[0].astype(np.float64) - want).max() <= ATTN_TOL
    with pytest.raises(KeyError):
        U.BatchDecodeWithPagedKVCacheWrapper("DHN")


def test_decode_topk_integer_selection_survives_views_and_copies(gpu_device):
    """decode_topk picks the single-pass integer selection for any view of the estimate the
    controller handed out, falls back to the arbitrary-key selection for a copy, and both give the
    same set (ties to the lowest index)."""
    L, budget = 5000, 64
    seq = synth.make_sequence(L, 4, torch.Generator().manual_seed(12))
    ctrl = T.make_controller(gpu_device, L, budget, 16)
    T.fill_sequence(ctrl, seq.k[:-1].to(gpu_device), seq.v[:-1].to(gpu_device))
    q_code = T.decode_append(ctrl, seq.q[None].to(gpu_device), seq.k[-1:].to(gpu_device),
                             seq.v[-1:].to(gpu_device))
    est = U.decode_estimate(q_code, ctrl, 0)
    want = np.sort(np.argsort(T.np16(est).astype(np.int64), axis=1, kind="stable")[:, :budget - 1], axis=1)
    for variant in (est, est[:, :], est.view(32, -1), est.clone(), est.contiguous()):
        ctrl.topk_dindices_buffer.fill_(-7)
        U.decode_topk(variant, ctrl)
        got = np.sort(T.np16(ctrl.topk_dindices_buffer).astype(np.int64), axis=1)
        assert np.array_equal(got, want)
    U.decode_topk(est.clone(), ctrl, integer_keys=True)     # the explicit promise
    assert np.array_equal(np.sort(T.np16(ctrl.topk_dindices_buffer).astype(np.int64), axis=1), want)


def test_decode_topk_takes_arbitrary_keys_for_tensors_it_did_not_fill(gpu_device):
    """Scores that are not the controller's own estimate (another tensor of the same shape made after
    the caller dropped the estimate, or the estimate edited in place) hold arbitrary fp16 values:
    decode_topk must select by value, not truncate them to integer distances."""
    L, budget = 5000, 64
    seq = synth.make_sequence(L, 4, torch.Generator().manual_seed(13))
    ctrl = T.make_controller(gpu_device, L, budget, 16)
    T.fill_sequence(ctrl, seq.k[:-1].to(gpu_device), seq.v[:-1].to(gpu_device))
    q_code = T.decode_append(ctrl, seq.q[None].to(gpu_device), seq.k[-1:].to(gpu_device),
                             seq.v[-1:].to(gpu_device))

    def picked():
        return np.sort(T.np16(ctrl.topk_dindices_buffer).astype(np.int64), axis=1)

    def stable_smallest(scores):
        return np.sort(np.argsort(scores.astype(np.float64), axis=1, kind="stable")[:, :budget - 1], axis=1)

    est = U.decode_estimate(q_code, ctrl, 0)
    shape = est.shape
    del est
    torch.cuda.synchronize()
    # fractional and negative scores of the same shape: the allocator may well reuse the block
    g = torch.Generator(device=gpu_device).manual_seed(1)
    other = (torch.rand(shape, generator=g, device=gpu_device) * 3 - 1).half()
    U.decode_topk(other, ctrl)
    assert np.array_equal(picked(), stable_smallest(T.np16(other)))
    # the estimate itself, scaled in place: values are no longer the integers the kernel wrote
    est = U.decode_estimate(q_code, ctrl, 0)
    est.mul_(0.001)
    U.decode_topk(est, ctrl)
    assert np.array_equal(picked(), stable_smallest(T.np16(est)))
    # and an untouched estimate still takes the integer selection (same result as by value)
    est = U.decode_estimate(q_code, ctrl, 0)
    U.decode_topk(est, ctrl)
    assert np.array_equal(picked(), stable_smallest(T.np16(est)))
