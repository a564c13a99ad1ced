"""The Llama-shaped decoder that drives the HIP path (adamas_amd/decoder.py): prefill and decode
against a plain torch fp32 model with dense attention on the same weights, the captured HIP graph
against the eager loop, and the sparse regime against the dense one where they must agree."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from adamas_amd.decoder import DecoderConfig, LlamaShapedDecoder

pytestmark = pytest.mark.gpu

CFG = DecoderConfig(num_layers=3, hidden=4096, num_heads=32, head_dim=128, intermediate=512,
                    vocab=512, dense_layers=1)
PROMPT = 300


def reference_logits(model, token_ids):
    """fp32, dense causal attention, no cache: logits of every position [N, vocab]."""
    c = model.cfg
    n = token_ids.shape[0]
    x = model.embed[token_ids].float()
    half = c.head_dim // 2
    cos, sin = model.rope_cos[:n, None, :], model.rope_sin[:n, None, :]

    def norm(t, w):
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + c.rms_eps) * w.float()

    def rope(t):
        t1, t2 = t[..., :half], t[..., half:]
        return torch.cat((t1 * cos - t2 * sin, t2 * cos + t1 * sin), -1)

    mask = torch.ones(n, n, dtype=torch.bool, device=x.device).tril()
    for lw in model.layers:
        qkv = (norm(x, lw["attn_norm"]) @ lw["wqkv"].float().T).view(n, -1, c.head_dim)
        hq, hkv = c.num_heads, c.kv_heads
        q, k, v = qkv[:, :hq], qkv[:, hq:hq + hkv], qkv[:, hq + hkv:]
        # the HIP path sees q, k, v rounded to fp16
        q, k, v = rope(q).half().float(), rope(k).half().float(), v.half().float()
        k, v = k.repeat_interleave(hq // hkv, dim=1), v.repeat_interleave(hq // hkv, dim=1)
        s = torch.einsum("ihd,jhd->hij", q, k) / math.sqrt(c.head_dim)
        p = torch.softmax(s.masked_fill(~mask, float("-inf")), -1)
        o = torch.einsum("hij,jhd->ihd", p, v).reshape(n, -1)
        x = x + o @ lw["wo"].float().T
        gu = norm(x, lw["mlp_norm"]) @ lw["w_gate_up"].float().T
        x = x + (F.silu(gu[:, :c.intermediate]) * gu[:, c.intermediate:]) @ lw["w_down"].float().T
    return norm(x, model.final_norm) @ model.lm_head.float().T


@pytest.fixture(scope="module")
def model(gpu_device):
    m = LlamaShapedDecoder(CFG, gpu_device, seed=5)
    return m


def _prompt(gpu_device):
    return torch.randint(0, CFG.vocab, (PROMPT,), generator=torch.Generator().manual_seed(1)).to(gpu_device)


def _close(a, b, tol=0.03):
    a, b = a.float(), b.float()
    return (a - b).abs().max().item() <= tol * max(1.0, b.abs().max().item())


def test_prefill_and_dense_decode_match_fp32_model(model, gpu_device):
    ids = _prompt(gpu_device)
    model.init_cache(page_size=16, max_seq_len=512, token_budget=64)
    logits = model.prefill(ids)
    ref = reference_logits(model, ids)
    assert _close(logits[0], ref[-1])
    # four eager dense steps, teacher-forced with the reference's greedy tokens
    seq = ids
    for _ in range(4):
        nxt = reference_logits(model, seq)[-1].argmax().view(1)
        got = model.decode_step_eager(nxt, sparse=False)
        seq = torch.cat((seq, nxt))
        assert _close(got[0], reference_logits(model, seq)[-1])
    model.clear()


@pytest.mark.parametrize("sparse", [False, True])
def test_graph_replay_equals_eager_loop(model, gpu_device, sparse):
    ids = _prompt(gpu_device)
    outs = []
    for use_graph in (False, True):
        model.init_cache(page_size=16, max_seq_len=512, token_budget=64)
        first = model.prefill(ids).argmax(-1)
        toks, _ = model.generate(first, 12, sparse=sparse, use_graph=use_graph)
        assert model.ctrl.seqs.lengths[0] == PROMPT + 12
        assert int(model.ctrl.seq_lens[0]) == PROMPT + 12
        outs.append(toks.numpy())
        model.clear()
    assert np.array_equal(outs[0], outs[1])


def test_sparse_regime_with_budget_above_length_is_dense(model, gpu_device):
    ids = _prompt(gpu_device)
    res = []
    for sparse, budget in ((False, 64), (True, 480)):
        model.init_cache(page_size=16, max_seq_len=512, token_budget=budget)
        first = model.prefill(ids).argmax(-1)
        res.append(model.decode_step_eager(first, sparse=sparse)[0].clone())
        model.clear()
    assert _close(res[1], res[0], tol=0.01)


def test_sparse_selection_keeps_output_close_when_budget_is_generous(model, gpu_device):
    """Budget 256 of 300 tokens: the sparse layers drop only the 44 most distant tokens per head."""
    ids = _prompt(gpu_device)
    res = []
    for sparse in (False, True):
        model.init_cache(page_size=16, max_seq_len=512, token_budget=256)
        first = model.prefill(ids).argmax(-1)
        res.append(model.decode_step_eager(first, sparse=sparse)[0].clone())
        assert model.ctrl.need_estimate()
        model.clear()
    assert _close(res[1], res[0], tol=0.25)


def test_stage_ranges_do_not_change_results(model, gpu_device):
    """Profiler ranges around the stages (the reference's NVTX names) are host calls only: prefill
    logits and the eager sparse decode give the same bits with them on, and the graph loop still
    captures and replays."""
    from adamas_amd import decoder as D
    ids = _prompt(gpu_device)
    res = []
    for on in (False, True):
        D.set_stage_ranges(on)
        try:
            model.init_cache(page_size=16, max_seq_len=512, token_budget=64)
            logits = model.prefill(ids)
            first = logits.argmax(-1)
            step = model.decode_step_eager(first, sparse=True).clone()
            toks, _ = model.generate(step.argmax(-1), 4, sparse=True, use_graph=True)
            res.append((logits.clone(), step, toks.numpy().copy()))
            model.clear()
        finally:
            D.set_stage_ranges(False)
    assert torch.equal(res[0][0], res[1][0])
    assert torch.equal(res[0][1], res[1][1])
    assert np.array_equal(res[0][2], res[1][2])


# ------------------------------------------------------- the one-launch operators of the decoder --
@pytest.mark.parametrize("rows,hidden", [(1, 4096), (7, 4096), (300, 512), (3, 11008)])
def test_rmsnorm_matches_torch(gpu_device, rows, hidden):
    import adamas_amd.utils as U
    g = torch.Generator().manual_seed(rows + hidden)
    x = (torch.randn(rows, hidden, generator=g) * 3).half().to(gpu_device)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).half().to(gpu_device)
    got = U.rms_norm_forward(x, w, 1e-5)
    xf = x.float()
    want = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).half() * w
    # fp32 sums in a different order: the normalised value may round to the neighbouring fp16
    assert (got.float() - want.float()).abs().max().item() <= 2 ** -9 * want.float().abs().max().item()


def test_add_rms_norm_updates_residual_in_place(gpu_device):
    import adamas_amd.utils as U
    g = torch.Generator().manual_seed(4)
    x = torch.randn(6, 4096, generator=g).half().to(gpu_device)
    d = torch.randn(6, 4096, generator=g).half().to(gpu_device)
    w = (1 + 0.1 * torch.randn(4096, generator=g)).half().to(gpu_device)
    s = x + d
    want = U.rms_norm_forward(s, w, 1e-5)
    got = U.add_rms_norm(x, d, w, 1e-5)
    assert torch.equal(x, s)
    assert torch.equal(got, want)


@pytest.mark.parametrize("decode", [True, False])
def test_rope_split_matches_torch(gpu_device, decode):
    import adamas_amd.utils as U
    g = torch.Generator().manual_seed(3)
    n, H, D = (4, 32, 128) if decode else (50, 32, 128)
    qkv = torch.randn(n, 3, H, D, generator=g).half().to(gpu_device)
    half = D // 2
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) / half))
    ang = torch.arange(1000, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = ang.cos().float().to(gpu_device), ang.sin().float().to(gpu_device)
    if decode:
        lens = torch.tensor([5, 1000, 17, 333], dtype=torch.int32, device=gpu_device)
        pos = (lens - 1).long()
        q, k, v = U.rope_split(qkv, cos, sin, seq_lens=lens)
    else:
        pos = torch.arange(n, device=gpu_device) + 123
        q, k, v = U.rope_split(qkv, cos, sin, start_pos=123)

    def rope(t):
        t = t.float()
        c, s = cos[pos][:, None, :], sin[pos][:, None, :]
        t1, t2 = t[..., :half], t[..., half:]
        return torch.cat((t1 * c - t2 * s, t2 * c + t1 * s), -1)

    assert (q.float() - rope(qkv[:, 0])).abs().max().item() <= 2e-3
    assert (k.float() - rope(qkv[:, 1])).abs().max().item() <= 2e-3
    assert torch.equal(v, qkv[:, 2])


def test_silu_mul_matches_torch(gpu_device):
    import adamas_amd.utils as U
    g = torch.Generator().manual_seed(9)
    gu = (torch.randn(5, 2 * 11008, generator=g) * 2).half().to(gpu_device)
    got = U.silu_mul(gu)
    want = F.silu(gu[:, :11008].float()).half() * gu[:, 11008:]
    assert (got.float() - want.float()).abs().max().item() <= 4e-3


# 1024 workgroups of four rows and fewer take the instance with early weight loads: both sides of
# that limit, the widest row (16384) and rows shorter than one step of the workgroup
@pytest.mark.parametrize("n,k", [(4096, 4096), (4096, 11008), (22016, 4096), (1003, 520), (5, 8),
                                 (64, 16384), (4096, 2048), (4100, 2048), (4097, 16384)])
def test_gemv_matches_fp32_matmul(gpu_device, n, k):
    import adamas_amd.utils as U
    g = torch.Generator().manual_seed(n + k)
    w = (torch.randn(n, k, generator=g) * 0.05).half().to(gpu_device)
    x = torch.randn(1, k, generator=g).half().to(gpu_device)
    got = U.gemv(w, x)
    want = x.float() @ w.float().T
    assert got.shape == (1, n)
    assert (got.float() - want).abs().max().item() <= 2e-3 * max(1.0, want.abs().max().item())


def test_rope_append_decode_equals_rope_split_plus_append(gpu_device):
    """The one-launch decode append against the two operators it replaces: same q, same query code,
    same cache contents (K, V, codes), bit for bit."""
    import adamas_amd.utils as U
    from tests import helpers as T
    g = torch.Generator().manual_seed(8)
    B, H, D = 3, 32, 128
    lens = [40, 333, 17]
    half = D // 2
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) / half))
    ang = torch.arange(512, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = ang.cos().float().to(gpu_device), ang.sin().float().to(gpu_device)
    qkv = (torch.randn(B, 3, H, D, generator=g) * 3).half().to(gpu_device)
    results = []
    for fused in (False, True):
        ctrl = T.make_controller(gpu_device, 512, 64, 16, batch_size=B, shuffle_seed=3)
        for b, L in enumerate(lens):
            kk = torch.randn(L - 1, H, D, generator=torch.Generator().manual_seed(b)).half().to(gpu_device)
            T.fill_sequence(ctrl, kk, kk, seq_idx=b)
        ctrl.prepare_hadamard(1)
        ctrl.begin_forward(1)
        if fused:
            q, q_code = U.rope_append_decode(qkv, cos, sin, ctrl, 0)
        else:
            q, k, v = U.rope_split(qkv, cos, sin, seq_lens=ctrl.seq_lens)
            q_code = U.append_kvh(k, v, None, ctrl, 0, q=q)
        caches = [T.read_logical_cache(ctrl, 0, b) for b in range(B)]
        results.append((q.clone(), q_code.clone(), caches))
    (q0, c0, k0), (q1, c1, k1) = results
    assert torch.equal(q0, q1) and torch.equal(c0, c1)
    for a, b in zip(k0, k1):
        for x, y in zip(a, b):
            assert np.array_equal(x.view(np.uint16), y.view(np.uint16))


@pytest.mark.parametrize("lens,hq,hkv,page_size,budget", [
    ([700], 32, 32, 16, 64),             # narrow estimator workgroups (short launch)
    ([40, 333, 17, 2], 32, 32, 16, 64),  # ragged batch, sequences below the budget
    ([1500], 32, 8, 16, 96),             # grouped queries: four workgroups share a new key
    ([1500, 900], 64, 16, 5, 96),        # odd page size, 64 heads
    ([33000], 32, 32, 16, 128),          # 65 chunks: one more than the chip has CUs per head group
    ([9000], 32, 32, 1, 200),            # page size 1
])
@pytest.mark.parametrize("scale", [1.0, 128 ** -0.5])
@pytest.mark.parametrize("fmt", ["fp16-nhd", "bf16-nhd", "fp16-hnd", "bf16-hnd"])
def test_layer_step_equals_append_then_step(gpu_device, lens, hq, hkv, page_size, budget, scale, fmt):
    """adamas_decode_layer_step (query code, rotary embedding, append and step in two launches)
    against rope_append_decode + decode_step: same cache contents and codes bit for bit, same
    selections, outputs equal up to the order of the softmax accumulation; float16 and bfloat16
    data, both page layouts."""
    import adamas_amd.utils as U
    from tests import helpers as T
    dtype = torch.bfloat16 if fmt.startswith("bf16") else torch.float16
    layout = U.TensorLayout.HND if fmt.endswith("hnd") else U.TensorLayout.NHD
    B, D = len(lens), 128
    cap = max(lens) + 8
    g = torch.Generator().manual_seed(sum(lens) + hq)
    half = D // 2
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) / half))
    ang = torch.arange(cap, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = ang.cos().float().to(gpu_device), ang.sin().float().to(gpu_device)
    qkv = (torch.randn(B, hq + 2 * hkv, D, generator=g) * 2).to(dtype).to(gpu_device)
    past = [((torch.randn(L - 1, hkv, D, generator=g) * 2).to(dtype).to(gpu_device),
             torch.randn(L - 1, hkv, D, generator=g).to(dtype).to(gpu_device)) for L in lens]
    results = []
    for fused in (False, True):
        ctrl = T.make_controller(gpu_device, cap, budget, page_size, batch_size=B, shuffle_seed=3,
                                 num_heads=hq, num_kv_heads=hkv, scale=scale, dtype=dtype,
                                 layout=layout)
        for b, (kk, vv) in enumerate(past):
            if kk.shape[0]:
                T.fill_sequence(ctrl, kk, vv, seq_idx=b)
        ctrl.prepare_hadamard(1)
        ctrl.begin_forward(1)
        assert U.layer_step_supported(ctrl)
        if fused:
            o, sel = U.decode_layer_step(qkv, cos, sin, ctrl, 0, return_indices=True)
        else:
            q, q_code = U.rope_append_decode(qkv, cos, sin, ctrl, 0)
            o, sel = U.decode_step(q, q_code, ctrl, 0, return_indices=True)
        caches = [T.read_logical_cache(ctrl, 0, b) for b in range(B)]
        results.append((o.clone(), T.np16(sel).copy(), caches))
    (o0, s0, c0), (o1, s1, c1) = results
    for a, b in zip(c0, c1):
        for x, y in zip(a, b):
            assert np.array_equal(x.view(np.uint16), y.view(np.uint16))
    assert np.array_equal(np.sort(s0, axis=1), np.sort(s1, axis=1))
    # (bfloat16 outputs are a few units of their last place apart at most: 2^-8 relative)
    tol = 1e-3 if dtype == torch.float16 else 2e-3 + 2.0 ** -7 * o1.float().abs().max().item()
    assert (o0.float() - o1.float()).abs().max().item() <= tol


@pytest.mark.parametrize("n,k", [(4096, 4096), (4096, 11008), (1008, 520)])
def test_gemv_add_and_normed_fold_the_residual_and_the_norm(gpu_device, n, k):
    """gemv_add writes resid += w . x (fp16 roundings of the unfused sequence) and the partial sums
    of squares; gemv_normed gives the projection of RMSNorm(resid) from them, plain and gated."""
    import adamas_amd.utils as U
    g = torch.Generator().manual_seed(n + k)
    w = (torch.randn(n, k, generator=g) * 0.05).half().to(gpu_device)
    x = torch.randn(1, k, generator=g).half().to(gpu_device)
    resid = torch.randn(1, n, generator=g).half().to(gpu_device)
    want = (resid.float() + (x.float() @ w.float().T).half().float()).half()
    ps = torch.empty(n // 4, dtype=torch.float32, device=gpu_device)
    got = resid.clone()
    U.gemv_add(w, x, got, ps)
    # the fp16 projection may differ from the fp32 reference by one fp16 step before the add
    assert (got.float() - want.float()).abs().max().item() <= 4e-3 * max(1.0, want.abs().max().item())
    sq = (got.float() ** 2).view(-1, 4).sum(-1)
    assert torch.allclose(ps, sq, rtol=1e-5, atol=1e-6)
    ps2 = torch.empty_like(ps)
    U.sumsq_partials(got, ps2)
    assert torch.allclose(ps2, sq, rtol=1e-5, atol=1e-6)
    # the projection of the normalised row: n rows of n-wide weights
    eps = 1e-5
    w2 = (torch.randn(2 * 256, n, generator=g) * 0.05).half().to(gpu_device)
    normed = got.float() * torch.rsqrt((got.float() ** 2).mean() + eps)
    y = U.gemv_normed(w2, got, ps, eps)
    ref = normed @ w2.float().T
    assert (y.float() - ref).abs().max().item() <= 2e-3 * max(1.0, ref.abs().max().item())
    yg = U.gemv_normed(w2, got, ps, eps, gated=True)
    gate, up = ref[:, :256], ref[:, 256:]
    refg = torch.nn.functional.silu(gate) * up
    assert (yg.float() - refg).abs().max().item() <= 4e-3 * max(1.0, refg.abs().max().item())


def test_layer_step_is_refused_where_the_two_launch_step_does_not_apply(gpu_device):
    """Budgets above 256 are served by rope_append_decode + decode_step: the one-call step says so
    instead of computing something; and it checks the format of the projection it is given."""
    import adamas_amd.utils as U
    from tests import helpers as T
    cos = torch.ones(1100, 64, device=gpu_device)
    sin = torch.zeros(1100, 64, device=gpu_device)
    qkv = torch.zeros(1, 96, 128, dtype=torch.float16, device=gpu_device)
    kk = torch.zeros(1000, 32, 128, dtype=torch.float16, device=gpu_device)
    ctrl = T.make_controller(gpu_device, 1100, 512, 16)
    T.fill_sequence(ctrl, kk, kk)
    ctrl.prepare_hadamard(1)
    ctrl.begin_forward(1)
    assert not U.layer_step_supported(ctrl)
    with pytest.raises(RuntimeError):
        U.decode_layer_step(qkv, cos, sin, ctrl, 0)
    ctrl = T.make_controller(gpu_device, 1100, 64, 16, dtype=torch.bfloat16)
    T.fill_sequence(ctrl, kk.bfloat16(), kk.bfloat16())
    ctrl.prepare_hadamard(1)
    ctrl.begin_forward(1)
    assert U.layer_step_supported(ctrl)
    with pytest.raises(RuntimeError):   # a float16 projection for bfloat16 caches
        U.decode_layer_step(qkv, cos, sin, ctrl, 0)


@pytest.mark.parametrize("inter,k", [(11008, 4096), (1002, 264)])
def test_gemv_silu_gate_equals_gemv_then_silu_mul(gpu_device, inter, k):
    import adamas_amd.utils as U
    g = torch.Generator().manual_seed(inter)
    w = (torch.randn(2 * inter, k, generator=g) * 0.05).half().to(gpu_device)
    x = torch.randn(1, k, generator=g).half().to(gpu_device)
    assert torch.equal(U.gemv_silu_gate(w, x), U.silu_mul(U.gemv(w, x)))


@pytest.mark.parametrize("heads", [64, 40])
def test_other_head_counts(gpu_device, heads):
    """Every kernel takes any multiple of 8 heads (40: the 13B shape of the model family); the other
    tests use 32."""
    cfg = DecoderConfig(num_layers=2, hidden=128 * heads, num_heads=heads, head_dim=128, intermediate=256,
                        vocab=256, dense_layers=1)
    m = LlamaShapedDecoder(cfg, gpu_device, seed=6)
    ids = torch.randint(0, cfg.vocab, (200,), generator=torch.Generator().manual_seed(2)).to(gpu_device)
    m.init_cache(page_size=16, max_seq_len=256, token_budget=48)
    logits = m.prefill(ids)
    ref = reference_logits(m, ids)
    assert _close(logits[0], ref[-1])
    nxt = ref[-1].argmax().view(1)
    got = m.decode_step_eager(nxt, sparse=False)
    assert _close(got[0], reference_logits(m, torch.cat((ids, nxt)))[-1])
    m.clear()
    outs = []
    for use_graph in (False, True):
        m.init_cache(page_size=16, max_seq_len=256, token_budget=48)
        first = m.prefill(ids).argmax(-1)
        toks, _ = m.generate(first, 6, sparse=True, use_graph=use_graph)
        outs.append(toks.numpy())
        m.clear()
    assert np.array_equal(outs[0], outs[1])


def test_grouped_query_decoder(gpu_device):
    """32 query heads over 8 key/value heads: prefill, dense decode against the fp32 model, sparse
    decode through the HIP graph against the eager loop."""
    cfg = DecoderConfig(num_layers=2, hidden=4096, num_heads=32, head_dim=128, intermediate=256,
                        vocab=256, dense_layers=1, num_kv_heads=8)
    m = LlamaShapedDecoder(cfg, gpu_device, seed=9)
    ids = torch.randint(0, cfg.vocab, (260,), generator=torch.Generator().manual_seed(3)).to(gpu_device)
    m.init_cache(page_size=16, max_seq_len=320, token_budget=48)
    logits = m.prefill(ids)
    ref = reference_logits(m, ids)
    assert _close(logits[0], ref[-1])
    nxt = ref[-1].argmax().view(1)
    got = m.decode_step_eager(nxt, sparse=False)
    assert _close(got[0], reference_logits(m, torch.cat((ids, nxt)))[-1])
    m.clear()
    outs = []
    for use_graph in (False, True):
        m.init_cache(page_size=16, max_seq_len=320, token_budget=48)
        first = m.prefill(ids).argmax(-1)
        toks, _ = m.generate(first, 6, sparse=True, use_graph=use_graph)
        outs.append(toks.numpy())
        m.clear()
    assert np.array_equal(outs[0], outs[1])
