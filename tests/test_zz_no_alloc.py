"""adamas_decode_step_noalloc (the decode step working in the library's static device scratch, for
callers that cannot allocate) against adamas_decode_step_f with a caller workspace: same outputs
and selections bit for bit, on calls in a row that share the scratch, the later ones smaller."""
import math

import numpy as np
import pytest
import torch

from adamas_amd import _lib, synth

import helpers as T

pytestmark = pytest.mark.gpu


def _state(gpu_device, L, budget, page_size, seed):
    seq = synth.make_sequence(L, 4, torch.Generator().manual_seed(seed))
    ctrl = T.make_controller(gpu_device, L, budget, page_size, shuffle_seed=seed)
    T.fill_sequence(ctrl, seq.k[:-1].to(gpu_device), seq.v[:-1].to(gpu_device))
    q = seq.q[None].to(gpu_device)
    q_code = T.decode_append(ctrl, q, seq.k[-1:].to(gpu_device), seq.v[-1:].to(gpu_device))
    return ctrl, q, q_code


def _both(lib, ctrl, q, q_code, budget):
    c = ctrl
    L = c.max_len_now
    common = (q.data_ptr(), q_code.data_ptr(), c.pool.kv[0].data_ptr(), c.pool.codes[0].data_ptr(),
              c.seqs.table_dev.data_ptr(), c.seqs.indptr_dev.data_ptr(),
              c.seqs.seq_lens_dev.data_ptr(), budget)
    tail = (c.batch_size, c.num_heads, c.num_kv_heads, 128, c.page_size, 1.0 / math.sqrt(128), L,
            c.seqs.max_pages, 0, _lib.current_stream())
    out_a, out_b = torch.full_like(q, float("nan")), torch.full_like(q, float("nan"))
    sel_a = torch.full((c.batch_size * 32, budget - 1), -9, dtype=torch.int32, device=q.device)
    sel_b = sel_a.clone()
    ws = torch.zeros(lib.adamas_workspace_bytes(c.batch_size, 32, L, budget), dtype=torch.uint8,
                     device=q.device)
    rc = lib.adamas_decode_step_f(*common, out_a.data_ptr(), sel_a.data_ptr(), ws.data_ptr(),
                                  ws.numel(), *tail)
    assert rc == 0, _lib.error_string(rc)
    rc = lib.adamas_decode_step_noalloc(*common, out_b.data_ptr(), sel_b.data_ptr(), *tail)
    assert rc == 0, _lib.error_string(rc)
    torch.cuda.synchronize()
    return out_a, sel_a, out_b, sel_b


def test_noalloc_step_equals_workspace_step_on_consecutive_calls(gpu_device):
    lib = _lib.load()
    # the two-launch step, a smaller one, the three-launch step (budget 300, page size 3), a tiny
    # one at page size 1, then the first size again: every call finds the scratch as the previous,
    # differently sized call left it
    cases = [(20000, 128, 16, 1), (3000, 64, 16, 2), (9000, 300, 3, 3), (700, 16, 1, 4),
             (20000, 128, 16, 1)]
    states = {}
    for L, budget, page, seed in cases:
        if (L, seed) not in states:
            states[(L, seed)] = _state(gpu_device, L, budget, page, seed)
        ctrl, q, q_code = states[(L, seed)]
        before = torch.cuda.memory_allocated()
        out_a, sel_a, out_b, sel_b = _both(lib, ctrl, q, q_code, budget)
        assert torch.equal(out_a, out_b), (L, budget)
        assert torch.equal(sel_a, sel_b), (L, budget)
        assert torch.isfinite(out_b.float()).all()
        assert (sel_b >= 0).all() and (sel_b < L - 1).all()
        del out_a, sel_a, out_b, sel_b
        assert torch.cuda.memory_allocated() <= before   # nothing of torch's was allocated and kept


def test_noalloc_step_rejects_sizes_beyond_its_scratch(gpu_device):
    lib = _lib.load()
    ctrl, q, q_code = _state(gpu_device, 600, 32, 16, 5)
    c = ctrl
    out = torch.empty_like(q)
    args = [q.data_ptr(), q_code.data_ptr(), c.pool.kv[0].data_ptr(), c.pool.codes[0].data_ptr(),
            c.seqs.table_dev.data_ptr(), c.seqs.indptr_dev.data_ptr(), c.seqs.seq_lens_dev.data_ptr(),
            32, out.data_ptr(), None, 1, 32, 32, 128, 16, 1.0 / math.sqrt(128), 600, c.seqs.max_pages,
            0, _lib.current_stream()]
    assert lib.adamas_decode_step_noalloc(*args) == 0
    # a length bound whose workspace exceeds the scratch is refused before anything is launched
    big = list(args)
    big[16] = 1 << 20
    assert lib.adamas_workspace_bytes(1, 32, 1 << 20, 32) > _lib.STATIC_SCRATCH_BYTES
    assert lib.adamas_decode_step_noalloc(*big) == _lib.E_SCRATCH
    assert "scratch" in _lib.error_string(_lib.E_SCRATCH)
    big = list(args)
    big[10] = 16          # 16 sequences of 32768 tokens
    big[16] = 32768
    assert lib.adamas_decode_step_noalloc(*big) == _lib.E_SCRATCH
    torch.cuda.synchronize()
