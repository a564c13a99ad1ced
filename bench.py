#!/usr/bin/env python3
"""Benchmark of the Adamas decode-time sparse-attention path on one MI355X.

A "step" is one pass of the hot path for one layer and one decode token at the headline shape:
batch 1, 32 heads x 128, fp16 paged KV of 32768 tokens (page size 16), token budget 128:
distance estimate over the 2-bit code cache -> top-k -> sparse paged attention (adamas_decode_step).
The caches are resident in HBM before the timed region.  To keep MI355X's 256 MB Infinity Cache from
serving the 32 MiB code scan, consecutive steps rotate over `--layers` distinct layer caches and
every timed replay starts behind an untimed flush of that cache.

Timed region: the K steps are recorded once into a HIP graph and replayed between two events on
the same stream (launch overhead of the Python host would otherwise dominate kernels that run for
a few microseconds); `value` is the median over the replays, the eager figure is reported next to it.
The same run also times each kernel on its own, a launch that only reads a code cache (the practical
ceiling of the estimator, `roofline.ceiling_us`), checks the timed path against the three stand-alone
operators, times the CPU restatement of the reference's PyTorch path, and runs the end-to-end
decode of the Llama-2-7B shape (`e2e`: tok/s with the sparse path against dense attention).

Prints ONE JSON line.  Usage: python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth

PROFILE_TRAFFIC_MD = os.path.join(ROOT, "profiles", "decode_step_kernels_c2_32k_b128.md")


def strip_c_comments(text: str) -> str:
    """C/C++ source without comments and without runs of white space (string and character
    literals are kept as they are)."""
    out = []
    i, n = 0, len(text)
    while i < n:
        c = text[i]
        if c in "\"'":                              # literal: copy to the closing quote
            j = i + 1
            while j < n and text[j] != c:
                j += 2 if text[j] == "\\" else 1
            out.append(text[i:j + 1])
            i = j + 1
        elif text.startswith("//", i):
            j = text.find("\n", i)
            i = n if j < 0 else j
        elif text.startswith("/*", i):
            j = text.find("*/", i + 2)
            i = n if j < 0 else j + 2
            out.append(" ")
        else:
            out.append(c)
            i += 1
    return " ".join("".join(out).split())


def kernel_sources_digest() -> str:
    """Digest of the HIP sources the library is built from, comments and white space left out: a
    counter run recorded in profiles/ speaks for the kernels of the same code, and an edit of a
    comment does not change the code."""
    import glob
    import hashlib
    h = hashlib.sha256()
    for path in sorted(glob.glob(os.path.join(ROOT, "adamas_amd", "csrc", "*"))):
        with open(path, "r", encoding="utf-8") as f:
            h.update(os.path.basename(path).encode() + b"\0" + strip_c_comments(f.read()).encode())
    return h.hexdigest()[:16]


def measured_traffic_bytes(workload: str, kernel: str):
    """HBM bytes per launch of `kernel` from the counter run recorded in profiles/ (rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE, scaled there by the same counters on a device copy of known size), or
    None when that summary was not made from the present kernel sources, names another workload or
    has no row for this template instance.  The summary carries machine-readable lines
        traffic-sources-digest: <digest>
        traffic: <workload> | <kernel instance> | <fetch KiB> | <write KiB>"""
    try:
        text = open(PROFILE_TRAFFIC_MD).read()
    except OSError:
        return None
    digest = None
    rows = {}
    for line in text.splitlines():
        line = line.strip().strip("`")
        if line.startswith("traffic-sources-digest:"):
            digest = line.split(":", 1)[1].strip()
        elif line.startswith("traffic:"):
            parts = [x.strip() for x in line.split(":", 1)[1].split("|")]
            if len(parts) == 4:
                rows[(parts[0], parts[1])] = (float(parts[2]) + float(parts[3])) * 1024
    if digest != kernel_sources_digest():
        return None
    v = rows.get((workload, kernel))
    return int(v) if v is not None else None


def estimator_instance(_lib, page_size: int, heads: int, batch: int, max_seq_len: int, budget: int) -> str:
    """Name of the fused estimator's template instance the library launches for these sizes
    (page size, passes, partial last pass, histogram mode, heads per workgroup, fused projection),
    from the library's own plan."""
    p = _lib.step_plan(batch, heads, max_seq_len, budget)
    flag = lambda v: "true" if v else "false"
    return (f"estimate_select_kernel<{16 if page_size == 16 else 0}, {p['passes']}, "
            f"{flag(p['partial'])}, false, {p['heads']}, false>")


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=320)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--layers", type=int, default=16, help="distinct layer caches to rotate over")
    ap.add_argument("--workload", default="c2_32k_b128")
    ap.add_argument("--page-size", type=int, default=0,
                    help="override the page size of the workload (the reference only works at 1)")
    ap.add_argument("--kv-len", type=int, default=0,
                    help="override the sequence length of a single-sequence workload (the reference's "
                         "kernel benchmarks use 8192, 16384 and 32768)")
    ap.add_argument("--budget", type=int, default=0,
                    help="override the token budget of the workload (the reference's kernel benchmarks "
                         "go up to 4096; budgets above 256 run as two launches of other kernels)")
    ap.add_argument("--kv-heads", type=int, default=32,
                    help="key/value heads (grouped-query attention when below the 32 query heads); "
                         "the CPU baseline is skipped then")
    ap.add_argument("--gqa-vector-alu", action="store_true",
                    help="with --kv-heads below 32: time dense attention with the vector-ALU kernel "
                         "(ADAMAS_F_NO_MFMA) instead of the matrix-core kernel")
    ap.add_argument("--kv-dtype", choices=("fp16", "bf16"), default="fp16",
                    help="16-bit format of q, K, V and the output (single-sequence workloads; the "
                         "reference and the headline figure are fp16)")
    ap.add_argument("--kv-layout", choices=("nhd", "hnd"), default="nhd",
                    help="page layout of the KV cache: [2, page, heads, 128] (the reference's) or "
                         "[2, heads, page, 128]")
    ap.add_argument("--hadamard-scale", type=float, default=1.0,
                    help="scale of the Hadamard transform behind the codes of the timed caches: 1.0 = raw "
                         "+-1 butterfly (all four code levels on the synthetic inputs; the headline), "
                         "0.08838834764831845 = 128**-0.5, the orthonormal transform (the library default)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="time box of the CPU baseline")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra-legs", action="store_true",
                    help="headline workload only: skip the two extra timings of the step (caches built "
                         "with the other scale of the transform; a sequence of 33024 tokens)")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="headline workload only: skip the step timings of configs 1, 3 and 4 that ride "
                         "in the same record")
    ap.add_argument("--no-e2e", action="store_true",
                    help="skip the end-to-end decode leg (random-init Llama-2-7B shape, 32768-token "
                         "prompt, 256 greedy tokens, sparse path against dense attention)")
    ap.add_argument("--e2e-prompt", type=int, default=32768)
    ap.add_argument("--e2e-new-tokens", type=int, default=256)
    ap.add_argument("--profile", action="store_true",
                    help="for rocprofv3: eager launches only (no HIP graphs), no CPU baseline, plus one "
                         "plain device copy of known size to calibrate the byte counters")
    return ap.parse_args()


class CacheFlusher:
    """Untimed traffic between timed replays: streams a buffer larger than MI355X's 256 MB Infinity
    Cache, so that a replay never starts on layer caches the previous replay left there."""

    def __init__(self, torch, lib, _lib, dev, nbytes: int = 640 << 20):
        self.buf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        self.buf.zero_()
        self.lib, self._lib = lib, _lib

    def __call__(self):
        rc = self.lib.adamas_read_probe(self.buf.data_ptr(), self.buf.numel(), None,
                                        self._lib.current_stream())
        if rc:
            self._lib.check(rc, "adamas_read_probe")


def record_graph(torch, fn_enqueue, n_iters: int):
    """Record n_iters calls of fn_enqueue(i) into a HIP graph (every kernel warmed outside of the
    capture first) and replay it once, untimed."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(min(n_iters, 4)):
            fn_enqueue(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(n_iters):
            fn_enqueue(i)
    g.replay()
    torch.cuda.synchronize()
    return g


def time_replays(torch, graph, n_iters: int, replays: int, flush=None):
    """Microseconds per call for each of `replays` replays of the graph (events on the replay
    stream; the cache flush, if any, runs before the first event and is waited for)."""
    out = []
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(replays):
        if flush is not None:
            flush()
        torch.cuda.synchronize()
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        out.append(e0.elapsed_time(e1) * 1e3 / n_iters)
    return out


def time_graph(torch, fn_enqueue, n_iters: int, replays: int = 5, flush=None) -> float:
    """Median microseconds per call of fn_enqueue over `replays` replays of a graph of n_iters calls."""
    import statistics
    g = record_graph(torch, fn_enqueue, n_iters)
    return float(statistics.median(time_replays(torch, g, n_iters, replays, flush)))


def check_against_operators(np, out_step, sel_step, out_ops, sel_ops, what: str, tol: float = 2e-3):
    """The timed path against the three stand-alone operators on the same state: identical index
    sets per (sequence, head), outputs within the attention tolerance."""
    a = np.sort(sel_step.cpu().numpy().astype(np.int64), axis=1)
    b = np.sort(sel_ops.cpu().numpy().astype(np.int64), axis=1)
    if not np.array_equal(a, b):
        bad = int(np.nonzero((a != b).any(axis=1))[0][0])
        raise AssertionError(f"{what}: the timed step and the stand-alone operators select "
                             f"different tokens (first differing row {bad})")
    err = float(np.abs(out_step.float().cpu().numpy() - out_ops.float().cpu().numpy()).max())
    if not err <= tol:
        raise AssertionError(f"{what}: outputs differ by {err:.3e} (tolerance {tol})")
    return err


def run_batched(args, w, lib, torch, U, _lib, dev):
    """Batched ragged decode (several sequences, one shared shuffled page pool): times the whole
    step for the batch.  Inputs are drawn on the device (same distribution, no needles)."""
    import numpy as np
    H, D, P, budget = 32, 128, w.page_size, w.budget
    B, lens = len(w.seq_lens), w.seq_lens
    cap = (max(lens) + P - 1) // P * P
    n_layers = min(args.layers, 4)
    n_pages = (cap // P) * B
    order = np.random.default_rng(w.seed).permutation(n_pages).tolist()
    ctrl = U.InferenceController(n_layers, H, D, P, budget, cap, torch.float16, dev, batch_size=B,
                                 page_order=order, hadamard_scale=args.hadamard_scale)
    g = torch.Generator(device=dev).manual_seed(w.seed)
    gain = torch.ones(H, D, device=dev)
    for h in range(H):
        gain[h, torch.randperm(D, generator=g, device=dev)[:4]] = 8.0
    q = (torch.randn(B, H, D, generator=g, device=dev) * gain).half()
    k_new = (torch.randn(B, H, D, generator=g, device=dev) * gain).half()
    v_new = torch.randn(B, H, D, generator=g, device=dev).half()
    for b, L in enumerate(lens):
        k = (torch.randn(L - 1, H, D, generator=g, device=dev) * gain).half()
        v = torch.randn(L - 1, H, D, generator=g, device=dev).half()
        for s0 in range(0, L - 1, 8192):
            m = min(8192, L - 1 - s0)
            new = [0] * B
            new[b] = m
            ctrl.prepare_hadamard(new)
            for layer in range(n_layers):
                U.append_kvh(k[s0:s0 + m].contiguous(), v[s0:s0 + m].contiguous(), None, ctrl, layer,
                             seq_idx=b)
        del k, v
    ctrl.prepare_hadamard(1)
    ctrl.begin_forward(1)
    q_codes = [U.append_kvh(k_new, v_new, None, ctrl, layer, q=q) for layer in range(n_layers)]
    torch.cuda.synchronize()
    log(f"workload {w.name}: {B} sequences, {sum(lens)} tokens, {n_layers} layer caches resident")
    ws = ctrl.workspace(budget)
    out = torch.empty_like(q)
    Lmax = ctrl.max_len_now
    tbl, indptr, sl = (ctrl.seqs.table_dev.data_ptr(), ctrl.seqs.indptr_dev.data_ptr(),
                       ctrl.seqs.seq_lens_dev.data_ptr())
    sm_scale = 1.0 / math.sqrt(D)

    def step(i):
        ly = i % n_layers
        rc = lib.adamas_decode_step(q.data_ptr(), q_codes[ly].data_ptr(), ctrl.pool.kv[ly].data_ptr(),
                                    ctrl.pool.codes[ly].data_ptr(), tbl, indptr, sl, budget,
                                    out.data_ptr(), None, ws.data_ptr(), ws.numel(), B, H, H, D, P,
                                    sm_scale, Lmax, ctrl.seqs.max_pages, _lib.current_stream())
        if rc:
            _lib.check(rc, "adamas_decode_step")

    def k_cand(i):
        ly = i % n_layers
        rc = lib.adamas_step_candidates(q_codes[ly].data_ptr(), ctrl.pool.codes[ly].data_ptr(), tbl,
                                        indptr, sl, budget, ws.data_ptr(), ws.numel(), B, H, H, P, Lmax,
                                        ctrl.seqs.max_pages, _lib.current_stream())
        if rc:
            _lib.check(rc, "adamas_step_candidates")

    def k_attend(i):
        ly = i % n_layers
        rc = lib.adamas_step_attend(q.data_ptr(), ctrl.pool.kv[ly].data_ptr(),
                                    ctrl.pool.codes[ly].data_ptr(), tbl, indptr, sl, budget,
                                    out.data_ptr(), None, ws.data_ptr(), ws.numel(), B, H, H, D, P,
                                    sm_scale, Lmax, ctrl.seqs.max_pages, _lib.current_stream())
        if rc:
            _lib.check(rc, "adamas_step_attend")

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    steps = min(args.steps, 64)
    flush = CacheFlusher(torch, lib, _lib, dev)
    step_us = time_graph(torch, step, steps, flush=flush)
    cand_us = time_graph(torch, k_cand, steps, flush=flush)
    attend_us = time_graph(torch, k_attend, steps, flush=flush)
    # the timed path against the three stand-alone operators on layer 0 of the same state
    sel_step = torch.empty((B * H, budget - 1), dtype=torch.int32, device=dev)
    rc = lib.adamas_decode_step(q.data_ptr(), q_codes[0].data_ptr(), ctrl.pool.kv[0].data_ptr(),
                                ctrl.pool.codes[0].data_ptr(), tbl, indptr, sl, budget,
                                out.data_ptr(), sel_step.data_ptr(), ws.data_ptr(), ws.numel(), B, H, H,
                                D, P, sm_scale, Lmax, ctrl.seqs.max_pages, _lib.current_stream())
    _lib.check(rc, "adamas_decode_step")
    est = U.decode_estimate(q_codes[0], ctrl, 0)
    U.decode_topk(est, ctrl)
    out_ops = U.decode_sparse_attn(q, ctrl, 0, ctrl.topk_dindices_buffer)
    torch.cuda.synchronize()
    check_err = check_against_operators(np, out, sel_step, out_ops, ctrl.topk_dindices_buffer, w.name)
    log(f"timed step == stand-alone operators on every sequence (max output difference {check_err:.1e})")
    code_bytes = sum(L - 1 for L in lens) * H * 32
    step_bytes = sum(lens) * H * (D // 4) + B * 2 * budget * H * D * 2
    achieved = code_bytes / (cand_us * 1e-6) / 1e9
    return {
        "metric": "decode_attn_us_per_layer_batched_ragged", "value": round(step_us, 3), "unit": "us",
        "n_gpus": 1, "steps": steps, "warmup": args.warmup, "ms_per_step": round(step_us / 1e3, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "u32 popcount on 2-bit codes + fp16 KV with fp32 softmax", "data": "synthetic",
        "config": {"workload": w.name, "batch": B, "heads": H, "head_dim": D, "seq_lens": lens,
                   "page_size": P, "token_budget": budget, "hadamard_scale": args.hadamard_scale,
                   "rotated_layer_caches": n_layers,
                   "timed_region": "HIP graph of K steps", "launches_per_step": 2},
        "achieved_hbm_GBps": round(step_bytes / (step_us * 1e-6) / 1e9, 1),
        "frac_of_hbm_roofline": round(step_bytes / (step_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
        "algorithmic_bytes_per_step": step_bytes,
        "step_kernels_us": {"estimate_select": round(cand_us, 3), "select_attend": round(attend_us, 3)},
        "check": {"against": "estimate + top-k + sparse attention operators, same state",
                  "index_sets": "identical", "max_output_diff": check_err},
        "roofline": {"bound": "hbm",
                     "kernel": estimator_instance(_lib, P, H, B, Lmax, budget),
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "algorithmic_bytes_per_launch": code_bytes, "avg_launch_us": round(cand_us, 3)},
        "cpu_baseline": None,
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures the single-GPU decode path only; run with --gpus 1 "
              "(the path shards by head or by sequence without any exchange, nothing to measure "
              "across GPUs here)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import adamas_amd.utils as U
    from adamas_amd import _lib, synth

    if not _lib.LIB_PATH.exists():
        from adamas_amd.build import build_library
        build_library()
    lib = _lib.load()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    w = synth.WORKLOADS[args.workload]
    if args.page_size:
        import dataclasses
        w = dataclasses.replace(w, page_size=args.page_size)
    if args.budget:
        import dataclasses
        w = dataclasses.replace(w, budget=args.budget)
    if args.kv_len and len(w.seq_lens) == 1:
        import dataclasses
        w = dataclasses.replace(w, seq_lens=(args.kv_len,))
    if len(w.seq_lens) > 1:
        print(json.dumps(run_batched(args, w, lib, torch, U, _lib, dev)), flush=True)
        return
    result = run_single(args, w, lib, torch, U, _lib, dev, np, synth)
    if result is None:
        return
    # ---- config 5 in the same record: end-to-end decode on the Llama-2-7B shape -----------------
    # (the layer caches of the kernel measurements above are released when run_single returns)
    if not args.no_e2e and not args.profile:
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        from bench_e2e import run_e2e
        e2e = run_e2e(prompt=args.e2e_prompt, new_tokens=args.e2e_new_tokens, budget=128, page_size=16,
                      layers=32, model_name="llama2_7b", use_graph=True, log=log)
        a, d = e2e["adamas"], e2e["dense"]
        result["e2e"] = {"tok_per_s": a["tok_per_s"], "ms_per_token": a["ms_per_token"],
                         "dense_tok_per_s": d["tok_per_s"], "dense_ms_per_token": d["ms_per_token"],
                         "speedup_vs_dense": e2e["speedup_vs_dense"], "prefill_s": a["prefill_s"],
                         "config": e2e["config"]}
    print(json.dumps(result), flush=True)


class StepState:
    """Resident state of one single-sequence workload: `n_layers` distinct layer caches (token-rolled
    copies of the same seeded data, shuffled page table), the query codes of the current token and
    the launch closures of the timed step and of its two kernels."""

    def __init__(self, args, w, L, scale, n_layers, lib, torch, U, _lib, dev, np, synth):
        import dataclasses
        H, D, P, budget, Hkv = 32, 128, w.page_size, w.budget, args.kv_heads
        self.L, self.scale, self.n_layers = L, scale, n_layers
        seq = synth.make_workload(dataclasses.replace(w, seq_lens=(L,)))[0]
        self.seq = seq
        n_pages = (L + P - 1) // P
        order = np.random.default_rng(w.seed).permutation(n_pages).tolist()   # non-contiguous pages
        bf16 = args.kv_dtype == "bf16"
        fdt = torch.bfloat16 if bf16 else torch.float16
        layout = U.TensorLayout.HND if args.kv_layout == "hnd" else U.TensorLayout.NHD
        ctrl = U.InferenceController(n_layers, H, D, P, budget, L, fdt, dev, page_order=order,
                                     num_kv_heads=Hkv, layout=layout, hadamard_scale=scale)
        self.ctrl, self.fdt = ctrl, fdt
        kv_flags = ctrl.kv_flags   # the *_f entry points with flags 0 are the plain ones
        k_dev, v_dev, q_dev = (seq.k[:, :Hkv].to(dev).to(fdt), seq.v[:, :Hkv].to(dev).to(fdt),
                               seq.q.to(dev).to(fdt))
        chunk = 8192
        for s0 in range(0, L - 1, chunk):
            m = min(chunk, L - 1 - s0)
            ctrl.prepare_hadamard(m)
            for layer in range(n_layers):
                idx = (torch.arange(s0, s0 + m, device=dev) + 997 * layer) % (L - 1)
                U.append_kvh(k_dev[idx].contiguous(), v_dev[idx].contiguous(), None, ctrl, layer)
        ctrl.prepare_hadamard(1)
        ctrl.begin_forward(1)
        q3 = q_dev[None].contiguous()
        self.k_new, self.v_new = k_dev[L - 1:].contiguous(), v_dev[L - 1:].contiguous()
        q_codes = [U.append_kvh(self.k_new, self.v_new, None, ctrl, layer, q=q3)
                   for layer in range(n_layers)]
        assert ctrl.need_estimate()
        torch.cuda.synchronize()
        self.q3, self.q_codes = q3, q_codes
        self.ws = ctrl.workspace(budget)
        self.out = torch.empty_like(q3)
        self.sel = torch.empty((H, budget - 1), dtype=torch.int32, device=dev)
        sm_scale = 1.0 / math.sqrt(D)
        tbl, indptr, lens = (ctrl.seqs.table_dev.data_ptr(), ctrl.seqs.indptr_dev.data_ptr(),
                             ctrl.seqs.seq_lens_dev.data_ptr())
        tbl_stride = ctrl.seqs.max_pages   # fixed-stride page tables: rows start at b * max_pages
        kv_ptr = [ctrl.pool.kv[i].data_ptr() for i in range(n_layers)]
        code_ptr = [ctrl.pool.codes[i].data_ptr() for i in range(n_layers)]
        qc_ptr = [c.data_ptr() for c in q_codes]
        self.ptrs = (tbl, indptr, lens, tbl_stride, kv_ptr, code_ptr, qc_ptr, sm_scale, kv_flags)
        ws, out, sel = self.ws, self.out, self.sel

        def step(i):
            ly = i % n_layers
            rc = lib.adamas_decode_step_f(q3.data_ptr(), qc_ptr[ly], kv_ptr[ly], code_ptr[ly], tbl,
                                          indptr, lens, budget, out.data_ptr(), sel.data_ptr(),
                                          ws.data_ptr(), ws.numel(), 1, H, Hkv, D, P, sm_scale, L,
                                          tbl_stride, kv_flags, _lib.current_stream())
            if rc:
                _lib.check(rc, "adamas_decode_step")

        def k_cand(i):
            ly = i % n_layers
            rc = lib.adamas_step_candidates(qc_ptr[ly], code_ptr[ly], tbl, indptr, lens, budget,
                                            ws.data_ptr(), ws.numel(), 1, H, Hkv, P, L, tbl_stride,
                                            _lib.current_stream())
            if rc:
                _lib.check(rc, "adamas_step_candidates")

        def k_attend(i):
            ly = i % n_layers
            rc = lib.adamas_step_attend_f(q3.data_ptr(), kv_ptr[ly], code_ptr[ly], tbl, indptr, lens,
                                          budget, out.data_ptr(), sel.data_ptr(), ws.data_ptr(),
                                          ws.numel(), 1, H, Hkv, D, P, sm_scale, L, tbl_stride,
                                          kv_flags, _lib.current_stream())
            if rc:
                _lib.check(rc, "adamas_step_attend")

        self.step, self.k_cand, self.k_attend = step, k_cand, k_attend


def time_step_leg(args, w, L, scale, lib, torch, U, _lib, dev, np, synth, flush):
    """The timed step and its two kernels for another sequence length or another scale of the
    transform than the headline's, same protocol (graph replays behind a cache flush, rotating over
    the layer caches); the state is released afterwards."""
    st = StepState(args, w, L, scale, args.layers, lib, torch, U, _lib, dev, np, synth)
    for i in range(args.warmup):
        st.step(i)
    torch.cuda.synchronize()
    k_iters = (max(64, min(args.steps, 512)) + st.n_layers - 1) // st.n_layers * st.n_layers
    graph = record_graph(torch, st.step, args.steps)
    step_us = float(np.median(time_replays(torch, graph, args.steps, 11, flush)))
    leg = {"value": round(step_us, 3), "unit": "us", "kv_len": L, "hadamard_scale": scale}
    if lib.adamas_step_fused_supported(1, 32, L, w.budget):
        leg["estimate_select"] = round(time_graph(torch, st.k_cand, k_iters, flush=flush), 3)
        st.k_cand(0)
        leg["select_attend"] = round(time_graph(torch, st.k_attend, k_iters, flush=flush), 3)
    del graph, st
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    return leg


def run_single(args, w, lib, torch, U, _lib, dev, np, synth):
    """The single-sequence kernel workloads (configs 1, 2 and 4): returns the result record."""
    L, budget, P, H, D = w.seq_lens[0], w.budget, w.page_size, 32, 128
    Hkv = args.kv_heads
    assert H % Hkv == 0
    n_layers = args.layers
    t0 = time.time()
    st = StepState(args, w, L, args.hadamard_scale, n_layers, lib, torch, U, _lib, dev, np, synth)
    log(f"workload {w.name}: L={L} budget={budget} page={P}, caches resident after {time.time() - t0:.1f}s: "
        f"{n_layers} layers x ({L * Hkv * D * 4 / 2**20:.0f} MiB KV + {L * Hkv * 32 / 2**20:.0f} MiB codes)")
    seq, ctrl, fdt, bf16 = st.seq, st.ctrl, st.fdt, args.kv_dtype == "bf16"
    q3, ws, out, sel = st.q3, st.ws, st.out, st.sel
    tbl, indptr, lens, tbl_stride, kv_ptr, code_ptr, qc_ptr, sm_scale, kv_flags = st.ptrs
    k_new, v_new = st.k_new, st.v_new
    step, k_cand, k_attend = st.step, st.k_cand, st.k_attend
    dist = torch.empty((H, (L + 7) // 8 * 8), dtype=torch.int16, device=dev)
    topk_ws = torch.zeros(lib.adamas_topk_workspace_bytes(H, L - 1, budget - 1), dtype=torch.uint8,
                          device=dev)

    def k_estimate(i):
        ly = i % n_layers
        rc = lib.adamas_estimate(qc_ptr[ly], code_ptr[ly], tbl, indptr, lens, dist.data_ptr(),
                                 H * dist.shape[1], dist.shape[1], _lib.DIST_U16, 1, H, Hkv, P, L,
                                 _lib.current_stream())
        if rc:
            _lib.check(rc, "adamas_estimate")

    def k_topk(i):
        rc = lib.adamas_topk(dist.data_ptr(), dist.shape[1], L - 1, None, H, 0, None, 0, H,
                             budget - 1, sel.data_ptr(), None, budget - 1, _lib.KEY_U16_INT,
                             topk_ws.data_ptr(), topk_ws.numel(), _lib.current_stream())
        if rc:
            _lib.check(rc, "adamas_topk")

    def k_attn(i):
        ly = i % n_layers
        rc = lib.adamas_sparse_decode_f(q3.data_ptr(), kv_ptr[ly], tbl, indptr, lens,
                                        sel.data_ptr(), budget - 1, budget - 1, out.data_ptr(),
                                        ws.data_ptr(), ws.numel(), 1, H, Hkv, D, P, sm_scale, L,
                                        kv_flags, _lib.current_stream())
        if rc:
            _lib.check(rc, "adamas_sparse_decode")

    def k_dense(i):   # dense decode attention over all L tokens (layers 0-1 and short sequences)
        ly = i % n_layers
        rc = lib.adamas_sparse_decode_f(q3.data_ptr(), kv_ptr[ly], tbl, indptr, lens, None, 0, 0,
                                        out.data_ptr(), ws.data_ptr(), ws.numel(), 1, H, Hkv, D, P,
                                        sm_scale, L, dense_flags, _lib.current_stream())
        if rc:
            _lib.check(rc, "adamas_sparse_decode (dense)")

    dense_flags = kv_flags | (_lib.F_NO_MFMA if args.gqa_vector_alu else 0)
    qc_tmp = torch.empty((1, H, 16), dtype=torch.int16, device=dev)

    def k_append(i):
        ly = i % n_layers
        rc = lib.adamas_append_decode(q3.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), None,
                                      qc_tmp.data_ptr(), kv_ptr[ly], code_ptr[ly], tbl, indptr, lens,
                                      1, H, Hkv, D, P, args.hadamard_scale, _lib.dtype_flags(fdt),
                                      _lib.current_stream())
        if rc:
            _lib.check(rc, "adamas_append_decode")

    code_bytes_layer = ctrl.pool.codes[0].numel() * 2

    def k_read(i):   # a launch that only reads one layer's code cache
        rc = lib.adamas_read_probe(code_ptr[i % n_layers], code_bytes_layer, None, _lib.current_stream())
        if rc:
            _lib.check(rc, "adamas_read_probe")

    # ---- warm-up (untimed) ----
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()

    if args.profile:
        # a copy of known size (256 MiB read + 256 MiB written) for scaling FETCH_SIZE / WRITE_SIZE
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        for i in range(args.steps):
            step(i)
        torch.cuda.synchronize()
        for fn in (k_estimate, k_topk, k_attn, k_append, k_read):
            for i in range(16):
                fn(i)
        for i in range(4):
            k_dense(i)
        torch.cuda.synchronize()
        print(json.dumps({"profile_run": True, "steps": args.steps, "workload": w.name,
                          "calibration_copy_bytes": 256 << 20,
                          "kernel_sources_digest": kernel_sources_digest()}), flush=True)
        return None

    # ---- eager K steps (host launch overhead included), for the record ----
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for i in range(args.steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    eager_us = e0.elapsed_time(e1) * 1e3 / args.steps

    # ---- the timed region: exactly K steps, recorded in one HIP graph, between two events ----
    # Every replay starts behind a flush of the Infinity Cache (untimed), so no timed step finds
    # a layer cache the previous replay left there, whatever K is; inside a replay a layer cache
    # comes round again only after the n_layers - 1 others (n_layers x 32 MiB of codes) went by.
    flush = CacheFlusher(torch, lib, _lib, dev)
    graph = record_graph(torch, step, args.steps)
    replay_times = time_replays(torch, graph, args.steps, 21, flush)
    p10, p50, p90 = (float(x) for x in np.percentile(replay_times, [10, 50, 90]))
    step_us = p50           # the reported value: median over the replays
    log(f"step: graph median {step_us:.2f} us over {len(replay_times)} replays (p10 {p10:.2f}, p90 {p90:.2f}), "
        f"eager {eager_us:.2f} us")

    # ---- each kernel on its own (graph of back-to-back launches, rotating layers) ----
    k_iters = max(64, min(args.steps, 512))
    k_iters = (k_iters + n_layers - 1) // n_layers * n_layers
    fused = bool(lib.adamas_step_fused_supported(1, H, L, budget))
    if fused:   # the two launches of the timed step
        cand_us = time_graph(torch, k_cand, k_iters, flush=flush)
        cand_hot_us = time_graph(torch, lambda i: k_cand(0), k_iters)   # one cache: Infinity-Cache hot
        k_cand(0)
        attend_us = time_graph(torch, k_attend, k_iters, flush=flush)
    else:
        cand_us = cand_hot_us = attend_us = float("nan")
    # the four stand-alone operators of the reference API
    est_us = time_graph(torch, k_estimate, k_iters, flush=flush)
    k_estimate(0)           # distances of layer 0 feed the stand-alone top-k and attention timings
    topk_us = time_graph(torch, k_topk, k_iters)
    attn_us = time_graph(torch, k_attn, k_iters, flush=flush)
    append_us = time_graph(torch, k_append, k_iters)
    dense_us = time_graph(torch, k_dense, max(16, k_iters // 8), flush=flush)
    dense_gbps = 2 * L * Hkv * D * 2 / (dense_us * 1e-6) / 1e9
    # the practical ceiling: a kernel that only reads the same rotated code caches, in this run
    read_us = time_graph(torch, k_read, k_iters, flush=flush)
    log(f"step kernels: estimate+select {cand_us:.2f} us (cache-hot {cand_hot_us:.2f}), "
        f"select+attend {attend_us:.2f}; plain read of one code cache {read_us:.2f} us "
        f"({code_bytes_layer / read_us / 1e3:.0f} GB/s)")
    log(f"stand-alone operators: estimate {est_us:.2f}, topk {topk_us:.2f}, attn {attn_us:.2f}, "
        f"append {append_us:.2f}, dense attention {dense_us:.2f} ({dense_gbps:.0f} GB/s)")

    # ---- the timed path against the three stand-alone operators on the same state (layer 0) ----
    step(0)
    out_step, sel_step = out.clone(), sel.clone()
    k_estimate(0)
    k_topk(0)
    k_attn(0)
    torch.cuda.synchronize()
    check_err = check_against_operators(np, out_step, sel_step, out, sel, w.name)
    log(f"timed step == stand-alone operators (identical index sets, max output difference {check_err:.1e})")

    # ---- the same step on the other scale of the transform and just past the headline length ------
    # (the headline workload only: caches built with the orthonormal transform, whose codes take two
    # of the four levels on these inputs, and a sequence of 33024 tokens, which is what a decode loop
    # sees a few hundred tokens after a 32768-token prompt)
    extra_legs = {}
    if (args.workload == "c2_32k_b128" and (L, budget) == (32768, 128) and Hkv == H and not bf16
            and args.kv_layout == "nhd" and not args.no_extra_legs):
        other = U.ORTHONORMAL_SCALE if args.hadamard_scale == 1.0 else 1.0
        key = "orthonormal_scale" if other == U.ORTHONORMAL_SCALE else "raw_scale"
        extra_legs[key] = time_step_leg(args, w, L, other, lib, torch, U, _lib, dev, np, synth, flush)
        extra_legs["kv_len_33024"] = time_step_leg(args, w, 33024, args.hadamard_scale, lib, torch, U,
                                                   _lib, dev, np, synth, flush)
        for name, leg in extra_legs.items():
            log(f"{name}: step {leg['value']:.2f} us (estimate+select {leg.get('estimate_select')}, "
                f"select+attend {leg.get('select_attend')})")

    # ---- roofline of the dominant kernel of the timed step: the fused estimator -----------------
    # algorithmic bytes of one launch = the 2-bit codes of the L-1 past tokens (32 bytes per token
    # and head); what the kernel writes (candidates, histograms) is overhead, not counted
    dom_name, dom_us = ((estimator_instance(_lib, P, H, 1, L, budget), cand_us) if fused
                        else (f"estimate_kernel<{16 if P == 16 else 0}>", est_us))
    est_bytes = (L - 1) * Hkv * 32
    step_bytes = L * Hkv * (D // 4) + 2 * budget * H * D * 2   # codes + selected K and V rows
    achieved = est_bytes / (dom_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "kernel": dom_name, "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "traffic": measured_traffic_bytes(w.name, dom_name) if Hkv == H and not bf16 else None,
                "algorithmic_bytes_per_launch": est_bytes, "avg_launch_us": round(dom_us, 3),
                # a launch that only reads the same bytes (one rotated code cache), timed in this run
                "ceiling_us": round(read_us, 3),
                "ceiling_GBps": round(code_bytes_layer / (read_us * 1e-6) / 1e9, 1),
                "frac_of_ceiling": round(read_us * est_bytes / code_bytes_layer / dom_us, 4)}

    # ---- CPU baseline: torch restatement of the reference's PyTorch path on the host cores ----
    cpu = None
    if not args.no_cpu_baseline and Hkv == H:
        from oracle import torch_cpu_path as P_cpu
        torch.set_num_threads(os.cpu_count() or 1)
        hmat = P_cpu.hadamard_matrix()
        qf, kf, vf = seq.q.float(), seq.k.float(), seq.v.float()
        P_cpu.decode_layer_step(qf, kf[:4096], vf[:4096], budget, hmat, args.hadamard_scale)      # warm
        times = []
        t_start = time.time()
        while len(times) < 3 or (time.time() - t_start < args.cpu_seconds and len(times) < 50):
            t1 = time.perf_counter()
            P_cpu.decode_layer_step(qf, kf, vf, budget, hmat, args.hadamard_scale)
            times.append(time.perf_counter() - t1)
        cpu_us = float(np.median(times)) * 1e6
        cpu = {"value": round(cpu_us, 1), "unit": "us", "cores": torch.get_num_threads(),
               "kind": "port",
               "sample": f"{len(times)} layer-steps of the same workload ({w.name}), torch "
                         f"{torch.__version__} fp32 on the host, key codes recomputed every step as "
                         "the reference's PyTorch path does; median"}
        # the same with the key codes kept from step to step (what a code cache would give the CPU)
        kc = P_cpu.codes(kf.transpose(0, 1), hmat, args.hadamard_scale)
        cached = []
        t_start = time.time()
        while len(cached) < 3 or (time.time() - t_start < args.cpu_seconds / 3 and len(cached) < 50):
            t1 = time.perf_counter()
            P_cpu.decode_layer_step(qf, kf, vf, budget, hmat, args.hadamard_scale, k_codes=kc)
            cached.append(time.perf_counter() - t1)
        cpu["cached_codes_value"] = round(float(np.median(cached)) * 1e6, 1)
        log(f"cpu baseline: {cpu_us:.0f} us per layer-step on {cpu['cores']} threads "
            f"({cpu['cached_codes_value']:.0f} us with cached key codes)")

    result = {
        # the headline metric is quoted on 32768 tokens / budget 128; other shapes say what they are
        "metric": ("decode_attn_us_per_layer_32k_budget128" if (L, budget) == (32768, 128)
                   else f"decode_attn_us_per_layer_{L}_budget{budget}"),
        "value": round(step_us, 3),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_us / 1e3, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": f"u32 popcount on 2-bit codes + {args.kv_dtype} KV with fp32 softmax",
        "data": "synthetic",
        "config": {"workload": w.name, "batch": 1, "heads": H, "kv_heads": Hkv, "head_dim": D,
                   "kv_len": L,
                   "page_size": P, "kv_layout": args.kv_layout.upper(), "token_budget": budget,
                   "hadamard_scale": args.hadamard_scale,
                   "rotated_layer_caches": n_layers,
                   "timed_region": "HIP graph of K steps",
                   "launches_per_step": 2,
                   "step_path": "candidate lists" if fused else "distances and histograms"},
        "achieved_hbm_GBps": round(step_bytes / (step_us * 1e-6) / 1e9, 1),
        "frac_of_hbm_roofline": round(step_bytes / (step_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
        "algorithmic_bytes_per_step": step_bytes,
        "eager_us_per_step": round(eager_us, 3),
        "replays_us_per_step": {"p10": round(p10, 3), "median": round(p50, 3), "p90": round(p90, 3),
                                "replays": len(replay_times),
                                "infinity_cache": "flushed (untimed) before every replay"},
        "check": {"against": "estimate + top-k + sparse attention operators, same state",
                  "index_sets": "identical", "max_output_diff": check_err},
        "step_kernels_us": {"estimate_select": round(cand_us, 3),
                            "estimate_select_cache_hot": round(cand_hot_us, 3),
                            "select_attend": round(attend_us, 3)},
        "operator_kernels_us": {"append_decode": round(append_us, 3), "estimate": round(est_us, 3),
                                "topk": round(topk_us, 3), "sparse_attn": round(attn_us, 3),
                                "dense_attn": round(dense_us, 3),
                                "dense_attn_GBps": round(dense_gbps, 1)},
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    result.update(extra_legs)
    # ---- the other kernel workloads of the benchmark definition, same protocol, in the same record --
    # (configs 1, 3 and 4: the step and its two kernels; the full record of each is what
    # `bench.py --workload <name>` prints)
    if extra_legs and not args.no_other_workloads:
        others = {}
        # 4 layer caches for the long sequence: 128K tokens x 4 layers = 8.6 GB
        few = argparse.Namespace(**{**vars(args), "layers": min(args.layers, 4)})
        for name in ("c1_4k_b64", "c4_128k_b256"):
            w2 = synth.WORKLOADS[name]
            leg = time_step_leg(few if name.startswith("c4") else args, w2, w2.seq_lens[0],
                                args.hadamard_scale, lib, torch, U, _lib, dev, np, synth, flush)
            bytes2 = w2.seq_lens[0] * H * (D // 4) + 2 * w2.budget * H * D * 2
            leg["token_budget"] = w2.budget
            leg["algorithmic_bytes_per_step"] = bytes2
            leg["frac_of_hbm_roofline"] = round(bytes2 / (leg["value"] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)
            others[name] = leg
            log(f"{name}: step {leg['value']:.2f} us (estimate+select {leg.get('estimate_select')}, "
                f"select+attend {leg.get('select_attend')})")
        rb = run_batched(args, synth.WORKLOADS["c3_ragged16_b128"], lib, torch, U, _lib, dev)
        others["c3_ragged16_b128"] = {k: rb[k] for k in ("value", "unit", "step_kernels_us",
                                                           "frac_of_hbm_roofline",
                                                           "algorithmic_bytes_per_step")}
        others["c3_ragged16_b128"]["seq_lens"] = rb["config"]["seq_lens"]
        others["c3_ragged16_b128"]["estimator_frac_of_hbm_roofline"] = rb["roofline"]["frac"]
        log(f"c3_ragged16_b128: step {rb['value']:.2f} us {rb['step_kernels_us']}")
        result["other_workloads"] = others
    return result


if __name__ == "__main__":
    main()
