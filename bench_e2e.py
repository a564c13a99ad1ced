#!/usr/bin/env python3
"""End-to-end decode benchmark on one MI355X: a random-init Llama-2-7B-shaped model (32 layers,
hidden 4096, 32 heads x 128, fp16), prefill of seeded uniform-random token ids, then greedy decoding
with the Adamas sparse attention path (token budget 128) on layers 2-31 and dense attention on
layers 0-1, against the same model with dense decode attention on every layer.

Counterpart of the reference's scripts/bench_textgen.py (time per generated token).  Prints one JSON
line.  `python bench_e2e.py --prompt 32768 --new-tokens 256` is the configuration the benchmark
definition names; smaller values give a quick check.
"""
import argparse
import json
import sys
import time


def log(msg):
    print(f"[bench_e2e] {msg}", file=sys.stderr, flush=True)


def run_e2e(prompt=32768, new_tokens=256, budget=128, page_size=16, layers=32,
            model_name="llama2_7b", use_graph=True, log=log, hadamard_scale=None):
    """Prefill + greedy decoding, sparse path against dense attention on every layer; returns the
    result record (protocol of the reference's scripts/bench_textgen.py:89-116: time per generated
    token after the prefill, here between device events around the whole decode loop)."""
    import torch
    from adamas_amd import _lib
    from adamas_amd.utils import ORTHONORMAL_SCALE
    from adamas_amd.decoder import DecoderConfig, LlamaShapedDecoder

    if not torch.cuda.is_available():
        raise SystemExit("the end-to-end benchmark needs a GPU")
    _lib.load()
    dev = torch.device("cuda:0")
    cfg = getattr(DecoderConfig, model_name)()
    cfg.num_layers = layers
    t0 = time.time()
    model = LlamaShapedDecoder(cfg, dev, seed=0)
    torch.cuda.synchronize()
    log(f"model ready in {time.time() - t0:.1f}s "
        f"({torch.cuda.memory_allocated() / 2**30:.1f} GiB allocated)")
    ids = torch.randint(0, cfg.vocab, (prompt,), generator=torch.Generator().manual_seed(5)).to(dev)
    max_len = prompt + new_tokens
    # the codes of the caches: the library's default transform (orthonormal) unless told otherwise
    scale = ORTHONORMAL_SCALE if hadamard_scale is None else float(hadamard_scale)

    results = {}
    for mode, sparse in (("adamas", True), ("dense", False)):
        model.init_cache(page_size, max_len, budget, hadamard_scale=scale)
        torch.cuda.synchronize()
        t0 = time.time()
        first = model.prefill(ids).argmax(-1)
        torch.cuda.synchronize()
        prefill_s = time.time() - t0
        toks, s_per_tok = model.generate(first, new_tokens, sparse=sparse, use_graph=use_graph)
        results[mode] = {"ms_per_token": round(s_per_tok * 1e3, 4),
                         "tok_per_s": round(1.0 / s_per_tok, 2),
                         "prefill_s": round(prefill_s, 2),
                         "first_tokens": toks[:8].tolist()}
        log(f"{mode}: prefill {prefill_s:.2f}s, decode {s_per_tok * 1e3:.3f} ms/token "
            f"({1.0 / s_per_tok:.1f} tok/s)")
        model.clear()
        model.ctrl = None
        torch.cuda.empty_cache()

    a, d = results["adamas"], results["dense"]
    return {
        "metric": "e2e_decode_tok_per_s", "value": a["tok_per_s"], "unit": "tok/s", "n_gpus": 1,
        "higher_is_better": True, "dtype": "fp16", "data": "synthetic (random-init weights, seeded "
        "uniform-random prompt ids)",
        "config": {"workload": f"c5_e2e_{model_name}_shape", "layers": cfg.num_layers,
                   "query_heads": cfg.num_heads, "kv_heads": cfg.kv_heads,
                   "prompt_tokens": prompt, "new_tokens": new_tokens,
                   "token_budget": budget, "page_size": page_size, "hadamard_scale": scale,
                   "dense_layers": cfg.dense_layers, "decode_loop": "one HIP graph per token"
                   if use_graph else "eager"},
        "adamas": a, "dense": d,
        "speedup_vs_dense": round(d["ms_per_token"] / a["ms_per_token"], 3),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--prompt", type=int, default=32768)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--budget", type=int, default=128)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--model", choices=["llama2_7b", "llama3_8b"], default="llama2_7b",
                    help="shape of the random-init model (llama3_8b: 8 key/value heads)")
    ap.add_argument("--no-graph", action="store_true", help="eager decode loop (host work per step)")
    ap.add_argument("--hadamard-scale", type=float, default=None,
                    help="scale of the Hadamard transform behind the codes (default: 128**-0.5)")
    args = ap.parse_args()
    print(json.dumps(run_e2e(args.prompt, args.new_tokens, args.budget, args.page_size, args.layers,
                             args.model, not args.no_graph, hadamard_scale=args.hadamard_scale)),
          flush=True)


if __name__ == "__main__":
    main()
