"""Llama-shaped decoder that drives the Adamas HIP path end to end.

Counterparts in the reference (restated, not imported):
  * AdamasAttention      - the attention forward of adamas/models/Adamas.py:68-225: prefill appends K, V
                           and the 2-bit codes of every prompt token (:118-142); a decode step appends
                           one token and runs estimate -> top-k -> sparse attention (:143-201), or dense
                           attention through the same kernels when no estimate is needed (:165-173).
  * LlamaShapedDecoder   - the decode loop of adamas/models/llama.py:420-486 with its policy of keeping
                           the first two layers dense (`_Adamas_skip_layer = 2`, llama.py:538 and
                           :427-439), and the state set-up of Adamas_init (llama.py:520-552).
  * generate()           - the timing loop of scripts/bench_textgen.py (time per generated token).

What is different by design: a decode step does no host work.  Page tables and lengths live on the
device, the pages of the tokens to come are reserved up front, and the whole step (32 layers, sampling
included) is recorded once into a HIP graph and replayed per token.  Weights are random (there is no
checkpoint to load here); the prefill uses torch matmuls (rocBLAS / hipBLASLt) and torch's
scaled_dot_product_attention.  This package's own code is the decode attention path plus the
one-launch operators around it (RMSNorm, rotary embedding fused with the q/k/v split, SiLU-gated
product, one-row matrix-vector product), without which a one-token step is mostly launch overhead.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional

import torch
import torch.nn.functional as F

from . import utils as U
from .utils.controller import ALL_PAST_TOKENS, ORTHONORMAL_SCALE, InferenceController


@dataclass
class DecoderConfig:
    num_layers: int = 32
    hidden: int = 4096
    num_heads: int = 32
    head_dim: int = 128
    intermediate: int = 11008
    vocab: int = 32000
    rope_theta: float = 10000.0
    rms_eps: float = 1e-5
    dense_layers: int = 2          # leading layers that always attend to everything (llama.py:538)
    num_kv_heads: int = 0          # key/value heads; 0 = num_heads (no grouped-query attention)

    @property
    def kv_heads(self) -> int:
        return self.num_kv_heads or self.num_heads

    @staticmethod
    def llama2_7b() -> "DecoderConfig":
        return DecoderConfig()

    @staticmethod
    def llama3_8b() -> "DecoderConfig":
        """Grouped-query attention: 32 query heads over 8 key/value heads."""
        return DecoderConfig(intermediate=14336, vocab=128256, rope_theta=500000.0, num_kv_heads=8)


# Profiler ranges around the stages of the attention module, with the names the reference gives its
# NVTX ranges (adamas/models/Adamas.py:112-220: "RoPE", "hadamard_transform", "append_kvh",
# "prefill_attn", "full_attn", "estimate", "topk", "approx_attn", "o_proj").  On ROCm torch's nvtx
# calls are roctx calls, so `rocprofv3 --marker-trace` shows them.  Where one launch covers several
# of the reference's stages the range carries their names joined by "+".  Off by default: a range
# is two host calls per stage and the eager decode loop is host-bound.
_STAGE_RANGES = False


def set_stage_ranges(enabled: bool) -> None:
    global _STAGE_RANGES
    _STAGE_RANGES = bool(enabled)


class stage:
    """`with stage("estimate+topk+approx_attn"):` = range_push / range_pop when ranges are on."""

    def __init__(self, name: str):
        self.name = name

    def __enter__(self):
        if _STAGE_RANGES:
            torch.cuda.nvtx.range_push(self.name)

    def __exit__(self, *exc):
        if _STAGE_RANGES:
            torch.cuda.nvtx.range_pop()
        return False


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x [N, K] @ w[M, K]^T.  One row goes through this package's matrix-vector kernel, which streams
    the weights faster than the library routines do for these shapes (measured for the 4096 x 11008
    down projection: 20 us against 29 us for torch.mv and 30 us for a one-row GEMM)."""
    if x.shape[0] == 1 and w.shape[1] % 8 == 0 and w.shape[1] <= 16384:
        return U.gemv(w, x)
    return F.linear(x, w)


class AdamasAttention:
    """Attention over the paged caches of one controller; stateless apart from it."""

    def __init__(self, ctrl: InferenceController):
        self.ctrl = ctrl

    def prefill(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layer: int) -> torch.Tensor:
        """q, k, v [N, H, D] of a fresh sequence whose N positions are already reserved.  Appends K, V
        and codes (Hadamard inside the kernel), returns causal attention [N, H, D]."""
        with stage("hadamard_transform+append_kvh"):
            U.append_kvh(k, v, None, self.ctrl, layer)
        with stage("prefill_attn"):
            o = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None],
                                               v.transpose(0, 1)[None], is_causal=True,
                                               enable_gqa=k.shape[1] != q.shape[1])
            return o[0].transpose(0, 1).contiguous()

    def decode(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layer: int,
               sparse: bool) -> torch.Tensor:
        """q, k, v [B, H, D], one new token per sequence (its slot is reserved and counted)."""
        with stage("hadamard_transform+append_kvh"):
            q_code = U.append_kvh(k, v, None, self.ctrl, layer, q=q)
        return self.attend(q, q_code, layer, sparse)

    def decode_from_qkv(self, qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, layer: int,
                        sparse: bool) -> torch.Tensor:
        """The same from the raw fused projection [B, Hq + 2*Hkv, D]: rotary embedding, append and
        codes are one launch, or none at all where the sparse step takes the projection itself."""
        c = self.ctrl
        if sparse and c.need_estimate() and U.layer_step_supported(c):
            # the append rides in the two launches of the step
            with stage("RoPE+hadamard_transform+append_kvh+estimate+topk+approx_attn"):
                return U.decode_layer_step(qkv, cos, sin, c, layer)
        with stage("RoPE+hadamard_transform+append_kvh"):
            q, q_code = U.rope_append_decode(qkv, cos, sin, c, layer)
        return self.attend(q, q_code, layer, sparse)

    def attend(self, q: torch.Tensor, q_code: torch.Tensor, layer: int, sparse: bool) -> torch.Tensor:
        c = self.ctrl
        if sparse and c.need_estimate():
            with stage("estimate+topk+approx_attn"):
                return U.decode_step(q, q_code, c, layer)
        with stage("full_attn"):
            return U.decode_sparse_attn(q, c, layer, ALL_PAST_TOKENS)


class LlamaShapedDecoder:
    def __init__(self, cfg: DecoderConfig, device, seed: int = 0, dtype=torch.float16):
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        g = torch.Generator(device=self.device).manual_seed(seed)   # weights are drawn on the device

        def w(*shape, std=0.02):
            return (torch.randn(*shape, generator=g, device=self.device) * std).to(dtype)

        c = cfg
        self.embed = w(c.vocab, c.hidden)
        self.lm_head = w(c.vocab, c.hidden)
        self.final_norm = torch.ones(c.hidden, dtype=dtype, device=self.device)
        self.layers: List[dict] = []
        for _ in range(c.num_layers):
            self.layers.append({
                "attn_norm": torch.ones(c.hidden, dtype=dtype, device=self.device),
                "wqkv": w((c.num_heads + 2 * c.kv_heads) * c.head_dim, c.hidden),
                "wo": w(c.hidden, c.num_heads * c.head_dim),
                "mlp_norm": torch.ones(c.hidden, dtype=dtype, device=self.device),
                "w_gate_up": w(2 * c.intermediate, c.hidden),
                "w_down": w(c.hidden, c.intermediate),
            })
        self.ctrl: Optional[InferenceController] = None
        self.attn: Optional[AdamasAttention] = None
        self._graph = None

    # --- state ------------------------------------------------------------------------------------
    def init_cache(self, page_size: int, max_seq_len: int, token_budget: int, page_order=None,
                   hadamard_scale: float = ORTHONORMAL_SCALE):
        """Counterpart of Adamas_init(page_size, max_seq_len, token_budget), llama.py:520-552."""
        c = self.cfg
        self.ctrl = InferenceController(c.num_layers, c.num_heads, c.head_dim, page_size,
                                        token_budget, max_seq_len, self.dtype, self.device,
                                        page_order=page_order, hadamard_scale=hadamard_scale,
                                        num_kv_heads=c.kv_heads)
        self.attn = AdamasAttention(self.ctrl)
        self.token_budget = token_budget
        half = c.head_dim // 2
        inv = 1.0 / (c.rope_theta ** (torch.arange(half, dtype=torch.float64) / half))
        ang = torch.arange(max_seq_len, dtype=torch.float64)[:, None] * inv[None, :]
        self.rope_cos = ang.cos().float().to(self.device)
        self.rope_sin = ang.sin().float().to(self.device)
        self._graph = None

    def clear(self):
        self.ctrl.clean_states()
        self._graph = None

    # --- one layer ---------------------------------------------------------------------------------
    # x is the residual stream, n its RMSNorm: every residual add is fused with the norm that follows
    # it (U.add_rms_norm updates x in place and returns the normalised rows).
    def _qkv(self, lw, n, seq_lens=None, start_pos=0):
        """n [N, hidden] (normalised) -> q, k (rotary applied), v, each [N, H, D].  Decode passes the
        device-side lengths (position = length - 1), prefill the first position."""
        c = self.cfg
        qkv = linear(n, lw["wqkv"]).view(-1, c.num_heads + 2 * c.kv_heads, c.head_dim)
        return U.rope_split(qkv, self.rope_cos, self.rope_sin, seq_lens=seq_lens, start_pos=start_pos,
                            num_kv_heads=c.kv_heads)

    def _mlp(self, lw, n):
        if n.shape[0] == 1 and n.shape[1] % 8 == 0 and n.shape[1] <= 16384:
            return linear(U.gemv_silu_gate(lw["w_gate_up"], n), lw["w_down"])   # activation fused
        return linear(U.silu_mul(linear(n, lw["w_gate_up"])), lw["w_down"])

    def _next_norm(self, li):
        return self.layers[li + 1]["attn_norm"] if li + 1 < len(self.layers) else self.final_norm

    # --- prefill -----------------------------------------------------------------------------------
    @torch.no_grad()
    def prefill(self, token_ids: torch.Tensor, mlp_chunk: int = 8192) -> torch.Tensor:
        """token_ids [N] int64 on the device; fills the caches, returns the logits of the last token."""
        eps = self.cfg.rms_eps
        n_tok = token_ids.shape[0]
        self.ctrl.prepare_hadamard(n_tok)
        self.ctrl.begin_forward(n_tok)
        x = self.embed[token_ids]
        n = U.rms_norm_forward(x, self.layers[0]["attn_norm"], eps)
        for li, lw in enumerate(self.layers):
            with stage("RoPE"):
                q, k, v = self._qkv(lw, n, start_pos=0)
            o = self.attn.prefill(q, k, v, li)
            with stage("o_proj"):
                d = F.linear(o.view(n_tok, -1), lw["wo"])
            for s0 in range(0, n_tok, mlp_chunk):
                xs = x[s0:s0 + mlp_chunk]
                m = U.add_rms_norm(xs, d[s0:s0 + mlp_chunk], lw["mlp_norm"], eps)
                n[s0:s0 + mlp_chunk] = U.add_rms_norm(xs, self._mlp(lw, m), self._next_norm(li), eps)
        self.ctrl.end_forward()
        return F.linear(n[-1:], self.lm_head)

    # --- decode ------------------------------------------------------------------------------------
    def _decode_layers(self, tok: torch.Tensor, sparse: bool) -> torch.Tensor:
        """The body of one decode step: tok [1] int64 -> logits [1, vocab].  The new token's slot must
        be reserved and counted in the device-side length already."""
        c, ctrl, eps = self.cfg, self.ctrl, self.cfg.rms_eps
        x = self.embed[tok]
        if c.hidden % 8 == 0 and c.hidden <= 16384:
            return self._decode_layers_folded(x, sparse)
        n = U.rms_norm_forward(x, self.layers[0]["attn_norm"], eps)
        for li, lw in enumerate(self.layers):
            qkv = linear(n, lw["wqkv"]).view(-1, c.num_heads + 2 * c.kv_heads, c.head_dim)
            o = self.attn.decode_from_qkv(qkv, self.rope_cos, self.rope_sin, li,
                                          sparse and li >= c.dense_layers)
            with stage("o_proj"):
                d = linear(o.view(1, -1), lw["wo"])
            m = U.add_rms_norm(x, d, lw["mlp_norm"], eps)
            n = U.add_rms_norm(x, self._mlp(lw, m), self._next_norm(li), eps)
        return linear(n, self.lm_head)

    def _folded_weights(self):
        """The projections that follow a norm, with the norm weight folded in (w[n][c] * g[c]); the
        same tensor where the norm weight is all ones."""
        if getattr(self, "_folded", None) is None:
            def fold(w, g):
                if bool((g == 1).all()):
                    return w
                return (w.float() * g.float()[None, :]).to(w.dtype)
            self._folded = {
                "layers": [(fold(lw["wqkv"], lw["attn_norm"]), fold(lw["w_gate_up"], lw["mlp_norm"]))
                           for lw in self.layers],
                "lm_head": fold(self.lm_head, self.final_norm),
                "partials": torch.empty(self.cfg.hidden // 4, dtype=torch.float32, device=self.device),
            }
        return self._folded

    def _decode_layers_folded(self, x: torch.Tensor, sparse: bool) -> torch.Tensor:
        """The same step with the residual adds and the norms folded into the projections: the
        output and down projections add into the residual stream x and leave partial sums of its
        squares, the projections after a norm scale their result by rsqrt(mean square).  Six
        launches per sparse layer (qkv, the two of the attention step, o, gate/up, down)."""
        c, eps = self.cfg, self.cfg.rms_eps
        fw = self._folded_weights()
        ps = fw["partials"]
        U.sumsq_partials(x, ps)
        for li, lw in enumerate(self.layers):
            wqkv_n, w_gate_up_n = fw["layers"][li]
            qkv = U.gemv_normed(wqkv_n, x, ps, eps).view(-1, c.num_heads + 2 * c.kv_heads, c.head_dim)
            o = self.attn.decode_from_qkv(qkv, self.rope_cos, self.rope_sin, li,
                                          sparse and li >= c.dense_layers)
            with stage("o_proj"):
                U.gemv_add(lw["wo"], o.view(1, -1), x, ps)
            U.gemv_add(lw["w_down"], U.gemv_normed(w_gate_up_n, x, ps, eps, gated=True), x, ps)
        return U.gemv_normed(fw["lm_head"], x, ps, eps)

    @torch.no_grad()
    def decode_step_eager(self, tok: torch.Tensor, sparse: bool = True) -> torch.Tensor:
        """One step with the host-side bookkeeping of the reference's loop (llama.py:420-486)."""
        ctrl = self.ctrl
        ctrl.prepare_hadamard(1)
        ctrl.set_page_budget(self.token_budget)
        ctrl.begin_forward(1)
        logits = self._decode_layers(tok, sparse)
        ctrl.end_forward()
        return logits

    @torch.no_grad()
    def generate(self, first_tok: torch.Tensor, n_tokens: int, sparse: bool = True,
                 use_graph: bool = True):
        """Greedy decoding of n_tokens tokens after first_tok [1] int64.  Returns (tokens [n_tokens]
        on the host, seconds per token measured with device events around the whole loop)."""
        ctrl = self.ctrl
        out = torch.empty(n_tokens, dtype=torch.int64, device=self.device)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if not use_graph:
            tok = first_tok.clone()
            torch.cuda.synchronize()
            e0.record()
            for i in range(n_tokens):
                tok = self.decode_step_eager(tok, sparse).argmax(-1)
                out[i] = tok[0]
            e1.record()
            torch.cuda.synchronize()
            return out.cpu(), e0.elapsed_time(e1) * 1e-3 / n_tokens

        # graph mode: pages for all tokens up front, one captured step replayed n_tokens times
        ctrl.begin_graph_decode(n_tokens)
        ctrl.set_page_budget(self.token_budget)
        ctrl.begin_forward(1)
        ctrl.workspace(ctrl.inference_page_budget)          # allocate before capture
        tok_buf = first_tok.clone()
        lens0 = ctrl.seq_lens.clone()

        def step():
            ctrl.advance_on_device()
            tok_buf.copy_(self._decode_layers(tok_buf, sparse).argmax(-1))

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):     # warm-up outside capture (library handles, allocator)
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        ctrl.seq_lens.copy_(lens0)        # undo the warm-up step
        tok_buf.copy_(first_tok)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        ctrl.seq_lens.copy_(lens0)        # capture does not execute, but keep the state explicit
        tok_buf.copy_(first_tok)
        torch.cuda.synchronize()
        e0.record()
        for i in range(n_tokens):
            graph.replay()
            out[i:i + 1].copy_(tok_buf, non_blocking=True)
        e1.record()
        torch.cuda.synchronize()
        ctrl.end_graph_decode(n_tokens)
        ctrl.end_forward()
        return out.cpu(), e0.elapsed_time(e1) * 1e-3 / n_tokens
