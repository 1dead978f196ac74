"""A Qwen2-shaped decoder for the decode step of the LLM benchmark configuration: random-init W8A16
weights (int8 per output channel, fp16 activations), RMSNorm, rotary embedding, a block-paged fp16
KV cache and greedy sampling, recorded once as a resident `hip` function (one HIP-graph replay per
generated token for the whole batch).

Per layer:  h = x + O(attn(rope(QKV(rmsnorm(x)))));  x' = h + Down(silu(Gate(n)) * Up(n)), n = rmsnorm(h)
Last:       logits = LMHead(rmsnorm(x));  next token = argmax(logits)
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np

from . import runtime as rt
from .runtime import Context, Function


@dataclass
class DecoderConfig:
    layers: int = 24
    hidden: int = 896
    q_heads: int = 14
    kv_heads: int = 2
    head_dim: int = 64
    mlp: int = 4864
    vocab: int = 151936
    rms_eps: float = 1e-6
    rope_theta: float = 1e6
    block_size: int = 16


def quantize_rows(w: np.ndarray):
    """Per-output-channel symmetric int8: w[n, :] ~ scale[n] * q[n, :], q in [-127, 127]."""
    amax = np.maximum(np.abs(w).max(axis=1), 1e-8)
    scale = (amax / 127.0).astype(np.float32)
    q = np.clip(np.rint(w / scale[:, None]), -127, 127).astype(np.int8)
    return q, scale


def random_weights(cfg: DecoderConfig, seed: int = 5) -> Dict[str, object]:
    """Host-side weights of the whole model (numpy), shared by the device model and the float64 reference."""
    rng = np.random.default_rng(seed)
    qd = cfg.q_heads * cfg.head_dim
    kvd = cfg.kv_heads * cfg.head_dim

    def lin(n, k, std):
        return quantize_rows((rng.standard_normal((n, k), dtype=np.float32) * std))

    layers = []
    for _ in range(cfg.layers):
        layers.append({
            "ln1": (1.0 + 0.1 * rng.standard_normal(cfg.hidden)).astype(np.float16),
            "qkv": lin(qd + 2 * kvd, cfg.hidden, cfg.hidden ** -0.5),
            "qkv_bias": (rng.standard_normal(qd + 2 * kvd) * 0.1).astype(np.float32),
            "o": lin(cfg.hidden, qd, qd ** -0.5 * 0.5),
            "ln2": (1.0 + 0.1 * rng.standard_normal(cfg.hidden)).astype(np.float16),
            "gate_up": lin(2 * cfg.mlp, cfg.hidden, cfg.hidden ** -0.5),
            "down": lin(cfg.hidden, cfg.mlp, cfg.mlp ** -0.5 * 0.5),
        })
    emb = (rng.standard_normal((cfg.vocab, cfg.hidden), dtype=np.float32) * 0.5).astype(np.float16)
    return {"layers": layers, "embedding": emb, "ln_f": (1.0 + 0.1 * rng.standard_normal(cfg.hidden)).astype(np.float16),
            "lm_head": lin(cfg.vocab, cfg.hidden, cfg.hidden ** -0.5)}


class HipDecoder:
    """The decode step resident on the device.  The KV cache is pre-filled by the caller (`k_cache`, `v_cache`
    numpy arrays in the paged layouts) for the given context lengths; step() appends one token per sequence."""

    def __init__(self, ctx: Context, cfg: DecoderConfig, weights: Dict[str, object], batch: int, max_blocks_per_seq: int,
                 block_table: np.ndarray, ctx_lens: np.ndarray, k_caches: List[np.ndarray], v_caches: List[np.ndarray],
                 capture_graph: bool = True, feedback: bool = False, fuse_norm: bool = True, lanes: int = 1):
        self.ctx, self.cfg, self.batch = ctx, cfg, batch
        c = cfg
        qd, kvd = c.q_heads * c.head_dim, c.kv_heads * c.head_dim
        num_blocks = k_caches[0].shape[0]
        f16 = 2
        self.tokens = ctx.alloc(batch * 4)
        self.next_tokens = ctx.alloc(batch * 4)
        self.block_table = ctx.to_device(np.ascontiguousarray(block_table, np.int32))
        self.ctx_lens = ctx.to_device(np.ascontiguousarray(ctx_lens, np.int32))
        self.x = [ctx.alloc(batch * c.hidden * f16), ctx.alloc(batch * c.hidden * f16)]
        self.norm = ctx.alloc(batch * c.hidden * f16)
        self.qkv = ctx.alloc(batch * (qd + 2 * kvd) * f16)
        self.q = ctx.alloc(batch * qd * f16)
        self.att = ctx.alloc(batch * qd * f16)
        self.act = ctx.alloc(batch * c.mlp * f16)
        self.logits = ctx.alloc(batch * c.vocab * 4)
        self.embedding = ctx.to_device(weights["embedding"])
        self.ln_f = ctx.to_device(weights["ln_f"])
        self.lm_head = ctx.prepack_w8a16(*weights["lm_head"])
        self.geometry = rt.PagedAttnArgs(batch, c.q_heads, c.kv_heads, c.head_dim, c.block_size, max_blocks_per_seq, num_blocks,
                                         float(c.head_dim ** -0.5), rt.DT_F16)
        self.attn_args = rt.PagedAttnArgs(batch, c.q_heads, c.kv_heads, c.head_dim, c.block_size, max_blocks_per_seq, num_blocks,
                                          float(c.head_dim ** -0.5), rt.DT_F16, 1)
        self.layers = []
        assert batch % lanes == 0, "lanes split the batch evenly"
        self.lanes = lanes
        bl = batch // lanes
        lane_args = rt.PagedAttnArgs(bl, c.q_heads, c.kv_heads, c.head_dim, c.block_size, max_blocks_per_seq, num_blocks,
                                     float(c.head_dim ** -0.5), rt.DT_F16, 1)
        lane_geometry = rt.PagedAttnArgs(bl, c.q_heads, c.kv_heads, c.head_dim, c.block_size, max_blocks_per_seq, num_blocks,
                                         float(c.head_dim ** -0.5), rt.DT_F16)
        for lw in weights["layers"]:
            self.layers.append({"ln1": ctx.to_device(lw["ln1"]), "ln2": ctx.to_device(lw["ln2"]),
                                "qkv": ctx.prepack_w8a16(lw["qkv"][0], lw["qkv"][1], lw["qkv_bias"]), "o": ctx.prepack_w8a16(*lw["o"]),
                                "gate_up": ctx.prepack_w8a16(*lw["gate_up"]), "down": ctx.prepack_w8a16(*lw["down"])})
        for li, L in enumerate(self.layers):
            L["k"] = ctx.to_device(np.ascontiguousarray(k_caches[li], np.float16))
            L["v"] = ctx.to_device(np.ascontiguousarray(v_caches[li], np.float16))
        fn = Function(ctx)
        # feedback: the arg-max lands in the token buffer the next step's embedding reads (greedy generation
        # without a host round trip); otherwise the caller feeds every step's tokens
        self.feedback = feedback
        # lanes > 1: the sequences are split into that many equal ranges and the whole step is recorded once per range,
        # each on a lane of its own; a captured step replays the lanes side by side, so the launch and memory latency
        # of one range's short kernels is covered by the other ranges' kernels.  Every range reads the same weights and
        # owns its rows of every buffer, so the result is that of lanes == 1 row for row, up to the order in which a
        # product's or an attention's partial sums are added (kernels pick their splits by the number of rows).
        for lane in range(lanes):
            if lanes > 1:
                fn.set_lane(lane)

            def R(buf, row_bytes):                  # this lane's rows of a [batch, ...] buffer
                return buf if lanes == 1 else buf.view(lane * bl * row_bytes, bl * row_bytes)

            tokens, next_tokens, ctx_lens = R(self.tokens, 4), R(self.next_tokens, 4), R(self.ctx_lens, 4)
            block_table = R(self.block_table, max_blocks_per_seq * 4)
            xs = [R(self.x[0], c.hidden * f16), R(self.x[1], c.hidden * f16)]
            norm, qkv, q = R(self.norm, c.hidden * f16), R(self.qkv, (qd + 2 * kvd) * f16), R(self.q, qd * f16)
            att, act, logits = R(self.att, qd * f16), R(self.act, c.mlp * f16), R(self.logits, c.vocab * 4)
            fn.add_embedding_f16(self.embedding, tokens, xs[0], bl, c.hidden, c.vocab)
            for L in self.layers:
                x, h = xs[0], xs[1]
                # the three normalisations run inside the products that consume them (fuse_norm), or as operators of their own
                if fuse_norm:
                    # (and the rotary embedding and the cache append in the projection's epilogue)
                    fn.add_w8a16_gemm_rope_kv_append(x, L["ln1"], c.rms_eps, L["qkv"], qkv, q, L["k"], L["v"], block_table, ctx_lens,
                                                     lane_geometry, c.rope_theta)
                else:
                    fn.add_rmsnorm_f16(x, L["ln1"], norm, bl, c.hidden, c.rms_eps)
                    fn.add_w8a16_gemm(norm, L["qkv"], qkv, bl)
                    fn.add_rope_kv_append(qkv, q, L["k"], L["v"], block_table, ctx_lens, lane_geometry, c.rope_theta)
                # the appended token takes part in its own attention (lengths + 1); the lengths themselves advance
                # once, at the end of the step
                fn.add_paged_attention_decode(q, L["k"], L["v"], block_table, ctx_lens, att, lane_args)
                fn.add_w8a16_gemm(att, L["o"], h, bl, residual=x)
                if fuse_norm:
                    fn.add_rmsnorm_w8a16_gemm(h, L["ln2"], c.rms_eps, L["gate_up"], act, bl, mode=rt.GEMM_SWIGLU)
                else:
                    fn.add_rmsnorm_f16(h, L["ln2"], norm, bl, c.hidden, c.rms_eps)
                    fn.add_w8a16_gemm(norm, L["gate_up"], act, bl, mode=rt.GEMM_SWIGLU)
                fn.add_w8a16_gemm(act, L["down"], x, bl, residual=h)
            if lanes > 1 and lane + 1 < lanes:
                continue
            # The vocabulary head reads its 136 MB of weights once for however many rows: behind the join of the lanes it
            # runs once over the whole batch (as do the two small operators after it), not once per lane.
            if lanes > 1:
                fn.set_lane(Function.LANE_JOINED)
                tokens, next_tokens, ctx_lens, norm, logits, bl_ = self.tokens, self.next_tokens, self.ctx_lens, self.norm, self.logits, batch
                xs = [self.x[0], self.x[1]]
            else:
                bl_ = bl
            if fuse_norm:
                fn.add_rmsnorm_w8a16_gemm(xs[0], self.ln_f, c.rms_eps, self.lm_head, logits, bl_, out_dtype=rt.DT_F32)
            else:
                fn.add_rmsnorm_f16(xs[0], self.ln_f, norm, bl_, c.hidden, c.rms_eps)
                fn.add_w8a16_gemm(norm, self.lm_head, logits, bl_, out_dtype=rt.DT_F32)
            fn.add_argmax_f32(logits, tokens if feedback else next_tokens, bl_, c.vocab)
            fn.add_add_i32(ctx_lens, bl_, 1)   # the step is complete: the caches hold one more token
        self.fn = fn
        # nothing to warm up: recording the attention operators has already sized their workspace
        if capture_graph:
            fn.capture()

    def set_tokens(self, ids: np.ndarray):
        self.tokens.upload(np.ascontiguousarray(ids, np.int32))

    def step(self):
        """One decode step for the whole batch (asynchronous)."""
        self.fn.invoke()

    def result(self) -> np.ndarray:
        return (self.tokens if self.feedback else self.next_tokens).download((self.batch,), np.int32)

    def weight_bytes(self) -> int:
        c = self.cfg
        qd, kvd = c.q_heads * c.head_dim, c.kv_heads * c.head_dim
        per_layer = (qd + 2 * kvd) * c.hidden + c.hidden * qd + 2 * c.mlp * c.hidden + c.hidden * c.mlp
        return c.layers * per_layer + c.vocab * c.hidden
