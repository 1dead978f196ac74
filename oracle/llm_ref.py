"""float64 restatement of the decode-step operators and of the whole decode step.
TEST INFRASTRUCTURE ONLY.  No counterpart in the reference tree (parity unpinned by the reference):
each function is the textbook definition; tests/test_llm_ref.py pins them against closed forms and
invariants that a swapped operand, a wrong pairing or a misplaced epsilon would break (rotary embedding:
identity at position 0, norms kept, inner products that depend on the position difference only, the
(i, i + d/2) pairing on one-hot vectors; RMS norm: constant rows, scale invariance, epsilon under the
root; SwiGLU: gate / up order; the W8A16 product on small integers; one decode step of a one-layer model
against a hand calculation)."""
from __future__ import annotations

import numpy as np


def w8a16_linear(a_f16, q_i8, scale_f32, bias_f32=None, acc=np.float64):
    """out[m, n] = scale[n] * sum_k a[m, k] * q[n, k] (+ bias[n]); `acc`: the type the sums are formed in."""
    y = (a_f16.astype(acc) @ q_i8.astype(acc).T).astype(np.float64) * scale_f32.astype(np.float64)[None, :]
    return y if bias_f32 is None else y + bias_f32.astype(np.float64)[None, :]


def rmsnorm(x, w, eps):
    x = x.astype(np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * w.astype(np.float64)


def silu(x):
    return x / (1.0 + np.exp(-x))


def rope(x, pos, theta):
    """x [..., d] with rotate-half pairing (i, i + d/2); angle pos * theta^(-2i/d)."""
    d = x.shape[-1]
    half = d // 2
    inv = theta ** (-2.0 * np.arange(half, dtype=np.float64) / d)
    ang = pos * inv
    c, s = np.cos(ang), np.sin(ang)
    x0, x1 = x[..., :half].astype(np.float64), x[..., half:].astype(np.float64)
    return np.concatenate([x0 * c - x1 * s, x1 * c + x0 * s], axis=-1)


def f16(x):
    """Round to fp16 and back: the storage precision of every activation tensor."""
    return np.asarray(x, np.float64).astype(np.float16).astype(np.float64)


def decode_step(cfg, weights, tokens, block_table, ctx_lens, k_caches, v_caches, acc=np.float64):
    """One greedy decode step in float64 with fp16 rounding wherever the device stores fp16.
    k_caches / v_caches (lists of numpy fp16 arrays in the paged layouts, K [blocks, Hkv, block, d],
    V [blocks, Hkv, d, block]) are updated in place.  Returns (next tokens, logits float64).
    acc=np.float32 forms the sums of the weight products in float32 instead (numpy's blocked order): a second valid
    evaluation, whose distance from the float64 one shows how far fp16 storage lets two correct implementations drift
    apart over the layers (a sum that differs in its last bits can round to the other fp16 neighbour)."""
    c = cfg
    B = len(tokens)
    G = c.q_heads // c.kv_heads
    x = weights["embedding"][np.asarray(tokens)].astype(np.float64)
    for li, lw in enumerate(weights["layers"]):
        n = f16(rmsnorm(x, lw["ln1"], c.rms_eps))
        qkv = f16(w8a16_linear(n.astype(np.float16), lw["qkv"][0], lw["qkv"][1], lw["qkv_bias"], acc=acc))
        att = np.zeros((B, c.q_heads * c.head_dim))
        for b in range(B):
            pos = int(ctx_lens[b])
            heads = qkv[b].reshape(c.q_heads + 2 * c.kv_heads, c.head_dim)
            q = f16(rope(heads[:c.q_heads], pos, c.rope_theta))
            k_new = f16(rope(heads[c.q_heads:c.q_heads + c.kv_heads], pos, c.rope_theta))
            v_new = heads[c.q_heads + c.kv_heads:]
            pb, off = block_table[b, pos // c.block_size], pos % c.block_size
            k_caches[li][pb, :, off, :] = k_new.astype(np.float16)
            v_caches[li][pb, :, :, off] = v_new.astype(np.float16)
            n_tok = pos + 1
            blocks = block_table[b, :(n_tok + c.block_size - 1) // c.block_size]
            K = k_caches[li][blocks].astype(np.float64).transpose(1, 0, 2, 3).reshape(c.kv_heads, -1, c.head_dim)[:, :n_tok]
            V = v_caches[li][blocks].astype(np.float64).transpose(1, 0, 3, 2).reshape(c.kv_heads, -1, c.head_dim)[:, :n_tok]
            for h in range(c.q_heads):
                s = K[h // G] @ q[h] * c.head_dim ** -0.5
                p = np.exp(s - s.max())
                att[b, h * c.head_dim:(h + 1) * c.head_dim] = (p / p.sum()) @ V[h // G]
        att = f16(att)
        h_ = f16(x + w8a16_linear(att.astype(np.float16), *lw["o"], acc=acc))
        n2 = f16(rmsnorm(h_, lw["ln2"], c.rms_eps))
        gu = w8a16_linear(n2.astype(np.float16), *lw["gate_up"], acc=acc)
        act = f16(silu(gu[:, :c.mlp]) * gu[:, c.mlp:])
        x = f16(h_ + w8a16_linear(act.astype(np.float16), *lw["down"], acc=acc))
    nf = f16(rmsnorm(x, weights["ln_f"], c.rms_eps))
    logits = w8a16_linear(nf.astype(np.float16), *weights["lm_head"], acc=acc)
    return logits.argmax(axis=-1).astype(np.int32), logits
