"""GPU parity of the decode-step operators and of a whole decode step against float64 restatements.
The reference tree has no counterpart (parity unpinned by the reference); tolerance 1e-3 relative to the
largest magnitude of each output row, as for attention."""
import numpy as np
import pytest

from nncase_amd import llm
from nncase_amd import runtime as rt
from oracle import llm_ref as R

pytestmark = pytest.mark.gpu
RTOL = 1e-3


def close(got, want, rtol=RTOL, atol=1e-3):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    tol = rtol * np.abs(want).max(axis=-1, keepdims=True) + atol
    assert (np.abs(got - want) <= tol).all(), f"max err {np.abs(got - want).max()} (max |want| {np.abs(want).max()})"


@pytest.mark.parametrize("m,k,n", [(1, 64, 16), (32, 896, 1152), (7, 128, 48), (33, 192, 64), (64, 4864, 896), (16, 896, 2048),
                                   # many output tiles: a tile per wave, the token rows shared through LDS (1, 2 and 4 row tiles)
                                   (32, 896, 20480), (5, 128, 16400), (64, 256, 16384), (33, 192, 16384)])
@pytest.mark.parametrize("out32", [False, True])
def test_w8a16_gemm(hip_ctx, m, k, n, out32):
    rng = np.random.default_rng(m + k + n)
    a = rng.standard_normal((m, k)).astype(np.float16)
    q = rng.integers(-127, 128, (n, k), dtype=np.int8)
    q[0, :] = -128 if k > 64 else q[0, :]                       # the full int8 range
    scale = rng.uniform(0.001, 0.01, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float16)
    w = hip_ctx.prepack_w8a16(q, scale, bias)
    da, dres = hip_ctx.to_device(a), hip_ctx.to_device(res)
    dt = np.float32 if out32 else np.float16
    out = hip_ctx.alloc(m * n * np.dtype(dt).itemsize)
    hip_ctx.w8a16_gemm(da, w, out, m, out_dtype=rt.DT_F32 if out32 else rt.DT_F16)
    close(out.download((m, n), dt), R.w8a16_linear(a, q, scale, bias))
    hip_ctx.w8a16_gemm(da, w, out, m, residual=dres, out_dtype=rt.DT_F32 if out32 else rt.DT_F16)
    close(out.download((m, n), dt), R.w8a16_linear(a, q, scale, bias) + res.astype(np.float64))
    # exact case: small integers survive fp16 and the fp32 accumulator exactly
    ai = rng.integers(-4, 5, (m, k)).astype(np.float16)
    w1 = hip_ctx.prepack_w8a16(q, np.ones(n, np.float32))
    o32 = hip_ctx.alloc(m * n * 4)
    hip_ctx.w8a16_gemm(hip_ctx.to_device(ai), w1, o32, m, out_dtype=rt.DT_F32)
    assert np.array_equal(o32.download((m, n), np.float32), (ai.astype(np.int64) @ q.astype(np.int64).T).astype(np.float32))


def test_w8a16_swiglu(hip_ctx):
    rng = np.random.default_rng(3)
    m, k, mlp = 32, 896, 4864
    a = rng.standard_normal((m, k)).astype(np.float16)
    q = rng.integers(-127, 128, (2 * mlp, k), dtype=np.int8)
    scale = rng.uniform(0.0005, 0.002, 2 * mlp).astype(np.float32)
    w = hip_ctx.prepack_w8a16(q, scale)
    out = hip_ctx.alloc(m * mlp * 2)
    hip_ctx.w8a16_gemm(hip_ctx.to_device(a), w, out, m, mode=rt.GEMM_SWIGLU)
    gu = R.w8a16_linear(a, q, scale)
    close(out.download((m, mlp), np.float16), R.silu(gu[:, :mlp]) * gu[:, mlp:])


@pytest.mark.parametrize("m,k,n,mode", [(1, 64, 16, "plain"), (32, 896, 1152, "plain"), (7, 128, 48, "residual"), (33, 192, 64, "plain"),
                                        (32, 896, 9728, "swiglu"), (64, 896, 2048, "f32"), (32, 896, 151936 // 16 * 16, "f32")])
def test_rmsnorm_fused_into_gemm_equals_the_two_operators(hip_ctx, m, k, n, mode):
    """The product that normalises its own rows writes, bit for bit, what rmsnorm_f16 followed by w8a16_gemm writes:
    split and per-wave reductions, SwiGLU, residual, fp32 output, the vocabulary head."""
    rng = np.random.default_rng(m * 3 + k + n)
    x = (rng.standard_normal((m, k)) * rng.uniform(0.1, 4.0, (m, 1))).astype(np.float16)
    lnw = (1.0 + 0.2 * rng.standard_normal(k)).astype(np.float16)
    q = rng.integers(-127, 128, (n, k), dtype=np.int8)
    scale = rng.uniform(0.001, 0.01, n).astype(np.float32)
    w = hip_ctx.prepack_w8a16(q, scale, rng.standard_normal(n).astype(np.float32))
    gemm_mode = rt.GEMM_SWIGLU if mode == "swiglu" else rt.GEMM_PLAIN
    n_out = n // 2 if mode == "swiglu" else n
    dt, code = (np.float32, rt.DT_F32) if mode == "f32" else (np.float16, rt.DT_F16)
    res = hip_ctx.to_device(rng.standard_normal((m, n_out)).astype(np.float16)) if mode == "residual" else None
    dx, dln = hip_ctx.to_device(x), hip_ctx.to_device(lnw)
    norm = hip_ctx.alloc(m * k * 2)
    two, one = hip_ctx.alloc(m * n_out * np.dtype(dt).itemsize), hip_ctx.alloc(m * n_out * np.dtype(dt).itemsize)
    hip_ctx.rmsnorm_f16(dx, dln, norm, m, k, 1e-6)
    hip_ctx.w8a16_gemm(norm, w, two, m, mode=gemm_mode, residual=res, out_dtype=code)
    hip_ctx.rmsnorm_w8a16_gemm(dx, dln, 1e-6, w, one, m, mode=gemm_mode, residual=res, out_dtype=code)
    a, b = two.download((m, n_out), dt), one.download((m, n_out), dt)
    assert np.array_equal(a.view(np.uint32 if mode == "f32" else np.uint16), b.view(np.uint32 if mode == "f32" else np.uint16))
    assert np.isfinite(a.astype(np.float64)).all() and np.abs(a.astype(np.float64)).max() > 0


def test_decoder_with_fused_normalisation_equals_separate_operators(hip_ctx):
    cfg = llm.DecoderConfig(layers=2, hidden=256, q_heads=4, kv_heads=2, head_dim=64, mlp=512, vocab=2048)
    rng = np.random.default_rng(5)
    weights = llm.random_weights(cfg, seed=4)
    batch = 5
    max_blocks, lens, bt, kcs, vcs = make_state(cfg, rng, batch, 70)
    tokens = rng.integers(0, cfg.vocab, batch).astype(np.int32)
    outs = []
    for fuse in (True, False):
        dec = llm.HipDecoder(hip_ctx, cfg, weights, batch, max_blocks, bt, lens.copy(), [k.copy() for k in kcs], [v.copy() for v in vcs],
                             capture_graph=True, fuse_norm=fuse)
        assert len(dec.fn) == (3 + cfg.layers * 5 + 1 if fuse else 3 + cfg.layers * 8 + 2)
        tk = tokens
        logs = []
        for _ in range(2):
            dec.set_tokens(tk)
            dec.step()
            hip_ctx.sync()
            tk = dec.result()
            logs.append(dec.logits.download((batch, cfg.vocab), np.float32))
        outs.append((tk, logs))
    assert np.array_equal(outs[0][0], outs[1][0])
    for a, b in zip(outs[0][1], outs[1][1]):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_w8a16_error_paths(hip_ctx):
    q = np.zeros((16, 64), np.int8)
    with pytest.raises(rt.HipError) as e:
        hip_ctx.prepack_w8a16(np.zeros((16, 48), np.int8), np.ones(16, np.float32))       # k not a multiple of 64
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH
    with pytest.raises(rt.HipError):
        hip_ctx.prepack_w8a16(np.zeros((10, 64), np.int8), np.ones(10, np.float32))       # n not a multiple of 16
    w = hip_ctx.prepack_w8a16(q, np.ones(16, np.float32))
    buf = hip_ctx.alloc(65 * 64 * 2)
    with pytest.raises(rt.HipError):
        hip_ctx.w8a16_gemm(buf, w, buf, 65)                                                 # more than 64 token rows


@pytest.mark.parametrize("rows,hidden", [(1, 64), (32, 896), (5, 1000), (64, 4864)])
def test_rmsnorm(hip_ctx, rows, hidden):
    rng = np.random.default_rng(rows + hidden)
    x = (rng.standard_normal((rows, hidden)) * 3).astype(np.float16)
    w = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    out = hip_ctx.alloc(rows * hidden * 2)
    hip_ctx.rmsnorm_f16(hip_ctx.to_device(x), hip_ctx.to_device(w), out, rows, hidden, 1e-6)
    close(out.download((rows, hidden), np.float16), R.rmsnorm(x, w, 1e-6))


def test_rope_and_kv_append(hip_ctx):
    rng = np.random.default_rng(9)
    B, hq, hkv, d, blk, max_blocks = 5, 14, 2, 64, 16, 8
    nb = B * max_blocks + 2
    lens = np.array([0, 1, 15, 16, 100], np.int32)
    bt = rng.permutation(nb)[:B * max_blocks].reshape(B, max_blocks).astype(np.int32)
    qkv = rng.standard_normal((B, (hq + 2 * hkv) * d)).astype(np.float16)
    kc = rng.standard_normal((nb, hkv, blk, d)).astype(np.float16)
    vc = rng.standard_normal((nb, hkv, d, blk)).astype(np.float16)
    dk, dv = hip_ctx.to_device(kc), hip_ctx.to_device(vc)
    dq = hip_ctx.alloc(B * hq * d * 2)
    geo = rt.PagedAttnArgs(B, hq, hkv, d, blk, max_blocks, nb, 0.125, rt.DT_F16)
    hip_ctx.rope_kv_append(hip_ctx.to_device(qkv), dq, dk, dv, hip_ctx.to_device(bt), hip_ctx.to_device(lens), geo, 1e6)
    q = dq.download((B, hq, d), np.float16)
    k2, v2 = dk.download(kc.shape, np.float16), dv.download(vc.shape, np.float16)
    want_k, want_v = kc.copy(), vc.copy()
    for b in range(B):
        heads = qkv[b].reshape(hq + 2 * hkv, d)
        close(q[b], R.rope(heads[:hq], int(lens[b]), 1e6), atol=2e-3)
        pb, off = bt[b, lens[b] // blk], lens[b] % blk
        close(k2[pb, :, off, :], R.rope(heads[hq:hq + hkv], int(lens[b]), 1e6), atol=2e-3)
        assert np.array_equal(v2[pb, :, :, off], heads[hq + hkv:])        # v is copied, not rotated
        want_k[pb, :, off, :] = k2[pb, :, off, :]
        want_v[pb, :, :, off] = v2[pb, :, :, off]
    assert np.array_equal(k2, want_k) and np.array_equal(v2, want_v)       # nothing else in the caches moved
    assert np.array_equal(q[0], qkv[0].reshape(-1, d)[:hq])                # position 0: rotation by zero


@pytest.mark.parametrize("B,k,norm", [(32, 896, True), (16, 896, True), (5, 256, False), (32, 1024, True), (7, 1536, True), (40, 896, True)])
def test_projection_that_rotates_and_appends_equals_the_two_operators(hip_ctx, B, k, norm):
    """nncase_hip_w8a16_gemm_rope_kv_append against the projection into fp16 followed by nncase_hip_rope_kv_append: the same
    bytes in the query buffer and in both caches (the last two cases take the two-launch form inside the entry point: a
    reduction too long for the rows to be normalised in one block, more than 32 rows)."""
    rng = np.random.default_rng(B + k)
    hq, hkv, d, blk, max_blocks = 14, 2, 64, 16, 8
    n = (hq + 2 * hkv) * d
    nb = B * max_blocks + 2
    lens = rng.integers(0, max_blocks * blk, B).astype(np.int32)
    lens[0] = 0
    bt = rng.permutation(nb)[:B * max_blocks].reshape(B, max_blocks).astype(np.int32)
    x = (rng.standard_normal((B, k)) * 0.7).astype(np.float16)
    ln = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float16)
    wq, sc = llm.quantize_rows((rng.standard_normal((n, k)) * k ** -0.5).astype(np.float32))
    bias = (rng.standard_normal(n) * 0.1).astype(np.float32)
    w = hip_ctx.prepack_w8a16(wq, sc, bias)
    kc = rng.standard_normal((nb, hkv, blk, d)).astype(np.float16)
    vc = rng.standard_normal((nb, hkv, d, blk)).astype(np.float16)
    geo = rt.PagedAttnArgs(B, hq, hkv, d, blk, max_blocks, nb, 0.125, rt.DT_F16)
    dx, dln, dbt, dlens = hip_ctx.to_device(x), hip_ctx.to_device(ln), hip_ctx.to_device(bt), hip_ctx.to_device(lens)
    got = []
    for fused in (True, False):
        dk, dv = hip_ctx.to_device(kc), hip_ctx.to_device(vc)
        dq, dqkv = hip_ctx.alloc(B * hq * d * 2), hip_ctx.alloc(B * n * 2)
        dq.fill(0)
        if fused:
            hip_ctx.w8a16_gemm_rope_kv_append(dx, dln if norm else None, 1e-6, w, dqkv, dq, dk, dv, dbt, dlens, geo, 1e6)
        else:
            if norm:
                hip_ctx.rmsnorm_w8a16_gemm(dx, dln, 1e-6, w, dqkv, B)
            else:
                hip_ctx.w8a16_gemm(dx, w, dqkv, B)
            hip_ctx.rope_kv_append(dqkv, dq, dk, dv, dbt, dlens, geo, 1e6)
        got.append((dq.download((B, hq, d), np.uint16), dk.download(kc.shape, np.uint16), dv.download(vc.shape, np.uint16)))
    for a, b in zip(*got):
        assert np.array_equal(a, b)
    assert not np.array_equal(got[0][1], kc.view(np.uint16))     # something was appended


def test_kv_append_ignores_lengths_outside_the_table(hip_ctx):
    """A negative or over-long context length appends nothing (the query is still rotated): the caches keep every byte."""
    rng = np.random.default_rng(10)
    B, hq, hkv, d, blk, max_blocks = 3, 4, 2, 64, 16, 2
    nb = B * max_blocks
    lens = np.array([-5, max_blocks * blk, 7], np.int32)
    bt = rng.permutation(nb).reshape(B, max_blocks).astype(np.int32)
    qkv = rng.standard_normal((B, (hq + 2 * hkv) * d)).astype(np.float16)
    kc = rng.standard_normal((nb, hkv, blk, d)).astype(np.float16)
    vc = rng.standard_normal((nb, hkv, d, blk)).astype(np.float16)
    dk, dv = hip_ctx.to_device(kc), hip_ctx.to_device(vc)
    dq = hip_ctx.alloc(B * hq * d * 2)
    geo = rt.PagedAttnArgs(B, hq, hkv, d, blk, max_blocks, nb, 0.125, rt.DT_F16)
    hip_ctx.rope_kv_append(hip_ctx.to_device(qkv), dq, dk, dv, hip_ctx.to_device(bt), hip_ctx.to_device(lens), geo, 1e6)
    k2, v2 = dk.download(kc.shape, np.float16), dv.download(vc.shape, np.float16)
    pb = bt[2, 0]
    want_k, want_v = kc.copy(), vc.copy()
    want_k[pb, :, 7, :], want_v[pb, :, :, 7] = k2[pb, :, 7, :], v2[pb, :, :, 7]
    assert np.array_equal(k2, want_k) and np.array_equal(v2, want_v)       # only sequence 2 appended
    assert np.array_equal(v2[pb, :, :, 7], qkv[2].reshape(-1, d)[hq + hkv:])


def test_argmax_embedding_and_counter(hip_ctx):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((7, 151936)).astype(np.float32)
    x[2, 777] = x[2, 5] = 50.0                                   # a tie: the lower index wins
    x[3, :] = -np.inf
    x[4, 9] = x[4, 8] = 60.0                                     # ties inside one 16-byte load,
    x[5, 4136] = x[5, 40] = 70.0                                 # in two loads of one thread's batch,
    x[6, 151935] = x[6, 40 + 4 * 1024 * 8] = 80.0                # and in two batches of one thread
    x[0, 100] = np.nan                                           # not a candidate
    out = hip_ctx.alloc(7 * 4)
    hip_ctx.argmax_f32(hip_ctx.to_device(x), out, 7, x.shape[1])
    got = out.download((7,), np.int32)
    want = np.where(np.isnan(x), -np.inf, x).argmax(axis=1)
    assert np.array_equal(got, want) and got[2] == 5 and got[3] == 0 and got[4] == 8 and got[5] == 40 and got[6] == 40 + 4 * 1024 * 8
    y = rng.standard_normal((3, 1001)).astype(np.float32)       # rows that are not whole 16-byte vectors
    y[1, 1000] = y[1, 3] = 9.0
    hip_ctx.argmax_f32(hip_ctx.to_device(y), out, 3, 1001)
    assert np.array_equal(out.download((3,), np.int32), y.argmax(axis=1))
    table = rng.standard_normal((1000, 96)).astype(np.float16)
    ids = np.array([0, 999, 5, 5, 123], np.int32)
    o = hip_ctx.alloc(5 * 96 * 2)
    hip_ctx.embedding_f16(hip_ctx.to_device(table), hip_ctx.to_device(ids), o, 5, 96, 1000)
    assert np.array_equal(o.download((5, 96), np.float16), table[ids])
    c = hip_ctx.to_device(np.arange(10, dtype=np.int32))
    hip_ctx.add_i32(c, 10, 3)
    hip_ctx.add_i32(c, 10, -1)
    assert np.array_equal(c.download((10,), np.int32), np.arange(10) + 2)


def make_state(cfg, rng, batch, max_ctx):
    max_blocks = -(-(max_ctx + 8) // cfg.block_size)
    nb = batch * max_blocks + 1
    lens = rng.integers(max_ctx // 2, max_ctx + 1, batch).astype(np.int32)
    bt = rng.permutation(nb)[:batch * max_blocks].reshape(batch, max_blocks).astype(np.int32)
    kcs = [rng.standard_normal((nb, cfg.kv_heads, cfg.block_size, cfg.head_dim)).astype(np.float16) for _ in range(cfg.layers)]
    vcs = [rng.standard_normal((nb, cfg.kv_heads, cfg.head_dim, cfg.block_size)).astype(np.float16) for _ in range(cfg.layers)]
    return max_blocks, lens, bt, kcs, vcs


@pytest.mark.parametrize("capture,lanes", [(False, 1), (True, 1), (True, 2), (False, 3)])
def test_decode_steps_small_model(hip_ctx, capture, lanes):
    """Three greedy steps of a 3-layer model (Qwen2 head geometry, reduced widths) against the float64 step:
    logits to 1e-3, the same tokens whenever the float64 top-2 margin exceeds the tolerance, and the caches
    the steps leave behind.  lanes > 1: the six sequences recorded as that many independent chains (each with
    its own rows of every buffer and its own attention scratch), replayed side by side when captured."""
    cfg = llm.DecoderConfig(layers=3, hidden=256, q_heads=4, kv_heads=2, head_dim=64, mlp=512, vocab=2048)
    rng = np.random.default_rng(12)
    weights = llm.random_weights(cfg, seed=3)
    batch = 6
    max_blocks, lens, bt, kcs, vcs = make_state(cfg, rng, batch, 90)
    dec = llm.HipDecoder(hip_ctx, cfg, weights, batch, max_blocks, bt, lens, kcs, vcs, capture_graph=capture, lanes=lanes)
    ref_k, ref_v = [k.copy() for k in kcs], [v.copy() for v in vcs]
    ref_lens = lens.copy()
    tokens = rng.integers(0, cfg.vocab, batch).astype(np.int32)
    for step in range(3):
        dec.set_tokens(tokens)
        dec.step()
        hip_ctx.sync()
        got = dec.result()
        logits = dec.logits.download((batch, cfg.vocab), np.float32)
        want_tok, want_logits = R.decode_step(cfg, weights, tokens, bt, ref_lens, ref_k, ref_v)
        close(logits, want_logits, rtol=2e-3, atol=2e-3)
        top2 = np.sort(want_logits, axis=1)[:, -2:]
        sure = (top2[:, 1] - top2[:, 0]) > 4e-3 * np.abs(want_logits).max(axis=1)
        assert sure.any() and np.array_equal(got[sure], want_tok[sure])
        ref_lens += 1
        assert np.array_equal(dec.ctx_lens.download((batch,), np.int32), ref_lens)
        tokens = want_tok
    for li in range(cfg.layers):   # the appended K / V rows
        close(dec.layers[li]["k"].download(kcs[li].shape, np.float16).reshape(-1, cfg.head_dim), ref_k[li].reshape(-1, cfg.head_dim), atol=4e-3)
        close(dec.layers[li]["v"].download(vcs[li].shape, np.float16).reshape(-1, cfg.block_size), ref_v[li].reshape(-1, cfg.block_size), atol=4e-3)


@pytest.mark.parametrize("lanes", [1, 2])
def test_decode_step_at_the_benchmark_shape(hip_ctx, lanes):
    """One greedy step of the decode benchmark's own model and state (24 layers, hidden 896, 14 query / 2 KV heads of 64,
    MLP 4864, vocabulary 151 936, batch 32, context lengths uniform in [512, 4096], one random cache image per layer) against
    the float64 step.  Twenty-four layers of fp16 storage amplify last-bit differences of the sums (a sum that differs in
    its last bits can round to the other fp16 neighbour, 1e-3 apart, and the layers behind it see that): the float64 step
    evaluated a second time with float32 sums (numpy's own blocked order) already drifts from itself by some 2e-3 of a
    row's largest logit.  The device is held to that yardstick: every logit within 1e-3 of the row maximum or 1.5 times the
    drift of the float32 evaluation, whichever is larger; the same next token wherever the float64 top-2 margin exceeds
    twice that; the appended K / V rows of the first and last layer, by the same yardstick; the advanced lengths."""
    cfg = llm.DecoderConfig()
    batch, max_ctx = 32, 4096
    rng = np.random.default_rng(5)
    weights = llm.random_weights(cfg, seed=5)
    lens = rng.integers(512, max_ctx + 1, batch).astype(np.int32)
    max_blocks = (max_ctx + 64) // cfg.block_size + 1
    nblocks = batch * max_blocks
    bt = rng.permutation(nblocks).reshape(batch, max_blocks).astype(np.int32)
    kc = rng.standard_normal((nblocks, cfg.kv_heads, cfg.block_size, cfg.head_dim), dtype=np.float32).astype(np.float16)
    vc = rng.standard_normal((nblocks, cfg.kv_heads, cfg.head_dim, cfg.block_size), dtype=np.float32).astype(np.float16)
    dec = llm.HipDecoder(hip_ctx, cfg, weights, batch, max_blocks, bt, lens, [kc] * cfg.layers, [vc] * cfg.layers, capture_graph=True, lanes=lanes)
    tokens = rng.integers(0, cfg.vocab, batch).astype(np.int32)
    dec.set_tokens(tokens)
    dec.step()
    hip_ctx.sync()
    got = dec.result()
    logits = dec.logits.download((batch, cfg.vocab), np.float32).astype(np.float64)
    ref_k, ref_v = [kc.copy() for _ in range(cfg.layers)], [vc.copy() for _ in range(cfg.layers)]
    want_tok, want_logits = R.decode_step(cfg, weights, tokens, bt, lens.copy(), ref_k, ref_v)
    drift_k, drift_v = [kc.copy() for _ in range(cfg.layers)], [vc.copy() for _ in range(cfg.layers)]
    _, drift_logits = R.decode_step(cfg, weights, tokens, bt, lens.copy(), drift_k, drift_v, acc=np.float32)
    scale = np.abs(want_logits).max(axis=1, keepdims=True)
    err = np.abs(logits - want_logits) / scale
    drift = np.abs(drift_logits - want_logits) / scale
    tol = max(1e-3, 1.5 * float(drift.max()))
    print(f"decode step at the benchmark shape: largest logit error {err.max():.2e} of the row maximum (mean {err.mean():.2e}); "
          f"float32-sum evaluation of the reference: {drift.max():.2e} (mean {drift.mean():.2e})")
    assert err.max() <= tol, f"logits differ by {err.max():.3e} of the row maximum (tolerance {tol:.3e})"
    assert err.mean() <= 5e-4
    top2 = np.sort(want_logits, axis=1)[:, -2:]
    sure = (top2[:, 1] - top2[:, 0]) > 2 * tol * scale[:, 0]
    assert sure.sum() >= batch // 2 and np.array_equal(got[sure], want_tok[sure])
    assert np.array_equal(dec.ctx_lens.download((batch,), np.int32), lens + 1)
    for li in (0, cfg.layers - 1):
        k_dev = dec.layers[li]["k"].download(kc.shape, np.float16).astype(np.float64)
        v_dev = dec.layers[li]["v"].download(vc.shape, np.float16).astype(np.float64)
        for name, dev, ref, other in (("k", k_dev, ref_k[li].astype(np.float64), drift_k[li].astype(np.float64)),
                                      ("v", v_dev, ref_v[li].astype(np.float64), drift_v[li].astype(np.float64))):
            d = np.abs(dev - ref)
            # fp16 storage: one unit in the last place of the stored value, on top of 1e-3 of the row's scale -- or, behind
            # 23 layers, 1.5 times what the float32-sum evaluation's own appended rows drift by (the logits' yardstick)
            bound = max(1e-3 * max(1.0, float(np.abs(ref).max())) + 4e-3, 1.5 * float(np.abs(other - ref).max()))
            print(f"layer {li} {name} cache: largest difference {d.max():.2e}, float32-sum evaluation {np.abs(other - ref).max():.2e}, bound {bound:.2e}")
            assert d.max() <= bound, f"layer {li} {name} cache differs by {d.max():.3e} (bound {bound:.3e})"
