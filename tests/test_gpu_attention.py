"""GPU parity: paged-attention decode vs the float64 brute-force oracle.  The reference tree
has no attention operator (parity unpinned by the reference); tolerance is the north-star
1e-3 relative error, taken against the largest magnitude of each output row."""
import numpy as np
import pytest

from nncase_amd import kernels as K
from oracle import oracle as O

pytestmark = pytest.mark.gpu
RTOL = 1e-3


def make_case(rng, bsz, hq, hkv, d, blk, max_ctx, ctx_lens=None):
    max_blocks = -(-max_ctx // blk)
    nb = bsz * max_blocks + 3
    q = rng.standard_normal((bsz, hq, d)).astype(np.float16)
    kc = rng.standard_normal((nb, hkv, blk, d)).astype(np.float16)
    vc = rng.standard_normal((nb, hkv, blk, d)).astype(np.float16)
    perm = rng.permutation(nb)[: bsz * max_blocks].reshape(bsz, max_blocks).astype(np.int32)  # scattered physical blocks
    cl = np.asarray(ctx_lens if ctx_lens is not None else rng.integers(1, max_ctx + 1, bsz), np.int32)
    return q, kc, vc, perm, cl


def check(hip_ctx, q, kc, vc, bt, cl, scale, out_dtype=np.float32):
    """vc is token-major [blocks, Hkv, block, D] (easy to index in the expectations); the kernel and
    the oracle both take the d-major cache layout."""
    vt = K.v_cache_from_token_major(vc)
    got = K.paged_attention_decode(q, kc, vt, bt, cl, scale, out_dtype, ctx=hip_ctx).astype(np.float64)
    want = O.paged_attention_decode(q.view(np.uint16), kc.view(np.uint16), vt.view(np.uint16), bt, cl, scale)
    tol = RTOL * np.abs(want).max(axis=-1, keepdims=True) + (1e-3 if out_dtype == np.float16 else 1e-6)
    assert (np.abs(got - want) <= tol).all(), f"max err {np.abs(got - want).max()}"
    return got


@pytest.mark.parametrize("bsz,hq,hkv,d,blk,max_ctx", [
    (2, 14, 2, 64, 16, 700),     # Qwen2-0.5B head geometry, two splits
    (3, 4, 4, 64, 16, 100),      # MHA
    (2, 8, 1, 64, 32, 1100),     # MQA, 8 query heads on one kv head, block 32, three splits
    (2, 8, 2, 128, 16, 600),     # head_dim 128
    (1, 2, 2, 64, 64, 64),
    (2, 16, 1, 64, 48, 500),     # 16 query heads on one kv head; block size not a power of two
    (2, 32, 2, 128, 16, 300),    # 16 per kv head at head_dim 128
    (3, 1, 1, 128, 32, 257),     # a single head
])
def test_random_cases(hip_ctx, bsz, hq, hkv, d, blk, max_ctx):
    rng = np.random.default_rng(bsz * 1000 + hq)
    case = make_case(rng, bsz, hq, hkv, d, blk, max_ctx)
    check(hip_ctx, *case, 1.0 / np.sqrt(d))
    check(hip_ctx, *case, 1.0 / np.sqrt(d), np.float16)


def test_edge_context_lengths(hip_ctx):
    rng = np.random.default_rng(7)
    lens = [0, 1, 15, 16, 17, 511, 512, 513, 1024]
    q, kc, vc, bt, cl = make_case(rng, len(lens), 14, 2, 64, 16, 1024, lens)
    got = check(hip_ctx, q, kc, vc, bt, cl, 0.125)
    assert (got[0] == 0).all()                                  # empty context -> zeros
    for h in range(14):                                         # ctx == 1 -> that token's V row
        assert np.array_equal(got[1, h], vc[bt[1, 0], h // 7, 0].astype(np.float64))


def test_closed_forms(hip_ctx):
    rng = np.random.default_rng(11)
    q, kc, vc, bt, cl = make_case(rng, 2, 14, 2, 64, 16, 900, [900, 333])
    base = check(hip_ctx, q, kc, vc, bt, cl, 0.125)
    # uniform keys -> plain mean of the cached values
    ku = np.ones_like(kc)
    got = K.paged_attention_decode(q, ku, K.v_cache_from_token_major(vc), bt, cl, 0.125, ctx=hip_ctx)
    for b in range(2):
        toks = [(bt[b, t // 16], t % 16) for t in range(cl[b])]
        for kvh in range(2):
            mean = np.mean([vc[p, kvh, o].astype(np.float64) for p, o in toks], axis=0)
            np.testing.assert_allclose(got[b, kvh * 7 + 3], mean, rtol=RTOL, atol=1e-4)
    # relabelling physical blocks leaves the output bit-identical
    perm = rng.permutation(kc.shape[0])
    inv = np.argsort(perm).astype(np.int32)
    again = K.paged_attention_decode(q, kc[perm], K.v_cache_from_token_major(vc[perm]), inv[bt], cl, 0.125, ctx=hip_ctx)
    assert np.array_equal(again.astype(np.float64), base)
    # large logits do not overflow the softmax; a negative scale is honoured
    check(hip_ctx, (q * 30).astype(np.float16), kc, vc, bt, cl, 1.0)
    check(hip_ctx, q, kc, vc, bt, cl, -0.125)


def test_slots_past_the_context_are_ignored(hip_ctx):
    """Cache slots of the last block beyond ctx_len (and blocks the table lists past it) may hold
    anything, NaN and Inf included, without touching the result."""
    rng = np.random.default_rng(13)
    lens = [5, 16, 37, 600]
    q, kc, vc, bt, cl = make_case(rng, len(lens), 14, 2, 64, 16, 640, lens)
    base = check(hip_ctx, q, kc, vc, bt, cl, 0.125)
    kc2, vc2 = kc.copy(), vc.copy()
    poison = np.array([np.nan, np.inf, -np.inf, 65504.0], np.float16)
    for b, n in enumerate(lens):
        for t in range(n, bt.shape[1] * 16):
            kc2[bt[b, t // 16], :, t % 16, :] = poison[t % 4]
            vc2[bt[b, t // 16], :, t % 16, :] = poison[(t + 1) % 4]
    vt2 = K.v_cache_from_token_major(vc2)
    again = K.paged_attention_decode(q, kc2, vt2, bt, cl, 0.125, ctx=hip_ctx).astype(np.float64)
    assert np.array_equal(again, base)


def test_config5_shape(hip_ctx):
    """BASELINE config 5 attention geometry: batch 32, 14 q / 2 kv heads, d 64, block 16, ctx U[512, 4096]."""
    rng = np.random.default_rng(5)
    q, kc, vc, bt, cl = make_case(rng, 32, 14, 2, 64, 16, 4096, rng.integers(512, 4097, 32))
    check(hip_ctx, q, kc, vc, bt, cl, 0.125, np.float16)


def test_long_runs_per_wave(hip_ctx):
    """Enough sequences that the kernel takes its longest per-wave runs (8 tiles of 16 tokens at head_dim 64,
    4 at head_dim 128), with ragged lengths around the split boundaries."""
    rng = np.random.default_rng(17)
    lens = np.concatenate([[1, 511, 512, 513, 1023, 1025, 2048], rng.integers(1, 2049, 89)])
    q, kc, vc, bt, cl = make_case(rng, len(lens), 8, 4, 64, 16, 2048, lens)
    check(hip_ctx, q, kc, vc, bt, cl, 0.125)
    lens = np.concatenate([[1, 255, 256, 257, 1024], rng.integers(1, 1025, 91)])
    q, kc, vc, bt, cl = make_case(rng, len(lens), 8, 8, 128, 16, 1024, lens)
    check(hip_ctx, q, kc, vc, bt, cl, 0.09)


def test_repeated_calls_reuse_the_workspace(hip_ctx):
    """The completion counters return to zero after every call: different shapes back to back."""
    rng = np.random.default_rng(19)
    for bsz, hq, hkv, d, max_ctx in [(4, 14, 2, 64, 2000), (2, 8, 8, 128, 700), (4, 14, 2, 64, 2000), (1, 4, 1, 64, 90)]:
        case = make_case(rng, bsz, hq, hkv, d, 16, max_ctx)
        check(hip_ctx, *case, 0.125)
        check(hip_ctx, *case, 0.125)


def test_error_paths(hip_ctx):
    from nncase_amd import runtime as rt
    rng = np.random.default_rng(1)
    q, kc, vc, bt, cl = make_case(rng, 1, 3, 2, 64, 16, 32)   # 3 query heads on 2 kv heads
    with pytest.raises(rt.HipError) as e:
        K.paged_attention_decode(q, kc, K.v_cache_from_token_major(vc), bt, cl, 0.125, ctx=hip_ctx)
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH
    q, kc, vc, bt, cl = make_case(rng, 1, 2, 2, 32, 16, 32)   # unsupported head_dim
    with pytest.raises(rt.HipError) as e:
        K.paged_attention_decode(q, kc, K.v_cache_from_token_major(vc), bt, cl, 0.125, ctx=hip_ctx)
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH
    q, kc, vc, bt, cl = make_case(rng, 1, 2, 2, 64, 8, 32)    # block size not a multiple of 16
    with pytest.raises(rt.HipError) as e:
        K.paged_attention_decode(q, kc, K.v_cache_from_token_major(vc), bt, cl, 0.125, ctx=hip_ctx)
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH
    q, kc, vc, bt, cl = make_case(rng, 1, 17, 1, 64, 16, 32)  # 17 query heads on one kv head
    with pytest.raises(rt.HipError) as e:
        K.paged_attention_decode(q, kc, K.v_cache_from_token_major(vc), bt, cl, 0.125, ctx=hip_ctx)
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH


def test_capture_without_a_warm_up_and_pinned_workspace(hip_ctx):
    """Recording the operator sizes the context's split workspace, so a capture needs no eager call first;
    while the captured function lives, a call that would have to move the workspace is refused (-EBUSY)
    instead of freeing memory the graph still addresses."""
    import errno
    from nncase_amd import runtime as rt
    from nncase_amd.runtime import Context, Function
    ctx = Context(0)  # a context of its own: its workspace starts empty
    try:
        rng = np.random.default_rng(99)
        q, kc, vc, bt, cl = make_case(rng, 3, 14, 2, 64, 16, 2048, [2048, 700, 33])
        vt = K.v_cache_from_token_major(vc)
        dq, dk, dv, dbt, dcl = (ctx.to_device(t) for t in (q, kc, vt, bt, cl))
        dout = ctx.alloc(q.size * 4)
        args = rt.PagedAttnArgs(3, 14, 2, 64, 16, bt.shape[1], kc.shape[0], 0.125, rt.DT_F32)
        fn = Function(ctx)
        fn.add_paged_attention_decode(dq, dk, dv, dbt, dcl, dout, args)
        fn.capture()                       # no eager call came before
        want = O.paged_attention_decode(q.view(np.uint16), kc.view(np.uint16), vt.view(np.uint16), bt, cl, 0.125)
        first = None
        for _ in range(3):
            dout.fill(0)
            fn.invoke()
            ctx.sync()
            got = dout.download(q.shape, np.float32)
            assert (np.abs(got - want) <= RTOL * np.abs(want).max(axis=-1, keepdims=True) + 1e-6).all()
            first = got if first is None else first
            assert np.array_equal(got, first)
        # a larger geometry on the same context would move the workspace under the graph
        q2, kc2, vc2, bt2, cl2 = make_case(rng, 16, 14, 2, 64, 16, 4096)
        big = rt.PagedAttnArgs(16, 14, 2, 64, 16, bt2.shape[1], kc2.shape[0], 0.125, rt.DT_F32)
        d2 = [ctx.to_device(t) for t in (q2, kc2, K.v_cache_from_token_major(vc2), bt2, cl2)]
        dout2 = ctx.alloc(q2.size * 4)
        with pytest.raises(rt.HipError) as e:
            ctx.paged_attention_decode(*d2, dout2, big)
        assert e.value.code == -errno.EBUSY
        fn.invoke()                        # the graph still replays on intact memory
        ctx.sync()
        assert np.array_equal(dout.download(q.shape, np.float32), first)
        fn.destroy()                       # nothing refers to the workspace any more: growth is allowed again
        ctx.paged_attention_decode(*d2, dout2, big)
        ctx.sync()
        want2 = O.paged_attention_decode(q2.view(np.uint16), kc2.view(np.uint16), d2 and K.v_cache_from_token_major(vc2).view(np.uint16), bt2, cl2, 0.125)
        got2 = dout2.download(q2.shape, np.float32)
        assert (np.abs(got2 - want2) <= RTOL * np.abs(want2).max(axis=-1, keepdims=True) + 1e-6).all()
    finally:
        ctx.close()
