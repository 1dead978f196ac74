"""GPU: the paged-attention entry point that allocates nothing (static device scratch) gives, through the
C ABI, bit for bit what nncase_hip_paged_attention_decode gives -- on two calls in a row, the second with a
smaller input (the scratch keeps the first call's partials and must not leak them) -- and refuses
geometries beyond its scratch."""
import errno

import numpy as np
import pytest

from nncase_amd import kernels as K
from nncase_amd import runtime as rt

pytestmark = pytest.mark.gpu


def _case(rng, bsz, hq, hkv, d, blk, max_ctx, lens):
    max_blocks = -(-max_ctx // blk)
    nb = bsz * max_blocks + 2
    q = rng.standard_normal((bsz, hq, d)).astype(np.float16)
    kc = rng.standard_normal((nb, hkv, blk, d)).astype(np.float16)
    vt = K.v_cache_from_token_major(rng.standard_normal((nb, hkv, blk, d)).astype(np.float16))
    bt = rng.permutation(nb)[: bsz * max_blocks].reshape(bsz, max_blocks).astype(np.int32)
    return q, kc, vt, bt, np.asarray(lens, np.int32)


def _both(ctx, q, kc, vt, bt, cl, out_dtype):
    bsz, hq, d = q.shape
    nb, hkv, blk, _ = kc.shape
    dq, dk, dv, dbt, dcl = (ctx.to_device(t) for t in (q, kc, vt, bt, cl))
    args = rt.PagedAttnArgs(bsz, hq, hkv, d, blk, bt.shape[1], nb, float(d ** -0.5), rt.NP_TO_DT[np.dtype(out_dtype)])
    outs = []
    for call in (ctx.paged_attention_decode_noalloc, ctx.paged_attention_decode):
        dout = ctx.alloc(bsz * hq * d * np.dtype(out_dtype).itemsize).fill(0xEE)
        call(dq, dk, dv, dbt, dcl, dout, args)
        ctx.sync()
        outs.append(dout.download((bsz, hq, d), out_dtype))
    return outs


def test_noalloc_matches_the_allocating_entry_point_twice_in_a_row(hip_ctx):
    rng = np.random.default_rng(2024)
    # first call: config-5 head geometry, several splits per sequence, lengths from empty to full
    big = _case(rng, 6, 14, 2, 64, 16, 4096, [4096, 2049, 513, 1, 0, 3000])
    got, want = _both(hip_ctx, *big, np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.isfinite(got).all() and (got[4] == 0).all()
    # second call, smaller in every extent, right behind the first: stale partials and counters must not show
    small = _case(rng, 2, 8, 2, 128, 32, 700, [700, 97])
    got, want = _both(hip_ctx, *small, np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # and the large one again after the small one
    got, want = _both(hip_ctx, *big, np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_noalloc_refuses_what_its_scratch_cannot_hold(hip_ctx):
    rng = np.random.default_rng(5)
    q, kc, vt, bt, cl = _case(rng, 1, 2, 2, 64, 16, 64, [64])
    dq, dk, dv, dbt, dcl = (hip_ctx.to_device(t) for t in (q, kc, vt, bt, cl))
    dout = hip_ctx.alloc(1 << 20)
    # the host-side plan only looks at the extents: 4096 sequences x 64 heads x many splits cannot fit 8 MiB
    args = rt.PagedAttnArgs(4096, 64, 4, 64, 16, 4096, 8, 0.125, rt.DT_F32)
    with pytest.raises(rt.HipError) as e:
        hip_ctx.paged_attention_decode_noalloc(dq, dk, dv, dbt, dcl, dout, args)
    assert e.value.code == -errno.ENOSPC


def test_noalloc_call_recorded_into_a_hip_graph_replays_correctly(hip_ctx):
    """The entry point is meant for code under HIP graph capture: its first call on a context may be the captured one (the
    scratch address was taken when the context was created, so the call itself only launches).  The graph is replayed
    three times, with eager work and synchronisations of the same context in between, and every replay gives the bytes of
    the eager call (the counters are cleared by a kernel inside the graph, not by a memset node)."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    ctx = rt.Context(0)                                      # a context whose first attention call is the captured one
    rng = np.random.default_rng(77)
    q, kc, vt, bt, cl = _case(rng, 5, 14, 2, 64, 16, 2048, [2048, 1500, 17, 600, 1025])
    bsz, hq, d = q.shape
    nb, hkv, blk, _ = kc.shape
    dq, dk, dv, dbt, dcl = (ctx.to_device(t) for t in (q, kc, vt, bt, cl))
    args = rt.PagedAttnArgs(bsz, hq, hkv, d, blk, bt.shape[1], nb, float(d ** -0.5), rt.DT_F32)
    dout = ctx.alloc(bsz * hq * d * 4).fill(0xEE)
    stream = C.c_void_p(ctx.stream)
    graph, gexec = C.c_void_p(), C.c_void_p()
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    assert hip.hipStreamBeginCapture(stream, 2) == 0         # hipStreamCaptureModeRelaxed
    try:
        ctx.paged_attention_decode_noalloc(dq, dk, dv, dbt, dcl, dout, args)
    finally:
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0 and graph.value
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
    want_out = ctx.alloc(bsz * hq * d * 4).fill(0x11)
    ctx.paged_attention_decode(dq, dk, dv, dbt, dcl, want_out, args)   # eager, allocating entry point
    ctx.sync()
    want = want_out.download((bsz, hq, d), np.float32)
    for replay in range(3):
        dout.fill(0xEE)
        ctx.sync()
        assert hip.hipGraphLaunch(gexec, stream) == 0
        ctx.sync()
        got = dout.download((bsz, hq, d), np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"replay {replay}"
        # eager work of the same context between the replays (it uses the same static scratch)
        other = ctx.alloc(bsz * hq * d * 4)
        ctx.paged_attention_decode_noalloc(dq, dk, dv, dbt, dcl, other, args)
        ctx.sync()
        assert np.array_equal(other.download((bsz, hq, d), np.float32).view(np.uint32), want.view(np.uint32))
    hip.hipGraphExecDestroy(gexec)
    hip.hipGraphDestroy(graph)
    ctx.close()
