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
    got = K.paged_attention_decode(q, kc, vc, bt, cl, scale, out_dtype, ctx=hip_ctx).astype(np.float64)
    want = O.paged_attention_decode(q.view(np.uint16), kc.view(np.uint16), vc.view(np.uint16), bt, cl, scale)
    tol = RTOL * np.abs(want).max(axis=-1, keepdims=True) + (1e-3 if out_dtype == np.float16 else 1e-6)
    assert (np.abs(got - want) <= tol).all(), f"max err {np.abs(got - want).max()}"
    return got


@pytest.mark.parametrize("bsz,hq,hkv,d,blk,max_ctx", [
    (2, 14, 2, 64, 16, 700),     # Qwen2-0.5B head geometry, two splits
    (3, 4, 4, 64, 16, 100),      # MHA
    (2, 8, 1, 64, 32, 1100),     # MQA, 8 query heads on one kv head, block 32, three splits
    (2, 8, 2, 128, 16, 600),     # head_dim 128
    (1, 2, 2, 64, 64, 64),
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
    got = K.paged_attention_decode(q, ku, vc, bt, cl, 0.125, ctx=hip_ctx)
    for b in range(2):
        toks = [(bt[b, t // 16], t % 16) for t in range(cl[b])]
        for kvh in range(2):
            mean = np.mean([vc[p, kvh, o].astype(np.float64) for p, o in toks], axis=0)
            np.testing.assert_allclose(got[b, kvh * 7 + 3], mean, rtol=RTOL, atol=1e-4)
    # relabelling physical blocks leaves the output bit-identical
    perm = rng.permutation(kc.shape[0])
    inv = np.argsort(perm).astype(np.int32)
    again = K.paged_attention_decode(q, kc[perm], vc[perm], inv[bt], cl, 0.125, ctx=hip_ctx)
    assert np.array_equal(again.astype(np.float64), base)
    # large logits do not overflow the softmax
    check(hip_ctx, (q * 30).astype(np.float16), kc, vc, bt, cl, 1.0)


def test_config5_shape(hip_ctx):
    """BASELINE config 5 attention geometry: batch 32, 14 q / 2 kv heads, d 64, block 16, ctx U[512, 4096]."""
    rng = np.random.default_rng(5)
    q, kc, vc, bt, cl = make_case(rng, 32, 14, 2, 64, 16, 4096, rng.integers(512, 4097, 32))
    check(hip_ctx, q, kc, vc, bt, cl, 0.125, np.float16)


def test_error_paths(hip_ctx):
    from nncase_amd import runtime as rt
    rng = np.random.default_rng(1)
    q, kc, vc, bt, cl = make_case(rng, 1, 3, 2, 64, 16, 32)   # 3 query heads on 2 kv heads
    with pytest.raises(rt.HipError) as e:
        K.paged_attention_decode(q, kc, vc, bt, cl, 0.125, ctx=hip_ctx)
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH
    q, kc, vc, bt, cl = make_case(rng, 1, 2, 2, 32, 16, 32)   # unsupported head_dim
    with pytest.raises(rt.HipError) as e:
        K.paged_attention_decode(q, kc, vc, bt, cl, 0.125, ctx=hip_ctx)
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH
