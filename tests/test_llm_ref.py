"""Pins oracle/llm_ref.py (the float64 restatement the LLM decode GPU tests compare with) on the CPU: the
reference tree has no counterpart, so each function is held to closed forms and invariants chosen so that
a plausible slip -- a swapped gate / up, the interleaved instead of the rotate-half pairing, epsilon
outside the root, a transposed weight -- fails at least one of them."""
import numpy as np
import pytest

from oracle import llm_ref as R
from oracle import oracle as O


def test_rope_is_a_rotation_of_the_rotate_half_pairs():
    rng = np.random.default_rng(0)
    d, theta = 64, 10000.0
    x = rng.standard_normal((3, d))
    assert np.array_equal(R.rope(x, 0, theta), x)                                   # position 0: identity
    for pos in (1, 17, 4095):
        y = R.rope(x, pos, theta)
        np.testing.assert_allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-12)
        # each pair (i, i + d/2) keeps its own length: a rotation inside the pair, nothing leaks between pairs
        np.testing.assert_allclose(y[:, :32] ** 2 + y[:, 32:] ** 2, x[:, :32] ** 2 + x[:, 32:] ** 2, rtol=1e-11)
    # one-hot at index i moves only into indices i and i + d/2, by the angle pos * theta^(-2i/d)
    for i in (0, 5, 31):
        e = np.zeros(d)
        e[i] = 1.0
        y = R.rope(e, 3, theta)
        ang = 3 * theta ** (-2.0 * i / d)
        want = np.zeros(d)
        want[i], want[i + 32] = np.cos(ang), np.sin(ang)
        np.testing.assert_allclose(y, want, atol=1e-15)
        e2 = np.zeros(d)
        e2[i + 32] = 1.0
        want2 = np.zeros(d)
        want2[i], want2[i + 32] = -np.sin(ang), np.cos(ang)
        np.testing.assert_allclose(R.rope(e2, 3, theta), want2, atol=1e-15)
    # <rope(q, m), rope(k, n)> depends on m - n only
    q, k = rng.standard_normal(d), rng.standard_normal(d)
    base = R.rope(q, 9, theta) @ R.rope(k, 4, theta)
    for shift in (1, 100, 2000):
        np.testing.assert_allclose(R.rope(q, 9 + shift, theta) @ R.rope(k, 4 + shift, theta), base, rtol=1e-9, atol=1e-9)
    assert abs(R.rope(q, 9, theta) @ R.rope(k, 5, theta) - base) > 1e-6              # and does change with m - n


def test_rmsnorm_closed_forms():
    w = np.linspace(0.5, 1.5, 8)
    row = np.full((1, 8), 3.0)
    np.testing.assert_allclose(R.rmsnorm(row, w, 0.0), w[None, :], rtol=1e-15)       # constant row -> the weights
    np.testing.assert_allclose(R.rmsnorm(-row, w, 0.0), -w[None, :], rtol=1e-15)     # sign kept
    rng = np.random.default_rng(1)
    x = rng.standard_normal((4, 8))
    np.testing.assert_allclose(R.rmsnorm(7.0 * x, w, 0.0), R.rmsnorm(x, w, 0.0), rtol=1e-12)   # scale invariant at eps 0
    # epsilon sits under the root, added to the mean square: x = (2, 0, 0, 0), eps = 3 -> 2 / sqrt(1 + 3) = 1
    got = R.rmsnorm(np.array([[2.0, 0.0, 0.0, 0.0]]), np.ones(4), 3.0)
    np.testing.assert_allclose(got, [[1.0, 0.0, 0.0, 0.0]], rtol=1e-15)
    # mean, not sum: all-ones row of any width normalises to itself
    np.testing.assert_allclose(R.rmsnorm(np.ones((1, 896)), np.ones(896), 0.0), np.ones((1, 896)), rtol=1e-15)


def test_silu_and_w8a16_linear():
    assert R.silu(np.array([0.0]))[0] == 0.0
    np.testing.assert_allclose(R.silu(np.array([1.0, -1.0])), [1 / (1 + np.exp(-1.0)), -1 / (1 + np.exp(1.0))], rtol=1e-15)
    rng = np.random.default_rng(2)
    a = rng.integers(-8, 9, (3, 16)).astype(np.float16)
    q = rng.integers(-128, 128, (5, 16)).astype(np.int8)
    scale = np.array([1, 2, 0.5, 4, 0.25], np.float32)
    bias = np.array([1, -2, 3, -4, 5], np.float32)
    want = np.zeros((3, 5))
    for m in range(3):
        for n in range(5):
            want[m, n] = float(scale[n]) * sum(int(a[m, k]) * int(q[n, k]) for k in range(16)) + float(bias[n])
    assert np.array_equal(R.w8a16_linear(a, q, scale, bias), want)                   # out[m, n] = s[n] * sum_k a[m,k] q[n,k] + b[n]
    assert np.array_equal(R.w8a16_linear(a, q, scale), want - bias[None, :])


class _Cfg:
    layers, hidden, q_heads, kv_heads, head_dim, mlp, vocab = 1, 4, 2, 1, 2, 2, 4
    rms_eps, rope_theta, block_size = 0.0, 10000.0, 16


def _tiny_weights(gate_rows, up_rows):
    """One layer with integer weights and unit scales; normalisation weights of one."""
    c = _Cfg
    qd, kvd = c.q_heads * c.head_dim, c.kv_heads * c.head_dim
    ones = lambda n: np.ones(n, np.float32)
    eye = np.eye(4, dtype=np.int8)
    layer = {
        "ln1": np.ones(c.hidden, np.float16), "ln2": np.ones(c.hidden, np.float16),
        # q head 0 = x[0:2], q head 1 = x[2:4], k = x[0:2], v = x[2:4]
        "qkv": (np.concatenate([eye, eye[0:2], eye[2:4]]).astype(np.int8), ones(qd + 2 * kvd)), "qkv_bias": np.zeros(qd + 2 * kvd, np.float32),
        "o": (eye, ones(c.hidden)),
        "gate_up": (np.concatenate([gate_rows, up_rows]).astype(np.int8), ones(2 * c.mlp)),
        "down": (np.array([[1, 0], [0, 1], [0, 0], [0, 0]], np.int8), ones(c.hidden)),
    }
    emb = np.array([[1, 0, 2, 0], [0, 1, 0, 2], [2, 2, 2, 2], [1, 1, 1, 1]], np.float16)
    return {"layers": [layer], "embedding": emb, "ln_f": np.ones(c.hidden, np.float16), "lm_head": (np.eye(4, dtype=np.int8), ones(4))}


def test_decode_step_against_a_hand_calculation():
    """Empty context (position 0: the rotary embedding is the identity and the only attended token is the one
    just appended, so attention returns its V row), epsilon 0, integer weights: every stage is computable by hand."""
    c = _Cfg
    gate = np.array([[1, 0, 0, 0], [0, 1, 0, 0]])
    up = np.array([[0, 0, 1, 0], [0, 0, 0, 1]])
    w = _tiny_weights(gate, up)
    kc = [np.zeros((2, 1, 16, 2), np.float16)]
    vc = [np.zeros((2, 1, 2, 16), np.float16)]
    bt = np.array([[1]], np.int32)
    nxt, logits = R.decode_step(c, w, [3], bt, np.array([0], np.int32), kc, vc)       # token 3: x = (1, 1, 1, 1)
    f16 = lambda v: np.asarray(v, np.float64).astype(np.float16).astype(np.float64)
    x = np.ones(4)
    n = x / np.sqrt(np.mean(x * x))                                                  # (1, 1, 1, 1)
    v_row = n[2:4]                                                                   # v = x[2:4]
    att = np.concatenate([v_row, v_row])                                             # both heads share the kv head
    h = f16(x + att)                                                                 # o = identity: (2, 2, 2, 2)
    n2 = f16(h / np.sqrt(np.mean(h * h)))                                            # (1, 1, 1, 1)
    g, u = n2[0:2], n2[2:4]
    act = f16(g / (1 + np.exp(-g)) * u)
    out = f16(h + np.array([act[0], act[1], 0, 0]))
    nf = f16(out / np.sqrt(np.mean(out * out)))
    np.testing.assert_allclose(logits[0], nf, rtol=1e-12)
    assert nxt[0] == 0                                                               # lowest index among the two largest
    # the new token's k and v went to slot 0 of physical block 1, V d-major
    assert np.array_equal(kc[0][1, 0, 0], np.array([1, 1], np.float16)) and np.array_equal(vc[0][1, 0, :, 0], np.array([1, 1], np.float16))
    assert not kc[0][0].any() and not vc[0][0].any()


def test_swiglu_takes_the_gate_from_the_first_half():
    """silu(gate) * up with the gate in rows [0, mlp): with gate = -x and up = +x swapping them changes the result
    (silu(-1) * 1 = -0.269 against silu(1) * -1 = -0.731)."""
    c = _Cfg
    gate = -np.array([[1, 0, 0, 0], [0, 1, 0, 0]])
    up = np.array([[1, 0, 0, 0], [0, 1, 0, 0]])
    w = _tiny_weights(gate, up)
    w["layers"][0]["down"] = (np.zeros((4, 2), np.int8), np.ones(4, np.float32))
    w["layers"][0]["down"][0][0, 0] = 64                                              # logit 0 carries 64 * act[0]
    kc, vc = [np.zeros((1, 1, 16, 2), np.float16)], [np.zeros((1, 1, 2, 16), np.float16)]
    _, logits = R.decode_step(c, w, [3], np.array([[0]], np.int32), np.array([0], np.int32), kc, vc)
    f16 = lambda v: np.asarray(v, np.float64).astype(np.float16).astype(np.float64)
    h = np.full(4, 2.0)
    act0 = f16((-1.0) / (1 + np.exp(1.0)) * 1.0)                                      # silu(gate = -1) * up = 1
    out = f16(h + np.array([64 * act0, 0, 0, 0]))
    nf = f16(out / np.sqrt(np.mean(out * out)))
    np.testing.assert_allclose(logits[0], nf, rtol=1e-12)
    swapped = f16(1.0 / (1 + np.exp(-1.0)) * -1.0)
    assert abs(64 * act0 - 64 * swapped) > 20                                         # the other order is far away


def test_cosine_follows_the_reference_harness():
    a = np.array([1.0, 2.0, 3.0])
    assert O.cosine(a, a) == 1.0
    assert O.cosine(np.zeros(3), np.zeros(3)) == 1.0                                 # identical all-zero arrays
    np.testing.assert_allclose(O.cosine(a, 2 * a), 1.0, rtol=1e-15)
    np.testing.assert_allclose(O.cosine(np.array([1.0, 0.0]), np.array([0.0, 1.0])), 0.0)
    nan, inf = float("nan"), float("inf")
    assert O.cosine(np.array([1.0, nan, 3.0]), np.array([1.0, nan, 3.0])) == 1.0     # same-position NaN is dropped
    assert O.cosine(np.array([1.0, inf, 3.0]), np.array([1.0, inf, 3.0])) == 1.0     # same-position Inf is dropped
    assert O.cosine(np.array([1.0, 2.0, 3.0]), np.array([1.0, nan, 3.0])) == -1.0    # one-sided NaN fails
    assert O.cosine(np.array([1.0, nan, 3.0]), np.array([1.0, 2.0, 3.0])) == -1.0
    assert O.cosine(np.array([1.0, 2.0, 3.0]), np.array([1.0, inf, 3.0])) == -1.0    # one-sided Inf fails
    assert O.cosine(np.array([nan, 2.0, 3.0]), np.array([1.0, nan, 3.0])) == -1.0    # NaN on both sides, different places
    assert O.cosine(np.zeros(3), a) == -1.0                                          # 0 / 0 -> NaN -> -1
