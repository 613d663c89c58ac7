"""CPU: the oracle's chunked cross-entropy (kernels/cross_entropy.cu:201-305) pinned by closed forms, the
sum-to-zero of a softmax gradient and a double-precision recomputation.  The reference holds no vector for it."""
import numpy as np

import oracle_lib as orc


def bits(x):
    return orc.bf16_from_f32(np.asarray(x, dtype=np.float32))


def reference_f64(logit_bits, labels, n_valid):
    x = orc.bf16_to_f32(logit_bits).astype(np.float64)
    p = np.exp(x - x.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    g = p.copy()
    valid = labels >= 0
    g[np.arange(len(labels))[valid], labels[valid]] -= 1.0
    g[~valid] = 0.0
    n = max(n_valid, 1)
    loss = -(np.log(p[np.arange(len(labels))[valid], labels[valid]] + 1e-9)).sum() / n
    return g / n, loss


def test_count_valid():
    labels = np.array([3, -100, 0, -1, 7, 7, -100], np.int32)
    assert orc.cross_entropy_count_valid(labels) == 4
    assert orc.cross_entropy_count_valid(np.zeros(0, np.int32)) == 0


def test_uniform_logits_and_one_dominant_logit():
    V = 1024                                   # a power of two: 1/V and every partial sum are exact
    logits = bits(np.full((2, V), 0.75))
    logits[1, 5] = bits([60.0])[0]             # exp(0.75 - 60) underflows against 1: p = one-hot
    labels = np.array([9, 5], np.int32)
    grad, loss = orc.cross_entropy_fwd_bwd_chunk(logits, labels, n_valid=2)
    g = orc.bf16_to_f32(grad)
    assert np.all(g[0, np.arange(V) != 9] == np.float32(1.0 / V / 2))
    assert grad[0, 9] == bits([(1.0 / V - 1.0) / 2])[0]                 # the label's term, rounded to bf16
    assert g[1, 5] == 0.0 and np.all(np.abs(g[1]) < 1e-20)
    want = -(np.log(np.float32(1.0 / V) + np.float32(1e-9)) + np.log(np.float32(1.0) + np.float32(1e-9))) / 2
    assert abs(loss - want) < 1e-6


def test_against_double_precision_and_row_sums():
    rng = np.random.default_rng(1)
    for V in (100, 1000, 4099):
        rows = 24
        logits = bits(rng.standard_normal((rows, V)) * 3.0)
        labels = rng.integers(0, V, rows).astype(np.int32)
        labels[::5] = -100
        n_valid = int((labels >= 0).sum())
        grad, loss = orc.cross_entropy_fwd_bwd_chunk(logits, labels, n_valid)
        ref, ref_loss = reference_f64(logits, labels, n_valid)
        g = orc.bf16_to_f32(grad).astype(np.float64)
        assert np.all(np.abs(g - ref) <= 0.5 * orc.bf16_ulp(ref) + 2e-6 * np.abs(ref) + 1e-30)
        assert np.all(grad[labels < 0] == 0)
        # a softmax gradient row sums to zero; what is left is the bf16 rounding of V terms
        assert np.all(np.abs(g.sum(axis=1)) <= 2.0 ** -8 * np.abs(g).sum(axis=1))
        assert abs(loss - ref_loss) <= 1e-5 * abs(ref_loss)
    # the loss accumulates into what the caller passes in
    _, loss2 = orc.cross_entropy_fwd_bwd_chunk(logits, labels, n_valid, loss_in=1.5)
    assert abs((loss2 - 1.5) - loss) < 1e-5
