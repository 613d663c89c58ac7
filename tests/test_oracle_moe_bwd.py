"""CPU: the oracle of the MoE expert-bank backward helpers against what the mathematics fixes
(kernels/moe.cu:510-521, 623-674, 1148-1167).  The reference holds no vectors for these kernels."""
import math

import numpy as np
import pytest

import oracle_lib as orc


def bf(x):
    return orc.bf16_from_f32(np.asarray(x, np.float32))


def f(bits):
    return orc.bf16_to_f32(bits).astype(np.float64)


def all_finite_bf16():
    bits = np.arange(1 << 16, dtype=np.uint16)
    return bits[np.isfinite(orc.bf16_to_f32(bits))]


def test_gelu_forward_every_bf16_value_against_double():
    bits = all_finite_bf16()
    x = f(bits)
    exact = 0.5 * x * (1.0 + np.vectorize(math.erf)(x / math.sqrt(2.0)))
    got = f(orc.gelu_forward(bits))
    # float32 evaluation then one bf16 rounding: within one bf16 ulp of the exact value, plus what the float32
    # rounding of 1 + erf costs where it cancels (x < 0: an ulp of 1 times |x| / 2); equal to the correctly
    # rounded value almost everywhere the cancellation plays no part
    assert np.all(np.abs(got - exact) <= orc.bf16_ulp(exact) + np.abs(x) * 2.0 ** -24)
    mild = x > -2.0
    assert np.mean(got[mild] != f(bf(exact[mild]))) < 2e-3
    # landmarks: gelu(0) = 0, gelu(x) -> x for large x, -> 0 for very negative x
    assert f(orc.gelu_forward(bf([0.0, 10.0, -10.0])))[0] == 0.0
    assert np.array_equal(f(orc.gelu_forward(bf([10.0, 37.5]))), [10.0, 37.5])
    assert abs(f(orc.gelu_forward(bf([-10.0])))[0]) == 0.0


def test_gelu_backward_is_the_derivative_of_the_forward():
    x = np.linspace(-6.0, 6.0, 2001)
    xb = bf(x)
    xs = f(xb)
    ones = bf(np.ones_like(xs))
    got = f(orc.gelu_backward(xb, ones))
    g = lambda v: 0.5 * v * (1.0 + np.vectorize(math.erf)(v / math.sqrt(2.0)))
    h = 1e-6
    central = (g(xs + h) - g(xs - h)) / (2 * h)
    assert np.all(np.abs(got - central) <= orc.bf16_ulp(central) + 1e-7)
    # gelu'(0) = 1/2 exactly; gelu'(x) + gelu'(-x) = 1 (Phi(x) + Phi(-x) = 1 and x phi(x) is odd)
    assert f(orc.gelu_backward(bf([0.0]), bf([1.0])))[0] == 0.5
    pos, neg = f(orc.gelu_backward(bf(xs), ones)), f(orc.gelu_backward(bf(-xs), ones))
    assert np.all(np.abs(pos + neg - 1.0) <= 2.0 ** -7)
    # linear in the upstream gradient up to the final rounding
    gup = bf(np.full_like(xs, -3.0))
    assert np.all(np.abs(f(orc.gelu_backward(xb, gup)) + 3.0 * central) <= 3.0 * orc.bf16_ulp(central) + 1e-6)


@pytest.mark.parametrize("H", [256, 512, 2048, 64, 8, 1000])
def test_row_dot_exact_sums_and_routing(H):
    """Small integers: every product and every partial sum is exact, so any summation order gives the integer
    dot product; what is checked is which rows are paired and where the result lands."""
    rng = np.random.default_rng(H)
    rows, n = 40, 17
    a = rng.integers(-4, 5, (rows, H)).astype(np.float32)
    b = rng.integers(-4, 5, (n, H)).astype(np.float32)
    ri = np.sort(rng.choice(rows, n, replace=False)).astype(np.int32)
    out0 = np.full((rows, 5), 7.25, np.float32)
    out = orc.moe_row_dot_selected(bf(a), bf(b), out0, ri, 3)
    want = out0.copy()
    want[ri, 3] = (a[ri] * b).sum(axis=1)
    assert np.array_equal(out, want)


def test_row_dot_follows_the_strided_halving_tree():
    """A row on which the order matters: thread 0's chain holds 2^24 then two ones, which a float32 chain
    swallows one at a time (2^24 + 1 = 2^24), while any tree that first adds the ones keeps them."""
    H = 1024
    a = np.zeros((1, H), np.float32)
    a[0, 0] = 4096.0          # product 2^24 with b = 4096
    a[0, 256] = 1.0           # same thread (h % 256 == 0), later links of the chain
    a[0, 512] = 1.0
    a[0, 1] = 1.0             # thread 1: survives as its own partial and is added in the tree: 2^24 + 1 -> 2^24 (tie to even)
    b = np.zeros((1, H), np.float32)
    b[0, 0] = 4096.0
    b[0, [256, 512, 1]] = 1.0
    out = orc.moe_row_dot_selected(bf(a), bf(b), np.zeros((1, 1), np.float32), np.zeros(1, np.int32), 0)
    assert out[0, 0] == 16777216.0                      # all three ones are lost, one at a time
    # two ones that meet each other in the tree before they meet the large partial survive as a 2
    a[0, 512] = 0.0; b[0, 512] = 0.0
    a[0, 256] = 0.0; b[0, 256] = 0.0
    a[0, 129] = 1.0; b[0, 129] = 1.0                    # thread 129 meets thread 1 at stride 128: 1 + 1 = 2 survives
    out = orc.moe_row_dot_selected(bf(a), bf(b), np.zeros((1, 1), np.float32), np.zeros(1, np.int32), 0)
    assert out[0, 0] == 16777218.0


def test_row_dot_against_double_and_the_192_thread_tree():
    rng = np.random.default_rng(3)
    rows, n, H = 12, 12, 768
    a = bf(rng.standard_normal((rows, H)))
    b = bf(rng.standard_normal((n, H)))
    ri = np.arange(n, dtype=np.int32)
    out = orc.moe_row_dot_selected(a, b, np.zeros((rows, 1), np.float32), ri, 0)[:, 0]
    exact = (f(a) * f(b)).sum(axis=1)
    assert np.all(np.abs(out - exact) <= 2.0 ** -21 * (np.abs(f(a) * f(b))).sum(axis=1))
    # H = 192 launches 192 threads; strides 96, 48, 24, 12, 6, 3, 1: after stride 3 the partial of slot 2 is
    # never added (3 >> 1 = 1).  Slot 2 holds threads t with t % 3 == 2 ... every thread index congruent to 2
    # modulo 3 is dropped.  With all-ones rows the result is 192 - 64 = 128.
    ones = bf(np.ones((1, 192)))
    out = orc.moe_row_dot_selected(ones, ones, np.zeros((1, 1), np.float32), np.zeros(1, np.int32), 0)
    assert out[0, 0] == 128.0


def test_gather_scale_and_scatter_add_closed_forms():
    rng = np.random.default_rng(11)
    rows, E, H = 50, 6, 40
    src = bf(rng.standard_normal((rows, H)))
    rw = rng.uniform(0.1, 0.9, (rows, E)).astype(np.float32)
    ri = np.sort(rng.choice(rows, 23, replace=False)).astype(np.int32)
    got = orc.moe_gather_scale_rows(src, rw, ri, 4)
    want = bf((rw[ri, 4][:, None] * orc.bf16_to_f32(src[ri])).astype(np.float32))
    assert np.array_equal(got, want)
    # weight 1 is a gather, weight 0 gives signed zeros
    rw1 = np.ones_like(rw)
    assert np.array_equal(orc.moe_gather_scale_rows(src, rw1, ri, 0), src[ri])
    assert np.all(f(orc.moe_gather_scale_rows(src, np.zeros_like(rw), ri, 0)) == 0.0)

    dst = bf(rng.standard_normal((rows, H)))
    comp = bf(rng.standard_normal((ri.size, H)))
    got = orc.moe_scatter_add_rows(dst, comp, ri)
    want = dst.copy()
    want[ri] = bf((orc.bf16_to_f32(dst[ri]) + orc.bf16_to_f32(comp)).astype(np.float32))
    assert np.array_equal(got, want)
    # equals the weighted scatter with unit route weights (fma(1, c, m) = m + c)
    assert np.array_equal(got, orc.moe_scatter_accumulate(dst, comp, np.ones((rows, 1), np.float32), ri, 0))
    # rows outside the list are untouched
    mask = np.ones(rows, bool); mask[ri] = False
    assert np.array_equal(got[mask], dst[mask])
