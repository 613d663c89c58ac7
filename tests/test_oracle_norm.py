"""CPU: the oracle's RMSNorm and row clip pinned by closed forms, a double-precision recomputation and the
symmetries of the reference's reduction tree (kernels/rmsnorm.cu:13-54, src/trainer.cu:3822-3842,3940-3958).
The reference holds no test vector for these kernels."""
import numpy as np
import pytest

import oracle_lib as orc

f32 = np.float32


def bits(x):
    return orc.bf16_from_f32(np.asarray(x, dtype=np.float32))


def vals(b):
    return orc.bf16_to_f32(b)


def closed_form(x_val, total, H, w_val, eps):
    """rms and one output element from an exactly known sum of squares, in IEEE fp32 steps."""
    rms = np.sqrt(f32(total) / f32(H) + f32(eps), dtype=np.float32)
    inv = f32(1.0) / rms
    return rms, bits([(f32(x_val) * inv) * f32(w_val)])[0]


@pytest.mark.parametrize("H", [32, 96, 512, 1024, 4096, 5120])
def test_rmsnorm_rows_with_exact_sums(H):
    eps = 1e-6
    w = bits(np.full(H, 1.5))
    # a constant row, a row of +-1, a one-hot row: every partial sum is exact, so the order cannot matter
    const = np.full(H, 2.0, np.float32)
    signs = np.where(np.arange(H) % 3 == 0, -1.0, 1.0).astype(np.float32)
    onehot = np.zeros(H, np.float32); onehot[H // 3] = 8.0
    x = bits(np.stack([const, signs, onehot]))
    out, rms = orc.rmsnorm_forward(x, w, eps)
    for r, (total, probe, xv) in enumerate([(4.0 * H, 0, 2.0), (float(H), 1, 1.0), (64.0, H // 3, 8.0)]):
        want_rms, want_out = closed_form(xv, total, H, 1.5, eps)
        assert rms[r] == want_rms
        assert out[r, probe] == want_out
    assert np.all(out[2, np.arange(H) != H // 3] == 0)          # zeros stay zero
    assert np.all(out[1] == np.where(signs < 0, out[1, 0], out[1, 1]))


def test_rmsnorm_against_double_precision():
    rng = np.random.default_rng(5)
    for H in (512, 1024, 4096):
        x = bits(rng.standard_normal((16, H)) * 3.0)
        w = bits(1.0 + 0.1 * rng.standard_normal(H))
        out, rms = orc.rmsnorm_forward(x, w)
        xd, wd = vals(x).astype(np.float64), vals(w).astype(np.float64)
        rms_d = np.sqrt((xd * xd).mean(axis=1) + 1e-6)
        assert np.allclose(rms, rms_d, rtol=2e-6, atol=0)
        ref = xd / rms_d[:, None] * wd
        got = vals(out).astype(np.float64)
        assert np.all(np.abs(got - ref) <= 0.5 * orc.bf16_ulp(ref) + 4e-7 * np.abs(ref)), "more than half a bf16 ulp (plus fp32 slack) from the exact value"


def test_rmsnorm_sum_has_the_butterfly_symmetry_and_no_other():
    """Moving every thread's elements to thread t ^ c maps the xor butterfly onto itself, so the fp32 sum keeps
    its bits; rotating the threads by one regroups the additions and must change some rows."""
    rng = np.random.default_rng(11)
    H, T = 4096, 512
    x = bits(rng.standard_normal((64, H)) * np.exp(rng.standard_normal((64, H))))
    w = bits(np.ones(H))
    _, rms = orc.rmsnorm_forward(x, w)
    cols = np.arange(H)
    t, j = cols % T, cols // T
    for c in (1, 16, 21, 32, 256, 0x1ff):
        perm = (t ^ c) + T * j
        _, rms_p = orc.rmsnorm_forward(np.ascontiguousarray(x[:, perm]), w)
        assert np.array_equal(rms_p.view(np.uint32), rms.view(np.uint32)), f"xor {c}"
    rot = ((t + 1) % T) + T * j
    _, rms_r = orc.rmsnorm_forward(np.ascontiguousarray(x[:, rot]), w)
    assert np.any(rms_r.view(np.uint32) != rms.view(np.uint32))
    assert np.allclose(rms_r, rms, rtol=1e-5)
    # a per-thread chain is sequential in j: swapping two of a thread's own elements may change bits, too
    swap = cols.copy(); swap[t + T * 0], swap[t + T * 7] = cols[t + T * 7], cols[t + T * 0]
    _, rms_s = orc.rmsnorm_forward(np.ascontiguousarray(x[:, swap]), w)
    assert np.allclose(rms_s, rms, rtol=1e-5)


def test_rmsnorm_rejects_partial_warps():
    with pytest.raises(ValueError):
        orc.rmsnorm_forward(bits(np.ones((1, 100))), bits(np.ones(100)))


@pytest.mark.parametrize("cols", [32, 96, 256, 1000, 4096])
def test_row_clip_closed_forms(cols):
    # rows of constant magnitude: sum of squares exact; ceiling between the two rows' norms
    small = np.full(cols, 0.5, np.float32)
    big = np.full(cols, 4.0, np.float32); big[::2] *= -1
    x = bits(np.stack([small, big]))
    norm_small, norm_big = np.sqrt(f32(0.25 * cols)), np.sqrt(f32(16.0 * cols))
    ceiling = f32(0.5) * (norm_small + norm_big)
    out, normsq = orc.act_row_clip_abs(x, ceiling)
    assert normsq[0] == f32(0.25 * cols) and normsq[1] == f32(16.0 * cols)
    assert np.array_equal(out[0], x[0])                                  # at or under the ceiling: untouched
    scalef = ceiling / norm_big
    assert np.array_equal(out[1], bits(vals(x[1]) * scalef))
    # exactly at the ceiling is not clipped; a non-positive ceiling disables the clip
    out_eq, _ = orc.act_row_clip_abs(x, norm_big)
    assert np.array_equal(out_eq, x)
    out_off, _ = orc.act_row_clip_abs(x, 0.0)
    assert np.array_equal(out_off, x)


def test_row_clip_against_double_precision():
    rng = np.random.default_rng(3)
    x = bits(rng.standard_normal((32, 2048)) * np.linspace(0.2, 5.0, 32)[:, None])
    xd = vals(x).astype(np.float64)
    norms = np.sqrt((xd * xd).sum(axis=1))
    ceiling = f32(np.median(norms))
    out, normsq = orc.act_row_clip_abs(x, ceiling)
    assert np.allclose(normsq, norms ** 2, rtol=2e-6)
    clipped = norms > float(ceiling) * (1 + 1e-5)
    kept = norms < float(ceiling) * (1 - 1e-5)
    assert clipped.sum() > 4 and kept.sum() > 4
    assert np.array_equal(out[kept], x[kept])
    got = vals(out[clipped]).astype(np.float64)
    ref = xd[clipped] * (float(ceiling) / norms[clipped])[:, None]
    assert np.all(np.abs(got - ref) <= 0.5 * orc.bf16_ulp(ref) + 4e-7 * np.abs(ref))
    # the clipped rows sit on the ceiling
    assert np.allclose(np.sqrt((got * got).sum(axis=1)), float(ceiling), rtol=2e-3)
