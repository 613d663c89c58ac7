"""Pins the CPU oracle's routing / dispatch / GEMM-reference functions: the reference's
router fixture, double-precision closed forms, invariants and brute force on tiny cases."""
import itertools
import json
from pathlib import Path

import numpy as np
import pytest

import oracle_lib as orc

GOLD = Path(__file__).resolve().parent / "golden"


def test_expf_within_2ulp_of_exp():
    x = np.concatenate([np.linspace(-104, 89, 2_000_001), np.linspace(-1, 1, 200001),
                        np.array([0.0, -0.0, -87.5, -103.9, 88.7])]).astype(np.float32)
    got = orc.expf(x).astype(np.float64)
    want = np.exp(x.astype(np.float64))
    with np.errstate(over="ignore"):
        want32 = want.astype(np.float32)
    ulp = np.spacing(np.maximum(np.abs(want32), np.float32(2.0 ** -126))).astype(np.float64)
    fin = np.isfinite(want32)
    assert np.max(np.abs(got[fin] - want[fin]) / ulp[fin]) <= 2.0
    assert orc.expf(np.array([0.0], np.float32))[0] == 1.0
    assert orc.expf(np.array([-200.0], np.float32))[0] == 0.0 and np.isinf(orc.expf(np.array([90.0], np.float32))[0])
    assert np.all(np.diff(orc.expf(np.linspace(-20, 0, 100001).astype(np.float32))) >= 0)   # monotone where the router uses it


def test_softmax_against_float64():
    rng = np.random.default_rng(0)
    for cols in (1, 3, 8, 64, 100, 300):
        x = (rng.standard_normal((37, cols)) * 3).astype(np.float32)
        got = orc.softmax(x)
        e = np.exp(x.astype(np.float64) - x.max(1, keepdims=True))
        want = e / e.sum(1, keepdims=True)
        assert np.max(np.abs(got - want)) <= 4e-7
        assert np.all(np.abs(got.sum(1) - 1) <= 1e-5)


def test_topk_reference_fixture():
    g = json.loads((GOLD / "moe_router_parity.json").read_text())
    c = g["cases"]["unpacked_case"]
    got = orc.moe_topk_route(np.array(c["logits"], np.float32), g["top_k"])
    want = np.array(c["route_weights_pre_inhibition"], np.float32)
    assert np.array_equal(got > 0, want > 0)                    # same experts selected
    assert np.max(np.abs(got - want)) <= 2e-7                   # values to fp32 rounding of the fixture


def py_topk(probs, k, normalize=True):
    out = np.zeros_like(probs)
    for r, s in enumerate(probs):
        kept = []
        for _ in range(min(k, len(s))):
            best, best_v = -1, np.float32(-1.0)
            for e in range(len(s)):
                if e not in kept and s[e] > best_v:
                    best, best_v = e, s[e]
            if best < 0:
                break
            kept.append(best)
        tot = np.float32(0)
        for e in sorted(kept):
            tot = np.float32(tot + s[e])
        inv = np.float32(1.0) / tot if (normalize and tot > 0) else np.float32(1.0)
        for e in kept:
            out[r, e] = s[e] * inv
    return out


def test_topk_invariants_and_ties():
    rng = np.random.default_rng(1)
    for E, k in ((3, 2), (8, 2), (64, 6), (64, 64), (5, 9), (40, 1)):
        logits = rng.standard_normal((200, E)).astype(np.float32)
        logits[::7, : E // 2] = 0.25                              # many exact ties
        probs = orc.softmax(logits)
        got, row_sum, save = orc.moe_topk_route(logits, k, want_saves=True)
        assert np.array_equal(save, probs)
        assert np.array_equal(got, py_topk(probs, k))
        kk = min(k, E)
        assert np.all((got > 0).sum(1) == kk)
        assert np.all(np.abs(got.sum(1) - 1) <= 1e-5)
        # kept set = the k largest probabilities, lowest index first among equals
        for r in range(0, 200, 13):
            order = sorted(range(E), key=lambda e: (-probs[r, e], e))[:kk]
            assert set(np.nonzero(got[r])[0]) == set(order)
        raw = orc.moe_topk_route(logits, k, normalize=False)
        assert np.array_equal(raw[raw > 0], probs[raw > 0])
        assert np.allclose(row_sum, raw.sum(1), rtol=1e-6)


def test_topk_brute_force_all_tie_patterns_tiny():
    vals = [np.float32(-1.0), np.float32(0.0), np.float32(0.5)]
    for E in (2, 3, 4):
        logits = np.array(list(itertools.product(vals, repeat=E)), np.float32)
        for k in range(1, E + 1):
            got = orc.moe_topk_route(logits, k)
            assert np.array_equal(got, py_topk(orc.softmax(logits), k))


def fma32(a, b, c):
    """Correctly rounded fp32 fused multiply-add, by exact rational arithmetic."""
    from fractions import Fraction
    a, b, c = np.broadcast_arrays(np.asarray(a, np.float32), np.asarray(b, np.float32), np.asarray(c, np.float32))
    out = np.empty(a.shape, np.float32)
    for i in np.ndindex(a.shape):
        exact = Fraction(float(a[i])) * Fraction(float(b[i])) + Fraction(float(c[i]))
        guess = np.float32(float(exact))                       # may be double-rounded: repair against the neighbours
        cands = [guess, np.nextafter(guess, np.float32(np.inf)), np.nextafter(guess, np.float32(-np.inf))]
        best = min(cands, key=lambda v: (abs(Fraction(float(v)) - exact), int(np.float32(v).view(np.uint32)) & 1))
        out[i] = best
    return out


def test_row_lists_offsets_gather_scatter():
    rng = np.random.default_rng(2)
    rows, E, k, H = 301, 16, 3, 24
    rw = orc.moe_topk_route(rng.standard_normal((rows, E)).astype(np.float32), k)
    counts, idx = orc.moe_build_expert_row_lists(rw)
    assert counts.sum() == rows * k
    for e in range(E):
        want = np.nonzero(rw[:, e] > 0)[0]
        assert counts[e] == len(want) and np.array_equal(idx[e, : counts[e]], want)   # ascending rows
        assert np.all(idx[e, counts[e]:] == -1)                                        # tail untouched
    off = orc.moe_expert_offsets(counts)
    assert np.array_equal(off, np.concatenate([[0], np.cumsum(counts)[:-1]]))
    src8 = rng.integers(0, 256, (rows, H)).astype(np.uint8)
    assert np.array_equal(orc.moe_gather_rows_u8(src8, idx[3, : counts[3]]), src8[idx[3, : counts[3]]])
    src16 = rng.integers(0, 65536, (rows, H)).astype(np.uint16)
    assert np.array_equal(orc.moe_gather_rows_bf16(src16, idx[5, : counts[5]]), src16[idx[5, : counts[5]]])
    # weighted unpermute: one FUSED multiply-add and one bf16 rounding per element, only selected rows change
    mixed = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))
    compact = orc.bf16_from_f32(rng.standard_normal((counts[3], H)).astype(np.float32))
    out = orc.moe_scatter_accumulate(mixed, compact, rw, idx[3, : counts[3]], 3)
    sel = idx[3, : counts[3]]
    want = mixed.copy()
    want[sel] = orc.bf16_from_f32(fma32(rw[sel, 3][:, None], orc.bf16_to_f32(compact), orc.bf16_to_f32(mixed[sel])))
    assert np.array_equal(out, want)
    dense = orc.moe_scale_accumulate(mixed, mixed, rw, 3)
    assert np.array_equal(dense, orc.bf16_from_f32(fma32(rw[:, 3][:, None], orc.bf16_to_f32(mixed), orc.bf16_to_f32(mixed))))


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_gemm_reference_reduces_to_numpy_matmul(mode):
    rng = np.random.default_rng(3 + mode)
    M, N, K = 37, 150, 300
    A = rng.integers(0, 0x7f, (M, K)).astype(np.uint8) | (rng.integers(0, 2, (M, K)).astype(np.uint8) << 7)
    B = rng.integers(0, 0x7f, (N, K)).astype(np.uint8) | (rng.integers(0, 2, (N, K)).astype(np.uint8) << 7)
    A[(A & 0x7f) == 0x7f] = 0x10
    B[(B & 0x7f) == 0x7f] = 0x10
    kb = (K + 127) // 128
    if mode == 0:
        sa, sb = np.array([0.37], np.float32), np.array([1.9], np.float32)
        fa, fb = sa[0], sb[0]
    elif mode == 1:
        sa, sb = rng.uniform(0.1, 2, M).astype(np.float32), rng.uniform(0.1, 2, N).astype(np.float32)
        fa, fb = sa[:, None], sb[:, None]
    else:
        sa = rng.uniform(0.1, 2, (M, kb)).astype(np.float32)
        sb = rng.uniform(0.1, 2, ((N + 127) // 128, kb)).astype(np.float32)
        fa = np.repeat(sa, 128, axis=1)[:, :K]
        fb = np.repeat(np.repeat(sb, 128, axis=0)[:N], 128, axis=1)[:, :K]
    ref, absdot = orc.gemm_nt_ref(A, B, sa, sb, scale_mode=mode)
    a = (orc.e4m3_unpack(A) * fa).astype(np.float32).astype(np.float64)
    b = (orc.e4m3_unpack(B) * fb).astype(np.float32).astype(np.float64)
    want = a @ b.T
    assert np.max(np.abs(ref - want)) <= 1e-9 * np.abs(want).max()
    assert np.max(np.abs(absdot - np.abs(a) @ np.abs(b).T)) <= 1e-9 * absdot.max()
    # E5M2 A operand and a padded row stride
    Apad = np.concatenate([A, np.full((M, 20), 0x7f, np.uint8)], axis=1)
    ref5, _ = orc.gemm_nt_ref(Apad, B, np.array([1.0], np.float32), np.array([1.0], np.float32), a_e5m2=True, lda=K + 20)
    a5 = orc.e5m2_unpack(A).astype(np.float64)
    a5[~np.isfinite(a5)] = np.nan
    ok = np.isfinite(a5).all(1)
    want5 = np.nan_to_num(a5) @ orc.e4m3_unpack(B).astype(np.float64).T
    assert np.allclose(ref5[ok], want5[ok], rtol=1e-12, atol=0)


def test_linear_forward_is_sequential_fp32_dot_and_thread_invariant():
    rng = np.random.default_rng(5)
    T, K, N = 19, 257, 33
    x = rng.standard_normal((T, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    y1 = orc.linear_forward_f32(x, w, threads=1)
    y8 = orc.linear_forward_f32(x, w, threads=8)
    assert np.array_equal(y1, y8)
    acc = np.zeros((T, N), np.float32)
    for k in range(K):
        acc = (acc + (x[:, k][:, None] * w[:, k][None, :]).astype(np.float32)).astype(np.float32)
    assert np.array_equal(y1, orc.bf16_from_f32(acc))
    bias = orc.bf16_from_f32(rng.standard_normal(N).astype(np.float32))
    yb = orc.linear_forward_f32(x, w, bias=bias, threads=3)
    assert np.array_equal(yb, orc.bf16_from_f32(orc.bf16_to_f32(y1) + orc.bf16_to_f32(bias)[None, :]))


def test_grouped_gelu_expert_reference_against_numpy():
    from math import erf
    rng = np.random.default_rng(6)
    rows, H, Ie, E, k = 40, 32, 24, 4, 2
    hidden = orc.e4m3_satfinite(rng.standard_normal((rows, H)).astype(np.float32) * 50)
    w_in = orc.e4m3_satfinite(rng.standard_normal((E, Ie, H)).astype(np.float32) * 50)
    w_out = orc.e4m3_satfinite(rng.standard_normal((E, H, Ie)).astype(np.float32) * 50)
    dh, din, dout = np.float32(0.02), np.float32(0.004), np.float32(0.005)
    rw = orc.moe_topk_route(rng.standard_normal((rows, E)).astype(np.float32), k)
    counts, idx = orc.moe_build_expert_row_lists(rw)
    mixed0 = rng.standard_normal((rows, H))
    got = orc.moe_grouped_expert_forward_fp8_ref(hidden, dh, False, rw, counts, idx, w_in, din, w_out, dout, mixed0)
    h = (orc.e4m3_unpack(hidden) * dh).astype(np.float64)
    want = mixed0.copy()
    gelu = np.vectorize(lambda v: 0.5 * v * (1 + erf(v / np.sqrt(2))))
    for e in range(E):
        wi = (orc.e4m3_unpack(w_in[e]) * din).astype(np.float64)
        wo = (orc.e4m3_unpack(w_out[e]) * dout).astype(np.float64)
        sel = np.nonzero(rw[:, e] > 0)[0]
        want[sel] += rw[sel, e][:, None].astype(np.float64) * (gelu(h[sel] @ wi.T) @ wo.T)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)


def test_expert_bank_formula_against_the_reference_fixture():
    """The reference's own router-parity case also holds the expert bank's inputs and its output `mixed`
    (tests/fixtures/moe_router_parity).  It fixes what the grouped expert forward computes:
    mixed = trunk(h) + sum_e w[sample, e] * fc_out_e(gelu_erf(fc_in_e(h))), weights laid out [E, Ie, H] and [E, H, Ie].
    (1) a float64 restatement reproduces `mixed` with the exact-erf GELU and visibly not with the tanh form;
    (2) the oracle's FP8 expert-bank reference, fed the same operands quantized to E4M3, lands on mixed - trunk to
        within the quantization error: a transposed weight or a dropped route weight would be off by the full scale."""
    import math
    g = json.loads((GOLD / "moe_expert_bank.json").read_text())
    hg, rw, mixed = np.array(g["hidden_gated"]), np.array(g["route_weights"]), np.array(g["mixed"])
    tin, tout = np.array(g["trunk_fc_in_w"]), np.array(g["trunk_fc_out_w"])
    ein, eout = np.array(g["expert_fc_in_w"]), np.array(g["expert_fc_out_w"])
    B, S, H = hg.shape
    E, Ie, _ = ein.shape
    erf = np.vectorize(math.erf)
    gelu_erf = lambda x: 0.5 * x * (1.0 + erf(x / math.sqrt(2.0)))
    gelu_tanh = lambda x: 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))

    def bank(act):
        out = np.zeros_like(mixed)
        for e in range(E):
            out += rw[:, None, e:e + 1] * (act(hg @ ein[e].T) @ eout[e].T)
        return out
    trunk = gelu_erf(hg @ tin.T) @ tout.T
    assert np.abs(trunk + bank(gelu_erf) - mixed).max() < 1e-6
    assert np.abs(gelu_tanh(hg @ tin.T) @ tout.T + bank(gelu_tanh) - mixed).max() > 5e-5
    want = (mixed - trunk).reshape(B * S, H)

    rows = B * S
    route = np.repeat(rw, S, axis=0).astype(np.float32)              # the route weight is per sample: every token of it
    counts, idx = orc.moe_build_expert_row_lists(route)

    def q(x):                                                        # per-tensor E4M3 as the reference's slots do
        amax = np.float32(np.abs(x).max())
        s, d = orc.scale_from_amax(amax, 448.0)
        return orc.e4m3_satfinite((x.astype(np.float32) * s).astype(np.float32)).reshape(x.shape), d
    hq, hd = q(hg.reshape(rows, H))
    wiq, wid = q(ein)
    woq, wod = q(eout)
    got = orc.moe_grouped_expert_forward_fp8_ref(hq, hd, False, route, counts, idx, wiq, wid, woq, wod, np.zeros((rows, H)))
    scale = np.abs(want).max()
    assert np.abs(got - want).max() < 0.06 * scale, (np.abs(got - want).max(), scale)      # measured: 0.027
    # sensitivity: the same call with the experts' weights in the wrong order misses by much more
    wrong = orc.moe_grouped_expert_forward_fp8_ref(hq, hd, False, route, counts, idx, wiq[::-1].copy(), wid, woq, wod, np.zeros((rows, H)))
    assert np.abs(wrong - want).max() > 0.3 * scale


def test_expert_bank_bf16_ref_on_the_reference_fixture():
    """The bf16 sibling's reference against the same fixture: with the operands rounded to bf16 it lands on the
    fixture's `mixed` minus its trunk term to bf16 rounding of the operands (2^-9 each), and a transposed expert
    order misses by far more; with two experts' rows swapped in the lists it changes."""
    import math
    g = json.loads((GOLD / "moe_expert_bank.json").read_text())
    hg, rw, mixed = np.array(g["hidden_gated"]), np.array(g["route_weights"]), np.array(g["mixed"])
    tin, tout = np.array(g["trunk_fc_in_w"]), np.array(g["trunk_fc_out_w"])
    ein, eout = np.array(g["expert_fc_in_w"]), np.array(g["expert_fc_out_w"])
    B, S, H = hg.shape
    rows = B * S
    erf = np.vectorize(math.erf)
    trunk = (lambda x: 0.5 * x * (1.0 + erf(x / math.sqrt(2.0))))(hg @ tin.T) @ tout.T
    want = (mixed - trunk).reshape(rows, H)
    route = np.repeat(rw, S, axis=0).astype(np.float32)
    counts, idx = orc.moe_build_expert_row_lists(route)
    b = lambda x: orc.bf16_from_f32(x.astype(np.float32))
    got = orc.moe_grouped_expert_forward_bf16_ref(b(hg.reshape(rows, H)), route, counts, idx, b(ein), b(eout), np.zeros((rows, H)))
    scale = np.abs(want).max()
    assert np.abs(got - want).max() < 0.01 * scale, (np.abs(got - want).max(), scale)
    wrong = orc.moe_grouped_expert_forward_bf16_ref(b(hg.reshape(rows, H)), route, counts, idx, b(ein)[::-1].copy(), b(eout),
                                                    np.zeros((rows, H)))
    assert np.abs(wrong - want).max() > 0.3 * scale
