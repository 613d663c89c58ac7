"""GPU parity: the bf16 GEMMs of the selected-expert MoE backward (gemm_bf16 / gemm_bf16_tn_f32 of
src/trainer.cu:3069-3160 as called at :7727-7740), dense and grouped per expert, against the matmul of the
same bf16 operands carried in double.  The reference's cuBLAS calls accumulate in fp32 in an order that is
not defined, so the bar is the GEMM bar of the FP8 path: the bf16 results within half a bf16 ulp of the
double reference plus an fp32 accumulation allowance; exactly summable operands must match to the bit."""
import ctypes

import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_arr, dev_bf16, host, stream

pytestmark = pytest.mark.gpu

ACC = 16.0 * 2.0 ** -24          # fp32 accumulation on the matrix cores, as a multiple of sum |a_k b_k|


def rand_bf16(rng, shape, sigma=1.0):
    return orc.bf16_from_f32((rng.standard_normal(shape) * sigma).astype(np.float32))


def absdot(A, B, tn=False):
    a = np.abs(orc.bf16_to_f32(A).astype(np.float64))
    b = np.abs(orc.bf16_to_f32(B).astype(np.float64))
    return (a.T if tn else a) @ b


def check_bf16_out(got_bits, ref, ad, what):
    got = orc.bf16_to_f32(got_bits).astype(np.float64)
    tol = 0.505 * orc.bf16_ulp(np.maximum(np.abs(ref), np.abs(got))) + ACC * ad
    bad = np.abs(got - ref) > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} outside tolerance, worst {float((np.abs(got - ref) / tol).max()):.3f}"


def padded(bits, ld):
    """[r, c] bit patterns -> [r, ld] with NaN padding (a kernel that reads the padding shows up)."""
    out = np.full((bits.shape[0], ld), 0x7fc0, np.uint16)
    out[:, :bits.shape[1]] = bits
    return out


@pytest.mark.parametrize("M,N,K,pad", [(256, 128, 64, 0), (300, 200, 136, 8), (1, 8, 8, 0), (513, 264, 1000, 16), (1024, 1408, 2048, 0),
                                       (40, 136, 72, 0)])
def test_gemm_bf16_nn(cf, dev, M, N, K, pad):
    case(f"bf16 nn {M}x{N}x{K} pad {pad}")
    rng = np.random.default_rng(M + N + K)
    A, B = rand_bf16(rng, (M, K)), rand_bf16(rng, (K, N), 0.02)
    lda, ldb, ldc = K + pad, N + pad, N + pad
    C = torch.full((M, ldc), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_gemm_bf16_nn(M, N, K, dev_bf16(padded(A, lda), dev), lda, dev_bf16(padded(B, ldb), dev), ldb, C, ldc, stream())
    torch.cuda.synchronize()
    got = bf16_bits(C)
    assert np.all((got[:, N:] & 0x7fff) > 0x7f80)                      # row padding of C left alone
    check_bf16_out(got[:, :N], orc.gemm_bf16_nn_ref(A, B), absdot(A, B), f"nn {M}x{N}x{K}")


def test_gemm_bf16_exact_integers_equal_numpy(cf, dev):
    """Small integers: every product and partial sum is exact in fp32, so all three forms must match numpy to the
    bit; the operands are far from symmetric, so a transposed or misindexed operand cannot pass."""
    case("bf16 GEMMs, exact integers")
    rng = np.random.default_rng(3)
    M, N, K = 300, 264, 200
    a = rng.integers(-4, 5, (M, K)).astype(np.float32)
    b = rng.integers(-3, 4, (K, N)).astype(np.float32)
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_gemm_bf16_nn(M, N, K, dev_bf16(orc.bf16_from_f32(a), dev), K, dev_bf16(orc.bf16_from_f32(b), dev), N, C, N, stream())
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(C), orc.bf16_from_f32((a @ b).astype(np.float32)))
    # tn: C[M2,N2] += A2[K2,M2]^T . B2[K2,N2]
    K2, M2, N2 = 333, 264, 136
    a2 = rng.integers(-4, 5, (K2, M2)).astype(np.float32)
    b2 = rng.integers(-3, 4, (K2, N2)).astype(np.float32)
    c0 = rng.integers(-50, 51, (M2, N2)).astype(np.float32)
    Cf = torch.from_numpy(c0).to(dev)
    cf.cf_gemm_bf16_tn_accum_f32(M2, N2, K2, dev_bf16(orc.bf16_from_f32(a2), dev), M2, dev_bf16(orc.bf16_from_f32(b2), dev), N2, Cf, N2, stream())
    Cb = dev_bf16(orc.bf16_from_f32(c0), dev)
    cf.cf_gemm_bf16_tn_accum_bf16(M2, N2, K2, dev_bf16(orc.bf16_from_f32(a2), dev), M2, dev_bf16(orc.bf16_from_f32(b2), dev), N2, Cb, N2, stream())
    torch.cuda.synchronize()
    want = c0 + a2.T @ b2
    assert np.array_equal(host(Cf), want)
    assert np.array_equal(bf16_bits(Cb), orc.bf16_from_f32(want))
    assert not np.array_equal(want[:136, :136], want[:136, :136].T)


@pytest.mark.parametrize("K", [64, 72, 200])
def test_gemm_bf16_more_tiles_than_workgroups_exact(cf, dev, K):
    """306 output tiles on at most 256 persistent workgroups: a workgroup walks from one tile into the next with its
    operand fetch two K-tiles ahead (at K = 64 and 72 a tile has one or two real K-tiles, so the fetch is two tiles
    ahead of the MFMAs).  Small integers, exact in fp32: all three forms must match numpy to the bit."""
    case(f"bf16 GEMMs, 306 tiles, K={K}")
    rng = np.random.default_rng(K)
    M, N = 17 * 256, 17 * 256 + 8
    a = rng.integers(-4, 5, (M, K)).astype(np.float32)
    b = rng.integers(-3, 4, (K, N)).astype(np.float32)
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_gemm_bf16_nn(M, N, K, dev_bf16(orc.bf16_from_f32(a), dev), K, dev_bf16(orc.bf16_from_f32(b), dev), N, C, N, stream())
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(C), orc.bf16_from_f32(a @ b))
    # tn: the same product from the transposed left operand, added to C
    at = np.ascontiguousarray(a.T)
    c0 = rng.integers(-50, 51, (M, N)).astype(np.float32)
    Cf = torch.from_numpy(c0).to(dev)
    cf.cf_gemm_bf16_tn_accum_f32(M, N, K, dev_bf16(orc.bf16_from_f32(at), dev), M, dev_bf16(orc.bf16_from_f32(b), dev), N, Cf, N, stream())
    Cb = dev_bf16(orc.bf16_from_f32(c0), dev)
    cf.cf_gemm_bf16_tn_accum_bf16(M, N, K, dev_bf16(orc.bf16_from_f32(at), dev), M, dev_bf16(orc.bf16_from_f32(b), dev), N, Cb, N, stream())
    torch.cuda.synchronize()
    want = c0 + a @ b
    assert np.array_equal(host(Cf), want)
    assert np.array_equal(bf16_bits(Cb), orc.bf16_from_f32(want))


def test_gemm_bf16_seeded_shapes_exact(cf, dev):
    """Forty seeded shapes (ragged rows, columns and k, padded strides; some with several tiles per workgroup), small
    integers: the dense forms against numpy, to the bit."""
    rng = np.random.default_rng(2024)
    for it in range(40):
        M = int(rng.integers(1, 900)); N = 8 * int(rng.integers(1, 90)); K = 8 * int(rng.integers(1, 60))
        pa, pb, pc = (8 * int(rng.integers(0, 3)) for _ in range(3))
        case(f"bf16 nn seeded {it}: {M}x{N}x{K} pads {pa} {pb} {pc}")
        a = rng.integers(-4, 5, (M, K)).astype(np.float32)
        b = rng.integers(-3, 4, (K, N)).astype(np.float32)
        C = torch.full((M, N + pc), float("nan"), dtype=torch.bfloat16, device=dev)
        cf.cf_gemm_bf16_nn(M, N, K, dev_bf16(padded(orc.bf16_from_f32(a), K + pa), dev), K + pa,
                           dev_bf16(padded(orc.bf16_from_f32(b), N + pb), dev), N + pb, C, N + pc, stream())
        torch.cuda.synchronize()
        got = bf16_bits(C)
        assert np.array_equal(got[:, :N], orc.bf16_from_f32(a @ b)), f"nn {M}x{N}x{K}"
        assert np.all((got[:, N:] & 0x7fff) > 0x7f80)
        # tn with the contraction over M rows: C2[K, N2] += a^T . b2, any M
        N2 = 8 * int(rng.integers(1, 60))
        b2 = rng.integers(-3, 4, (M, N2)).astype(np.float32)
        c0 = rng.integers(-50, 51, (K, N2)).astype(np.float32)
        Cf = torch.from_numpy(c0).to(dev)
        Cb = dev_bf16(orc.bf16_from_f32(c0), dev)
        a_dev, b2_dev = dev_bf16(padded(orc.bf16_from_f32(a), K + pa), dev), dev_bf16(orc.bf16_from_f32(b2), dev)
        cf.cf_gemm_bf16_tn_accum_f32(K, N2, M, a_dev, K + pa, b2_dev, N2, Cf, N2, stream())
        cf.cf_gemm_bf16_tn_accum_bf16(K, N2, M, a_dev, K + pa, b2_dev, N2, Cb, N2, stream())
        torch.cuda.synchronize()
        want = c0 + a.T @ b2
        assert np.array_equal(host(Cf), want), f"tn f32 {K}x{N2}x{M}"
        assert np.array_equal(bf16_bits(Cb), orc.bf16_from_f32(want)), f"tn bf16 {K}x{N2}x{M}"


def test_grouped_bf16_seeded_routings_exact(cf, dev):
    """Twenty seeded expert banks (1 to 12 experts of 0 to 400 rows, ragged widths), small integers: both grouped forms
    against numpy per expert, to the bit."""
    rng = np.random.default_rng(77)
    for it in range(20):
        E = int(rng.integers(1, 13)); H = 8 * int(rng.integers(1, 50)); Ie = 8 * int(rng.integers(1, 70))
        counts = rng.integers(0, 401, E).astype(np.int32)
        counts[rng.integers(0, E)] = 0
        offsets = orc.moe_expert_offsets(counts)
        total = int(counts.sum()) + int(rng.integers(0, 300))
        case(f"grouped bf16 seeded {it}: E={E} H={H} Ie={Ie} total={total}")
        if total == 0:
            continue
        d_out = rng.integers(-4, 5, (total, H)).astype(np.float32)
        act = rng.integers(-3, 4, (total, Ie)).astype(np.float32)
        w = rng.integers(-3, 4, (E, H, Ie)).astype(np.float32)
        g0 = rng.integers(-40, 41, (E, H, Ie)).astype(np.float32)
        dc, do = dev_arr(counts, dev), dev_arr(offsets, dev)
        ws, ws_bytes = workspace(cf, dev, total, E)
        d_act = torch.full((total, Ie), float("nan"), dtype=torch.bfloat16, device=dev)
        cf.cf_moe_grouped_gemm_bf16_nn(total, Ie, H, E, dc, do, dev_bf16(orc.bf16_from_f32(d_out), dev), H, dev_bf16(orc.bf16_from_f32(w), dev),
                                       d_act, Ie, ws, ws_bytes, stream())
        g_bf = dev_bf16(orc.bf16_from_f32(g0), dev)
        g_f32 = torch.from_numpy(g0.copy()).to(dev)
        cf.cf_moe_grouped_gemm_bf16_tn_accum_bf16(H, Ie, total, E, dc, do, dev_bf16(orc.bf16_from_f32(d_out), dev), H, dev_bf16(orc.bf16_from_f32(act), dev), Ie, g_bf, stream())
        cf.cf_moe_grouped_gemm_bf16_tn_accum_f32(H, Ie, total, E, dc, do, dev_bf16(orc.bf16_from_f32(d_out), dev), H, dev_bf16(orc.bf16_from_f32(act), dev), Ie, g_f32, stream())
        torch.cuda.synchronize()
        got_act, got_g, got_gf = bf16_bits(d_act), bf16_bits(g_bf), host(g_f32)
        filled = int(counts.sum())
        assert np.all((got_act[filled:] & 0x7fff) > 0x7f80), "rows past the experts' lists were written"
        for e in range(E):
            n, o = int(counts[e]), int(offsets[e])
            want_g = g0[e] + d_out[o:o + n].T @ act[o:o + n]
            assert np.array_equal(got_gf[e], want_g), f"bank {it} expert {e} g (fp32)"
            assert np.array_equal(got_g[e], orc.bf16_from_f32(want_g)), f"bank {it} expert {e} g (bf16)"
            if n:
                assert np.array_equal(got_act[o:o + n], orc.bf16_from_f32(d_out[o:o + n] @ w[e])), f"bank {it} expert {e} d_act"


def test_grouped_bf16_weight_gradient_cuts_row_ranges_at_total_rows(cf, dev):
    """Counts that run past the rows the compact buffers hold (a caller passing an upper bound that is too small):
    the row ranges are cut at total_rows, nothing beyond the buffers is read (NaN rows lie behind them)."""
    case("grouped bf16 wgrad, counts beyond total_rows")
    rng = np.random.default_rng(12)
    E, H, Ie = 4, 136, 264
    counts = np.array([100, 70, 90, 30], np.int32)
    offsets = orc.moe_expert_offsets(counts)
    total = 200                                         # cuts expert 2 after 30 rows and expert 3 entirely
    d_out, act = rand_bf16(rng, (total, H), 1e-2), rand_bf16(rng, (total, Ie))
    nan_rows = np.full((96, max(H, Ie)), 0x7fc0, np.uint16)
    a_dev = dev_bf16(np.concatenate([d_out, nan_rows[:, :H]]), dev)
    b_dev = dev_bf16(np.concatenate([act, nan_rows[:, :Ie]]), dev)
    g0 = rand_bf16(rng, (E, H, Ie), 1e-2)
    g_bf = dev_bf16(g0, dev)
    dc, do = dev_arr(counts, dev), dev_arr(offsets, dev)
    cf.cf_moe_grouped_gemm_bf16_tn_accum_bf16(H, Ie, total, E, dc, do, a_dev, H, b_dev, Ie, g_bf, stream())
    torch.cuda.synchronize()
    got = bf16_bits(g_bf)
    for e in range(E):
        o = min(int(offsets[e]), total)
        n = min(int(counts[e]), total - o)
        if n == 0:
            assert np.array_equal(got[e], g0[e]), f"expert {e}"
            continue
        ref = orc.bf16_to_f32(g0[e]).astype(np.float64) + orc.gemm_bf16_tn_ref(d_out[o:o + n], act[o:o + n])
        check_bf16_out(got[e], ref, absdot(d_out[o:o + n], act[o:o + n], tn=True), f"g_out expert {e}")


def test_grouped_bf16_weight_gradient_leaves_empty_experts_alone(cf, dev):
    """An expert without rows adds nothing: its block of C keeps its bits, negative zeros included (a sum with an
    all-zero product would turn them into +0), also when such experts sit between experts of a few rows each."""
    case("grouped bf16 wgrad, empty experts between short ones")
    rng = np.random.default_rng(11)
    E, H, Ie = 19, 520, 1032                           # 15 tiles per expert, 360 tile positions on 256 workgroups
    counts = np.array([0, 3, 0, 0, 70, 1, 0, 130, 0, 64, 0, 0, 0, 5, 0, 65, 0, 0, 0], np.int32)
    offsets = orc.moe_expert_offsets(counts)
    total = int(counts.sum()) + 7                      # the compact buffers may hold more rows than the lists fill
    d_out, act = rand_bf16(rng, (total, H), 1e-2), rand_bf16(rng, (total, Ie))
    g0 = np.full((E, H, Ie), 0x8000, np.uint16)        # -0.0 everywhere
    g_bf = dev_bf16(g0, dev)
    g_f32 = torch.from_numpy(orc.bf16_to_f32(g0)).to(dev)
    dc, do = dev_arr(counts, dev), dev_arr(offsets, dev)
    cf.cf_moe_grouped_gemm_bf16_tn_accum_bf16(H, Ie, total, E, dc, do, dev_bf16(d_out, dev), H, dev_bf16(act, dev), Ie, g_bf, stream())
    cf.cf_moe_grouped_gemm_bf16_tn_accum_f32(H, Ie, total, E, dc, do, dev_bf16(d_out, dev), H, dev_bf16(act, dev), Ie, g_f32, stream())
    torch.cuda.synchronize()
    got_g, got_gf = bf16_bits(g_bf), host(g_f32)
    for e in range(E):
        n, o = int(counts[e]), int(offsets[e])
        if n == 0:
            assert np.array_equal(got_g[e], g0[e]), f"expert {e}"
            assert np.array_equal(got_gf[e].view(np.uint32), np.full((H, Ie), 0x80000000, np.uint32)), f"expert {e}"
            continue
        ref = orc.gemm_bf16_tn_ref(d_out[o:o + n], act[o:o + n])
        ad = absdot(d_out[o:o + n], act[o:o + n], tn=True)
        check_bf16_out(got_g[e], ref, ad, f"g_out expert {e}")
        assert np.all(np.abs(got_gf[e] - ref) <= ACC * ad + 2.0 ** -22 * np.abs(ref))


@pytest.mark.parametrize("M,N,K", [(256, 128, 64), (264, 200, 131), (8, 8, 1), (1408, 512, 777), (520, 136, 2000)])
def test_gemm_bf16_tn_accumulate(cf, dev, M, N, K):
    case(f"bf16 tn {M}x{N}x{K}")
    rng = np.random.default_rng(M * 3 + N + K)
    A, B = rand_bf16(rng, (K, M), 1e-2), rand_bf16(rng, (K, N))
    ref, ad = orc.gemm_bf16_tn_ref(A, B), absdot(A, B, tn=True)
    c0 = (rng.standard_normal((M, N)) * np.abs(ref).mean()).astype(np.float32)
    Cf = torch.from_numpy(c0).to(dev)
    cf.cf_gemm_bf16_tn_accum_f32(M, N, K, dev_bf16(A, dev), M, dev_bf16(B, dev), N, Cf, N, stream())
    c0b = orc.bf16_from_f32(c0)
    Cb = dev_bf16(c0b, dev)
    cf.cf_gemm_bf16_tn_accum_bf16(M, N, K, dev_bf16(A, dev), M, dev_bf16(B, dev), N, Cb, N, stream())
    torch.cuda.synchronize()
    want = c0.astype(np.float64) + ref
    assert np.all(np.abs(host(Cf).astype(np.float64) - want) <= ACC * ad + 2.0 ** -22 * (np.abs(want) + np.abs(c0)))
    check_bf16_out(bf16_bits(Cb), orc.bf16_to_f32(c0b).astype(np.float64) + ref, ad, f"tn bf16 {M}x{N}x{K}")


def routing(rng, rows, E, k, zero_expert=None):
    logits = rng.standard_normal((rows, E)).astype(np.float32)
    if zero_expert is not None:
        logits[:, zero_expert] = -50.0
    rw = orc.moe_topk_route(logits, k)
    counts, _ = orc.moe_build_expert_row_lists(rw)
    return counts, orc.moe_expert_offsets(counts)


def workspace(cf, dev, total, E):
    sz = ctypes.c_size_t(0)
    assert cf.raw_cf_fp8_grouped_gemm_workspace_bytes(total, E, ctypes.byref(sz)) == 0
    return torch.empty(sz.value, dtype=torch.uint8, device=dev), sz.value


@pytest.mark.parametrize("rows,E,k,H,Ie,zero", [(600, 5, 2, 256, 384, None), (300, 4, 2, 264, 136, 2), (1500, 3, 1, 512, 640, None), (40, 8, 3, 128, 72, None)])
def test_grouped_bf16_backward_gemms(cf, dev, rows, E, k, H, Ie, zero):
    """The four GEMMs of the selected-expert backward over a ragged routing (src/trainer.cu:7727-7740), each expert
    against the double reference, and bit for bit against the dense entry point called per expert the way the
    reference's loop does."""
    case(f"grouped bf16 backward GEMMs rows={rows} E={E} k={k} H={H} Ie={Ie}")
    rng = np.random.default_rng(rows + E + H)
    counts, offsets = routing(rng, rows, E, k, zero)
    total = rows * k
    filled = int(counts.sum())
    d_out = rand_bf16(rng, (total, H), 1e-2)          # d_expert_out, compact
    act = rand_bf16(rng, (total, Ie))                 # post-GELU activations, compact
    w_out = rand_bf16(rng, (E, H, Ie), 0.02)          # fc_out_w [E, H, Ie]
    dc, do = dev_arr(counts, dev), dev_arr(offsets, dev)
    ws, ws_bytes = workspace(cf, dev, total, E)
    # input gradient: d_act[n, Ie] = d_out[n, H] . fc_out_w[e]   (K = H, N = Ie)
    d_act = torch.full((total, Ie), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_moe_grouped_gemm_bf16_nn(total, Ie, H, E, dc, do, dev_bf16(d_out, dev), H, dev_bf16(w_out, dev), d_act, Ie, ws, ws_bytes, stream())
    # weight gradient: g_out[e][H, Ie] += d_out[n, H]^T . act[n, Ie]   (M = H, N = Ie, contraction over the expert's rows)
    g0 = rand_bf16(rng, (E, H, Ie), 1e-2)
    g_bf = dev_bf16(g0, dev)
    g_f32 = torch.from_numpy(orc.bf16_to_f32(g0)).to(dev)
    cf.cf_moe_grouped_gemm_bf16_tn_accum_bf16(H, Ie, total, E, dc, do, dev_bf16(d_out, dev), H, dev_bf16(act, dev), Ie, g_bf, stream())
    cf.cf_moe_grouped_gemm_bf16_tn_accum_f32(H, Ie, total, E, dc, do, dev_bf16(d_out, dev), H, dev_bf16(act, dev), Ie, g_f32, stream())
    torch.cuda.synchronize()
    got_act, got_g, got_gf = bf16_bits(d_act), bf16_bits(g_bf), host(g_f32)
    assert np.all((got_act[filled:] & 0x7fff) > 0x7f80), "rows past the experts' lists were written"
    for e in range(E):
        n, o = int(counts[e]), int(offsets[e])
        if n == 0:
            assert np.array_equal(got_g[e], g0[e]) and np.array_equal(got_gf[e], orc.bf16_to_f32(g0[e]))
            continue
        check_bf16_out(got_act[o:o + n], orc.gemm_bf16_nn_ref(d_out[o:o + n], w_out[e]), absdot(d_out[o:o + n], w_out[e]), f"d_act expert {e}")
        ref = orc.gemm_bf16_tn_ref(d_out[o:o + n], act[o:o + n])
        ad = absdot(d_out[o:o + n], act[o:o + n], tn=True)
        base = orc.bf16_to_f32(g0[e]).astype(np.float64)
        check_bf16_out(got_g[e], base + ref, ad, f"g_out expert {e}")
        assert np.all(np.abs(got_gf[e] - (base + ref)) <= ACC * ad + 2.0 ** -22 * (np.abs(base + ref) + np.abs(base)))
        # the reference's loop: one dense call per expert on that expert's slice
        one = torch.full((n, Ie), float("nan"), dtype=torch.bfloat16, device=dev)
        cf.cf_gemm_bf16_nn(n, Ie, H, dev_bf16(d_out[o:o + n], dev), H, dev_bf16(w_out[e], dev), Ie, one, Ie, stream())
        ge = dev_bf16(g0[e], dev)
        cf.cf_gemm_bf16_tn_accum_bf16(H, Ie, n, dev_bf16(d_out[o:o + n], dev), H, dev_bf16(act[o:o + n], dev), Ie, ge, Ie, stream())
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(one), got_act[o:o + n]) and np.array_equal(bf16_bits(ge), got_g[e])


def test_grouped_bf16_backward_gemms_config5_size(cf, dev):
    """16384 tokens, 64 experts, top-6, H = 2048, Ie = 1408: the four GEMMs at full size, sampled against the
    double reference (every expert, a few rows or weight-gradient rows each)."""
    case("grouped bf16 backward GEMMs, config 5 size")
    rows, E, k, H, Ie = 16384, 64, 6, 2048, 1408
    rng = np.random.default_rng(55)
    counts, offsets = routing(rng, rows, E, k)
    total = rows * k
    g = torch.Generator(device=dev).manual_seed(5)
    d_out = (torch.randn((total, H), generator=g, device=dev) * 1e-2).to(torch.bfloat16)
    d_pre = (torch.randn((total, Ie), generator=g, device=dev) * 1e-2).to(torch.bfloat16)
    x = torch.randn((total, H), generator=g, device=dev).to(torch.bfloat16)
    w_out = (torch.randn((E, H, Ie), generator=g, device=dev) * 0.02).to(torch.bfloat16)
    w_in = (torch.randn((E, Ie, H), generator=g, device=dev) * 0.02).to(torch.bfloat16)
    dc, do = dev_arr(counts, dev), dev_arr(offsets, dev)
    ws, ws_bytes = workspace(cf, dev, total, E)
    d_act = torch.empty((total, Ie), dtype=torch.bfloat16, device=dev)
    d_x = torch.empty((total, H), dtype=torch.bfloat16, device=dev)
    g_out = torch.zeros((E, H, Ie), dtype=torch.bfloat16, device=dev)
    g_in = torch.zeros((E, Ie, H), dtype=torch.bfloat16, device=dev)
    cf.cf_moe_grouped_gemm_bf16_nn(total, Ie, H, E, dc, do, d_out, H, w_out, d_act, Ie, ws, ws_bytes, stream())
    cf.cf_moe_grouped_gemm_bf16_tn_accum_bf16(H, Ie, total, E, dc, do, d_out, H, d_pre, Ie, g_out, stream())
    cf.cf_moe_grouped_gemm_bf16_nn(total, H, Ie, E, dc, do, d_pre, Ie, w_in, d_x, H, ws, ws_bytes, stream())
    cf.cf_moe_grouped_gemm_bf16_tn_accum_bf16(Ie, H, total, E, dc, do, d_pre, Ie, x, H, g_in, stream())
    torch.cuda.synchronize()
    for e in range(0, E, 7):
        n, o = int(counts[e]), int(offsets[e])
        sel = np.sort(np.random.default_rng(e).choice(n, 6, replace=False)) + o
        sidx = torch.from_numpy(sel).to(dev)
        A = bf16_bits(d_out[sidx]); W = bf16_bits(w_out[e])
        check_bf16_out(bf16_bits(d_act[sidx]), orc.gemm_bf16_nn_ref(A, W), absdot(A, W), f"d_act expert {e}")
        A = bf16_bits(d_pre[sidx]); W = bf16_bits(w_in[e])
        check_bf16_out(bf16_bits(d_x[sidx]), orc.gemm_bf16_nn_ref(A, W), absdot(A, W), f"d_x expert {e}")
        # weight gradients: a few output rows (columns of the M-side operand), the whole contraction
        mrows = np.sort(np.random.default_rng(100 + e).choice(Ie, 5, replace=False))
        midx = torch.from_numpy(mrows).to(dev)
        A = bf16_bits(d_out[o:o + n][:, midx]); Bm = bf16_bits(d_pre[o:o + n])
        check_bf16_out(bf16_bits(g_out[e][midx]), orc.gemm_bf16_tn_ref(A, Bm), absdot(A, Bm, tn=True), f"g_out expert {e}")
        A = bf16_bits(d_pre[o:o + n][:, midx]); Bm = bf16_bits(x[o:o + n])
        check_bf16_out(bf16_bits(g_in[e][midx]), orc.gemm_bf16_tn_ref(A, Bm), absdot(A, Bm, tn=True), f"g_in expert {e}")


def test_gemm_bf16_argument_errors(cf, dev):
    a = torch.zeros(64 * 64, dtype=torch.bfloat16, device=dev)
    c = torch.zeros(64 * 64, dtype=torch.bfloat16, device=dev)
    p = lambda t: t.data_ptr()
    assert cf.raw_cf_gemm_bf16_nn(-1, 8, 8, p(a), 8, p(a), 8, p(c), 8, None) == -1
    assert cf.raw_cf_gemm_bf16_nn(8, 8, 8, None, 8, p(a), 8, p(c), 8, None) == -1
    assert cf.raw_cf_gemm_bf16_nn(8, 8, 16, p(a), 8, p(a), 8, p(c), 8, None) == -1          # lda < K
    assert cf.raw_cf_gemm_bf16_nn(8, 12, 8, p(a), 8, p(a), 16, p(c), 16, None) == -2        # N % 8
    assert cf.raw_cf_gemm_bf16_nn(8, 8, 8, p(a) + 2, 8, p(a), 8, p(c), 8, None) == -2       # unaligned operand
    assert cf.raw_cf_gemm_bf16_nn(0, 8, 8, p(a), 8, p(a), 8, p(c), 8, None) == 0
    assert cf.raw_cf_gemm_bf16_nn(1, 8, 8, p(a), 8, p(a), 8, p(c), 1 << 21, None) == -2     # a row stride of C the epilogue's 32-bit offsets do not cover
    assert cf.raw_cf_gemm_bf16_tn_accum_bf16(12, 8, 8, p(a), 16, p(a), 8, p(c), 8, None) == -2   # M % 8
    assert cf.raw_cf_gemm_bf16_tn_accum_bf16(8, 8, 0, p(a), 8, p(a), 8, p(c), 8, None) == 0
    torch.cuda.synchronize()
    assert torch.all(c == 0)
