"""GPU parity: the scaled FP8 GEMM against the CPU oracle (matmul of the dequantised operands,
carried in double).  Bar: relative L2 error <= 1e-3 and max error <= 2 bf16 ulps of |ref|
(see oracle_lib.assert_gemm_close for the accumulation-order term near cancellation)."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_arr, dev_bf16, host, scalar, stream

pytestmark = pytest.mark.gpu

PER_TENSOR, ROW_COL = 0, 1
EPI_NONE, EPI_BIAS, EPI_SILU = 0, 1, 2
NAIVE = 1


def rand_fp8(rng, shape, e5m2=False, sigma=1.0):
    """Quantised operand bytes drawn like a real tensor: N(0, sigma) scaled to the format's range."""
    x = (rng.standard_normal(shape) * sigma).astype(np.float32)
    fmax = 57344.0 if e5m2 else 448.0
    s = np.float32(fmax) / np.abs(x).max()
    q = orc.e5m2_satfinite(x * s) if e5m2 else orc.e4m3_satfinite(x * s)
    return q, np.float32(1.0) / s


def silu_ref(gate_ref, up_ref):
    """The reference epilogue on exact inputs: bf16(gate), bf16(up) -> bf16(silu*up) (kernels/activations.cu:28-40)."""
    g = orc.bf16_to_f32(orc.bf16_from_f32(gate_ref.astype(np.float32))).astype(np.float64)
    u = orc.bf16_to_f32(orc.bf16_from_f32(up_ref.astype(np.float32))).astype(np.float64)
    return g / (1.0 + np.exp(-g)) * u


def run_gemm(cf, dev, A, B, sa, sb, *, lda=None, a_e5m2=False, mode=PER_TENSOR, epi=EPI_NONE, bias=None,
             B2=None, sb2=None, flags=0, ldc=None):
    M, K = A.shape[0], B.shape[1]
    N = B.shape[0]
    lda = A.shape[1] if lda is None else lda
    ldc = N if ldc is None else ldc
    Ad, Bd = dev_arr(A, dev), dev_arr(B, dev)
    C = torch.full((M, ldc), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, Ad, lda, int(a_e5m2), dev_arr(np.atleast_1d(sa).astype(np.float32), dev),
                              Bd, K, dev_arr(np.atleast_1d(sb).astype(np.float32), dev), mode, epi,
                              None if bias is None else dev_bf16(bias, dev),
                              None if B2 is None else dev_arr(B2, dev),
                              None if sb2 is None else dev_arr(np.atleast_1d(sb2).astype(np.float32), dev),
                              C, ldc, flags, stream())
    torch.cuda.synchronize()
    return orc.bf16_to_f32(bf16_bits(C)).astype(np.float64)


# (300, 512, 512) and (770, 256, 384): persistent kernel with a ragged last row tile; (1024, 1024, 256): several tiles per workgroup, two K-tiles;
# (300, 264, 512), (512, 1000, 384), (256, 8, 256): persistent kernel with a last column tile that N cuts short at a multiple of 8
SHAPES = [(256, 256, 128), (512, 768, 1024), (300, 200, 144), (1, 1, 16), (33, 500, 208), (257, 129, 4096), (64, 1408, 2048),
          (300, 512, 512), (770, 256, 384), (1024, 1024, 256), (300, 264, 512), (512, 1000, 384), (256, 8, 256)]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("flags", [0, NAIVE])
def test_gemm_per_tensor(cf, dev, M, N, K, flags):
    case(f"gemm per-tensor {M}x{N}x{K} flags={flags}")
    rng = np.random.default_rng(M + N + K)
    A, sa = rand_fp8(rng, (M, K))
    B, sb = rand_fp8(rng, (N, K), sigma=0.02)
    got = run_gemm(cf, dev, A, B, sa, sb, flags=flags)
    ref, absdot = orc.gemm_nt_ref(A, B, [sa], [sb])
    orc.assert_gemm_close(got, ref, absdot, what=f"{M}x{N}x{K}", acc=orc.ACC_FP32 if flags else orc.ACC_MFMA)
    # without any allowance: only cancellation points (|ref| << sum|a b|) may exceed 2 bf16 ulps
    off = np.abs(got - ref) > 2 * orc.bf16_ulp(ref)
    assert off.mean() <= 0.03 and np.all(np.abs(ref[off]) <= 2.0 ** -9 * absdot[off])


@pytest.mark.parametrize("epi", [EPI_NONE, EPI_BIAS])
def test_gemm_short_last_column_tile_leaves_row_padding_alone(cf, dev, epi):
    """N = 3 x 256 + 136 with rows of C padded to ldc > N: the persistent kernel stores whole 8-column chunks up to
    N and nothing after it; the element-per-thread kernel is the cross-check."""
    case(f"gemm N=904 ldc=960 epi={epi}")
    rng = np.random.default_rng(904)
    M, N, K, ldc = 300, 904, 512, 960
    A, _ = rand_fp8(rng, (M, K))
    B, _ = rand_fp8(rng, (N, K), sigma=0.02)
    sa = rng.uniform(0.001, 0.02, M).astype(np.float32)
    sb = rng.uniform(1e-5, 1e-4, N).astype(np.float32)
    bias = orc.bf16_from_f32((rng.standard_normal(N) * 1e-3).astype(np.float32)) if epi == EPI_BIAS else None
    got = run_gemm(cf, dev, A, B, sa, sb, mode=ROW_COL, epi=epi, bias=bias, ldc=ldc)
    naive = run_gemm(cf, dev, A, B, sa, sb, mode=ROW_COL, epi=epi, bias=bias, ldc=ldc, flags=NAIVE)
    assert np.all(np.isnan(got[:, N:])) and not np.any(np.isnan(got[:, :N]))
    ref, absdot = orc.gemm_nt_ref(A, B, sa, sb, scale_mode=1)
    if epi == EPI_BIAS:
        # bias is added to the bf16-rounded product: exact given the plain result
        plain = run_gemm(cf, dev, A, B, sa, sb, mode=ROW_COL, ldc=ldc)[:, :N]
        want = orc.bf16_to_f32(orc.bf16_from_f32((plain + orc.bf16_to_f32(bias)[None, :].astype(np.float64)).astype(np.float32)))
        assert np.array_equal(got[:, :N], want)
    else:
        orc.assert_gemm_close(got[:, :N], ref, absdot)
    assert np.all(np.isnan(naive[:, N:]))
    assert np.mean(got[:, :N] != naive[:, :N]) < 0.25      # two accumulation orders: mostly the same bf16 value


def test_gemm_exact_small_integers_equals_numpy_matmul(cf, dev):
    """All scales 1 and operands small integers: every product and partial sum is exact in fp32,
    so the GEMM must equal numpy's matmul to the last bit of the bf16 rounding."""
    case("gemm exact integers")
    rng = np.random.default_rng(0)
    M, N, K = 256, 512, 256
    ai = rng.integers(-3, 4, (M, K)).astype(np.float32)
    bi = rng.integers(-2, 3, (N, K)).astype(np.float32)
    A, B = orc.e4m3_satfinite(ai), orc.e4m3_satfinite(bi)
    got = run_gemm(cf, dev, A, B, 1.0, 1.0)
    want = orc.bf16_to_f32(orc.bf16_from_f32((ai @ bi.T).astype(np.float32)))
    assert np.array_equal(got, want)
    # a transposed or misindexed operand cannot pass this: the matrix is far from symmetric
    assert not np.array_equal(got[:256, :256], got[:256, :256].T)


@pytest.mark.parametrize("flags", [0, NAIVE])
def test_gemm_e5m2_activations_and_row_stride(cf, dev, flags):
    case(f"gemm e5m2 A + lda flags={flags}")
    rng = np.random.default_rng(5)
    M, N, K, lda = 200, 300, 512, 512 + 64
    A, sa = rand_fp8(rng, (M, lda), e5m2=True, sigma=1e-3)
    B, sb = rand_fp8(rng, (N, K), sigma=0.02)
    got = run_gemm(cf, dev, A, B, sa, sb, lda=lda, a_e5m2=True, flags=flags, ldc=N + 8)[:, :N]
    ref, absdot = orc.gemm_nt_ref(A, B, [sa], [sb], a_e5m2=True, lda=lda)
    orc.assert_gemm_close(got, ref, absdot)


@pytest.mark.parametrize("M,N,K", [(300, 260, 384), (300, 512, 384), (1100, 256, 640), (300, 264, 384), (520, 904, 640)])
@pytest.mark.parametrize("flags", [0, NAIVE])
def test_gemm_row_col_scales_and_bias(cf, dev, M, N, K, flags):
    case(f"gemm row/col scales + bias {M}x{N}x{K} flags={flags}")
    rng = np.random.default_rng(6)
    A, _ = rand_fp8(rng, (M, K))
    B, _ = rand_fp8(rng, (N, K), sigma=0.02)
    sa = rng.uniform(0.001, 0.02, M).astype(np.float32)
    sb = rng.uniform(1e-5, 1e-4, N).astype(np.float32)
    got = run_gemm(cf, dev, A, B, sa, sb, mode=ROW_COL, flags=flags)
    ref, absdot = orc.gemm_nt_ref(A, B, sa, sb, scale_mode=1)
    orc.assert_gemm_close(got, ref, absdot)
    bias = orc.bf16_from_f32((rng.standard_normal(N) * np.abs(ref).mean()).astype(np.float32))
    gotb = run_gemm(cf, dev, A, B, sa, sb, mode=ROW_COL, epi=EPI_BIAS, bias=bias, flags=flags)
    # bias is added to the bf16-rounded product (GEMM then bias_add_strided_bf16): exact given the plain result
    want = orc.bf16_to_f32(orc.bf16_from_f32((got + orc.bf16_to_f32(bias)[None, :].astype(np.float64)).astype(np.float32)))
    assert np.array_equal(gotb, want)


@pytest.mark.parametrize("M,N,K", [(256, 128, 256), (300, 200, 512), (512, 1408, 2048), (300, 256, 512), (1024, 384, 256)])
@pytest.mark.parametrize("mode", [PER_TENSOR, ROW_COL])
def test_gemm_fused_silu_gate(cf, dev, M, N, K, mode):
    case(f"gemm silu-gate {M}x{N}x{K} mode={mode}")
    rng = np.random.default_rng(M + N + mode)
    A, sa = rand_fp8(rng, (M, K))
    Bg, sg = rand_fp8(rng, (N, K), sigma=0.02)
    Bu, su = rand_fp8(rng, (N, K), sigma=0.02)
    if mode == ROW_COL:
        sa = (sa * rng.uniform(0.5, 2, M)).astype(np.float32)
        sg = (sg * rng.uniform(0.5, 2, N)).astype(np.float32)
        su = (su * rng.uniform(0.5, 2, N)).astype(np.float32)
    fused = run_gemm(cf, dev, A, Bg, sa, sg, mode=mode, epi=EPI_SILU, B2=Bu, sb2=su)
    # (1) identical to running the two plain GEMMs and the stand-alone swiglu kernel
    gate = run_gemm(cf, dev, A, Bg, sa, sg, mode=mode)
    up = run_gemm(cf, dev, A, Bu, sa, su, mode=mode)
    want = orc.bf16_to_f32(orc.swiglu_forward(orc.bf16_from_f32(gate.astype(np.float32)), orc.bf16_from_f32(up.astype(np.float32)))).astype(np.float64)
    # the fused epilogue evaluates the sigmoid on the hardware exp2 / reciprocal (1 ulp fp32 each): the bf16
    # result may land on the neighbouring value when the product sits at a rounding boundary
    assert np.all(np.abs(fused - want) <= orc.bf16_ulp(want)) and (fused != want).mean() < 0.01
    naive = run_gemm(cf, dev, A, Bg, sa, sg, mode=mode, epi=EPI_SILU, B2=Bu, sb2=su, flags=NAIVE)
    # the cross-check kernel uses the reproducible expf: bit-exact against the oracle's swiglu of ITS gate / up
    gate_n = run_gemm(cf, dev, A, Bg, sa, sg, mode=mode, flags=NAIVE)
    up_n = run_gemm(cf, dev, A, Bu, sa, su, mode=mode, flags=NAIVE)
    want_n = orc.bf16_to_f32(orc.swiglu_forward(orc.bf16_from_f32(gate_n.astype(np.float32)), orc.bf16_from_f32(up_n.astype(np.float32))))
    assert np.array_equal(naive, want_n)
    # (2) close to the exact-input reference epilogue; gate/up each carry <= 1 bf16 ulp of input rounding
    gref, _ = orc.gemm_nt_ref(A, Bg, np.atleast_1d(sa), np.atleast_1d(sg), scale_mode=mode, want_abs=False)
    uref, _ = orc.gemm_nt_ref(A, Bu, np.atleast_1d(sa), np.atleast_1d(su), scale_mode=mode, want_abs=False)
    exact = silu_ref(gref, uref)
    for got in (fused, naive):
        rel = np.sqrt(((got - exact) ** 2).sum() / (exact ** 2).sum())
        assert rel <= 4e-3, rel      # three bf16 roundings (gate, up, product): ~2^-9 * sqrt(3) relative


DUO, DUO_IN_STEP = 4, 12


# (300, 256, 384): ragged last row tile, three K-tiles; (1100, 384, 256): two K-tiles (the copy stream a whole tile ahead);
# (3000, 768, 512): more tiles than workgroups; (128, 128, 1024): a single tile
@pytest.mark.parametrize("M,N,K", [(300, 256, 384), (1100, 384, 256), (3000, 768, 512), (128, 128, 1024), (520, 512, 640)])
@pytest.mark.parametrize("epi", [EPI_NONE, EPI_SILU])
def test_gemm_two_workgroups_per_cu_kernel_matches_the_ring_kernel(cf, dev, M, N, K, epi):
    """CF_GEMM_FLAG_DUO: the 128 x 128-tile kernel accumulates every output over the same sequence of MFMA steps as the
    256 x 256-tile kernel and runs the same epilogue arithmetic, so the bits are the same; started in step or half a tile apart."""
    case(f"gemm duo {M}x{N}x{K} epi={epi}")
    rng = np.random.default_rng(M + N + K + epi)
    A, sa = rand_fp8(rng, (M, K))
    Bg, sg = rand_fp8(rng, (N, K), sigma=0.02)
    Bu, su = rand_fp8(rng, (N, K), sigma=0.02)
    sa = (sa * rng.uniform(0.5, 2, M)).astype(np.float32)
    sg = (sg * rng.uniform(0.5, 2, N)).astype(np.float32)
    su = (su * rng.uniform(0.5, 2, N)).astype(np.float32)
    kw = dict(mode=ROW_COL, epi=epi, B2=Bu if epi == EPI_SILU else None, sb2=su if epi == EPI_SILU else None)
    ring = run_gemm(cf, dev, A, Bg, sa, sg, **kw)
    assert np.array_equal(run_gemm(cf, dev, A, Bg, sa, sg, flags=DUO, **kw), ring)
    assert np.array_equal(run_gemm(cf, dev, A, Bg, sa, sg, flags=DUO_IN_STEP, **kw), ring)
    if epi == EPI_NONE:
        ref, absdot = orc.gemm_nt_ref(A, Bg, sa, sg, scale_mode=ROW_COL)
        orc.assert_gemm_close(ring, ref, absdot, what=f"duo {M}x{N}x{K}")
    # a row stride wider than N: the padding stays untouched
    wide = run_gemm(cf, dev, A, Bg, sa, sg, flags=DUO, ldc=N + 40, **kw)
    assert np.array_equal(wide[:, :N], ring) and np.isnan(wide[:, N:]).all()


MFMA32 = 16


# (300, 256, 384): ragged last row tile, three K-tiles (odd); (1100, 384, 256): two K-tiles; (3000, 768, 512): more tiles than
# workgroups; (520, 904, 640): a last column tile cut short at a multiple of 8, five K-tiles; (257, 128, 4096): 32 K-tiles
@pytest.mark.parametrize("M,N,K", [(300, 256, 384), (1100, 384, 256), (3000, 768, 512), (520, 904, 640), (257, 128, 4096)])
@pytest.mark.parametrize("epi", [EPI_NONE, EPI_BIAS, EPI_SILU])
@pytest.mark.parametrize("mode", [PER_TENSOR, ROW_COL])
def test_gemm_both_mfma_shapes_of_the_ring_kernel(cf, dev, M, N, K, epi, mode):
    """The persistent kernel exists on two MFMA shapes: v_mfma_f32_16x16x128_f8f6f4 (the default for the bf16 epilogues)
    and v_mfma_f32_32x32x64_f8f6f4 (CF_GEMM_FLAG_MFMA32; also what the accumulate and term-split forms run on).  Same
    tiles, same drain arithmetic; the two differ at most by the order in which a K-tile's 128 products are added."""
    if epi == EPI_SILU and N % 128:
        pytest.skip("the fused gate/up form keeps whole column tiles on either kernel")
    case(f"gemm 16x16x128 / 32x32x64 {M}x{N}x{K} epi={epi} mode={mode}")
    rng = np.random.default_rng(M + N + K + 3 * epi + mode)
    A, sa = rand_fp8(rng, (M, K))
    Bg, sg = rand_fp8(rng, (N, K), sigma=0.02)
    Bu, su = rand_fp8(rng, (N, K), sigma=0.02)
    if mode == ROW_COL:
        sa = (sa * rng.uniform(0.5, 2, M)).astype(np.float32)
        sg = (sg * rng.uniform(0.5, 2, N)).astype(np.float32)
        su = (su * rng.uniform(0.5, 2, N)).astype(np.float32)
    bias = orc.bf16_from_f32((rng.standard_normal(N) * 0.05).astype(np.float32)) if epi == EPI_BIAS else None
    kw = dict(mode=mode, epi=epi, bias=bias, B2=Bu if epi == EPI_SILU else None, sb2=su if epi == EPI_SILU else None)
    new = run_gemm(cf, dev, A, Bg, sa, sg, ldc=N + 24, **kw)
    old = run_gemm(cf, dev, A, Bg, sa, sg, flags=MFMA32, ldc=N + 24, **kw)
    assert np.isnan(new[:, N:]).all() and np.isnan(old[:, N:]).all()
    new, old = new[:, :N], old[:, :N]
    if epi == EPI_NONE:
        ref, absdot = orc.gemm_nt_ref(A, Bg, np.atleast_1d(sa), np.atleast_1d(sg), scale_mode=mode)
        orc.assert_gemm_close(new, ref, absdot, what=f"16x16x128 {M}x{N}x{K}")
        orc.assert_gemm_close(old, ref, absdot, what=f"32x32x64 {M}x{N}x{K}")
    # against each other: the same value, or neighbouring bf16 values where the accumulation order moves a sum across a
    # rounding boundary (gate, up and product each round once in the fused form)
    tol = (3 if epi == EPI_SILU else 1) * np.maximum(orc.bf16_ulp(old), orc.bf16_ulp(new))
    assert np.all(np.abs(new - old) <= tol), float(np.abs(new - old).max())
    assert (new != old).mean() < 0.02


def test_gemm_exact_integers_on_both_mfma_shapes(cf, dev):
    case("gemm exact small integers, 16x16x128 and 32x32x64")
    rng = np.random.default_rng(21)
    M, N, K = 520, 384, 640
    ai = rng.integers(-3, 4, (M, K)).astype(np.float32)
    bi = rng.integers(-2, 3, (N, K)).astype(np.float32)
    A, B = orc.e4m3_satfinite(ai), orc.e4m3_satfinite(bi)
    want = orc.bf16_to_f32(orc.bf16_from_f32((ai @ bi.T).astype(np.float32))).astype(np.float64)
    one = np.float32(1.0)
    for flags in (0, MFMA32):
        assert np.array_equal(run_gemm(cf, dev, A, B, one, one, flags=flags), want), flags


def test_gemm_duo_flag_on_other_shapes_takes_the_usual_kernels(cf, dev):
    case("gemm duo flag on shapes the kernel does not take")
    rng = np.random.default_rng(9)
    A, sa = rand_fp8(rng, (300, 384))
    B, sb = rand_fp8(rng, (200, 384), sigma=0.02)                # N not a multiple of 128
    assert np.array_equal(run_gemm(cf, dev, A, B, sa, sb, flags=DUO), run_gemm(cf, dev, A, B, sa, sb))
    B, sb = rand_fp8(rng, (256, 384), sigma=0.02)                # per-tensor scales
    assert np.array_equal(run_gemm(cf, dev, A, B, sa, sb, flags=DUO), run_gemm(cf, dev, A, B, sa, sb))


def test_gemm_config2_shape_sampled_rows_and_naive_crosscheck(cf, dev):
    """M=8192, K=4096, N=14336 (the benchmark shape): per-token / per-channel scales, outliers at +-40."""
    case("gemm config 2 full size")
    M, N, K = 8192, 14336, 4096
    g = torch.Generator(device=dev).manual_seed(22)
    x = torch.randn((M, K), generator=g, device=dev)
    u = torch.rand((M, K), generator=g, device=dev)
    x = torch.where(u < 0.0005, torch.full_like(x, 40.0), x)
    x = torch.where(u > 0.9995, torch.full_like(x, -40.0), x).to(torch.bfloat16)
    w = (torch.randn((N, K), generator=g, device=dev) * 0.02).to(torch.bfloat16)
    xq = torch.empty((M, K), dtype=torch.uint8, device=dev); xs = torch.empty(M, device=dev); xd = torch.empty(M, device=dev)
    wq = torch.empty((N, K), dtype=torch.uint8, device=dev); ws = torch.empty(N, device=dev); wd = torch.empty(N, device=dev)
    cf.cf_fp8_quantize_rows(x, M, K, 0, xq, xs, xd, stream())
    cf.cf_fp8_quantize_rows(w, N, K, 0, wq, ws, wd, stream())
    C = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    Cn = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wq, K, wd, ROW_COL, EPI_NONE, None, None, None, C, N, 0, stream())
    cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wq, K, wd, ROW_COL, EPI_NONE, None, None, None, Cn, N, NAIVE, stream())
    torch.cuda.synchronize()
    # tiled vs naive over the whole output: both are fp32 accumulations of the same products
    diff = (C.float() - Cn.float()).abs()
    ulp = torch.maximum(Cn.float().abs(), torch.tensor(1e-30, device=dev)).log2().floor().sub(7).exp2()
    frac_off = (diff > 2 * ulp).float().mean().item()
    assert frac_off < 5e-3, frac_off      # cancellation points only: the MFMA keeps fewer bits than an fp32 FMA chain
    rel = (diff.double().pow(2).sum() / Cn.double().pow(2).sum()).sqrt().item()
    assert rel < 1e-3
    # sampled rows against the CPU oracle
    rows = np.sort(np.random.default_rng(1).choice(M, 48, replace=False))
    ridx = torch.from_numpy(rows).to(dev)
    ref, absdot = orc.gemm_nt_ref(host(xq[ridx]), host(wq), host(xd[ridx]), host(wd), scale_mode=1)
    got = orc.bf16_to_f32(bf16_bits(C[ridx])).astype(np.float64)
    orc.assert_gemm_close(got, ref, absdot, what="config 2 sampled rows")
    report_strict("config 2 gate projection (plain epilogue)", got, ref)


def silu_grad(g):
    """d/dg of g * sigmoid(g)."""
    sg = 1.0 / (1.0 + np.exp(-g))
    return sg * (1.0 + g * (1.0 - sg))


def report_strict(config, got, ref):
    """Prints the fraction of elements beyond 2 bf16 ulps of |ref| with no accumulation allowance at all (the bar as
    literally stated); the assertions use assert_gemm_close, which adds the accumulation term at cancellation points."""
    frac = orc.strict_ulp_fraction(got, ref)
    print(f"[strict-2ulp] {config}: {frac:.3e} of {got.size} elements beyond 2 bf16 ulps of |ref|", flush=True)
    return frac


def test_config1_linear_forward_end_to_end(cf, dev):
    """Config 1 through the library end to end: X fp32 [512,1024] ~ N(0,1), W fp32 [1024,1024] ~ N(0,0.02), per-tensor
    amax -> scale -> E4M3 bytes, Y = dequant(X) . dequant(W)^T as bf16.  Bytes and scales bit-exact; Y against the
    CPU path's scalar fp32 loop over the dequantised operands (src/cpu_trainer.cpp:89-108, 306-324) and against the
    double-precision matmul."""
    case("config 1 end to end")
    rng = np.random.default_rng(11)
    T, K, N = 512, 1024, 1024
    x = rng.standard_normal((T, K)).astype(np.float32)
    w = (0.02 * rng.standard_normal((N, K))).astype(np.float32)
    got_q = []
    for t in (x, w):
        td = torch.from_numpy(t).to(dev)
        amax, scale, desc = scalar(0.0, dev), scalar(0.0, dev), scalar(0.0, dev)
        q = torch.empty(t.shape, dtype=torch.uint8, device=dev)
        cf.cf_fp8_amax_f32(td, t.size, amax, stream())
        cf.cf_fp8_scale_from_amax(amax, 448.0, scale, desc, stream())
        cf.cf_fp8_quantize_f32_e4m3(td, q, scale, t.size, stream())
        torch.cuda.synchronize()
        want_amax = orc.amax_f32(t)
        assert want_amax == np.float32(np.abs(t).max())
        want_scale, want_desc = orc.scale_from_amax(want_amax, 448.0)
        assert host(amax)[0] == want_amax and host(scale)[0] == want_scale and host(desc)[0] == want_desc
        assert np.array_equal(host(q), orc.quantize_f32_e4m3(t, want_scale))
        got_q.append((q, desc))
    (xq, xd), (wq, wd) = got_q
    y = torch.full((T, N), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16(T, N, K, xq, K, 0, xd, wq, wd, y, N, stream())
    torch.cuda.synchronize()
    got = orc.bf16_to_f32(bf16_bits(y)).astype(np.float64)
    # (1) the stated bar against the double-precision matmul of the dequantised operands
    ref, absdot = orc.gemm_nt_ref(host(xq), host(wq), host(xd), host(wd))
    orc.assert_gemm_close(got, ref, absdot, what="config 1 Y")
    report_strict("config 1 Y", got, ref)
    # (2) the CPU path itself: scalar fp32 dot in k order over the dequantised fp32 operands, bf16 output; the two
    # fp32 accumulation orders may land on neighbouring bf16 values at rounding boundaries, never further apart
    xf = orc.dequant(host(xq), host(xd)[0])
    wf = orc.dequant(host(wq), host(wd)[0])
    cpu = orc.bf16_to_f32(orc.linear_forward_f32(xf, wf, threads=4)).astype(np.float64)
    assert np.all(np.abs(got - cpu) <= orc.bf16_ulp(cpu) + orc.ACC_MFMA * absdot)
    assert (got != cpu).mean() < 0.02


def test_config2_full_size_step(cf, dev):
    """The step the benchmark times, at its size, checked link by link: per-token quantize of X -> fused gate/up GEMM
    with the SiLU-gate epilogue (M=8192, K=4096, N=14336, per-token x per-channel scales) -> per-token quantize of H ->
    down projection (K=14336, N=4096)."""
    case("config 2 full-size step")
    M, K, N = 8192, 4096, 14336
    g = torch.Generator(device=dev).manual_seed(2)
    x = torch.randn((M, K), generator=g, device=dev)
    u = torch.rand((M, K), generator=g, device=dev)
    x = torch.where(u < 0.0005, torch.full_like(x, 40.0), x)
    x = torch.where(u > 0.9995, torch.full_like(x, -40.0), x).to(torch.bfloat16)
    del u

    def qrows(t):
        r, c = t.shape
        q = torch.empty((r, c), dtype=torch.uint8, device=dev)
        s = torch.empty(r, device=dev); d = torch.empty(r, device=dev)
        cf.cf_fp8_quantize_rows(t, r, c, 0, q, s, d, stream())
        return q, s, d

    def wquant(rows, cols):
        w = (torch.randn((rows, cols), generator=g, device=dev) * 0.02).to(torch.bfloat16)
        q, _, d = qrows(w)
        return q, d

    wgq, wgd = wquant(N, K)
    wuq, wud = wquant(N, K)
    wdq, wdd = wquant(K, N)
    xq, xs, xd = qrows(x)
    h = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wgq, K, wgd, ROW_COL, EPI_SILU, None, wuq, wud, h, N, 0, stream())
    hq, hs, hd = qrows(h)
    y = torch.full((M, K), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16_ex(M, K, N, hq, N, 0, hd, wdq, N, wdd, ROW_COL, EPI_NONE, None, None, None, y, K, 0, stream())
    torch.cuda.synchronize()
    rows = np.sort(np.random.default_rng(12).choice(M, 40, replace=False))
    ridx = torch.from_numpy(rows).to(dev)

    # link 1: X bytes and scales, bit-exact on sampled rows (the quantize tests cover the kernel exhaustively)
    oq, os_, od = orc.quantize_rows(bf16_bits(x[ridx]))
    assert np.array_equal(host(xq[ridx]), oq) and np.array_equal(host(xs[ridx]), os_) and np.array_equal(host(xd[ridx]), od)

    # link 2a: the fused kernel against the one-lane-per-output kernel over the WHOLE of H: same products, two fp32
    # accumulation orders, the reproducible expf instead of the hardware exp2 / reciprocal
    hn = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wgq, K, wgd, ROW_COL, EPI_SILU, None, wuq, wud, hn, N, NAIVE, stream())
    torch.cuda.synchronize()
    assert not torch.isnan(h).any()
    hf, hnf = h.float(), hn.float()
    diff = (hf - hnf).abs()
    ulp = torch.maximum(hnf.abs(), torch.tensor(1e-30, device=dev)).log2().floor().sub(7).exp2()
    frac_off = (diff > 2 * ulp).float().mean().item()
    rel = (diff.double().pow(2).sum() / hnf.double().pow(2).sum()).sqrt().item()
    print(f"[config 2 step] H fused vs naive over {M * N} elements: rel L2 {rel:.3e}, beyond 2 ulp {frac_off:.3e}", flush=True)
    assert rel < 2e-3 and frac_off < 2e-2
    del hn, hf, hnf, diff, ulp

    # link 2b: sampled rows of H against the reference epilogue on the exact (double) gate / up products
    xr, xdr = host(xq[ridx]), host(xd[ridx])
    gref, gabs = orc.gemm_nt_ref(xr, host(wgq), xdr, host(wgd), scale_mode=1)
    uref, uabs = orc.gemm_nt_ref(xr, host(wuq), xdr, host(wud), scale_mode=1)
    exact = silu_ref(gref, uref)
    got_h = orc.bf16_to_f32(bf16_bits(h[ridx])).astype(np.float64)
    rel = np.sqrt(((got_h - exact) ** 2).sum() / (exact ** 2).sum())
    assert rel <= 4e-3, rel        # three bf16 roundings (gate, up, product): ~2^-9 * sqrt(3) relative
    # elementwise.  `exact` rounds the exact gate and up to bf16 itself, so without accumulation error the kernel could
    # differ only by its own rounding and the hardware sigmoid: one ulp of the larger of the two values (a result that
    # rounds up into the next binade is half of ITS ulp away).  The MFMA's accumulation error moves gate and up before
    # they are rounded: by the accumulation allowance itself (it dominates where the dot product cancels), and by a
    # whole ulp of that input when it flips the bf16 rounding (on the percent of elements that sit that close to a
    # rounding boundary).  That is the loose bound; the tight one may be exceeded only on a few percent.
    g16 = orc.bf16_to_f32(orc.bf16_from_f32(gref.astype(np.float32))).astype(np.float64)
    u16 = orc.bf16_to_f32(orc.bf16_from_f32(uref.astype(np.float32))).astype(np.float64)
    err = np.abs(got_h - exact)
    tight = orc.bf16_ulp(np.maximum(np.abs(exact), np.abs(got_h)))
    sg = g16 / (1.0 + np.exp(-g16))
    dg = orc.bf16_ulp(g16) + orc.ACC_MFMA * gabs
    du = orc.bf16_ulp(u16) + orc.ACC_MFMA * uabs
    # |silu'| <= 1.1 everywhere and silu is convex-concave with |silu''| <= 0.5: second order covers dg that is not small
    loose = tight + (np.abs(silu_grad(g16)) * dg + 0.25 * dg * dg) * (np.abs(u16) + du) + np.abs(sg) * du
    assert np.all(err <= 1.05 * loose), float((err / loose).max())
    flips = float((err > 1.05 * tight).mean())
    print(f"[config 2 step] H sampled rows: {flips:.3e} of elements beyond one ulp (an input's bf16 rounding flipped)", flush=True)
    assert flips < 0.03
    report_strict("config 2 H (fused SiLU-gate, against silu of the exact gate / up)", got_h, exact)

    # link 3: Hq bytes and scales bit-exact against the oracle's quantize of the GPU's own H
    sel = np.sort(np.random.default_rng(13).choice(M, 512, replace=False))
    sidx = torch.from_numpy(sel).to(dev)
    oq, os_, od = orc.quantize_rows(bf16_bits(h[sidx]))
    assert np.array_equal(host(hq[sidx]), oq) and np.array_equal(host(hs[sidx]), os_) and np.array_equal(host(hd[sidx]), od)

    # link 4: the down projection on sampled rows against the oracle on the GPU's own Hq
    ref, absdot = orc.gemm_nt_ref(host(hq[ridx]), host(wdq), host(hd[ridx]), host(wdd), scale_mode=1)
    got_y = orc.bf16_to_f32(bf16_bits(y[ridx])).astype(np.float64)
    assert not torch.isnan(y).any()
    orc.assert_gemm_close(got_y, ref, absdot, what="config 2 down projection, sampled rows")
    report_strict("config 2 Y (down projection)", got_y, ref)


def test_gemm_argument_errors(cf, dev):
    a = torch.zeros(16, dtype=torch.uint8, device=dev)
    c = torch.zeros(16, dtype=torch.bfloat16, device=dev)
    s = scalar(1.0, dev)
    assert cf.raw_cf_fp8_gemm_nt_bf16(-1, 1, 16, a.data_ptr(), 16, 0, s.data_ptr(), a.data_ptr(), s.data_ptr(), c.data_ptr(), 1, None) == -1
    assert cf.raw_cf_fp8_gemm_nt_bf16(1, 1, 16, None, 16, 0, s.data_ptr(), a.data_ptr(), s.data_ptr(), c.data_ptr(), 1, None) == -1
    assert cf.raw_cf_fp8_gemm_nt_bf16(1, 1, 16, a.data_ptr(), 8, 0, s.data_ptr(), a.data_ptr(), s.data_ptr(), c.data_ptr(), 1, None) == -1
    assert cf.raw_cf_fp8_gemm_nt_bf16(0, 1, 16, a.data_ptr(), 16, 0, s.data_ptr(), a.data_ptr(), s.data_ptr(), c.data_ptr(), 1, None) == 0


# ---- backward-pass GEMMs (benchmark config 4) ------------------------------------------------
def run_accum(cf, dev, A, B, sa, sb, C0, *, a_e5m2, b_e5m2, flags=0, bf16_out=False, ldc=None):
    M, K = A.shape
    N = B.shape[0]
    ldc = N if ldc is None else ldc
    s = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    if bf16_out:
        C = dev_bf16(orc.bf16_from_f32(C0.astype(np.float32)), dev)
        assert a_e5m2 is False and b_e5m2 is True
        cf.cf_fp8_gemm_tn_accum_bf16(M, N, K, dev_arr(A, dev), s(sa), dev_arr(B, dev), s(sb), C, ldc, stream())
        torch.cuda.synchronize()
        return orc.bf16_to_f32(bf16_bits(C)).astype(np.float64)
    C = torch.from_numpy(C0.astype(np.float32)).to(dev)
    cf.cf_fp8_gemm_nt_accum_f32_ex(M, N, K, dev_arr(A, dev), K, int(a_e5m2), s(sa), dev_arr(B, dev), K, int(b_e5m2), s(sb),
                                   C, ldc, flags, stream())
    torch.cuda.synchronize()
    return host(C).astype(np.float64)


@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (300, 200, 384), (512, 1024, 2048), (130, 260, 80), (300, 512, 512), (1024, 768, 256)])
@pytest.mark.parametrize("flags", [0, NAIVE])
def test_wgrad_tn_accumulate_f32(cf, dev, M, N, K, flags):
    """dW[M,N] fp32 += X^T[M,K](E4M3) . dY^T[N,K](E5M2)^T, beta = 1 (lt_gemm_fp8_tn_accum_f32)."""
    case(f"wgrad accumulate f32 {M}x{N}x{K} flags={flags}")
    rng = np.random.default_rng(M + N + K + flags)
    Xt, sx = rand_fp8(rng, (M, K))
    dYt, sy = rand_fp8(rng, (N, K), e5m2=True, sigma=1e-3)
    C0 = rng.standard_normal((M, N)) * 1e-3
    ref, absdot = orc.gemm_nt_ref(Xt, dYt, [sx], [sy], b_e5m2=True)
    got = run_accum(cf, dev, Xt, dYt, sx, sy, C0, a_e5m2=False, b_e5m2=True, flags=flags)
    want = C0.astype(np.float32).astype(np.float64) + ref
    # fp32 output: relative L2 against the unrounded reference, elementwise within the accumulation allowance
    rel = np.sqrt(((got - want) ** 2).sum() / (want ** 2).sum())
    assert rel <= 1e-3, rel
    acc = orc.ACC_FP32 if flags else orc.ACC_MFMA
    assert np.all(np.abs(got - want) <= acc * absdot + 2.0 ** -22 * (np.abs(want) + np.abs(C0)))
    if flags == 0 and K % 128 == 0:
        # the named entry point is the same kernel
        C = torch.from_numpy(C0.astype(np.float32)).to(dev)
        s = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
        cf.cf_fp8_gemm_tn_accum_f32(M, N, K, dev_arr(Xt, dev), s(sx), dev_arr(dYt, dev), s(sy), C, N, stream())
        torch.cuda.synchronize()
        assert np.array_equal(host(C).astype(np.float64), got)


@pytest.mark.parametrize("M,N,K", [(300, 260, 512), (300, 512, 512), (1024, 768, 256), (700, 256, 1152)])
def test_wgrad_tn_accumulate_bf16(cf, dev, M, N, K):
    """N a multiple of 256 takes the persistent kernel (ragged last row tile included), 260 the staged one."""
    case(f"wgrad accumulate bf16 {M}x{N}x{K}")
    rng = np.random.default_rng(77 + M + N + K)
    Xt, sx = rand_fp8(rng, (M, K))
    dYt, sy = rand_fp8(rng, (N, K), e5m2=True, sigma=1e-3)
    ref, absdot = orc.gemm_nt_ref(Xt, dYt, [sx], [sy], b_e5m2=True)
    C0 = rng.standard_normal((M, N)) * np.abs(ref).mean()
    got = run_accum(cf, dev, Xt, dYt, sx, sy, C0, a_e5m2=False, b_e5m2=True, bf16_out=True)
    want = orc.bf16_to_f32(orc.bf16_from_f32(C0.astype(np.float32))).astype(np.float64) + ref
    assert np.all(np.abs(got - want) <= 1.01 * orc.bf16_ulp(want) / 2 + orc.ACC_MFMA * absdot)


def test_config4_backward_shapes_sampled(cf, dev):
    """dgrad: dY[8192,14336] E5M2 (per-tensor, ~N(0,1e-3)) . W[4096,14336] E4M3 -> bf16 [8192,4096];
    wgrad: dY^T[14336... as X^T[14336,8192] E4M3 . dY^T[4096,8192] E5M2 accumulated into fp32 [14336,4096]."""
    case("config 4 backward, full size")
    g = torch.Generator(device=dev).manual_seed(4)
    M, N, K = 8192, 4096, 14336
    dy = (torch.randn((M, K), generator=g, device=dev) * 1e-3).to(torch.bfloat16)
    w = (torch.randn((N, K), generator=g, device=dev) * 0.02).to(torch.bfloat16)
    sc = lambda: torch.zeros(1, device=dev)
    amax, s_dy, d_dy, s_w, d_w = sc(), sc(), sc(), sc(), sc()
    dyq = torch.empty((M, K), dtype=torch.uint8, device=dev); wq = torch.empty((N, K), dtype=torch.uint8, device=dev)
    cf.cf_fp8_amax_bf16(dy, dy.numel(), amax, stream()); cf.cf_fp8_scale_from_amax(amax, 57344.0, s_dy, d_dy, stream())
    cf.cf_fp8_quantize_e5m2(dy, dyq, s_dy, dy.numel(), stream())
    cf.cf_fp8_amax_bf16(w, w.numel(), amax, stream()); cf.cf_fp8_scale_from_amax(amax, 448.0, s_w, d_w, stream())
    cf.cf_fp8_quantize_e4m3(w, wq, s_w, w.numel(), stream())
    dx = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16(M, N, K, dyq, K, 1, d_dy, wq, d_w, dx, N, stream())
    torch.cuda.synchronize()
    assert host(amax)[0] > 0 and np.array_equal(host(dyq), orc.quantize_e5m2(bf16_bits(dy), host(s_dy)[0]))
    rows = np.sort(np.random.default_rng(2).choice(M, 32, replace=False)); ridx = torch.from_numpy(rows).to(dev)
    ref, absdot = orc.gemm_nt_ref(host(dyq[ridx]), host(wq), host(d_dy), host(d_w), a_e5m2=True)
    got_dx = orc.bf16_to_f32(bf16_bits(dx[ridx])).astype(np.float64)
    orc.assert_gemm_close(got_dx, ref, absdot, what="config 4 dgrad")
    report_strict("config 4 dgrad", got_dx, ref)
    del dx, w, wq
    # wgrad: M=14336, N=4096, K=8192, both operands K-contiguous (pre-transposed); dY^T via the byte transpose
    Mw, Nw, Kw = 14336, 4096, 8192
    x = torch.randn((Kw, Mw), generator=g, device=dev).to(torch.bfloat16)          # swiglu_out [tokens, I]
    s_x, d_x = sc(), sc()
    cf.cf_fp8_amax_bf16(x, x.numel(), amax, stream()); cf.cf_fp8_scale_from_amax(amax, 448.0, s_x, d_x, stream())
    act8 = torch.empty((Kw, Mw), dtype=torch.uint8, device=dev); snap = torch.empty((Mw, Kw), dtype=torch.uint8, device=dev)
    cf.cf_fp8_quant_and_transpose_e4m3(x, act8, snap, s_x, Kw, Mw, stream())          # X^T [14336, 8192]
    dyh = (torch.randn((Kw, Nw), generator=g, device=dev) * 1e-3).to(torch.bfloat16)  # dY [tokens, H]
    cf.cf_fp8_amax_bf16(dyh, dyh.numel(), amax, stream()); cf.cf_fp8_scale_from_amax(amax, 57344.0, s_dy, d_dy, stream())
    dyhq = torch.empty((Kw, Nw), dtype=torch.uint8, device=dev); dyt = torch.empty((Nw, Kw), dtype=torch.uint8, device=dev)
    cf.cf_fp8_quantize_e5m2(dyh, dyhq, s_dy, dyh.numel(), stream())
    cf.cf_transpose_u8(dyhq, dyt, Kw, Nw, stream())                                   # dY^T [4096, 8192]
    dW = torch.full((Mw, Nw), 0.125, device=dev)
    cf.cf_fp8_gemm_tn_accum_f32(Mw, Nw, Kw, snap, d_x, dyt, d_dy, dW, Nw, stream())
    torch.cuda.synchronize()
    assert torch.equal(snap, act8.t()) and torch.equal(dyt, dyhq.t())                 # the transposes are permutations
    rows = np.sort(np.random.default_rng(3).choice(Mw, 32, replace=False)); ridx = torch.from_numpy(rows).to(dev)
    ref, absdot = orc.gemm_nt_ref(host(snap[ridx]), host(dyt), host(d_x), host(d_dy), b_e5m2=True)
    got = host(dW[ridx]).astype(np.float64)
    want = 0.125 + ref
    assert np.sqrt(((got - want) ** 2).sum() / (want ** 2).sum()) <= 1e-3
    assert np.all(np.abs(got - want) <= orc.ACC_MFMA * absdot + 2.0 ** -22 * (np.abs(want) + 0.125))


# ---- block-scaled GEMM (benchmark config 3) ----------------------------------------------------
BLOCK = 2


def block_quant_gpu(cf, dev, x_bf16, kind):
    rows, K = x_bf16.shape
    kb = (K + 127) // 128
    q = torch.empty((rows, K), dtype=torch.uint8, device=dev)
    shape = (rows, kb) if kind == "1x128" else ((rows + 127) // 128, kb)
    s = torch.empty(shape, device=dev); d = torch.empty(shape, device=dev)
    fn = cf.cf_fp8_quantize_block_1x128 if kind == "1x128" else cf.cf_fp8_quantize_block_128x128
    fn(x_bf16, rows, K, q, s, d, stream())
    return q, s, d


# (300, 512, 640), (1000, 256, 384), (3000, 768, 512): the persistent kernel (ragged rows; three K-tiles per tile; many tiles per workgroup)
@pytest.mark.parametrize("M,N,K", [(128, 256, 128), (256, 256, 256), (300, 200, 384), (130, 260, 208), (64, 512, 1024),
                                   (300, 512, 640), (1000, 256, 384), (3000, 768, 512)])
@pytest.mark.parametrize("flags", [0, NAIVE])
def test_gemm_block_scaled(cf, dev, M, N, K, flags):
    case(f"gemm block-scaled {M}x{N}x{K} flags={flags}")
    rng = np.random.default_rng(M * 3 + N + K)
    xb = orc.bf16_from_f32((rng.standard_normal((M, K)) * np.exp(rng.standard_normal((M, 1)))).astype(np.float32))
    wb = orc.bf16_from_f32((0.02 * rng.standard_normal((N, K))).astype(np.float32))
    xq, xs, xd = block_quant_gpu(cf, dev, dev_bf16(xb, dev), "1x128")
    wq, ws, wd = block_quant_gpu(cf, dev, dev_bf16(wb, dev), "128x128")
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wq, K, wd, BLOCK, EPI_NONE, None, None, None, C, N, flags, stream())
    torch.cuda.synchronize()
    # the quantized operands and scales are bit-exact (checked in the quantize tests); reference on the same bytes
    oq, osx, odx = orc.quantize_block_1x128(xb)
    assert np.array_equal(host(xq), oq) and np.array_equal(host(xd), odx)
    ref, absdot = orc.gemm_nt_ref(host(xq), host(wq), host(xd), host(wd), scale_mode=2)
    got = orc.bf16_to_f32(bf16_bits(C)).astype(np.float64)
    orc.assert_gemm_close(got, ref, absdot, what=f"block {M}x{N}x{K}", acc=orc.ACC_FP32 * 4 if flags else orc.ACC_MFMA)


@pytest.mark.parametrize("pad", [4, 2, 8])
def test_gemm_block_scaled_row_strides_of_c(cf, dev, pad):
    """The persistent block-scaled kernel stores whole 128-byte lines when C's rows allow 16-byte accesses and falls
    back to 8-byte or 2-byte stores otherwise: the same bits in all three, and the padding of C's rows untouched."""
    case(f"gemm block-scaled, ldc = N + {pad}")
    M, N, K = 300, 512, 640
    rng = np.random.default_rng(pad)
    xb = orc.bf16_from_f32(rng.standard_normal((M, K)).astype(np.float32))
    wb = orc.bf16_from_f32((0.02 * rng.standard_normal((N, K))).astype(np.float32))
    xq, xs, xd = block_quant_gpu(cf, dev, dev_bf16(xb, dev), "1x128")
    wq, ws, wd = block_quant_gpu(cf, dev, dev_bf16(wb, dev), "128x128")
    C0 = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wq, K, wd, BLOCK, EPI_NONE, None, None, None, C0, N, 0, stream())
    C1 = torch.full((M, N + pad), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wq, K, wd, BLOCK, EPI_NONE, None, None, None, C1, N + pad, 0, stream())
    torch.cuda.synchronize()
    got = bf16_bits(C1)
    assert np.array_equal(got[:, :N], bf16_bits(C0))
    assert np.all((got[:, N:] & 0x7fff) > 0x7f80)


def test_config3_block_scaled_full_size_sampled(cf, dev):
    """M=4096, N=7168, K=7168; activations 1x128 groups, weights 128x128 blocks, fp32 scale tensors."""
    case("config 3 block-scaled, full size")
    M, N, K = 4096, 7168, 7168
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn((M, K), generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn((N, K), generator=g, device=dev) * 0.02).to(torch.bfloat16)
    xq, xs, xd = block_quant_gpu(cf, dev, x, "1x128")
    wq, ws, wd = block_quant_gpu(cf, dev, w, "128x128")
    C = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wq, K, wd, BLOCK, EPI_NONE, None, None, None, C, N, 0, stream())
    torch.cuda.synchronize()
    rows = np.sort(np.random.default_rng(6).choice(M, 24, replace=False)); ridx = torch.from_numpy(rows).to(dev)
    ref, absdot = orc.gemm_nt_ref(host(xq[ridx]), host(wq), host(xd[ridx]), host(wd), scale_mode=2)
    got_c3 = orc.bf16_to_f32(bf16_bits(C[ridx])).astype(np.float64)
    orc.assert_gemm_close(got_c3, ref, absdot, what="config 3 sampled rows")
    report_strict("config 3 block-scaled", got_c3, ref)
    # weight block scales against the oracle on a few blocks
    wb = bf16_bits(w[:256, :256])
    oq, _, od = orc.quantize_block_128x128(wb)
    assert np.array_equal(host(wq[:256, :256]), oq) and np.array_equal(host(wd[:2, :2]), od)
