"""GPU parity: RMSNorm, the row clip and their fusion with the FP8 quantize against the CPU oracle, bit for bit,
through the C ABI (reference sequence: src/trainer.cu:6281-6304)."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_bf16, host, scalar, stream

pytestmark = pytest.mark.gpu

EPS = 1e-6


def make_rows(rows, H, seed, loud_every=5):
    """N(0,1) rows with a spread of row scales; every loud_every-th row is loud enough to be clipped."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, H)).astype(np.float32) * np.exp(rng.standard_normal((rows, 1))).astype(np.float32)
    w = (1.0 + 0.2 * rng.standard_normal(H)).astype(np.float32)
    w[::loud_every] *= 6.0
    return orc.bf16_from_f32(x), orc.bf16_from_f32(w)


def ceiling_for(normed_bits):
    n = orc.bf16_to_f32(normed_bits).astype(np.float64)
    norms = np.sqrt((n * n).sum(axis=1))
    return np.float32(np.percentile(norms, 60))


def oracle_sequence(xb, wb, ceiling, e5m2):
    normed, rms = orc.rmsnorm_forward(xb, wb, EPS)
    clipped, normsq = orc.act_row_clip_abs(normed, ceiling)
    q, s, d = orc.quantize_rows(clipped, e5m2)
    return normed, rms, clipped, normsq, q, s, d


@pytest.mark.parametrize("rows,H", [(1, 32), (7, 96), (33, 512), (5, 520), (9, 516), (64, 1024), (37, 4096), (3, 8192), (2, 16384)])
def test_rmsnorm_forward_matches_oracle(cf, dev, rows, H):
    case(f"rmsnorm rows={rows} H={H}")
    xb, wb = make_rows(rows, H, rows * 131 + H)
    x, w = dev_bf16(xb, dev), dev_bf16(wb, dev)
    out = torch.empty_like(x)
    rms = torch.empty(rows, dtype=torch.float32, device=dev)
    cf.cf_rmsnorm_forward(x, w, out, rms, rows, H, EPS, stream())
    torch.cuda.synchronize()
    want, want_rms = orc.rmsnorm_forward(xb, wb, EPS)
    assert np.array_equal(host(rms).view(np.uint32), want_rms.view(np.uint32))
    assert np.array_equal(bf16_bits(out), want)


def test_rmsnorm_unaligned_rows_and_in_place(cf, dev):
    rows, H = 11, 1032                     # rows start 2 bytes off a 16-byte boundary: the element-wise path
    case("rmsnorm unaligned / in place")
    xb, wb = make_rows(rows, H, 77)
    buf = torch.zeros(rows * H + 8, dtype=torch.bfloat16, device=dev)
    x = buf[1:1 + rows * H]
    x.copy_(dev_bf16(xb, dev).reshape(-1))
    w = dev_bf16(wb, dev)
    cf.cf_rmsnorm_forward(x, w, x, None, rows, H, EPS, stream())
    torch.cuda.synchronize()
    want, _ = orc.rmsnorm_forward(xb, wb, EPS)
    assert np.array_equal(bf16_bits(x).reshape(rows, H), want)
    assert float(buf[0]) == 0.0 and float(buf[1 + rows * H]) == 0.0


@pytest.mark.parametrize("rows,cols", [(4, 32), (6, 96), (9, 256), (21, 1000), (40, 4096), (3, 12288)])
def test_row_clip_matches_oracle(cf, dev, rows, cols):
    case(f"row clip rows={rows} cols={cols}")
    xb, _ = make_rows(rows, cols, rows + cols)
    ceiling = ceiling_for(xb)
    x = dev_bf16(xb, dev)
    normsq = torch.zeros(rows, dtype=torch.float32, device=dev)
    cf.cf_act_row_clip_abs(x, rows, cols, float(ceiling), normsq, stream())
    torch.cuda.synchronize()
    want, want_normsq = orc.act_row_clip_abs(xb, ceiling)
    assert np.any(want != xb) and np.any(np.all(want == xb, axis=1)), "the case must clip some rows and keep others"
    assert np.array_equal(host(normsq).view(np.uint32), want_normsq.view(np.uint32))
    assert np.array_equal(bf16_bits(x), want)
    # a non-positive ceiling leaves everything alone
    y = dev_bf16(xb, dev)
    cf.cf_act_row_clip_abs(y, rows, cols, 0.0, None, stream())
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(y), xb)


@pytest.mark.parametrize("e5m2", [False, True])
@pytest.mark.parametrize("rows,H,clip", [(1, 64, True), (19, 512, True), (8, 776, False), (50, 2048, True), (130, 4096, True),
                                         (130, 4096, False), (6, 5120, True), (7, 7168, True), (4, 8192, True), (5, 1028, True),
                                         (3, 12288, True), (9, 1024, True)])
def test_fused_rows_matches_the_launch_sequence(cf, dev, rows, H, clip, e5m2):
    case(f"fused norm/clip/quantize rows={rows} H={H} clip={clip} e5m2={e5m2}")
    xb, wb = make_rows(rows, H, rows * 7 + H + int(e5m2))
    normed0, _ = orc.rmsnorm_forward(xb, wb, EPS)
    ceiling = ceiling_for(normed0) if clip else np.float32(0.0)
    _, rms_w, clipped_w, _, q_w, s_w, d_w = oracle_sequence(xb, wb, ceiling, e5m2)
    if clip and rows > 4:
        assert np.any(np.any(clipped_w != normed0, axis=1)) and np.any(np.all(clipped_w == normed0, axis=1))
    x, w = dev_bf16(xb, dev), dev_bf16(wb, dev)
    normed = torch.empty_like(x)
    rms = torch.empty(rows, dtype=torch.float32, device=dev)
    q = torch.empty((rows, H), dtype=torch.uint8, device=dev)
    s = torch.empty(rows, dtype=torch.float32, device=dev)
    d = torch.empty(rows, dtype=torch.float32, device=dev)
    cf.cf_rmsnorm_clip_quantize_rows(x, w, rows, H, EPS, float(ceiling), int(e5m2), normed, rms, q, s, d, stream())
    torch.cuda.synchronize()
    assert np.array_equal(host(rms).view(np.uint32), rms_w.view(np.uint32))
    assert np.array_equal(bf16_bits(normed), clipped_w)
    assert np.array_equal(host(s).view(np.uint32), s_w.view(np.uint32))
    assert np.array_equal(host(d).view(np.uint32), d_w.view(np.uint32))
    assert np.array_equal(host(q), q_w)
    # without the bf16 row and the rms: same fp8 bytes
    q2 = torch.empty_like(q)
    cf.cf_rmsnorm_clip_quantize_rows(x, w, rows, H, EPS, float(ceiling), int(e5m2), None, None, q2, s, d, stream())
    torch.cuda.synchronize()
    assert torch.equal(q2, q)


@pytest.mark.parametrize("e5m2", [False, True])
@pytest.mark.parametrize("rows,H", [(300, 2048), (33, 7168), (21, 1000 * 8), (64, 4096)])
def test_fused_record_matches_the_launch_sequence(cf, dev, rows, H, e5m2):
    case(f"fused norm/clip/quantize-record rows={rows} H={H} e5m2={e5m2}")
    xb, wb = make_rows(rows, H, 901 + int(e5m2))
    normed0, _ = orc.rmsnorm_forward(xb, wb, EPS)
    ceiling = ceiling_for(normed0)
    clipped_w, _ = orc.act_row_clip_abs(normed0, ceiling)
    qscale = np.float32(37.5)
    q_w, amax_w = orc.quantize_record(clipped_w.reshape(-1), qscale, np.float32(0.125), e5m2)
    x, w = dev_bf16(xb, dev), dev_bf16(wb, dev)
    normed = torch.empty_like(x)
    q = torch.empty((rows, H), dtype=torch.uint8, device=dev)
    amax = scalar(0.125, dev)
    cf.cf_rmsnorm_clip_quantize_record(x, w, rows, H, EPS, float(ceiling), int(e5m2), normed, None, q,
                                       scalar(float(qscale), dev), amax, stream())
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(normed), clipped_w)
    assert np.array_equal(host(q).reshape(-1), q_w)
    assert host(amax).view(np.uint32)[0] == np.float32(amax_w).view(np.uint32)


def test_fused_full_size_equals_separate_library_calls(cf, dev):
    """Benchmark configuration 2's activation (8192 x 4096): the fused launch against rmsnorm -> clip -> per-row
    quantize as three library calls, every byte; a sample of rows against the oracle."""
    rows, H = 8192, 4096
    case("fused norm/clip/quantize 8192x4096")
    g = torch.Generator(device=dev); g.manual_seed(4)
    x = (torch.randn(rows, H, device=dev, generator=g) * torch.exp(torch.randn(rows, 1, device=dev, generator=g))).to(torch.bfloat16)
    w = (1.0 + 0.2 * torch.randn(H, device=dev, generator=g)).to(torch.bfloat16)
    a = torch.empty_like(x)
    cf.cf_rmsnorm_forward(x, w, a, None, rows, H, EPS, stream())
    ceiling = float(a.float().norm(dim=1).median())        # normalised rows differ little in norm: clip the upper half
    cf.cf_act_row_clip_abs(a, rows, H, ceiling, None, stream())
    qa = torch.empty((rows, H), dtype=torch.uint8, device=dev)
    sa = torch.empty(rows, dtype=torch.float32, device=dev); da = torch.empty_like(sa)
    cf.cf_fp8_quantize_rows(a, rows, H, 0, qa, sa, da, stream())
    b = torch.empty_like(x)
    qb = torch.empty_like(qa); sb = torch.empty_like(sa); db = torch.empty_like(sa)
    cf.cf_rmsnorm_clip_quantize_rows(x, w, rows, H, EPS, ceiling, 0, b, None, qb, sb, db, stream())
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert torch.equal(qa, qb) and torch.equal(sa, sb) and torch.equal(da, db)
    pick = np.arange(0, rows, 257)
    xb, wb = bf16_bits(x)[pick], bf16_bits(w)
    _, _, clipped_w, _, q_w, s_w, _ = oracle_sequence(xb, wb, np.float32(ceiling), False)
    assert np.any(np.any(clipped_w != orc.rmsnorm_forward(xb, wb, EPS)[0], axis=1)), "the sample must contain clipped rows"
    assert np.array_equal(bf16_bits(b)[pick], clipped_w)
    assert np.array_equal(host(qb)[pick], q_w)
    assert np.array_equal(host(sb)[pick].view(np.uint32), s_w.view(np.uint32))


def test_shape_and_argument_errors(cf, dev):
    x = torch.zeros(4 * 100, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(100, dtype=torch.bfloat16, device=dev)
    assert cf.raw_cf_rmsnorm_forward(x.data_ptr(), w.data_ptr(), x.data_ptr(), None, 4, 100, EPS, None) == -2   # 100 % 32 != 0
    assert cf.raw_cf_rmsnorm_forward(x.data_ptr(), w.data_ptr(), x.data_ptr(), None, 4, 32768, EPS, None) == -2
    assert cf.raw_cf_rmsnorm_forward(None, None, None, None, 4, 64, EPS, None) == -1
    assert cf.raw_cf_rmsnorm_forward(None, None, None, None, 0, 64, EPS, None) == 0
    assert cf.raw_cf_rmsnorm_forward(None, None, None, None, -1, 64, EPS, None) == -1
    assert cf.raw_cf_act_row_clip_abs(None, 4, 64, 1.0, None, None) == -1
    assert cf.raw_cf_act_row_clip_abs(None, 4, 64, 0.0, None, None) == 0
