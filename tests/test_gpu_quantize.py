"""GPU parity: the HIP quantize family against the CPU oracle, bit for bit, through the C ABI."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_arr, dev_bf16, host, scalar, stream

pytestmark = pytest.mark.gpu

SCALES = [1.0, 0.5, 3.0, 448.0 / 3.7, 448.0 / 41.5, 1e-3, 7.123e4, 57344.0 / 2.3e-3, 1.0 / 3.0]


def all_bf16_bits():
    return np.arange(65536, dtype=np.uint32).astype(np.uint16)


def q_gpu(cf, dev, bits, scale, e5m2=False):
    x = dev_bf16(bits, dev)
    out = torch.empty(x.shape, dtype=torch.uint8, device=dev)
    fn = cf.cf_fp8_quantize_e5m2 if e5m2 else cf.cf_fp8_quantize_e4m3
    fn(x, out, scalar(scale, dev), x.numel(), stream())
    torch.cuda.synchronize()
    return host(out)


@pytest.mark.parametrize("e5m2", [False, True])
def test_hardware_convert_matches_oracle_on_every_bf16_input(cf, dev, e5m2):
    bits = all_bf16_bits()
    enc = orc.quantize_e5m2 if e5m2 else orc.quantize_e4m3
    for s in SCALES:
        case(f"all bf16 x scale {s} e5m2={e5m2}")
        got = q_gpu(cf, dev, bits, np.float32(s), e5m2)
        want = enc(bits, np.float32(s))
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, f"scale {s}: {bad.size} differ, first bits {bits[bad[0]]:#06x} got {got[bad[0]]:#x} want {want[bad[0]]:#x}"


@pytest.mark.parametrize("e5m2", [False, True])
def test_recording_quantize_on_every_bf16_input(cf, dev, e5m2):
    """The recording form on all 65536 patterns, in an order that mixes finite and non-finite vectors: same bytes
    as the plain form, and an amax that ignores the NaNs (here +inf, the largest non-NaN magnitude present)."""
    case(f"record, all bf16, e5m2={e5m2}")
    rng = np.random.default_rng(3)
    bits = rng.permutation(np.concatenate([all_bf16_bits(), np.tile(orc.bf16_from_f32(rng.standard_normal(4096).astype(np.float32)), 64)]))
    x = dev_bf16(bits, dev)
    fn = cf.cf_fp8_quantize_e5m2_record if e5m2 else cf.cf_fp8_quantize_e4m3_record
    for sc in (1.0, 37.5, 0.0, float("inf")):
        out = torch.empty(bits.size, dtype=torch.uint8, device=dev)
        amax = scalar(0.0, dev)
        fn(x, out, scalar(sc, dev), amax, bits.size, stream())
        torch.cuda.synchronize()
        wq, wamax = orc.quantize_record(bits, np.float32(sc), np.float32(0.0), e5m2)
        assert np.array_equal(host(out), wq), f"scale {sc}"
        assert host(amax).view(np.uint32)[0] == np.float32(wamax).view(np.uint32), f"scale {sc}"
    finite_only = bits[(bits & 0x7fff) < 0x7f80]
    xf = dev_bf16(finite_only, dev)
    out = torch.empty(finite_only.size, dtype=torch.uint8, device=dev)
    amax = scalar(0.0, dev)
    fn(xf, out, scalar(2.0, dev), amax, finite_only.size, stream())
    torch.cuda.synchronize()
    wq, wamax = orc.quantize_record(finite_only, np.float32(2.0), np.float32(0.0), e5m2)
    assert np.array_equal(host(out), wq) and host(amax)[0] == wamax


@pytest.mark.parametrize("e5m2", [False, True])
def test_hardware_convert_matches_oracle_on_fp32_sweep(cf, dev, e5m2):
    # 2^26 fp32 bit patterns at stride 64 plus a random offset: every exponent, every rounding position
    case(f"fp32 sweep e5m2={e5m2}")
    bits = (np.arange(2 ** 26, dtype=np.uint64) * 64 + 29).astype(np.uint32)
    x = torch.from_numpy(bits.view(np.int32)).to(dev).view(torch.float32)
    out = torch.empty(x.shape, dtype=torch.uint8, device=dev)
    fn = cf.cf_fp8_quantize_f32_e5m2 if e5m2 else cf.cf_fp8_quantize_f32_e4m3
    fn(x, out, scalar(1.0, dev), x.numel(), stream())
    torch.cuda.synchronize()
    xf = bits.view(np.float32)
    want = orc.e5m2_satfinite(xf) if e5m2 else orc.e4m3_satfinite(xf)
    got = host(out)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, f"{bad.size} differ, first bits {bits[bad[0]]:#010x} got {got[bad[0]]:#x} want {want[bad[0]]:#x}"


@pytest.mark.parametrize("n,offset", [(0, 0), (1, 0), (15, 0), (16, 0), (4097, 0), (100003, 0), (100003, 1), (65536, 3), (1 << 20, 0)])
def test_amax_scale_quantize_record(cf, dev, n, offset):
    case(f"amax/quantize n={n} offset={offset}")
    rng = np.random.default_rng(n + offset)
    bits = orc.bf16_from_f32(rng.standard_normal(n + offset).astype(np.float32) * 2.5)
    if n > 100:
        bits[offset + 7] = 0x7fc0   # a NaN is ignored by amax and encodes as NaN
    xfull = dev_bf16(bits, dev)
    x = xfull[offset:]
    hb = bits[offset:]
    amax = scalar(123.0, dev); scale = scalar(0, dev); desc = scalar(0, dev)
    cf.cf_fp8_amax_bf16(x, n, amax, stream())
    cf.cf_fp8_scale_from_amax(amax, 448.0, scale, desc, stream())
    torch.cuda.synchronize()
    want_amax = orc.amax_bf16(hb)
    ws, wd = orc.scale_from_amax(want_amax, 448.0)
    assert host(amax)[0] == want_amax and host(scale)[0] == ws and host(desc)[0] == wd
    for e5m2 in (False, True):
        outfull = torch.full((n + offset + 32,), 0xAA, dtype=torch.uint8, device=dev)
        out = outfull[offset:offset + n]
        (cf.cf_fp8_quantize_e5m2 if e5m2 else cf.cf_fp8_quantize_e4m3)(x, out, scale, n, stream())
        torch.cuda.synchronize()
        want = (orc.quantize_e5m2 if e5m2 else orc.quantize_e4m3)(hb, ws)
        assert np.array_equal(host(out), want)
        assert np.all(host(outfull[:offset]) == 0xAA) and np.all(host(outfull[offset + n:]) == 0xAA)   # no stray writes
        rec = scalar(0.0, dev)
        out2 = torch.empty(n, dtype=torch.uint8, device=dev)
        (cf.cf_fp8_quantize_e5m2_record if e5m2 else cf.cf_fp8_quantize_e4m3_record)(x, out2, scale, rec, n, stream())
        torch.cuda.synchronize()
        assert np.array_equal(host(out2), want) and host(rec)[0] == want_amax
        rec = scalar(1e9, dev)                               # max-combines with the previous content
        (cf.cf_fp8_quantize_e5m2_record if e5m2 else cf.cf_fp8_quantize_e4m3_record)(x, out2, scale, rec, n, stream())
        torch.cuda.synchronize()
        assert host(rec)[0] == np.float32(1e9)


def test_fp32_input_quantize_config1(cf, dev):
    case("fp32 input, config 1 shapes")
    rng = np.random.default_rng(11)
    for shape, sigma in (((512, 1024), 1.0), ((1024, 1024), 0.02), ((7, 13), 1.0)):
        xh = (rng.standard_normal(shape) * sigma).astype(np.float32)
        x = torch.from_numpy(xh).to(dev)
        amax = scalar(0, dev); scale = scalar(0, dev); desc = scalar(0, dev)
        out = torch.empty(shape, dtype=torch.uint8, device=dev)
        cf.cf_fp8_amax_f32(x, x.numel(), amax, stream())
        cf.cf_fp8_scale_from_amax(amax, 448.0, scale, desc, stream())
        cf.cf_fp8_quantize_f32_e4m3(x, out, scale, x.numel(), stream())
        torch.cuda.synchronize()
        wa = orc.amax_f32(xh)
        ws, wd = orc.scale_from_amax(wa, 448.0)
        assert host(amax)[0] == wa and host(scale)[0] == ws and host(desc)[0] == wd
        assert np.array_equal(host(out), orc.quantize_f32_e4m3(xh, ws))


@pytest.mark.parametrize("hlen,cursor,count", [(0, 0, 0), (1, 0, 0), (8, 0, 0), (16, 0, 0), (8, 99, 3), (8, -4, 0)])
def test_update_delayed_scale(cf, dev, hlen, cursor, count):
    case(f"delayed scale len={hlen}")
    rng = np.random.default_rng(hlen)
    amaxes = np.abs(rng.standard_normal(40)).astype(np.float32) * 10
    amaxes[5] = 0.0
    st = orc.DelayedState(hlen, cursor, count)
    hist = torch.zeros(max(hlen, 1), device=dev)
    cur = scalar(cursor, dev, torch.int32); cnt = scalar(count, dev, torch.int32)
    scale = scalar(0, dev); desc = scalar(0, dev)
    for a in amaxes:
        st.update(a, 57344.0)
        cf.cf_fp8_update_delayed_scale(scalar(a, dev), 57344.0, scale, desc, hist, hlen, cur, cnt, stream())
        torch.cuda.synchronize()
        assert host(scale)[0] == st.scale[0] and host(desc)[0] == st.descale[0]
        if hlen > 0:
            assert host(cur)[0] == st.cursor[0] and host(cnt)[0] == st.count[0]
            assert np.array_equal(host(hist), st.history)


@pytest.mark.parametrize("K,N", [(128, 128), (256, 384), (1024, 2048), (1, 1), (3, 5), (65, 130), (200, 77), (128, 130)])
def test_transposing_kernels(cf, dev, K, N):
    case(f"transposes K={K} N={N}")
    rng = np.random.default_rng(K * 7 + N)
    wb = orc.bf16_from_f32(rng.standard_normal((K, N)).astype(np.float32))
    s = np.float32(448.0) / orc.amax_bf16(wb)
    if K * N > 64:        # a few non-finite elements: those vectors take the NaN-restoring convert
        flat = wb.reshape(-1)
        flat[rng.integers(0, flat.size, 6)] = np.array([0x7fc0, 0xffc1, 0x7f80, 0xff80, 0x7f81, 0x7fc0], dtype=np.uint16)
    w = dev_bf16(wb, dev)
    sc = scalar(s, dev)
    q = orc.quantize_e4m3(wb, s)
    out = torch.empty((N, K), dtype=torch.uint8, device=dev)
    cf.cf_fp8_quantize_transpose_e4m3(w, out, sc, K, N, stream())
    torch.cuda.synchronize()
    assert np.array_equal(host(out), q.T)
    act8 = torch.empty((K, N), dtype=torch.uint8, device=dev)
    snap = torch.empty((N, K), dtype=torch.uint8, device=dev)
    cf.cf_fp8_quant_and_transpose_e4m3(w, act8, snap, sc, K, N, stream())
    torch.cuda.synchronize()
    assert np.array_equal(host(act8), q) and np.array_equal(host(snap), q.T)
    qd = dev_arr(q, dev)
    t = torch.empty((N, K), dtype=torch.uint8, device=dev)
    cf.cf_transpose_u8(qd, t, K, N, stream())
    torch.cuda.synchronize()
    assert np.array_equal(host(t), q.T)


@pytest.mark.parametrize("rows,K", [(8, 4096), (5, 1024), (3, 14336), (130, 2048), (4, 1408), (7, 300), (2, 20000), (1, 16),
                                    (5, 28672), (2, 32768), (2, 40000), (3, 20001)])
@pytest.mark.parametrize("e5m2", [False, True])
def test_per_row_quantize(cf, dev, rows, K, e5m2):
    case(f"rows quantize {rows}x{K} e5m2={e5m2}")
    rng = np.random.default_rng(rows * 31 + K)
    xh = rng.standard_normal((rows, K)).astype(np.float32)
    xh[rng.random((rows, K)) < 0.001] = 40.0
    if rows > 2:
        xh[2] = 0.0                                       # an all-zero row takes the 1e-12 floor
    xb = orc.bf16_from_f32(xh)
    x = dev_bf16(xb, dev)
    out = torch.empty((rows, K), dtype=torch.uint8, device=dev)
    s = torch.empty(rows, device=dev); d = torch.empty(rows, device=dev)
    cf.cf_fp8_quantize_rows(x, rows, K, int(e5m2), out, s, d, stream())
    torch.cuda.synchronize()
    wq, ws, wd = orc.quantize_rows(xb, e5m2)
    assert np.array_equal(host(s), ws) and np.array_equal(host(d), wd)
    assert np.array_equal(host(out), wq)


@pytest.mark.parametrize("K", [1024, 4096, 14336])
@pytest.mark.parametrize("e5m2", [False, True])
def test_per_row_quantize_with_nonfinite_elements(cf, dev, K, e5m2):
    """Rows holding NaN or infinities: the row maximum ignores NaN, an infinite maximum gives scale 0 and
    the products 0 x inf become NaN codes, exactly as the element-wise definition says."""
    case(f"rows quantize non-finite K={K} e5m2={e5m2}")
    rng = np.random.default_rng(K + int(e5m2))
    xh = rng.standard_normal((6, K)).astype(np.float32)
    xh[1, 5] = np.nan
    xh[2, K - 1] = np.inf
    xh[3, 7] = -np.inf; xh[3, 9] = np.nan
    xh[4, :] = np.nan
    xb = orc.bf16_from_f32(xh)
    x = dev_bf16(xb, dev)
    out = torch.empty((6, K), dtype=torch.uint8, device=dev)
    s = torch.empty(6, device=dev); d = torch.empty(6, device=dev)
    cf.cf_fp8_quantize_rows(x, 6, K, int(e5m2), out, s, d, stream())
    torch.cuda.synchronize()
    wq, ws, wd = orc.quantize_rows(xb, e5m2)
    assert np.array_equal(host(s).view(np.uint32), ws.view(np.uint32))
    assert np.array_equal(host(d).view(np.uint32), wd.view(np.uint32))
    assert np.array_equal(host(out), wq)


@pytest.mark.parametrize("rows,K", [(128, 128), (4, 7168), (130, 384), (37, 300), (256, 1408)])
def test_block_scaled_quantize(cf, dev, rows, K):
    case(f"block quantize {rows}x{K}")
    rng = np.random.default_rng(rows + K)
    xb = orc.bf16_from_f32(rng.standard_normal((rows, K)).astype(np.float32) * np.exp(rng.standard_normal((rows, 1))).astype(np.float32))
    x = dev_bf16(xb, dev)
    kb, rb = (K + 127) // 128, (rows + 127) // 128
    out = torch.empty((rows, K), dtype=torch.uint8, device=dev)
    s = torch.empty((rows, kb), device=dev); d = torch.empty((rows, kb), device=dev)
    cf.cf_fp8_quantize_block_1x128(x, rows, K, out, s, d, stream())
    torch.cuda.synchronize()
    wq, ws, wd = orc.quantize_block_1x128(xb)
    assert np.array_equal(host(s), ws) and np.array_equal(host(d), wd) and np.array_equal(host(out), wq)
    s = torch.empty((rb, kb), device=dev); d = torch.empty((rb, kb), device=dev)
    cf.cf_fp8_quantize_block_128x128(x, rows, K, out, s, d, stream())
    torch.cuda.synchronize()
    wq, ws, wd = orc.quantize_block_128x128(xb)
    assert np.array_equal(host(s), ws) and np.array_equal(host(d), wd) and np.array_equal(host(out), wq)


def test_block_scaled_quantize_with_nonfinite_elements(cf, dev):
    """Groups holding NaN or infinities take the float maximum (NaNs ignored) and the NaN-restoring convert."""
    case("block quantize, non-finite groups")
    rng = np.random.default_rng(21)
    rows, K = 256, 512
    xh = rng.standard_normal((rows, K)).astype(np.float32)
    xh[3, 5] = np.nan; xh[3, 200] = np.inf; xh[130, 300] = -np.inf; xh[200, 129] = np.nan; xh[255, 511] = np.nan
    xb = orc.bf16_from_f32(xh)
    x = dev_bf16(xb, dev)
    for fn, ofn, nscale in ((cf.cf_fp8_quantize_block_1x128, orc.quantize_block_1x128, rows * (K // 128)),
                            (cf.cf_fp8_quantize_block_128x128, orc.quantize_block_128x128, (rows // 128) * (K // 128))):
        out = torch.empty((rows, K), dtype=torch.uint8, device=dev)
        s = torch.empty(nscale, device=dev); d = torch.empty(nscale, device=dev)
        fn(x, rows, K, out, s, d, stream())
        torch.cuda.synchronize()
        wq, ws, wd = ofn(xb)
        assert np.array_equal(host(s).view(np.uint32), ws.reshape(-1).view(np.uint32))
        assert np.array_equal(host(d).view(np.uint32), wd.reshape(-1).view(np.uint32))
        assert np.array_equal(host(out), wq)


def test_raw_pack_path(cf, dev):
    case("raw pack")
    rng = np.random.default_rng(21)
    for poison in (False, True):
        bits = orc.bf16_from_f32(rng.standard_normal(70001).astype(np.float32))
        if poison:
            bits[5] = 0x7f80; bits[9] = 0xffc0; bits[60000] = 0xff80
        x = dev_bf16(bits, dev)
        out = torch.empty(bits.size, dtype=torch.uint8, device=dev)
        deq = torch.empty(bits.size, dtype=torch.bfloat16, device=dev)
        amax = scalar(5, dev); scale = scalar(0, dev); desc = scalar(0, dev); bad = scalar(77, dev, torch.int32)
        cf.cf_fp8_pack_bf16_e4m3_raw_and_dequant(x, out, deq, amax, scale, desc, bad, bits.size, stream())
        torch.cuda.synchronize()
        wq, wdeq, wa, ws, wd, wbad = orc.pack_raw(bits, dequant=True)
        assert host(amax)[0] == wa and host(scale)[0] == ws and host(desc)[0] == wd
        assert np.array_equal(host(out), wq) and np.array_equal(bf16_bits(deq), wdeq)
        assert int(host(bad)[0]) == wbad and (wbad > 0) == poison
        out2 = torch.empty_like(out)
        cf.cf_fp8_pack_bf16_e4m3_raw(x, out2, amax, scale, desc, bad, bits.size, stream())
        un = torch.empty_like(deq)
        cf.cf_fp8_unpack_e4m3_raw_bf16(out2, desc, un, bits.size, stream())
        torch.cuda.synchronize()
        assert np.array_equal(host(out2), wq) and int(host(bad)[0]) == wbad
        assert np.array_equal(bf16_bits(un), orc.unpack_raw(wq, wd))


def test_clip_probes_and_calibration_minmax(cf, dev):
    case("clip probes")
    stats = torch.zeros(3, device=dev)
    want = np.zeros(3, np.float32)
    for a, s in ((10.0, 448.0 / 5.0), (4.0, 448.0 / 5.0), (6.0, 448.0 / 5.0), (1.0, 0.0)):
        cf.cf_fp8_clip_probe(scalar(a, dev), scalar(s, dev), 448.0, stats, stream())
        want = orc.clip_probe(a, s, 448.0, want)
    torch.cuda.synchronize()
    assert np.array_equal(host(stats), want)
    rng = np.random.default_rng(3)
    bits = orc.bf16_from_f32(rng.standard_normal(100000).astype(np.float32))
    out = torch.zeros(2, device=dev)
    sc = np.float32(448.0 / 2.0)
    cf.cf_fp8_elem_clip_count(dev_bf16(bits, dev), scalar(sc, dev), 448.0, bits.size, out, stream())
    torch.cuda.synchronize()
    assert np.array_equal(host(out), orc.elem_clip_count(bits, sc, 448.0, np.zeros(2, np.float32)))
    mn = scalar(3.0, dev); mx = scalar(3.0, dev)
    cf.cf_fp8_calib_minmax_update(scalar(0.0, dev), mn, mx, stream())
    cf.cf_fp8_calib_minmax_update(scalar(9.0, dev), mn, mx, stream())
    torch.cuda.synchronize()
    assert host(mn)[0] == np.float32(1e-12) and host(mx)[0] == np.float32(9.0)


def test_swiglu_and_bias_add(cf, dev):
    case("swiglu / bias")
    rng = np.random.default_rng(13)
    for n, off in ((0, 0), (5, 0), (4096, 0), (100003, 0), (100003, 1), (300007, 0)):     # the last one: table path + tail
        gb = orc.bf16_from_f32(rng.standard_normal(n + off).astype(np.float32) * 4)
        ub = orc.bf16_from_f32(rng.standard_normal(n + off).astype(np.float32))
        if n > 10:
            gb[off:off + 6] = orc.bf16_from_f32(np.array([-100, 100, -20, 20, 0, -0.0], np.float32))
        out = torch.empty(n + off, dtype=torch.bfloat16, device=dev)
        cf.cf_swiglu_forward(dev_bf16(gb, dev)[off:], dev_bf16(ub, dev)[off:], out[off:], n, stream())
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(out[off:]), orc.swiglu_forward(gb[off:], ub[off:]))
    xb = orc.bf16_from_f32(rng.standard_normal((37, 96)).astype(np.float32))
    bb = orc.bf16_from_f32(rng.standard_normal(40).astype(np.float32))
    x = dev_bf16(xb, dev)
    cf.cf_bias_add_strided_bf16(x, dev_bf16(bb, dev), 37, 40, 96, 17, stream())
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(x), orc.bias_add_strided(xb, bb, 37, 40, 96, 17))


def test_swiglu_on_every_bf16_gate(cf, dev):
    """All 65536 gate patterns (NaNs and infinities included) against a handful of up values."""
    case("swiglu, every bf16 gate")
    gate = np.tile(all_bf16_bits(), 8)
    ups = orc.bf16_from_f32(np.array([1.0, -0.75, 0.0, 3.0e38, 1e-30, np.inf, -np.inf, np.nan], np.float32))
    up = np.repeat(ups, 65536)
    out = torch.empty(gate.size, dtype=torch.bfloat16, device=dev)
    cf.cf_swiglu_forward(dev_bf16(gate, dev), dev_bf16(up, dev), out, gate.size, stream())
    torch.cuda.synchronize()
    got, want = bf16_bits(out), orc.swiglu_forward(gate, up)
    # a NaN result must be a NaN; its sign and payload are not defined by the arithmetic (x86 and the GPU
    # propagate different operands' payloads)
    nan_w, nan_g = (want & 0x7fff) > 0x7f80, (got & 0x7fff) > 0x7f80
    assert np.array_equal(nan_w, nan_g)
    got, want = np.where(nan_g, 0x7fc0, got), np.where(nan_w, 0x7fc0, want)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, f"{bad.size} differ; first gate {gate[bad[0]]:#06x} up {up[bad[0]]:#06x} got {got[bad[0]]:#06x} want {want[bad[0]]:#06x}"


def test_swiglu_backward(cf, dev):
    """swiglu_backward against the oracle, bit for bit: ragged and unaligned lengths, then every bf16 gate pattern."""
    case("swiglu backward")
    rng = np.random.default_rng(14)
    for n, off in ((0, 0), (5, 0), (4096, 0), (100003, 0), (100003, 1), (300007, 0)):     # the last one: table path + tail
        gb = orc.bf16_from_f32(rng.standard_normal(n + off).astype(np.float32) * 4)
        ub = orc.bf16_from_f32(rng.standard_normal(n + off).astype(np.float32))
        db = orc.bf16_from_f32(rng.standard_normal(n + off).astype(np.float32) * 1e-2)
        if n > 10:
            gb[off:off + 6] = orc.bf16_from_f32(np.array([-100, 100, -20, 20, 0, -0.0], np.float32))
        dg = torch.empty(n + off, dtype=torch.bfloat16, device=dev)
        du = torch.empty(n + off, dtype=torch.bfloat16, device=dev)
        cf.cf_swiglu_backward(dev_bf16(db, dev)[off:], dev_bf16(gb, dev)[off:], dev_bf16(ub, dev)[off:], dg[off:], du[off:], n, stream())
        torch.cuda.synchronize()
        wg, wu = orc.swiglu_backward(db[off:], gb[off:], ub[off:])
        assert np.array_equal(bf16_bits(dg[off:]), wg) and np.array_equal(bf16_bits(du[off:]), wu)
    gate = np.tile(all_bf16_bits(), 6)
    ups = orc.bf16_from_f32(np.array([1.0, -0.75, 0.0, 3.0e38, 1e-30, -2.5], np.float32))
    grads = orc.bf16_from_f32(np.array([1.0, 0.5, -3.0, 1e-30, 3.0e38, 0.0], np.float32))
    up, grad = np.repeat(ups, 65536), np.repeat(grads, 65536)
    dg = torch.empty(gate.size, dtype=torch.bfloat16, device=dev)
    du = torch.empty(gate.size, dtype=torch.bfloat16, device=dev)
    cf.cf_swiglu_backward(dev_bf16(grad, dev), dev_bf16(gate, dev), dev_bf16(up, dev), dg, du, gate.size, stream())
    torch.cuda.synchronize()
    wg, wu = orc.swiglu_backward(grad, gate, up)
    for got, want in ((bf16_bits(dg), wg), (bf16_bits(du), wu)):
        # a NaN result must be a NaN; its sign and payload are not defined by the arithmetic
        nan_w, nan_g = (want & 0x7fff) > 0x7f80, (got & 0x7fff) > 0x7f80
        assert np.array_equal(nan_w, nan_g)
        bad = np.nonzero(np.where(nan_g, 0x7fc0, got) != np.where(nan_w, 0x7fc0, want))[0]
        assert bad.size == 0, f"{bad.size} differ; first gate {gate[bad[0]]:#06x}"
    assert cf.raw_cf_swiglu_backward(None, None, None, None, None, -1, None) == -1
    assert cf.raw_cf_swiglu_backward(None, None, None, None, None, 4, None) == -1
    assert cf.raw_cf_swiglu_backward(None, None, None, None, None, 0, None) == 0


@pytest.mark.parametrize("rows,cols,stride,base", [(300, 70, 96, 11), (1, 1, 1, 0), (129, 64, 64, 0), (1000, 200, 256, 8),
                                                   (4096, 1024, 3072, 2048), (0, 5, 8, 0), (257, 130, 136, 0)])
def test_col_sum_strided(cf, dev, rows, cols, stride, base):
    """The bias gradient: fp32 column sums in ascending row order, added to the accumulator; bit for bit against the
    oracle's sequential loop (16-byte and element-wise fetch paths, ragged row and column tiles)."""
    case(f"col_sum {rows}x{cols} stride {stride} base {base}")
    rng = np.random.default_rng(rows + cols)
    xb = orc.bf16_from_f32((rng.standard_normal((max(rows, 1), stride)) * np.exp(rng.standard_normal((max(rows, 1), 1)))).astype(np.float32))
    acc0 = rng.standard_normal(cols).astype(np.float32)
    acc = torch.from_numpy(acc0).to(dev)
    cf.cf_col_sum_strided_bf16(dev_bf16(xb, dev), acc, rows, cols, stride, base, stream())
    torch.cuda.synchronize()
    assert np.array_equal(host(acc), orc.col_sum_strided(xb, acc0, rows, cols, stride, base))


def test_col_sum_is_sequential_in_rows(cf, dev):
    """2^24 followed by ones: added one at a time every 1 is lost (ties to even); any tree keeps some."""
    case("col_sum order")
    col = np.array([16777216.0] + [1.0] * 300, np.float32).reshape(-1, 1)
    x = np.repeat(orc.bf16_from_f32(col), 8, axis=1)
    acc = torch.zeros(8, device=dev)
    cf.cf_col_sum_strided_bf16(dev_bf16(x, dev), acc, 301, 8, 8, 0, stream())
    torch.cuda.synchronize()
    assert np.all(host(acc) == np.float32(16777216.0))


def test_config2_activation_quantize_full_size(cf, dev):
    """M=8192 x K=4096 bf16 ~N(0,1) with 0.1% outliers at +-40 -> E4M3 with per-token scales."""
    case("config 2 activations, full size")
    g = torch.Generator(device=dev).manual_seed(2)
    x = torch.randn((8192, 4096), generator=g, device=dev)
    u = torch.rand((8192, 4096), generator=g, device=dev)
    x = torch.where(u < 0.0005, torch.full_like(x, 40.0), x)
    x = torch.where(u > 0.9995, torch.full_like(x, -40.0), x).to(torch.bfloat16)
    out = torch.empty((8192, 4096), dtype=torch.uint8, device=dev)
    s = torch.empty(8192, device=dev); d = torch.empty(8192, device=dev)
    cf.cf_fp8_quantize_rows(x, 8192, 4096, 0, out, s, d, stream())
    torch.cuda.synchronize()
    wq, ws, wd = orc.quantize_rows(bf16_bits(x))
    assert np.array_equal(host(s), ws) and np.array_equal(host(d), wd) and np.array_equal(host(out), wq)
    # size-independent property: every row's largest magnitude encodes as 448 and dequantises back to its amax
    assert np.all((host(out) & 0x7f).max(1) == 0x7e)
