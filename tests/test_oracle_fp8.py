"""Pins the CPU oracle's FP8 functions against what does not depend on the oracle:
the reference's own E4M3 header (oracle/_ref), the bytes its probe pins, torch's OCP
casts, nearest-value brute force over all 256 codes, closed forms and identities."""
import ctypes
import json
from pathlib import Path

import numpy as np
import pytest
import torch

import oracle_lib as orc

GOLD = Path(__file__).resolve().parent / "golden"


def all_bf16_bits():
    return np.arange(65536, dtype=np.uint32).astype(np.uint16)


def f32_from_bits(bits):
    return np.asarray(bits, dtype=np.uint32).view(np.float32)


SCALES = [1.0, 0.5, 3.0, 448.0 / 3.7, 448.0 / 41.5, 1e-3, 7.123e4, 57344.0 / 2.3e-3, 1.0 / 3.0]


# ---- bf16 helper ------------------------------------------------------------------
def test_bf16_rne_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * 10,
                        f32_from_bits(rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32))])
    x = x[np.isfinite(x)]
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.bf16_from_f32(x), want)
    # ties: exactly half way between two bf16 values rounds to the even one
    assert orc.bf16_from_f32(f32_from_bits([0x3f808000]))[0] == 0x3f80
    assert orc.bf16_from_f32(f32_from_bits([0x3f818000]))[0] == 0x3f82
    assert np.array_equal(orc.bf16_to_f32(all_bf16_bits()).view(np.uint32) >> 16, np.arange(65536, dtype=np.uint32))


# ---- E4M3 vs the reference's own header ----------------------------------------------
needs_ref = pytest.mark.skipif(not orc.ref_available(), reason="oracle/_ref not built")


def ref_pack(x):
    r = orc.ref_lib()
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint8)
    fin = np.empty(x.shape, np.uint8)
    r.ref_e4m3_pack_n(x.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p),
                      fin.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(x.size))
    return out, fin.astype(bool)


@needs_ref
def test_e4m3_pack_matches_reference_header_all_bf16_times_scales():
    x = orc.bf16_to_f32(all_bf16_bits())
    for s in SCALES:
        with np.errstate(over="ignore", invalid="ignore"):
            v = (x * np.float32(s)).astype(np.float32)
        got, gfin = orc.e4m3_pack(v)
        want, wfin = ref_pack(v)
        assert np.array_equal(got, want), f"scale {s}"
        assert np.array_equal(gfin, wfin)


@needs_ref
def test_e4m3_pack_matches_reference_header_fp32_sweep():
    # every 61st fp32 bit pattern (70M values, all exponents, every rounding position);
    # the full 2^32 sweep (ref_e4m3_sweep with stride 1) was run once: 0 mismatches.
    r = orc.ref_lib()
    r.ref_e4m3_sweep.restype = ctypes.c_uint64
    r.ref_e4m3_sweep.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64,
                                 ctypes.POINTER(ctypes.c_uint32)]
    first_bad = ctypes.c_uint32(0)
    mine = ctypes.cast(orc._o.orc_e4m3_pack, ctypes.c_void_p)
    bad = r.ref_e4m3_sweep(mine, 17, 61, (2 ** 32) // 61, ctypes.byref(first_bad))
    assert bad == 0, f"first mismatch at bits {first_bad.value:#x}"


@needs_ref
def test_e4m3_unpack_matches_reference_header():
    b = np.arange(256, dtype=np.uint8)
    r = orc.ref_lib()
    want = np.empty(256, np.float32)
    r.ref_e4m3_unpack_n(b.ctypes.data_as(ctypes.c_void_p), want.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(256))
    got = orc.e4m3_unpack(b)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.array_equal(np.isnan(got), np.isnan(want))


def test_e4m3_probe_bytes():
    g = json.loads((GOLD / "e4m3_probe.json").read_text())
    x = np.array([float(v) for v in g["inputs"]], np.float32)
    got, fin = orc.e4m3_pack(x)
    for i, b in g["pinned"].items():
        assert got[int(i)] == b
    assert list(fin) == [True] * 8 + [False] * 3
    assert got[2] == 0x38 and got[3] == 0xb8 and got[4] == 0x08 and got[7] == 0x7e   # 1, -1, 2^-6, 447->448
    # the quantize kernels' conversion saturates infinities instead (kernels/fp8.cu:333-337)
    sat = orc.e4m3_satfinite(x)
    assert sat[9] == 0x7e and sat[10] == 0xfe and sat[8] == 0x7f
    assert np.array_equal(sat[:8], got[:8])


def test_e4m3_matches_torch_cast_after_clamp():
    x = orc.bf16_to_f32(all_bf16_bits())
    for s in SCALES:
        with np.errstate(over="ignore", invalid="ignore"):
            v = (x * np.float32(s)).astype(np.float32)
        ok = np.isfinite(v)
        want = torch.from_numpy(v[ok]).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(orc.e4m3_satfinite(v)[ok], want), f"scale {s}"


def nearest_code_bruteforce(v, values, codes):
    """Round-to-nearest, ties to the code with an even low bit, over an explicit table of finite values."""
    order = np.argsort(values)
    vals, cds = values[order].astype(np.float64), codes[order]
    hi = np.clip(np.searchsorted(vals, v), 1, len(vals) - 1)
    lo = hi - 1
    dlo, dhi = np.abs(v - vals[lo]), np.abs(vals[hi] - v)
    pick_hi = (dhi < dlo) | ((dhi == dlo) & ((cds[hi] & 1) == 0))
    return np.where(pick_hi, cds[hi], cds[lo])


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_fp8_is_nearest_even_by_brute_force(fmt):
    codes = np.arange(256, dtype=np.uint8)
    if fmt == "e4m3":
        vals, enc, fmax = orc.e4m3_unpack(codes), orc.e4m3_satfinite, 448.0
    else:
        vals, enc, fmax = orc.e5m2_unpack(codes), orc.e5m2_satfinite, 57344.0
    pos = np.isfinite(vals) & (codes < 0x80)
    pv, pc = vals[pos], codes[pos]
    rng = np.random.default_rng(3)
    mags = np.concatenate([
        np.exp(rng.uniform(np.log(1e-9), np.log(fmax * 1.5), 400000)),
        (pv[:-1] + pv[1:]) / 2,                              # exact midpoints: tie cases
        pv, pv * (1 + 2.0 ** -23), pv * (1 - 2.0 ** -24)]).astype(np.float32)
    mags = mags[mags >= 0]
    want = nearest_code_bruteforce(np.minimum(mags.astype(np.float64), fmax), pv, pc)
    assert np.array_equal(enc(mags), want)
    assert np.array_equal(enc(-mags), want | 0x80)
    # decode(encode(v)) == v for every finite code value
    assert np.array_equal(enc(vals[np.isfinite(vals)]) & 0x7f, codes[np.isfinite(vals)] & 0x7f)


def test_e5m2_matches_torch_cast_after_clamp():
    x = orc.bf16_to_f32(all_bf16_bits())
    for s in SCALES:
        with np.errstate(over="ignore", invalid="ignore"):
            v = (x * np.float32(s)).astype(np.float32)
        ok = np.isfinite(v)
        want = torch.from_numpy(v[ok]).clamp(-57344, 57344).to(torch.float8_e5m2).view(torch.uint8).numpy()
        assert np.array_equal(orc.e5m2_satfinite(v)[ok], want), f"scale {s}"
    special = np.array([np.inf, -np.inf, 61440.0, 1e30], np.float32)
    assert list(orc.e5m2_satfinite(special)) == [0x7b, 0xfb, 0x7b, 0x7b]
    assert np.array_equal(orc.e5m2_unpack(np.arange(256, dtype=np.uint8))[:0x7c],
                          torch.arange(0x7c, dtype=torch.uint8).view(torch.float8_e5m2).float().numpy())


# ---- amax / scale ---------------------------------------------------------------------
def test_amax_is_max_of_sign_cleared_patterns():
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 65536, 100001).astype(np.uint16)
    bits = bits[(bits & 0x7fff) <= 0x7f80]                 # drop NaN patterns
    want = orc.bf16_to_f32(np.array([(bits & 0x7fff).max()], np.uint16))[0]
    assert orc.amax_bf16(bits) == want
    assert orc.amax_bf16(np.zeros(0, np.uint16)) == 0.0
    # NaN elements are ignored by fmaxf
    withnan = np.concatenate([bits[:10], np.array([0x7fc0], np.uint16)])
    assert orc.amax_bf16(withnan) == orc.amax_bf16(bits[:10])


def test_scale_from_amax_closed_form():
    for a in [0.0, 1e-20, 1e-12, 3.7, 448.0, 41.5, 6.1e4]:
        for fmax in (448.0, 57344.0):
            s, d = orc.scale_from_amax(a, fmax)
            af = max(np.float32(a), np.float32(1e-12))
            assert s == np.float32(fmax) / af and d == af / np.float32(fmax)


def test_quantize_is_multiply_then_convert():
    rng = np.random.default_rng(2)
    bits = orc.bf16_from_f32(rng.standard_normal(50000).astype(np.float32) * 3)
    s, _ = orc.scale_from_amax(orc.amax_bf16(bits), 448.0)
    q = orc.quantize_e4m3(bits, s)
    assert np.array_equal(q, orc.e4m3_satfinite(orc.bf16_to_f32(bits) * s))
    assert (q & 0x7f).max() == 0x7e                         # the amax element lands on 448
    q5 = orc.quantize_e5m2(bits, np.float32(2.0))
    assert np.array_equal(q5, orc.e5m2_satfinite(orc.bf16_to_f32(bits) * np.float32(2.0)))
    qr, amax = orc.quantize_record(bits, s, 0.0)
    assert np.array_equal(qr, q) and amax == orc.amax_bf16(bits)
    _, amax2 = orc.quantize_record(bits, s, 1e9)            # max-combines with what is there
    assert amax2 == np.float32(1e9)


# ---- delayed scaling ring -----------------------------------------------------------------
def py_delayed(amaxes, fmax, hlen, cursor=0, count=0):
    hist = [np.float32(0)] * max(hlen, 1)
    out = []
    for a in amaxes:
        a = max(np.float32(a), np.float32(1e-12))
        if hlen <= 0:
            out.append((np.float32(fmax) / a, a / np.float32(fmax), cursor, count))
            continue
        if cursor < 0 or cursor >= hlen:
            cursor = 0
        hist[cursor] = a
        cursor = (cursor + 1) % hlen
        count = min(count + 1, hlen)
        m = max(max(hist[:count]), np.float32(1e-12))
        out.append((np.float32(fmax) / m, m / np.float32(fmax), cursor, count))
    return out


@pytest.mark.parametrize("hlen,cursor,count", [(0, 0, 0), (1, 0, 0), (8, 0, 0), (16, 0, 0), (8, 99, 3), (8, -4, 0), (4, 3, 4)])
def test_update_delayed_scale_sequences(hlen, cursor, count):
    rng = np.random.default_rng(hlen + 5)
    amaxes = np.abs(rng.standard_normal(40)).astype(np.float32) * 10
    amaxes[7] = 0.0
    st = orc.DelayedState(hlen, cursor, count)
    want = py_delayed(amaxes, 448.0, hlen, cursor, count)
    for a, (s, d, cur, cnt) in zip(amaxes, want):
        st.update(a, 448.0)
        assert st.scale[0] == s and st.descale[0] == d
        if hlen > 0:
            assert st.cursor[0] == cur and st.count[0] == cnt
    if hlen > 0:
        # window property: the scale is fp8_max / max(last min(len, calls) amaxes)
        tail = np.maximum(amaxes[-hlen:], np.float32(1e-12))
        assert st.scale[0] == np.float32(448.0) / tail.max()


# ---- permutations ---------------------------------------------------------------------------
@pytest.mark.parametrize("K,N", [(1, 1), (3, 5), (64, 64), (65, 130), (128, 256), (200, 77)])
def test_transposing_quantizers_are_permutations_of_the_plain_one(K, N):
    rng = np.random.default_rng(K * 1000 + N)
    w = orc.bf16_from_f32(rng.standard_normal((K, N)).astype(np.float32))
    s = np.float32(37.5)
    q = orc.quantize_e4m3(w, s)
    assert np.array_equal(orc.quantize_transpose_e4m3(w, s), q.T)
    act8, snap = orc.quant_and_transpose_e4m3(w, s)
    assert np.array_equal(act8, q) and np.array_equal(snap, q.T)
    assert np.array_equal(orc.transpose_u8(q), q.T)


# ---- probes / raw path ------------------------------------------------------------------------
def test_clip_probe_and_elem_count():
    st = orc.clip_probe(10.0, 448.0 / 5.0, 448.0, np.zeros(3, np.float32))
    assert list(st) == [1.0, 2.0, 1.0]
    st = orc.clip_probe(4.0, 448.0 / 5.0, 448.0, st)
    assert list(st) == [1.0, 2.0, 2.0]
    bits = orc.bf16_from_f32(np.array([1, -6, 5, 5.5, -4.9], np.float32))
    out = orc.elem_clip_count(bits, np.float32(448.0 / 5.0), 448.0, np.zeros(2, np.float32))
    assert list(out) == [2.0, 5.0]


def test_raw_pack_roundtrip_and_bad_count():
    rng = np.random.default_rng(9)
    bits = orc.bf16_from_f32(rng.standard_normal(4099).astype(np.float32))
    q, amax, s, d, bad = orc.pack_raw(bits)
    assert bad == 0 and amax == orc.amax_bf16(bits)
    assert np.array_equal(q, orc.quantize_e4m3(bits, s))          # finite input: same bytes as the cast
    q2, deq, *_ = orc.pack_raw(bits, dequant=True)
    assert np.array_equal(q2, q)
    assert np.array_equal(deq, orc.bf16_from_f32(orc.e4m3_unpack(q) * d))
    assert np.array_equal(orc.unpack_raw(q, d), deq)
    bits[5] = 0x7f80   # +inf
    bits[9] = 0xffc0   # NaN
    q, amax, s, d, bad = orc.pack_raw(bits)
    assert bad > 0 and q[5] == 0x7f and q[9] == 0xff and np.isfinite(amax)


# ---- scale groups --------------------------------------------------------------------------------
def test_group_quantizers_equal_per_tensor_on_each_group():
    rng = np.random.default_rng(4)
    x = orc.bf16_from_f32(rng.standard_normal((130, 300)).astype(np.float32))
    q, s, d = orc.quantize_rows(x)
    for r in (0, 17, 129):
        sr, dr = orc.scale_from_amax(orc.amax_bf16(x[r]), 448.0)
        assert s[r] == sr and d[r] == dr and np.array_equal(q[r], orc.quantize_e4m3(x[r], sr))
    q, s, d = orc.quantize_block_1x128(x)
    assert s.shape == (130, 3)
    sr, _ = orc.scale_from_amax(orc.amax_bf16(x[5, 256:300]), 448.0)
    assert s[5, 2] == sr and np.array_equal(q[5, 256:], orc.quantize_e4m3(x[5, 256:], sr))
    q, s, d = orc.quantize_block_128x128(x)
    assert s.shape == (2, 3)
    blk = np.ascontiguousarray(x[128:130, 128:256])
    sr, _ = orc.scale_from_amax(orc.amax_bf16(blk), 448.0)
    assert s[1, 1] == sr and np.array_equal(q[128:130, 128:256], orc.quantize_e4m3(blk, sr))


# ---- epilogue ops ------------------------------------------------------------------------------------
def test_swiglu_probe_values_and_closed_form():
    g = json.loads((GOLD / "swiglu_probe.json").read_text())
    gate, up = np.array(g["gate"], np.float32), np.array(g["up"], np.float32)
    out = orc.bf16_to_f32(orc.swiglu_forward(orc.bf16_from_f32(gate), orc.bf16_from_f32(up)))
    want = gate / (1 + np.exp(-gate.astype(np.float64))) * up
    assert np.all(np.abs(out - want) <= g["tolerance"])
    rng = np.random.default_rng(6)
    gb = orc.bf16_from_f32(rng.standard_normal(20000).astype(np.float32) * 4)
    ub = orc.bf16_from_f32(rng.standard_normal(20000).astype(np.float32))
    gf, uf = orc.bf16_to_f32(gb).astype(np.float64), orc.bf16_to_f32(ub).astype(np.float64)
    exact = gf / (1 + np.exp(-gf)) * uf
    got = orc.bf16_to_f32(orc.swiglu_forward(gb, ub))
    assert np.all(np.abs(got - exact) <= 1.01 * orc.bf16_ulp(exact) / 2 + 1e-30 + 3e-7 * np.abs(exact))


def test_swiglu_backward_is_the_derivative_of_the_forward():
    """grad_up = grad * silu(gate) is the forward's product with (gate, grad) -- one commutative multiply, so the
    bits must equal swiglu_forward(gate, grad).  grad_gate against the closed form d/dg [g sigmoid(g)] u grad in double,
    and against a central difference of the forward's own formula (a dropped `1 +` or a sign error in `1 - sigmoid`
    misses by tens of percent)."""
    rng = np.random.default_rng(16)
    n = 30000
    gb = orc.bf16_from_f32(rng.standard_normal(n).astype(np.float32) * 4)
    ub = orc.bf16_from_f32(rng.standard_normal(n).astype(np.float32))
    db = orc.bf16_from_f32(rng.standard_normal(n).astype(np.float32) * 1e-2)
    gb[:6] = orc.bf16_from_f32(np.array([-100, 100, -20, 20, 0, -0.0], np.float32))
    dg, du = orc.swiglu_backward(db, gb, ub)
    assert np.array_equal(du, orc.swiglu_forward(gb, db))
    g, u, d = (orc.bf16_to_f32(v).astype(np.float64) for v in (gb, ub, db))
    sg = 1.0 / (1.0 + np.exp(-g))
    exact = d * u * sg * (1.0 + g * (1.0 - sg))
    got = orc.bf16_to_f32(dg).astype(np.float64)
    assert np.all(np.abs(got - exact) <= 1.01 * orc.bf16_ulp(exact) / 2 + 1e-30 + 6e-7 * np.abs(d * u))
    silu = lambda x: x / (1.0 + np.exp(-x))
    h = 1e-4
    numeric = d * u * (silu(g + h) - silu(g - h)) / (2 * h)
    assert np.all(np.abs(exact - numeric) <= 1e-6 * np.abs(d * u) + 1e-30)
    # silu'(0) = 1/2, silu'(large) = 1, silu'(-large) = 0
    one = orc.bf16_from_f32(np.ones(3, np.float32))
    dg, _ = orc.swiglu_backward(one, orc.bf16_from_f32(np.array([0.0, 60.0, -60.0], np.float32)), one)
    assert np.array_equal(orc.bf16_to_f32(dg), np.array([0.5, 1.0, 0.0], np.float32)) or \
        np.allclose(orc.bf16_to_f32(dg), [0.5, 1.0, 0.0], atol=1e-20)


def test_col_sum_strided_order_and_accumulate():
    rng = np.random.default_rng(17)
    rows, cols, stride, base = 300, 70, 96, 11
    xi = rng.integers(-8, 9, (rows, stride)).astype(np.float32)          # every partial sum is exact
    x = orc.bf16_from_f32(xi)
    acc0 = rng.integers(-4, 5, cols).astype(np.float32)
    got = orc.col_sum_strided(x, acc0, rows, cols, stride, base)
    assert np.array_equal(got, acc0 + xi[:, base:base + cols].sum(0))
    # a column that separates the sequential order from any tree: 2^24 then ones.  Added one at a time every 1 is
    # lost to rounding (ties to even); any grouping that first adds two ones together keeps them.
    col = np.array([16777216.0] + [1.0] * 7, np.float32)
    x = orc.bf16_from_f32(col.reshape(-1, 1))
    assert orc.col_sum_strided(x, np.zeros(1, np.float32), 8, 1, 1, 0)[0] == np.float32(16777216.0)
    # the sum starts from zero and is added to the accumulator once (not accumulated into it term by term)
    assert orc.col_sum_strided(x[1:], np.array([16777216.0], np.float32), 7, 1, 1, 0)[0] == np.float32(16777224.0)
    # random data: the float32 chain, restated with numpy scalars
    xr = orc.bf16_from_f32(rng.standard_normal((257, 5)).astype(np.float32))
    want = np.zeros(5, np.float32)
    for r in range(257):
        want = (want + orc.bf16_to_f32(xr[r])).astype(np.float32)
    assert np.array_equal(orc.col_sum_strided(xr, np.zeros(5, np.float32), 257, 5, 5, 0), want)


def test_bias_add_strided():
    rng = np.random.default_rng(8)
    x = orc.bf16_from_f32(rng.standard_normal((5, 12)).astype(np.float32))
    b = orc.bf16_from_f32(rng.standard_normal(4).astype(np.float32))
    out = orc.bias_add_strided(x, b, 5, 4, 12, 3)
    want = x.copy()
    want[:, 3:7] = orc.bf16_from_f32(orc.bf16_to_f32(x[:, 3:7]) + orc.bf16_to_f32(b)[None, :])
    assert np.array_equal(out, want)


def test_running_maximum_ignores_every_kind_of_nan():
    """CUDA's fmaxf returns the non-NaN operand for quiet and signaling NaNs alike; a signaling NaN must not
    reset the oracle's running maximum (glibc's fmaxf would turn it into a NaN result)."""
    bits = np.array([0x4000, 0x7f81, 0x3f80, 0xffa0, 0x7fc0, 0xc040, 0x7fbf, 0x3e00], dtype=np.uint16)   # 2, sNaN, 1, -sNaN, qNaN, -3, sNaN, .125
    assert orc.amax_bf16(bits) == np.float32(3.0)
    _, amax = orc.quantize_record(bits, np.float32(1.0), np.float32(0.0))
    assert amax == np.float32(3.0)
    _, amax = orc.quantize_record(bits, np.float32(1.0), np.float32(0.0), e5m2=True)
    assert amax == np.float32(3.0)
    with_inf = np.concatenate([bits, np.array([0xff80, 0x7f85], dtype=np.uint16)])
    assert np.isposinf(orc.amax_bf16(with_inf))
