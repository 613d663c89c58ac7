"""GPU parity: grouped (per-expert) FP8 GEMM and the SwiGLU expert bank of benchmark config 5.

Integer / byte stages (compact index, per-token quantize of the activations, weighted unpermute) are bit-exact
against the oracle given their inputs; the GEMM stages meet the GEMM bar against the oracle's double reference."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_arr, dev_bf16, host, stream
from test_gpu_gemm import silu_ref

pytestmark = pytest.mark.gpu
ROW_COL, EPI_NONE, EPI_SILU = 1, 0, 2


def quant_rows_np(x):
    """float32 [r,c] -> (E4M3 bytes, descale[r]) with the library's per-row scale formula."""
    q, s, d = orc.quantize_rows(orc.bf16_from_f32(x))
    return q, d


class Bank:
    """Synthetic expert bank + routing, everything the stages need on host and device."""

    def __init__(self, dev, rows, E, k, H, Ie, seed, zero_expert=None):
        rng = np.random.default_rng(seed)
        self.rows, self.E, self.k, self.H, self.Ie = rows, E, k, H, Ie
        logits = rng.standard_normal((rows, E)).astype(np.float32)
        if zero_expert is not None:
            logits[:, zero_expert] = -50.0                   # an expert nobody selects
        self.rw = orc.moe_topk_route(logits, k)
        self.counts, self.idx = orc.moe_build_expert_row_lists(self.rw)
        self.offsets = orc.moe_expert_offsets(self.counts)
        self.total = rows * k
        self.hq, self.hd = quant_rows_np(rng.standard_normal((rows, H)).astype(np.float32))
        self.wg, self.wgd = quant_rows_np((0.02 * rng.standard_normal((E * Ie, H))).astype(np.float32))
        self.wu, self.wud = quant_rows_np((0.02 * rng.standard_normal((E * Ie, H))).astype(np.float32))
        self.wd, self.wdd = quant_rows_np((0.02 * rng.standard_normal((E * H, Ie))).astype(np.float32))
        self.mixed0 = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))
        d = lambda a: dev_arr(a, dev)
        self.d = {n: d(getattr(self, n)) for n in ("rw", "counts", "offsets", "idx", "hq", "hd", "wg", "wgd", "wu", "wud", "wd", "wdd")}
        self.dev = dev

    def compact_index(self):
        return np.concatenate([self.idx[e, : self.counts[e]] for e in range(self.E)])


def run_stages(cf, b: Bank):
    """The bank through the individual entry points; returns every intermediate."""
    dev, E, H, Ie, total = b.dev, b.E, b.H, b.Ie, b.total
    nbytes = np.zeros(1, np.uint64)
    import ctypes
    sz = ctypes.c_size_t(0)
    assert cf.raw_cf_fp8_grouped_gemm_workspace_bytes(total, E, ctypes.byref(sz)) == 0
    ws = torch.empty(sz.value, dtype=torch.uint8, device=dev)
    cidx = torch.full((total,), -1, dtype=torch.int32, device=dev)
    cf.cf_moe_compact_row_index(b.d["counts"], b.d["offsets"], b.d["idx"], b.rows, E, cidx, stream())
    act = torch.zeros((total, Ie), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_grouped_gemm_nt_bf16_ex(total, Ie, H, E, b.d["counts"], b.d["offsets"], b.d["hq"], b.rows, H, cidx, b.d["hd"],
                                      b.d["wg"], b.d["wgd"], ROW_COL, EPI_SILU, b.d["wu"], b.d["wud"], act, Ie, ws, sz.value, stream())
    actq = torch.empty((total, Ie), dtype=torch.uint8, device=dev)
    a_s = torch.empty(total, device=dev); a_d = torch.empty(total, device=dev)
    cf.cf_fp8_quantize_rows(act, total, Ie, 0, actq, a_s, a_d, stream())
    y = torch.zeros((total, H), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_grouped_gemm_nt_bf16_ex(total, H, Ie, E, b.d["counts"], b.d["offsets"], actq, total, Ie, None, a_d,
                                      b.d["wd"], b.d["wdd"], ROW_COL, EPI_NONE, None, None, y, H, ws, sz.value, stream())
    mixed = dev_bf16(b.mixed0, dev)
    cf.cf_moe_unpermute_weighted_bf16(mixed, y, b.d["rw"], b.d["counts"], b.d["offsets"], b.d["idx"], b.rows, E, H, stream())
    torch.cuda.synchronize()
    return dict(cidx=host(cidx), act=bf16_bits(act), actq=host(actq), a_s=host(a_s), a_d=host(a_d), y=bf16_bits(y), mixed=bf16_bits(mixed))


def run_fused(cf, b: Bank):
    import ctypes
    sz = ctypes.c_size_t(0)
    assert cf.raw_cf_moe_grouped_swiglu_workspace_bytes(b.total, b.E, b.H, b.Ie, ctypes.byref(sz)) == 0
    ws = torch.empty(sz.value + 256, dtype=torch.uint8, device=b.dev)
    off = (-ws.data_ptr()) % 256
    mixed = dev_bf16(b.mixed0, b.dev)
    cf.cf_moe_grouped_swiglu_forward_fp8(b.d["hq"], b.d["hd"], b.d["rw"], b.d["counts"], b.d["offsets"], b.d["idx"],
                                         b.d["wg"], b.d["wgd"], b.d["wu"], b.d["wud"], b.d["wd"], b.d["wdd"], mixed,
                                         b.rows, b.H, b.Ie, b.E, b.total, ws.data_ptr() + off, sz.value, stream())
    torch.cuda.synchronize()
    return bf16_bits(mixed)


def check_stages(b: Bank, r, experts=None, sample=None):
    E, H, Ie = b.E, b.H, b.Ie
    cidx = b.compact_index()
    assert np.array_equal(r["cidx"], cidx)                                     # permutation indices: bit-exact
    # per-token quantize of the GPU's own activations: bit-exact
    wq, ws_, wd_ = orc.quantize_rows(r["act"])
    assert np.array_equal(r["actq"], wq) and np.array_equal(r["a_s"], ws_) and np.array_equal(r["a_d"], wd_)
    # weighted unpermute of the GPU's own expert outputs: bit-exact, experts applied in ascending order
    mixed = b.mixed0
    for e in range(E):
        n, o = int(b.counts[e]), int(b.offsets[e])
        mixed = orc.moe_scatter_accumulate(mixed, r["y"][o:o + n], b.rw, b.idx[e, :n], e)
    assert np.array_equal(r["mixed"], mixed)
    # GEMM stages against the double reference, per expert (optionally on a sample of each expert's rows)
    for e in (range(E) if experts is None else experts):
        n, o = int(b.counts[e]), int(b.offsets[e])
        if n == 0:
            continue
        sel = np.arange(n) if sample is None or n <= sample else np.sort(np.random.default_rng(e).choice(n, sample, replace=False))
        rows = b.idx[e, :n][sel]
        A, sa = b.hq[rows], b.hd[rows]
        gref, _ = orc.gemm_nt_ref(A, b.wg[e * Ie:(e + 1) * Ie], sa, b.wgd[e * Ie:(e + 1) * Ie], scale_mode=1, want_abs=False)
        uref, _ = orc.gemm_nt_ref(A, b.wu[e * Ie:(e + 1) * Ie], sa, b.wud[e * Ie:(e + 1) * Ie], scale_mode=1, want_abs=False)
        exact = silu_ref(gref, uref)
        got = orc.bf16_to_f32(r["act"][o:o + n][sel]).astype(np.float64)
        rel = np.sqrt(((got - exact) ** 2).sum() / (exact ** 2).sum())
        assert rel <= 4e-3, (e, rel)                                           # three bf16 roundings, as in the dense fused test
        yref, yabs = orc.gemm_nt_ref(r["actq"][o:o + n][sel], b.wd[e * H:(e + 1) * H], r["a_d"][o:o + n][sel],
                                     b.wdd[e * H:(e + 1) * H], scale_mode=1)
        orc.assert_gemm_close(orc.bf16_to_f32(r["y"][o:o + n][sel]).astype(np.float64), yref, yabs, what=f"down expert {e}")


@pytest.mark.parametrize("rows,E,k,H,Ie,zero", [(600, 5, 2, 256, 384, None), (300, 4, 2, 256, 256, 2), (1500, 3, 1, 512, 640, None), (40, 8, 3, 256, 256, None),
                                                  (500, 4, 2, 384, 256, None), (300, 3, 2, 640, 384, None)])
def test_grouped_bank_small(cf, dev, rows, E, k, H, Ie, zero):
    case(f"grouped swiglu bank rows={rows} E={E} k={k} H={H} Ie={Ie}")
    b = Bank(dev, rows, E, k, H, Ie, seed=rows + E, zero_expert=zero)
    r = run_stages(cf, b)
    check_stages(b, r)
    assert np.array_equal(run_fused(cf, b), r["mixed"])                        # the one-call form is the same computation


def test_grouped_gemm_leaves_rows_of_other_experts_alone(cf, dev):
    case("grouped gemm write footprint")
    b = Bank(dev, 700, 6, 2, 256, 256, seed=9)
    r = run_stages(cf, b)
    # every compact row was written exactly by its expert: rows are a permutation, no zero rows left behind
    assert np.all((r["act"] != 0).any(axis=1)) and np.all((r["y"] != 0).any(axis=1))


def test_config5_full_size(cf, dev):
    """16384 tokens, hidden 2048, 64 experts, top-6, expert width 1408."""
    case("config 5 full size")
    b = Bank(dev, 16384, 64, 6, 2048, 1408, seed=5)
    assert b.counts.sum() == 98304
    r = run_stages(cf, b)
    check_stages(b, r, experts=[0, 31, 63], sample=24)
    assert np.array_equal(run_fused(cf, b), r["mixed"])


@pytest.mark.parametrize("rows,E,k,H,Ie,e5m2", [(90, 4, 2, 96, 72, False), (300, 6, 3, 256, 300, True), (33, 3, 3, 40, 1408, False),
                                                 # whole MFMA steps (H % 128 == 0, Ie % 64 == 0): the matrix-core form
                                                 (300, 6, 3, 256, 320, True), (200, 4, 2, 128, 64, False), (1000, 5, 2, 384, 448, False),
                                                 (70, 3, 3, 2048, 1408, False),
                                                 # three unequal chunks of Ie in the 32-row form; H > 2048: the 16-row form
                                                 (50, 2, 2, 2048, 1472, True), (40, 3, 2, 2304, 128, False), (90, 2, 1, 2176, 192, True)])
def test_grouped_gelu_expert_bank_reference_form(cf, dev, rows, E, k, H, Ie, e5m2):
    """moe_grouped_expert_forward_fp8: per-tensor descales, float GELU intermediate, bf16 CAS accumulate."""
    case(f"grouped gelu bank rows={rows} E={E} k={k} H={H} Ie={Ie} e5m2={e5m2}")
    rng = np.random.default_rng(rows + Ie)
    x = rng.standard_normal((rows, H)).astype(np.float32)
    fmax = 57344.0 if e5m2 else 448.0
    sx = np.float32(fmax) / np.abs(x).max()
    hq = (orc.e5m2_satfinite if e5m2 else orc.e4m3_satfinite)(x * sx)
    win = (0.05 * rng.standard_normal((E, Ie, H))).astype(np.float32)
    wout = (0.05 * rng.standard_normal((E, H, Ie))).astype(np.float32)
    s_in, s_out = np.float32(448.0) / np.abs(win).max(), np.float32(448.0) / np.abs(wout).max()
    winq, woutq = orc.e4m3_satfinite(win * s_in), orc.e4m3_satfinite(wout * s_out)
    d_h, d_in, d_out = np.float32(1) / sx, np.float32(1) / s_in, np.float32(1) / s_out
    rw = orc.moe_topk_route(rng.standard_normal((rows, E)).astype(np.float32), k)
    counts, idx = orc.moe_build_expert_row_lists(rw)
    mixed0 = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))
    mixed = dev_bf16(mixed0, dev)
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    cf.cf_moe_grouped_expert_forward_fp8(dev_arr(hq, dev), sc(d_h), int(e5m2), dev_arr(rw, dev), dev_arr(counts, dev), None,
                                         dev_arr(idx, dev), dev_arr(winq, dev), sc(d_in), dev_arr(woutq, dev), sc(d_out),
                                         mixed, rows, H, Ie, E, rows * k, stream())
    torch.cuda.synchronize()
    start = orc.bf16_to_f32(mixed0).astype(np.float64)
    ref = orc.moe_grouped_expert_forward_fp8_ref(hq, d_h, e5m2, rw, counts, idx, winq, d_in, woutq, d_out, start)
    got = orc.bf16_to_f32(bf16_bits(mixed)).astype(np.float64)
    rel = np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum())
    assert rel <= 4e-3, rel
    # every one of the k accumulations rounds the running value to bf16 (relative 2^-9 each), and the running value
    # can exceed both end points when contributions cancel: bound it by start, result and the typical contribution
    typical = np.sqrt(((ref - start) ** 2).mean())
    bound = (k + 1) * 2.0 ** -8 * (np.abs(start) + np.abs(ref) + 2.0 * typical)
    assert np.all(np.abs(got - ref) <= bound)
    # rows routed to no expert keep their value
    untouched = ~(rw > 0).any(axis=1)
    assert np.array_equal(bf16_bits(mixed)[untouched], mixed0[untouched])


def test_grouped_gelu_expert_bank_on_the_reference_fixture(cf, dev):
    """The expert bank of the reference's own router-parity case (tests/fixtures/moe_router_parity), operands
    quantized to E4M3 with per-tensor scales: the kernel must land on the fixture's `mixed` minus its trunk term to
    within the quantization error, and on the oracle's reference of the same quantized operands to bf16 rounding."""
    import json
    import math
    from pathlib import Path
    case("grouped gelu bank, reference fixture")
    g = json.loads((Path(__file__).resolve().parent / "golden" / "moe_expert_bank.json").read_text())
    hg, rw, mixed = np.array(g["hidden_gated"]), np.array(g["route_weights"]), np.array(g["mixed"])
    tin, tout = np.array(g["trunk_fc_in_w"]), np.array(g["trunk_fc_out_w"])
    ein, eout = np.array(g["expert_fc_in_w"]), np.array(g["expert_fc_out_w"])
    B, S, H = hg.shape
    E, Ie, _ = ein.shape
    rows = B * S
    erf = np.vectorize(math.erf)
    trunk = (lambda x: 0.5 * x * (1.0 + erf(x / math.sqrt(2.0))))(hg @ tin.T) @ tout.T
    want = (mixed - trunk).reshape(rows, H)
    route = np.repeat(rw, S, axis=0).astype(np.float32)
    counts, idx = orc.moe_build_expert_row_lists(route)

    def q(x):
        s, d = orc.scale_from_amax(np.float32(np.abs(x).max()), 448.0)
        return orc.e4m3_satfinite((x.astype(np.float32) * s).astype(np.float32)).reshape(x.shape), d
    hq, hd = q(hg.reshape(rows, H)); wiq, wid = q(ein); woq, wod = q(eout)
    out = torch.zeros((rows, H), dtype=torch.bfloat16, device=dev)
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    cf.cf_moe_grouped_expert_forward_fp8(dev_arr(hq, dev), sc(hd), 0, dev_arr(route, dev), dev_arr(counts, dev), None,
                                         dev_arr(idx, dev), dev_arr(wiq, dev), sc(wid), dev_arr(woq, dev), sc(wod),
                                         out, rows, H, Ie, E, int(counts.sum()), stream())
    torch.cuda.synchronize()
    got = orc.bf16_to_f32(bf16_bits(out)).astype(np.float64)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() < 0.06 * scale
    ref = orc.moe_grouped_expert_forward_fp8_ref(hq, hd, False, route, counts, idx, wiq, wid, woq, wod, np.zeros((rows, H)))
    assert np.all(np.abs(got - ref) <= (E + 1) * 2.0 ** -8 * (np.abs(ref) + scale))


# ---- the GELU expert loop on the matrix cores ----------------------------------------------------------------------

@pytest.mark.parametrize("rows,K,off", [(37, 1408, 0), (9, 300, 0), (5, 8192, 0), (3, 20480, 0), (11, 256, 1), (4, 16, 0)])
def test_gelu_quantize_rows_is_gelu_forward_then_quantize_rows(cf, dev, rows, K, off):
    """One pass over the projections: bytes and scales equal the two launches it replaces, and equal the oracle's
    per-row quantize of the GELU values the GPU produced (the GELU itself is pinned to one bf16 ulp elsewhere)."""
    case(f"gelu + per-row quantize rows={rows} K={K} offset={off}")
    rng = np.random.default_rng(rows * K)
    x = orc.bf16_from_f32((2.5 * rng.standard_normal((rows, K))).astype(np.float32))
    x[0, :] = 0                                                             # an all-zero row: the 1e-12 floor
    flat = torch.zeros(rows * K + 8, dtype=torch.bfloat16, device=dev)
    flat[off:off + rows * K] = dev_bf16(x, dev).reshape(-1)
    dx = flat[off:off + rows * K]
    q = torch.zeros((rows, K), dtype=torch.uint8, device=dev); s = torch.zeros(rows, device=dev); d = torch.zeros(rows, device=dev)
    cf.cf_gelu_quantize_rows_e4m3(dx, rows, K, q, s, d, stream())
    g = torch.zeros(rows * K, dtype=torch.bfloat16, device=dev)
    cf.cf_gelu_forward_bf16(dx, g, rows * K, stream())
    q2 = torch.zeros_like(q); s2 = torch.zeros_like(s); d2 = torch.zeros_like(d)
    cf.cf_fp8_quantize_rows(g, rows, K, 0, q2, s2, d2, stream())
    torch.cuda.synchronize()
    assert np.array_equal(host(q), host(q2)) and np.array_equal(host(s), host(s2)) and np.array_equal(host(d), host(d2))
    wq, ws_, wd_ = orc.quantize_rows(bf16_bits(g).reshape(rows, K))
    assert np.array_equal(host(q), wq) and np.array_equal(host(s), ws_) and np.array_equal(host(d), wd_)


class GeluBank:
    """Per-tensor-scaled expert bank (the operands moe_grouped_expert_forward_fp8 takes) + routing."""

    def __init__(self, dev, rows, E, k, H, Ie, seed, e5m2=False, zero_expert=None):
        rng = np.random.default_rng(seed)
        self.rows, self.E, self.k, self.H, self.Ie, self.e5m2, self.dev = rows, E, k, H, Ie, e5m2, dev
        logits = rng.standard_normal((rows, E)).astype(np.float32)
        if zero_expert is not None:
            logits[:, zero_expert] = -50.0
        self.rw = orc.moe_topk_route(logits, k)
        self.counts, self.idx = orc.moe_build_expert_row_lists(self.rw)
        self.offsets = orc.moe_expert_offsets(self.counts)
        self.total = int(self.counts.sum())

        def q(x, fmax, sat):
            s, d = orc.scale_from_amax(np.float32(np.abs(x).max()), fmax)
            return sat((x * s).astype(np.float32)).reshape(x.shape), np.float32(d)
        x = rng.standard_normal((rows, H)).astype(np.float32)
        self.hq, self.hd = q(x, 57344.0, orc.e5m2_satfinite) if e5m2 else q(x, 448.0, orc.e4m3_satfinite)
        self.wi, self.wid = q((0.05 * rng.standard_normal((E * Ie, H))).astype(np.float32), 448.0, orc.e4m3_satfinite)
        self.wo, self.wod = q((0.05 * rng.standard_normal((E * H, Ie))).astype(np.float32), 448.0, orc.e4m3_satfinite)
        self.mixed0 = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))
        self.d = {n: dev_arr(getattr(self, n), dev) for n in ("rw", "counts", "offsets", "idx", "hq", "wi", "wo")}
        for n in ("hd", "wid", "wod"):
            self.d[n] = torch.tensor([getattr(self, n)], dtype=torch.float32, device=dev)


def run_gelu_fused(cf, b: GeluBank):
    import ctypes
    sz = ctypes.c_size_t(0)
    assert cf.raw_cf_moe_grouped_gelu_workspace_bytes(b.rows, b.total, b.E, b.H, b.Ie, ctypes.byref(sz)) == 0
    ws = torch.empty(sz.value + 256, dtype=torch.uint8, device=b.dev)
    off = (-ws.data_ptr()) % 256
    mixed = dev_bf16(b.mixed0, b.dev)
    cf.cf_moe_grouped_gelu_forward_fp8(b.d["hq"], b.d["hd"], int(b.e5m2), b.d["rw"], b.d["counts"], b.d["offsets"], b.d["idx"],
                                       b.d["wi"], b.d["wid"], b.d["wo"], b.d["wod"], mixed, b.rows, b.H, b.Ie, b.E, b.total,
                                       ws.data_ptr() + off, sz.value, stream())
    torch.cuda.synchronize()
    return bf16_bits(mixed)


def run_gelu_stages(cf, b: GeluBank):
    """The same bank through the public per-stage entry points (E4M3 hidden states), per-tensor descales spread
    into vectors on the host."""
    import ctypes
    dev, E, H, Ie, total = b.dev, b.E, b.H, b.Ie, b.total
    sz = ctypes.c_size_t(0)
    assert cf.raw_cf_fp8_grouped_gemm_workspace_bytes(total, E, ctypes.byref(sz)) == 0
    ws = torch.empty(sz.value, dtype=torch.uint8, device=dev)
    full = lambda v, n: torch.full((n,), float(v), dtype=torch.float32, device=dev)
    cidx = torch.full((total,), -1, dtype=torch.int32, device=dev)
    cf.cf_moe_compact_row_index(b.d["counts"], b.d["offsets"], b.d["idx"], b.rows, E, cidx, stream())
    act = torch.zeros((total, Ie), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_grouped_gemm_nt_bf16_ex(total, Ie, H, E, b.d["counts"], b.d["offsets"], b.d["hq"], b.rows, H, cidx, full(b.hd, b.rows),
                                      b.d["wi"], full(b.wid, E * Ie), ROW_COL, EPI_NONE, None, None, act, Ie, ws, sz.value, stream())
    actq = torch.empty((total, Ie), dtype=torch.uint8, device=dev)
    a_s = torch.empty(total, device=dev); a_d = torch.empty(total, device=dev)
    cf.cf_gelu_quantize_rows_e4m3(act, total, Ie, actq, a_s, a_d, stream())
    y = torch.zeros((total, H), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_grouped_gemm_nt_bf16_ex(total, H, Ie, E, b.d["counts"], b.d["offsets"], actq, total, Ie, None, a_d,
                                      b.d["wo"], full(b.wod, E * H), ROW_COL, EPI_NONE, None, None, y, H, ws, sz.value, stream())
    mixed = dev_bf16(b.mixed0, dev)
    cf.cf_moe_unpermute_weighted_bf16(mixed, y, b.d["rw"], b.d["counts"], b.d["offsets"], b.d["idx"], b.rows, E, H, stream())
    torch.cuda.synchronize()
    return dict(act=bf16_bits(act), actq=host(actq), a_d=host(a_d), y=bf16_bits(y), mixed=bf16_bits(mixed))


def check_gelu_stages(b: GeluBank, r, experts=None, sample=None):
    E, H, Ie = b.E, b.H, b.Ie
    mixed = b.mixed0
    for e in range(E):
        n, o = int(b.counts[e]), int(b.offsets[e])
        mixed = orc.moe_scatter_accumulate(mixed, r["y"][o:o + n], b.rw, b.idx[e, :n], e)
    assert np.array_equal(r["mixed"], mixed)                                   # weighted unpermute: bit-exact
    for e in (range(E) if experts is None else experts):
        n, o = int(b.counts[e]), int(b.offsets[e])
        if n == 0:
            continue
        sel = np.arange(n) if sample is None or n <= sample else np.sort(np.random.default_rng(e).choice(n, sample, replace=False))
        rows = b.idx[e, :n][sel]
        ref, absdot = orc.gemm_nt_ref(b.hq[rows], b.wi[e * Ie:(e + 1) * Ie], [b.hd], [b.wid], a_e5m2=b.e5m2, scale_mode=0)
        orc.assert_gemm_close(orc.bf16_to_f32(r["act"][o:o + n][sel]).astype(np.float64), ref, absdot, what=f"fc_in expert {e}")
        yref, yabs = orc.gemm_nt_ref(r["actq"][o:o + n][sel], b.wo[e * H:(e + 1) * H], r["a_d"][o:o + n][sel],
                                     np.full(H, b.wod, np.float32), scale_mode=1)
        orc.assert_gemm_close(orc.bf16_to_f32(r["y"][o:o + n][sel]).astype(np.float64), yref, yabs, what=f"fc_out expert {e}")


def gelu_loop_ref(b: GeluBank):
    """The reference's expert loop restated on the host from the oracle's pieces (bf16 roundings where the loop has
    them): returns mixed as bf16 bits."""
    mixed = b.mixed0
    for e in range(b.E):
        n = int(b.counts[e])
        if n == 0:
            continue
        rows = b.idx[e, :n]
        a, _ = orc.gemm_nt_ref(b.hq[rows], b.wi[e * b.Ie:(e + 1) * b.Ie], [b.hd], [b.wid], a_e5m2=b.e5m2, scale_mode=0, want_abs=False)
        g = orc.gelu_forward(orc.bf16_from_f32(a.astype(np.float32)))
        q, _, d = orc.quantize_rows(g)
        y, _ = orc.gemm_nt_ref(q, b.wo[e * b.H:(e + 1) * b.H], d, np.full(b.H, b.wod, np.float32), scale_mode=1, want_abs=False)
        mixed = orc.moe_scatter_accumulate(mixed, orc.bf16_from_f32(y.astype(np.float32)), b.rw, rows, e)
    return mixed


@pytest.mark.parametrize("rows,E,k,H,Ie,zero", [(600, 5, 2, 256, 384, None), (300, 4, 2, 256, 256, 2), (40, 8, 3, 384, 256, None)])
def test_grouped_gelu_bank_on_the_matrix_cores(cf, dev, rows, E, k, H, Ie, zero):
    case(f"grouped gelu bank (mfma) rows={rows} E={E} k={k} H={H} Ie={Ie}")
    b = GeluBank(dev, rows, E, k, H, Ie, seed=rows + Ie, zero_expert=zero)
    r = run_gelu_stages(cf, b)
    check_gelu_stages(b, r)
    got = run_gelu_fused(cf, b)
    assert np.array_equal(got, r["mixed"])                                     # the one-call form is the same computation
    # against the loop restated from the oracle end to end: a GELU value one bf16 ulp apart can move a quantized
    # byte, so this is the GEMM bar on the sum rather than bit equality
    want = orc.bf16_to_f32(gelu_loop_ref(b)).astype(np.float64)
    g = orc.bf16_to_f32(got).astype(np.float64)
    assert np.sqrt(((g - want) ** 2).sum() / (want ** 2).sum()) <= 4e-3
    # and against moe_grouped_expert_forward_fp8's semantics (GELU output kept in fp32): apart by the E4M3
    # rounding of the activations, relative 2^-4 / sqrt(3) per element
    start = orc.bf16_to_f32(b.mixed0).astype(np.float64)
    ref = orc.moe_grouped_expert_forward_fp8_ref(b.hq, b.hd, b.e5m2, b.rw, b.counts, b.idx, b.wi.reshape(E, Ie, H), b.wid,
                                                 b.wo.reshape(E, H, Ie), b.wod, start)
    assert np.sqrt(((g - ref) ** 2).sum() / ((ref - start) ** 2).sum()) <= 0.06
    untouched = ~(b.rw > 0).any(axis=1)
    assert np.array_equal(got[untouched], b.mixed0[untouched])


def test_grouped_gelu_bank_e5m2_hidden_states(cf, dev):
    case("grouped gelu bank (mfma), E5M2 hidden states")
    b = GeluBank(dev, 500, 4, 2, 256, 384, seed=77, e5m2=True)
    got = orc.bf16_to_f32(run_gelu_fused(cf, b)).astype(np.float64)
    want = orc.bf16_to_f32(gelu_loop_ref(b)).astype(np.float64)
    assert np.sqrt(((got - want) ** 2).sum() / (want ** 2).sum()) <= 4e-3
    assert np.all(np.abs(got - want) <= (b.k + 1) * 2.0 ** -7 * (np.abs(want) + np.abs(want).mean()))


def test_grouped_gelu_bank_config5_size(cf, dev):
    """16384 tokens, hidden 2048, 64 experts, top-6, expert width 1408, per-tensor scales."""
    case("grouped gelu bank (mfma), config 5 size")
    b = GeluBank(dev, 16384, 64, 6, 2048, 1408, seed=6)
    assert b.total == 98304
    r = run_gelu_stages(cf, b)
    check_gelu_stages(b, r, experts=[0, 40, 63], sample=24)
    assert np.array_equal(run_gelu_fused(cf, b), r["mixed"])


def test_grouped_gelu_bank_argument_errors(cf, dev):
    case("grouped gelu bank argument checks")
    import ctypes
    sz = ctypes.c_size_t(0)
    assert cf.raw_cf_moe_grouped_gelu_workspace_bytes(16, 32, 4, 256, 256, None) != 0
    assert cf.raw_cf_moe_grouped_gelu_workspace_bytes(-1, 32, 4, 256, 256, ctypes.byref(sz)) != 0
    b = GeluBank(dev, 64, 4, 2, 256, 256, seed=3)
    assert cf.raw_cf_moe_grouped_gelu_workspace_bytes(b.rows, b.total, b.E, b.H, b.Ie, ctypes.byref(sz)) == 0
    ws = torch.empty(sz.value + 256, dtype=torch.uint8, device=dev)
    p = ws.data_ptr() + (-ws.data_ptr()) % 256
    mixed = dev_bf16(b.mixed0, dev)
    args = lambda wsp, nbytes, H=b.H: (b.d["hq"].data_ptr(), b.d["hd"].data_ptr(), 0, b.d["rw"].data_ptr(), b.d["counts"].data_ptr(),
                                       b.d["offsets"].data_ptr(), b.d["idx"].data_ptr(), b.d["wi"].data_ptr(), b.d["wid"].data_ptr(),
                                       b.d["wo"].data_ptr(), b.d["wod"].data_ptr(), mixed.data_ptr(), b.rows, H, b.Ie, b.E, b.total,
                                       wsp, nbytes, None)
    assert cf.raw_cf_moe_grouped_gelu_forward_fp8(*args(p, sz.value - 1)) == -1            # workspace too small
    assert cf.raw_cf_moe_grouped_gelu_forward_fp8(*args(p + 16, sz.value)) == -1           # workspace misaligned
    assert cf.raw_cf_moe_grouped_gelu_forward_fp8(*args(None, sz.value)) == -1
    assert cf.raw_cf_moe_grouped_gelu_forward_fp8(*args(p, sz.value, H=200)) == -2         # K not a multiple of 128
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(mixed), b.mixed0)                                      # nothing ran


def test_grouped_gelu_expert_bank_reference_form_config5_size(cf, dev):
    """moe_grouped_expert_forward_fp8 at 16384 tokens, hidden 2048, 64 experts, top-6, width 1408: a sample of token rows
    against the double reference of exactly those rows."""
    case("grouped gelu bank, reference form, config 5 size")
    b = GeluBank(dev, 16384, 64, 6, 2048, 1408, seed=8)
    mixed = dev_bf16(b.mixed0, dev)
    cf.cf_moe_grouped_expert_forward_fp8(b.d["hq"], b.d["hd"], 0, b.d["rw"], b.d["counts"], None, b.d["idx"], b.d["wi"], b.d["wid"],
                                         b.d["wo"], b.d["wod"], mixed, b.rows, b.H, b.Ie, b.E, b.total, stream())
    torch.cuda.synchronize()
    sel = np.sort(np.random.default_rng(1).choice(b.rows, 40, replace=False))
    sel[0], sel[-1] = 0, b.rows - 1
    rw = np.ascontiguousarray(b.rw[sel])
    counts, idx = orc.moe_build_expert_row_lists(rw)
    start = orc.bf16_to_f32(b.mixed0[sel]).astype(np.float64)
    ref = orc.moe_grouped_expert_forward_fp8_ref(b.hq[sel], b.hd, False, rw, counts, idx, b.wi.reshape(b.E, b.Ie, b.H), b.wid,
                                                 b.wo.reshape(b.E, b.H, b.Ie), b.wod, start)
    got = orc.bf16_to_f32(bf16_bits(mixed)[sel]).astype(np.float64)
    assert np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum()) <= 4e-3
    typical = np.sqrt(((ref - start) ** 2).mean())
    assert np.all(np.abs(got - ref) <= (b.k + 1) * 2.0 ** -8 * (np.abs(start) + np.abs(ref) + 2.0 * typical))


@pytest.mark.parametrize("rows,E,k,H,Ie", [(90, 4, 2, 96, 72), (33, 3, 3, 40, 1408),
                                            # H % 64 == 0 and Ie % 64 == 0: the matrix-core form
                                            (300, 6, 3, 256, 320), (70, 3, 3, 2048, 1408), (200, 4, 2, 64, 64), (21, 5, 2, 192, 448)])
def test_grouped_gelu_expert_bank_bf16_sibling(cf, dev, rows, E, k, H, Ie):
    """moe_grouped_expert_forward_bf16: bf16 hidden states and weights, float GELU intermediate, bf16 CAS accumulate."""
    case(f"grouped gelu bank, bf16 sibling rows={rows} E={E} k={k} H={H} Ie={Ie}")
    rng = np.random.default_rng(rows + Ie + 1)
    hidden = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))
    win = orc.bf16_from_f32((0.05 * rng.standard_normal((E, Ie, H))).astype(np.float32))
    wout = orc.bf16_from_f32((0.05 * rng.standard_normal((E, H, Ie))).astype(np.float32))
    rw = orc.moe_topk_route(rng.standard_normal((rows, E)).astype(np.float32), k)
    counts, idx = orc.moe_build_expert_row_lists(rw)
    mixed0 = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))
    mixed = dev_bf16(mixed0, dev)
    cf.cf_moe_grouped_expert_forward_bf16(dev_bf16(hidden, dev), dev_arr(rw, dev), dev_arr(counts, dev), None, dev_arr(idx, dev),
                                          dev_bf16(win, dev), dev_bf16(wout, dev), mixed, rows, H, Ie, E, rows * k, stream())
    torch.cuda.synchronize()
    start = orc.bf16_to_f32(mixed0).astype(np.float64)
    ref = orc.moe_grouped_expert_forward_bf16_ref(hidden, rw, counts, idx, win, wout, start)
    got = orc.bf16_to_f32(bf16_bits(mixed)).astype(np.float64)
    assert np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum()) <= 4e-3
    typical = np.sqrt(((ref - start) ** 2).mean())
    assert np.all(np.abs(got - ref) <= (k + 1) * 2.0 ** -8 * (np.abs(start) + np.abs(ref) + 2.0 * typical))
    untouched = ~(rw > 0).any(axis=1)
    assert np.array_equal(bf16_bits(mixed)[untouched], mixed0[untouched])
    assert cf.raw_cf_moe_grouped_expert_forward_bf16(None, None, None, None, None, None, None, None, 4, 8, 8, 2, 8, None) == -1


@pytest.mark.parametrize("rows,E,k,H,Ie,zero", [(100, 4, 2, 256, 128, 1), (5, 3, 1, 128, 64, None), (37, 3, 2, 2304, 64, 0)])
def test_grouped_gelu_reference_form_ragged_and_empty_experts(cf, dev, rows, E, k, H, Ie, zero):
    """The matrix-core forms with experts nobody selects, lists shorter than one row tile, and a last tile that ends
    inside the first group of 16 rows."""
    case(f"grouped gelu bank, reference form, ragged rows={rows} E={E} k={k} H={H} Ie={Ie} zero={zero}")
    b = GeluBank(dev, rows, E, k, H, Ie, seed=rows + H, zero_expert=zero)
    if zero is not None:
        assert b.counts[zero] == 0
    mixed = dev_bf16(b.mixed0, dev)
    cf.cf_moe_grouped_expert_forward_fp8(b.d["hq"], b.d["hd"], 0, b.d["rw"], b.d["counts"], None, b.d["idx"], b.d["wi"], b.d["wid"],
                                         b.d["wo"], b.d["wod"], mixed, b.rows, b.H, b.Ie, b.E, b.total, stream())
    torch.cuda.synchronize()
    start = orc.bf16_to_f32(b.mixed0).astype(np.float64)
    ref = orc.moe_grouped_expert_forward_fp8_ref(b.hq, b.hd, False, b.rw, b.counts, b.idx, b.wi.reshape(E, Ie, H), b.wid,
                                                 b.wo.reshape(E, H, Ie), b.wod, start)
    got = orc.bf16_to_f32(bf16_bits(mixed)).astype(np.float64)
    assert np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum()) <= 4e-3
    typical = np.sqrt(((ref - start) ** 2).mean())
    assert np.all(np.abs(got - ref) <= (k + 1) * 2.0 ** -8 * (np.abs(start) + np.abs(ref) + 2.0 * typical))


def test_gelu_quantize_rows_argument_errors(cf, dev):
    case("gelu + per-row quantize argument checks")
    z = torch.zeros(64, dtype=torch.bfloat16, device=dev)
    q = torch.zeros(64, dtype=torch.uint8, device=dev)
    s = torch.zeros(4, device=dev)
    assert cf.raw_cf_gelu_quantize_rows_e4m3(None, 4, 16, q.data_ptr(), s.data_ptr(), s.data_ptr(), None) == -1
    assert cf.raw_cf_gelu_quantize_rows_e4m3(z.data_ptr(), 4, 16, None, s.data_ptr(), s.data_ptr(), None) == -1
    assert cf.raw_cf_gelu_quantize_rows_e4m3(z.data_ptr(), 4, 16, q.data_ptr(), None, s.data_ptr(), None) == -1
    assert cf.raw_cf_gelu_quantize_rows_e4m3(z.data_ptr(), -1, 16, q.data_ptr(), s.data_ptr(), s.data_ptr(), None) == -1
    assert cf.raw_cf_gelu_quantize_rows_e4m3(None, 0, 16, None, None, None, None) == 0
    # K = 0: nothing to convert, the scales of an empty row are those of amax = 0
    assert cf.raw_cf_gelu_quantize_rows_e4m3(None, 4, 0, None, s.data_ptr(), s.data_ptr(), None) == 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("rows,K", [(49152, 1408), (16384, 4096)])
def test_gelu_quantize_rows_table_form(cf, dev, rows, K):
    """Enough rows for the form that looks GELU up in a per-workgroup table of all 65536 bf16 values: bytes and scales
    must equal gelu_forward followed by the per-row quantize (both pinned against the oracle elsewhere), NaN and
    infinity rows included."""
    case(f"gelu + per-row quantize, table form rows={rows} K={K}")
    g = torch.Generator(device=dev); g.manual_seed(rows + K)
    x = (torch.randn(rows, K, device=dev, generator=g) * 2.5).to(torch.bfloat16)
    x[0, :] = 0
    x[1, 5] = float("nan"); x[2, 7] = float("inf"); x[3, 9] = float("-inf")
    x[4] = torch.arange(K, device=dev).to(torch.bfloat16) - K / 2                  # large magnitudes
    q = torch.zeros((rows, K), dtype=torch.uint8, device=dev); s = torch.zeros(rows, device=dev); d = torch.zeros(rows, device=dev)
    cf.cf_gelu_quantize_rows_e4m3(x, rows, K, q, s, d, stream())
    y = torch.empty_like(x)
    cf.cf_gelu_forward_bf16(x, y, rows * K, stream())
    q2 = torch.zeros_like(q); s2 = torch.zeros_like(s); d2 = torch.zeros_like(d)
    cf.cf_fp8_quantize_rows(y, rows, K, 0, q2, s2, d2, stream())
    torch.cuda.synchronize()
    assert torch.equal(q, q2)
    assert torch.equal(s.view(torch.int32), s2.view(torch.int32)) and torch.equal(d.view(torch.int32), d2.view(torch.int32))
