"""GPU parity: moe_grouped_expert_forward_fp8 (/root/reference/kernels/moe.cu:950-1127) as whole-matrix launches with
a workspace (cf_moe_grouped_expert_forward_fp8_ws), and its bf16 sibling (cf_moe_grouped_expert_forward_bf16_ws).

Every stage is checked on the intermediates the call leaves in its workspace, given that stage's own (GPU) inputs:
the fp32 projections against the double product of the dequantized operands; the three-term E4M3 split of the GELU
against the exact-erf GELU of those projections (12 bits and better, and the row maximum lands on 448); the fc_out
GEMM, whose matrix-core scales weight term t by 16^-t, against the double product of the recombined terms at fp32
accumulation error; the result against the oracle of the reference kernel at the bars of the one-kernel form's test."""
import ctypes
import math

import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_arr, dev_bf16, host, stream

pytestmark = pytest.mark.gpu

NAMES = ["TILE_MAP", "OFFSETS", "INDEX", "SLOT", "PRE", "SPLIT", "SPLIT_DESCALE", "Y", "X"]
# the block-scaled FP8 MFMA aligns the products of a K-block to the largest one before adding them, so the terms it
# scales by 2^-4 and 2^-8 lose low bits: measured up to 2 x the unscaled FP8 MFMA's accumulation error
ACC_MX = 4.0 * orc.ACC_MFMA
ACC_BF16 = 16.0 * 2.0 ** -24          # fp32 accumulation of bf16 products on the matrix cores, per sum |a_k b_k|
erf = np.vectorize(math.erf, otypes=[np.float64])


def gelu64(x):
    return 0.5 * x * (1.0 + erf(x * 0.70710678118654752440))


class Bank:
    def __init__(self, dev, rows, E, k, H, Ie, e5m2, seed, zero_expert=None):
        rng = np.random.default_rng(seed)
        self.rows, self.E, self.k, self.H, self.Ie, self.e5m2, self.dev = rows, E, k, H, Ie, e5m2, dev
        x = rng.standard_normal((rows, H)).astype(np.float32)
        fmax = 57344.0 if e5m2 else 448.0
        sx = np.float32(fmax) / np.abs(x).max()
        self.hq = (orc.e5m2_satfinite if e5m2 else orc.e4m3_satfinite)(x * sx)
        win = (0.05 * rng.standard_normal((E, Ie, H))).astype(np.float32)
        wout = (0.05 * rng.standard_normal((E, H, Ie))).astype(np.float32)
        s_in, s_out = np.float32(448.0) / np.abs(win).max(), np.float32(448.0) / np.abs(wout).max()
        self.winq, self.woutq = orc.e4m3_satfinite(win * s_in), orc.e4m3_satfinite(wout * s_out)
        self.d_h, self.d_in, self.d_out = np.float32(1) / sx, np.float32(1) / s_in, np.float32(1) / s_out
        logits = rng.standard_normal((rows, E)).astype(np.float32)
        if zero_expert is not None:
            logits[:, zero_expert] = -50.0
        self.rw = orc.moe_topk_route(logits, k)
        self.counts, self.idx = orc.moe_build_expert_row_lists(self.rw)
        self.total = int(self.counts.sum())
        self.mixed0 = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))

    def compact_index(self):
        return np.concatenate([self.idx[e, : self.counts[e]] for e in range(self.E)])

    def expert_of_compact(self):
        return np.repeat(np.arange(self.E), self.counts)


def workspace(cf, b):
    offs = (ctypes.c_size_t * len(NAMES))()
    nbytes = ctypes.c_size_t()
    cf.cf_moe_grouped_expert_forward_fp8_workspace(b.rows, b.total, b.E, b.H, b.Ie, offs, ctypes.byref(nbytes))
    return {n: int(offs[i]) for i, n in enumerate(NAMES)}, int(nbytes.value)


def run(cf, b, pass_offsets=False):
    dev = b.dev
    off, nbytes = workspace(cf, b)
    ws = torch.empty(max(nbytes, 256) + 256, dtype=torch.uint8, device=dev)
    ws.fill_(0xCD)
    shift = (-ws.data_ptr()) % 256
    ws = ws[shift:shift + max(nbytes, 256)]
    mixed = dev_bf16(b.mixed0, dev)
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    offsets = dev_arr(orc.moe_expert_offsets(b.counts), dev) if pass_offsets else None
    cf.cf_moe_grouped_expert_forward_fp8_ws(dev_arr(b.hq, dev), sc(b.d_h), int(b.e5m2), dev_arr(b.rw, dev), dev_arr(b.counts, dev), offsets,
                                            dev_arr(b.idx, dev), dev_arr(b.winq, dev), sc(b.d_in), dev_arr(b.woutq, dev), sc(b.d_out),
                                            mixed, b.rows, b.H, b.Ie, b.E, b.total, ws if nbytes else None, nbytes, stream())
    torch.cuda.synchronize()
    return mixed, ws, off, nbytes


def check_result(b, mixed):
    start = orc.bf16_to_f32(b.mixed0).astype(np.float64)
    ref = orc.moe_grouped_expert_forward_fp8_ref(b.hq, b.d_h, b.e5m2, b.rw, b.counts, b.idx, b.winq, b.d_in, b.woutq, b.d_out, start)
    got = orc.bf16_to_f32(bf16_bits(mixed)).astype(np.float64)
    rel = np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum())
    assert rel <= 4e-3, rel
    # every one of the k accumulations rounds the running value to bf16: the bound of the one-kernel form's test
    typical = np.sqrt(((ref - start) ** 2).mean())
    bound = (b.k + 1) * 2.0 ** -8 * (np.abs(start) + np.abs(ref) + 2.0 * typical)
    assert np.all(np.abs(got - ref) <= bound)
    untouched = ~(b.rw > 0).any(axis=1)
    assert np.array_equal(bf16_bits(mixed)[untouched], b.mixed0[untouched])
    return rel


@pytest.mark.parametrize("rows,E,k,H,Ie,e5m2,zero", [
    (70, 3, 3, 2048, 1408, False, None),       # config 5's widths: 11 K-tiles per term
    (40, 3, 2, 2304, 128, False, None),        # one K-tile per term: the weight columns wrap at every K-tile
    (300, 6, 3, 256, 384, True, None),         # E5M2 hidden states, two K-tiles of fc_in
    (1000, 5, 2, 384, 256, False, 2),          # several row tiles per expert, ragged last ones, an expert with no rows
    (64, 2, 1, 256, 4096, False, None),        # the widest row the split keeps in registers
])
def test_staged_bank_stage_by_stage(cf, dev, rows, E, k, H, Ie, e5m2, zero):
    case(f"staged gelu bank rows={rows} E={E} k={k} H={H} Ie={Ie} e5m2={e5m2} zero_expert={zero}")
    b = Bank(dev, rows, E, k, H, Ie, e5m2, seed=rows + Ie, zero_expert=zero)
    mixed, ws, off, nbytes = run(cf, b)
    assert nbytes > 0
    T = b.total
    raw = host(ws)
    take = lambda name, dtype, count: raw[off[name]: off[name] + count * np.dtype(dtype).itemsize].view(dtype)
    index = take("INDEX", np.int32, T)
    assert np.array_equal(index, b.compact_index())
    assert np.array_equal(take("OFFSETS", np.int32, E), orc.moe_expert_offsets(b.counts))
    expert = b.expert_of_compact()

    # fc_in: fp32 projections of the gathered rows
    hx = (orc.e5m2_unpack if e5m2 else orc.e4m3_unpack)(b.hq).astype(np.float64)
    win = orc.e4m3_unpack(b.winq).astype(np.float64)
    wout = orc.e4m3_unpack(b.woutq).astype(np.float64)
    pre = take("PRE", np.float32, T * Ie).reshape(T, Ie).astype(np.float64)
    s_in = float(np.float32(b.d_h) * np.float32(b.d_in))
    for e in range(E):
        sel = expert == e
        if not sel.any():
            continue
        want = (hx[index[sel]] @ win[e].T) * s_in
        ad = (np.abs(hx[index[sel]]) @ np.abs(win[e]).T) * s_in
        assert np.all(np.abs(pre[sel] - want) <= 2.0 ** -22 * np.abs(want) + orc.ACC_MFMA * ad), f"fc_in expert {e}"

    # split: three terms recombine to the exact-erf GELU of the GPU's projections
    q = take("SPLIT", np.uint8, T * 3 * Ie).reshape(T, 3, Ie)
    d = take("SPLIT_DESCALE", np.float32, T).astype(np.float64)
    terms = orc.e4m3_unpack(q).astype(np.float64)
    recon = (terms[:, 0] + terms[:, 1] / 16.0 + terms[:, 2] / 256.0) * d[:, None]
    g = gelu64(pre)
    amax = np.abs(g).max(axis=1)
    assert np.allclose(d, amax / 448.0, rtol=1e-5), "row descale is amax / 448"
    assert np.all(np.abs(terms[:, 0]).max(axis=1) == 448.0), "the row maximum lands on the largest E4M3 value"
    tol = 2.0 ** -12 * np.abs(g) + (amax * 2.0 ** -17 / 448.0)[:, None] + 4e-7 * (np.abs(pre) + 1e-3)
    worst = np.abs(recon - g) / tol
    assert worst.max() <= 1.0, f"split worst {worst.max():.3f}"
    # ... and carries more than bf16 would: compare the two errors over the elements that matter
    big = np.abs(g) >= amax[:, None] * 2.0 ** -6
    bf = orc.bf16_to_f32(orc.bf16_from_f32(g.astype(np.float32))).astype(np.float64)
    assert np.abs(recon - g)[big].max() / np.abs(g)[big].max() < 2.0 ** -12
    assert np.sqrt(((recon - g)[big] ** 2).mean()) < 0.125 * np.sqrt(((bf - g)[big] ** 2).mean())

    # fc_out: the matrix cores weight the terms; the fp32 sum is stored as it is
    y = take("Y", np.float32, T * H).reshape(T, H).astype(np.float64)
    act = terms[:, 0] + terms[:, 1] / 16.0 + terms[:, 2] / 256.0
    act_abs = np.abs(terms[:, 0]) + np.abs(terms[:, 1]) / 16.0 + np.abs(terms[:, 2]) / 256.0
    for e in range(E):
        sel = expert == e
        if not sel.any():
            continue
        rowscale = d[sel][:, None] * float(b.d_out)
        want = (act[sel] @ wout[e].T) * rowscale
        ad = (act_abs[sel] @ np.abs(wout[e]).T) * rowscale
        tol = 2.0 ** -22 * np.abs(want) + ACC_MX * ad
        worst = np.abs(y[sel] - want) / tol
        print(f"fc_out expert {e}: worst error / tolerance {worst.max():.3f}")
        assert worst.max() <= 1.0, f"fc_out expert {e}: worst {worst.max():.3f}"
        # end to end from the exact-erf GELU in double: what the split and the matrix cores lose together, against what
        # rounding the activations to bf16 would lose
        exact = (g[sel] @ wout[e].T) * float(b.d_out)
        lost = np.sqrt(((y[sel] - exact) ** 2).sum() / (exact ** 2).sum())
        lost_bf16 = np.sqrt((((bf[sel] @ wout[e].T) * float(b.d_out) - exact) ** 2).sum() / (exact ** 2).sum())
        print(f"fc_out expert {e}: rel L2 from exact GELU {lost:.2e}, with bf16 activations {lost_bf16:.2e}")
        assert lost < 0.1 * lost_bf16

    check_result(b, mixed)


def test_staged_bank_takes_offsets_and_repeats(cf, dev):
    """Offsets handed in or recomputed, and a second call on a dirty workspace: the same bits."""
    case("staged gelu bank, offsets given / recomputed, repeated")
    b = Bank(dev, 500, 8, 2, 512, 256, False, seed=5)
    m1, ws, off, nbytes = run(cf, b)
    m2, _, _, _ = run(cf, b, pass_offsets=True)
    assert np.array_equal(bf16_bits(m1), bf16_bits(m2))
    check_result(b, m1)


def test_other_shapes_pass_through_without_a_workspace(cf, dev):
    case("staged gelu bank entry on a shape of the one-kernel forms")
    b = Bank(dev, 200, 4, 2, 128, 64, False, seed=9)
    mixed, _, _, nbytes = run(cf, b)
    assert nbytes == 0
    start = orc.bf16_to_f32(b.mixed0).astype(np.float64)
    ref = orc.moe_grouped_expert_forward_fp8_ref(b.hq, b.d_h, False, b.rw, b.counts, b.idx, b.winq, b.d_in, b.woutq, b.d_out, start)
    got = orc.bf16_to_f32(bf16_bits(mixed)).astype(np.float64)
    assert np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum()) <= 4e-3


def cf_conv(v):
    return v.data_ptr() if hasattr(v, "data_ptr") else v


def test_staged_bank_rejects_a_short_workspace(cf, dev):
    case("staged gelu bank, short or missing workspace")
    b = Bank(dev, 64, 2, 1, 256, 128, False, seed=3)
    off, nbytes = workspace(cf, b)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    mixed = dev_bf16(b.mixed0, dev)
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    args = lambda w, n: (dev_arr(b.hq, dev), sc(b.d_h), 0, dev_arr(b.rw, dev), dev_arr(b.counts, dev), None, dev_arr(b.idx, dev),
                         dev_arr(b.winq, dev), sc(b.d_in), dev_arr(b.woutq, dev), sc(b.d_out), mixed, b.rows, b.H, b.Ie, b.E, b.total,
                         w, n, stream())
    assert cf.raw_cf_moe_grouped_expert_forward_fp8_ws(*[cf_conv(a) for a in args(ws, nbytes - 1)]) == -1
    assert cf.raw_cf_moe_grouped_expert_forward_fp8_ws(*[cf_conv(a) for a in args(None, nbytes)]) == -1
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(mixed), b.mixed0)


# ---- the bf16 sibling --------------------------------------------------------------------------------------------

class Bank16:
    def __init__(self, dev, rows, E, k, H, Ie, seed, zero_expert=None):
        rng = np.random.default_rng(seed)
        self.rows, self.E, self.k, self.H, self.Ie, self.dev = rows, E, k, H, Ie, dev
        self.hidden = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))
        self.win = orc.bf16_from_f32((0.05 * rng.standard_normal((E, Ie, H))).astype(np.float32))
        self.wout = orc.bf16_from_f32((0.05 * rng.standard_normal((E, H, Ie))).astype(np.float32))
        logits = rng.standard_normal((rows, E)).astype(np.float32)
        if zero_expert is not None:
            logits[:, zero_expert] = -50.0
        self.rw = orc.moe_topk_route(logits, k)
        self.counts, self.idx = orc.moe_build_expert_row_lists(self.rw)
        self.total = int(self.counts.sum())
        self.mixed0 = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))


def run16(cf, b):
    dev = b.dev
    offs = (ctypes.c_size_t * len(NAMES))()
    nbytes = ctypes.c_size_t()
    cf.cf_moe_grouped_expert_forward_bf16_workspace(b.rows, b.total, b.E, b.H, b.Ie, offs, ctypes.byref(nbytes))
    off, nbytes = {n: int(offs[i]) for i, n in enumerate(NAMES)}, int(nbytes.value)
    ws = torch.empty(max(nbytes, 256) + 256, dtype=torch.uint8, device=dev)
    ws.fill_(0xCD)
    shift = (-ws.data_ptr()) % 256
    ws = ws[shift:shift + max(nbytes, 256)]
    mixed = dev_bf16(b.mixed0, dev)
    cf.cf_moe_grouped_expert_forward_bf16_ws(dev_bf16(b.hidden, dev), dev_arr(b.rw, dev), dev_arr(b.counts, dev), None, dev_arr(b.idx, dev),
                                             dev_bf16(b.win, dev), dev_bf16(b.wout, dev), mixed, b.rows, b.H, b.Ie, b.E, b.total,
                                             ws if nbytes else None, nbytes, stream())
    torch.cuda.synchronize()
    return mixed, ws, off, nbytes


def check_result16(b, mixed):
    start = orc.bf16_to_f32(b.mixed0).astype(np.float64)
    ref = orc.moe_grouped_expert_forward_bf16_ref(b.hidden, b.rw, b.counts, b.idx, b.win, b.wout, start)
    got = orc.bf16_to_f32(bf16_bits(mixed)).astype(np.float64)
    assert np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum()) <= 4e-3
    typical = np.sqrt(((ref - start) ** 2).mean())
    assert np.all(np.abs(got - ref) <= (b.k + 1) * 2.0 ** -8 * (np.abs(start) + np.abs(ref) + 2.0 * typical))
    untouched = ~(b.rw > 0).any(axis=1)
    assert np.array_equal(bf16_bits(mixed)[untouched], b.mixed0[untouched])


@pytest.mark.parametrize("rows,E,k,H,Ie,zero", [
    (70, 3, 3, 2048, 1408, None),        # config 5's widths
    (300, 6, 3, 256, 320, None),         # Ie = 5 K-tiles
    (200, 4, 2, 64, 64, None),           # one K-tile per projection
    (1000, 5, 2, 192, 448, 2),           # several row tiles per expert, ragged, an expert with no rows; N = 448 and 192 end inside a column tile
    (21, 5, 2, 200, 128, None),          # H % 64 != 0: the k range of fc_in ends inside a K-tile
])
def test_staged_bf16_bank_stage_by_stage(cf, dev, rows, E, k, H, Ie, zero):
    case(f"staged bf16 gelu bank rows={rows} E={E} k={k} H={H} Ie={Ie} zero_expert={zero}")
    b = Bank16(dev, rows, E, k, H, Ie, seed=rows + Ie + 1, zero_expert=zero)
    mixed, ws, off, nbytes = run16(cf, b)
    assert nbytes > 0
    T = b.total
    raw = host(ws)
    take = lambda name, dtype, count: raw[off[name]: off[name] + count * np.dtype(dtype).itemsize].view(dtype)
    index = take("INDEX", np.int32, T)
    assert np.array_equal(index, np.concatenate([b.idx[e, : b.counts[e]] for e in range(E)]))
    expert = np.repeat(np.arange(E), b.counts)

    hx = orc.bf16_to_f32(b.hidden).astype(np.float64)
    win = orc.bf16_to_f32(b.win).astype(np.float64)
    wout = orc.bf16_to_f32(b.wout).astype(np.float64)
    pre = take("PRE", np.float32, T * Ie).reshape(T, Ie).astype(np.float64)
    for e in range(E):
        sel = expert == e
        if not sel.any():
            continue
        want = hx[index[sel]] @ win[e].T
        ad = np.abs(hx[index[sel]]) @ np.abs(win[e]).T
        assert np.all(np.abs(pre[sel] - want) <= 2.0 ** -22 * np.abs(want) + ACC_BF16 * ad), f"fc_in expert {e}"

    # the GELU output rounded to bf16, as the reference kernel parks it before fc_out (kernels/moe.cu:845)
    act_bits = take("SPLIT", np.uint16, T * Ie).reshape(T, Ie)
    act = orc.bf16_to_f32(act_bits).astype(np.float64)
    g = gelu64(pre)
    gb = orc.bf16_from_f32(g.astype(np.float32))
    # the erf form is good to 4e-7 (|pre| + 1e-3) absolute: away from zero that can only flip a rounding now and then
    big = np.abs(g) >= 2.0 ** -6
    off_by = np.abs(act_bits.astype(np.int64) - gb.astype(np.int64))[big]
    assert off_by.max() <= 1 and (off_by != 0).mean() < 2e-2, (off_by.max(), (off_by != 0).mean())
    assert (np.abs(act - g) <= 2.0 ** -8 * np.abs(g) + 4e-7 * (np.abs(pre) + 1e-3)).all()

    y = take("Y", np.float32, T * H).reshape(T, H).astype(np.float64)
    for e in range(E):
        sel = expert == e
        if not sel.any():
            continue
        want = act[sel] @ wout[e].T
        ad = np.abs(act[sel]) @ np.abs(wout[e]).T
        tol = 2.0 ** -22 * np.abs(want) + ACC_BF16 * ad
        worst = np.abs(y[sel] - want) / tol
        assert worst.max() <= 1.0, f"fc_out expert {e}: worst {worst.max():.3f}"
    check_result16(b, mixed)


def test_staged_bf16_bank_other_shapes_pass_through(cf, dev):
    case("staged bf16 gelu bank entry on a shape of the one-kernel forms")
    b = Bank16(dev, 50, 3, 2, 64, 40, seed=2)
    mixed, _, _, nbytes = run16(cf, b)
    assert nbytes == 0
    check_result16(b, mixed)


# ---- config 5 size: a sample of token rows against the double reference of exactly those rows -------------------

def sample_rows(rows):
    sel = np.sort(np.random.default_rng(1).choice(rows, 40, replace=False))
    sel[0], sel[-1] = 0, rows - 1
    return sel


def test_staged_bank_config5_size(cf, dev):
    case("staged gelu bank, config 5 size")
    b = Bank(dev, 16384, 64, 6, 2048, 1408, False, seed=8)
    assert b.total == 98304
    mixed, ws, off, nbytes = run(cf, b)
    sel = sample_rows(b.rows)
    rw = np.ascontiguousarray(b.rw[sel])
    counts, idx = orc.moe_build_expert_row_lists(rw)
    start = orc.bf16_to_f32(b.mixed0[sel]).astype(np.float64)
    ref = orc.moe_grouped_expert_forward_fp8_ref(b.hq[sel], b.d_h, False, rw, counts, idx, b.winq, b.d_in, b.woutq, b.d_out, start)
    got = orc.bf16_to_f32(bf16_bits(mixed)[sel]).astype(np.float64)
    assert np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum()) <= 4e-3
    typical = np.sqrt(((ref - start) ** 2).mean())
    assert np.all(np.abs(got - ref) <= (b.k + 1) * 2.0 ** -8 * (np.abs(start) + np.abs(ref) + 2.0 * typical))
    # rows nobody samples: every row moved, and by a plausible amount (a tile that was skipped or written twice shows)
    all_got = orc.bf16_to_f32(bf16_bits(mixed)).astype(np.float64)
    delta = np.abs(all_got - orc.bf16_to_f32(b.mixed0).astype(np.float64)).mean(axis=1)
    assert delta.min() > 0.1 * np.median(delta) and delta.max() < 10.0 * np.median(delta)
    # a second call on the same workspace gives the same bits
    mixed2, _, _, _ = run(cf, b)
    assert np.array_equal(bf16_bits(mixed2), bf16_bits(mixed))


def test_staged_bf16_bank_config5_size(cf, dev):
    case("staged bf16 gelu bank, config 5 size")
    b = Bank16(dev, 16384, 64, 6, 2048, 1408, seed=9)
    assert b.total == 98304
    mixed, ws, off, nbytes = run16(cf, b)
    sel = sample_rows(b.rows)
    rw = np.ascontiguousarray(b.rw[sel])
    counts, idx = orc.moe_build_expert_row_lists(rw)
    start = orc.bf16_to_f32(b.mixed0[sel]).astype(np.float64)
    ref = orc.moe_grouped_expert_forward_bf16_ref(b.hidden[sel], rw, counts, idx, b.win, b.wout, start)
    got = orc.bf16_to_f32(bf16_bits(mixed)[sel]).astype(np.float64)
    assert np.sqrt(((got - ref) ** 2).sum() / (ref ** 2).sum()) <= 4e-3
    typical = np.sqrt(((ref - start) ** 2).mean())
    assert np.all(np.abs(got - ref) <= (b.k + 1) * 2.0 ** -8 * (np.abs(start) + np.abs(ref) + 2.0 * typical))
    all_got = orc.bf16_to_f32(bf16_bits(mixed)).astype(np.float64)
    delta = np.abs(all_got - orc.bf16_to_f32(b.mixed0).astype(np.float64)).mean(axis=1)
    assert delta.min() > 0.1 * np.median(delta) and delta.max() < 10.0 * np.median(delta)


# ---- total_selected_rows is the caller's upper bound (rows * top_k, /root/reference/src/trainer.cu:6863) ------------

def run_total(cf, b, total, guard=4096, st=None, form="fp8"):
    """The workspace form with `total` as the bound: workspace sized for it, guard bytes behind it that must survive."""
    dev = b.dev
    nbytes = ctypes.c_size_t()
    if form == "fp8":
        cf.cf_moe_grouped_expert_forward_fp8_workspace(b.rows, total, b.E, b.H, b.Ie, None, ctypes.byref(nbytes))
    else:
        cf.cf_moe_grouped_expert_forward_bf16_workspace(b.rows, total, b.E, b.H, b.Ie, None, ctypes.byref(nbytes))
    nbytes = int(nbytes.value)
    buf = torch.empty(nbytes + 256 + guard, dtype=torch.uint8, device=dev)
    buf.fill_(0xA7)
    shift = (-buf.data_ptr()) % 256
    ws = buf[shift:shift + nbytes]
    mixed = dev_bf16(b.mixed0, dev)
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    # the operands are returned with the result: a call on a side stream may still be reading them when this returns
    if form == "fp8":
        ops = [dev_arr(b.hq, dev), sc(b.d_h), dev_arr(b.rw, dev), dev_arr(b.counts, dev), dev_arr(b.idx, dev), dev_arr(b.winq, dev),
               sc(b.d_in), dev_arr(b.woutq, dev), sc(b.d_out)]
    else:
        ops = [dev_bf16(b.hidden, dev), dev_arr(b.rw, dev), dev_arr(b.counts, dev), dev_arr(b.idx, dev), dev_bf16(b.win, dev),
               dev_bf16(b.wout, dev)]
    if st is not None:
        st.wait_stream(torch.cuda.current_stream())      # the uploads above ran on the current stream
    s = stream() if st is None else st.cuda_stream
    if form == "fp8":
        cf.cf_moe_grouped_expert_forward_fp8_ws(ops[0], ops[1], int(b.e5m2), ops[2], ops[3], None, ops[4], ops[5], ops[6], ops[7], ops[8],
                                                mixed, b.rows, b.H, b.Ie, b.E, total, ws, nbytes, s)
    else:
        cf.cf_moe_grouped_expert_forward_bf16_ws(ops[0], ops[1], ops[2], None, ops[3], ops[4], ops[5], mixed, b.rows, b.H,
                                                 b.Ie, b.E, total, ws, nbytes, s)
    return mixed, (buf, ops), shift + nbytes


def test_total_is_an_upper_bound(cf, dev):
    case("workspace forms with total_selected_rows = rows * top_k above the sum of the counts (an expert nobody selects)")
    b8 = Bank(dev, 500, 8, 2, 512, 256, False, seed=21, zero_expert=5)
    b16 = Bank16(dev, 500, 8, 2, 512, 256, seed=22)
    # some rows select fewer than k experts once a weight underflows to zero: make that certain
    b8.rw[::7, :] = 0.0
    b8.rw[::7, 1] = 1.0
    b8.counts, b8.idx = orc.moe_build_expert_row_lists(b8.rw)
    b8.total = int(b8.counts.sum())
    assert b8.total < b8.rows * b8.k and b8.counts[5] == 0
    want8 = bf16_bits(run(cf, b8)[0])
    want16 = bf16_bits(run16(cf, b16)[0])
    for total in (b8.rows * b8.k, b8.rows * b8.k + 777):
        mixed, keep, end = run_total(cf, b8, total)
        torch.cuda.synchronize()
        # the whole-matrix form is deterministic: the bound changes the layout, not a bit of the result
        assert np.array_equal(bf16_bits(mixed), want8), total
        assert bool((keep[0][end:] == 0xA7).all())
    mixed, keep, end = run_total(cf, b16, b16.rows * b16.k + 300, form="bf16")
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(mixed), want16)
    assert bool((keep[0][end:] == 0xA7).all())
    # the calls under the reference's own argument lists do not use the bound at all (kernels/moe.cu:1070)
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    for total in (b8.rows * b8.k + 5, 0):
        mixed = dev_bf16(b8.mixed0, dev)
        cf.cf_moe_grouped_expert_forward_fp8(dev_arr(b8.hq, dev), sc(b8.d_h), 0, dev_arr(b8.rw, dev), dev_arr(b8.counts, dev), None,
                                             dev_arr(b8.idx, dev), dev_arr(b8.winq, dev), sc(b8.d_in), dev_arr(b8.woutq, dev), sc(b8.d_out),
                                             mixed, b8.rows, b8.H, b8.Ie, b8.E, total, stream())
        torch.cuda.synchronize()
        check_result(b8, mixed)


def test_counts_beyond_the_bound_are_cut_not_written(cf, dev):
    case("workspace forms with total_selected_rows BELOW the sum of the counts: rows beyond the bound are left out")
    b = Bank(dev, 600, 6, 2, 512, 256, False, seed=31)
    offs = orc.moe_expert_offsets(b.counts)
    total = int(offs[4]) + 37                      # expert 4 keeps 37 rows, expert 5 none
    assert total < b.total
    mixed, keep, end = run_total(cf, b, total, guard=1 << 20)
    torch.cuda.synchronize()
    assert bool((keep[0][end:] == 0xA7).all()), "a write went past the workspace the bound sized"
    # what is inside the bound is computed as ever: compare with a bank that holds exactly those pairs
    kept = Bank(dev, 600, 6, 2, 512, 256, False, seed=31)
    for e in range(b.E):
        n_keep = max(0, min(int(b.counts[e]), total - int(offs[e])))
        for s_ in range(n_keep, int(b.counts[e])):
            kept.rw[b.idx[e, s_], e] = 0.0
    kept.counts, kept.idx = orc.moe_build_expert_row_lists(kept.rw)
    kept.total = int(kept.counts.sum())
    assert kept.total == total
    check_result(kept, mixed)


def test_two_streams_two_workspaces(cf, dev):
    case("two banks in flight at once on two streams, each with its own workspace")
    a = Bank(dev, 700, 8, 2, 512, 384, False, seed=41)
    b = Bank(dev, 650, 6, 3, 768, 256, False, seed=42)
    want_a = bf16_bits(run(cf, a)[0])
    want_b = bf16_bits(run(cf, b)[0])
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    outs = []
    for rep in range(3):
        ma, keepa, _ = run_total(cf, a, a.rows * a.k, st=s1)
        mb, keepb, _ = run_total(cf, b, b.rows * b.k, st=s2)
        outs.append((ma, mb, keepa, keepb))
    torch.cuda.synchronize()
    for ma, mb, _, _ in outs:
        assert np.array_equal(bf16_bits(ma), want_a)
        assert np.array_equal(bf16_bits(mb), want_b)
