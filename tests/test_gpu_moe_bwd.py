"""GPU parity: the custom kernels of the MoE expert-bank backward with forward-owned routes against the CPU
oracle.  Row dot, route-weighted gather and scatter-add: bit-exact.  GELU pair: within one bf16 ulp (the
device's erff / expf against libm's)."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_arr, dev_bf16, host, stream

pytestmark = pytest.mark.gpu


def bf(x):
    return orc.bf16_from_f32(np.asarray(x, np.float32))


def ulp_close(got_bits, want_bits, ulps=1, extra=0.0):
    """Within `ulps` bf16 ulps (+ `extra`, absolute), identical infinities, NaN where NaN is expected."""
    got, want = orc.bf16_to_f32(got_bits).astype(np.float64), orc.bf16_to_f32(want_bits).astype(np.float64)
    same = (np.isnan(got) & np.isnan(want)) | (got == want)
    with np.errstate(invalid="ignore"):
        near = np.abs(got - want) <= ulps * orc.bf16_ulp(want) + extra
    return np.all(same | near)


def test_gelu_forward_every_bf16_value(cf, dev):
    case("gelu forward, all 65536 bf16 values")
    bits = np.arange(1 << 16, dtype=np.uint16)
    out = torch.empty(1 << 16, dtype=torch.bfloat16, device=dev)
    cf.cf_gelu_forward_bf16(dev_bf16(bits, dev), out, bits.size, stream())
    torch.cuda.synchronize()
    got, want = bf16_bits(out), orc.gelu_forward(bits)
    # 1 + erf(x / sqrt 2) cancels for x < 0: one float32 ulp of erf (2^-24 near -1) is worth |x| 2^-25 of output,
    # and two erf implementations may differ by a couple of such ulps
    x = np.nan_to_num(np.abs(orc.bf16_to_f32(bits).astype(np.float64)), nan=0.0, posinf=0.0)
    assert ulp_close(got, want, extra=x * 2.0 ** -23)
    mild = orc.bf16_to_f32(bits) > -2.0
    assert np.mean(got[mild] != want[mild]) < 5e-3


@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
def test_gelu_backward(cf, dev, n):
    case(f"gelu backward n={n}")
    rng = np.random.default_rng(n)
    pre = bf(rng.standard_normal(n) * 2.5)
    g = bf(rng.standard_normal(n) * 1e-2)
    out = torch.empty(n, dtype=torch.bfloat16, device=dev)
    cf.cf_gelu_backward_bf16(dev_bf16(pre, dev), dev_bf16(g, dev), out, n, stream())
    torch.cuda.synchronize()
    got, want = bf16_bits(out), orc.gelu_backward(pre, g)
    assert ulp_close(got, want, extra=2.0 ** -23 * 0.05)
    assert np.mean(got != want) < 5e-3


def test_gelu_backward_every_pre_activation(cf, dev):
    case("gelu backward, all bf16 pre-activations, unit gradient")
    bits = np.arange(1 << 16, dtype=np.uint16)
    ones = bf(np.ones(1 << 16))
    out = torch.empty(1 << 16, dtype=torch.bfloat16, device=dev)
    cf.cf_gelu_backward_bf16(dev_bf16(bits, dev), dev_bf16(ones, dev), out, bits.size, stream())
    torch.cuda.synchronize()
    got, want = bf16_bits(out), orc.gelu_backward(bits, ones)
    fin = np.isfinite(orc.bf16_to_f32(bits))
    # the same cancellation in Phi(x) for x < 0: absolute 2^-23 on a derivative of order one
    assert ulp_close(got[fin], want[fin], extra=2.0 ** -23)


def test_gelu_unaligned_and_in_place(cf, dev):
    case("gelu on an unaligned view, backward in place over the gradient")
    rng = np.random.default_rng(2)
    n = 1001
    pre = bf(rng.standard_normal(n + 1))
    g = bf(rng.standard_normal(n + 1))
    dpre, dg = dev_bf16(pre, dev), dev_bf16(g, dev)
    cf.cf_gelu_backward_bf16(dpre[1:], dg[1:], dg[1:], n, stream())       # the reference calls it in place (src/trainer.cu:7730)
    torch.cuda.synchronize()
    got = bf16_bits(dg)
    assert got[0] == g[0] and ulp_close(got[1:], orc.gelu_backward(pre[1:], g[1:]), extra=2.0 ** -21)


@pytest.mark.parametrize("rows,n,H", [(300, 170, 2048), (64, 64, 256), (500, 333, 1024), (90, 41, 192), (90, 41, 1000), (33, 20, 64),
                                      (70, 70, 8)])
def test_row_dot_selected_per_expert_form(cf, dev, rows, n, H):
    case(f"row dot selected rows={rows} n={n} H={H}")
    rng = np.random.default_rng(rows + H)
    a = bf(rng.standard_normal((rows, H)))
    b = bf(rng.standard_normal((n, H)))
    ri = np.sort(rng.choice(rows, n, replace=False)).astype(np.int32)
    E, col = 5, 3
    out0 = rng.standard_normal((rows, E)).astype(np.float32)
    dout = dev_arr(out0, dev)
    cf.cf_moe_row_dot_selected_bf16(dev_bf16(a, dev), dev_bf16(b, dev), dout, dev_arr(ri, dev), n, H, E, col, stream())
    torch.cuda.synchronize()
    want = orc.moe_row_dot_selected(a, b, out0, ri, col)
    assert np.array_equal(host(dout).view(np.uint32), want.view(np.uint32))


def test_row_dot_order_sensitive_row(cf, dev):
    """The crafted row of the oracle's own test: only the reference's tree gives these two sums."""
    case("row dot order-sensitive row")
    H = 1024
    a = np.zeros((1, H), np.float32); b = np.zeros((1, H), np.float32)
    a[0, 0] = b[0, 0] = 4096.0
    for h in (256, 512, 1):
        a[0, h] = b[0, h] = 1.0
    out = torch.zeros(1, dtype=torch.float32, device=dev)
    ri = dev_arr(np.zeros(1, np.int32), dev)
    cf.cf_moe_row_dot_selected_bf16(dev_bf16(bf(a), dev), dev_bf16(bf(b), dev), out, ri, 1, H, 1, 0, stream())
    torch.cuda.synchronize()
    assert host(out)[0] == 16777216.0
    for h in (256, 512):
        a[0, h] = b[0, h] = 0.0
    a[0, 129] = b[0, 129] = 1.0
    cf.cf_moe_row_dot_selected_bf16(dev_bf16(bf(a), dev), dev_bf16(bf(b), dev), out, ri, 1, H, 1, 0, stream())
    torch.cuda.synchronize()
    assert host(out)[0] == 16777218.0


@pytest.mark.parametrize("rows,n,H", [(300, 170, 2048), (90, 41, 1000), (64, 64, 256), (50, 9, 24)])
def test_gather_scale_and_scatter_add_per_expert_form(cf, dev, rows, n, H):
    case(f"gather-scale / scatter-add rows={rows} n={n} H={H}")
    rng = np.random.default_rng(rows * 3 + H)
    E, e = 6, 2
    src = bf(rng.standard_normal((rows, H)))
    rw = rng.uniform(0.05, 0.9, (rows, E)).astype(np.float32)
    ri = np.sort(rng.choice(rows, n, replace=False)).astype(np.int32)
    dst = torch.zeros((n, H), dtype=torch.bfloat16, device=dev)
    cf.cf_moe_gather_scale_rows_bf16(dev_bf16(src, dev), dst, dev_arr(rw, dev), dev_arr(ri, dev), n, e, E, H, stream())
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(dst), orc.moe_gather_scale_rows(src, rw, ri, e))

    full = bf(rng.standard_normal((rows, H)))
    comp = bf(rng.standard_normal((n, H)))
    dfull = dev_bf16(full, dev)
    cf.cf_moe_scatter_add_rows_bf16(dfull, dev_bf16(comp, dev), dev_arr(ri, dev), n, H, stream())
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(dfull), orc.moe_scatter_add_rows(full, comp, ri))


class Routes:
    def __init__(self, dev, rows, E, k, H, seed, zero_expert=None):
        rng = np.random.default_rng(seed)
        logits = rng.standard_normal((rows, E)).astype(np.float32)
        if zero_expert is not None:
            logits[:, zero_expert] = -50.0
        self.rw = orc.moe_topk_route(logits, k)
        self.counts, self.idx = orc.moe_build_expert_row_lists(self.rw)
        self.offsets = orc.moe_expert_offsets(self.counts)
        self.total = int(self.counts.sum())
        self.rows, self.E, self.H = rows, E, H
        self.d_mixed = bf(rng.standard_normal((rows, H)))
        self.expert_out = bf(rng.standard_normal((self.total, H)))
        self.d = {n: dev_arr(getattr(self, n), dev) for n in ("rw", "counts", "offsets", "idx")}


@pytest.mark.parametrize("rows,E,k,H,zero", [(600, 5, 2, 256, None), (300, 4, 2, 1024, 2), (1000, 16, 3, 2048, None), (200, 6, 2, 1000, None),
                                             (64, 3, 3, 192, None)])
def test_grouped_route_grad_equals_the_per_expert_launches(cf, dev, rows, E, k, H, zero):
    case(f"grouped route grad rows={rows} E={E} k={k} H={H}")
    r = Routes(dev, rows, E, k, H, seed=rows + E + H, zero_expert=zero)
    eo = dev_bf16(r.expert_out, dev)
    dlog = torch.full((rows, E), 3.5, dtype=torch.float32, device=dev)
    cf.cf_moe_grouped_route_grad_bf16(dev_bf16(r.d_mixed, dev), eo, dlog, r.d["rw"], r.d["counts"], r.d["offsets"], r.d["idx"],
                                      rows, E, H, stream())
    torch.cuda.synchronize()
    want_log = np.zeros((rows, E), np.float32)
    want_out = np.empty_like(r.expert_out)
    for e in range(E):
        n, o = int(r.counts[e]), int(r.offsets[e])
        ri = r.idx[e, :n]
        want_log = orc.moe_row_dot_selected(r.d_mixed, r.expert_out[o:o + n], want_log, ri, e)
        want_out[o:o + n] = orc.moe_gather_scale_rows(r.d_mixed, r.rw, ri, e)
    assert np.array_equal(host(dlog).view(np.uint32), want_log.view(np.uint32))
    assert np.array_equal(bf16_bits(eo), want_out)


@pytest.mark.parametrize("rows,E,k,H", [(600, 5, 2, 256), (300, 70, 4, 1000), (1000, 16, 3, 2048)])
def test_grouped_scatter_add_equals_the_per_expert_launches(cf, dev, rows, E, k, H):
    case(f"grouped scatter-add rows={rows} E={E} k={k} H={H}")
    r = Routes(dev, rows, E, k, H, seed=rows + E)
    full = bf(np.random.default_rng(1).standard_normal((rows, H)))
    dfull = dev_bf16(full, dev)
    cf.cf_moe_unpermute_add_bf16(dfull, dev_bf16(r.expert_out, dev), r.d["rw"], r.d["counts"], r.d["offsets"], r.d["idx"],
                                 rows, E, H, stream())
    torch.cuda.synchronize()
    want = full
    for e in range(E):
        n, o = int(r.counts[e]), int(r.offsets[e])
        want = orc.moe_scatter_add_rows(want, r.expert_out[o:o + n], r.idx[e, :n])
    assert np.array_equal(bf16_bits(dfull), want)


@pytest.mark.parametrize("rows,E,k,H", [(600, 5, 2, 256), (300, 70, 4, 1000), (1000, 16, 3, 2048), (16384, 64, 6, 2048)])
@pytest.mark.parametrize("unit", [0, 1])
def test_indexed_unpermute_equals_the_searching_one(cf, dev, rows, E, k, H, unit):
    """The slot table is the search's answer computed once: both forms must agree bit for bit, weighted
    (forward) and with unit factors (backward scatter-add)."""
    case(f"indexed unpermute rows={rows} E={E} k={k} H={H} unit={unit}")
    r = Routes(dev, rows, E, k, H, seed=rows + E + unit)
    full = bf(np.random.default_rng(2).standard_normal((rows, H)))
    y = dev_bf16(r.expert_out, dev)
    a, b = dev_bf16(full, dev), dev_bf16(full, dev)
    slot = torch.full((rows, E), -12345, dtype=torch.int32, device=dev)
    cf.cf_moe_build_slot_index(r.d["counts"], r.d["offsets"], r.d["idx"], rows, E, slot, stream())
    cf.cf_moe_unpermute_indexed_bf16(a, y, r.d["rw"], slot, rows, E, H, unit, stream())
    if unit:
        cf.cf_moe_unpermute_add_bf16(b, y, r.d["rw"], r.d["counts"], r.d["offsets"], r.d["idx"], rows, E, H, stream())
    else:
        cf.cf_moe_unpermute_weighted_bf16(b, y, r.d["rw"], r.d["counts"], r.d["offsets"], r.d["idx"], rows, E, H, stream())
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(a), bf16_bits(b))
    # the table itself: listed pairs hold their slot, every other cell is untouched
    hs = host(slot)
    want = np.full((rows, E), -12345, np.int32)
    for e in range(E):
        n = int(r.counts[e])
        want[r.idx[e, :n], e] = r.offsets[e] + np.arange(n)
    assert np.array_equal(hs, want)
    if rows <= 1000:
        ref = full
        for e in range(E):
            n, o = int(r.counts[e]), int(r.offsets[e])
            ref = (orc.moe_scatter_add_rows(ref, r.expert_out[o:o + n], r.idx[e, :n]) if unit else
                   orc.moe_scatter_accumulate(ref, r.expert_out[o:o + n], r.rw, r.idx[e, :n], e))
        assert np.array_equal(bf16_bits(a), ref)


def test_route_grad_config5_size(cf, dev):
    """16384 tokens, hidden 2048, 64 experts, top-6: the full-size launch against the oracle on three experts
    and through the identity sum_e w[row, e] * d_w[row, e] = dot(d_mixed[row], sum_e w expert_out) per row."""
    case("grouped route grad, config 5 size")
    r = Routes(dev, 16384, 64, 6, 2048, seed=5)
    assert r.total == 98304
    eo = dev_bf16(r.expert_out, dev)
    dlog = torch.empty((r.rows, r.E), dtype=torch.float32, device=dev)
    cf.cf_moe_grouped_route_grad_bf16(dev_bf16(r.d_mixed, dev), eo, dlog, r.d["rw"], r.d["counts"], r.d["offsets"], r.d["idx"],
                                      r.rows, r.E, r.H, stream())
    torch.cuda.synchronize()
    got_log, got_out = host(dlog), bf16_bits(eo)
    assert np.all(got_log[r.rw == 0.0] == 0.0) and np.count_nonzero(got_log) > 0.99 * r.total
    for e in (0, 31, 63):
        n, o = int(r.counts[e]), int(r.offsets[e])
        ri = r.idx[e, :n]
        want = orc.moe_row_dot_selected(r.d_mixed, r.expert_out[o:o + n], np.zeros((r.rows, r.E), np.float32), ri, e)
        assert np.array_equal(got_log[ri, e].view(np.uint32), want[ri, e].view(np.uint32))
        assert np.array_equal(got_out[o:o + n], orc.moe_gather_scale_rows(r.d_mixed, r.rw, ri, e))
    # every slot was rewritten with a multiple of its token's gradient row: slot / row ratio is the route weight
    e = 17
    n, o = int(r.counts[e]), int(r.offsets[e])
    ri = r.idx[e, :n]
    ratio = orc.bf16_to_f32(got_out[o:o + n]).astype(np.float64) / orc.bf16_to_f32(r.d_mixed[ri]).astype(np.float64)
    assert np.all(np.abs(ratio / r.rw[ri, e][:, None] - 1.0) <= 2.0 ** -8)


def test_argument_errors(cf, dev):
    import ctypes
    z = torch.zeros(16, dtype=torch.bfloat16, device=dev)
    zi = torch.zeros(4, dtype=torch.int32, device=dev)
    zf = torch.zeros(16, dtype=torch.float32, device=dev)
    assert cf.raw_cf_moe_row_dot_selected_bf16(z.data_ptr(), z.data_ptr(), zf.data_ptr(), zi.data_ptr(), -1, 8, 1, 0, None) != 0
    assert cf.raw_cf_moe_gather_scale_rows_bf16(z.data_ptr(), z.data_ptr(), zf.data_ptr(), zi.data_ptr(), 1, 3, 2, 8, None) != 0
    assert cf.raw_cf_gelu_forward_bf16(None, z.data_ptr(), 4, None) != 0
    assert cf.raw_cf_gelu_forward_bf16(None, None, 0, None) == 0


def test_gelu_forward_table_form_matches_the_plain_kernel(cf, dev):
    """Tensors of 64 Mi elements and more take the form that looks results up in a per-workgroup table; it must give
    the bits of the plain kernel (run here on the same data in pieces below that size), an unaligned tail included."""
    case("gelu forward, table form")
    n = (64 << 20) + 8 * 1000 + 3
    g = torch.Generator(device=dev); g.manual_seed(4)
    x = (torch.randn(n, device=dev, generator=g) * 3.0).to(torch.bfloat16)
    x[:65536] = torch.arange(65536, device=dev, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)   # every bf16 value
    out = torch.empty_like(x)
    cf.cf_gelu_forward_bf16(x, out, n, stream())
    want = torch.empty_like(x)
    piece = 16 << 20
    for a in range(0, n, piece):
        m = min(piece, n - a)
        cf.cf_gelu_forward_bf16(x[a:a + m], want[a:a + m], m, stream())
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


def test_gelu_backward_table_form_matches_the_plain_kernel(cf, dev):
    """Tensors of 1 Mi elements and more take the form that looks the derivative up in a per-workgroup table; it must
    give the bits of the plain kernel (run here on the same data in pieces below that size), every bf16 pre-activation
    and an unaligned tail included."""
    case("gelu backward, table form")
    n = (2 << 20) + 8 * 100 + 5
    g = torch.Generator(device=dev); g.manual_seed(6)
    pre = (torch.randn(n, device=dev, generator=g) * 3.0).to(torch.bfloat16)
    pre[:65536] = torch.arange(65536, device=dev, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    grad = (torch.randn(n, device=dev, generator=g) * 1e-2).to(torch.bfloat16)
    out = torch.empty_like(pre)
    cf.cf_gelu_backward_bf16(pre, grad, out, n, stream())
    want = torch.empty_like(pre)
    piece = 1 << 19
    for a in range(0, n, piece):
        m = min(piece, n - a)
        cf.cf_gelu_backward_bf16(pre[a:a + m], grad[a:a + m], want[a:a + m], m, stream())
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
