"""GPU parity: MoE routing / dispatch against the CPU oracle.  Route weights, selected expert sets,
counts, row lists, offsets, gathers and the weighted unpermute are all bit-exact."""
import json
from pathlib import Path

import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_arr, dev_bf16, host, stream

pytestmark = pytest.mark.gpu
GOLD = Path(__file__).resolve().parent / "golden"


def test_device_expf_is_bit_identical_to_the_oracle(cf, dev):
    # softmax of [x, 0] at x <= 0 exposes expf(x): p0 = e/(e+1) in a fixed order; compare whole softmax rows instead
    case("softmax vs oracle, dense sweep")
    x = np.concatenate([np.linspace(-104, 0, 400001), -np.exp(np.linspace(-20, 4.6, 100000))]).astype(np.float32)
    rows = np.stack([x, np.zeros_like(x)], axis=1)
    d = torch.from_numpy(rows.copy()).to(dev)
    cf.cf_softmax_inplace_f32(d, rows.shape[0], 2, stream())
    torch.cuda.synchronize()
    assert np.array_equal(host(d).view(np.uint32), orc.softmax(rows).view(np.uint32))


@pytest.mark.parametrize("rows,cols", [(1, 1), (5, 3), (33, 32), (100, 33), (1000, 64), (7, 65), (50, 100), (9, 256), (6, 300), (4, 1000)])
def test_softmax(cf, dev, rows, cols):
    case(f"softmax {rows}x{cols}")
    rng = np.random.default_rng(rows * 1000 + cols)
    x = (rng.standard_normal((rows, cols)) * 4).astype(np.float32)
    d = torch.from_numpy(x.copy()).to(dev)
    cf.cf_softmax_inplace_f32(d, rows, cols, stream())
    torch.cuda.synchronize()
    assert np.array_equal(host(d).view(np.uint32), orc.softmax(x).view(np.uint32))


def route_gpu(cf, dev, logits, k, normalize=True, saves=False):
    rows, E = logits.shape
    d = torch.from_numpy(logits.copy()).to(dev)
    rs = torch.empty(rows, device=dev) if saves else None
    sv = torch.empty((rows, E), device=dev) if saves else None
    cf.cf_moe_topk_route_f32(d, rows, E, k, stream(), rs, sv, int(normalize))
    torch.cuda.synchronize()
    return (host(d), host(rs), host(sv)) if saves else host(d)


def test_topk_reference_fixture(cf, dev):
    case("top-k fixture")
    g = json.loads((GOLD / "moe_router_parity.json").read_text())
    c = g["cases"]["unpacked_case"]
    got = route_gpu(cf, dev, np.array(c["logits"], np.float32), g["top_k"])
    want = np.array(c["route_weights_pre_inhibition"], np.float32)
    assert np.array_equal(got > 0, want > 0) and np.max(np.abs(got - want)) <= 2e-7


@pytest.mark.parametrize("E,k", [(3, 2), (8, 2), (64, 6), (64, 64), (5, 9), (40, 1), (65, 4), (128, 8), (300, 3), (1000, 100), (2048, 7)])
@pytest.mark.parametrize("normalize", [True, False])
def test_topk_route_bit_exact(cf, dev, E, k, normalize):
    case(f"top-k E={E} k={k} normalize={normalize}")
    rng = np.random.default_rng(E * 100 + k)
    rows = 777
    logits = rng.standard_normal((rows, E)).astype(np.float32)
    logits[::7, : max(E // 2, 1)] = 0.25                           # exact ties: the lowest index must win
    logits[5] = 0.0
    got, rs, sv = route_gpu(cf, dev, logits, k, normalize, saves=True)
    want, wrs, wsv = orc.moe_topk_route(logits, k, normalize, want_saves=True)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(rs.view(np.uint32), wrs.view(np.uint32)) and np.array_equal(sv.view(np.uint32), wsv.view(np.uint32))
    assert np.all((got > 0).sum(1) == min(k, E))


def test_config5_routing_and_dispatch_full_size(cf, dev):
    """16384 tokens, 64 experts, top-6: route weights, counts, row lists, offsets bit-exact."""
    case("config 5 routing")
    rows, E, k, H = 16384, 64, 6, 2048
    rng = np.random.default_rng(55)
    logits = rng.standard_normal((rows, E)).astype(np.float32)
    rw_d = torch.from_numpy(logits.copy()).to(dev)
    cf.cf_moe_topk_route_f32(rw_d, rows, E, k, stream(), None, None, 1)
    counts_d = torch.full((E,), -7, dtype=torch.int32, device=dev)
    idx_d = torch.full((E, rows), -1, dtype=torch.int32, device=dev)
    off_d = torch.empty(E, dtype=torch.int32, device=dev)
    cf.cf_moe_build_expert_row_lists(rw_d, counts_d, idx_d, rows, E, stream())
    cf.cf_moe_expert_offsets_from_counts(counts_d, off_d, E, stream())
    torch.cuda.synchronize()
    rw = orc.moe_topk_route(logits, k)
    counts, idx = orc.moe_build_expert_row_lists(rw)
    assert np.array_equal(host(rw_d).view(np.uint32), rw.view(np.uint32))
    assert np.array_equal(host(counts_d), counts) and counts.sum() == rows * k
    assert np.array_equal(host(idx_d), idx)                         # ascending rows, tails untouched
    assert np.array_equal(host(off_d), orc.moe_expert_offsets(counts))
    # token permute of fp8 rows and the weighted unpermute, one expert at a time
    hidden = rng.integers(0, 256, (rows, H)).astype(np.uint8)
    hid_d = dev_arr(hidden, dev)
    mixed = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))
    mixed_d = dev_bf16(mixed, dev)
    for e in (0, 17, 63):
        n = int(counts[e])
        comp_d = torch.empty((n, H), dtype=torch.uint8, device=dev)
        cf.cf_moe_gather_rows_u8(hid_d, comp_d, idx_d[e], n, H, stream())
        torch.cuda.synchronize()
        assert np.array_equal(host(comp_d), hidden[idx[e, :n]])
        out = orc.bf16_from_f32(rng.standard_normal((n, H)).astype(np.float32))
        cf.cf_moe_scatter_accumulate_rows_bf16(mixed_d, dev_bf16(out, dev), rw_d, idx_d[e], n, e, E, H, stream())
        torch.cuda.synchronize()
        mixed = orc.moe_scatter_accumulate(mixed, out, rw, idx[e, :n], e)
        assert np.array_equal(bf16_bits(mixed_d), mixed)


@pytest.mark.parametrize("rows,E,H", [(1, 1, 1), (301, 16, 24), (1030, 7, 40), (64, 3, 5), (40000, 5, 8), (16385, 2, 8)])
def test_dispatch_small_and_ragged(cf, dev, rows, E, H):
    case(f"dispatch rows={rows} E={E} H={H}")
    rng = np.random.default_rng(rows + E)
    rw = orc.moe_topk_route(rng.standard_normal((rows, E)).astype(np.float32), min(2, E))
    rw[rows // 2] = 0.0                                                # a row routed nowhere
    rw_d = torch.from_numpy(rw.copy()).to(dev)
    counts_d = torch.empty(E, dtype=torch.int32, device=dev)
    idx_d = torch.full((E, rows), -1, dtype=torch.int32, device=dev)
    cf.cf_moe_build_expert_row_lists(rw_d, counts_d, idx_d, rows, E, stream())
    torch.cuda.synchronize()
    counts, idx = orc.moe_build_expert_row_lists(rw)
    assert np.array_equal(host(counts_d), counts) and np.array_equal(host(idx_d), idx)
    e = int(np.argmax(counts))
    n = int(counts[e])
    src16 = rng.integers(0, 65536, (rows, H)).astype(np.uint16)
    dst = torch.empty((n, H), dtype=torch.bfloat16, device=dev)
    cf.cf_moe_gather_rows_bf16(dev_bf16(src16, dev), dst, idx_d[e], n, H, stream())
    src8 = rng.integers(0, 256, (rows, H)).astype(np.uint8)
    dst8 = torch.empty((n, H), dtype=torch.uint8, device=dev)
    cf.cf_moe_gather_rows_u8(dev_arr(src8, dev), dst8, idx_d[e], n, H, stream())
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(dst), src16[idx[e, :n]]) and np.array_equal(host(dst8), src8[idx[e, :n]])
    mixed = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))
    term = orc.bf16_from_f32(rng.standard_normal((rows, H)).astype(np.float32))
    md = dev_bf16(mixed, dev)
    cf.cf_moe_scale_accumulate_bf16(md, dev_bf16(term, dev), rw_d, rows, e, E, H, stream())
    comp = orc.bf16_from_f32(rng.standard_normal((n, H)).astype(np.float32))
    cf.cf_moe_scatter_accumulate_rows_bf16(md, dev_bf16(comp, dev), rw_d, idx_d[e], n, e, E, H, stream())
    torch.cuda.synchronize()
    want = orc.moe_scatter_accumulate(orc.moe_scale_accumulate(mixed, term, rw, e), comp, rw, idx[e, :n], e)
    assert np.array_equal(bf16_bits(md), want)
