"""GPU parity of the grouped FP8 GEMM entry point that allocates nothing (cf_fp8_grouped_gemm_nt_bf16_static): its
tile table lives in a fixed array inside the library instead of a caller's workspace.  Two calls in a row, the second
on a smaller routing, each bit for bit against cf_fp8_grouped_gemm_nt_bf16_ex on the same inputs; then the size
limit."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import bf16_bits, case, stream
from test_gpu_moe_grouped import Bank, EPI_NONE, EPI_SILU, ROW_COL

pytestmark = pytest.mark.gpu


def both_forms(cf, b, epi):
    """The gate/up projection (SiLU-gate) or a plain projection of the bank's hidden rows through both entry points."""
    dev, E, H, Ie, total = b.dev, b.E, b.H, b.Ie, b.total
    cidx = torch.full((total,), -1, dtype=torch.int32, device=dev)
    cf.cf_moe_compact_row_index(b.d["counts"], b.d["offsets"], b.d["idx"], b.rows, E, cidx, stream())
    sz = ctypes.c_size_t(0)
    assert cf.raw_cf_fp8_grouped_gemm_workspace_bytes(total, E, ctypes.byref(sz)) == 0
    ws = torch.empty(sz.value, dtype=torch.uint8, device=dev)
    up, upd = (b.d["wu"], b.d["wud"]) if epi == EPI_SILU else (None, None)
    want = torch.full((total, Ie), float("nan"), dtype=torch.bfloat16, device=dev)
    got = torch.full((total, Ie), float("nan"), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_grouped_gemm_nt_bf16_ex(total, Ie, H, E, b.d["counts"], b.d["offsets"], b.d["hq"], b.rows, H, cidx, b.d["hd"],
                                      b.d["wg"], b.d["wgd"], ROW_COL, epi, up, upd, want, Ie, ws, sz.value, stream())
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    cf.cf_fp8_grouped_gemm_nt_bf16_static(total, Ie, H, E, b.d["counts"], b.d["offsets"], b.d["hq"], b.rows, H, cidx, b.d["hd"],
                                          b.d["wg"], b.d["wgd"], ROW_COL, epi, up, upd, got, Ie, stream())
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    return bf16_bits(got), bf16_bits(want), int(b.counts.sum())


def test_static_grouped_gemm_matches_workspace_form_twice(cf, dev):
    case("no-alloc grouped GEMM: 1500 rows x 6 experts, then 300 rows x 3 experts")
    big = Bank(dev, 1500, 6, 2, 512, 384, seed=71)
    small = Bank(dev, 300, 3, 1, 256, 256, seed=72, zero_expert=1)
    for bank, epi in ((big, EPI_SILU), (small, EPI_NONE), (big, EPI_NONE), (small, EPI_SILU)):
        got, want, filled = both_forms(cf, bank, epi)
        # rows past the experts' lists are written by neither form
        assert np.array_equal(got, want)
        g = got[:filled]
        assert not np.any((g & 0x7fff) > 0x7f80), "a routed row was left unwritten"
        assert np.all((got[filled:] & 0x7fff) > 0x7f80)


def test_static_grouped_gemm_size_limit(cf, dev):
    case("no-alloc grouped GEMM: size limit")
    mx = ctypes.c_size_t(0)
    assert cf.raw_cf_fp8_grouped_gemm_static_max_bytes(ctypes.byref(mx)) == 0 and mx.value == 64 * 1024
    b = Bank(dev, 40, 4, 1, 256, 256, seed=73)
    cidx = torch.zeros(b.total, dtype=torch.int32, device=dev)
    out = torch.full((b.total, b.Ie), 7.0, dtype=torch.bfloat16, device=dev)
    # a table for total_rows / 256 + num_experts = 3277 row tiles is one entry too large: rejected before any launch
    args = lambda total, E: (total, b.Ie, b.H, E, b.d["counts"].data_ptr(), b.d["offsets"].data_ptr(), b.d["hq"].data_ptr(), b.rows, b.H,
                             cidx.data_ptr(), b.d["hd"].data_ptr(), b.d["wg"].data_ptr(), b.d["wgd"].data_ptr(), ROW_COL, EPI_NONE, None, None,
                             out.data_ptr(), b.Ie, stream())
    need = ctypes.c_size_t(0)
    assert cf.raw_cf_fp8_grouped_gemm_workspace_bytes(256 * 3273, 4, ctypes.byref(need)) == 0 and need.value > mx.value
    assert cf.raw_cf_fp8_grouped_gemm_nt_bf16_static(*args(256 * 3273, 4)) == -2
    assert cf.raw_cf_fp8_grouped_gemm_workspace_bytes(256 * 3272, 4, ctypes.byref(need)) == 0 and need.value <= mx.value
    torch.cuda.synchronize()
    assert torch.all(out == 7.0)
    assert cf.raw_cf_fp8_grouped_gemm_nt_bf16_static(*args(-1, 4)) == -1
