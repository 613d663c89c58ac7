"""GPU parity: the selected-expert backward of the GELU expert bank in one call
(cf_moe_grouped_gelu_backward_fp8; the reference's per-expert host loop is src/trainer.cu:7669-7741).

Every stage is checked on the intermediates the call leaves in its workspace, given that stage's own (GPU) inputs, the
way the reference's loop would produce them expert by expert: index, quantized bytes and scales, the route-weight
gradient's row dots, the scaled gather and the scatter-add bit for bit against the oracle; the GELU pair within one
bf16 ulp (device erff against libm's); the FP8 and bf16 GEMM stages at their bars against the double reference."""
import ctypes

import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_arr, dev_bf16, host, stream
from test_gpu_gemm_bf16 import absdot, check_bf16_out
from test_gpu_moe_bwd import ulp_close

pytestmark = pytest.mark.gpu

NAMES = ["TILE_MAP", "INDEX", "HIDDEN_DESCALE", "IN_DESCALE", "OUT_DESCALE", "PRE", "POST", "POSTQ", "POST_SCALE", "POST_DESCALE",
         "D_OUT", "D_POST", "D_PRE", "X", "D_X"]


def per_tensor_e4m3(x):
    """float32 -> (E4M3 bytes, descale) with one scale for the tensor (kernels/fp8.cu:34-49)."""
    scale, descale = orc.scale_from_amax(orc.amax_f32(x), 448.0)
    return orc.quantize_f32_e4m3(x, scale), np.float32(descale)


class BwdBank:
    def __init__(self, dev, rows, E, k, H, Ie, seed, zero_expert=None):
        rng = np.random.default_rng(seed)
        self.rows, self.E, self.k, self.H, self.Ie, self.dev = rows, E, k, H, Ie, dev
        logits = rng.standard_normal((rows, E)).astype(np.float32)
        if zero_expert is not None:
            logits[:, zero_expert] = -50.0
        self.rw = orc.moe_topk_route(logits, k)
        self.counts, self.idx = orc.moe_build_expert_row_lists(self.rw)
        self.offsets = orc.moe_expert_offsets(self.counts)
        self.total = int(self.counts.sum())
        hidden = rng.standard_normal((rows, H)).astype(np.float32)
        self.hidden_bf16 = orc.bf16_from_f32(hidden)
        self.hq, self.hd = per_tensor_e4m3(orc.bf16_to_f32(self.hidden_bf16))
        w_in = (0.05 * rng.standard_normal((E, Ie, H))).astype(np.float32)
        w_out = (0.05 * rng.standard_normal((E, H, Ie))).astype(np.float32)
        self.w_in, self.w_out = orc.bf16_from_f32(w_in), orc.bf16_from_f32(w_out)
        self.w_in8, self.w_in_d = per_tensor_e4m3(orc.bf16_to_f32(self.w_in))
        self.w_out8, self.w_out_d = per_tensor_e4m3(orc.bf16_to_f32(self.w_out))
        self.d_mixed = orc.bf16_from_f32((rng.standard_normal((rows, H)) * 1e-2).astype(np.float32))
        self.g_in0 = orc.bf16_from_f32((rng.standard_normal((E, Ie, H)) * 1e-3).astype(np.float32))
        self.g_out0 = orc.bf16_from_f32((rng.standard_normal((E, H, Ie)) * 1e-3).astype(np.float32))
        self.d_hidden0 = orc.bf16_from_f32((rng.standard_normal((rows, H)) * 1e-2).astype(np.float32))

    def compact_index(self):
        return np.concatenate([self.idx[e, : self.counts[e]] for e in range(self.E)]) if self.total else np.zeros(0, np.int32)


def run_backward(cf, b, bound=None, slots=None, guard=0):
    """bound: what the caller passes as total_selected_rows (an upper bound on the sum of the counts; default the sum);
    slots: (state tensor, stride words, history_len, is_e5m2) of the per-expert activation slots;
    guard: bytes behind the workspace that must come back untouched."""
    dev = b.dev
    bound = b.total if bound is None else bound
    offs = (ctypes.c_size_t * len(NAMES))()
    size = ctypes.c_size_t(0)
    assert cf.raw_cf_moe_grouped_gelu_backward_workspace(b.rows, bound, b.E, b.H, b.Ie, offs, ctypes.byref(size)) == 0
    ws = torch.zeros(size.value + 256 + guard, dtype=torch.uint8, device=dev)
    shift = (-ws.data_ptr()) % 256
    ws[shift + size.value:].fill_(0xA7)
    f32 = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    d_rw = torch.full((b.rows, b.E), float("nan"), device=dev)
    g_in, g_out, d_hidden = dev_bf16(b.g_in0, dev), dev_bf16(b.g_out0, dev), dev_bf16(b.d_hidden0, dev)
    args = (dev_bf16(b.d_mixed, dev), dev_arr(b.hq, dev), f32(b.hd), 0, dev_bf16(b.hidden_bf16, dev), dev_arr(b.rw, dev),
            dev_arr(b.counts, dev), dev_arr(b.offsets, dev), dev_arr(b.idx, dev),
            dev_arr(b.w_in8, dev), f32(b.w_in_d), dev_arr(b.w_out8, dev), f32(b.w_out_d), dev_bf16(b.w_in, dev), dev_bf16(b.w_out, dev),
            d_rw, g_in, g_out, d_hidden, b.rows, b.H, b.Ie, b.E, bound)
    if slots is None:
        cf.cf_moe_grouped_gelu_backward_fp8(*args, ws.data_ptr() + shift, size.value, stream())
    else:
        cf.cf_moe_grouped_gelu_backward_fp8_slots(*args, slots[0], slots[1], slots[2], int(slots[3]), ws.data_ptr() + shift, size.value,
                                                  stream())
    torch.cuda.synchronize()
    assert bool((ws[shift + size.value:] == 0xA7).all()), "a write went past the workspace"
    raw = ws[shift:]
    t, H, Ie = min(b.total, bound), b.H, b.Ie

    def grab(name, dtype, shape):
        o = offs[NAMES.index(name)]
        n = int(np.prod(shape)) * np.dtype(dtype).itemsize
        return raw[o:o + n].cpu().numpy().view(dtype).reshape(shape)

    r = dict(index=grab("INDEX", np.int32, (t,)), pre=grab("PRE", np.uint16, (t, Ie)), post=grab("POST", np.uint16, (t, Ie)),
             postq=grab("POSTQ", np.uint8, (t, Ie)), post_scale=grab("POST_SCALE", np.float32, (t,)),
             post_descale=grab("POST_DESCALE", np.float32, (t,)), d_out=grab("D_OUT", np.uint16, (t, H)),
             d_post=grab("D_POST", np.uint16, (t, Ie)), d_pre=grab("D_PRE", np.uint16, (t, Ie)), x=grab("X", np.uint16, (t, H)),
             d_x=grab("D_X", np.uint16, (t, H)), d_rw=host(d_rw), g_in=bf16_bits(g_in), g_out=bf16_bits(g_out),
             d_hidden=bf16_bits(d_hidden))
    # the expert outputs before the route gradient overwrote them: the same grouped FP8 GEMM on the same operands
    sz = ctypes.c_size_t(0)
    cf.raw_cf_fp8_grouped_gemm_workspace_bytes(t, b.E, ctypes.byref(sz))
    ws2 = torch.empty(max(sz.value, 4), dtype=torch.uint8, device=dev)
    out = torch.zeros((max(t, 1), H), dtype=torch.bfloat16, device=dev)
    if t:
        cf.cf_fp8_grouped_gemm_nt_bf16_ex(t, H, Ie, b.E, dev_arr(b.counts, dev), dev_arr(b.offsets, dev), dev_arr(r["postq"], dev), t, Ie,
                                          None, dev_arr(r["post_descale"], dev), dev_arr(b.w_out8, dev),
                                          torch.full((b.E * H,), float(b.w_out_d), device=dev), 1, 0, None, None, out, H, ws2, sz.value,
                                          stream())
        torch.cuda.synchronize()
    r["out"] = bf16_bits(out)[:t]
    return r


def check_backward(b, r, gemm_experts=None, gemm_rows=None, gelu_stride=1, slot_oracles=None):
    """gemm_experts / gemm_rows: the experts whose GEMM stages are compared with the double reference and how many of
    their rows (None: all); gelu_stride: every n-th row of the GELU pair is compared; slot_oracles: the per-expert slot
    state machines whose recompute call gives the activation bytes (None: one scale per token row)."""
    E, H, Ie = b.E, b.H, b.Ie
    cidx = b.compact_index()
    assert np.array_equal(r["index"], cidx)
    assert np.array_equal(r["x"], b.hidden_bf16[cidx])                                             # moe_gather_rows_bf16
    # recompute: gelu_forward within an ulp of the oracle; the quantize of the GPU's own activations bit for bit
    gs = slice(None, None, gelu_stride)
    assert ulp_close(r["post"][gs], orc.gelu_forward(r["pre"][gs]), extra=np.abs(orc.bf16_to_f32(r["pre"][gs]).astype(np.float64)) * 2.0 ** -23)
    if slot_oracles is None:
        q, s, d = orc.quantize_rows(r["post"])
        assert np.array_equal(r["postq"], q) and np.array_equal(r["post_scale"], s) and np.array_equal(r["post_descale"], d)
    else:
        # fp8_quant_act(slot_e, ..., is_recompute = true), src/trainer.cu:7707-7712: the forward call's snapshot scale
        for e in range(E):
            n, o = int(b.counts[e]), int(b.offsets[e])
            if n == 0:
                continue
            want = slot_oracles[e].quant_act(r["post"][o:o + n].reshape(-1), is_recompute=True)
            assert np.array_equal(r["postq"][o:o + n].reshape(-1), want), f"expert {e}"
            assert np.all(r["post_descale"][o:o + n] == slot_oracles[e].descale_snapshot), f"expert {e}"
    assert ulp_close(r["d_pre"][gs], orc.gelu_backward(r["pre"][gs], r["d_post"][gs]), extra=2.0 ** -23 * 0.05)
    # route-weight gradient and the scaled gather, expert by expert as the loop runs them; then the scatter-add
    d_rw = np.zeros((b.rows, E), np.float32)
    d_hidden = b.d_hidden0
    for e in range(E):
        n, o = int(b.counts[e]), int(b.offsets[e])
        if n == 0:
            assert np.array_equal(r["g_in"][e], b.g_in0[e]) and np.array_equal(r["g_out"][e], b.g_out0[e])
            continue
        rows = b.idx[e, :n]
        d_rw = orc.moe_row_dot_selected(b.d_mixed, r["out"][o:o + n], d_rw, rows, e)
        assert np.array_equal(r["d_out"][o:o + n], orc.moe_gather_scale_rows(b.d_mixed, b.rw, rows, e))
        d_hidden = orc.moe_scatter_add_rows(d_hidden, r["d_x"][o:o + n], rows)
        if gemm_experts is not None and e not in gemm_experts:
            continue
        sel = np.arange(n) if gemm_rows is None or n <= gemm_rows else np.sort(np.random.default_rng(e).choice(n, gemm_rows, replace=False))
        # FP8 recompute GEMMs against the double reference (per-tensor descales)
        ref, ad = orc.gemm_nt_ref(b.hq[rows[sel]], b.w_in8[e], [b.hd], [b.w_in_d])
        orc.assert_gemm_close(orc.bf16_to_f32(r["pre"][o:o + n][sel]).astype(np.float64), ref, ad, what=f"pre expert {e}")
        ref, ad = orc.gemm_nt_ref(r["postq"][o:o + n][sel], b.w_out8[e], r["post_descale"][o:o + n][sel], np.full(H, b.w_out_d, np.float32),
                                  scale_mode=1)
        orc.assert_gemm_close(orc.bf16_to_f32(r["out"][o:o + n][sel]).astype(np.float64), ref, ad, what=f"out expert {e}")
        # the four bf16 GEMMs on the GPU's own operands: the weight gradients contract over all of the expert's rows
        dO, post, dpre, x = r["d_out"][o:o + n], r["post"][o:o + n], r["d_pre"][o:o + n], r["x"][o:o + n]
        check_bf16_out(r["g_out"][e], orc.bf16_to_f32(b.g_out0[e]).astype(np.float64) + orc.gemm_bf16_tn_ref(dO, post),
                       absdot(dO, post, tn=True), f"g_out expert {e}")
        check_bf16_out(r["d_post"][o:o + n][sel], orc.gemm_bf16_nn_ref(dO[sel], b.w_out[e]), absdot(dO[sel], b.w_out[e]), f"d_post expert {e}")
        check_bf16_out(r["g_in"][e], orc.bf16_to_f32(b.g_in0[e]).astype(np.float64) + orc.gemm_bf16_tn_ref(dpre, x),
                       absdot(dpre, x, tn=True), f"g_in expert {e}")
        check_bf16_out(r["d_x"][o:o + n][sel], orc.gemm_bf16_nn_ref(dpre[sel], b.w_in[e]), absdot(dpre[sel], b.w_in[e]), f"d_x expert {e}")
    assert np.array_equal(r["d_rw"], d_rw)
    assert np.array_equal(r["d_hidden"], d_hidden)


@pytest.mark.parametrize("rows,E,k,H,Ie,zero", [(600, 5, 2, 256, 384, None), (300, 4, 2, 256, 256, 2), (1100, 3, 1, 512, 640, None)])
def test_grouped_gelu_backward_stage_by_stage(cf, dev, rows, E, k, H, Ie, zero):
    case(f"grouped GELU backward rows={rows} E={E} k={k} H={H} Ie={Ie} zero={zero}")
    b = BwdBank(dev, rows, E, k, H, Ie, seed=rows + E, zero_expert=zero)
    check_backward(b, run_backward(cf, b))


def test_grouped_gelu_backward_total_is_an_upper_bound(cf, dev):
    case("grouped GELU backward with total_selected_rows = rows * top_k + slack above the sum of the counts")
    b = BwdBank(dev, 500, 5, 2, 256, 384, seed=77, zero_expert=3)
    b.rw[::5, :] = 0.0                                   # every fifth row selects one expert only
    b.rw[::5, 0] = 1.0
    b.counts, b.idx = orc.moe_build_expert_row_lists(b.rw)
    b.offsets = orc.moe_expert_offsets(b.counts)
    b.total = int(b.counts.sum())
    assert b.total < b.rows * b.k
    check_backward(b, run_backward(cf, b, bound=b.rows * b.k + 333, guard=1 << 16))


def test_grouped_gelu_backward_counts_beyond_the_bound(cf, dev):
    case("grouped GELU backward with total_selected_rows below the sum of the counts: nothing is written past the workspace")
    b = BwdBank(dev, 400, 4, 2, 256, 256, seed=78)
    bound = int(b.offsets[2]) + 21                       # expert 2 keeps 21 rows, expert 3 none
    r = run_backward(cf, b, bound=bound, guard=1 << 20)  # run_backward asserts that the guard bytes survive
    # the pairs inside the bound are computed as ever
    assert np.array_equal(r["index"], b.compact_index()[:bound])
    n0 = int(b.counts[0])
    assert np.array_equal(r["d_out"][:n0], orc.moe_gather_scale_rows(b.d_mixed, b.rw, b.idx[0, :n0], 0))
    assert np.array_equal(r["g_in"][3], b.g_in0[3]) and np.array_equal(r["g_out"][3], b.g_out0[3])


def test_grouped_gelu_backward_with_per_expert_slots(cf, dev):
    case("grouped GELU backward whose recompute quantizes through the per-expert slots (is_recompute)")
    from oracle_slots import ActSlotOracle
    from test_gpu_moe_slots import SlotBank
    b = BwdBank(dev, 500, 4, 2, 256, 384, seed=79, zero_expert=1)
    bank = SlotBank(cf, dev, b.E, 8, 448.0, 0)
    try:
        # slots as a forward call leaves them: a snapshot pair per expert (different ones) and a newer scale that the
        # recompute must not use
        st = bank.words()
        for e in range(b.E):
            st[e, 1], st[e, 2] = 100.0 + e, 1.0 / (100.0 + e)                      # scale, descale: not to be used
            st[e, 3] = np.float32(448.0) / np.float32(1.5 + 0.5 * e)               # scale_snapshot
            st[e, 4] = np.float32(1.5 + 0.5 * e) / np.float32(448.0)               # descale_snapshot
            bank.oracle[e].scale_snapshot, bank.oracle[e].descale_snapshot = st[e, 3], st[e, 4]
        bank.state.copy_(torch.from_numpy(st.reshape(-1)))
        before = bank.words().view(np.uint32).copy()
        r = run_backward(cf, b, slots=(bank.state, bank.stride, 8, False))
        check_backward(b, r, slot_oracles=bank.oracle)
        assert np.array_equal(bank.words().view(np.uint32), before), "a recompute call must leave the slots as they are"
    finally:
        bank.close()


def test_grouped_gelu_backward_config5_size(cf, dev):
    case("grouped GELU backward at config 5 size: 16384 rows x 64 experts x top-6, H 2048, Ie 1408")
    b = BwdBank(dev, 16384, 64, 6, 2048, 1408, seed=5)
    assert b.total == 98304
    r = run_backward(cf, b)
    # bit-exact stages on all rows and experts; the GELU pair on every 16th row; the GEMM stages on three experts
    # (the weight gradients over all of their rows, the row-wise products on 48 sampled rows each)
    check_backward(b, r, gemm_experts=(0, 31, 63), gemm_rows=48, gelu_stride=16)


def test_grouped_gelu_backward_argument_errors(cf, dev):
    size = ctypes.c_size_t(0)
    assert cf.raw_cf_moe_grouped_gelu_backward_workspace(-1, 1, 1, 256, 256, None, ctypes.byref(size)) == -1
    assert cf.raw_cf_moe_grouped_gelu_backward_workspace(8, 8, 2, 256, 256, None, ctypes.byref(size)) == 0 and size.value > 0
    nul = [None] * 18
    assert cf.raw_cf_moe_grouped_gelu_backward_fp8(*nul[:3], 0, *nul[3:18], 8, 256, 256, 2, 8, None, 0, None) == -1
    assert cf.raw_cf_moe_grouped_gelu_backward_fp8(*nul[:3], 0, *nul[3:18], 0, 256, 256, 2, 0, None, 0, None) == 0
