"""GPU parity: the FP8 expert loop's per-expert activation slots (/root/reference/src/trainer.cu:6886-6934).

Between its two GEMMs the loop runs, for every expert WITH rows, gelu_forward in place and then fp8_quant_act on that
expert's own delayed-scaling slot (moe_fcout_act_slot(f8, layer, base + e), :6910-6918); fc_out dequantizes with the
slot's descale_snapshot (:6921-6924).  cf_moe_grouped_quantize_delayed is that step for all experts in one launch.
The oracle is the slot state machine restated in tests/oracle_slots.py, one instance per expert, stepping alongside
over several calls: the first calls (calibration, commit, first use) go per expert through cf_fp8_quant_act, as the
loop itself would, the later ones through the grouped launch; activation bytes, snapshots and every state word are
compared bit for bit per expert, and an expert without rows must keep its state."""
import ctypes

import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_arr, dev_bf16, host, stream
from oracle_slots import ActSlotOracle

pytestmark = pytest.mark.gpu

W = dict(amax=0, scale=1, descale=2, scale_snapshot=3, descale_snapshot=4, cursor=8, count=9, running=10, arrived=11, history=16)


class SlotBank:
    """E device slots in one block (stride words apart) with their host objects, and E oracles."""

    def __init__(self, cf, dev, E, history_len, fp8_max, calib_calls):
        self.cf, self.dev, self.E, self.hist, self.fp8_max = cf, dev, E, history_len, fp8_max
        self.stride = cf.raw_cf_act_slot_state_words(history_len) + 5          # not a multiple of anything in particular
        self.state = torch.zeros(E * self.stride, dtype=torch.float32, device=dev)
        self.h = []
        for e in range(E):
            h = ctypes.c_void_p()
            assert cf.raw_cf_act_slot_create(ctypes.byref(h), self.state.data_ptr() + 4 * e * self.stride, history_len, fp8_max,
                                             calib_calls, 4.0, stream()) == 0
            self.h.append(h)
        self.oracle = [ActSlotOracle(history_len=history_len, fp8_max=fp8_max, calib_calls=calib_calls) for _ in range(E)]

    def words(self):
        return self.state.cpu().numpy().reshape(self.E, self.stride)

    def check_state(self, what):
        st = self.words()
        for e, o in enumerate(self.oracle):
            w, wi = st[e], st[e].view(np.int32)
            got = (w[W["amax"]], w[W["scale"]], w[W["descale"]], w[W["scale_snapshot"]], w[W["descale_snapshot"]],
                   int(wi[W["cursor"]]), int(wi[W["count"]]))
            want = (o.amax, o.scale, o.descale, o.scale_snapshot, o.descale_snapshot, int(o.delayed.cursor[0]), int(o.delayed.count[0]))
            assert got == want, (what, e, got, want)
            assert np.array_equal(w[W["history"]:W["history"] + self.hist], o.delayed.history[:self.hist]), (what, e)
            assert w[W["running"]] == 0.0 and wi[W["arrived"]] == 0, (what, e)

    def close(self):
        for h in self.h:
            self.cf.cf_act_slot_destroy(h)


def routing(rng, rows, E, k, empty=()):
    logits = rng.standard_normal((rows, E)).astype(np.float32)
    for e in empty:
        logits[:, e] = -50.0
    rw = orc.moe_topk_route(logits, k)
    counts, idx = orc.moe_build_expert_row_lists(rw)
    return rw, counts, idx, orc.moe_expert_offsets(counts)


@pytest.mark.parametrize("E,K,rows,k,history_len,fp8_max", [(5, 384, 300, 2, 8, 448.0), (4, 256, 200, 2, 16, 448.0),
                                                            (6, 1408, 90, 3, 8, 57344.0), (3, 128, 1500, 1, 0, 448.0)])
def test_grouped_delayed_quantize_follows_the_per_expert_slots(cf, dev, E, K, rows, k, history_len, fp8_max):
    case(f"grouped delayed quantize E={E} K={K} rows={rows} k={k} history={history_len} fp8_max={fp8_max}")
    rng = np.random.default_rng(E * 1000 + K)
    e5m2 = fp8_max > 1000
    calib = 2
    bank = SlotBank(cf, dev, E, history_len, fp8_max, calib)
    quant = orc.quantize_e5m2 if e5m2 else orc.quantize_e4m3
    try:
        for call in range(9):
            empty = () if call < 4 else ((call % E,) if call % 2 == 0 else (call % E, (call + 2) % E))
            rw, counts, idx, offsets = routing(rng, rows, E, k, empty)
            total = int(counts.sum())
            bound = rows * k + (call % 3) * 17                                   # what the caller knows: an upper bound
            pre = orc.bf16_from_f32((rng.standard_normal((bound, K)) * (1.0 + 0.2 * rng.random())).astype(np.float32))
            d_pre = dev_bf16(pre, dev)
            g = torch.empty_like(d_pre)
            cf.cf_gelu_forward_bf16(d_pre, g, bound * K, stream())
            g_bits = bf16_bits(g)                                                # the GPU's own GELU values (pinned to an ulp elsewhere)
            out = torch.full((bound, K), 0xEE, dtype=torch.uint8, device=dev)
            row_descale = torch.full((bound,), -1.0, dtype=torch.float32, device=dev)
            before = bank.words().copy()
            if call < calib + 2:
                # calibration calls, the call that commits the calibration, the first steady call: per expert on the host,
                # as the reference loop runs them
                for e in range(E):
                    n, o = int(counts[e]), int(offsets[e])
                    if n == 0:
                        continue
                    cf.cf_fp8_quant_act(bank.h[e], g[o:o + n], out[o:o + n], n * K, 0, stream())
            else:
                cf.cf_moe_grouped_quantize_delayed(d_pre, out, K, E, dev_arr(counts, dev), dev_arr(offsets, dev), bound, bank.state,
                                                   bank.stride, history_len, int(e5m2), 1, 0, row_descale, stream())
            torch.cuda.synchronize()
            got = host(out)
            for e in range(E):
                n, o = int(counts[e]), int(offsets[e])
                if n == 0:
                    continue
                want = bank.oracle[e].quant_act(g_bits[o:o + n].reshape(-1))
                assert np.array_equal(got[o:o + n].reshape(-1), want), (call, e)
                if call >= calib + 2:
                    assert np.all(host(row_descale)[o:o + n] == bank.oracle[e].descale_snapshot), (call, e)
            assert np.all(got[total:] == 0xEE), "rows past the experts' lists were written"
            bank.check_state(f"call {call}")
            after = bank.words()
            for e in empty:
                assert np.array_equal(after[e].view(np.uint32), before[e].view(np.uint32)), f"call {call}: expert {e} has no rows and must keep its slot"
            if call >= calib + 2:
                # the backward's recompute: the bytes of the forward call, nothing changes
                out2 = torch.full((bound, K), 0xEE, dtype=torch.uint8, device=dev)
                rd2 = torch.full((bound,), -1.0, dtype=torch.float32, device=dev)
                cf.cf_moe_grouped_quantize_delayed(g, out2, K, E, dev_arr(counts, dev), dev_arr(offsets, dev), bound, bank.state,
                                                   bank.stride, history_len, int(e5m2), 0, 1, rd2, stream())
                torch.cuda.synchronize()
                assert np.array_equal(host(out2), got) and np.array_equal(host(rd2), host(row_descale))
                assert np.array_equal(bank.words().view(np.uint32), after.view(np.uint32))
            assert not any(o.is_e5m2() != e5m2 for o in bank.oracle)
    finally:
        bank.close()


def test_counts_beyond_the_bound(cf, dev):
    case("grouped delayed quantize with counts that sum past total_rows: cut at the bound")
    E, K, hist = 3, 128, 8
    bank = SlotBank(cf, dev, E, hist, 448.0, 0)
    try:
        st = bank.words()
        st[:, W["scale"]] = 4.0
        st[:, W["descale"]] = 0.25
        bank.state.copy_(torch.from_numpy(st.reshape(-1)))
        counts = np.array([40, 50, 60], np.int32)
        offsets = np.array([0, 40, 90], np.int32)
        bound = 100                                                        # expert 1 keeps 50, expert 2 keeps 10
        x = orc.bf16_from_f32(np.random.default_rng(3).standard_normal((bound, K)).astype(np.float32))
        out = torch.full((bound + 64, K), 0xEE, dtype=torch.uint8, device=dev)
        rd = torch.full((bound + 64,), -1.0, dtype=torch.float32, device=dev)
        cf.cf_moe_grouped_quantize_delayed(dev_bf16(x, dev), out, K, E, dev_arr(counts, dev), dev_arr(offsets, dev), bound, bank.state,
                                           bank.stride, hist, 0, 0, 0, rd, stream())
        torch.cuda.synchronize()
        got = host(out)
        assert np.array_equal(got[:bound].reshape(-1), orc.quantize_e4m3(x.reshape(-1), np.float32(4.0)))
        assert np.all(got[bound:] == 0xEE) and np.all(host(rd)[bound:] == -1.0) and np.all(host(rd)[:bound] == 0.25)
        st = bank.words()
        assert st[2, W["amax"]] == orc.amax_bf16(x[90:100].reshape(-1))     # the amax of the rows kept, not of rows beyond
    finally:
        bank.close()


@pytest.mark.parametrize("e5m2", [False, True])
def test_large_banks_take_the_table_form_with_the_same_bits(cf, dev, e5m2):
    """From 64 Mi elements (rows of the bound x K) the GELU form looks bf16(gelu(x)) up in a table held in LDS by
    workgroups that stay resident; total_rows being an upper bound, the same routing runs through both forms."""
    case(f"grouped delayed GELU quantize, table form against the direct form, e5m2={e5m2}")
    E, K, hist = 8, 1408, 8
    counts = np.array([9000, 0, 7001, 300, 11000, 1, 8000, 4698], np.int32)
    offsets = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.int32)
    total = int(counts.sum())                                              # 40000 rows: 56 Mi elements, the direct form
    bound = 50000                                                          # 70 Mi elements: the table form
    assert total * K < (64 << 20) <= bound * K
    gen = torch.Generator(device=dev).manual_seed(11)
    x = (torch.randn(bound, K, device=dev, generator=gen) * 1.7).to(torch.bfloat16)
    fp8_max = 57344.0 if e5m2 else 448.0
    stride = cf.raw_cf_act_slot_state_words(hist) + 3
    init = np.zeros((E, stride), np.float32)
    init[:, W["scale"]] = fp8_max / 6.0
    init[:, W["descale"]] = 6.0 / fp8_max
    init[:, W["history"]] = 6.0
    init.view(np.int32)[:, W["cursor"]] = 1
    init.view(np.int32)[:, W["count"]] = 1
    d_counts, d_offsets = dev_arr(counts, dev), dev_arr(offsets, dev)
    results = []
    for rows_bound in (total, bound):
        state = torch.from_numpy(init.reshape(-1).copy()).to(dev)
        per_call = []
        for call in range(2):
            out = torch.full((bound, K), 0xEE, dtype=torch.uint8, device=dev)
            rd = torch.full((bound,), -1.0, dtype=torch.float32, device=dev)
            cf.cf_moe_grouped_quantize_delayed(x, out, K, E, d_counts, d_offsets, rows_bound, state, stride, hist, int(e5m2), 1, 0, rd, stream())
            out_r = torch.full((bound, K), 0xEE, dtype=torch.uint8, device=dev)
            rd_r = torch.full((bound,), -1.0, dtype=torch.float32, device=dev)
            cf.cf_moe_grouped_quantize_delayed(x, out_r, K, E, d_counts, d_offsets, rows_bound, state, stride, hist, int(e5m2), 1, 1, rd_r, stream())
            torch.cuda.synchronize()
            assert torch.equal(out_r, out) and torch.equal(rd_r, rd), "the recompute pass gives the forward call's bytes"
            assert bool((out[total:] == 0xEE).all()) and bool((rd[total:] == -1.0).all())
            per_call.append((out, rd, state.clone()))
        results.append(per_call)
    for call in range(2):
        (o_a, rd_a, st_a), (o_b, rd_b, st_b) = results[0][call], results[1][call]
        assert torch.equal(o_a, o_b), f"call {call}: bytes differ between the two forms"
        assert torch.equal(rd_a, rd_b)
        assert torch.equal(st_a.view(torch.int32), st_b.view(torch.int32)), f"call {call}: slot states differ"
    # and one expert against the oracle (the GPU's own GELU values as its input)
    e = 3
    o, n = int(offsets[e]), int(counts[e])
    g = torch.empty((n, K), dtype=torch.bfloat16, device=dev)
    cf.cf_gelu_forward_bf16(x[o:o + n].contiguous(), g, n * K, stream())
    torch.cuda.synchronize()
    quant = orc.quantize_e5m2 if e5m2 else orc.quantize_e4m3
    g_bits = bf16_bits(g).reshape(-1)
    assert np.array_equal(host(results[1][0][0][o:o + n]).reshape(-1), quant(g_bits, np.float32(fp8_max / 6.0)))
    st = results[1][0][2].cpu().numpy().reshape(E, stride)
    amax = orc.amax_bf16(g_bits)
    assert st[e, W["amax"]] == amax and st[e, W["history"] + 1] == max(amax, np.float32(1e-12))
    assert st[e, W["scale"]] == np.float32(fp8_max) / max(amax, np.float32(6.0))
    assert np.array_equal(st[1], init[1]), "an expert without rows keeps its slot"
    second = results[1][1][0]
    want_scale = st[e, W["scale"]]
    assert np.array_equal(host(second[o:o + n]).reshape(-1), quant(g_bits, np.float32(want_scale)))


class LoopBank:
    """Inputs of the FP8 GELU expert loop with per-tensor descales (the reference's slots are per tensor)."""

    def __init__(self, dev, rows, E, k, H, Ie, seed):
        rng = np.random.default_rng(seed)
        self.dev, self.rows, self.E, self.k, self.H, self.Ie = dev, rows, E, k, H, Ie

        def q(x):
            s, d = orc.scale_from_amax(np.float32(np.abs(x).max()), 448.0)
            return orc.e4m3_satfinite((x * s).astype(np.float32)).reshape(x.shape), np.float32(d)
        self.wi, self.wid = q((0.05 * rng.standard_normal((E * Ie, H))).astype(np.float32))
        self.wo, self.wod = q((0.05 * rng.standard_normal((E * H, Ie))).astype(np.float32))
        self.q = q
        self.rng = rng

    def step_inputs(self, empty=()):
        x = (self.rng.standard_normal((self.rows, self.H)) * (1.0 + 0.3 * self.rng.random())).astype(np.float32)
        hq, hd = self.q(x)
        rw, counts, idx, offsets = routing(self.rng, self.rows, self.E, self.k, empty)
        mixed0 = orc.bf16_from_f32(self.rng.standard_normal((self.rows, self.H)).astype(np.float32))
        return hq, hd, rw, counts, idx, offsets, mixed0


@pytest.mark.parametrize("history_len", [8, 16])
def test_gelu_bank_with_per_expert_slots_is_the_reference_loop(cf, dev, history_len):
    case(f"GELU expert bank in one call with per-expert delayed-scale slots, history {history_len}")
    rows, E, k, H, Ie = 400, 5, 2, 256, 384
    b = LoopBank(dev, rows, E, k, H, Ie, seed=history_len)
    bank = SlotBank(cf, dev, E, history_len, 448.0, 0)          # no calibration calls: call 0 is the first use, then steady state
    sc = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    full = lambda v, n: torch.full((n,), float(v), dtype=torch.float32, device=dev)
    d_wi, d_wo = dev_arr(b.wi, dev), dev_arr(b.wo, dev)
    sz, gsz = ctypes.c_size_t(0), ctypes.c_size_t(0)
    bound = rows * k
    assert cf.raw_cf_moe_grouped_gelu_workspace_bytes(rows, bound, E, H, Ie, ctypes.byref(sz)) == 0
    assert cf.raw_cf_fp8_grouped_gemm_workspace_bytes(bound, E, ctypes.byref(gsz)) == 0
    ws = torch.empty(sz.value + 256, dtype=torch.uint8, device=dev)
    ws_ptr = ws.data_ptr() + (-ws.data_ptr()) % 256
    gws = torch.empty(gsz.value, dtype=torch.uint8, device=dev)
    try:
        for call in range(7):
            hq, hd, rw, counts, idx, offsets, mixed0 = b.step_inputs(empty=() if call < 2 else (call % E,))
            total = int(counts.sum())
            d = dict(hq=dev_arr(hq, dev), rw=dev_arr(rw, dev), counts=dev_arr(counts, dev), offsets=dev_arr(offsets, dev), idx=dev_arr(idx, dev))
            # the loop's stages through the public entry points: gather + fc_in for all experts ...
            cidx = torch.zeros((bound,), dtype=torch.int32, device=dev)
            cf.cf_moe_compact_row_index(d["counts"], d["offsets"], d["idx"], rows, E, cidx, stream())
            act = torch.zeros((bound, Ie), dtype=torch.bfloat16, device=dev)
            cf.cf_fp8_grouped_gemm_nt_bf16_ex(bound, Ie, H, E, d["counts"], d["offsets"], d["hq"], rows, H, cidx, full(hd, rows), d_wi,
                                              full(b.wid, E * Ie), 1, 0, None, None, act, Ie, gws, gsz.value, stream())
            g = torch.empty_like(act)
            cf.cf_gelu_forward_bf16(act, g, bound * Ie, stream())
            torch.cuda.synchronize()
            g_bits = bf16_bits(g)
            # ... the oracle's slots step over the GPU's GELU values, expert by expert, as the loop's fp8_quant_act calls do
            want_q = np.zeros((bound, Ie), np.uint8)
            want_d = np.zeros(bound, np.float32)
            for e in range(E):
                n, o = int(counts[e]), int(offsets[e])
                if n == 0:
                    continue
                want_q[o:o + n] = bank.oracle[e].quant_act(g_bits[o:o + n].reshape(-1)).reshape(n, Ie)
                want_d[o:o + n] = bank.oracle[e].descale_snapshot
            if call == 0:
                # first use of every slot (exact amax): per expert on the host objects, as the reference runs it
                actq = torch.zeros((bound, Ie), dtype=torch.uint8, device=dev)
                for e in range(E):
                    n, o = int(counts[e]), int(offsets[e])
                    cf.cf_fp8_quant_act(bank.h[e], g[o:o + n], actq[o:o + n], n * Ie, 0, stream())
                torch.cuda.synchronize()
                assert np.array_equal(host(actq)[:total], want_q[:total])
                bank.check_state("first use")
                continue
            # fc_out on the oracle's bytes and snapshots, unpermute: what the loop leaves in `mixed`
            y = torch.zeros((bound, H), dtype=torch.bfloat16, device=dev)
            cf.cf_fp8_grouped_gemm_nt_bf16_ex(bound, H, Ie, E, d["counts"], d["offsets"], dev_arr(want_q, dev), bound, Ie, None,
                                              dev_arr(want_d, dev), d_wo, full(b.wod, E * H), 1, 0, None, None, y, H, gws, gsz.value, stream())
            want_mixed = dev_bf16(mixed0, dev)
            cf.cf_moe_unpermute_weighted_bf16(want_mixed, y, d["rw"], d["counts"], d["offsets"], d["idx"], rows, E, H, stream())
            # the one call, on the device's slots
            mixed = dev_bf16(mixed0, dev)
            cf.cf_moe_grouped_gelu_forward_fp8_slots(d["hq"], sc(hd), 0, d["rw"], d["counts"], d["offsets"], d["idx"], d_wi, sc(b.wid), d_wo,
                                                     sc(b.wod), mixed, rows, H, Ie, E, bound, bank.state, bank.stride, history_len, 0, 0,
                                                     ws_ptr, sz.value, stream())
            torch.cuda.synchronize()
            assert np.array_equal(bf16_bits(mixed), bf16_bits(want_mixed)), f"call {call}"
            bank.check_state(f"call {call}")
            # and the unpermute itself against the oracle's scatter-accumulate, expert by expert
            m = mixed0
            yb = bf16_bits(y)
            for e in range(E):
                n, o = int(counts[e]), int(offsets[e])
                m = orc.moe_scatter_accumulate(m, yb[o:o + n], rw, idx[e, :n], e)
            assert np.array_equal(bf16_bits(mixed), m)
            # replay for the backward: same bits, state untouched
            state_before = bank.words().view(np.uint32).copy()
            mixed2 = dev_bf16(mixed0, dev)
            cf.cf_moe_grouped_gelu_forward_fp8_slots(d["hq"], sc(hd), 0, d["rw"], d["counts"], d["offsets"], d["idx"], d_wi, sc(b.wid), d_wo,
                                                     sc(b.wod), mixed2, rows, H, Ie, E, bound, bank.state, bank.stride, history_len, 0, 1,
                                                     ws_ptr, sz.value, stream())
            torch.cuda.synchronize()
            assert np.array_equal(bf16_bits(mixed2), bf16_bits(mixed))
            assert np.array_equal(bank.words().view(np.uint32), state_before)
    finally:
        bank.close()
