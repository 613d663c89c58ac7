"""The delayed-scaling slot state machine: oracle properties on the CPU, device parity on the GPU."""
import ctypes

import numpy as np
import pytest

import oracle_lib as orc
from oracle_slots import ActSlotOracle, refresh_weight


def batches(seed, n, calls, growth=1.0):
    rng = np.random.default_rng(seed)
    return [orc.bf16_from_f32((rng.standard_normal(n) * (growth ** i) * (1 + 0.3 * rng.random())).astype(np.float32)) for i in range(calls)]


def test_oracle_slot_phases_and_scale_lag():
    slot = ActSlotOracle(history_len=8, calib_calls=3)
    xs = batches(0, 4096, 10)
    for i, x in enumerate(xs):
        q = slot.quant_act(x)
        if i < 3:   # calibration: exact amax of THIS tensor
            s, _ = orc.scale_from_amax(orc.amax_bf16(x), 448.0)
            assert slot.scale_snapshot == s and np.array_equal(q, orc.quantize_e4m3(x, s))
        else:       # steady state: the scale derived from the history of PREVIOUS calls
            window = [orc.amax_bf16(v) for v in xs[max(0, i - 8):i]]
            s, _ = orc.scale_from_amax(max(window), 448.0)
            assert slot.scale_snapshot == s and np.array_equal(q, orc.quantize_e4m3(x, s))
        # recompute reproduces the forward bytes and changes nothing
        before = (slot.scale, slot.amax, slot.delayed.cursor[0], slot.delayed.count[0])
        assert np.array_equal(slot.quant_act(x, is_recompute=True), q)
        assert before == (slot.scale, slot.amax, slot.delayed.cursor[0], slot.delayed.count[0])
    assert not slot.is_e5m2() and slot.calib_remaining == 0


def test_oracle_slot_switches_to_e5m2_when_the_range_moves():
    slot = ActSlotOracle(history_len=16, calib_calls=4, spread_threshold=4.0)
    xs = batches(1, 2048, 8, growth=2.0)          # amax doubles every call: spread 8 over the calibration window
    for i, x in enumerate(xs):
        slot.quant_act(x)
        assert slot.is_e5m2() == (i >= 4)         # committed on the first call AFTER calibration ends
    steady = ActSlotOracle(history_len=16, calib_calls=4)
    for x in batches(2, 2048, 8):
        steady.quant_act(x)
    assert not steady.is_e5m2()


def test_oracle_refresh_weight_layouts():
    rng = np.random.default_rng(3)
    w = orc.bf16_from_f32((0.02 * rng.standard_normal((96, 160))).astype(np.float32))
    fwd, bwd, amax, s, d = refresh_weight(w.reshape(-1), in_dim=96, out_dim=160, stored_out_major=False)
    assert fwd.shape == (160, 96) and bwd.shape == (96, 160) and np.array_equal(fwd, bwd.T)
    fwd2, bwd2, *_ = refresh_weight(w.reshape(-1), in_dim=160, out_dim=96, stored_out_major=True)
    assert fwd2.shape == (96, 160) and np.array_equal(fwd2, bwd) and np.array_equal(bwd2, fwd)


# ---- device parity ------------------------------------------------------------------------------
FIELDS = dict(amax=0, scale=1, descale=2, scale_snapshot=3, descale_snapshot=4, history=5, cursor=6, count=7, calib_min=8, calib_max=9)


class DevSlot:
    def __init__(self, cf, dev, history_len, fp8_max, calib_calls, spread=4.0):
        import torch
        from gpu_util import stream
        self.cf, self.dev = cf, dev
        words = cf.raw_cf_act_slot_state_words(history_len)
        self.state = torch.empty(words, dtype=torch.float32, device=dev)
        h = ctypes.c_void_p()
        rc = cf.raw_cf_act_slot_create(ctypes.byref(h), self.state.data_ptr(), history_len, fp8_max, calib_calls, spread, stream())
        assert rc == 0, f"cf_act_slot_create returned {rc}"
        self.h, self.history_len = h, history_len

    def quant(self, x_bits, recompute=False):
        import torch
        from gpu_util import dev_bf16, host, stream
        x = dev_bf16(x_bits, self.dev)
        out = torch.empty(x_bits.size, dtype=torch.uint8, device=self.dev)
        self.cf.cf_fp8_quant_act(self.h, x, out, x_bits.size, int(recompute), stream())
        torch.cuda.synchronize()
        return host(out)

    def field(self, name):
        base = self.state.data_ptr()
        p = ctypes.c_void_p()
        assert self.cf.raw_cf_act_slot_device_field(self.h, FIELDS[name], ctypes.byref(p)) == 0
        off = (p.value - base) // 4
        st = self.state.cpu().numpy()
        if name == "history":
            return st[off:off + self.history_len]
        if name in ("cursor", "count"):
            return st.view(np.int32)[off]
        return st[off]

    def close(self):
        self.cf.cf_act_slot_destroy(self.h)


@pytest.mark.gpu
@pytest.mark.parametrize("history_len,fp8_max,calib,growth", [(8, 448.0, 8, 1.0), (16, 448.0, 8, 1.0), (16, 448.0, 4, 2.0),
                                                             (8, 57344.0, 0, 1.0), (1, 448.0, 2, 1.3), (0, 448.0, 0, 1.0)])
def test_device_slot_follows_the_oracle(cf, dev, history_len, fp8_max, calib, growth):
    from gpu_util import case
    case(f"act slot history={history_len} fp8_max={fp8_max} calib={calib} growth={growth}")
    ds = DevSlot(cf, dev, history_len, fp8_max, calib)
    oslot = ActSlotOracle(history_len, fp8_max, calib)
    n = 70001
    for i, x in enumerate(batches(int(history_len + calib), n, 22, growth)):
        got = ds.quant(x)
        want = oslot.quant_act(x)
        assert np.array_equal(got, want), f"call {i}"
        assert bool(cf.raw_cf_act_slot_is_e5m2(ds.h)) == oslot.is_e5m2()
        for name, val in (("amax", oslot.amax), ("scale", oslot.scale), ("descale", oslot.descale),
                          ("scale_snapshot", oslot.scale_snapshot), ("descale_snapshot", oslot.descale_snapshot)):
            assert ds.field(name) == val, (i, name)
        if history_len > 0:
            assert ds.field("cursor") == oslot.delayed.cursor[0] and ds.field("count") == oslot.delayed.count[0]
            assert np.array_equal(ds.field("history"), oslot.delayed.history)
        if i % 5 == 2:      # the backward recompute of the same tensor: same bytes, no state change
            assert np.array_equal(ds.quant(x, recompute=True), want)
            assert ds.field("scale") == oslot.scale and ds.field("amax") == oslot.amax
    ds.close()


@pytest.mark.gpu
@pytest.mark.parametrize("in_dim,out_dim,out_major", [(128, 256, False), (256, 128, True), (96, 200, False), (4096, 1408, False)])
def test_device_refresh_weight(cf, dev, in_dim, out_dim, out_major):
    import torch
    from gpu_util import case, dev_bf16, host, stream
    case(f"refresh weight {in_dim}x{out_dim} out_major={out_major}")
    rng = np.random.default_rng(in_dim + out_dim)
    w = orc.bf16_from_f32((0.02 * rng.standard_normal(in_dim * out_dim)).astype(np.float32))
    fwd = torch.empty((out_dim, in_dim), dtype=torch.uint8, device=dev)
    bwd = torch.empty((in_dim, out_dim), dtype=torch.uint8, device=dev)
    sc = [torch.zeros(1, device=dev) for _ in range(3)]
    cf.cf_fp8_refresh_weight(dev_bf16(w, dev), fwd, bwd, sc[0], sc[1], sc[2], in_dim, out_dim, int(out_major), 1, stream())
    torch.cuda.synchronize()
    wf, wb, amax, s, d = refresh_weight(w, in_dim, out_dim, out_major)
    assert host(sc[0])[0] == amax and host(sc[1])[0] == s and host(sc[2])[0] == d
    assert np.array_equal(host(fwd), wf) and np.array_equal(host(bwd), wb)
    # without recompute the supplied amax (e.g. from the optimizer's fused side channel) is used as is
    sc[0].fill_(float(amax) * 2)
    cf.cf_fp8_refresh_weight(dev_bf16(w, dev), fwd, bwd, sc[0], sc[1], sc[2], in_dim, out_dim, int(out_major), 0, stream())
    torch.cuda.synchronize()
    wf2, wb2, *_ = refresh_weight(w, in_dim, out_dim, out_major, amax=np.float32(amax) * 2)
    assert np.array_equal(host(fwd), wf2) and np.array_equal(host(bwd), wb2)


@pytest.mark.gpu
@pytest.mark.parametrize("n,offset,history_len,e5m2", [(1 << 22, 0, 16, False), (100003, 1, 8, True), (5, 0, 0, False), (0, 0, 4, False)])
def test_one_launch_delayed_step_equals_the_separate_launches(cf, dev, n, offset, history_len, e5m2):
    """cf_fp8_quantize_delayed_step against snapshot copy + zeroed amax + quantize_record + update_delayed_scale,
    every byte and every state word, over several calls (history wrap-around included)."""
    import torch
    from gpu_util import case, dev_bf16, host, stream
    case(f"delayed step n={n} offset={offset} history={history_len} e5m2={e5m2}")
    fp8_max = 57344.0 if e5m2 else 448.0
    f32 = lambda *v: torch.tensor(v, dtype=torch.float32, device=dev)

    def fresh():
        return dict(amax=f32(0.0), scale=f32(3.5), descale=f32(1 / 3.5), ssnap=f32(0.0), dsnap=f32(0.0),
                    hist=torch.zeros(max(history_len, 1), dtype=torch.float32, device=dev),
                    cursor=torch.zeros(1, dtype=torch.int32, device=dev), count=torch.zeros(1, dtype=torch.int32, device=dev),
                    running=f32(0.0), arrived=torch.zeros(1, dtype=torch.int32, device=dev))
    a, b = fresh(), fresh()
    rng = np.random.default_rng(n + history_len)
    record = cf.cf_fp8_quantize_e5m2_record if e5m2 else cf.cf_fp8_quantize_e4m3_record
    for call in range(history_len + 3):
        xb = orc.bf16_from_f32((rng.standard_normal(n + offset) * (1.0 + call)).astype(np.float32))
        x = dev_bf16(xb, dev)[offset:]
        qa = torch.zeros(n + offset, dtype=torch.uint8, device=dev)[offset:]
        qb = torch.zeros(n + offset, dtype=torch.uint8, device=dev)[offset:]
        # the reference's sequence
        a["ssnap"].copy_(a["scale"]); a["dsnap"].copy_(a["descale"]); a["amax"].zero_()
        record(x, qa, a["scale"], a["amax"], n, stream())
        cf.cf_fp8_update_delayed_scale(a["amax"], fp8_max, a["scale"], a["descale"], a["hist"], history_len, a["cursor"], a["count"], stream())
        # one launch
        cf.cf_fp8_quantize_delayed_step(x, qb, n, int(e5m2), b["amax"], b["scale"], b["descale"], b["ssnap"], b["dsnap"],
                                        b["hist"], history_len, b["cursor"], b["count"], b["running"], b["arrived"], stream())
        torch.cuda.synchronize()
        assert torch.equal(qa, qb), f"call {call}"
        for k in ("amax", "scale", "descale", "ssnap", "dsnap", "hist", "cursor", "count"):
            assert torch.equal(a[k], b[k]), (call, k)
        assert float(b["running"]) == 0.0 and int(b["arrived"]) == 0
        if n:
            assert host(b["amax"])[0] == orc.amax_bf16(xb[offset:])
