"""GPU: the library's launches can be recorded into a HIP graph (they allocate nothing, never synchronize and clear
device scalars with kernels, not memset nodes).  A config-2-shaped MLP step and a delayed-scaling step are captured
once and replayed several times on changing inputs, with eager work and synchronizations between the replays; every
replay must reproduce the eager result bit for bit."""
import numpy as np
import pytest
import torch

from gpu_util import case, stream

pytestmark = pytest.mark.gpu


def fp8_weights(n, k, dev, g):
    w = torch.randn(n, k, device=dev, generator=g) * 0.02
    s = w.abs().amax(dim=1).clamp_min(1e-12)
    q = (w * (448.0 / s)[:, None]).to(torch.float8_e4m3fn).view(torch.uint8)
    return q, (s / 448.0).contiguous()


def test_mlp_step_replays_from_a_graph(cf, dev):
    case("graph capture: quantize -> gate/up -> quantize -> down")
    M, K, N = 512, 1024, 1536
    g = torch.Generator(device=dev); g.manual_seed(11)
    wg, wgd = fp8_weights(N, K, dev, g); wu, wud = fp8_weights(N, K, dev, g); wd, wdd = fp8_weights(K, N, dev, g)
    x = torch.empty((M, K), dtype=torch.bfloat16, device=dev)
    xq = torch.empty((M, K), dtype=torch.uint8, device=dev); xs = torch.empty(M, device=dev); xd = torch.empty(M, device=dev)
    h = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    hq = torch.empty((M, N), dtype=torch.uint8, device=dev); hs = torch.empty(M, device=dev); hd = torch.empty(M, device=dev)
    y = torch.empty((M, K), dtype=torch.bfloat16, device=dev)
    amax = torch.zeros(1, device=dev)

    def step():
        s = stream()
        cf.cf_fp8_quantize_rows(x, M, K, 0, xq, xs, xd, s)
        cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wg, K, wgd, 1, 2, None, wu, wud, h, N, 0, s)
        cf.cf_fp8_amax_bf16(h, h.numel(), amax, s)                  # clears its scalar with a kernel
        cf.cf_fp8_quantize_rows(h, M, N, 0, hq, hs, hd, s)
        cf.cf_fp8_gemm_nt_bf16_ex(M, K, N, hq, N, 0, hd, wd, N, wdd, 1, 0, None, None, None, y, K, 0, s)

    inputs = [(torch.randn(M, K, device=dev, generator=g) * (1.0 + i)).to(torch.bfloat16) for i in range(4)]
    x.copy_(inputs[0]); step(); torch.cuda.synchronize()          # warm-up outside the capture (one-time kernel attributes)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for i, xin in enumerate(inputs):
        x.copy_(xin)
        step()
        torch.cuda.synchronize()
        want_y, want_h, want_amax = y.clone(), h.clone(), amax.clone()
        y.zero_(); h.zero_(); amax.fill_(-1.0)
        scratch = torch.randn(1 << 20, device=dev).sum()           # unrelated eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), want_y.view(torch.int16)), f"replay {i}"
        assert torch.equal(h.view(torch.int16), want_h.view(torch.int16)) and torch.equal(amax, want_amax), f"replay {i}"
        assert float(scratch) == float(scratch)


def test_delayed_scaling_step_replays_from_a_graph(cf, dev):
    case("graph capture: one-launch delayed-scaling step")
    n, hist_len = 300000, 4
    g = torch.Generator(device=dev); g.manual_seed(12)
    x = torch.empty(n, dtype=torch.bfloat16, device=dev)
    q = torch.empty(n, dtype=torch.uint8, device=dev)

    def fresh():
        f32 = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
        return [f32(0.0), f32(2.0), f32(0.5), f32(0.0), f32(0.0), torch.zeros(hist_len, device=dev),
                torch.zeros(1, dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int32, device=dev),
                f32(0.0), torch.zeros(1, dtype=torch.int32, device=dev)]
    eager, captured = fresh(), fresh()

    def step(st):
        cf.cf_fp8_quantize_delayed_step(x, q, n, 0, st[0], st[1], st[2], st[3], st[4], st[5], hist_len, st[6], st[7], st[8], st[9], stream())

    graph = torch.cuda.CUDAGraph()
    x.copy_(torch.randn(n, device=dev, generator=g).to(torch.bfloat16))
    with torch.cuda.graph(graph):
        step(captured)
    for i in range(7):
        x.copy_((torch.randn(n, device=dev, generator=g) * (1.0 + 0.5 * i)).to(torch.bfloat16))
        step(eager)
        torch.cuda.synchronize()
        want_q = q.clone()
        q.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(q, want_q), f"replay {i}"
        for a, b in zip(eager, captured):
            assert torch.equal(a, b), f"replay {i}"


def test_moe_layer_replays_from_a_graph(cf, dev):
    """Routing, row lists, offsets and the one-call expert banks (SwiGLU; GELU with re-quantized activations; the workspace
    forms of moe_grouped_expert_forward_fp8 and _bf16, which take no offsets) in one captured graph: every buffer the routing fills is consumed on the device, so a replay on new logits and new hidden
    states must reproduce the eager run bit for bit."""
    import ctypes
    case("graph capture: top-k route -> row lists -> offsets -> SwiGLU bank -> GELU bank")
    T, E, k, H, Ie = 768, 8, 2, 256, 384
    total = T * k
    g = torch.Generator(device=dev); g.manual_seed(23)
    wg, wgd = fp8_weights(E * Ie, H, dev, g); wu, wud = fp8_weights(E * Ie, H, dev, g); wd, wdd = fp8_weights(E * H, Ie, dev, g)
    one = torch.full((1,), 0.02, device=dev)
    logits = torch.empty((T, E), device=dev)
    rw = torch.empty((T, E), device=dev)
    hq = torch.empty((T, H), dtype=torch.uint8, device=dev); hd = torch.empty(T, device=dev)
    counts = torch.zeros(E, dtype=torch.int32, device=dev); offs = torch.zeros(E, dtype=torch.int32, device=dev)
    idx = torch.zeros(E * T, dtype=torch.int32, device=dev)
    out_swiglu = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    out_gelu = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    out_ref8 = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    out_ref16 = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    h16 = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    wi16 = (0.05 * torch.randn(E * Ie, H, device=dev, generator=g)).to(torch.bfloat16)
    wo16 = (0.05 * torch.randn(E * H, Ie, device=dev, generator=g)).to(torch.bfloat16)
    s3, s4 = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert cf.raw_cf_moe_grouped_expert_forward_fp8_workspace(T, total, E, H, Ie, None, ctypes.byref(s3)) == 0 and s3.value > 0
    assert cf.raw_cf_moe_grouped_expert_forward_bf16_workspace(T, total, E, H, Ie, None, ctypes.byref(s4)) == 0 and s4.value > 0
    ws3 = torch.empty(s3.value + 256, dtype=torch.uint8, device=dev); p3 = ws3.data_ptr() + (-ws3.data_ptr()) % 256
    ws4 = torch.empty(s4.value + 256, dtype=torch.uint8, device=dev); p4 = ws4.data_ptr() + (-ws4.data_ptr()) % 256
    s1, s2 = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert cf.raw_cf_moe_grouped_swiglu_workspace_bytes(total, E, H, Ie, ctypes.byref(s1)) == 0
    assert cf.raw_cf_moe_grouped_gelu_workspace_bytes(T, total, E, H, Ie, ctypes.byref(s2)) == 0
    ws1 = torch.empty(s1.value + 256, dtype=torch.uint8, device=dev); p1 = ws1.data_ptr() + (-ws1.data_ptr()) % 256
    ws2 = torch.empty(s2.value + 256, dtype=torch.uint8, device=dev); p2 = ws2.data_ptr() + (-ws2.data_ptr()) % 256

    def step():
        s = stream()
        rw.copy_(logits)
        out_swiglu.zero_(); out_gelu.zero_(); out_ref8.zero_(); out_ref16.zero_()
        cf.cf_moe_topk_route_f32(rw, T, E, k, s, None, None, 1)
        cf.cf_moe_build_expert_row_lists(rw, counts, idx, T, E, s)
        cf.cf_moe_expert_offsets_from_counts(counts, offs, E, s)
        cf.cf_moe_grouped_swiglu_forward_fp8(hq, hd, rw, counts, offs, idx, wg, wgd, wu, wud, wd, wdd, out_swiglu, T, H, Ie, E, total,
                                             p1, s1.value, s)
        cf.cf_moe_grouped_gelu_forward_fp8(hq, one, 0, rw, counts, offs, idx, wg, one, wd, one, out_gelu, T, H, Ie, E, total,
                                           p2, s2.value, s)
        cf.cf_moe_grouped_expert_forward_fp8_ws(hq, one, 0, rw, counts, None, idx, wg, one, wd, one, out_ref8, T, H, Ie, E, total,
                                                p3, s3.value, s)
        cf.cf_moe_grouped_expert_forward_bf16_ws(h16, rw, counts, None, idx, wi16, wo16, out_ref16, T, H, Ie, E, total, p4, s4.value, s)

    def new_inputs(i):
        logits.copy_(torch.randn(T, E, device=dev, generator=g))
        x = torch.randn(T, H, device=dev, generator=g) * (1.0 + i)
        amax = x.abs().amax(dim=1).clamp_min(1e-12)
        hq.copy_((x * (448.0 / amax)[:, None]).to(torch.float8_e4m3fn).view(torch.uint8)); hd.copy_(amax / 448.0)
        h16.copy_(x.to(torch.bfloat16))

    new_inputs(0); step(); torch.cuda.synchronize()                 # warm-up outside the capture
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for i in range(4):
        new_inputs(i)
        step()
        torch.cuda.synchronize()
        want = (out_swiglu.clone(), out_gelu.clone(), counts.clone(), rw.clone(), out_ref8.clone(), out_ref16.clone())
        assert float(out_ref8.float().abs().max()) > 0 and float(out_ref16.float().abs().max()) > 0
        assert int(counts.sum()) == total
        out_swiglu.fill_(7.0); out_gelu.fill_(7.0); counts.fill_(-1); rw.fill_(0.5); out_ref8.fill_(7.0); out_ref16.fill_(7.0)
        scratch = torch.randn(1 << 20, device=dev).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(counts, want[2]) and torch.equal(rw, want[3]), f"replay {i}"
        assert torch.equal(out_swiglu.view(torch.int16), want[0].view(torch.int16)), f"replay {i}"
        assert torch.equal(out_gelu.view(torch.int16), want[1].view(torch.int16)), f"replay {i}"
        assert torch.equal(out_ref8.view(torch.int16), want[4].view(torch.int16)), f"replay {i}"
        assert torch.equal(out_ref16.view(torch.int16), want[5].view(torch.int16)), f"replay {i}"
        assert float(scratch) == float(scratch)


def test_moe_backward_and_static_grouped_gemm_replay_from_a_graph(cf, dev):
    """The one-call selected-expert backward (its route-weight gradient is cleared by a kernel, not a memset node) and
    the grouped GEMM whose tile table lives in the library's own device array (set up before the capture) in one
    captured graph; replays on new gradients must reproduce the eager run bit for bit."""
    import ctypes
    import numpy as np
    import oracle_lib as orc
    from gpu_util import dev_arr
    case("graph capture: GELU bank backward + static grouped GEMM")
    T, E, k, H, Ie = 512, 4, 2, 256, 256
    g = torch.Generator(device=dev); g.manual_seed(31)
    rng = np.random.default_rng(31)
    rw_h = orc.moe_topk_route(rng.standard_normal((T, E)).astype(np.float32), k)
    counts_h, idx_h = orc.moe_build_expert_row_lists(rw_h)
    offs_h = orc.moe_expert_offsets(counts_h)
    total = int(counts_h.sum())
    rw, counts, offs, idx = dev_arr(rw_h, dev), dev_arr(counts_h, dev), dev_arr(offs_h, dev), dev_arr(idx_h, dev)
    w_in8, w_in_d = fp8_weights(E * Ie, H, dev, g); w_out8, w_out_d = fp8_weights(E * H, Ie, dev, g)
    one = torch.full((1,), 0.02, device=dev)
    w_in = (torch.randn(E * Ie, H, device=dev, generator=g) * 0.05).to(torch.bfloat16)
    w_out = (torch.randn(E * H, Ie, device=dev, generator=g) * 0.05).to(torch.bfloat16)
    hidden = torch.randn(T, H, device=dev, generator=g).to(torch.bfloat16)
    hq = (hidden.float() * (448.0 / hidden.float().abs().max())).to(torch.float8_e4m3fn).view(torch.uint8)
    hd = (hidden.float().abs().max() / 448.0).reshape(1)
    hrow_d = hd.expand(T).contiguous()
    d_mixed = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    d_rw = torch.empty((T, E), device=dev)
    g_in = torch.zeros((E * Ie, H), dtype=torch.bfloat16, device=dev); g_out = torch.zeros((E * H, Ie), dtype=torch.bfloat16, device=dev)
    d_hidden = torch.zeros((T, H), dtype=torch.bfloat16, device=dev)
    cidx = torch.empty(total, dtype=torch.int32, device=dev)
    static_out = torch.empty((total, Ie), dtype=torch.bfloat16, device=dev)
    size = ctypes.c_size_t(0)
    assert cf.raw_cf_moe_grouped_gelu_backward_workspace(T, total, E, H, Ie, None, ctypes.byref(size)) == 0
    ws = torch.empty(size.value + 256, dtype=torch.uint8, device=dev); wp = ws.data_ptr() + (-ws.data_ptr()) % 256
    mx = ctypes.c_size_t(0)
    assert cf.raw_cf_fp8_grouped_gemm_static_max_bytes(ctypes.byref(mx)) == 0          # set-up: before any capture

    def step():
        s = stream()
        g_in.zero_(); g_out.zero_(); d_hidden.zero_()
        cf.cf_moe_grouped_gelu_backward_fp8(d_mixed, hq, hd, 0, hidden, rw, counts, offs, idx, w_in8, one, w_out8, one, w_in, w_out,
                                            d_rw, g_in, g_out, d_hidden, T, H, Ie, E, total, wp, size.value, s)
        cf.cf_moe_compact_row_index(counts, offs, idx, T, E, cidx, s)
        cf.cf_fp8_grouped_gemm_nt_bf16_static(total, Ie, H, E, counts, offs, hq, T, H, cidx, hrow_d, w_in8, w_in_d, 1, 0, None, None,
                                              static_out, Ie, s)

    d_mixed.copy_((torch.randn(T, H, device=dev, generator=g) * 1e-2).to(torch.bfloat16)); step(); torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for i in range(3):
        d_mixed.copy_((torch.randn(T, H, device=dev, generator=g) * 1e-2 * (1 + i)).to(torch.bfloat16))
        step()
        torch.cuda.synchronize()
        want = [t.clone() for t in (d_rw, g_in, g_out, d_hidden, static_out)]
        for t in (d_rw, g_in, g_out, d_hidden, static_out):
            t.fill_(3.0)
        scratch = torch.randn(1 << 20, device=dev).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("d_rw", "g_in", "g_out", "d_hidden", "static_out"), (d_rw, g_in, g_out, d_hidden, static_out), want):
            assert torch.equal(a.view(torch.int32 if a.dtype == torch.float32 else torch.int16),
                               b.view(torch.int32 if b.dtype == torch.float32 else torch.int16)), f"replay {i}: {name}"
        assert float(scratch) == float(scratch)
