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
