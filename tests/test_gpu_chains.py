"""GPU parity of two call chains at their real sizes, every link checked on the bytes the link before it wrote.

LM head (/root/reference/src/trainer.cu:8015-8060), one chunk of token rows: fp8_quant_act of the final hidden states
-> lt_gemm_fp8_nt with N = vocabulary -> cross_entropy_fwd_bwd_chunk -> fp8_quant_act of the logits' gradient as E5M2
-> lt_gemm_fp8_nt with K = vocabulary against the transposed head.

Benchmark config 3: 16 and more consecutive calls of the delayed-scaling flow with a history of 16
(/root/reference/kernels/fp8.cu:67-142: record-quantize with the previous scale, then the history update), each
followed by the 1 x 128 / 128 x 128 block-scaled GEMM on that call's activations, the oracle's state stepping alongside."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, host, scalar, stream
from test_oracle_ce import reference_f64

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("V,check_rows", [(50304, 24), (128256, 12)])
def test_lm_head_chain(cf, dev, V, check_rows):
    rows, H = 2048, 4096
    case(f"LM head chain: {rows} rows, hidden {H}, vocabulary {V}")
    g = torch.Generator(device=dev).manual_seed(V)
    normed = torch.randn((rows, H), generator=g, device=dev).to(torch.bfloat16)
    head = (torch.randn((V, H), generator=g, device=dev) * 0.02).to(torch.bfloat16)
    labels = torch.randint(0, V, (rows,), device=dev, generator=g, dtype=torch.int32)
    labels[::9] = -100
    st = stream()
    z = lambda: scalar(0.0, dev)

    # Fp8Slot of the head: forward layout [V,H] and backward layout [H,V] from one amax (refresh_fp8_weights, :4694-4712)
    w_amax, w_s, w_d = z(), z(), z()
    fwd8 = torch.empty((V, H), dtype=torch.uint8, device=dev)
    bwd8 = torch.empty((H, V), dtype=torch.uint8, device=dev)
    cf.cf_fp8_refresh_weight(head, fwd8, bwd8, w_amax, w_s, w_d, H, V, 1, 1, st)
    # activations: per-tensor E4M3 (the first-use branch of fp8_quant_act: exact amax)
    a_amax, a_s, a_d = z(), z(), z()
    act8 = torch.empty((rows, H), dtype=torch.uint8, device=dev)
    cf.cf_fp8_amax_bf16(normed, normed.numel(), a_amax, st)
    cf.cf_fp8_scale_from_amax(a_amax, 448.0, a_s, a_d, st)
    cf.cf_fp8_quantize_e4m3(normed, act8, a_s, normed.numel(), st)
    # logits_chunk = act8 . fwd8^T
    logits = torch.empty((rows, V), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16(rows, V, H, act8, H, 0, a_d, fwd8, w_d, logits, V, st)
    # cross entropy, gradient as bf16 and as E5M2 under a scale known before the call (the steady-state branch)
    nv = torch.zeros(1, dtype=torch.int32, device=dev)
    cf.cf_cross_entropy_count_valid(labels, rows, nv, st)
    torch.cuda.synchronize()
    n_valid = int(nv)
    qscale = np.float32(57344.0 * n_valid / 2.0)
    qdescale = np.float32(1.0) / qscale
    grad = torch.empty_like(logits)
    g8 = torch.empty((rows, V), dtype=torch.uint8, device=dev)
    loss, g_amax = z(), z()
    cf.cf_cross_entropy_fwd_bwd_chunk_quant_e5m2(logits, labels, loss, grad, g8, scalar(float(qscale), dev), g_amax, rows, V, nv, st)
    # dW_lm_head[V,H] += grad_chunk^T . normed_c (bf16 operands, fp32 accumulation into the gradient buffer)
    g_head = torch.full((V, H), 0.5, dtype=torch.float32, device=dev)
    cf.cf_gemm_bf16_tn_accum_f32(V, H, rows, grad, V, normed, H, g_head, H, st)
    # d(normed) chunk = g8 . bwd8^T, K = vocabulary
    d_hidden = torch.empty((rows, H), dtype=torch.bfloat16, device=dev)
    cf.cf_fp8_gemm_nt_bf16(rows, H, V, g8, V, 1, scalar(float(qdescale), dev), bwd8, w_d, d_hidden, H, st)
    torch.cuda.synchronize()

    pick = np.sort(np.random.default_rng(V).choice(rows, check_rows, replace=False))
    pick[0], pick[-1] = 0, rows - 1
    pidx = torch.from_numpy(pick).to(dev)
    # weight layouts: the transposed bytes are the forward bytes transposed; a block against the oracle
    hb = bf16_bits(head[:300, :200])
    assert np.array_equal(host(fwd8[:300, :200]), orc.quantize_e4m3(hb, host(w_s)[0]))
    assert np.array_equal(host(bwd8[:200, :300]), host(fwd8[:300, :200]).T)
    assert np.array_equal(host(bwd8[:, V - 64:]), host(fwd8[V - 64:, :]).T)
    # activations bit-exact, logits at the GEMM bar (the last column tile ends inside a tile for V = 50304)
    nb = bf16_bits(normed[pidx])
    assert np.array_equal(host(act8[pidx]), orc.quantize_e4m3(nb, host(a_s)[0]))
    ref, absdot = orc.gemm_nt_ref(host(act8[pidx]), host(fwd8), host(a_d), host(w_d))
    orc.assert_gemm_close(orc.bf16_to_f32(bf16_bits(logits[pidx])).astype(np.float64), ref, absdot, what=f"logits V={V}")
    del ref, absdot
    # the loss head on the GPU's logits: gradient within an ulp of double precision, bytes exactly its quantization
    lb, lab = bf16_bits(logits[pidx]), host(labels)[pick]
    gref, _ = reference_f64(lb, lab, n_valid)
    gb = bf16_bits(grad[pidx])
    got = orc.bf16_to_f32(gb).astype(np.float64)
    assert np.all(np.abs(got - gref) <= orc.bf16_ulp(gref) + 1e-30)
    want8, _ = orc.quantize_record(gb.reshape(-1), qscale, np.float32(0.0), e5m2=True)
    assert np.array_equal(host(g8[pidx]).reshape(-1), want8)
    assert float(g_amax) == float(grad.float().abs().max())
    # the head's weight gradient on sampled vocabulary entries (the labels' own among them), in double
    vs = np.unique(np.concatenate([np.random.default_rng(1).choice(V, 40, replace=False), host(labels)[pick][host(labels)[pick] >= 0],
                                   [0, V - 1]]))
    vidx = torch.from_numpy(vs).to(dev)
    gcol = grad[:, vidx].float().double()                                   # [rows, picked]
    want = 0.5 + (gcol.T @ normed.double()).cpu().numpy()
    mass = (gcol.abs().T @ normed.double().abs()).cpu().numpy()
    gotw = host(g_head[vidx]).astype(np.float64)
    assert np.all(np.abs(gotw - want) <= 2.0 ** -22 * np.abs(want) + 16.0 * 2.0 ** -24 * mass + 1e-30), "g_lm_head"
    del g_head
    # the input gradient over K = vocabulary, E5M2 activations
    ref, absdot = orc.gemm_nt_ref(host(g8[pidx]), host(bwd8), [qdescale], host(w_d), a_e5m2=True)
    orc.assert_gemm_close(orc.bf16_to_f32(bf16_bits(d_hidden[pidx])).astype(np.float64), ref, absdot, what=f"d_hidden V={V}")
    # rows nobody sampled: every row of the result moved by a plausible amount (a skipped or doubled tile shows)
    mag = d_hidden.float().abs().mean(dim=1)
    valid = labels >= 0
    assert float(mag[~valid].max()) == 0.0
    med = float(mag[valid].median())
    assert float(mag[valid].min()) > 0.2 * med and float(mag[valid].max()) < 5.0 * med


def test_config3_sixteen_calls_with_the_history_advancing(cf, dev):
    case("config 3: 20 calls of record-quantize -> history (16) -> block-scaled GEMM, 4096 x 7168 x 7168")
    M, N, K, HIST, CALLS = 4096, 7168, 7168, 16, 20
    g = torch.Generator(device=dev).manual_seed(33)
    st = stream()
    w = (torch.randn((N, K), generator=g, device=dev) * 0.02).to(torch.bfloat16)
    kb = K // 128
    wq = torch.empty((N, K), dtype=torch.uint8, device=dev)
    ws = torch.empty((N // 128, kb), device=dev); wd = torch.empty((N // 128, kb), device=dev)
    cf.cf_fp8_quantize_block_128x128(w, N, K, wq, ws, wd, st)
    del w
    # the slot's device scalars, as alloc_act_slot leaves them, after one first-use call that seeds the scale
    amax, scale, descale = scalar(0.0, dev), scalar(0.0, dev), scalar(0.0, dev)
    history = torch.zeros(HIST, device=dev)
    cursor = torch.zeros(1, dtype=torch.int32, device=dev); count = torch.zeros(1, dtype=torch.int32, device=dev)
    oracle = orc.DelayedState(HIST)
    xq_pt = torch.empty((M, K), dtype=torch.uint8, device=dev)
    xq = torch.empty((M, K), dtype=torch.uint8, device=dev)
    xs = torch.empty((M, kb), device=dev); xd = torch.empty((M, kb), device=dev)
    C = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    rng = np.random.default_rng(3)
    wq_h, wd_h = host(wq), host(wd)
    scales = []
    for call in range(CALLS):
        # the activations' range drifts and jumps, so the history maximum moves in and out of the window
        gain = float(1.0 + 0.5 * np.sin(call / 2.0) + (3.0 if call in (2, 19) else 0.0))
        x = (torch.randn((M, K), generator=g, device=dev) * gain).to(torch.bfloat16)
        pick = np.sort(rng.choice(M, 3, replace=False))
        pidx = torch.from_numpy(pick).to(dev)
        if call == 0:
            cf.cf_fp8_amax_bf16(x, x.numel(), amax, st)
            cf.cf_fp8_scale_from_amax(amax, 448.0, scale, descale, st)
            torch.cuda.synchronize()
            s0, d0 = orc.scale_from_amax(orc.amax_bf16(bf16_bits(x)), 448.0)
            oracle.scale[0], oracle.descale[0] = s0, d0
            prev_scale = s0
            cf.cf_fp8_quantize_e4m3(x, xq_pt, scale, x.numel(), st)
            a = host(amax)[0]
        else:
            prev_scale = host(scale)[0]
            amax.zero_()
            cf.cf_fp8_quantize_e4m3_record(x, xq_pt, scale, amax, x.numel(), st)      # with the PREVIOUS call's scale
            torch.cuda.synchronize()
            a = host(amax)[0]
            assert a == orc.amax_bf16(bf16_bits(x))
        cf.cf_fp8_update_delayed_scale(amax, 448.0, scale, descale, history, HIST, cursor, count, st)
        oracle.update(a, 448.0)
        # this call's activations under 1 x 128 scales, and the block-scaled GEMM on them
        cf.cf_fp8_quantize_block_1x128(x, M, K, xq, xs, xd, st)
        cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wq, K, wd, 2, 0, None, None, None, C, N, 0, st)
        torch.cuda.synchronize()
        # state: every word of the ring, cursor wrapping at 16, count saturating, scale from the window's maximum
        assert host(scale)[0] == oracle.scale[0] and host(descale)[0] == oracle.descale[0], call
        assert np.array_equal(host(history), oracle.history[:HIST]), call
        assert int(cursor) == int(oracle.cursor[0]) == (call + 1) % HIST and int(count) == int(oracle.count[0]) == min(call + 1, HIST)
        # bytes of the per-tensor path (previous scale) and of the block path on sampled rows
        xb = bf16_bits(x[pidx])
        assert np.array_equal(host(xq_pt[pidx]), orc.quantize_e4m3(xb, prev_scale)), call
        oq, _, od = orc.quantize_block_1x128(xb)
        assert np.array_equal(host(xq[pidx]), oq) and np.array_equal(host(xd[pidx]), od), call
        ref, absdot = orc.gemm_nt_ref(oq, wq_h, od, wd_h, scale_mode=2)
        orc.assert_gemm_close(orc.bf16_to_f32(bf16_bits(C[pidx])).astype(np.float64), ref, absdot, what=f"config 3 call {call}")
        scales.append(float(host(scale)[0]))
    # the jump of call 2 leaves the window of sixteen with call 18: the scale recovers there and not before
    assert scales[18] > 2.0 * scales[17] and max(scales[2:18]) <= scales[2] * 1.0000001
