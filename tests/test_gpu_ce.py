"""GPU: chunked cross-entropy and its fusion with the E5M2 quantize of the gradient, through the C ABI, against
the CPU oracle and a double-precision softmax (reference: kernels/cross_entropy.cu:201-305, src/trainer.cu:8015-8060).
exp / log are hardware units on the GPU and libm on the CPU: gradients are compared to one bf16 ulp; the fp8
bytes are compared exactly against the quantization of the gradient the kernel itself wrote."""
import numpy as np
import pytest
import torch

import oracle_lib as orc
from gpu_util import bf16_bits, case, dev_bf16, host, scalar, stream
from test_oracle_ce import reference_f64

pytestmark = pytest.mark.gpu


def make(rows, V, seed, ignore_every=4):
    rng = np.random.default_rng(seed)
    logits = orc.bf16_from_f32((rng.standard_normal((rows, V)) * 4.0).astype(np.float32))
    labels = rng.integers(0, V, rows).astype(np.int32)
    if rows > 2:
        labels[::ignore_every] = -100
    return logits, labels


def check_grad(got_bits, logits, labels, n_valid):
    ref, ref_loss = reference_f64(logits, labels, n_valid)
    g = orc.bf16_to_f32(got_bits).astype(np.float64)
    assert np.all(np.abs(g - ref) <= 1.0 * orc.bf16_ulp(ref) + 1e-30), "more than one bf16 ulp from the exact gradient"
    want, _ = orc.cross_entropy_fwd_bwd_chunk(logits, labels, n_valid)
    w = orc.bf16_to_f32(want).astype(np.float64)
    assert np.all(np.abs(g - w) <= 1.0 * orc.bf16_ulp(w) + 1e-30), "more than one bf16 ulp from the oracle"
    assert np.all(got_bits[labels < 0] == 0)
    return ref_loss


@pytest.mark.parametrize("rows,V", [(1, 8), (9, 1000), (33, 4096), (7, 4099), (5, 32000), (3, 32768), (2, 50264), (2, 50257), (2, 128256), (2, 131072), (2, 131080)])
def test_cross_entropy_chunk(cf, dev, rows, V):
    case(f"cross entropy rows={rows} V={V}")
    logits, labels = make(rows, V, rows * 13 + V)
    n_valid_all = 57                                   # the chunk is part of a larger batch
    lab = torch.from_numpy(labels).to(dev)
    nv = torch.zeros(1, dtype=torch.int32, device=dev)
    cf.cf_cross_entropy_count_valid(lab, rows, nv, stream())
    torch.cuda.synchronize()
    assert int(nv) == int((labels >= 0).sum()) == orc.cross_entropy_count_valid(labels)
    nv.fill_(n_valid_all)
    x = dev_bf16(logits, dev)
    grad = torch.empty_like(x)
    loss = scalar(0.25, dev)
    cf.cf_cross_entropy_fwd_bwd_chunk(x, lab, loss, grad, rows, V, nv, stream())
    torch.cuda.synchronize()
    ref_loss = check_grad(bf16_bits(grad), logits, labels, n_valid_all)
    assert abs((float(loss) - 0.25) - ref_loss) <= 2e-5 * abs(ref_loss) + 1e-7
    # in place, as the trainer calls it
    cf.cf_cross_entropy_fwd_bwd_chunk(x, lab, loss, x, rows, V, nv, stream())
    torch.cuda.synchronize()
    assert torch.equal(x.view(torch.int16), grad.view(torch.int16))


@pytest.mark.parametrize("rows,V", [(12, 4096), (6, 32000), (5, 1001), (2, 40000), (3, 128256), (2, 131080)])
def test_cross_entropy_chunk_fused_with_e5m2_quantize(cf, dev, rows, V):
    case(f"cross entropy + e5m2 quantize rows={rows} V={V}")
    logits, labels = make(rows, V, rows * 17 + V)
    n_valid = int((labels >= 0).sum())
    lab = torch.from_numpy(labels).to(dev)
    nv = torch.tensor([n_valid], dtype=torch.int32, device=dev)
    x = dev_bf16(logits, dev)
    grad = torch.empty_like(x)
    plain = torch.empty_like(x)
    g8 = torch.empty((rows, V), dtype=torch.uint8, device=dev)
    loss, loss2 = scalar(0.0, dev), scalar(0.0, dev)
    amax = scalar(0.0, dev)
    qscale = np.float32(57344.0 * n_valid / 2.0)      # gradients are at most 1 / n_valid in magnitude
    cf.cf_cross_entropy_fwd_bwd_chunk(x, lab, loss2, plain, rows, V, nv, stream())
    cf.cf_cross_entropy_fwd_bwd_chunk_quant_e5m2(x, lab, loss, grad, g8, scalar(float(qscale), dev), amax, rows, V, nv, stream())
    torch.cuda.synchronize()
    gb = bf16_bits(grad)
    assert np.array_equal(gb, bf16_bits(plain))                          # the same gradient as the plain form
    check_grad(gb, logits, labels, n_valid)
    want8, want_amax = orc.quantize_record(gb.reshape(-1), qscale, np.float32(0.0), e5m2=True)
    assert np.array_equal(host(g8).reshape(-1), want8)                   # exactly the quantization of that gradient
    assert host(amax)[0] == want_amax
    assert abs(float(loss) - float(loss2)) <= 1e-6 * abs(float(loss2))


def test_cross_entropy_full_vocabulary_chunk(cf, dev):
    """A trainer-sized chunk: 2048 rows x 32000 logits, rows sampled against double precision."""
    rows, V = 2048, 32000
    case("cross entropy 2048 x 32000")
    g = torch.Generator(device=dev); g.manual_seed(9)
    x = (torch.randn(rows, V, device=dev, generator=g) * 3.0).to(torch.bfloat16)
    labels = torch.randint(0, V, (rows,), device=dev, generator=g, dtype=torch.int32)
    labels[::7] = -100
    nv = torch.zeros(1, dtype=torch.int32, device=dev)
    cf.cf_cross_entropy_count_valid(labels, rows, nv, stream())
    grad = torch.empty_like(x)
    g8 = torch.empty((rows, V), dtype=torch.uint8, device=dev)
    loss, amax = scalar(0.0, dev), scalar(0.0, dev)
    cf.cf_cross_entropy_fwd_bwd_chunk_quant_e5m2(x, labels, loss, grad, g8, scalar(1.0e6, dev), amax, rows, V, nv, stream())
    torch.cuda.synchronize()
    n_valid = int(nv)
    assert n_valid == int((labels >= 0).sum())
    pick = np.arange(0, rows, 97)
    lb, lab = bf16_bits(x)[pick], host(labels)[pick]
    ref, _ = reference_f64(lb, lab, n_valid)
    got = orc.bf16_to_f32(bf16_bits(grad)[pick]).astype(np.float64)
    assert np.all(np.abs(got - ref) <= orc.bf16_ulp(ref) + 1e-30)
    # the whole batch's loss against a float64 log-softmax on the device
    xl = x.double()
    lse = torch.logsumexp(xl, dim=1)
    valid = labels >= 0
    p_label = torch.exp(xl[valid, labels[valid].long()] - lse[valid])
    ref_loss = float(-torch.log(p_label + 1e-9).sum() / n_valid)          # the reference's epsilon inside the log
    assert abs(float(loss) - ref_loss) <= 2e-5 * ref_loss
    assert float(amax) == float(grad.float().abs().max())


def test_cross_entropy_argument_errors(cf):
    assert cf.raw_cf_cross_entropy_fwd_bwd_chunk(None, None, None, None, 4, 8, None, None) == -1
    assert cf.raw_cf_cross_entropy_fwd_bwd_chunk(None, None, None, None, 0, 8, None, None) == 0
    assert cf.raw_cf_cross_entropy_fwd_bwd_chunk(None, None, None, None, -1, 8, None, None) == -1
    assert cf.raw_cf_cross_entropy_count_valid(None, 0, None, None) == -1
