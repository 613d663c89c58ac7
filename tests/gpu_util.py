"""Small helpers for the GPU parity tests: numpy <-> device tensors, stream handle."""
import numpy as np
import torch


def stream():
    return torch.cuda.current_stream().cuda_stream


def dev_bf16(bits, dev):
    """uint16 bit patterns -> bf16 device tensor of the same shape."""
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.bfloat16)


def bf16_bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def dev_arr(a, dev):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(dev)
    return torch.from_numpy(a).to(dev)


def host(t):
    return t.cpu().numpy()


def scalar(v, dev, dtype=torch.float32):
    return torch.tensor([v], dtype=dtype, device=dev)


def case(msg):
    """Names the case before a GPU step so a fault can be attributed."""
    print(f"[gpu-case] {msg}", flush=True)
