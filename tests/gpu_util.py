"""Helpers shared by the GPU parity tests (torch is only the carrier of device memory)."""
import numpy as np
import torch


def require_gpu():
    if not torch.cuda.is_available():
        raise RuntimeError("GPU test run without a GPU")


def dev(a):
    """numpy (float32 / uint16 bf16 bits / uint32 / int32) -> contiguous GPU tensor."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    return torch.from_numpy(a).cuda()


def host(t):
    """GPU tensor -> numpy; bf16 comes back as uint16 bit patterns."""
    torch.cuda.synchronize()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def rel_err(a, b):
    """max |a-b| / max |b|  (the tolerance metric used for conv and softmax)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    den = np.max(np.abs(b))
    return float(np.max(np.abs(a - b)) / (den if den > 0 else 1.0))
