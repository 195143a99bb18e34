"""Helpers for the GPU parity tests: torch is used only for device memory and copies."""
import numpy as np
import torch

from turbogpt_amd.bridge import check, library


def rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-12))


def to_bf16_device(a):
    """float array -> (device bf16 tensor, the same values as float32 on the host)."""
    t = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).bfloat16()
    return t.cuda(), t.float().numpy()


def host(t):
    return t.float().cpu().numpy()


def stream():
    return torch.cuda.current_stream().cuda_stream


def sync():
    torch.cuda.synchronize()
