"""Helpers shared by the GPU tests: numpy <-> device tensors (uint32 kept as int32 bit patterns)."""
import numpy as np
import torch


def dev(a, device):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype == torch.uint32:
        t = t.view(torch.int32)
    return t.to(device)


def host_u32(t):
    return t.cpu().numpy().view(np.uint32)


def stream():
    return torch.cuda.current_stream().cuda_stream
