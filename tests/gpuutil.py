"""Helpers for the GPU parity tests: torch is used only for device memory and the
stream; every computation goes through the C ABI (cavs_amd.hip)."""
import ctypes as C

import numpy as np
import torch

from cavs_amd import hip


def stream():
    return torch.cuda.current_stream().cuda_stream


# Device tensors made by dev() stay referenced until release() so that a raw address
# taken from a temporary (P(devf(x)) inside a call expression) never outlives its memory.
_KEEP = []


def release():
    torch.cuda.synchronize()
    _KEEP.clear()


def dev(a, dtype=None):
    if a is None:
        return None
    a = np.ascontiguousarray(a, dtype=dtype or np.asarray(a).dtype)
    t = torch.from_numpy(a).cuda()
    _KEEP.append(t)
    return t


def devf(a):
    return dev(a, np.float32)


def devi(a):
    return dev(a, np.int32)


def zeros(*shape, fill=None):
    t = torch.zeros(*shape, dtype=torch.float32, device="cuda")
    if fill is not None:
        t.fill_(fill)
    _KEEP.append(t)
    return t


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def P(t):
    return hip.ptr(t)


def call(name, *args):
    print(f"[abi] {name}", flush=True)
    hip.call(name, *args)
