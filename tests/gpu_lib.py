"""Shared helpers for the GPU tests: loads the C-ABI library, moves numpy arrays to the device in
the library's storage type and back. torch is used only as a device allocator / dtype converter."""
import ctypes as C
import importlib.util
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def package():
    if "llmc_amd" in sys.modules:
        return sys.modules["llmc_amd"]
    spec = importlib.util.spec_from_file_location("llmc_amd", os.path.join(ROOT, "llm.c_amd", "__init__.py"))
    m = importlib.util.module_from_spec(spec)
    sys.modules["llmc_amd"] = m
    spec.loader.exec_module(m)
    return m


_inited = set()


def lib(precision):
    L = package().load(precision)
    if precision not in _inited:
        L.llmk_init(0)
        _inited.add(precision)
    return L


def torch_dtype(precision):
    import torch
    return torch.bfloat16 if precision == "bf16" else torch.float32


def dev(x, precision=None, dtype=None):
    """numpy -> cuda tensor. precision given: cast to the library's storage type."""
    import torch
    t = torch.from_numpy(np.ascontiguousarray(x)).cuda()
    if precision is not None:
        t = t.to(torch_dtype(precision))
    elif dtype is not None:
        t = t.to(dtype)
    return t.contiguous()


def host(t):
    """cuda tensor -> float32 numpy (int tensors keep their type)"""
    import torch
    torch.cuda.synchronize()
    if t.dtype in (torch.bfloat16, torch.float16):
        t = t.float()
    return t.cpu().numpy()


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def rounded(x, precision):
    """what the device holds after storing fp32 numpy data x in the storage type, as fp32 numpy"""
    if precision == "fp32":
        return np.ascontiguousarray(x, dtype=np.float32)
    import torch
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16).float().numpy()


def sync():
    import torch
    torch.cuda.synchronize()


def check_no_error(L):
    msg = L.llmk_last_error().decode()
    assert msg == "", msg
