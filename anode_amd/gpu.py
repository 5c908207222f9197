"""Calling the C ABI with torch-ROCm tensors.

torch is used for device memory and streams only; every computation goes
through the entry points of libanode_routines_gpu.so.  `call()` passes
arguments exactly as anode's Rust callers do (src/ops_gpu.rs:670-679): dims as
u32, device pointers, a host KernelConfig*, the stream handle.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ._lib import KernelConfig, load

# gpudevicemem's per-connection values are not visible in the reference; any
# power-of-two block size satisfies the reduction entry points' contract.
DEFAULT_CONFIG = KernelConfig(1024, 1024)


def _as_arg(a):
    if isinstance(a, torch.Tensor):
        if not a.is_cuda:
            raise ValueError("the ABI takes device pointers: tensor is not on the GPU")
        if not a.is_contiguous():
            raise ValueError("the ABI takes packed arrays: tensor is not contiguous")
        return a.data_ptr()
    return a


def call(name: str, *args, cfg: Optional[KernelConfig] = None, stream: Optional[int] = None):
    """Invoke entry point `name`; `args` are everything before (cfg, stream)."""
    lib = load()
    restype, argtypes, names = lib.prototypes[name]
    if len(args) != len(argtypes) - 2:
        raise TypeError(f"{name} takes {len(argtypes) - 2} arguments before (cfg, stream): {names[:-2]}")
    if cfg is None:
        cfg = DEFAULT_CONFIG
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    lib.symbol(name)(*[_as_arg(a) for a in args], ctypes.byref(cfg), ctypes.c_void_p(stream))


def take_last_error() -> int:
    return int(load().symbol("anode_gpu_take_last_error")())


def set_tuning(knob: int, value: int) -> int:
    return int(load().cdll.anode_gpu_set_tuning(knob, value))
