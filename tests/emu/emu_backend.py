"""Test-only: the package's operators bound to the CPU build of the kernel sources (libgdn_emu.so).

This exists so that kernel indexing, LDS use and barriers can be checked on a machine without a GPU, with
guard pages instead of GPU faults.  The shipped package never imports this module."""
import contextlib
import ctypes
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "mindspeed-mm_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

from mindspeed_mm_amd._lib import GdnLibrary  # noqa: E402
from mindspeed_mm_amd.ops import GdnOps  # noqa: E402

_ops = None


def emu_ops() -> GdnOps:
    global _ops
    if _ops is None:
        from . import build_emu
        path = build_emu.build()
        _ops = GdnOps(GdnLibrary(path, "cpu"))
        _ops.lib.cdll.emu_guard_alloc.restype = ctypes.c_void_p
        _ops.lib.cdll.emu_guard_alloc.argtypes = [ctypes.c_size_t, ctypes.c_int]
    return _ops


_keep = []


def guarded(t: torch.Tensor, at_end: bool = True) -> torch.Tensor:
    """Copy of `t` whose storage ends (or starts) flush against an inaccessible page."""
    lib = emu_ops().lib.cdll
    t = t.contiguous()
    nbytes = max(t.numel() * t.element_size(), 1)
    p = lib.emu_guard_alloc(nbytes, 1 if at_end else 0)
    buf = (ctypes.c_uint8 * nbytes).from_address(p)
    _keep.append(buf)
    raw = torch.frombuffer(buf, dtype=torch.uint8, count=nbytes)
    out = raw[: t.numel() * t.element_size()].view(t.dtype).view(t.shape)
    out.copy_(t)
    return out


@contextlib.contextmanager
def guarded_outputs():
    """While active, every CPU tensor made by torch.empty (the operators allocate their outputs, gradients and
    workspaces with it) ends flush against an inaccessible page, so that a kernel reading or writing past the end of
    an output is a SIGSEGV here."""
    real = torch.empty

    def empty(*size, **kw):
        t = real(*size, **kw)
        return guarded(t) if t.device.type == "cpu" and t.numel() > 0 and not kw.get("pin_memory") else t
    torch.empty = empty
    try:
        yield
    finally:
        torch.empty = real
