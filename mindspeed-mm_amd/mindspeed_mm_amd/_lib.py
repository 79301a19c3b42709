"""ctypes binding of the C ABI declared in include/gdn_mi355x.h.

There is no fallback: if libgdn_mi355x.so is missing or cannot be loaded, importing an op raises."""
import ctypes
import os
from ctypes import c_float, c_int, c_int64, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libgdn_mi355x.so")

P, I, L, F = c_void_p, c_int, c_int64, c_float

# name -> (restype, argtypes); must mirror include/gdn_mi355x.h (tests/test_capi_symbols.py checks it)
SIGNATURES = {
    "gdn_chunk_workspace_bytes": (L, [I] * 9),
    "gdn_chunk_fwd": (I, [P] * 10 + [L] + [I] * 7 + [F, I, I, P]),
    "gdn_chunk_bwd": (I, [P] * 16 + [L] + [I] * 7 + [F, I, I, P]),
    "gdn_chunk_fwd_strided": (I, [P] * 3 + [L] * 3 + [P] * 7 + [L] + [I] * 7 + [F, I, I, I, P]),
    "gdn_chunk_fwd_norm_strided": (I, [P] * 3 + [L] * 3 + [P] * 11 + [L] + [I] * 7 + [F, F, I, I, I, I, P]),
    "gdn_chunk_bwd_strided": (I, [P] * 3 + [L] * 3 + [P] * 9 + [L] * 3 + [P] * 4 + [L] + [I] * 7 + [F, I, I, I, P]),
    "gdn_chunk_bwd_parts": (I, [P] * 3 + [L] * 3 + [P] * 9 + [L] * 3 + [P] * 4 + [L, P, L] + [I] * 9 + [F, I, I, I, P]),
    "gdn_recurrent_fwd": (I, [P] * 8 + [I] * 6 + [F, I, I, P]),
    "gdn_recurrent_fwd_packed": (I, [P] * 9 + [I] * 6 + [F, I, I, P]),
    "gdn_recurrent_fwd_qkv": (I, [P, L] + [P] * 7 + [I] * 6 + [F, I, I, I, P]),
    "gdn_conv1d_fwd": (I, [P] * 8 + [I] * 7 + [P]),
    "gdn_conv1d_bwd_workspace_bytes": (L, [I] * 4),
    "gdn_conv1d_bwd": (I, [P] * 12 + [L] + [I] * 7 + [P]),
    "gdn_conv1d_update": (I, [P] * 5 + [I] * 7 + [P]),
    "gdn_rmsnorm_gated_fwd": (I, [P] * 5 + [L, I, F, I, I, I, P]),
    "gdn_rmsnorm_gated_bwd_workspace_bytes": (L, [L, I]),
    "gdn_rmsnorm_gated_bwd": (I, [P] * 9 + [L, L, I, I, I, I, P]),
    "gdn_gate_fwd": (I, [P] * 6 + [L, I, I, I, P]),
    "gdn_gate_bwd_workspace_bytes": (L, [L, I]),
    "gdn_gate_bwd": (I, [P] * 11 + [L, L, I, I, I, P]),
    "gdn_gate_bwd_noalloc": (I, [P] * 10 + [L, I, I, I, P]),
    "gdn_kda_workspace_bytes": (L, [I] * 8),
    "gdn_kda_fwd": (I, [P] * 12 + [L] + [I] * 6 + [F, I, I, I, F, I, I, I, I, I, P]),
    "gdn_kda_intermediate_states": (I, [P, L, P, P, L] + [I] * 8 + [P]),
    "gdn_kda_bwd": (I, [P] * 18 + [L] + [I] * 6 + [F, I, I, I, F, I, I, I, I, I, P]),
    "gdn_profile_enable": (I, [I]),
    "gdn_profile_kernel_count": (I, []),
    "gdn_profile_kernel_name": (ctypes.c_char_p, [I]),
    "gdn_profile_collect": (I, [P, P]),
}

DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}

_ERRORS = {
    -1: "null pointer for a required tensor",
    -2: "inconsistent shapes",
    -3: "unsupported size (K must be 64 or 128 (256 for decode), V a multiple of 64, conv width 1..8, D % 8 == 0, "
        "norm rows of 4/8/16/32/64 16-byte pieces)",
    -4: "unsupported dtype",
    -5: "workspace too small or misaligned",
    -6: "token stride not a multiple of 16 bytes or shorter than a token's heads, or a pointer not 16-byte aligned",
}


class GdnLibrary:
    """A loaded kernel library plus the device type its pointers live on."""

    def __init__(self, path: str, device_type: str = "cuda"):
        if not os.path.exists(path):
            raise RuntimeError(
                f"HIP kernel library not found at {path}; build it with "
                "`python -c 'import __graft_entry__ as g; g.build()'` (needs hipcc). There is no fallback path.")
        self.path = path
        self.device_type = device_type
        self.cdll = ctypes.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(self.cdll, name)
            fn.restype, fn.argtypes = res, args
            setattr(self, name, fn)

    def stream(self):
        if self.device_type == "cuda":
            return torch.cuda.current_stream().cuda_stream
        return None

    def check(self, code: int, what: str):
        if code == 0:
            return
        if code < 0:
            raise ValueError(f"{what}: {_ERRORS.get(code, 'invalid argument')} (code {code})")
        raise RuntimeError(f"{what}: HIP error {code}")


def kernel_timings(lib: "GdnLibrary"):
    """Collect the per-kernel event timings recorded since profiling was enabled:
    {kernel name: (total milliseconds, launches)}."""
    n = lib.gdn_profile_kernel_count()
    ms = (ctypes.c_double * n)()
    cnt = (ctypes.c_int64 * n)()
    rc = lib.gdn_profile_collect(ctypes.cast(ms, c_void_p), ctypes.cast(cnt, c_void_p))
    if rc != 0:
        raise RuntimeError("gdn_profile_collect failed")
    return {lib.gdn_profile_kernel_name(i).decode(): (ms[i], cnt[i]) for i in range(n) if cnt[i] > 0}


_default = None


def default_library() -> GdnLibrary:
    global _default
    if _default is None:
        _default = GdnLibrary(LIB_PATH, "cuda")
    return _default


def ptr(t):
    return None if t is None else t.data_ptr()
