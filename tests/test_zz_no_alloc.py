"""gdn_gate_bwd_noalloc (the entry point that allocates nothing: its partial sums live in a buffer inside the
library) against gdn_gate_bwd with a caller-provided workspace, through the C ABI: identical bits, on two calls in
a row, the second with a smaller input (the buffer then still holds the first call's partial sums)."""
import pytest
import torch

from mindspeed_mm_amd._lib import DTYPE_CODE, default_library, ptr

pytestmark = pytest.mark.gpu


def _inputs(tokens, Hv, dtype, seed, param_dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    dev = "cuda"
    a = torch.randn(tokens, Hv, generator=g).to(dev, dtype)
    b = torch.randn(tokens, Hv, generator=g).to(dev, dtype)
    A_log = torch.rand(Hv, generator=g).mul(2.7).to(dev, param_dtype)
    dt_bias = torch.rand(Hv, generator=g).mul(2).sub(4).to(dev, param_dtype)
    dg = torch.randn(tokens, Hv, generator=g).to(dev)
    dbeta = torch.randn(tokens, Hv, generator=g).to(dev, dtype)
    return a, b, A_log, dt_bias, dg, dbeta


def _run(lib, which, a, b, A_log, dt_bias, dg, dbeta):
    tokens, Hv = a.shape
    da, db = torch.empty_like(a), torch.empty_like(b)
    dA = torch.empty(Hv, dtype=torch.float32, device=a.device)
    dd = torch.empty(Hv, dtype=torch.float32, device=a.device)
    code, pcode = DTYPE_CODE[a.dtype], DTYPE_CODE[A_log.dtype]
    if which == "workspace":
        nbytes = lib.gdn_gate_bwd_workspace_bytes(tokens, Hv)
        ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=a.device)
        rc = lib.gdn_gate_bwd(ptr(a), ptr(b), ptr(A_log), ptr(dt_bias), ptr(dg), ptr(dbeta), ptr(da), ptr(db), ptr(dA),
                              ptr(dd), ptr(ws), nbytes, tokens, Hv, code, pcode, lib.stream())
    else:
        rc = lib.gdn_gate_bwd_noalloc(ptr(a), ptr(b), ptr(A_log), ptr(dt_bias), ptr(dg), ptr(dbeta), ptr(da), ptr(db),
                                      ptr(dA), ptr(dd), tokens, Hv, code, pcode, lib.stream())
    assert rc == 0, rc
    torch.cuda.synchronize()
    return da, db, dA, dd


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_no_alloc_entry_matches_workspace_entry(dtype):
    lib = default_library()
    for tokens, Hv, seed in ((40000, 32, 1), (777, 32, 2), (5000, 128, 3), (3, 8, 4)):   # large first, then smaller
        x = _inputs(tokens, Hv, dtype, seed)
        want = _run(lib, "workspace", *x)
        got = _run(lib, "noalloc", *x)
        for w, g_, name in zip(want, got, ("da", "db", "dA_log", "ddt_bias")):
            assert torch.equal(w, g_), (name, tokens, Hv)


def test_no_alloc_entry_with_half_precision_parameters_and_odd_head_counts():
    """A_log and dt_bias in bf16 (the layer's parameters under a bf16 policy), and head counts that do not divide the
    workgroup size: again two calls in a row per case, the second smaller."""
    lib = default_library()
    for tokens, Hv, seed in ((9000, 48, 6), (130, 48, 7), (2049, 6, 8), (64, 6, 9)):
        x = _inputs(tokens, Hv, torch.bfloat16, seed, param_dtype=torch.bfloat16)
        want = _run(lib, "workspace", *x)
        got = _run(lib, "noalloc", *x)
        for w, g_, name in zip(want, got, ("da", "db", "dA_log", "ddt_bias")):
            assert torch.equal(w, g_), (name, tokens, Hv)


def test_no_alloc_entry_rejects_what_its_buffer_cannot_hold():
    lib = default_library()
    x = _inputs(16, 256, torch.bfloat16, 5)
    a, b, A_log, dt_bias, dg, dbeta = x
    da, db = torch.empty_like(a), torch.empty_like(b)
    dA = torch.empty(256, dtype=torch.float32, device="cuda")
    rc = lib.gdn_gate_bwd_noalloc(ptr(a), ptr(b), ptr(A_log), ptr(dt_bias), ptr(dg), ptr(dbeta), ptr(da), ptr(db),
                                  ptr(dA), ptr(dA), 16, 256, 1, 0, lib.stream())
    assert rc == -3
    with pytest.raises(ValueError, match="unsupported size"):
        lib.check(rc, "gdn_gate_bwd_noalloc")
