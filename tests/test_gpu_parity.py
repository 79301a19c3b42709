"""GPU parity tests proper: the shipped HIP library (through the package's C-ABI binding) against the CPU
oracle on the same seeded inputs.  Run with `-m gpu` on an MI355X."""
import pytest
import torch

from tests import parity as P

pytestmark = pytest.mark.gpu
BF, F32 = torch.bfloat16, torch.float32


@pytest.fixture(scope="module")
def ops():
    from mindspeed_mm_amd.ops import _default_ops
    return _default_ops()


def test_library_is_the_hip_build(ops):
    assert ops.lib.device_type == "cuda" and ops.lib.path.endswith("libgdn_mi355x.so")


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V", [
    (F32, 2, 3, 1, 2, 64, 64), (BF, 4, 1, 16, 32, 128, 128), (F32, 3, 1, 2, 4, 128, 128), (BF, 2, 64, 2, 4, 128, 128),
    (F32, 1, 5, 1, 1, 128, 192), (BF, 1, 4, 1, 2, 256, 128), (BF, 2, 2, 1, 1, 64, 256),
])
def test_recurrent(ops, dtype, B, T, Hqk, Hv, K, V):
    print(f"recurrent {dtype} B{B} T{T} Hqk{Hqk} Hv{Hv} K{K} V{V}", flush=True)
    P.check_recurrent(ops, "cuda", B, T, Hqk, Hv, K, V, dtype)
    P.check_recurrent(ops, "cuda", B, T, Hqk, Hv, K, V, dtype, l2=False, with_state=False)


def test_recurrent_inplace_state(ops):
    x = P.gdn_inputs(2, 1, 2, 4, 128, 128, BF, seed=3)
    d = {n: t.cuda() for n, t in x.items()}
    o1, s1 = ops.fused_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=d["h0"],
                                                  output_final_state=True, use_qk_l2norm_in_kernel=True)
    st = d["h0"].clone()
    o2, s2 = ops.fused_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=st,
                                                  output_final_state=True, use_qk_l2norm_in_kernel=True,
                                                  inplace_state=True)
    assert s2.data_ptr() == st.data_ptr()
    assert torch.equal(o1, o2) and torch.equal(s1, st)


CHUNK_CASES = [
    # dtype, B, T, Hqk, Hv, K, V, l2, cu
    (F32, 1, 512, 4, 4, 64, 64, False, None),                    # BASELINE config 0 shape
    (F32, 2, 100, 2, 4, 128, 128, True, None),
    (BF, 1, 128, 4, 4, 64, 64, False, None),                     # reference test table rows
    (BF, 2, 256, 4, 4, 64, 64, False, None),
    (BF, 1, 128, 8, 8, 128, 128, True, None),
    (BF, 1, 360, 32, 32, 128, 128, True, None),
    (BF, 1, 1121, 2, 2, 128, 128, True, [0, 112, 209, 240, 281, 489, 523, 566, 689, 721, 785, 837, 985, 1071, 1121]),
    (BF, 1, 1024, 4, 4, 128, 128, True,
     [0, 112, 209, 240, 281, 489, 523, 566, 689, 721, 785, 837, 985] + list(range(986, 1025))),
    (BF, 1, 808, 2, 4, 128, 128, True, [0] + list(range(804, 809))),
    (BF, 3, 195, 2, 4, 128, 128, True, None),
    (BF, 1, 256, 1, 2, 128, 256, True, None),                    # wide value heads (config 4 head shape)
    (F32, 1, 96, 1, 2, 128, 192, True, [0, 1, 38, 96]),
]


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu", CHUNK_CASES)
def test_chunk_forward(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu):
    print(f"chunk fwd {dtype} B{B} T{T} Hqk{Hqk} Hv{Hv} K{K} V{V} l2={l2} varlen={cu is not None}", flush=True)
    P.check_chunk(ops, "cuda", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu", CHUNK_CASES)
def test_chunk_backward(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu):
    print(f"chunk bwd {dtype} B{B} T{T} Hqk{Hqk} Hv{Hv} K{K} V{V} l2={l2} varlen={cu is not None}", flush=True)
    P.check_chunk(ops, "cuda", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, backward=True)


def test_chunk_backward_without_initial_state(ops):
    P.check_chunk(ops, "cuda", 1, 200, 2, 2, 128, 128, BF, backward=True, with_h0=False)


@pytest.mark.parametrize("dtype,B,T,D,W,cu", [
    (F32, 2, 37, 16, 4, None), (BF, 1, 300, 64, 4, [0, 1, 3, 130, 131, 300]), (F32, 1, 9, 8, 3, [0, 2, 9]),
    (torch.float16, 2, 5, 8, 2, None), (F32, 3, 2, 8, 4, None), (BF, 2, 1024, 512, 4, None),
    (F32, 1, 2000, 256, 4, [0, 255, 257, 1200, 2000]),
])
def test_conv1d(ops, dtype, B, T, D, W, cu):
    print(f"conv1d {dtype} B{B} T{T} D{D} W{W} varlen={cu is not None}", flush=True)
    P.check_conv(ops, "cuda", B, T, D, W, dtype, cu=cu, residual=True)
    P.check_conv(ops, "cuda", B, T, D, W, dtype, cu=cu, bias=False, state=False, activation=None)


@pytest.mark.parametrize("dtype,B,T,D,W", [(F32, 2, 1, 16, 4), (BF, 3, 5, 8, 4), (BF, 16, 1, 8192, 4)])
def test_conv1d_update(ops, dtype, B, T, D, W):
    P.check_conv_update(ops, "cuda", B, T, D, W, dtype)


@pytest.mark.parametrize("dtype,shape,N,wdt", [
    (F32, (3, 5), 64, None), (BF, (70,), 128, None), (BF, (2, 9), 256, torch.float32), (F32, (33,), 16, None),
    (BF, (5,), 512, None), (F32, (4,), 256, None), (BF, (2, 1000, 32), 128, None),
])
def test_rms_norm_gated(ops, dtype, shape, N, wdt):
    P.check_rms_norm_gated(ops, "cuda", shape, N, dtype, weight_dtype=wdt)


def test_rms_norm_gated_module_matches_functional(ops):
    from mindspeed_mm_amd import RMSNormGated
    m = RMSNormGated(128).to("cuda", BF)
    x = torch.randn(4, 7, 128, device="cuda", dtype=BF)
    z = torch.randn(4, 7, 128, device="cuda", dtype=BF)
    assert torch.equal(m(x, z), ops.rms_norm_gated(x, z, m.weight, 1e-6))
    with pytest.raises(ValueError):
        ops.rms_norm_gated(x, None, m.weight)
    with pytest.raises(ValueError):
        ops.rms_norm_gated(x[..., :100].contiguous(), z[..., :100].contiguous(), m.weight[:100])

