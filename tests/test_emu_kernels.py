"""CPU checks of the HIP kernel sources themselves, compiled for the host against a fiber-based stand-in
for the HIP runtime (tests/emu).  Same operators, same C ABI, same oracle as the GPU parity tests, on
small shapes; buffers sit against guard pages so an out-of-range index is a SIGSEGV here rather than a
GPU fault.  The shipped library is not involved: these tests prove indexing/synchronisation logic, the
`-m gpu` tests prove the device build."""
import pytest
import torch

from tests import parity as P
from tests.emu.emu_backend import emu_ops, guarded, guarded_outputs

BF, F32 = torch.bfloat16, torch.float32


@pytest.fixture(scope="module")
def ops():
    return emu_ops()


@pytest.fixture(autouse=True)
def _outputs_against_guard_pages():
    """Every test here also runs with what the operators allocate themselves (outputs, gradients, workspaces)
    flush against guard pages, not only the inputs the test hands in."""
    with guarded_outputs():
        yield


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V", [
    (F32, 2, 3, 1, 2, 64, 64), (BF, 2, 2, 2, 4, 128, 128), (F32, 1, 1, 1, 1, 128, 192), (BF, 1, 4, 1, 2, 256, 128),
])
def test_recurrent(ops, dtype, B, T, Hqk, Hv, K, V):
    P.check_recurrent(ops, "cpu", B, T, Hqk, Hv, K, V, dtype, wrap=guarded)
    P.check_recurrent(ops, "cpu", B, T, Hqk, Hv, K, V, dtype, l2=False, with_state=False, wrap=guarded)


@pytest.mark.parametrize("dtype,T,cu,Hqk,Hv,K,V", [
    (F32, 12, [0, 3, 3, 8, 12], 1, 2, 64, 64), (BF, 9, [0, 1, 6], 1, 2, 128, 64),
])
def test_recurrent_packed_sequences(ops, dtype, T, cu, Hqk, Hv, K, V):
    P.check_recurrent_packed(ops, "cpu", T, cu, Hqk, Hv, K, V, dtype, wrap=guarded)
    P.check_recurrent_packed(ops, "cpu", T, cu, Hqk, Hv, K, V, dtype, l2=False, with_state=False, wrap=guarded)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu", [
    (F32, 1, 64, 1, 1, 64, 64, False, None),
    (F32, 2, 100, 2, 4, 128, 128, True, None),
    (BF, 1, 200, 1, 2, 128, 128, True, None),
    (BF, 1, 140, 2, 2, 64, 64, False, [0, 5, 70, 71, 140]),
    (BF, 1, 128, 1, 1, 128, 256, True, None),
    (F32, 1, 96, 1, 1, 128, 192, True, [0, 1, 38, 96]),
])
def test_chunk_forward(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu):
    P.check_chunk(ops, "cpu", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, wrap=guarded, h0_std=0.1)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu", [
    (F32, 1, 130, 1, 2, 64, 64, True, None),
    (F32, 2, 100, 2, 4, 128, 128, True, None),
    (BF, 1, 200, 1, 2, 128, 128, True, None),
    (BF, 1, 140, 2, 2, 64, 64, False, [0, 5, 70, 71, 140]),
    (F32, 1, 96, 1, 1, 128, 192, True, [0, 1, 38, 96]),
    (BF, 1, 100, 1, 6, 64, 64, True, None),          # more value heads per group than the prep kernel has waves
    (F32, 1, 70, 1, 3, 64, 64, True, [0, 3, 70]),
])
def test_chunk_backward(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu):
    P.check_chunk(ops, "cpu", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, backward=True, wrap=guarded, h0_std=0.1)


@pytest.mark.parametrize("cu", [[0, 0, 70], [0, 70, 70], [0, 30, 30, 100], [0, 0, 0, 64]])
def test_chunk_packed_with_empty_sequences(ops, cu):
    """A sequence of length 0 has no chunk: its final state is its initial state, its gradients are empty."""
    P.check_chunk(ops, "cpu", 1, cu[-1], 1, 2, 64, 64, F32, cu=cu, backward=True, wrap=guarded, h0_std=0.1)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,cu", [
    (BF, 1, 200, 1, 2, 128, 128, None), (F32, 1, 140, 1, 2, 64, 64, [0, 5, 70, 140]),
])
def test_chunk_backward_recompute_mode_equals_stored_mode(ops, dtype, B, T, Hqk, Hv, K, V, cu):
    P.check_chunk_recompute_equals_stored(ops, "cpu", B, T, Hqk, Hv, K, V, dtype, cu=cu, wrap=guarded, h0_std=0.1)


def test_chunk_backward_without_initial_state(ops):
    P.check_chunk(ops, "cpu", 1, 70, 1, 1, 64, 64, F32, backward=True, with_h0=False, wrap=guarded)


@pytest.mark.parametrize("dtype,B,T,D,W,cu", [
    (F32, 2, 37, 16, 4, None), (BF, 1, 300, 32, 4, [0, 1, 3, 130, 131, 300]), (F32, 1, 9, 8, 3, [0, 2, 9]),
    (torch.float16, 2, 5, 8, 2, None), (F32, 3, 2, 8, 4, None), (F32, 1, 600, 8, 4, [0, 255, 257, 600]),
])
def test_conv1d(ops, dtype, B, T, D, W, cu):
    P.check_conv(ops, "cpu", B, T, D, W, dtype, cu=cu, residual=True, wrap=guarded)
    P.check_conv(ops, "cpu", B, T, D, W, dtype, cu=cu, bias=False, state=False, activation=None, wrap=guarded)


@pytest.mark.parametrize("dtype,B,T,D,W", [(F32, 2, 1, 16, 4), (BF, 3, 5, 8, 4), (F32, 1, 3, 8, 2)])
def test_conv1d_update(ops, dtype, B, T, D, W):
    P.check_conv_update(ops, "cpu", B, T, D, W, dtype, wrap=guarded)


@pytest.mark.parametrize("dtype,shape,N,wdt", [
    (F32, (3, 5), 64, None), (BF, (70,), 128, None), (BF, (2, 9), 256, torch.float32), (F32, (33,), 16, None),
    (BF, (5,), 512, None), (F32, (4,), 256, None), (BF, (300,), 32, None),
])
def test_rms_norm_gated(ops, dtype, shape, N, wdt):
    P.check_rms_norm_gated(ops, "cpu", shape, N, dtype, weight_dtype=wdt, wrap=guarded)


@pytest.mark.parametrize("dtype,shape,N,wdt", [(F32, (3, 5), 64, None), (BF, (70,), 128, None), (BF, (2, 9), 128, torch.float32)])
def test_rms_norm_sigmoid_gated(ops, dtype, shape, N, wdt):
    P.check_rms_norm_gated(ops, "cpu", shape, N, dtype, weight_dtype=wdt, wrap=guarded, activation="sigmoid")


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu,pad", [
    (F32, 1, 100, 1, 2, 64, 64, True, None, 0),
    (BF, 2, 70, 2, 4, 128, 128, True, None, 0),
    (BF, 1, 140, 2, 2, 64, 64, False, [0, 5, 70, 71, 140], 16),
])
def test_chunk_on_unsplit_qkv(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu, pad):
    P.check_chunk_qkv(ops, "cpu", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, pad=pad, wrap=guarded, h0_std=0.1)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu,wdt,bwd", [
    (BF, 1, 100, 1, 2, 64, 128, True, None, None, True),
    (BF, 1, 140, 2, 2, 128, 64, False, [0, 5, 70, 71, 140], torch.float32, True),
    (F32, 1, 70, 1, 1, 64, 64, True, None, None, True),
    (BF, 2, 64, 1, 2, 64, 128, True, None, None, False),
])
def test_chunk_with_fused_norm(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu, wdt, bwd):
    P.check_chunk_norm(ops, "cpu", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, weight_dtype=wdt, backward=bwd,
                       wrap=guarded, h0_std=0.1)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu,bwd", [
    (BF, 1, 100, 1, 2, 64, 128, True, None, True),
    (BF, 1, 140, 2, 4, 64, 64, False, [0, 5, 70, 71, 140], False),
])
def test_chunk_on_unsplit_qkv_with_fused_norm(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu, bwd):
    P.check_chunk_qkv_norm(ops, "cpu", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, backward=bwd, wrap=guarded, h0_std=0.1)


@pytest.mark.parametrize("dtype,shape,Hv,pdt", [
    (F32, (2, 37), 6, None), (BF, (1, 300), 32, None), (BF, (3, 5), 48, torch.float32), (F32, (1,), 256, None),
    (BF, (1100,), 4, None),
])
def test_gdn_gates(ops, dtype, shape, Hv, pdt):
    P.check_gdn_gates(ops, "cpu", shape, Hv, dtype, param_dtype=pdt, wrap=guarded)


@pytest.mark.parametrize("dtype,B,steps,Hqk,Hv,K,V,W,pdt", [
    (F32, 2, 3, 1, 2, 64, 64, 4, None), (BF, 2, 4, 2, 4, 128, 128, 4, None), (BF, 1, 2, 1, 2, 64, 128, 3, torch.float32),
])
def test_decode_step(ops, dtype, B, steps, Hqk, Hv, K, V, W, pdt):
    P.check_decode_step(ops, "cpu", B, steps, Hqk, Hv, K, V, W, dtype, param_dtype=pdt, wrap=guarded)


@pytest.mark.parametrize("dtype,B,T,D,W,S", [(F32, 2, 3, 16, 4, 6), (BF, 2, 2, 8, 3, 3), (BF, 1, 1, 8, 4, 3)])
def test_conv1d_update_general_state_length(ops, dtype, B, T, D, W, S):
    P.check_conv_update(ops, "cpu", B, T, D, W, dtype, S=S, wrap=guarded)


def _random_case(seed):
    import random
    rng = random.Random(seed)
    B = rng.choice([1, 1, 2])
    T = rng.randint(1, 200)
    Hqk = rng.choice([1, 2])
    Hv = Hqk * rng.choice([1, 2, 4])
    K, V = rng.choice([64, 128]), rng.choice([64, 128, 192])
    cu = None
    if B == 1 and rng.random() < 0.6:
        cuts = sorted(rng.sample(range(0, T + 1), min(T + 1, rng.randint(0, 4))))
        cu = [0] + cuts + [T]
    return (BF if seed % 2 else F32), B, T, Hqk, Hv, K, V, rng.random() < 0.7, cu


def _one_output_gradients(ops, device, kda):
    """A loss that uses only one of the two outputs reaches the backward pass with the other gradient undefined (the
    functions ask autograd not to fill it with zeros): the gradients from o alone and from the final state alone add up
    to those of the loss over both (linearity), in fp32."""
    import tests.parity as P
    B, T, H, K, V = 1, 130, 2, 64, 128
    if kda:
        x = P.kda_inputs(B, T, H, K, V, torch.float32, seed=7)
        names = ("q", "k", "v", "g", "beta", "h0", "A_log", "dt_bias")
    else:
        x = P.gdn_inputs(B, T, H, 2 * H, K, V, torch.float32, seed=7)
        names = ("q", "k", "v", "g", "beta", "h0")
    d = {n: t.to(device) for n, t in x.items()}

    def grads(use_o, use_ht):
        leaves = {n: d[n].clone().requires_grad_(True) for n in names}
        if kda:
            o, ht = ops.chunk_kda(leaves["q"], leaves["k"], leaves["v"], leaves["g"], leaves["beta"],
                                  initial_state=leaves["h0"], output_final_state=True, use_qk_l2norm_in_kernel=True,
                                  use_gate_in_kernel=True, use_beta_sigmoid_in_kernel=True, A_log=leaves["A_log"],
                                  dt_bias=leaves["dt_bias"])
        else:
            o, ht = ops.chunk_gated_delta_rule(leaves["q"], leaves["k"], leaves["v"], leaves["g"], leaves["beta"],
                                               initial_state=leaves["h0"], output_final_state=True,
                                               use_qk_l2norm_in_kernel=True)
        loss = 0
        if use_o:
            loss = loss + (o * d["do"]).sum()
        if use_ht:
            loss = loss + (ht * d["dht"]).sum()
        return torch.autograd.grad(loss, list(leaves.values()))
    both, only_o, only_ht = grads(True, True), grads(True, False), grads(False, True)
    for n, a, b, c in zip(names, both, only_o, only_ht):
        scale = max(a.abs().max().item(), 1e-6)
        assert ((b + c) - a).abs().max().item() <= 2e-5 * scale + 1e-6, n
        if n in ("k", "v", "h0"):   # the final state does not depend on q
            assert c.abs().max().item() > 0, n
        if n == "q":
            assert c.abs().max().item() == 0


@pytest.mark.parametrize("kda", [False, True])
def test_gradient_from_one_output_only(ops, kda):
    _one_output_gradients(ops, "cpu", kda)


@pytest.mark.parametrize("seed", range(8))
def test_chunk_random_shapes(ops, seed):
    """Seeded random shapes: ragged lengths, packed sequences with empty and one-token members, grouped heads."""
    dtype, B, T, Hqk, Hv, K, V, l2, cu = _random_case(seed)
    P.check_chunk(ops, "cpu", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, backward=True, wrap=guarded, h0_std=0.1, seed=seed)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,cu", [
    (BF, 1, 70, 1, 2, 64, 64, None),               # last chunk of 6 tokens: its second 32-row half does not exist
    (BF, 1, 200, 2, 4, 128, 128, None),
    (F32, 1, 97, 1, 2, 64, 64, [0, 33, 97]),
])
def test_chunk_backward_stays_inside_its_outputs(ops, dtype, B, T, Hqk, Hv, K, V, cu):
    """Grouped heads (later value heads add to the dq, dk rows of the first) with a short last chunk, outputs and
    workspace against guard pages: no kernel may touch rows past the end of dq, dk, dv."""
    P.check_chunk(ops, "cpu", B, T, Hqk, Hv, K, V, dtype, cu=cu, backward=True, wrap=guarded, h0_std=0.1)


def _random_conv_case(seed):
    import random
    rng = random.Random(1000 + seed)
    dtype = rng.choice([BF, F32, BF])
    B, T, W = rng.choice([1, 1, 2, 3]), rng.randint(1, 300), rng.randint(1, 8)
    D = rng.choice([8, 16, 64, 72, 256])
    cu = None
    if B == 1 and rng.random() < 0.6:
        cuts = sorted(rng.sample(range(0, T + 1), min(T + 1, rng.randint(0, 5))))
        cu = [0] + cuts + [T]
    return dict(B=B, T=T, D=D, W=W, dtype=dtype, cu=cu, residual=rng.random() < 0.5, bias=rng.random() < 0.7,
                state=rng.random() < 0.7, activation=rng.choice(["silu", None]), seed=seed)


@pytest.mark.parametrize("seed", range(6))
def test_conv1d_random_shapes(ops, seed):
    """Seeded random shapes of the convolution: widths 1..8, ragged and packed lengths, with and without bias,
    residual, initial state and activation."""
    c = _random_conv_case(seed)
    P.check_conv(ops, "cpu", c.pop("B"), c.pop("T"), c.pop("D"), c.pop("W"), c.pop("dtype"), wrap=guarded, **c)


@pytest.mark.parametrize("dtype,B,T,H,K,V,cu,kw", [
    (F32, 1, 64, 1, 64, 64, None, {}),
    (F32, 2, 100, 2, 128, 128, None, {}),
    (BF, 1, 200, 2, 128, 128, None, {}),
    (BF, 1, 140, 2, 64, 64, [0, 5, 70, 71, 140], dict(lower_bound=-5.0)),
    (F32, 1, 96, 1, 128, 192, [0, 1, 38, 96], dict(gate_in_kernel=False, beta_sigmoid=False, l2=False, transpose_state=False)),
    (BF, 1, 130, 1, 128, 64, None, dict(allow_neg=True, with_h0=False, g_dtype=torch.float32)),
])
def test_kda_forward(ops, dtype, B, T, H, K, V, cu, kw):
    P.check_kda(ops, "cpu", B, T, H, K, V, dtype, cu=cu, wrap=guarded, h0_std=0.1, **kw)


@pytest.mark.parametrize("dtype,B,T,H,K,V,cu,kw", [
    (F32, 1, 64, 1, 64, 64, None, {}),
    (F32, 1, 100, 2, 128, 128, None, {}),
    (BF, 1, 200, 2, 128, 128, None, {}),
    (BF, 1, 140, 2, 64, 64, [0, 5, 70, 71, 140], dict(lower_bound=-5.0)),
    (F32, 1, 96, 1, 128, 64, [0, 1, 38, 96], dict(gate_in_kernel=False, beta_sigmoid=False, l2=False, transpose_state=False)),
    (BF, 1, 130, 1, 128, 64, None, dict(allow_neg=True, with_h0=False, g_dtype=torch.float32)),
])
def test_kda_backward(ops, dtype, B, T, H, K, V, cu, kw):
    errs = P.check_kda(ops, "cpu", B, T, H, K, V, dtype, cu=cu, backward=True, wrap=guarded, h0_std=0.1, **kw)
    print({n: f"{e:.2e}" for n, e in errs.items()})


def _random_kda_case(seed):
    import random
    rng = random.Random(1000 + seed)
    B = rng.choice([1, 1, 2])
    T = rng.randint(1, 200)
    H = rng.choice([1, 2, 3])
    K, V = rng.choice([64, 128]), rng.choice([64, 128, 192])
    cu = None
    if B == 1 and rng.random() < 0.6:
        cuts = sorted(rng.sample(range(0, T + 1), min(T + 1, rng.randint(0, 4))))
        cu = [0] + cuts + [T]
    kw = dict(gate_in_kernel=rng.random() < 0.7, beta_sigmoid=rng.random() < 0.7, l2=rng.random() < 0.7,
              transpose_state=rng.random() < 0.5, with_h0=rng.random() < 0.7, allow_neg=rng.random() < 0.3)
    if kw["gate_in_kernel"] and rng.random() < 0.4:
        kw["lower_bound"] = -5.0
    if not kw["beta_sigmoid"]:
        kw["allow_neg"] = False   # the doubled beta is an option of the in-kernel sigmoid
    return (BF if seed % 2 else F32), B, T, H, K, V, cu, kw


@pytest.mark.parametrize("seed", range(4))
def test_kda_random_shapes(ops, seed):
    """Seeded random shapes and options of chunk_kda, forward and backward: ragged and packed lengths with empty
    members, both state layouts, with and without the in-kernel gate, sigmoid and norm."""
    dtype, B, T, H, K, V, cu, kw = _random_kda_case(seed)
    P.check_kda(ops, "cpu", B, T, H, K, V, dtype, cu=cu, backward=True, wrap=guarded, h0_std=0.1, seed=seed, **kw)


@pytest.mark.parametrize("dtype,B,T,H,K,V,cu,kw", [
    (F32, 2, 100, 2, 128, 64, None, {}),
    (BF, 1, 200, 2, 64, 128, [0, 70, 70, 200], dict(transpose_state=False)),
    (BF, 1, 130, 1, 128, 128, None, dict(with_h0=False)),
])
def test_kda_intermediate_states(ops, dtype, B, T, H, K, V, cu, kw):
    """The states at chunk entries, written out from the workspace's tiles in both layouts."""
    errs = P.check_kda(ops, "cpu", B, T, H, K, V, dtype, cu=cu, wrap=guarded, h0_std=0.1, states=True, **kw)
    assert "h" in errs
