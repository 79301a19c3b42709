"""GPU parity tests proper: the shipped HIP library (through the package's C-ABI binding) against the CPU
oracle on the same seeded inputs.  Run with `-m gpu` on an MI355X."""
import pytest
import torch

from oracle import gdn_oracle as O
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


@pytest.mark.parametrize("dtype,T,cu,Hqk,Hv,K,V", [
    (F32, 20, [0, 3, 3, 9, 20], 1, 2, 64, 64),       # an empty sequence
    (BF, 70, [0, 1, 40, 70], 2, 4, 128, 128),
    (BF, 12, [0, 5, 9], 1, 2, 128, 64),              # a padded batch: tokens 9..11 belong to no sequence
])
def test_recurrent_packed_sequences(ops, dtype, T, cu, Hqk, Hv, K, V):
    """cu_seqlens at the decode entry: every listed sequence runs on its own from its own state."""
    print(f"recurrent packed {dtype} T{T} cu{cu} Hqk{Hqk} Hv{Hv} K{K} V{V}", flush=True)
    P.check_recurrent_packed(ops, "cuda", T, cu, Hqk, Hv, K, V, dtype)
    P.check_recurrent_packed(ops, "cuda", T, cu, Hqk, Hv, K, V, dtype, l2=False, with_state=False)
    x = P.gdn_inputs(2, 4, Hqk, Hv, K, V, dtype)
    d = {n: t.cuda() for n, t in x.items()}
    with pytest.raises(ValueError, match="batch size is expected to be 1"):
        ops.fused_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], cu_seqlens=[0, 2, 4])


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
    # (sequences x q/k groups) a multiple of 8 with grouped heads: the recurrence kernels renumber their workgroups
    (BF, 4, 200, 2, 4, 128, 128, True, None),
    (BF, 2, 130, 4, 16, 128, 128, True, None),
    (BF, 1, 600, 1, 2, 64, 64, False, [0, 64, 65, 130, 258, 300, 450, 599, 600]),
    (F32, 8, 70, 1, 2, 64, 64, True, None),
    (F32, 1, 1024, 2, 4, 128, 128, True, None),                  # fp32 with grouped heads over many chunks
    # value heads per q/k group other than 1, 2, 4: the prep kernel deals a group's heads to its four waves
    (BF, 1, 200, 1, 3, 128, 128, True, None),
    (BF, 1, 140, 2, 12, 64, 64, True, [0, 5, 70, 71, 140]),
    (F32, 1, 100, 1, 5, 64, 64, False, None),
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


def test_chunk_backward_wide_value_heads_group_of_four_slow_decay(ops):
    """Head shape of BASELINE config 4 (d_k 128, d_v 256, four value heads per q/k head) with its decay recipe
    (A_log ~ U(log 0.5, log 2), dt_bias ~ U(-6, -4): slow forgetting), forward and backward against the oracle."""
    print("chunk bwd bf16 B1 T512 Hqk1 Hv4 K128 V256 slow decay", flush=True)
    P.check_chunk(ops, "cuda", 1, 512, 1, 4, 128, 256, BF, backward=True, a_log=(0.5, 2.0), dt_bias=(-6.0, -4.0))


@pytest.mark.parametrize("B,T,H,K,V,l2,cu,heads", [
    # rows of the reference's own table (test_chunk_gated_delta_rule.py:116-140) with its input recipe (:158-175)
    (1, 128, 8, 128, 128, False, None, 2),
    (1, 1024, 64, 128, 128, True, None, 2),
    (1, 1121, 16, 128, 128, True, [0, 112, 209, 240, 281, 489, 523, 566, 689, 721, 785, 837, 985, 1071, 1121], 2),
    (21, 195, 32, 128, 128, True, None, 1),
    (1, 160, 32, 128, 128, True, None, 2),
    (1, 4608, 2, 128, 128, True, None, 2),
    (1, 4608, 32, 128, 128, True, None, 1),
    (1, 32832, 32, 128, 128, True, [0, 14012, 26600, 32766, 32832], 1),
])
def test_chunk_reference_test_table_and_recipe(ops, B, T, H, K, V, l2, cu, heads):
    print(f"chunk reference recipe B{B} T{T} H{H} K{K} V{V} l2={l2} varlen={cu is not None}", flush=True)
    P.check_chunk_reference_recipe(ops, "cuda", B, T, H, K, V, l2, cu=cu, oracle_heads=heads)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu", [
    (BF, 2, 300, 2, 4, 128, 128, True, None),
    (BF, 1, 1121, 2, 2, 128, 128, True, [0, 112, 209, 240, 281, 489, 523, 566, 689, 721, 785, 837, 985, 1071, 1121]),
    (BF, 1, 256, 1, 4, 128, 256, True, None),
    (BF, 1, 200, 2, 2, 64, 64, False, None),
    (F32, 1, 200, 1, 2, 128, 128, True, None),
])
def test_chunk_backward_recompute_mode_equals_stored_mode(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu):
    print(f"chunk recompute vs stored {dtype} B{B} T{T} Hqk{Hqk} Hv{Hv} K{K} V{V}", flush=True)
    P.check_chunk_recompute_equals_stored(ops, "cuda", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,cu", [
    (BF, 2, 300, 2, 4, 128, 128, None),
    (BF, 1, 333, 1, 2, 64, 128, [0, 70, 70, 333]),
    (F32, 1, 130, 1, 2, 128, 64, None),
])
def test_chunk_backward_in_phases_through_the_c_abi(ops, dtype, B, T, Hqk, Hv, K, V, cu):
    """gdn_chunk_bwd_parts on a two-part workspace against gdn_chunk_bwd_strided on one full workspace, bit for bit:
    all phases in one call; refill / reverse recurrence / chunk-local in three calls; with the prep part rebuilt as
    well (prep_valid = 0); a state part that is too small is refused."""
    from mindspeed_mm_amd._lib import DTYPE_CODE, ptr
    lib = ops.lib
    N = (len(cu) - 1) if cu is not None else B
    x = P.gdn_inputs(B, T, Hqk, Hv, K, V, dtype, seed=41, N=N)
    d = {n: t.cuda() for n, t in x.items()}
    q, k, v, g, do = d["q"], d["k"], d["v"], d["g"], d["do"]
    beta = d["beta"].float()
    h0, dht = d["h0"], d["dht"]
    cu_t = torch.tensor(cu, dtype=torch.int64, device="cuda") if cu is not None else None
    code, scale = DTYPE_CODE[dtype], K ** -0.5
    dims = (B, T, N, Hqk, Hv, K, V)

    def buf(mode):
        n = lib.gdn_chunk_workspace_bytes(*dims, code, mode)
        t = torch.empty(n + 256, dtype=torch.uint8, device="cuda")
        off = (-t.data_ptr()) % 256
        return t[off:off + n], n

    def grads():
        return [torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(g), torch.empty_like(beta),
                torch.empty_like(h0)]

    def fwd(ws, n, o):
        rc = lib.gdn_chunk_fwd_strided(ptr(q), ptr(k), ptr(v), 0, 0, 0, ptr(g), ptr(beta), ptr(h0), ptr(cu_t), ptr(o), None,
                                       ptr(ws), n, *dims, scale, 1, code, 0, lib.stream())
        assert rc == 0, rc

    def parts(G, wp, np_, wst, ns, phases, prep_valid):
        return lib.gdn_chunk_bwd_parts(ptr(q), ptr(k), ptr(v), 0, 0, 0, ptr(g), ptr(beta), ptr(h0), ptr(cu_t), ptr(do),
                                       ptr(dht), ptr(G[0]), ptr(G[1]), ptr(G[2]), 0, 0, 0, ptr(G[3]), ptr(G[4]), ptr(G[5]),
                                       ptr(wp), np_, ptr(wst), ns, phases, prep_valid, *dims, scale, 1, code, 0, lib.stream())

    o = torch.empty_like(v)
    full, nfull = buf(1)
    fwd(full, nfull, o)
    want = grads()
    rc = lib.gdn_chunk_bwd_strided(ptr(q), ptr(k), ptr(v), 0, 0, 0, ptr(g), ptr(beta), ptr(h0), ptr(cu_t), ptr(do), ptr(dht),
                                   ptr(want[0]), ptr(want[1]), ptr(want[2]), 0, 0, 0, ptr(want[3]), ptr(want[4]),
                                   ptr(want[5]), ptr(full), nfull, *dims, scale, 1, code, 0, lib.stream())
    assert rc == 0, rc
    prep, nprep = buf(2)
    state, nstate = buf(3)
    assert nprep + nstate >= nfull > nstate > 0 and nprep > 0
    if dtype == BF:
        fwd(prep, nprep, o)            # a 16-bit forward call that writes o needs the prep part only
        cases = [("one call", (7,), 1), ("three calls", (1, 2, 4), 1), ("prep rebuilt too", (7,), 0)]
    else:
        cases = [("prep rebuilt too", (7,), 0), ("three calls, prep rebuilt by the first", (1, 2, 4), 0)]
    for name, phases, prep_valid in cases:
        state.zero_()
        if not prep_valid:
            prep.zero_()
        got = grads()
        for ph in phases:
            rc = parts(got, prep, nprep, state, nstate, ph, prep_valid or ph != phases[0])
            assert rc == 0, (name, ph, rc)
        torch.cuda.synchronize()
        for w, g_, nm in zip(want, got, ("dq", "dk", "dv", "dg", "dbeta", "dh0")):
            assert torch.equal(w, g_), (name, nm)
    assert parts(grads(), prep, nprep, state, nstate - 256, 7, 1) == -5


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
    _one_output_gradients(ops, "cuda", kda)


def test_chunk_default_mode_on_one_stream_equals_two_streams(ops):
    """The default mode's backward pass rebuilds states and corrected values on a second stream beside the reverse
    recurrence; with that switched off (everything on the caller's stream) the gradients are the same bits."""
    x = P.gdn_inputs(2, 500, 2, 4, 128, 128, BF, seed=42)
    d = {n: t.cuda() for n, t in x.items()}
    outs = []
    was = ops.two_stream_backward
    try:
        for two in (True, False):
            ops.two_stream_backward = two
            L = {n: d[n].clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta", "h0")}
            o, ht = ops.chunk_gated_delta_rule(L["q"], L["k"], L["v"], L["g"], L["beta"], initial_state=L["h0"],
                                               output_final_state=True, use_qk_l2norm_in_kernel=True)
            ((o.float() * d["do"].float()).sum() + (ht * d["dht"]).sum()).backward()
            outs.append([o, ht] + [L[n].grad for n in L])
    finally:
        ops.two_stream_backward = was
    for a, b in zip(*outs):
        assert torch.equal(a, b)


def test_chunk_backward_stored_mode_against_oracle(ops):
    P.check_chunk(ops, "cuda", 2, 200, 2, 4, 128, 128, BF, backward=True, skip_recompute=True)


def test_chunk_beta_in_float32_and_in_the_activation_dtype(ops):
    """beta is read in its own dtype: bf16 in place (the layer's), anything else as float32; dbeta comes back in it."""
    x = P.gdn_inputs(1, 200, 2, 4, 128, 128, BF, seed=5)
    d = {n: t.cuda() for n, t in x.items()}
    outs = []
    for bdt in (BF, F32):
        L = {n: d[n].clone().requires_grad_(True) for n in ("q", "k", "v", "g")}
        beta = d["beta"].to(bdt).clone().detach().requires_grad_(True)
        o, _ = ops.chunk_gated_delta_rule(L["q"], L["k"], L["v"], L["g"], beta, use_qk_l2norm_in_kernel=True)
        (o.float() * d["do"].float()).sum().backward()
        assert beta.grad.dtype == bdt
        outs.append((o, beta.grad, L["q"].grad))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][2], outs[1][2])   # same values of beta
    assert torch.equal(outs[0][1], outs[1][1].to(BF))


def test_chunk_rejects_key_width_256(ops):
    """The chunk kernels hold K in {64, 128} (the reference allows up to 256, chunk_delta_h.py:259): a clean error."""
    q = torch.randn(1, 64, 1, 256, device="cuda", dtype=BF)
    g, b = -torch.rand(1, 64, 1, device="cuda"), torch.rand(1, 64, 1, device="cuda")
    with pytest.raises(ValueError, match="unsupported size"):
        ops.chunk_gated_delta_rule(q, q, q, g, b)


def test_chunk_rows_past_the_last_sequence_are_cleared(ops):
    """cu_seqlens on the device cannot be checked against the number of tokens without a synchronisation: rows after
    the last listed sequence belong to no chunk, and every output row there is written as zero (forward and
    backward), the rows before it as in a call on the covered tokens alone."""
    T, Tc, cu = 100, 90, [0, 30, 90]
    x = P.gdn_inputs(1, T, 1, 2, 64, 64, BF, seed=5, N=2)
    d = {n: t.cuda() for n, t in x.items()}
    cu_t = torch.tensor(cu, dtype=torch.int64, device="cuda")
    outs = []
    for t_len in (T, Tc):
        L = {n: d[n][:, :t_len].clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta")}
        o, ht = ops.chunk_gated_delta_rule(L["q"], L["k"], L["v"], L["g"], L["beta"], initial_state=d["h0"],
                                           output_final_state=True, use_qk_l2norm_in_kernel=True, cu_seqlens=cu_t)
        (o.float() * d["do"][:, :t_len].float()).sum().backward()
        outs.append((o, ht, {n: L[n].grad for n in L}))
    (o, ht, gr), (oc, htc, grc) = outs
    assert torch.equal(o[:, :Tc], oc) and torch.equal(ht, htc) and not o[:, Tc:].any()
    for n in gr:
        assert torch.equal(gr[n][:, :Tc], grc[n]), n
        assert not gr[n][:, Tc:].any(), n


def test_chunk_float16(ops):
    """float16 q, k, v (accepted by the reference's entry, chunk_gated_delta_rule.py:379-386) run through the float32
    kernels: the output and the gradients come back in float16 and meet the half-precision bounds against the oracle
    on the same float16-valued inputs."""
    H16 = torch.float16
    x = P.gdn_inputs(1, 200, 1, 2, 64, 64, F32, seed=9)
    x = {n: (t.to(H16) if n in ("q", "k", "v", "do") else t) for n, t in x.items()}
    d = {n: t.cuda() for n, t in x.items()}
    L = {n: d[n].clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta")}
    R = {n: x[n].float().clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta")}
    o, ht = ops.chunk_gated_delta_rule(L["q"], L["k"], L["v"], L["g"], L["beta"], initial_state=d["h0"],
                                       output_final_state=True, use_qk_l2norm_in_kernel=True)
    ro, rht = P.O.chunk_gated_delta_rule_ref(R["q"], R["k"], R["v"], R["g"], R["beta"], initial_state=x["h0"],
                                             output_final_state=True, use_qk_l2norm_in_kernel=True)
    assert o.dtype == H16 and ht.dtype == F32
    (o.float() * d["do"].float()).sum().backward()
    (ro * x["do"].float()).sum().backward()
    P._err("o", o, ro, H16, P.BF16_ABS_O)
    P._err("final_state", ht, rht, H16, P.BF16_ABS_O)
    for n in L:
        assert L[n].grad.dtype == L[n].dtype
        P._err("d" + n, L[n].grad, R[n].grad, H16, P.BF16_ABS_GRAD)


def test_chunk_head_first_warns_and_proceeds(ops):
    """head_first=True is deprecated in the reference, which warns and then treats the tensors as [B, T, H, ...]
    all the same (chunk_gated_delta_rule.py:392-396)."""
    x = P.gdn_inputs(1, 70, 1, 1, 64, 64, BF, seed=3)
    d = {n: t.cuda() for n, t in x.items()}
    with pytest.warns(UserWarning, match="head_first is deprecated"):
        o1, _ = ops.chunk_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], head_first=True)
    o2, _ = ops.chunk_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"])
    assert torch.equal(o1, o2)


def test_chunk_under_autocast_keeps_dtypes(ops):
    """custom_fwd / custom_bwd: under torch.autocast the operator still computes in the dtype of its inputs."""
    x = P.gdn_inputs(1, 130, 1, 2, 64, 64, F32, seed=2)
    d = {n: t.cuda() for n, t in x.items()}
    L = {n: d[n].clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta")}
    o0, _ = ops.chunk_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], use_qk_l2norm_in_kernel=True)
    with torch.autocast("cuda", dtype=BF):
        o, _ = ops.chunk_gated_delta_rule(L["q"], L["k"], L["v"], L["g"], L["beta"], use_qk_l2norm_in_kernel=True)
        (o * d["do"]).sum().backward()
    assert o.dtype == F32 and torch.equal(o, o0)
    assert all(L[n].grad.dtype == F32 for n in L)


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


@pytest.mark.parametrize("dtype,shape,N,wdt", [(F32, (3, 5), 64, None), (BF, (2, 70, 3), 128, None), (BF, (9,), 128, torch.float32)])
def test_rms_norm_sigmoid_gated(ops, dtype, shape, N, wdt):
    """The KDA layer's norm (KimiK_3_MoeRMSNormGated, modeling_kimi_linear.py:75-96), forward and backward."""
    errs = P.check_rms_norm_gated(ops, "cuda", shape, N, dtype, weight_dtype=wdt, activation="sigmoid")
    print("   ", {n: f"{e:.2e}" for n, e in errs.items()}, flush=True)
    import mindspeed_mm_amd as M
    norm = M.RMSNormGated(N, eps=1e-6, activation="sigmoid").cuda()        # as the layer constructs it (:603-604)
    x, g = torch.randn(4, N, device="cuda", dtype=dtype), torch.randn(4, N, device="cuda", dtype=dtype)
    assert torch.equal(norm(x, g), ops.rms_norm_gated(x, g, norm.weight, 1e-6, "sigmoid"))


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



@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu,pad", [
    (F32, 1, 100, 1, 2, 64, 64, True, None, 0),
    (BF, 2, 200, 2, 4, 128, 128, True, None, 0),
    (BF, 1, 140, 2, 2, 64, 64, False, [0, 5, 70, 71, 140], 16),
    (BF, 1, 512, 4, 8, 128, 128, True, [0, 100, 512], 0),
])
def test_chunk_on_unsplit_qkv(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu, pad):
    print(f"chunk qkv {dtype} B{B} T{T} Hqk{Hqk} Hv{Hv} K{K} V{V} l2={l2} varlen={cu is not None} pad={pad}", flush=True)
    P.check_chunk_qkv(ops, "cuda", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, pad=pad, h0_std=0.1)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu,wdt,bwd", [
    (BF, 2, 200, 2, 4, 128, 128, True, None, None, True),
    (BF, 1, 512, 4, 8, 128, 128, True, [0, 100, 101, 512], torch.float32, True),
    (BF, 1, 140, 2, 2, 64, 64, False, [0, 5, 70, 71, 140], None, True),
    (F32, 1, 100, 1, 2, 64, 128, True, None, None, True),
    (F32, 1, 130, 1, 1, 128, 64, True, None, None, False),
    (BF, 2, 1024, 4, 8, 128, 128, True, None, None, False),
])
def test_chunk_with_fused_norm(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu, wdt, bwd):
    print(f"chunk+norm {dtype} B{B} T{T} Hqk{Hqk} Hv{Hv} K{K} V{V} l2={l2} varlen={cu is not None} wdt={wdt} bwd={bwd}",
          flush=True)
    P.check_chunk_norm(ops, "cuda", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, weight_dtype=wdt, backward=bwd,
                       h0_std=0.1)


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,l2,cu,bwd", [
    (BF, 2, 200, 2, 4, 128, 128, True, None, True),
    (BF, 1, 512, 4, 8, 128, 128, True, [0, 100, 101, 512], False),
    (F32, 1, 100, 1, 2, 64, 64, True, None, True),
])
def test_chunk_on_unsplit_qkv_with_fused_norm(ops, dtype, B, T, Hqk, Hv, K, V, l2, cu, bwd):
    print(f"chunk qkv+norm {dtype} B{B} T{T} Hqk{Hqk} Hv{Hv} K{K} V{V} l2={l2} varlen={cu is not None} bwd={bwd}", flush=True)
    P.check_chunk_qkv_norm(ops, "cuda", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, backward=bwd, h0_std=0.1)


def test_fused_norm_rejects_other_head_dims(ops):
    q = torch.randn(1, 64, 1, 64, device="cuda", dtype=BF)
    v = torch.randn(1, 64, 1, 256, device="cuda", dtype=BF)
    g, b = -torch.rand(1, 64, 1, device="cuda"), torch.rand(1, 64, 1, device="cuda")
    with pytest.raises(ValueError):
        ops.chunk_gated_delta_rule_norm(q, q, v, g, b, torch.randn_like(v), torch.ones(256, device="cuda", dtype=BF),
                                        in_output_kernel=True)


def test_chunk_rejects_bad_strides(ops):
    """A token stride that breaks 16-byte alignment cannot be read in place: the op copies; the C ABI refuses."""
    B, T, H, K = 1, 64, 1, 64
    wide = torch.randn(B, T, 3 * K + 4, device="cuda", dtype=BF)
    q, k, v = (wide[..., i * K:(i + 1) * K].reshape(B, T, H, K) for i in range(3))
    g = -torch.rand(B, T, H, device="cuda")
    beta = torch.rand(B, T, H, device="cuda")
    o, _ = ops.chunk_gated_delta_rule(q, k, v, g, beta)
    o2, _ = ops.chunk_gated_delta_rule(q.contiguous(), k.contiguous(), v.contiguous(), g, beta)
    assert torch.equal(o, o2)
    lib = ops.lib
    ws = torch.empty(lib.gdn_chunk_workspace_bytes(B, T, B, H, H, K, K, 1, 0) + 256, dtype=torch.uint8, device="cuda")
    rc = lib.gdn_chunk_fwd_strided(q.data_ptr(), k.data_ptr(), v.data_ptr(), 3 * K + 4, 3 * K + 4, 3 * K + 4,
                                   g.data_ptr(), beta.data_ptr(), None, None, o.data_ptr(), None,
                                   ws.data_ptr() + (-ws.data_ptr()) % 256, ws.numel() - 256, B, T, B, H, H, K, K, 0.125, 0,
                                   1, 0, lib.stream())
    assert rc == -6


@pytest.mark.parametrize("dtype,shape,Hv,pdt", [
    (F32, (2, 37), 6, None), (BF, (1, 300), 32, None), (BF, (3, 5), 48, torch.float32), (F32, (1,), 256, None),
    (BF, (2, 8192), 32, None), (BF, (1, 65536), 64, torch.float32),
])
def test_gdn_gates(ops, dtype, shape, Hv, pdt):
    P.check_gdn_gates(ops, "cuda", shape, Hv, dtype, param_dtype=pdt)


def test_gdn_gates_feed_the_rule(ops):
    """The layer's chain: projections -> gates -> rule, gradients back to the projections and the parameters."""
    B, T, Hqk, Hv, K, V = 1, 128, 2, 4, 64, 64
    gen = torch.Generator().manual_seed(1)
    r = lambda *s: torch.randn(*s, generator=gen)
    a, b = r(B, T, Hv).to(BF), r(B, T, Hv).to(BF)
    A_log, dt_bias = torch.empty(Hv).uniform_(0, 2.7, generator=gen), torch.empty(Hv).uniform_(-4, -2, generator=gen)
    mixed = r(B, T, 2 * Hqk * K + Hv * V).to(BF)
    do = r(B, T, Hv, V).to(BF)
    L = [t.cuda().requires_grad_(True) for t in (mixed, a, b, A_log, dt_bias)]
    g, beta = ops.gdn_gates(L[1], L[2], L[3], L[4])
    o, _ = ops.chunk_gated_delta_rule_qkv(L[0], g, beta, Hqk, Hv, K, V, use_qk_l2norm_in_kernel=True)
    o.backward(do.cuda())
    R = [t.float().requires_grad_(True) for t in (mixed, a, b, A_log, dt_bias)]
    rg, rbeta = O.gdn_gates_ref(R[1], R[2], R[3], R[4])
    q, k, v = torch.split(R[0], [Hqk * K, Hqk * K, Hv * V], dim=-1)
    ro, _ = O.chunk_gated_delta_rule_ref(q.reshape(B, T, Hqk, K), k.reshape(B, T, Hqk, K), v.reshape(B, T, Hv, V), rg,
                                         rbeta.to(BF).float(), use_qk_l2norm_in_kernel=True)
    ro.backward(do.float())
    P._err("o", o, ro, BF, P.BF16_ABS_O)
    for name, l, rr in zip(("d_mixed", "da", "db"), L[:3], R[:3]):
        P._err(name, l.grad, rr.grad, BF, P.BF16_ABS_GRAD)
    for name, l, rr in zip(("dA_log", "ddt_bias"), L[3:], R[3:]):
        P._err(name, l.grad, rr.grad, BF, 2e-2 * max(rr.grad.abs().max().item(), 1.0), rtol=2e-2)


@pytest.mark.parametrize("dtype,B,steps,Hqk,Hv,K,V,W,pdt", [
    (F32, 2, 3, 1, 2, 64, 64, 4, None), (BF, 2, 4, 2, 4, 128, 128, 4, None), (BF, 1, 2, 1, 2, 64, 128, 3, torch.float32),
    (BF, 16, 8, 16, 32, 128, 128, 4, None),
])
def test_decode_step(ops, dtype, B, steps, Hqk, Hv, K, V, W, pdt):
    print(f"decode step {dtype} B{B} steps{steps} Hqk{Hqk} Hv{Hv} K{K} V{V} W{W}", flush=True)
    P.check_decode_step(ops, "cuda", B, steps, Hqk, Hv, K, V, W, dtype, param_dtype=pdt)


def test_decode_cache_prefill_then_steps(ops):
    """Prefill with the chunked operators, hand both states to the cache, decode two more tokens, reorder the beams:
    equal to running the chunked operators over the longer sequences of the reordered batch."""
    from mindspeed_mm_amd import GdnDecodeCache
    B, T, Hqk, Hv, K, V, W = 3, 70, 2, 4, 64, 64, 4
    nq, nv = Hqk * K, Hv * V
    D = 2 * nq + nv
    gen = torch.Generator().manual_seed(5)
    r = lambda *s: torch.randn(*s, generator=gen)
    xin = r(B, T + 2, D).to(BF).cuda()
    a, b = r(B, T + 2, Hv).to(BF).cuda(), r(B, T + 2, Hv).to(BF).cuda()
    cw, cb = (r(D, W) / 2).to(BF).cuda(), (r(D) / 4).to(BF).cuda()
    A_log, dt_bias = torch.empty(Hv).uniform_(0, 2.7, generator=gen).cuda(), torch.empty(Hv).uniform_(-4, -2, generator=gen).cuda()

    def layer(x, aa, bb):   # chunked path over whole sequences
        y, conv_fs = ops.causal_conv1d(x, cw.t().contiguous(), cb, activation="silu", output_final_state=True)
        g, beta = ops.gdn_gates(aa, bb, A_log, dt_bias)
        o, S = ops.chunk_gated_delta_rule_qkv(y, g, beta, Hqk, Hv, K, V, output_final_state=True,
                                              use_qk_l2norm_in_kernel=True)
        return o, conv_fs, S
    cache = GdnDecodeCache(1)
    assert not cache.has_previous_state(0)
    _, conv_fs, S = layer(xin[:, :T], a[:, :T], b[:, :T])
    cache.set_prefill(0, conv_fs, S)
    assert cache.has_previous_state(0) and cache.conv_states[0].shape == (B, D, W)
    o1 = ops.decode_step(xin[:, T:T + 1], a[:, T:T + 1], b[:, T:T + 1], cache.conv_states[0], cache.recurrent_states[0],
                         cw, cb, A_log, dt_bias, Hqk, Hv, K, V)
    beam = torch.tensor([2, 0, 0], device="cuda")
    cache.reorder_cache(beam)
    x2 = xin[:, T + 1:T + 2]
    o2 = ops.decode_step(x2, a[:, T + 1:T + 2], b[:, T + 1:T + 2], cache.conv_states[0], cache.recurrent_states[0], cw, cb,
                         A_log, dt_bias, Hqk, Hv, K, V)
    # whole-sequence run of the reordered batch: history of beam[i], last token of row i
    xfull = torch.cat([xin[beam][:, :T + 1], x2], dim=1)
    afull = torch.cat([a[beam][:, :T + 1], a[:, T + 1:T + 2]], dim=1)
    bfull = torch.cat([b[beam][:, :T + 1], b[:, T + 1:T + 2]], dim=1)
    ofull, conv_full, Sfull = layer(xfull, afull, bfull)
    ofull1, _, _ = layer(xin[:, :T + 1], a[:, :T + 1], b[:, :T + 1])
    P._err("decode token 1", o1, ofull1[:, T:T + 1], BF, P.BF16_ABS_O)
    P._err("decode token 2 after reorder", o2, ofull[:, T + 1:T + 2], BF, P.BF16_ABS_O)
    P._err("recurrent state", cache.recurrent_states[0], Sfull, BF, P.BF16_ABS_GRAD)
    assert torch.equal(cache.conv_states[0], conv_full)


@pytest.mark.parametrize("cu", [[0, 0, 70], [0, 70, 70], [0, 30, 30, 100], [0, 0, 0, 64]])
def test_chunk_packed_with_empty_sequences(ops, cu):
    print(f"chunk packed with empty sequences {cu}", flush=True)
    P.check_chunk(ops, "cuda", 1, cu[-1], 2, 4, 128, 128, BF, cu=cu, backward=True, h0_std=0.1)


@pytest.mark.parametrize("dtype,B,T,D,W,S", [(F32, 2, 3, 16, 4, 6), (BF, 2, 2, 8, 3, 3), (BF, 1, 1, 8, 4, 3)])
def test_conv1d_update_general_state_length(ops, dtype, B, T, D, W, S):
    P.check_conv_update(ops, "cuda", B, T, D, W, dtype, S=S)


@pytest.mark.parametrize("seed", range(12))
def test_chunk_random_shapes(ops, seed):
    """The seeded random shapes of the CPU emulation tests, on the device build."""
    from tests.test_emu_kernels import _random_case
    dtype, B, T, Hqk, Hv, K, V, l2, cu = _random_case(seed)
    print(f"chunk random {seed}: {dtype} B{B} T{T} Hqk{Hqk} Hv{Hv} K{K} V{V} l2={l2} cu={cu}", flush=True)
    P.check_chunk(ops, "cuda", B, T, Hqk, Hv, K, V, dtype, l2=l2, cu=cu, backward=True, h0_std=0.1, seed=seed)


def test_no_grad_forward_prepares_no_backward(ops):
    """Under torch.no_grad() inputs that require grad must not make the forward kernels write backward operands:
    the result is the same and nothing is attached to the graph."""
    x = P.gdn_inputs(1, 200, 2, 4, 128, 128, BF, seed=3)
    d = {n: t.cuda().requires_grad_(t.is_floating_point()) for n, t in x.items()}
    o1, h1 = ops.chunk_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=d["h0"],
                                        output_final_state=True, use_qk_l2norm_in_kernel=True)
    with torch.no_grad():
        o2, h2 = ops.chunk_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=d["h0"],
                                            output_final_state=True, use_qk_l2norm_in_kernel=True)
    assert o1.requires_grad and not o2.requires_grad and o2.grad_fn is None
    assert torch.equal(o1, o2) and torch.equal(h1, h2)


@pytest.mark.parametrize("seed", range(24))
def test_conv1d_random_shapes(ops, seed):
    """The seeded random convolution shapes of the CPU emulation tests (and more seeds), on the device build."""
    from tests.test_emu_kernels import _random_conv_case
    c = _random_conv_case(seed)
    print(f"conv random {seed}: {c}", flush=True)
    P.check_conv(ops, "cuda", c.pop("B"), c.pop("T"), c.pop("D"), c.pop("W"), c.pop("dtype"), **c)


# ---- KDA (one decay per key channel) ------------------------------------------------------------------------------

KDA_CASES = [
    # dtype, B, T, H, K, V, cu, options
    (F32, 1, 64, 1, 64, 64, None, {}),
    (F32, 2, 100, 2, 128, 128, None, {}),
    (F32, 1, 1024, 2, 128, 128, None, dict(a_log=(0.5, 2.0), dt_bias=(-6.0, -4.0))),          # slow decay, long memory
    (BF, 1, 200, 2, 128, 128, None, {}),
    (BF, 2, 512, 4, 128, 128, None, dict(a_log=(0.5, 2.0), dt_bias=(-6.0, -4.0))),
    (BF, 1, 140, 2, 64, 64, [0, 5, 70, 71, 140], dict(lower_bound=-5.0)),
    (BF, 1, 1121, 2, 128, 128, [0, 112, 209, 240, 281, 489, 523, 566, 689, 721, 785, 837, 985, 1071, 1121],
     dict(lower_bound=-5.0)),
    (F32, 1, 96, 1, 128, 192, [0, 1, 38, 96], dict(gate_in_kernel=False, beta_sigmoid=False, l2=False, transpose_state=False)),
    (BF, 1, 130, 1, 128, 64, None, dict(allow_neg=True, with_h0=False, g_dtype=torch.float32)),
    (BF, 1, 300, 3, 128, 256, [0, 0, 300], dict(gate_in_kernel=False)),                      # an empty sequence
    (BF, 1, 2048, 4, 128, 128, None, {}),                                                     # the layer's head shape
    (BF, 4, 130, 24, 128, 128, None, {}),                          # more 32-column slabs of the state than CUs: two per workgroup
]


@pytest.mark.parametrize("dtype,B,T,H,K,V,cu,kw", KDA_CASES)
def test_kda_forward(ops, dtype, B, T, H, K, V, cu, kw):
    print(f"kda {dtype} B{B} T{T} H{H} K{K} V{V} cu={'yes' if cu else 'no'} {kw}", flush=True)
    errs = P.check_kda(ops, "cuda", B, T, H, K, V, dtype, cu=cu, **kw)
    print("   ", {n: f"{e:.2e}" for n, e in errs.items()}, flush=True)


@pytest.mark.parametrize("dtype,B,T,H,K,V,cu,kw", KDA_CASES)
def test_kda_backward(ops, dtype, B, T, H, K, V, cu, kw):
    print(f"kda backward {dtype} B{B} T{T} H{H} K{K} V{V} cu={'yes' if cu else 'no'} {kw}", flush=True)
    errs = P.check_kda(ops, "cuda", B, T, H, K, V, dtype, cu=cu, backward=True, **kw)
    print("   ", {n: f"{e:.2e}" for n, e in errs.items()}, flush=True)


@pytest.mark.parametrize("dtype", [BF, torch.float32])
@pytest.mark.parametrize("B,T,H,K,V,cu,transposed", [
    (2, 150, 2, 128, 128, None, True),              # dense batch, a partial last chunk
    (1, 200, 3, 64, 128, [0, 70, 70, 200], False),  # packed, an empty sequence, [K,V] layout, K != V
    (1, 64, 1, 128, 64, None, False),               # one chunk: the state at its entry is the initial state
])
def test_kda_intermediate_states(ops, dtype, B, T, H, K, V, cu, transposed):
    """return_intermediate_states=True: the state at every chunk entry, [B, NT, H, K, V] or [.., V, K] in the input
    type (chunk_kda_naive.py:287-303), against the oracle; nothing else about the call changes."""
    e = P.check_kda(ops, "cuda", B, T, H, K, V, dtype, cu=cu, transpose_state=transposed, states=True, seed=21)
    assert "h" in e
    # under autograd the states come back without a gradient and the other results keep theirs
    e = P.check_kda(ops, "cuda", B, T, H, K, V, dtype, cu=cu, transpose_state=transposed, states=True, backward=True, seed=22)
    assert "dq" in e and "h" in e


def test_kda_output_from_the_recurrence_equals_the_output_kernel(ops):
    """With one 32-column slab of the state per workgroup the 16-bit recurrence writes the output itself; with more
    slabs than compute units it leaves states and v_new to the stand-alone output kernel.  Both accumulate a row in the
    same order: batch row 0 alone (the first way) and inside a batch of four (the second way) give the same bits."""
    B, T, H, K, V = 4, 200, 24, 128, 128
    d = {n: t.cuda() for n, t in P.kda_inputs(B, T, H, K, V, BF, seed=3).items()}
    kw = dict(output_final_state=True, use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True,
              use_beta_sigmoid_in_kernel=True, A_log=d["A_log"], dt_bias=d["dt_bias"])
    with torch.no_grad():
        o, ht = ops.chunk_kda(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=d["h0"], **kw)
        o1, ht1 = ops.chunk_kda(d["q"][:1], d["k"][:1], d["v"][:1], d["g"][:1], d["beta"][:1],
                                initial_state=d["h0"][:1], **kw)
    assert torch.equal(o[:1], o1) and torch.equal(ht[:1], ht1)


def test_kda_argument_checks(ops):
    x = P.kda_inputs(1, 64, 2, 64, 64, BF)
    d = {n: t.cuda() for n, t in x.items()}
    with pytest.raises(ValueError):
        ops.chunk_kda(d["q"], d["k"], d["v"], d["g"], d["beta"], use_gate_in_kernel=True)               # no A_log
    with pytest.raises(ValueError):
        ops.chunk_kda(d["q"], d["k"], d["v"], d["g"], d["beta"], allow_neg_eigval=True)
    with pytest.raises(ValueError):
        ops.chunk_kda(d["q"], d["k"], d["v"], d["g"][..., :32], d["beta"])
    with pytest.raises(ValueError):
        ops.chunk_kda(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=d["h0"].bfloat16())
    # the safe gate needs its bound, inside [-5, 0) (triton_ascend/chunk.py:373-377)
    gate = dict(use_gate_in_kernel=True, A_log=d["A_log"], dt_bias=d["dt_bias"], safe_gate=True)
    with pytest.raises(ValueError, match="must be specified"):
        ops.chunk_kda(d["q"], d["k"], d["v"], d["g"], d["beta"], **gate)
    with pytest.raises(ValueError, match="safe range"):
        ops.chunk_kda(d["q"], d["k"], d["v"], d["g"], d["beta"], lower_bound=-6.0, **gate)


def test_kda_log_decay_in_half_precision(ops):
    """The caller hands over the log decay itself (use_gate_in_kernel=False) in the dtype of q, k, v."""
    errs = P.check_kda(ops, "cuda", 1, 200, 2, 128, 128, BF, gate_in_kernel=False, g_dtype=BF, backward=True, seed=6)
    print({n: f"{e:.2e}" for n, e in errs.items()})


@pytest.mark.parametrize("dtype,B,T,D,W,cu", [(F32, 2, 37, 16, 4, None), (BF, 1, 300, 64, 4, [0, 1, 3, 130, 131, 300])])
def test_short_convolution_module(ops, dtype, B, T, D, W, cu):
    """The KDA layer's convolution module (short_conv.py:18-218) over this package's operators: the prefill call with
    a cache, a residual and the final state, its gradients down to the nn.Conv1d parameters, then the decoding call
    (one token per sequence) on the cache it returned, against the convolution oracle."""
    import mindspeed_mm_amd as M
    from oracle import gdn_oracle as O
    print(f"short convolution {dtype} B{B} T{T} D{D} W{W} varlen={cu is not None}", flush=True)
    gen = torch.Generator().manual_seed(3)
    r = lambda *s: torch.randn(*s, generator=gen)
    N = B if cu is None else len(cu) - 1
    conv = M.ShortConvolution(D, W, bias=True, activation="silu", device="cuda", dtype=dtype)
    assert tuple(conv.weight.shape) == (D, 1, W) and tuple(conv.bias.shape) == (D,)
    w0, b0 = (r(D, 1, W) / 2).to(dtype), r(D).to(dtype)
    with torch.no_grad():
        conv.weight.copy_(w0)
        conv.bias.copy_(b0)
    x, res, cache, dy = r(B, T, D).to(dtype), r(B, T, D).to(dtype), r(N, D, W).to(dtype), r(B, T, D).to(dtype)
    cu_t = None if cu is None else torch.tensor(cu, dtype=torch.int64, device="cuda")
    xd = x.cuda().requires_grad_(True)
    y, fs = conv(xd, residual=res.cuda(), cache=cache.cuda(), output_final_state=True, cu_seqlens=cu_t)
    R = dict(x=x.float().requires_grad_(True), w=w0.float().squeeze(1).t().contiguous().requires_grad_(True),
             b=b0.float().requires_grad_(True))
    ry, rfs = O.causal_conv1d_ref(R["x"], R["w"], R["b"], res.float(), cache.float(), "silu", cu, True)
    P._err("y", y, ry, dtype, 1e-2, 1e-2)
    P._err("final_state", fs, rfs, dtype, 1e-2, 1e-2)
    y.backward(dy.cuda())
    ry.backward(dy.float())
    tol = 5e-2 * max(1.0, B * T / 256)
    P._err("dx", xd.grad, R["x"].grad, dtype, 5e-2, 1e-2)
    P._err("dweight", conv.weight.grad.squeeze(1).t(), R["w"].grad, dtype, tol, 1e-2)
    P._err("dbias", conv.bias.grad, R["b"].grad, dtype, tol, 1e-2)
    # decoding: one token per sequence; the cache is rolled in place and handed back
    x1, res1 = r(N, 1, D).to(dtype), r(N, 1, D).to(dtype)
    if cu is not None:       # packed: [1, N, D] with one token per sequence
        x1, res1 = x1.transpose(0, 1).contiguous(), res1.transpose(0, 1).contiguous()
    step_cache = fs.detach().clone()
    cu1 = None if cu is None else torch.arange(N + 1, dtype=torch.int64, device="cuda")
    with torch.no_grad():
        y1, c1 = conv(x1.cuda(), residual=res1.cuda(), cache=step_cache, output_final_state=True, cu_seqlens=cu1)
    assert c1 is step_cache and y1.shape == x1.shape
    ref_state = rfs.detach().clone()
    ry1 = O.causal_conv1d_update_ref(x1.float().reshape(N, 1, D), ref_state, w0.float().squeeze(1), b0.float(), "silu")
    P._err("step y", y1.reshape(N, 1, D), ry1 + res1.float().reshape(N, 1, D), dtype, 1e-2, 1e-2)
    P._err("step cache", step_cache, ref_state, dtype, 1e-2, 1e-2)
    with torch.no_grad():    # without a cache the step starts from zeros and returns none unless asked
        y2, c2 = conv(x1.cuda(), cu_seqlens=cu1)
    assert c2 is None and y2.shape == x1.shape


def _random_kda_case(seed):
    """A seeded random KDA problem: shape, packing and every option of the operator."""
    import random
    rnd = random.Random(1000 + seed)
    dtype = rnd.choice([BF, BF, BF, F32])
    K, V = rnd.choice([64, 128]), rnd.choice([64, 128, 192, 256])
    H = rnd.choice([1, 2, 3, 5])
    if rnd.random() < 0.5:
        B, T, cu = rnd.choice([1, 2, 3]), rnd.choice([1, 17, 64, 65, 130, 200, 333]), None
    else:
        n = rnd.choice([1, 2, 4, 7])
        lens = [rnd.choice([0, 1, 5, 63, 64, 65, 100, 129, 200]) for _ in range(n)]
        if sum(lens) == 0:
            lens[-1] = 70
        cu = [0]
        for x in lens:
            cu.append(cu[-1] + x)
        B, T = 1, cu[-1]
    kw = dict(gate_in_kernel=rnd.random() < 0.7, beta_sigmoid=rnd.random() < 0.7, l2=rnd.random() < 0.7,
              transpose_state=rnd.random() < 0.5, with_h0=rnd.random() < 0.7)
    if kw["gate_in_kernel"] and rnd.random() < 0.5:
        kw["lower_bound"] = -5.0
    if kw["beta_sigmoid"] and rnd.random() < 0.3:
        kw["allow_neg"] = True
    if dtype == BF and rnd.random() < 0.3:
        kw["g_dtype"] = torch.float32
    return dtype, B, T, H, K, V, cu, kw


@pytest.mark.parametrize("seed", range(16))
def test_kda_random_shapes(ops, seed):
    dtype, B, T, H, K, V, cu, kw = _random_kda_case(seed)
    print(f"kda random {seed}: {dtype} B{B} T{T} H{H} K{K} V{V} cu={cu} {kw}", flush=True)
    errs = P.check_kda(ops, "cuda", B, T, H, K, V, dtype, cu=cu, backward=True, seed=seed, **kw)
    print("   ", {n: f"{e:.2e}" for n, e in errs.items()}, flush=True)

