#!/usr/bin/env python3
"""Benchmark of the GDN operator path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one chunked gated-delta-rule forward + backward over the configuration the metric is quoted on
(BASELINE.json configs[1]: B=2, T=8192, H_qk=16, H_v=32, d_k=d_v=128, bf16, in-kernel q/k L2 norm, N(0,0.02)
initial state, upstream grad ~ N(0,1)); inputs are synthetic and already resident in HBM.  Prints ONE JSON line.
The step keeps the forward pass's workspace for the backward pass (skip_recompute=True, an option the reference's
operator has as well); the operator's default call (skip_recompute=False: the input-only part of the workspace is
kept, states and corrected values are rebuilt in the backward pass) is timed right after it, same K and W, and
reported beside it in roofline.path.default_mode.

  value        tokens/s of fwd+bwd (B*T / step time), measured without per-kernel instrumentation
  roofline     the kernel with the largest share of the step: its algorithmic HBM bytes per launch divided by its
               mean launch duration, taken live with HIP events on the launch stream in a second, instrumented
               pass over the same K steps; peak = MI355X HBM3E (8 TB/s).  Its matmul FLOP rate against the dense
               bf16 MFMA peak (2.5 PFLOP/s) is given beside it
  cpu_baseline the CPU oracle (PyTorch fp32 restatement of the reference's torch path, autograd backward) timed on
               this box's host cores on a bounded sample of the same workload
               roofline.path gives the whole step against the two machine peaks: the reference's FLOP formula
               against the bf16 MFMA peak, and the minimal HBM bytes of the operator (inputs and outputs only)
               against the HBM peak, with the traffic the kernels really move beside it
  aux          the per-kernel split, the other BASELINE configurations (packed sequences, the long-context shape,
               the CPU-runnable case) and the HBM-bound siblings (batch-256 decode, the packed conv1d, the gated
               RMSNorm) with their achieved GB/s
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "mindspeed-mm_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

CFG = dict(B=2, T=8192, Hqk=16, Hv=32, K=128, V=128, C=64)

# HBM bytes per launch of each kernel on CFG, read + written, from the hardware counters FETCH_SIZE and WRITE_SIZE
# (rocprofv3 --pmc, one run per counter, each scaled by what the same counter reads for a 512 MiB copy).  They are
# collected offline and live in the tracked summary named below, which is the only place they are written down:
# this script reads its table of the benchmark shape and reports the figures beside the live timings.
TRAFFIC_SOURCE = "profiles/chunk_fwd_bwd_B2_T8192_bf16_hbm_traffic.md"


def measured_traffic_bytes_per_launch():
    """{kernel: bytes per launch} from the first table of TRAFFIC_SOURCE (rows `| kernel<...> | ... | bytes |`, the last
    column being bytes per launch); empty when the file is missing, and the traffic fields are then null."""
    out, in_main = {}, False
    try:
        with open(os.path.join(ROOT, TRAFFIC_SOURCE)) as f:
            lines = f.read().splitlines()
    except OSError:
        return out
    for ln in lines:
        if ln.startswith("## "):
            in_main = ln.startswith("## Chunk fwd+bwd at the benchmark shape")
        elif in_main and ln.startswith("| chunk_"):
            cells = [c.strip() for c in ln.strip().strip("|").split("|")]
            try:
                out[cells[0].split("<")[0]] = int(cells[-1])
            except ValueError:
                pass
    return out


CLOCK_RAMP_S = 0.5   # untimed run of the benchmark step before the warm-up steps (see main)


def ref_formula_flops(tokens, Hv, K, V, C=64):
    """fwd+bwd FLOP of the reference's own counter (mindspeed_mm/fsdp/tools/flops_tool/flops_qwen3_5.py:170-204)."""
    return 3 * 2 * tokens * Hv * (3 * V * C + 2 * K * C + 3 * K * V)


def minimal_bytes(B, T, N, Hqk, Hv, K, V, e=2):
    """HBM bytes the operator cannot avoid, fwd+bwd: every input read once and every output written once per pass
    (q, k, v, o and their gradients in `e` bytes, g, beta and the states in fp32), grouped q/k heads read natively."""
    tok = B * T
    fwd = tok * (e * (2 * Hqk * K + 2 * Hv * V) + 8 * Hv) + 2 * 4 * N * Hv * K * V
    bwd = tok * (e * (4 * Hqk * K + 3 * Hv * V) + 16 * Hv) + 2 * 4 * N * Hv * K * V
    return fwd + bwd


def kernel_matmul_flops(K, V, C=64):
    """Matmul FLOP each kernel performs per (chunk, value head): 2*M*N*K summed over its contractions."""
    g = lambda m, n, k: 2 * m * n * k
    return {
        "chunk_prep_kernel": 2 * g(C, C, K),                               # K K^T, Q K^T (the solve is not counted)
        # K S, Tm z, (decayed K)^T V', Q S, Aq V'
        "chunk_state_kernel": g(C, V, K) + g(C, V, C) + g(K, V, C) + g(C, V, K) + g(C, V, C),
        # Aq^T dO, K dS, Tm^T dV', Q^T dO, K^T R
        "chunk_state_bwd_kernel": g(C, V, C) + g(C, V, K) + g(C, V, C) + 2 * g(K, V, C),
        # dO V'^T, dO S^T, V' dS^T, dV' S^T, ds K, ds^T Q | Tm^T dW, dW K^T, Tm^T dV', dV' V^T, dTm Tm^T, Tm^T X, dM K, dM^T K
        "chunk_bwd_local_kernel": g(C, C, V) + 3 * g(C, K, V) + 2 * g(C, K, C)
                                  + g(C, K, C) + g(C, C, K) + g(C, V, C) + g(C, C, V) + 2 * g(C, C, C) + 2 * g(C, K, C),
    }


def kernel_algorithmic_bytes(K, V, grp, e=2, C=64):
    """HBM bytes each kernel has to move per (chunk, value head) given its interface: every input tile read once, every
    output tile written once (bf16 tiles, fp32 row vectors).  tk = [64,K] tile, tv = [64,V] tile, st = [K,V] state,
    cc = [64,64] tile (three of its four 32x32 tiles where it is triangular), row = 64 fp32 values."""
    tk, tv, st, cc, row = C * K * e, C * V * e, K * V * e, C * C * e, C * 4
    tri = 3 * cc // 4
    return {
        # g, beta -> G, Tm, Aq; once per q/k group: q, k -> K, Q^T tiles, 1/|q|, 1/|k|
        "chunk_prep_kernel": 2 * row + row + 2 * cc + (2 * tk + 2 * tk + 2 * row) // grp,
        # K, Q^T (per group), Tm, Aq, v, G, beta -> o, v_new, state before the chunk
        "chunk_state_kernel": 2 * tk // grp + 2 * tri + tv + 2 * row + tv + tv + st,
        # K, Q^T (per group), Tm, Aq, dO, G, beta -> dv_new, dS
        "chunk_state_bwd_kernel": 2 * tk // grp + 2 * tri + tv + 2 * row + tv + st,
        # v_new, dv_new, dO, S, dS, v, K, q, Tm, row vectors -> dv, dg, dbeta, dq/dk (written by the first head of a
        # group, read and re-written by the others)
        "chunk_bwd_local_kernel": 3 * tv + 2 * st + tv + 2 * tk + cc + 5 * row + tv + 2 * row
                                  + 2 * tk * (2 * grp - 1) // grp,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-side oracle timing")
    ap.add_argument("--no-aux", action="store_true", help="skip the decode / conv1d side measurements")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a 512 MiB device-to-device copy a few times (a kernel of known traffic for scaling "
                         "hardware counters collected over this command)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the operator path has no collective and this build runs on a single "
              "MI355X; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no host execution path for the operators)", file=sys.stderr)
        sys.exit(1)
    from mindspeed_mm_amd import _lib
    from mindspeed_mm_amd.inputs import gdn_inputs, packed_lengths
    from mindspeed_mm_amd.ops import _default_ops

    ops = _default_ops()
    lib = ops.lib
    dev = torch.device("cuda:0")
    c = CFG
    tokens = c["B"] * c["T"]
    x = gdn_inputs(c["B"], c["T"], c["Hqk"], c["Hv"], c["K"], c["V"], torch.bfloat16, seed=0)
    d = {n: t.to(dev) for n, t in x.items()}
    leaves = [d[n].requires_grad_(True) for n in ("q", "k", "v", "g", "beta", "h0")]

    def step(skip_recompute=True):
        o, ht = ops.chunk_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=d["h0"],
                                           output_final_state=True, use_qk_l2norm_in_kernel=True,
                                           skip_recompute=skip_recompute)
        return torch.autograd.grad([o], leaves, [d["do"]])

    # The GPU raises its clocks over the first half second of work of a process: steps timed right after start-up run
    # about 3 % slower than the same steps a second later.  The figure reported is the steady state, so the same step
    # runs untimed for CLOCK_RAMP_S before the W warm-up steps and the K timed ones.
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < CLOCK_RAMP_S:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    value = tokens / (ms_per_step * 1e-3)
    # the operator's default call, timed the same way
    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(False)
    torch.cuda.synchronize()
    ms_default = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- spread of the step time: each of max(steps, 50) further steps bracketed by events on the launch stream ----
    nspread = max(args.steps, 50)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(nspread)]
    for a, b in evs:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    per_step = sorted(a.elapsed_time(b) for a, b in evs)
    spread = {"n": nspread, "median_ms": round(per_step[nspread // 2], 4), "p10_ms": round(per_step[nspread // 10], 4),
              "p90_ms": round(per_step[(9 * nspread) // 10], 4)}

    # ---- instrumented pass: per-kernel durations from HIP events on the launch stream ----
    lib.gdn_profile_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    timings = _lib.kernel_timings(lib)
    lib.gdn_profile_enable(0)
    nchunk_heads = c["B"] * (c["T"] // c["C"]) * c["Hv"]
    per_kernel = {}
    total_kernel_ms = sum(ms for ms, _ in timings.values()) / args.steps
    flops = kernel_matmul_flops(c["K"], c["V"])
    for name, (ms, cnt) in timings.items():
        # a kernel launched several times per step (one launch per value head of a q/k group) splits the step's work
        # evenly over its launches: avg_ms is per launch, step_ms per step
        launches = cnt / args.steps
        avg, step_ms = ms / cnt, ms / args.steps
        per_kernel[name] = {"avg_ms": round(avg, 4), "launches_per_step": round(launches, 2),
                            "step_ms": round(step_ms, 4), "share": round(step_ms / total_kernel_ms, 3)}
        if name in flops:
            per_kernel[name]["tflops"] = round(flops[name] * nchunk_heads / (step_ms * 1e-3) / 1e12, 1)
    abytes = kernel_algorithmic_bytes(c["K"], c["V"], c["Hv"] // c["Hqk"])
    for name in per_kernel:
        if name in abytes:
            per_kernel[name]["GBps"] = round(abytes[name] * nchunk_heads / (per_kernel[name]["step_ms"] * 1e-3) / 1e9, 1)
    # The dominant kernel's arithmetic intensity (matmul FLOP / algorithmic byte) is far below the ridge of the machine
    # (2.5 PFLOP/s / 8 TB/s = 312 FLOP/B), like that of every kernel of the path: the roofline that bounds it is HBM.
    dom = max((n for n in per_kernel if n in abytes), key=lambda n: per_kernel[n]["step_ms"])
    launches = per_kernel[dom]["launches_per_step"]
    bytes_per_launch = abytes[dom] * nchunk_heads / launches
    dom_gbps = bytes_per_launch / (per_kernel[dom]["avg_ms"] * 1e-3) / 1e9
    dom_tflops = flops[dom] * nchunk_heads / (per_kernel[dom]["step_ms"] * 1e-3) / 1e12
    path_tflops = ref_formula_flops(tokens, c["Hv"], c["K"], c["V"]) / (ms_per_step * 1e-3) / 1e12
    min_bytes = minimal_bytes(c["B"], c["T"], c["B"], c["Hqk"], c["Hv"], c["K"], c["V"])
    interface_total = sum(abytes[n] * nchunk_heads for n in per_kernel if n in abytes)
    traffic_table = measured_traffic_bytes_per_launch()
    traffic_total = None
    if all(n in traffic_table for n in per_kernel if n in abytes):
        traffic_total = sum(traffic_table[n] * per_kernel[n]["launches_per_step"] for n in per_kernel if n in abytes)
    # the whole step against both roofs: the operator's minimal bytes (inputs and outputs only) and the reference's
    # FLOP count say what an ideal implementation would need; the kernels' own interfaces move more (intermediates
    # between the launches), which is what the per-kernel figures above are measured against
    path = {"ms_per_step": round(ms_per_step, 4),
            "minimal_bytes_per_step": int(min_bytes),
            "frac_hbm_minimal": round(min_bytes / (ms_per_step * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
            "flops_ref_formula_per_step": ref_formula_flops(tokens, c["Hv"], c["K"], c["V"]),
            "tflops_ref_formula": round(path_tflops, 2),
            "frac_mfma_ref_formula": round(path_tflops / PEAK_BF16_TFLOPS, 4),
            "kernel_interface_bytes_per_step": int(interface_total),
            "interface_over_minimal": round(interface_total / min_bytes, 2),
            "traffic_per_step_total": None if traffic_total is None else int(traffic_total),
            "traffic_over_minimal": None if traffic_total is None else round(traffic_total / min_bytes, 2),
            # skip_recompute=False, the call a user of the reference makes without changing anything
            "default_mode": {"ms_per_step": round(ms_default, 4), "tokens_per_s": round(tokens / (ms_default * 1e-3), 1),
                             "tflops_ref_formula": round(path_tflops * ms_per_step / ms_default, 2),
                             "frac_mfma_ref_formula": round(path_tflops * ms_per_step / ms_default / PEAK_BF16_TFLOPS, 4),
                             "frac_hbm_minimal": round(min_bytes / (ms_default * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                             "kept_between_passes_bytes": int(lib.gdn_chunk_workspace_bytes(
                                 c["B"], c["T"], c["B"], c["Hqk"], c["Hv"], c["K"], c["V"], 1, 2)),
                             "stored_mode_kept_bytes": int(lib.gdn_chunk_workspace_bytes(
                                 c["B"], c["T"], c["B"], c["Hqk"], c["Hv"], c["K"], c["V"], 1, 1))}}
    roofline = {"kernel": dom, "bound": "hbm", "achieved": round(dom_gbps, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(dom_gbps / PEAK_HBM_GBS, 4), "traffic": traffic_table.get(dom),
                "traffic_source": TRAFFIC_SOURCE + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, collected offline)",
                "algorithmic_bytes_per_launch": int(bytes_per_launch), "launches_per_step": launches,
                "avg_launch_ms": per_kernel[dom]["avg_ms"],
                "flop_per_byte": round(flops[dom] / abytes[dom], 1), "tflops": round(dom_tflops, 1),
                "frac_of_bf16_mfma_peak": round(dom_tflops / PEAK_BF16_TFLOPS, 4), "path": path}

    aux = {"path_tflops_ref_formula": round(path_tflops, 2),
           "path_frac_of_bf16_mfma_peak": round(path_tflops / PEAK_BF16_TFLOPS, 4),
           "kernel_ms_sum": round(total_kernel_ms, 3), "step_time_spread": spread, "kernels": per_kernel,
           "clock_ramp_before_warmup_s": CLOCK_RAMP_S}

    if not args.no_aux:
        # ---- decode: batch 256, 64 consecutive steps, state updated in place (BASELINE.json configs[3]) ----
        B3 = 256
        y = gdn_inputs(B3, 64, c["Hqk"], c["Hv"], c["K"], c["V"], torch.bfloat16, seed=3)
        e = {n: t.to(dev) for n, t in y.items()}
        state = e["h0"].clone()
        tok = [{n: e[n][:, t:t + 1].contiguous() for n in ("q", "k", "v", "g", "beta")} for t in range(64)]

        def decode64():
            for t in tok:
                ops.fused_recurrent_gated_delta_rule(t["q"], t["k"], t["v"], t["g"], t["beta"], initial_state=state,
                                                     output_final_state=True, use_qk_l2norm_in_kernel=True,
                                                     inplace_state=True)
        decode64()
        lib.gdn_profile_enable(1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        decode64()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / 64
        tm = _lib.kernel_timings(lib)["recurrent_kernel"]
        lib.gdn_profile_enable(0)
        kern_s = tm[0] / tm[1] * 1e-3
        # per step: fp32 state in + out, bf16 q,k,v,o, fp32 g,beta
        step_bytes = 2 * B3 * c["Hv"] * c["K"] * c["V"] * 4 + B3 * (2 * c["Hqk"] * c["K"] + 2 * c["Hv"] * c["V"]) * 2 \
            + 2 * B3 * c["Hv"] * 4
        aux["decode_b256"] = {"kernel_us": round(kern_s * 1e6, 1), "GBps": round(step_bytes / kern_s / 1e9, 1),
                              "frac_of_hbm_peak": round(step_bytes / kern_s / 1e9 / PEAK_HBM_GBS, 4),
                              "tokens_per_s_wall": round(B3 / wall, 1), "bytes_per_step": step_bytes}
        # ---- one decode step of the layer between the projections and the gated norm, batch 256: convolution update +
        # rule on its unsplit output with in-kernel gates (2 launches) against the same from separate operators ----
        nq3, nv3 = c["Hqk"] * c["K"], c["Hv"] * c["V"]
        D3 = 2 * nq3 + nv3
        g3 = torch.Generator().manual_seed(4)
        mx3 = torch.randn(B3, 1, D3, generator=g3).to(dev, torch.bfloat16)
        a3 = torch.randn(B3, 1, c["Hv"], generator=g3).to(dev, torch.bfloat16)
        b3 = torch.randn(B3, 1, c["Hv"], generator=g3).to(dev, torch.bfloat16)
        cw3 = (torch.randn(D3, 4, generator=g3) / 2).to(dev, torch.bfloat16)
        cb3 = torch.zeros(D3, device=dev, dtype=torch.bfloat16)
        Al3, db3 = torch.zeros(c["Hv"], device=dev), torch.full((c["Hv"],), -3.0, device=dev)
        conv3 = torch.zeros(B3, D3, 4, device=dev, dtype=torch.bfloat16)

        def layer_step_fused():
            ops.decode_step(mx3, a3, b3, conv3, state, cw3, cb3, Al3, db3, c["Hqk"], c["Hv"], c["K"], c["V"])

        def layer_step_separate():
            y_ = ops.causal_conv1d_update(mx3, conv3, cw3, cb3, "silu")
            q_, k_, v_ = torch.split(y_, [nq3, nq3, nv3], dim=-1)
            g_, be_ = ops.gdn_gates(a3, b3, Al3, db3)
            ops.fused_recurrent_gated_delta_rule(q_.reshape(B3, 1, c["Hqk"], c["K"]), k_.reshape(B3, 1, c["Hqk"], c["K"]),
                                                 v_.reshape(B3, 1, c["Hv"], c["V"]), g_, be_, initial_state=state,
                                                 output_final_state=True, use_qk_l2norm_in_kernel=True,
                                                 inplace_state=True)

        def wall_us(fn, n=64):
            for _ in range(8):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / n * 1e6
        aux["decode_layer_step_b256"] = {"conv_update_plus_rule_us": round(wall_us(layer_step_fused), 1),
                                         "separate_operators_us": round(wall_us(layer_step_separate), 1)}
        del mx3, conv3
        del e, y, state, tok
        # ---- packed causal conv1d fwd+bwd (BASELINE.json configs[2]: 32768 tokens, D=8192, W=4, SiLU) ----
        cu = torch.tensor(packed_lengths(), dtype=torch.int64, device=dev)
        D = 2 * c["Hqk"] * c["K"] + c["Hv"] * c["V"]
        gen = torch.Generator().manual_seed(2)
        xx = torch.randn(1, 32768, D, generator=gen).to(dev, torch.bfloat16).requires_grad_(True)
        ww = (torch.randn(4, D, generator=gen) / 2).to(dev, torch.bfloat16).requires_grad_(True)
        dy = torch.randn(1, 32768, D, generator=gen).to(dev, torch.bfloat16)

        def conv_step():
            yy, _ = ops.causal_conv1d(xx, ww, None, None, None, "silu", cu, False)
            torch.autograd.grad([yy], [xx, ww], [dy])
        conv_step()
        lib.gdn_profile_enable(1)
        for _ in range(5):
            conv_step()
        torch.cuda.synchronize()
        tm = _lib.kernel_timings(lib)
        lib.gdn_profile_enable(0)
        nb = xx.numel() * 2
        f_s = tm["conv1d_fwd_kernel"][0] / tm["conv1d_fwd_kernel"][1] * 1e-3
        b_s = tm["conv1d_bwd_kernel"][0] / tm["conv1d_bwd_kernel"][1] * 1e-3
        aux["conv1d_packed"] = {"fwd_ms": round(f_s * 1e3, 3), "fwd_GBps": round(2 * nb / f_s / 1e9, 1),
                                "bwd_ms": round(b_s * 1e3, 3), "bwd_GBps": round(3 * nb / b_s / 1e9, 1)}
        del xx, ww, dy
        # ---- gated RMSNorm on the chunk output of the benchmark shape: [tokens * H_v, d_v] rows, fwd+bwd ----
        rows = tokens * c["Hv"]
        xn = torch.randn(rows, c["V"], generator=gen).to(dev, torch.bfloat16).requires_grad_(True)
        zn = torch.randn(rows, c["V"], generator=gen).to(dev, torch.bfloat16).requires_grad_(True)
        wn = torch.ones(c["V"], device=dev, dtype=torch.bfloat16, requires_grad=True)
        dyn = torch.randn(rows, c["V"], generator=gen).to(dev, torch.bfloat16)

        def norm_step():
            yn = ops.rms_norm_gated(xn, zn, wn, 1e-6)
            torch.autograd.grad([yn], [xn, zn, wn], [dyn])
        norm_step()
        lib.gdn_profile_enable(1)
        for _ in range(5):
            norm_step()
        torch.cuda.synchronize()
        tm = _lib.kernel_timings(lib)
        lib.gdn_profile_enable(0)
        nb = xn.numel() * 2
        f_s = tm["rmsnorm_gated_fwd_kernel"][0] / tm["rmsnorm_gated_fwd_kernel"][1] * 1e-3
        b_s = tm["rmsnorm_gated_bwd_kernel"][0] / tm["rmsnorm_gated_bwd_kernel"][1] * 1e-3
        aux["rmsnorm_gated"] = {"fwd_ms": round(f_s * 1e3, 3), "fwd_GBps": round(3 * nb / f_s / 1e9, 1),
                                "bwd_ms": round(b_s * 1e3, 3), "bwd_GBps": round(5 * nb / b_s / 1e9, 1)}
        del xn, zn, dyn

        # ---- the rule inside the layer: on the unsplit convolution output (read and written in place) against the
        # reference's glue (split -> contiguous copies -> rule -> concatenated gradient), and the gate recipe ----
        nq, nv = c["Hqk"] * c["K"], c["Hv"] * c["V"]
        mixed = torch.cat([x[n].reshape(c["B"], c["T"], -1) for n in ("q", "k", "v")], dim=-1).to(dev)
        mixed.requires_grad_(True)
        gg, bb, hh0 = (d[n].detach().clone().requires_grad_(True) for n in ("g", "beta", "h0"))

        def unsplit_step():
            o_, _ = ops.chunk_gated_delta_rule_qkv(mixed, gg, bb, c["Hqk"], c["Hv"], c["K"], c["V"], initial_state=hh0,
                                                   output_final_state=True, use_qk_l2norm_in_kernel=True)
            torch.autograd.grad([o_], [mixed, gg, bb, hh0], [d["do"]])

        def split_step():
            q_, k_, v_ = torch.split(mixed, [nq, nq, nv], dim=-1)
            o_, _ = ops.chunk_gated_delta_rule(q_.reshape(c["B"], c["T"], c["Hqk"], c["K"]).contiguous(),
                                               k_.reshape(c["B"], c["T"], c["Hqk"], c["K"]).contiguous(),
                                               v_.reshape(c["B"], c["T"], c["Hv"], c["V"]).contiguous(), gg, bb,
                                               initial_state=hh0, output_final_state=True, use_qk_l2norm_in_kernel=True)
            torch.autograd.grad([o_], [mixed, gg, bb, hh0], [d["do"]])

        def wall_ms(fn, n=10, warm=3):
            for _ in range(warm):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / n * 1e3
        def prefill_step():
            with torch.no_grad():
                ops.chunk_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=d["h0"],
                                           output_final_state=True, use_qk_l2norm_in_kernel=True)
        pf = wall_ms(prefill_step, 20)
        aux["forward_only"] = {"ms": round(pf, 4), "tokens_per_s": round(tokens / (pf * 1e-3), 1)}
        two_streams = ops.two_stream_backward
        ops.two_stream_backward = False
        rc = wall_ms(lambda: step(False), 20)
        ops.two_stream_backward = two_streams
        aux["default_mode_on_one_stream"] = {
            "ms_per_step": round(rc, 4), "tokens_per_s": round(tokens / (rc * 1e-3), 1),
            "note": "skip_recompute=False with the backward pass's rebuild of states and corrected values queued in "
                    "front of the reverse recurrence instead of beside it on a second stream"}
        zg = torch.randn(c["B"], c["T"], c["Hv"], c["V"], generator=gen).to(dev, torch.bfloat16)
        nw = torch.ones(c["V"], device=dev, dtype=torch.bfloat16)

        def prefill_norm_fused():
            with torch.no_grad():
                ops.chunk_gated_delta_rule_norm(d["q"], d["k"], d["v"], d["g"], d["beta"], zg, nw,
                                                initial_state=d["h0"], output_final_state=True,
                                                use_qk_l2norm_in_kernel=True, in_output_kernel=True)

        def prefill_norm_separate():
            with torch.no_grad():
                o_, _ = ops.chunk_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=d["h0"],
                                                   output_final_state=True, use_qk_l2norm_in_kernel=True)
                ops.rms_norm_gated(o_, zg, nw, 1e-6)
        def kernel_sum_ms(fn, n=10):
            """GPU time of one call: the library's per-kernel event timings summed (no launch gaps, no host time)."""
            torch.cuda.synchronize()
            lib.gdn_profile_enable(1)
            for _ in range(n):
                fn()
            torch.cuda.synchronize()
            tm = _lib.kernel_timings(lib)
            lib.gdn_profile_enable(0)
            return sum(ms for ms, _ in tm.values()) / n
        # the host-side generation of the gate above leaves the GPU idle: longer warm-up before these
        aux["forward_only_with_gated_norm"] = {
            "separate_operators_ms": round(wall_ms(prefill_norm_separate, 20, 20), 4),
            "norm_in_output_kernel_ms": round(wall_ms(prefill_norm_fused, 20, 20), 4),
            "separate_operators_kernel_ms": round(kernel_sum_ms(prefill_norm_separate), 4),
            "norm_in_output_kernel_kernel_ms": round(kernel_sum_ms(prefill_norm_fused), 4)}
        del zg
        aux["rule_in_layer"] = {"unsplit_qkv_ms": round(wall_ms(unsplit_step), 4),
                                "split_with_copies_ms": round(wall_ms(split_step), 4)}
        del mixed
        aa = torch.randn(c["B"], c["T"], c["Hv"], generator=gen).to(dev, torch.bfloat16).requires_grad_(True)
        ab = torch.randn(c["B"], c["T"], c["Hv"], generator=gen).to(dev, torch.bfloat16).requires_grad_(True)
        A_log = torch.zeros(c["Hv"], device=dev, requires_grad=True)
        dt_b = torch.full((c["Hv"],), -3.0, device=dev, requires_grad=True)
        dgg = torch.randn(c["B"], c["T"], c["Hv"], generator=gen).to(dev)

        def gates_step():
            g_, b_ = ops.gdn_gates(aa, ab, A_log, dt_b)
            torch.autograd.grad([g_, b_], [aa, ab, A_log, dt_b], [dgg, dgg.to(torch.bfloat16)])

        def gates_eager_step():
            b_ = ab.sigmoid()
            g_ = -A_log.float().exp() * torch.nn.functional.softplus(aa.float() + dt_b)
            torch.autograd.grad([g_, b_], [aa, ab, A_log, dt_b], [dgg, dgg.to(torch.bfloat16)])
        # 0.5 M elements: both wall times are set by host-side launch work; the kernels' own time is given beside them
        aux["gates"] = {"fused_fwd_bwd_ms": round(wall_ms(gates_step, 100), 4),
                        "fused_fwd_bwd_kernel_ms": round(kernel_sum_ms(gates_step, 20), 4),
                        "torch_elementwise_fwd_bwd_ms": round(wall_ms(gates_eager_step, 100), 4)}

    if not args.no_aux:
        # ---- the other BASELINE configurations (parity-tested at full size in tests/test_gpu_full_size.py) ----
        def fwd_bwd_ms(dd, cu=None, n=5, warm=2, skip=True):
            L = [dd[m].requires_grad_(True) for m in ("q", "k", "v", "g", "beta", "h0")]

            def f():
                o_, _ = ops.chunk_gated_delta_rule(dd["q"], dd["k"], dd["v"], dd["g"], dd["beta"], initial_state=dd["h0"],
                                                   output_final_state=True, use_qk_l2norm_in_kernel=True, cu_seqlens=cu,
                                                   skip_recompute=skip)
                torch.autograd.grad([o_], L, [dd["do"]])
            for _ in range(warm):
                f()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                f()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / n * 1e3
        del d, leaves
        torch.cuda.empty_cache()
        cu2 = packed_lengths()
        x2 = gdn_inputs(1, cu2[-1], c["Hqk"], c["Hv"], c["K"], c["V"], torch.bfloat16, seed=2, N=len(cu2) - 1)
        d2 = {n: t.to(dev) for n, t in x2.items()}
        ms2 = fwd_bwd_ms(d2, torch.tensor(cu2, dtype=torch.int64, device=dev))
        fl2 = ref_formula_flops(cu2[-1], c["Hv"], c["K"], c["V"])
        aux["config2_packed_24_sequences_32768_tokens"] = {
            "ms_per_step": round(ms2, 4), "tokens_per_s": round(cu2[-1] / (ms2 * 1e-3), 1),
            "frac_mfma_ref_formula": round(fl2 / (ms2 * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)}
        del d2, x2
        torch.cuda.empty_cache()
        T4, Hv4, V4 = 65536, 64, 256
        x4 = gdn_inputs(1, T4, c["Hqk"], Hv4, c["K"], V4, torch.bfloat16, seed=4, a_log=(0.5, 2.0), dt_bias=(-6.0, -4.0))
        d4 = {n: t.to(dev) for n, t in x4.items()}
        del x4
        ms4 = fwd_bwd_ms(d4)
        fl4 = 3 * 2 * T4 * Hv4 * (3 * V4 * 64 + 2 * c["K"] * 64 + 3 * c["K"] * V4)
        aux["config4_T65536_Hv64_dv256"] = {
            "ms_per_step": round(ms4, 3), "tokens_per_s": round(T4 / (ms4 * 1e-3), 1),
            "frac_mfma_ref_formula": round(fl4 / (ms4 * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)}
        del d4
        torch.cuda.empty_cache()
        # KDA (one decay per key channel) at the benchmark's token count and the Kimi linear-attention head shape
        # (mindspeed_mm/fsdp/models/kimi_k3/modeling_kimi_linear.py:549-596: 32 heads of 128), with the layer's
        # options: raw gate and beta, l2 norm in the kernel, [N,H,V,K] states
        from mindspeed_mm_amd.inputs import kda_inputs
        Hk = c["Hv"]
        xk = kda_inputs(c["B"], c["T"], Hk, c["K"], c["V"], torch.bfloat16, seed=5)
        dk_ = {n: t.to(dev) for n, t in xk.items()}
        del xk
        kl = {n: dk_[n].clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta", "A_log", "dt_bias")}
        kh0 = dk_["h0"].transpose(-1, -2).contiguous().requires_grad_(True)
        kda_kw = dict(initial_state=kh0, output_final_state=True, use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True,
                      use_beta_sigmoid_in_kernel=True, transpose_state_layout=True, A_log=kl["A_log"], dt_bias=kl["dt_bias"])

        def kda_step():
            o_, _ = ops.chunk_kda(kl["q"], kl["k"], kl["v"], kl["g"], kl["beta"], **kda_kw)
            torch.autograd.grad([o_], list(kl.values()) + [kh0], [dk_["do"]])

        def kda_prefill():
            with torch.no_grad():
                ops.chunk_kda(kl["q"], kl["k"], kl["v"], kl["g"], kl["beta"], **kda_kw)
        kms, kpf = wall_ms(kda_step, 30, 5), wall_ms(kda_prefill, 30, 5)
        torch.cuda.synchronize()
        lib.gdn_profile_enable(1)
        for _ in range(5):
            kda_step()
        torch.cuda.synchronize()
        ktm = _lib.kernel_timings(lib)
        lib.gdn_profile_enable(0)
        aux["kda_B2_T8192_H32_d128"] = {
            "fwd_bwd_ms": round(kms, 4), "tokens_per_s": round(tokens / (kms * 1e-3), 1), "forward_only_ms": round(kpf, 4),
            "kernels_ms_per_step": {n: round(ms / 5, 4) for n, (ms, _) in ktm.items()}}
        del dk_, kl, kh0
        torch.cuda.empty_cache()

    if args.calibrate_copy:
        src = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    cpu = None
    if not args.no_cpu_baseline:
        from oracle import gdn_oracle as O
        # BASELINE configs[0], the reference's own CPU-runnable case: forward only, fp32, B=1 T=512 H=4 d=64
        x0 = gdn_inputs(1, 512, 4, 4, 64, 64, torch.float32, seed=0, l2norm_in_kernel=False)
        t0 = time.perf_counter()
        for _ in range(3):
            O.chunk_gated_delta_rule_ref(x0["q"], x0["k"], x0["v"], x0["g"], x0["beta"], output_final_state=True)
        dt0 = (time.perf_counter() - t0) / 3
        aux["config0_cpu_forward_fp32"] = {"ms": round(dt0 * 1e3, 2), "tokens_per_s": round(512 / dt0, 1),
                                           "cores": torch.get_num_threads()}
        Ts = 8192
        sample = {n: x[n][:1, :Ts] for n in ("q", "k", "v", "g", "beta", "do")}
        L = {n: sample[n].float().requires_grad_(True) for n in ("q", "k", "v", "g", "beta")}
        h0 = x["h0"][:1].clone().requires_grad_(True)
        t0 = time.perf_counter()
        o, _ = O.chunk_gated_delta_rule_ref(L["q"], L["k"], L["v"], L["g"], L["beta"], initial_state=h0,
                                            output_final_state=True, use_qk_l2norm_in_kernel=True)
        torch.autograd.grad([o], list(L.values()) + [h0], [sample["do"].float()])
        dt = time.perf_counter() - t0
        cpu = {"value": round(Ts / dt, 1), "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
               "sample": f"one of the two batch rows at full length: B=1, T={Ts}, H_qk=16, H_v=32, d=128, fp32, "
                         f"fwd+bwd once ({dt:.1f} s)"}

    out = {
        "metric": "GDN chunk fwd+bwd tokens/sec (H=32,d=128,bf16) on 1 GPU",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "GDN chunk forward+backward, B=2 T=8192 H_qk=16 H_v=32 d_k=d_v=128 chunk=64, "
                               "use_qk_l2norm_in_kernel, initial state N(0,0.02), native grouped q/k heads, "
                               "skip_recompute=True (forward workspace kept for the backward pass); the default call "
                               "(skip_recompute=False) is timed beside it: roofline.path.default_mode",
                   "global_batch": c["B"], "seq_len": c["T"], "parallelism": "single GPU"},
        "roofline": roofline, "cpu_baseline": cpu, "aux": aux,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
