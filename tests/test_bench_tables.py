"""bench.py's static tables: the measured-traffic figures it reports come from the tracked counter summary, and its
byte / FLOP models name the kernels that the library times."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402


def test_traffic_table_is_read_from_the_tracked_summary():
    t = bench.measured_traffic_bytes_per_launch()
    c = bench.CFG
    grp = c["Hv"] // c["Hqk"]
    algo = bench.kernel_algorithmic_bytes(c["K"], c["V"], grp)
    units = c["B"] * (c["T"] // c["C"]) * c["Hv"]
    assert set(t) == set(algo)
    for name, measured in t.items():
        launches = grp if name == "chunk_bwd_local_kernel" else 1
        modelled = algo[name] * units / launches
        # the counters may read somewhat more than the interface bytes (partial lines, re-reads), never far less
        assert 0.9 * modelled < measured < 1.5 * modelled, (name, measured, modelled)


def test_flop_and_byte_models_cover_the_same_kernels():
    c = bench.CFG
    assert set(bench.kernel_matmul_flops(c["K"], c["V"])) == set(bench.kernel_algorithmic_bytes(c["K"], c["V"], 2))
    # the reference's counter at the benchmark shape (flops_qwen3_5.py:170-204): 3 * 2 * tokens * Hv * (...)
    assert bench.ref_formula_flops(16384, 32, 128, 128) == 3 * 2 * 16384 * 32 * (3 * 128 * 64 + 2 * 128 * 64 + 3 * 128 * 128)
