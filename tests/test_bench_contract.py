"""bench.py's command-line contract that can be checked without a GPU: more than one GPU is refused with a message
(this build measures one GPU), and the workload table prices FLOPs by the documented formulas."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_algorithmic_flops_of_the_workloads():
    sys.path.insert(0, ROOT)
    import bench
    T, d, f, E, k, r = 4096, 4096, 14336, 8, 2, 16
    R = T * k
    base = 6 * R * d * f
    assert bench.flops(T, d, f, E, k, 0, False) == base + 2 * T * d * E                      # forward, no adapters
    lora = 6 * R * r * (d + f)
    assert bench.flops(T, d, f, E, k, r, True) == 2 * base + 2 * T * d * E + 2 * lora + 12 * R * r * (d + f)
    assert bench.flops(T, d, f, E, k, 0, True, True) == 3 * base + 2 * T * d * E             # full fine-tuning adds dW
    assert abs(bench.flops(T, d, f, E, k, r, True) - 5.830e12) / 5.830e12 < 1e-3              # the figure quoted for the default workload
    for name, cfg in bench.WORKLOADS.items():
        assert {"T", "d", "f", "E", "k", "r", "bwd", "skew", "desc"} <= set(cfg), name


def test_flops_of_the_expert_parallel_share_and_the_tiny_configuration():
    sys.path.insert(0, ROOT)
    import bench
    d, f, r = 4096, 14336, 16
    ep = bench.WORKLOADS["ep_share_fwd_bwd_lora"]
    assert (ep["T"], ep["E"], ep["k"], ep["r"], ep["bwd"]) == (8192, 2, 1, 16, True)
    R = 8192
    # the Mixtral fwd+bwd+LoRA formula on 8192 rows, without the router (it runs on the other side of the exchange)
    want = 12 * R * d * f + 24 * R * r * (d + f)
    got = bench.flops(ep["T"], ep["d"], ep["f"], ep["E"], ep["k"], ep["r"], ep["bwd"], False, True)
    assert got == want and abs(got - 5.830e12) / 5.830e12 < 1e-3
    tiny = bench.WORKLOADS["tiny_fp32_fwd"]
    assert (tiny["T"], tiny["d"], tiny["f"], tiny["E"], tiny["k"], tiny["dtype"], tiny["bwd"]) == (256, 128, 256, 4, 2, "fp32", False)
    got = bench.flops(tiny["T"], tiny["d"], tiny["f"], tiny["E"], tiny["k"], 0, False)
    assert got == 6 * 512 * 128 * 256 + 2 * 256 * 128 * 4 and abs(got - 1.007e8) / 1.007e8 < 5e-3


def test_roofline_traffic_is_read_from_the_committed_profile():
    sys.path.insert(0, ROOT)
    import bench
    t = bench.measured_traffic_bytes()
    stages = t["mixtral_fwd_bwd_lora"]
    assert set(stages) == {"fwd.gemm_w1w3_swiglu", "fwd.gemm_w2", "bwd.gemm_dx_w1w3", "bwd.gemm_dh_swiglu_bwd"}
    assert all(1e9 < v < 1e10 for v in stages.values())
    # the figures are the profile's own: each appears in its "scaled traffic per launch" table
    text = open(bench.TRAFFIC_PROFILE).read()
    for v in stages.values():
        assert f"= {v / 1e9:.2f} GB" in text
