#!/usr/bin/env python3
"""Benchmark of the MoE expert-MLP hot path on one MI355X.

A step = one pass of the hot path over one batch of synthetic input that is already resident in HBM:
router -> stable sort into expert-grouped order -> fused w1/w3 GEMM + SwiGLU -> w2 GEMM -> weighted combine,
then the backward pass (dX and the LoRA dA/dB of all three projections).  Default workload: the Mixtral-8x7B
shaped layer, T=4096, bf16, top-2, LoRA r=16 alpha=32, fwd+bwd.

Prints ONE JSON line: metric/value (TFLOP/s of algorithmic FLOPs), ms_per_step, tokens/s, a `roofline` object
for the dominant kernel (grouped GEMM, measured with events inside the timed region) and a `cpu_baseline`
object (the fp32 CPU oracle timed on a bounded sample on this box's host cores).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
PEAK_HBM_GBS = 8000.0
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "grouped_gemm_hbm_traffic_pmc.txt")


def measured_traffic_bytes(path=TRAFFIC_PROFILE):
    """HBM-side bytes per launch of the grouped GEMM stages, read from the committed rocprofv3 --pmc FETCH_SIZE /
    WRITE_SIZE summary (counters cannot be read from inside this process): its lines
    `traffic_bytes <workload> <stage> <bytes>` carry the calibrated figures."""
    out = {}
    try:
        with open(path) as fh:
            for line in fh:
                parts = line.split()
                if len(parts) == 4 and parts[0] == "traffic_bytes":
                    out.setdefault(parts[1], {})[parts[2]] = float(parts[3])
    except OSError:
        pass
    return out


WORKLOADS = {
    # name: (T, d, f, E, k, rank, backward, skew, description)
    "mixtral_fwd_bwd_lora": dict(T=4096, d=4096, f=14336, E=8, k=2, r=16, bwd=True, skew=False,
                                 desc="Mixtral-8x7B MoE layer fwd+bwd, T=4096, bf16, top-2, LoRA r=16 alpha=32 (BASELINE configs[2])"),
    "mixtral_fwd_bwd_lora_r32": dict(T=4096, d=4096, f=14336, E=8, k=2, r=32, bwd=True, skew=False,
                                     desc="Mixtral-8x7B MoE layer fwd+bwd, T=4096, bf16, top-2, LoRA r=32 alpha=32 (adapters as two 16-wide rank chunks)"),
    "mixtral_fwd_bwd_lora_r64": dict(T=4096, d=4096, f=14336, E=8, k=2, r=64, bwd=True, skew=False,
                                     desc="Mixtral-8x7B MoE layer fwd+bwd, T=4096, bf16, top-2, LoRA r=64 alpha=32 (adapters as four 16-wide rank chunks)"),
    "mixtral_fwd_bwd_lora_fp16": dict(T=4096, d=4096, f=14336, E=8, k=2, r=16, bwd=True, skew=False, dtype="fp16",
                                      desc="Mixtral-8x7B MoE layer fwd+bwd, T=4096, fp16 (the reference's fp16 switch), top-2, LoRA r=16 alpha=32"),
    "mixtral_fwd": dict(T=4096, d=4096, f=14336, E=8, k=2, r=0, bwd=False, skew=False,
                        desc="Mixtral-8x7B MoE layer forward, T=4096, bf16, top-2 (BASELINE configs[1])"),
    "mixtral_fwd_bwd_full": dict(T=4096, d=4096, f=14336, E=8, k=2, r=0, bwd=True, skew=False, train_base=True,
                                 desc="Mixtral-8x7B MoE layer fwd+bwd, T=4096, bf16, top-2, full fine-tuning (expert weights take gradients)"),
    "ep_share_fwd_bwd_lora": dict(T=8192, d=4096, f=14336, E=2, k=1, r=16, bwd=True, skew=False, ep_share=True,
                                  desc="one expert-parallel rank's share: 2 resident experts, 8192 pre-dispatched rows (0.55 / 0.45), "
                                       "bf16, LoRA r=16, fwd+bwd, no router / combine (BASELINE configs[4])"),
    "tiny_fp32_fwd": dict(T=256, d=128, f=256, E=4, k=2, r=0, bwd=False, skew=False, dtype="fp32",
                          desc="tiny MoE MLP, T=256, d=128, f=256, E=4, top-2, fp32, forward (BASELINE configs[0], the CPU-runnable case)"),
    "skewed_fwd_bwd_lora": dict(T=16384, d=4096, f=14336, E=8, k=2, r=16, bwd=True, skew=True,
                                desc="Zipf(1.2)-skewed routing, T=16384, fwd+bwd, LoRA r=16 (BASELINE configs[3])"),
}


def flops(T, d, f, E, k, r, bwd, train_base=False, ep_share=False):
    """Algorithmic FLOP of one step.  ep_share: rows arrive dispatched (T rows, one assignment each), the router runs
    on the other side of the exchange and is not counted."""
    R = T * k
    base = 6 * R * d * f
    router = 0 if ep_share else 2 * T * d * E
    lora_fwd = 6 * R * r * (d + f)
    total = base + router + lora_fwd
    if bwd:
        total += base + lora_fwd + 12 * R * r * (d + f)
        if train_base:
            total += base          # dW1, dW3, dW2: one more 2*R*d*f per projection
    return total


def make_inputs(cfg, dev, seed=0):
    import torch
    g = torch.Generator(device=dev).manual_seed(seed)
    T, d, f, E, r = cfg["T"], cfg["d"], cfg["f"], cfg["E"], cfg["r"]
    bf = {"fp32": torch.float32, "fp16": torch.float16}.get(cfg.get("dtype"), torch.bfloat16)

    def rn(*shape, std=1.0):
        return (torch.randn(*shape, generator=g, device=dev, dtype=torch.float32) * std).to(bf)

    x = rn(T, d)
    wg = rn(E, d, std=0.02)
    if cfg["skew"]:
        # per-expert logit offset ~ log Zipf(s=1.2) pmf, folded into the router weight along one input direction
        pmf = torch.tensor([1.0 / (i + 1) ** 1.2 for i in range(E)])
        pmf = pmf / pmf.sum()
        bias = (2.2 * torch.log(pmf)).to(dev)
        x[:, 0] = 1.0
        wg[:, 0] = bias.to(bf)
    w1, w2, w3 = rn(E, f, d, std=0.02), rn(E, f, d, std=0.02), rn(E, f, d, std=0.02)
    lora = None
    if r > 0:
        lora = dict(a1=rn(E, d, r, std=0.02), b1=rn(E, r, f, std=0.02), a3=rn(E, d, r, std=0.02), b3=rn(E, r, f, std=0.02),
                    a2=rn(E, f, r, std=0.02), b2=rn(E, r, d, std=0.02))
    dout = rn(T, d)
    return x, wg, w1, w2, w3, lora, dout


def ep_share_routing(cfg, dev, seed=1):
    """The local expert of each pre-dispatched row (a multinomial draw, 0.55 / 0.45 over the two resident experts; rows
    arrive in exchange order, i.e. the grouped order is a permutation of them) and what the rank's local re-sort hands
    to the kernels: sorted positions and inclusive expert offsets."""
    import torch
    from moe_distributed_training_amd.megablocks_utils.router import sort_assignments
    g = torch.Generator().manual_seed(seed)
    p = torch.tensor([0.55, 0.45] if cfg["E"] == 2 else [1.0 / cfg["E"]] * cfg["E"])
    e_of_row = torch.multinomial(p, cfg["T"], replacement=True, generator=g).to(dev)
    _sei, ssi, _counts, offsets, _inv = sort_assignments(e_of_row.int(), cfg["E"])
    return e_of_row, ssi, offsets


def read_profile(lib):
    n = lib.moe_profile_count()
    buf = ctypes.create_string_buffer(64)
    ms = ctypes.c_float()
    out = {}
    for i in range(n):
        lib.moe_profile_get(i, ctypes.cast(buf, ctypes.c_void_p), 64, ctypes.cast(ctypes.pointer(ms), ctypes.c_void_p))
        out.setdefault(buf.value.decode(), []).append(ms.value)
    return out


def cpu_baseline(cfg, x, wg, w1, w2, w3, lora, dout, budget_tokens, e_of_row=None):
    """fp32 CPU oracle (per-expert loop + index_add, autograd backward) on the first `budget_tokens` tokens: one
    untimed warm-up pass, then the median of 3 timed passes (5 for the tiny configuration)."""
    import statistics
    import torch
    from oracle import moe_oracle as oracle
    cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    cores = min(cores, os.cpu_count() or cores)
    torch.set_num_threads(cores)
    Ts = min(cfg["T"], budget_tokens)
    xs = x[:Ts].float().cpu()
    W = [t.detach().float().cpu() for t in (wg, w1, w2, w3)]
    if cfg.get("train_base"):
        for t in W[1:]:
            t.requires_grad_(True)
    lo = None
    if lora is not None:
        c = {k_: v.float().cpu().requires_grad_(cfg["bwd"]) for k_, v in lora.items()}
        lo = {"w1": (c["a1"], c["b1"]), "w3": (c["a3"], c["b3"]), "w2": (c["a2"], c["b2"])}
    ds = dout[:Ts].float().cpu()
    xs.requires_grad_(cfg["bwd"])
    routing = None
    if e_of_row is not None:   # pre-dispatched rows: the expert of each row is given, weight 1
        routing = (torch.ones(Ts, 1), e_of_row[:Ts].cpu().long()[:, None])

    def one_pass():
        t0 = time.perf_counter()
        with torch.set_grad_enabled(cfg["bwd"]):
            out, _ = oracle.moe_block(xs, None if routing else W[0], W[1], W[2], W[3], cfg["k"], lo, 32.0, routing=routing)
            if cfg["bwd"]:
                out.backward(ds)
        return time.perf_counter() - t0

    one_pass()
    passes = 5 if cfg["T"] <= 1024 else 3
    times = [one_pass() for _ in range(passes)]
    dt = statistics.median(times)
    fl = flops(Ts, cfg["d"], cfg["f"], cfg["E"], cfg["k"], cfg["r"], cfg["bwd"], bool(cfg.get("train_base")), bool(cfg.get("ep_share")))
    cpu_model = "unknown CPU"
    try:
        with open("/proc/cpuinfo") as fh:
            cpu_model = next(line.split(":", 1)[1].strip() for line in fh if line.startswith("model name"))
    except (OSError, StopIteration):
        pass
    return dict(value=fl / dt / 1e12, unit="TFLOP/s", cores=cores, kind="port",
                sample=f"first {Ts} of {cfg['T']} {'rows' if cfg.get('ep_share') else 'tokens'}, fp32 torch oracle, 1 warm-up pass + median of "
                       f"{passes} passes ({dt * 1e3:.1f} ms; all: {', '.join(f'{t * 1e3:.1f}' for t in times)} ms)",
                tokens_per_s=Ts / dt, cpu=cpu_model)


def library_gemm(torch, dev, R, d, f, launches=50):
    """The vendor library's dense bf16 GEMM of one projection's size, (R, d) x (d, f), as a practical ceiling beside the
    2.5 PFLOP/s datasheet figure: what a hand-tuned kernel without groups, gathers, adapters or epilogues reaches on
    this GPU under the same kind of short measurement.  Runs after the timed region."""
    a = torch.randn(R, d, device=dev).bfloat16()
    b = (torch.randn(f, d, device=dev) * 0.02).bfloat16()
    for _ in range(10):
        torch.matmul(a, b.t())
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        torch.matmul(a, b.t())
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / launches
    return {"kernel": f"torch.matmul (hipBLASLt) {R}x{d}x{f} bf16", "launch_ms": round(ms, 4),
            "value": round(2 * R * d * f / (ms * 1e-3) / 1e12, 1), "unit": "TFLOP/s", "launches": launches}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="mixtral_fwd_bwd_lora", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-tokens", type=int, default=4096)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    import moe_distributed_training_amd as moe
    from moe_distributed_training_amd._lib import lib
    from moe_distributed_training_amd.megablocks_utils.moe_mlp import LoraViews

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    cfg = WORKLOADS[args.workload]
    x, wg, w1, w2, w3, lora, dout = make_inputs(cfg, dev)
    views = None
    if lora is not None:
        for v in lora.values():
            v.requires_grad_(cfg["bwd"])
        views = LoraViews(lora["a1"], lora["b1"], lora["a3"], lora["b3"], lora["a2"], lora["b2"])
    x.requires_grad_(cfg["bwd"])
    train_base = bool(cfg.get("train_base"))
    if train_base:
        for w in (w1, w2, w3):
            w.requires_grad_(True)
    ep_share = bool(cfg.get("ep_share"))
    e_of_row = ep_ssi = ep_offsets = None
    if ep_share:
        e_of_row, ep_ssi, ep_offsets = ep_share_routing(cfg, dev)

    def clear_grads():
        x.grad = None
        if lora is not None:
            for v in lora.values():
                v.grad = None
        if train_base:
            w1.grad = w2.grad = w3.grad = None

    def step():
        with torch.set_grad_enabled(cfg["bwd"]):
            if ep_share:
                # the rows are here already, one assignment each: expert MLP on the local experts, output back in arrival order
                out = moe.fused_expert_mlp(x, w1, w2, w3, 1, ep_ssi, ep_offsets, views, 32.0)
            else:
                out, ew, ei = moe.moe_layer_forward(x, wg, w1, w2, w3, cfg["k"], views, 32.0)
            if cfg["bwd"]:
                clear_grads()
                out.backward(dout)
        return out

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # Timed region: only the grouped-GEMM launches (the roofline's kernels) are bracketed by events -- a bracket costs a few
    # microseconds of device time, and one around each of the ~26 stages of a step adds ~0.12 ms (2.5 %) to it.
    lib.moe_profile_select(b"gemm,group_bwd_w")
    lib.moe_profile_enable(1)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    prof = read_profile(lib)
    lib.moe_profile_enable(0)
    # Every stage, for the per-stage table and the HBM-bound stages' rates: a separate pass after the timed region
    stage_steps = max(1, min(args.steps, 20))
    lib.moe_profile_select(None)
    lib.moe_profile_enable(1)
    for _ in range(stage_steps):
        step()
    torch.cuda.synchronize()
    prof_all = read_profile(lib)
    lib.moe_profile_enable(0)

    fl = flops(cfg["T"], cfg["d"], cfg["f"], cfg["E"], cfg["k"], cfg["r"], cfg["bwd"], train_base, ep_share)
    tflops = fl / dt / 1e12
    stages = {k_: sum(v) / len(v) for k_, v in prof_all.items()}       # all stages, from the separate pass
    stages.update({k_: sum(v) / len(v) for k_, v in prof.items()})     # the GEMM launches, from the timed region
    # dominant kernel: the grouped GEMM launches; FLOPs per launch are the algorithmic ones of that projection pair
    R = cfg["T"] * cfg["k"]
    gemm_flops = {"fwd.gemm_w1w3_swiglu": 4 * R * cfg["d"] * cfg["f"], "fwd.gemm_w2": 2 * R * cfg["d"] * cfg["f"],
                  "bwd.gemm_dh_swiglu_bwd": 2 * R * cfg["d"] * cfg["f"], "bwd.gemm_dx_w1w3": 4 * R * cfg["d"] * cfg["f"],
                  "bwd.group_bwd_w": 2 * R * cfg["d"] * cfg["f"]}
    gemm_stages = {k_: v for k_, v in stages.items() if k_ in gemm_flops}
    fp32 = cfg.get("dtype") == "fp32"
    fp16 = cfg.get("dtype") == "fp16"   # same dense MFMA peak as bf16 (2.5 PFLOP/s)
    if gemm_stages:
        dom = max(gemm_stages, key=gemm_stages.get)
        ach = gemm_flops[dom] / (gemm_stages[dom] * 1e-3) / 1e12
        per_step = {k_: len(prof[k_]) / args.steps for k_ in gemm_stages}       # launches per step (3 for the weight gradients)
        gemm_ms = sum(gemm_stages[k_] * per_step[k_] for k_ in gemm_stages)
        gemm_all = sum(gemm_flops[k_] * per_step[k_] for k_ in gemm_stages) / (gemm_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "kernel": f"{'grouped_xty_mfma_kernel' if dom == 'bwd.group_bwd_w' else 'grouped_gemm_mfma_kernel'} [{dom}]",
                    "achieved": round(ach, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(ach / PEAK_BF16_TFLOPS, 4),
                    "traffic": measured_traffic_bytes().get(args.workload, {}).get(dom), "launch_ms": round(gemm_stages[dom], 4),
                    "all_gemm_launches_tflops": round(gemm_all, 2), "all_gemm_ms": round(gemm_ms, 4)}
    else:
        # fp32 runs on the generic (non matrix-core) kernels through the per-projection calls, which carry no stage timer: the
        # whole step stands for the kernel, against the fp32 vector peak
        peak = 157.3
        roofline = {"bound": "valu", "kernel": "generic_gemm_kernel (whole step: a few microseconds of fp32 vector arithmetic, launch bound)",
                    "achieved": round(tflops, 4), "peak": peak, "unit": "TFLOP/s", "frac": round(tflops / peak, 6), "traffic": None}
    what = ("fwd+bwd" if cfg["bwd"] else "fwd")
    metric = "MoE-layer fwd+bwd TFLOP/s & % bf16 MFMA peak, Mixtral shape T=4096, 1 GPU" if args.workload == "mixtral_fwd_bwd_lora" \
        else f"MoE-layer {what} TFLOP/s & % {'fp32' if fp32 else 'fp16 MFMA' if fp16 else 'bf16 MFMA'} peak, workload {args.workload}, 1 GPU"
    result = {
        "metric": metric,
        "value": round(tflops, 4 if fp32 else 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp32" if fp32 else "fp16" if fp16 else "bf16", "data": "synthetic",
        "config": {"workload": cfg["desc"], "tokens": cfg["T"], "d_model": cfg["d"], "d_ff": cfg["f"],
                   "experts": cfg["E"], "top_k": cfg["k"], "lora_rank": cfg["r"]},
        "tokens_per_s": round(cfg["T"] / dt, 1),
        "frac_of_bf16_peak": round(tflops / PEAK_BF16_TFLOPS, 6 if fp32 else 4),
        "algorithmic_flop_per_step": fl,
        "roofline": roofline,
        "stage_ms": {k_: round(v, 4) for k_, v in sorted(stages.items())},
        "stage_ms_source": f"grouped-GEMM stages: events inside the timed region ({args.steps} steps); all other stages: a separate pass of "
                           f"{stage_steps} steps after it with every stage bracketed (those brackets would add ~0.12 ms to a timed step)",
    }
    # HBM-bound stages: algorithmic bytes (read activations once, write results once) over the measured launch times
    T_, d_, E_, k_top = cfg["T"], cfg["d"], cfg["E"], cfg["k"]
    hbm = {}
    if "route.router_forward" in stages and "route.sort" in stages:
        hbm["routing (router + sort)"] = (stages["route.router_forward"] + stages["route.sort"],
                                         T_ * d_ * 2 + T_ * E_ * 4 + 2 * R * 8)
    if "rows.combine" in stages:
        hbm["combine (per launch)"] = (stages["rows.combine"], R * d_ * 2 + T_ * k_top * 4 + T_ * d_ * 2)
    if "rows.combine_dgates" in stages:
        hbm["combine d_gates"] = (stages["rows.combine_dgates"], R * d_ * 2 + T_ * d_ * 2 + T_ * k_top * 4)
    result["hbm_stages"] = {n: {"ms": round(ms, 4), "bytes": b, "GB_per_s": round(b / (ms * 1e-3) / 1e9, 1),
                                "frac_of_8TBps": round(b / (ms * 1e-3) / 8e12, 4)} for n, (ms, b) in hbm.items()}
    if not fp32:
        result["library_gemm"] = library_gemm(torch, dev, R, cfg["d"], cfg["f"])
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg, x.detach(), wg, w1, w2, w3,
                                              None if lora is None else {k_: v.detach() for k_, v in lora.items()},
                                              dout, args.cpu_tokens, e_of_row)
        result["cpu_baseline"]["value"] = round(result["cpu_baseline"]["value"], 4)
        result["cpu_baseline"]["tokens_per_s"] = round(result["cpu_baseline"]["tokens_per_s"], 1)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
