#!/usr/bin/env python3
"""Benchmark of the GRPO hot path on one MI355X.

One "step" = one fused logprob + loss forward and backward (loss and d_hidden)
over one packed batch of synthetic input at the Qwen2.5-7B shape (hidden 3584,
vocab 152064, 16384 positions = 32 trajectories of 512 tokens in 8 groups of 4,
40 % assistant mask).  Inputs are resident in HBM before the timed region.

Prints ONE JSON line.  `roofline` describes the dominant kernel (the lm_head
projection with fused log-sum-exp): algorithmic flops per launch divided by its
average launch duration measured with HIP events on the launch stream during the
timed steps.  `cpu_baseline` is the CPU oracle timed on the host cores on a
bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA peak
# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc runs
# (FETCH_SIZE + WRITE_SIZE scaled by a copy kernel of known size); None until
# measured for the workload.  Source: profiles/lmhead_fwd_c3_pmc.txt
TRAFFIC_BYTES = {"c3": 1.05e10, "c1": None}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3", choices=["c1", "c3", "c4"])
    ap.add_argument("--chunk-tokens", type=int, default=0, help="positions per logits scratch chunk")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-tokens", type=int, default=2048)
    ap.add_argument("--copy-calibration-mib", type=int, default=0,
                    help="also run one plain device copy of this size (scales FETCH_SIZE/WRITE_SIZE "
                         "counters when profiling with rocprofv3 --pmc)")
    return ap.parse_args()


def cpu_baseline(case, sample_tokens: int):
    """CPU oracle (fp32, autograd w.r.t. hidden) on the first `sample_tokens`
    positions of the same case; tokens/s on the host cores."""
    import torch

    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import grpo_oracle

    n = min(sample_tokens, case.hidden.shape[1])
    sl = lambda t: t[:, :n].contiguous()
    args = (sl(case.hidden), case.lm_head, sl(case.tokens), sl(case.logprobs), sl(case.advantages),
            sl(case.assistant_mask), sl(case.weights))
    chunk = 256 if n % 256 == 0 else n
    t0 = time.perf_counter()
    grpo_oracle.loss_and_grad(*args, chunk_size=chunk)
    dt = time.perf_counter() - t0
    return {
        "value": n / dt,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first {n} of {case.hidden.shape[1]} positions, full vocab, fp32 torch-CPU oracle "
                  f"fwd+bwd, 1 run of {dt:.1f} s",
    }


def main():
    args = parse()
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        print("bench.py: this build runs on ONE GPU only (the path shards over tokens with no "
              "exchange; see DESIGN.md). Re-run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    from art_amd import ops, synthetic

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    case = {"c1": synthetic.config1, "c3": synthetic.config3, "c4": synthetic.config4}[args.workload]()
    T, H = case.hidden.shape[1], case.hidden.shape[2]
    V = case.lm_head.shape[0]

    hidden = case.hidden.view(T, H).to(dev)
    lm_head = case.lm_head.to(dev)
    tokens = case.tokens.view(T).to(dev)
    # old logprobs = current logprobs + noise: the current ones come from the kernel itself
    new, _ = ops.logprob_fwd(hidden, lm_head, tokens, True, T)
    case.finish(new.cpu())
    old = case.logprobs.view(T).to(dev)
    adv = case.advantages.view(T).to(dev)
    mask = case.assistant_mask.view(T).to(dev)
    weights = case.weights.view(T).to(dev)
    lm_head_t = ops.transpose(lm_head)

    chunk = args.chunk_tokens or ops.DEFAULT_CHUNK_TOKENS
    ws = torch.empty(ops.grpo_fused_workspace_bytes(T, V, H, chunk), dtype=torch.uint8, device=dev)
    out = (torch.empty(4, dtype=torch.float32, device=dev),
           torch.empty(T, dtype=torch.float32, device=dev),
           torch.empty((T, H), dtype=torch.bfloat16, device=dev))

    def step():
        ops.grpo_fused(hidden, lm_head, lm_head_t, tokens, old, adv, mask, weights, None, T, 0.8,
                       1.2, 0.0, chunk, workspace=ws, out=out)

    if args.copy_calibration_mib:
        n = args.copy_calibration_mib << 20
        src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads n bytes, writes n bytes
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ops.profile_enable(True)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    fwd_ms, fwd_n = ops.profile_collect(ops.PROF_LMHEAD_FWD)
    bwd_ms, bwd_n = ops.profile_collect(ops.PROF_DHIDDEN_GEMM)
    sm_ms, sm_n = ops.profile_collect(ops.PROF_SOFTMAX_GRAD)
    ops.profile_enable(False)

    ms_per_step = dt / args.steps * 1e3
    tokens_per_s = T / (dt / args.steps)
    # rows whose loss coefficient is zero (non-assistant positions) have a zero d_hidden row
    # and are skipped by the backward: the algorithmic work counts them in the forward only
    t_active = int(out[0][3].item())
    alg_flops_step = 2.0 * T * V * H + 2.0 * t_active * V * H
    # dominant kernel: one launch covers `chunk` positions against the whole vocabulary
    fwd_launch_ms = fwd_ms / max(fwd_n, 1)
    launches_per_step = fwd_n / args.steps
    flops_per_launch = 2.0 * T * V * H / launches_per_step
    achieved = flops_per_launch / (fwd_launch_ms * 1e-3) / 1e12
    bwd_launch_ms = bwd_ms / max(bwd_n, 1)
    bwd_achieved = (2.0 * t_active * V * H / (bwd_n / args.steps)) / (bwd_launch_ms * 1e-3) / 1e12

    result = {
        "metric": "GRPO loss fwd+bwd tokens/sec @Qwen2.5-7B shape" if args.workload == "c3"
        else f"GRPO loss fwd+bwd tokens/sec ({case.name})",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": case.name, "tokens": T, "hidden": H, "vocab": V,
                   "chunk_tokens": chunk, "mask_fraction": float(case.assistant_mask.float().mean()),
                   "t_active": t_active},
        "algorithmic_flops_per_step": alg_flops_step,
        "tflops_algorithmic": alg_flops_step / (dt / args.steps) / 1e12,
        "frac_of_bf16_peak": alg_flops_step / (dt / args.steps) / 1e12 / PEAK_BF16_TFLOPS,
        "roofline": {
            "kernel": "lmhead_fwd_kernel<stash>",
            "bound": "mfma",
            "achieved": achieved,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / PEAK_BF16_TFLOPS,
            "traffic": TRAFFIC_BYTES.get(args.workload),
            "launch_ms": fwd_launch_ms,
            "launches_per_step": launches_per_step,
        },
        "kernels": {
            "dhidden_gemm_kernel": {"launch_ms": bwd_launch_ms, "tflops": bwd_achieved,
                                    "frac": bwd_achieved / PEAK_BF16_TFLOPS},
            "softmax_grad_kernel": {"launch_ms": sm_ms / max(sm_n, 1)},
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(case, args.cpu_sample_tokens)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
