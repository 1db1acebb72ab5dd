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
PEAK_HBM_GBPS = 8000.0     # MI355X HBM3E peak
# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc runs
# (FETCH_SIZE + WRITE_SIZE scaled by a copy kernel of known size); None until
# measured for the workload.  Source: profiles/lmhead_fwd_c3_pmc.md
TRAFFIC_BYTES = {"c3": 1.68e10, "c1": None}  # 7.87e6 x 2 KiB fetched + 0.70e6 KiB written per forward launch
# moe_gemm_kernel, mean bytes per launch over the 4 launches of the step with gate|up fused (FETCH_SIZE x 2 KiB +
# WRITE_SIZE x 1 KiB, the factors a 1 GiB copy gives): 1166 MB read + 211 MB written
MOE_TRAFFIC_BYTES = 1.38e9
# lora_multi_gemm_kernel, mean of the two gate|up launches (8192 x 2048 -> 11008 + 11008): y 1.41 GB read + 0.37 GB
# written, dx 1.08 GB read + 0.03 GB written
LORA_TRAFFIC_BYTES = 1.45e9
LORA_TRAFFIC_SOURCE = ("profiles/lora_c2_kernel_trace.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of "
                       "this command, scaled by a 1 GiB copy; not measured in this run)")
MOE_TRAFFIC_SOURCE = ("profiles/moe_c5_kernel_trace.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of "
                      "this command, scaled by a 1 GiB copy; not measured in this run)")
TRAFFIC_SOURCE = {"c3": "profiles/lmhead_fwd_c3_pmc.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier "
                        "run of this command, scaled by a 1 GiB copy; not measured in this run)"}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3", choices=["c1", "c3", "c4", "lora", "moe", "attn", "pack", "optim", "nf4", "ceiling"],
                    help="c3 (default, the headline): fused GRPO step at the Qwen2.5-7B shape; c1/c4: the "
                         "0.5B / 14B shapes; lora: LoRA linear fwd+bwd at the Qwen2.5-3B shapes; moe: "
                         "expert-LoRA grouped GEMMs at the Qwen3-30B-A3B-style share")
    ap.add_argument("--chunk-tokens", type=int, default=0, help="positions per logits scratch chunk")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="skip the secondary figures (c3/c1/c4: the skip_inactive variant), e.g. when profiling")
    ap.add_argument("--no-sub-records", action="store_true",
                    help="c3 only: leave out the lora / moe / ceiling records of the default line")
    ap.add_argument("--cpu-sample-tokens", type=int, default=4096,
                    help="positions of the CPU baseline sample (first half from the start, second from the end)")
    ap.add_argument("--copy-calibration-mib", type=int, default=0,
                    help="also run one plain device copy of this size (scales FETCH_SIZE/WRITE_SIZE "
                         "counters when profiling with rocprofv3 --pmc)")
    return ap.parse_args()


def cpu_baseline(case, sample_tokens: int, gpu_logprob=None, gpu_d_hidden=None, mask_count=None):
    """CPU oracle (autograd w.r.t. hidden) on a bounded sample of the same case: the first and
    the last `sample_tokens / 2` positions, full vocabulary; tokens/s on the host cores.
    fp32 (the parity reference): 1 warm-up + 3 runs, median.  bf16 (the dtype the reference
    itself runs in): the same, cut short if the host is slow at it.  With the GPU results of
    the whole batch given, the fp32 run doubles as the parity check of this run."""
    import torch

    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import grpo_oracle

    T = case.hidden.shape[1]
    half = max(min(sample_tokens // 2, T // 2), 1)
    spans = [(0, half), (T - half, T)]
    chunk = 256 if half % 256 == 0 else half

    def run(dtype):
        refs = []
        t0 = time.perf_counter()
        for a, b in spans:
            sl = lambda t: t[:, a:b].contiguous()
            refs.append(grpo_oracle.loss_and_grad(sl(case.hidden), case.lm_head, sl(case.tokens), sl(case.logprobs),
                                                  sl(case.advantages), sl(case.assistant_mask), sl(case.weights),
                                                  chunk_size=chunk, dtype=dtype))
        return time.perf_counter() - t0, refs

    def series(dtype, budget_s):
        """1 warm-up + up to 3 timed runs (fewer if `budget_s` runs out); (median seconds, runs, refs)."""
        t_start = time.perf_counter()
        warm, refs = run(dtype)
        times = []
        while len(times) < 3 and time.perf_counter() - t_start + warm < budget_s:
            times.append(run(dtype)[0])
        if not times:
            return warm, 0, refs
        return sorted(times)[len(times) // 2], len(times), refs

    n = 2 * half
    dt32, runs32, refs = series(torch.float32, 60.0)
    dt16, runs16, _ = series(torch.bfloat16, 30.0)
    out = {
        "value": n / dt32,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first and last {half} of {T} positions, full vocab, torch-CPU oracle fwd+bwd in fp32: "
                  f"1 warm-up + {runs32} runs, median {dt32:.1f} s",
        "bf16": {"value": n / dt16, "unit": "tokens/s",
                 "sample": f"same sample evaluated in bf16 (the reference's dtype): 1 warm-up + {runs16} runs, "
                           f"median {dt16:.1f} s" if runs16 else f"same sample in bf16: one run of {dt16:.1f} s"},
    }
    parity = None
    if gpu_logprob is not None and half > 1:
        # Every position's logprob and d_hidden row depend on the rest of the batch only through
        # the loss denominator (mask count + 1e-6).  The last position of the first span is left
        # out (its target lies outside the span); the last position of the batch has the pad target.
        lp_err, num, den, npos = 0.0, 0.0, 0.0, 0
        for (a, b), ref in zip(spans, refs):
            e = b - 1 if b < T else b
            m_span = float(grpo_oracle.shift_tensor(case.assistant_mask[:, a:b], False).sum())
            scale = (m_span + 1e-6) / (float(mask_count) + 1e-6)
            lp_err = max(lp_err, (gpu_logprob[a:e].float().cpu() - ref["logprobs"][0, : e - a]).abs().max().item())
            want = ref["d_hidden"][0, : e - a].double() * scale
            got = gpu_d_hidden[a:e].double().cpu()
            num += float((got - want).pow(2).sum())
            den += float(want.pow(2).sum())
            npos += e - a
        parity = {"positions": npos, "spans": [list(sp) for sp in spans], "logprob_max_abs_err": lp_err,
                  "d_hidden_rel_l2": (num / den) ** 0.5,
                  "tolerances": {"logprob_max_abs_err": 2e-3, "d_hidden_rel_l2": 1e-2}}
    return out, parity


def input_digests(case):
    """SHA-256 (first 16 hex digits) of the integer and boolean inputs of a case."""
    import hashlib

    import numpy as np

    arrays = {"tokens": case.tokens.numpy(), "assistant_mask": case.assistant_mask.numpy().astype(np.uint8),
              "traj_id": case.traj_id.numpy(), "group_of_traj": np.asarray(case.group_of_traj)}
    return {k: hashlib.sha256(np.ascontiguousarray(v).tobytes()).hexdigest()[:16] for k, v in arrays.items()}


def timed(fn, steps, warmup):
    """Seconds per call: `warmup` untimed calls, then `steps` calls between device syncs."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def base_result(args, metric, unit, value, ms_per_step, workload):
    return {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic", "config": {"workload": workload},
    }


def bench_lora(args):
    """LoRA linear fwd+bwd over the six projections of one Qwen2.5-3B layer that have
    in = 2048 (q, o: out 2048; k, v: out 256; gate, up: out 11008), T = 8192, r = 8, alpha = 16.
    One step = forward + backward of all six.  `value` = algorithmic TFLOP/s of the step as a user
    runs it: the modules of art_amd.lora (FusedLoRALinear for q|k|v and for gate|up, LoRALinear for o)
    called through torch autograd with one upstream gradient tensor per projection; the projections
    that read the same activations go through the library's multi-projection entry points (separate
    weights, adapters, outputs and gradients; nothing concatenated).  `raw_multi` = the same entry
    points called directly; `raw_concatenated` = the single-projection entry points on
    pre-concatenated weights / stacked adapters / concatenated upstream gradients (built outside the
    timed region); `separate` = six single-projection calls."""
    import math

    import torch

    from art_amd import ops
    from art_amd.lora import FusedLoRALinear, LoRALinear

    dev = torch.device("cuda:0")
    T, n_in, r, scale = 8192, 2048, 8, 2.0
    g = torch.Generator().manual_seed(1002)
    x_cpu = torch.randn(T, n_in, generator=g).to(torch.bfloat16)
    x = x_cpu.to(dev)
    names = ("q", "o", "k", "v", "gate", "up")
    cpu, shapes = {}, {}
    for name, n_out in zip(names, (2048, 2048, 256, 256, 11008, 11008)):
        W = (0.02 * torch.randn(n_out, n_in, generator=g)).to(torch.bfloat16)
        A = ((torch.rand(r, n_in, generator=g) * 2 - 1) / math.sqrt(n_in)).to(torch.bfloat16)
        B = (0.01 * torch.randn(n_out, r, generator=g)).to(torch.bfloat16)
        up = torch.randn(T, n_out, generator=g).to(torch.bfloat16)
        cpu[name] = (W, A, B, up)
        Wd = W.to(dev)
        shapes[name] = (n_out, Wd, ops.transpose(Wd), A.to(dev), B.to(dev), up.to(dev))
    flops = lambda n_out: 4.0 * T * n_in * n_out + 6.0 * T * r * (n_in + n_out)
    total = sum(flops(sh[0]) for sh in shapes.values())

    def one(sh):
        _, W, Wt, A, B, up = sh
        y, xa = ops.lora_linear_fwd(x, W, A, B, scale)
        return (y,) + ops.lora_linear_bwd(up, x, Wt, A, B, xa, scale)

    def multi(group):
        parts = [shapes[n] for n in group]
        ys, xas = ops.lora_linear_multi_fwd(x, [p[1] for p in parts], [p[3] for p in parts],
                                            [p[4] for p in parts], scale)
        dx, dAs, dBs = ops.lora_linear_multi_bwd([p[5] for p in parts], x, [p[2] for p in parts],
                                                 [p[3] for p in parts], [p[4] for p in parts], xas, scale)
        return ys, dx, dAs, dBs

    def fuse(group):
        parts = [shapes[n] for n in group]
        W = torch.cat([p[1] for p in parts], 0).contiguous()
        A = torch.cat([p[3] for p in parts], 0).contiguous()
        B = torch.zeros(W.shape[0], A.shape[0], dtype=torch.bfloat16, device=dev)
        o0 = r0 = 0
        for p in parts:
            B[o0:o0 + p[0], r0:r0 + r] = p[4]
            o0, r0 = o0 + p[0], r0 + r
        up = torch.cat([p[5] for p in parts], 1).contiguous()
        return (W.shape[0], W, ops.transpose(W), A, B, up)

    # the modules a user holds: one LoRALinear per projection (adapters in bf16, as peft keeps them
    # under the reference's bf16 training), grouped by the activations they read
    mods = {}
    for name in names:
        n_out, Wd, _, Ad, Bd, _ = shapes[name]
        m = LoRALinear(n_in, n_out, r=r, lora_alpha=int(scale * r), device=dev, dtype=torch.bfloat16)
        with torch.no_grad():
            m.weight.copy_(Wd)
            m.lora_A.copy_(Ad)
            m.lora_B.copy_(Bd)
        mods[name] = m
    groups = (("q", "k", "v"), ("o",), ("gate", "up"))
    fused_mods = [FusedLoRALinear([mods[n] for n in grp]) for grp in groups]
    ups = [[shapes[n][5] for n in grp] for grp in groups]
    # in the model the three groups read three different activations (the attention input, the attention
    # output, the MLP input): one leaf per group, all with the same values so that one oracle serves
    xgs = [x.detach().clone().requires_grad_(True) for _ in groups]
    params = [p for m in mods.values() for p in (m.lora_A, m.lora_B)]
    for m in fused_mods:   # transposed copies of the frozen weights are made once per weight version
        for l in m.layers:
            ops.transposed_weight(l.weight)

    def step_module():
        for p_ in params + xgs:
            p_.grad = None
        for m, u, xg in zip(fused_mods, ups, xgs):
            torch.autograd.backward(m(xg), u)

    def step_raw_multi():
        for grp in groups:
            multi(grp)

    def step_separate():
        for sh in shapes.values():
            one(sh)

    dt = timed(step_module, args.steps, args.warmup)
    dt_raw = timed(step_raw_multi, args.steps, args.warmup)
    per_group = {}
    for grp in (("q", "k", "v"), ("gate", "up")):
        fl = sum(flops(shapes[m][0]) for m in grp)
        gdt = timed(lambda: multi(grp), args.steps, args.warmup)
        per_group["|".join(grp)] = {"us_fwd_bwd": gdt * 1e6, "tflops": fl / gdt / 1e12,
                                    "frac": fl / gdt / 1e12 / PEAK_BF16_TFLOPS}
    per_shape = {}
    for name in ("q", "k", "gate"):
        sh = shapes[name]
        sdt = timed(lambda: one(sh), args.steps, args.warmup)
        per_shape[f"out={sh[0]}"] = {"us_fwd_bwd": sdt * 1e6, "tflops": flops(sh[0]) / sdt / 1e12,
                                     "frac": flops(sh[0]) / sdt / 1e12 / PEAK_BF16_TFLOPS}
    dt_sep = timed(step_separate, args.steps, args.warmup)
    cat = {"qkv": fuse(("q", "k", "v")), "o": shapes["o"], "gate_up": fuse(("gate", "up"))}
    dt_cat = timed(lambda: [one(sh) for sh in cat.values()], args.steps, args.warmup)
    cat_bytes = sum(sh[1].numel() * 2 * 2 + sh[5].numel() * 2 for k_, sh in cat.items() if k_ != "o")
    del cat
    # dominant kernel, from a separate burst with the library's HIP-event brackets on
    ops.profile_enable(True)
    for _ in range(args.steps):
        multi(("gate", "up"))
    torch.cuda.synchronize()
    gemm_ms, gemm_n = ops.profile_collect(ops.PROF_LORA_GEMM)
    ops.profile_enable(False)
    res = base_result(args, "LoRA linear fwd+bwd TFLOP/s (Qwen2.5-3B shapes)", "TFLOP/s", total / dt / 1e12,
                      dt * 1e3, "C2-lora-qwen2.5-3b")
    res["config"].update({"tokens": T, "in": n_in, "rank": r, "projections": "q,o,k,v,gate,up",
                          "path": "art_amd.lora modules under torch autograd: FusedLoRALinear(q,k,v), "
                                  "LoRALinear(o), FusedLoRALinear(gate,up); one upstream gradient per projection"})
    res["frac_of_bf16_peak"] = total / dt / 1e12 / PEAK_BF16_TFLOPS
    res["raw_multi"] = {"value": total / dt_raw / 1e12, "unit": "TFLOP/s", "ms_per_step": dt_raw * 1e3,
                        "frac_of_bf16_peak": total / dt_raw / 1e12 / PEAK_BF16_TFLOPS, "groups": per_group,
                        "note": "artk_lora_linear_multi_fwd/_bwd called directly: q|k|v, o, gate|up"}
    res["raw_concatenated"] = {"value": total / dt_cat / 1e12, "unit": "TFLOP/s", "ms_per_step": dt_cat * 1e3,
                               "extra_resident_bytes": cat_bytes,
                               "note": "single-projection entry points on weights, transposed weights and upstream "
                                       "gradients concatenated outside the timed region (extra_resident_bytes of "
                                       "copies), adapters stacked with a block-diagonal B"}
    res["separate"] = {"value": total / dt_sep / 1e12, "unit": "TFLOP/s", "ms_per_step": dt_sep * 1e3,
                       "frac_of_bf16_peak": total / dt_sep / 1e12 / PEAK_BF16_TFLOPS, "shapes": per_shape,
                       "note": "six separate calls; per shape: one projection fwd+bwd"}
    launch_ms = gemm_ms / max(gemm_n, 1)
    ach = 2.0 * T * n_in * 22016 / (launch_ms * 1e-3) / 1e12
    res["roofline"] = {"kernel": "lora_multi_gemm_kernel (gate|up: mean of the y launch and the dx launch)",
                       "bound": "mfma", "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                       "frac": ach / PEAK_BF16_TFLOPS, "traffic": LORA_TRAFFIC_BYTES,
                       "traffic_source": LORA_TRAFFIC_SOURCE, "launch_ms": launch_ms,
                       "flop_per_launch": 2.0 * T * n_in * 22016,
                       "algorithmic_bytes": 2.0 * (T * n_in + T * 22016 + n_in * 22016)}
    if not args.no_secondary:
        # The LoRA linear the way peft evaluates it, in stock torch ops on the same GPU:
        # base(x) + scale * lora_B(lora_A(x)), autograd for dx, dA, dB (W frozen).
        import torch.nn.functional as F

        def torch_step():
            for _, W, _, A, B, up in shapes.values():
                xg_ = x.detach().requires_grad_(True)
                Ag, Bg = A.detach().requires_grad_(True), B.detach().requires_grad_(True)
                y = F.linear(xg_, W) + scale * F.linear(F.linear(xg_, Ag), Bg)
                y.backward(up)

        tdt = timed(torch_step, max(args.steps // 2, 3), 2)
        res["torch_gpu_same_algorithm"] = {"value": total / tdt / 1e12, "unit": "TFLOP/s", "ms_per_step": tdt * 1e3,
                                           "note": "F.linear(x, W) + s * F.linear(F.linear(x, A), B) with autograd "
                                                   "(dx, dA, dB), bf16, same six projections"}
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import lora_oracle

        # CPU oracle (fp32) of all six projections: the timing sample (1 warm-up + 3 runs, median) and the
        # parity reference of this run for the module step and for the raw multi-projection calls
        ref, times = {}, []
        for rep in range(4):
            t0 = time.perf_counter()
            for name in names:
                W, A, B, up = cpu[name]
                out = lora_oracle.lora_linear_grads(x_cpu, W, A, B, scale, up)
                if rep == 0:
                    ref[name] = out
            if rep:
                times.append(time.perf_counter() - t0)
        cdt = sorted(times)[1]
        t0 = time.perf_counter()
        for name in names:
            W, A, B, up = cpu[name]
            lora_oracle.lora_linear_grads(x_cpu, W, A, B, scale, up, dtype=torch.bfloat16)
        cdt16 = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": total / cdt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                               "kind": "port",
                               "sample": f"all six projections fwd+bwd, fp32 torch-CPU oracle, 1 warm-up + 3 runs, "
                                         f"median {cdt:.2f} s",
                               "bf16": {"value": total / cdt16 / 1e12, "unit": "TFLOP/s",
                                        "sample": f"same in bf16, one run of {cdt16:.2f} s"}}
        rel = lambda a, b: ((a.double().cpu() - b.double()).norm() / b.double().norm()).item()
        parity = {}
        for name in ("q", "k"):
            got = one(shapes[name])
            parity[name] = dict(zip(("y", "dx", "dA", "dB"), (rel(a, b) for a, b in zip(got, ref[name]))))
        for grp in (("q", "k", "v"), ("gate", "up")):
            ys, dx, dAs, dBs = multi(grp)
            rec = {"dx": rel(dx, sum(ref[n][1] for n in grp))}
            for i, name in enumerate(grp):
                rec[f"y_{name}"] = rel(ys[i], ref[name][0])
                rec[f"dA_{name}"] = rel(dAs[i], ref[name][2])
                rec[f"dB_{name}"] = rel(dBs[i], ref[name][3])
            parity["multi_" + "_".join(grp)] = rec
            del ys, dx, dAs, dBs
        # the module step itself: the gradient of each group's input is the sum over its projections
        step_module()
        rec = {}
        for grp, xg in zip(groups, xgs):
            rec["x_grad_" + "_".join(grp)] = rel(xg.grad, sum(ref[n][1] for n in grp))
        for name in names:
            rec[f"dA_{name}"] = rel(mods[name].lora_A.grad, ref[name][2])
            rec[f"dB_{name}"] = rel(mods[name].lora_B.grad, ref[name][3])
        parity["module_step"] = rec
        parity["tolerance_rel_l2"] = 1e-2
        res["parity_same_run"] = parity
    return res


def bench_moe(args):
    """Expert-LoRA grouped GEMMs: 8192 tokens, hidden 2048, 128 experts, top-8, gate/up [768,2048],
    down [2048,768], rank 8.  One step = routing + forward and backward of the three projections."""
    import torch

    from art_amd import ops

    dev = torch.device("cuda:0")
    T, H, I, E, k, r, scale = 8192, 2048, 768, 128, 8, 8, 2.0
    g = torch.Generator().manual_seed(1005)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    logits = torch.randn(T, E, generator=g).to(dev)
    mk = lambda o, i: ((0.02 * torch.randn(E, o, i, generator=g)).to(torch.bfloat16).to(dev),
                       ((torch.rand(E, r, i, generator=g) * 2 - 1) / i ** 0.5).to(torch.bfloat16).to(dev),
                       (0.01 * torch.randn(E, o, r, generator=g)).to(torch.bfloat16).to(dev))
    Wg, Ag, Bg = mk(I, H)
    Wu, Au, Bu = mk(I, H)
    Wd, Ad, Bd = mk(H, I)
    Wgt, Wut, Wdt = (ops.transpose_batched(w) for w in (Wg, Wu, Wd))
    n = T * k
    h = torch.randn(n, I, generator=g).to(torch.bfloat16).to(dev)
    g_i = torch.randn(n, I, generator=g).to(torch.bfloat16).to(dev)
    g_h = torch.randn(n, H, generator=g).to(torch.bfloat16).to(dev)

    def step():
        rt = ops.moe_route(logits, k)
        yg, xag = ops.moe_lora_grouped_fwd(x, rt.row_token, Wg, Ag, Bg, scale, rt)
        yu, xau = ops.moe_lora_grouped_fwd(x, rt.row_token, Wu, Au, Bu, scale, rt)
        yd, xad = ops.moe_lora_grouped_fwd(h, None, Wd, Ad, Bd, scale, rt)
        ops.moe_lora_grouped_bwd(g_h, h, None, Wdt, Ad, Bd, xad, scale, rt)
        ops.moe_lora_grouped_bwd(g_i, x, rt.row_token, Wut, Au, Bu, xau, scale, rt)
        ops.moe_lora_grouped_bwd(g_i, x, rt.row_token, Wgt, Ag, Bg, xag, scale, rt)

    # secondary figure: gate and up as one grouped product (weights concatenated per expert,
    # adapters stacked / block-diagonal), the way art_amd.moe.MoELoRAExperts runs them
    Wgu = torch.cat([Wg, Wu], 1).contiguous()
    Wgut = ops.transpose_batched(Wgu)
    Agu = torch.cat([Ag, Au], 1).contiguous()
    Bgu = torch.zeros(E, 2 * I, 2 * r, dtype=torch.bfloat16, device=dev)
    Bgu[:, :I, :r], Bgu[:, I:, r:] = Bg, Bu
    g_i2 = torch.cat([g_i, g_i], 1).contiguous()

    def step_fused():
        rt = ops.moe_route(logits, k)
        ygu, xagu = ops.moe_lora_grouped_fwd(x, rt.row_token, Wgu, Agu, Bgu, scale, rt)
        yd, xad = ops.moe_lora_grouped_fwd(h, None, Wd, Ad, Bd, scale, rt)
        ops.moe_lora_grouped_bwd(g_h, h, None, Wdt, Ad, Bd, xad, scale, rt)
        ops.moe_lora_grouped_bwd(g_i2, x, rt.row_token, Wgut, Agu, Bgu, xagu, scale, rt)

    dt_sep = timed(step, args.steps, args.warmup)

    # headline: gate and up as one grouped product, the way art_amd.moe.MoELoRAExperts runs them
    for _ in range(args.warmup):
        step_fused()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_fused()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    # the grouped GEMM's own launch time, from a second burst with HIP events around each launch
    ops.profile_enable(True)
    for _ in range(args.steps):
        step_fused()
    torch.cuda.synchronize()
    gemm_ms, gemm_n = ops.profile_collect(ops.PROF_MOE_GEMM)
    ops.profile_enable(False)
    flops = 2 * (3 * 2.0 * n * H * I) + 3 * 6.0 * n * r * (H + I)  # fwd + dx of three projections + rank-r terms
    res = base_result(args, "MoE expert-LoRA grouped GEMM fwd+bwd TFLOP/s", "TFLOP/s", flops / dt / 1e12, dt * 1e3,
                      "C5-moe-qwen3-30b-a3b-share")
    res["config"].update({"tokens": T, "hidden": H, "intermediate": I, "experts": E, "top_k": k, "rank": r,
                          "gate_up": "one grouped product (weights concatenated per expert, adapters stacked)"})
    res["frac_of_bf16_peak"] = flops / dt / 1e12 / PEAK_BF16_TFLOPS
    res["separate"] = {"value": flops / dt_sep / 1e12, "unit": "TFLOP/s", "ms_per_step": dt_sep * 1e3,
                       "frac_of_bf16_peak": flops / dt_sep / 1e12 / PEAK_BF16_TFLOPS,
                       "note": "same algorithmic flops, gate and up as two grouped products"}
    # 4 launches per step, each 2 n H I' flop with I' = 2 I (gate|up) or I (down): mean over the launches
    launch_ms = gemm_ms / max(gemm_n, 1)
    ach = 3 * 2.0 * n * H * I * 2 / 4 / (launch_ms * 1e-3) / 1e12
    # Each expert's weights (3 MiB per projection) serve only ~512 rows: a launch moves, at the least, the
    # activations in, the weights once and the result out, and at 8 TB/s that takes longer than its flops
    # at 2.5 PFLOP/s, so HBM is the roofline that bounds this kernel.
    alg_bytes = (2.0 * (n * H + n * 2 * I + E * 2 * I * H) * 2 + 2.0 * (n * H + n * I + E * I * H) * 2) / 4
    res["roofline"] = {"kernel": "moe_gemm_kernel (mean of the 4 launches per step)", "bound": "hbm",
                       "achieved": alg_bytes / (launch_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                       "frac": alg_bytes / (launch_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                       "algorithmic_bytes": alg_bytes,
                       "traffic": MOE_TRAFFIC_BYTES, "traffic_source": MOE_TRAFFIC_SOURCE,
                       "launch_ms": launch_ms,
                       "mfma": {"achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                "frac": ach / PEAK_BF16_TFLOPS}}
    if not args.no_secondary:
        # The same work the way a stock torch MoE layer does it: softmax -> top-k, stable sort by
        # expert, then a Python loop over the experts with F.linear on each expert's rows, autograd
        # for dx, dA_e, dB_e (weights frozen).
        import torch.nn.functional as F

        def torch_step():
            probs = torch.softmax(logits, -1)
            topv, topi = torch.topk(probs, k, -1)
            order = torch.sort(topi.reshape(-1), stable=True).indices
            row_token = order // k
            counts = torch.bincount(topi.reshape(-1), minlength=E).tolist()
            xs = x[row_token].detach().requires_grad_(True)
            hs = h.detach().requires_grad_(True)
            params = [t.detach().requires_grad_(True) for t in (Ag, Bg, Au, Bu, Ad, Bd)]
            a_g, b_g, a_u, b_u, a_d, b_d = params
            outs, grads, lo = [], [], 0
            for e in range(E):
                hi = lo + counts[e]
                xe, he = xs[lo:hi], hs[lo:hi]
                yg = F.linear(xe, Wg[e]) + scale * F.linear(F.linear(xe, a_g[e]), b_g[e])
                yu = F.linear(xe, Wu[e]) + scale * F.linear(F.linear(xe, a_u[e]), b_u[e])
                yd = F.linear(he, Wd[e]) + scale * F.linear(F.linear(he, a_d[e]), b_d[e])
                outs += [yg, yu, yd]
                grads += [g_i[lo:hi], g_i[lo:hi], g_h[lo:hi]]
                lo = hi
            torch.autograd.backward(outs, grads)

        tdt = timed(torch_step, 3, 1)
        res["torch_gpu_same_algorithm"] = {"value": flops / tdt / 1e12, "unit": "TFLOP/s", "ms_per_step": tdt * 1e3,
                                           "note": "softmax/top-k/stable sort + per-expert F.linear loop with "
                                                   "autograd, bf16, same three projections"}
    if not args.no_cpu_baseline:
        import hashlib

        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import moe_oracle

        # CPU oracle (fp32) of routing and all three projections (gate, up over the gathered token rows,
        # down over the sorted rows): the timing sample, 1 warm-up + 3 runs, median
        cpu_in = {"gate": (x.cpu(), True, Wg.cpu(), Ag.cpu(), Bg.cpu(), g_i.cpu()),
                  "up": (x.cpu(), True, Wu.cpu(), Au.cpu(), Bu.cpu(), g_i.cpu()),
                  "down": (h.cpu(), False, Wd.cpu(), Ad.cpu(), Bd.cpu(), g_h.cpu())}
        times, ref, ref_out = [], None, {}
        for rep in range(4):
            t0 = time.perf_counter()
            ref = moe_oracle.route(logits.cpu(), k)
            for name, (xin, gathered, W_, A_, B_, up_) in cpu_in.items():
                out = moe_oracle.grouped_lora_grads(xin, ref["row_token"] if gathered else None, W_, A_, B_, scale,
                                                    ref["offsets"], up_)
                if rep == 0:
                    ref_out[name] = out
            if rep:
                times.append(time.perf_counter() - t0)
        cdt = sorted(times)[1]
        res["cpu_baseline"] = {"value": flops / cdt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                               "kind": "port",
                               "sample": f"routing + gate, up and down projections fwd+bwd, fp32 torch-CPU oracle, "
                                         f"1 warm-up + 3 runs, median {cdt:.1f} s"}
        # parity of this run: integer outputs of the routing by digest, the fused gate|up product (the
        # measured path) and the down product by rel-L2 against the oracle of each projection
        sha = lambda t: hashlib.sha256(t.cpu().to(torch.int64).contiguous().numpy().tobytes()).hexdigest()
        rt = ops.moe_route(logits, k)
        ints = {}
        for key in ("topk_idx", "perm", "inv_perm", "row_token", "offsets"):
            ints[key] = {"sha256": sha(getattr(rt, key))[:16], "equal": sha(getattr(rt, key)) == sha(ref[key])}
        rel = lambda a, b: ((a.double().cpu() - b.double()).norm() / b.double().norm()).item()
        ygu, xagu = ops.moe_lora_grouped_fwd(x, rt.row_token, Wgu, Agu, Bgu, scale, rt)
        dxr, dAgu, dBgu = ops.moe_lora_grouped_bwd(g_i2, x, rt.row_token, Wgut, Agu, Bgu, xagu, scale, rt)
        dx_tok = dxr[rt.inv_perm.long()].view(T, k, H).float().sum(1)
        yg0, dxg0, dAg0, dBg0 = ref_out["gate"]
        yu0, dxu0, dAu0, dBu0 = ref_out["up"]
        fused = {"y_gate": rel(ygu[:, :I], yg0), "y_up": rel(ygu[:, I:], yu0), "dx": rel(dx_tok, dxg0 + dxu0),
                 "dA_gate": rel(dAgu[:, :r], dAg0), "dA_up": rel(dAgu[:, r:], dAu0),
                 "dB_gate": rel(dBgu[:, :I, :r], dBg0), "dB_up": rel(dBgu[:, I:, r:], dBu0)}
        yd, xad = ops.moe_lora_grouped_fwd(h, None, Wd, Ad, Bd, scale, rt)
        dxd, dAd, dBd = ops.moe_lora_grouped_bwd(g_h, h, None, Wdt, Ad, Bd, xad, scale, rt)
        down = dict(zip(("y", "dx", "dA", "dB"), (rel(a, b) for a, b in zip((yd, dxd, dAd, dBd), ref_out["down"]))))
        res["parity_same_run"] = {"routing_bit_exact": ints, "fused_gate_up": fused, "down": down,
                                  "tolerance_rel_l2": 1e-2}
    return res


def bench_attn(args):
    """Packed-row attention of one layer at the Qwen2.5-7B head shape: a row of 16384 positions
    holding 8 prompts of 128 tokens, each with 4 completions of 480 tokens (the packer's layout),
    28 query / 4 key-value heads of 128.  One step = plan reuse + forward + backward; value =
    algorithmic TFLOP/s over the visible (query, key) pairs: 4 N D Hq forward + 10 N D Hq backward."""
    import torch

    from art_amd import ops, synthetic

    dev = torch.device("cuda:0")
    S, Hq, Hkv, D = 16384, 28, 4, 128
    layout = (8, 128, 4, 480)
    g = torch.Generator().manual_seed(1006)
    q = torch.randn(S, Hq, D, generator=g).to(torch.bfloat16).to(dev)
    k = torch.randn(S, Hkv, D, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(S, Hkv, D, generator=g).to(torch.bfloat16).to(dev)
    d_out = torch.randn(S, Hq, D, generator=g).to(torch.bfloat16).to(dev)
    group, parent = synthetic.packed_row_ids(1006, S, *layout)
    # visible pairs from the layout: a prompt token sees its prompt prefix, a completion token its
    # prompt and its completion prefix, a padding token the padding before it
    npr, pl, nc, cl = layout
    pad = S - npr * (pl + nc * cl)
    n_vis = npr * (pl * (pl + 1) // 2 + nc * (cl * pl + cl * (cl + 1) // 2)) + pad * (pad + 1) // 2
    plan = ops.attn_plan(group.to(dev), parent.to(dev))
    state = {}

    def step():
        out, lse = ops.attn_fwd(q, k, v, plan)
        state["fwd"] = (out, lse)
        state["grads"] = ops.attn_bwd(q, k, v, out, lse, d_out, plan)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ops.profile_enable(True)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    prof = {name: ops.profile_collect(kind) for name, kind in
            (("attn_fwd_kernel", ops.PROF_ATTN_FWD), ("attn_bwd_kv_kernel", ops.PROF_ATTN_BWD_KV),
             ("attn_bwd_dq_kernel", ops.PROF_ATTN_BWD_Q))}
    ops.profile_enable(False)
    unit_flops = 2.0 * n_vis * D * Hq           # one product over the visible pairs
    flops = 14.0 * n_vis * D * Hq
    res = base_result(args, "packed-row attention fwd+bwd TFLOP/s over visible pairs (7B head shape)",
                      "TFLOP/s", flops / dt / 1e12, dt * 1e3, "C3-attention")
    res["config"].update({"positions": S, "q_heads": Hq, "kv_heads": Hkv, "head_dim": D,
                          "layout": "8 x (prompt 128 + 4 completions x 480) + padding",
                          "visible_pairs": n_vis, "visible_fraction_of_causal": n_vis / (S * (S + 1) / 2)})
    executed = {"attn_fwd_kernel": 2, "attn_bwd_kv_kernel": 4, "attn_bwd_dq_kernel": 3}
    res["kernels"] = {}
    for name, (ms, n) in prof.items():
        launch_ms = ms / max(n, 1)
        tf = executed[name] * unit_flops / (launch_ms * 1e-3) / 1e12
        res["kernels"][name] = {"launch_ms": launch_ms, "tflops_executed_on_visible_pairs": tf,
                                "frac": tf / PEAK_BF16_TFLOPS}
    kv = res["kernels"]["attn_bwd_kv_kernel"]
    res["roofline"] = {"kernel": "attn_bwd_kv_kernel", "bound": "mfma",
                       "achieved": kv["tflops_executed_on_visible_pairs"], "peak": PEAK_BF16_TFLOPS,
                       "unit": "TFLOP/s", "frac": kv["frac"], "traffic": None, "launch_ms": kv["launch_ms"]}
    res["plan_ms"] = timed(lambda: ops.attn_plan(group.to(dev), parent.to(dev)), 3, 1) * 1e3
    if not args.no_secondary:
        # The same kernels on a dense causal row of the same shape (one group: every tile full but
        # the diagonal), where the per-kernel rate is not blurred by partly visible tiles.
        zero = torch.zeros(S, dtype=torch.int64, device=dev)
        dplan = ops.attn_plan(zero, zero)
        n_dense = S * (S + 1) // 2

        def dense_step():
            o, l = ops.attn_fwd(q, k, v, dplan)
            return ops.attn_bwd(q, k, v, o, l, d_out, dplan)

        dense_step()
        torch.cuda.synchronize()
        ops.profile_enable(True)
        for _ in range(3):
            dense_step()
        torch.cuda.synchronize()
        dprof = {name: ops.profile_collect(kind) for name, kind in
                 (("attn_fwd_kernel", ops.PROF_ATTN_FWD), ("attn_bwd_kv_kernel", ops.PROF_ATTN_BWD_KV),
                  ("attn_bwd_dq_kernel", ops.PROF_ATTN_BWD_Q))}
        ops.profile_enable(False)
        dunit = 2.0 * n_dense * D * Hq
        res["dense_causal_row"] = {
            name: {"launch_ms": ms / max(n, 1),
                   "tflops_executed": executed[name] * dunit / (ms / max(n, 1) * 1e-3) / 1e12}
            for name, (ms, n) in dprof.items()}
        del dplan
        # The reference's method on the same GPU: the dense [1, S, S] bias of calculate_attn_bias
        # (src/art/local/train.py:177-215) handed to torch's scaled_dot_product_attention.
        import torch.nn.functional as F

        from art_amd.train import calculate_attn_bias

        def torch_step(bias):
            qh, kh, vh = (t.detach().transpose(0, 1).unsqueeze(0).requires_grad_(True) for t in (q, k, v))
            o = F.scaled_dot_product_attention(qh, kh, vh, attn_mask=bias.unsqueeze(1), enable_gqa=True)
            o.backward(d_out.transpose(0, 1).unsqueeze(0))
            return o

        try:
            t0 = time.perf_counter()
            bias = calculate_attn_bias(1, S, dev, group.view(1, S).to(dev), parent.view(1, S).to(dev),
                                       torch.bfloat16)
            torch.cuda.synchronize()
            bias_ms = (time.perf_counter() - t0) * 1e3
            o_ref = torch_step(bias)
            rel = ((o_ref[0].transpose(0, 1).float() - state["fwd"][0].float()).norm()
                   / state["fwd"][0].float().norm()).item()
            tdt = timed(lambda: torch_step(bias), 3, 0)
            res["torch_gpu_same_algorithm"] = {
                "value": flops / tdt / 1e12, "unit": "TFLOP/s", "ms_per_step": tdt * 1e3,
                "bias_ms": bias_ms, "bias_bytes": bias.numel() * bias.element_size(),
                "note": f"dense bf16 bias + torch SDPA (enable_gqa) fwd+bwd, same visible-pair flop count; "
                        f"out rel-L2 against the kernels {rel:.1e}"}
            del bias, o_ref
        except Exception as e:  # the baseline is informative only
            res["torch_gpu_same_algorithm"] = {"error": f"{type(e).__name__}: {e}"[:200]}
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import attn_oracle

        # one prompt with its completions (2048 positions), all heads, dense bias, fwd + bwd
        n = pl + nc * cl
        sl = lambda t: t[:n].cpu()
        t0 = time.perf_counter()
        attn_oracle.attention_grads(sl(q), sl(k), sl(v), group[:n], parent[:n], sl(d_out))
        cdt = time.perf_counter() - t0
        vis_n = pl * (pl + 1) // 2 + nc * (cl * pl + cl * (cl + 1) // 2)
        res["cpu_baseline"] = {"value": 14.0 * vis_n * D * Hq / cdt / 1e12, "unit": "TFLOP/s",
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"first {n} positions (one prompt and its completions), all heads, "
                                         f"dense-bias fp32 torch-CPU oracle fwd+bwd, 1 run of {cdt:.1f} s; "
                                         "same visible-pair flop count"}
    return res


def bench_pack(args):
    """Packer (host code, no kernel): 64 prompts of 256 tokens with 8 completions of 768 tokens each,
    packed into rows of 16384.  value = packed tokens per second of `art_amd.pack`; the baseline is the
    list-based algorithm of the reference restated in oracle/pack_oracle.py on the same inputs."""
    import random

    import torch

    from art_amd import pack

    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import pack_oracle

    g = random.Random(1007)
    results = []
    for pid in range(64):
        prompt = [g.randint(0, 150000) for _ in range(256)]
        for _ in range(8):
            comp = [g.randint(0, 150000) for _ in range(768)]
            results.append(pack_oracle.Result(
                token_ids=prompt + comp, input_pos=list(range(1024)), assistant_mask=[0] * 256 + [1] * 768,
                logprobs=[float("nan")] * 256 + [-g.random() for _ in range(768)], advantage=g.uniform(-1, 1),
                prompt_id=pid, prompt_length=256))
    seq_len = 16384
    out = pack.packed_tensors_from_tokenized_results(results, seq_len, rng=random.Random(1))
    n_tokens = int((out["group_ids"] != -1).sum())
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = pack.packed_tensors_from_tokenized_results(results, seq_len, rng=random.Random(1))
    dt = (time.perf_counter() - t0) / args.steps
    res = base_result(args, "packer tokens/s (host)", "tokens/s", n_tokens / dt, dt * 1e3, "pack-64x8x1024")
    res["dtype"] = "int64/f32"
    res["config"].update({"results": len(results), "rows": out["tokens"].shape[0], "row_length": seq_len,
                          "packed_tokens": n_tokens})
    res["roofline"] = None  # host code: no kernel to place on a roofline
    if torch.cuda.is_available():
        stager = pack.RowStager(seq_len, torch.device("cuda:0"))
        stager.to_device(out, 0)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            stager.to_device(out, 0)
        torch.cuda.synchronize()
        res["row_to_device_ms"] = (time.perf_counter() - t0) / 20 * 1e3
        rows8 = {k: v[:1].expand(8, -1).contiguous() for k, v in out.items()}
        t0 = time.perf_counter()
        for _row in stager.rows(rows8):
            pass
        torch.cuda.synchronize()
        res["row_pipelined_ms"] = (time.perf_counter() - t0) / 8 * 1e3
    if not args.no_cpu_baseline:
        t0 = time.perf_counter()
        ref = pack_oracle.pack(results, seq_len, rng=random.Random(1))
        cdt = time.perf_counter() - t0
        assert all(torch.equal(ref[k].nan_to_num(0.0) if ref[k].is_floating_point() else ref[k],
                               out[k].nan_to_num(0.0) if out[k].is_floating_point() else out[k]) for k in ref)
        res["cpu_baseline"] = {"value": n_tokens / cdt, "unit": "tokens/s", "cores": 1, "kind": "port",
                               "sample": f"the same {len(results)} results, list-based algorithm, 1 run of {cdt:.2f} s"}
    return res


def bench_optim(args):
    """Fused AdamW + global gradient-norm clip over all rank-8 adapters of a Qwen2.5-7B (q, k, v, o, gate,
    up, down of 28 layers = 20.2 M parameters in one flat buffer).  value = parameters updated per second;
    roofline = HBM bytes (4 B for the norm + 16 B read + 14 B written per parameter)."""
    import torch

    from art_amd.optim import FlatParams, FusedAdamW

    dev = torch.device("cuda:0")
    H, KV, I, r, L = 3584, 512, 18944, 8, 28
    shapes = {}
    for l in range(L):
        for name, (i, o) in (("q", (H, H)), ("k", (H, KV)), ("v", (H, KV)), ("o", (H, H)), ("gate", (H, I)),
                             ("up", (H, I)), ("down", (I, H))):
            shapes[f"{l}.{name}.A"] = (r, i)
            shapes[f"{l}.{name}.B"] = (o, r)
    flat = FlatParams(shapes, dev)
    g = torch.Generator().manual_seed(1008)
    flat.master.copy_(0.02 * torch.randn(flat.numel, generator=g))
    flat.grad.copy_(0.01 * torch.randn(flat.numel, generator=g))
    opt = FusedAdamW(flat)
    dt = timed(opt.step, args.steps, args.warmup)
    n = flat.numel
    res = base_result(args, "fused AdamW + grad-norm clip, parameters/s", "params/s", n / dt, dt * 1e3,
                      "adapters-7B-r8")
    res["dtype"] = "f32"
    res["config"].update({"parameters": n, "tensors": len(shapes)})
    gbs = 34.0 * n / dt / 1e9
    res["roofline"] = {"kernel": "sumsq_partial_kernel + adamw_kernel", "bound": "hbm", "achieved": gbs,
                       "peak": 8000.0, "unit": "GB/s", "frac": gbs / 8000.0, "traffic": None}
    # the same step with the moments in the 8-bit block-wise form of `paged_adamw_8bit`:
    # 4 B for the norm + 10 B read + 8 B written per parameter, 2 B of state instead of 8
    from art_amd.optim import FusedAdamW8bit

    opt8 = FusedAdamW8bit(flat)
    dt8 = timed(opt8.step, args.steps, args.warmup)
    res["moments_8bit"] = {"value": n / dt8, "unit": "params/s", "ms_per_step": dt8 * 1e3,
                           "gb_per_s": 22.0 * n / dt8 / 1e9, "state_bytes_per_param": 2 + 8 / 256,
                           "state_bytes_per_param_f32": 8}
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import optim_oracle

        p0, gr = flat.master.cpu(), flat.grad.cpu()
        t0 = time.perf_counter()
        optim_oracle.adamw_steps(p0, [gr] * 3, 5e-6, (0.9, 0.99), 1e-8, 0.1, 0.1)
        cdt = (time.perf_counter() - t0) / 3
        res["cpu_baseline"] = {"value": n / cdt, "unit": "params/s", "cores": torch.get_num_threads(),
                               "kind": "port", "sample": f"torch.optim.AdamW + clip_grad_norm_ on the flat fp32 "
                                                         f"tensor, mean of 3 steps of {cdt:.3f} s"}
    return res


def bench_nf4(args):
    """NF4 -> bf16 dequantisation of one gate projection of a Qwen2.5-7B (18944 x 3584, block size 64).
    value = elements per second; roofline = HBM bytes (0.5625 B read + 2 B written per element)."""
    import numpy as np
    import torch

    from art_amd import ops

    dev = torch.device("cuda:0")
    n = 18944 * 3584
    g = torch.Generator().manual_seed(1009)
    packed = torch.randint(0, 256, (n // 2,), generator=g, dtype=torch.uint8).to(dev)
    absmax = (0.05 * torch.rand(n // 64, generator=g)).to(dev)
    out = torch.empty(n, dtype=torch.bfloat16, device=dev)
    dt = timed(lambda: ops.nf4_dequant(packed, absmax, out=out), args.steps, args.warmup)
    res = base_result(args, "NF4 dequantisation elements/s", "elements/s", n / dt, dt * 1e3, "gate-proj-7B")
    res["dtype"] = "u8->bf16"
    res["config"].update({"elements": n, "blocksize": 64})
    gbs = 2.5625 * n / dt / 1e9
    res["roofline"] = {"kernel": "nf4_dequant_kernel", "bound": "hbm", "achieved": gbs, "peak": 8000.0,
                       "unit": "GB/s", "frac": gbs / 8000.0, "traffic": None}
    # The two ways to run a LoRA projection on a 4-bit base weight (gate projection of config 2:
    # 8192 tokens, 2048 -> 11008, rank 8), forward + backward: bf16 weight and transposed copy
    # resident (dequantised once), or the 4-bit form only and the 16-bit weight inside each call.
    from art_amd.quant import NF4Weight

    T, n_in, n_out, r = 8192, 2048, 11008, 8
    q = NF4Weight(torch.randint(0, 256, (n_out * n_in // 2,), generator=g, dtype=torch.uint8).to(dev),
                  (n_out, n_in), absmax=(0.05 * torch.rand(n_out * n_in // 64, generator=g)).to(dev))
    x = torch.randn(T, n_in, generator=g).to(torch.bfloat16).to(dev)
    A = (0.02 * torch.randn(r, n_in, generator=g)).to(torch.bfloat16).to(dev)
    B = (0.01 * torch.randn(n_out, r, generator=g)).to(torch.bfloat16).to(dev)
    up = torch.randn(T, n_out, generator=g).to(torch.bfloat16).to(dev)
    Wd, Wt = q.dequantize(), q.dequantize_transposed()

    def resident():
        y, xa = ops.lora_linear_fwd(x, Wd, A, B, 2.0)
        ops.lora_linear_bwd(up, x, Wt, A, B, xa, 2.0)

    def transient():
        y, xa = ops.lora_linear_fwd_nf4(x, q, A, B, 2.0)
        ops.lora_linear_bwd_nf4(up, x, q, A, B, xa, 2.0)

    t_res = timed(resident, args.steps, args.warmup)
    t_tr = timed(transient, args.steps, args.warmup)
    res["lora_on_nf4_base"] = {
        "shape": {"tokens": T, "in": n_in, "out": n_out, "rank": r},
        "resident_bf16": {"us_fwd_bwd": t_res * 1e6, "weight_bytes_resident": 4 * n_out * n_in + q.nbytes()},
        "nf4_only": {"us_fwd_bwd": t_tr * 1e6, "weight_bytes_resident": q.nbytes(),
                     "transient_workspace_bytes": 2 * n_out * n_in},
        "time_ratio": t_tr / t_res}
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import quant_oracle

        m = 64 * 65536
        pk, am = packed[: m // 2].cpu().numpy(), absmax[: m // 64].cpu().numpy()
        t0 = time.perf_counter()
        quant_oracle.to_bf16_bits(quant_oracle.dequantize(pk, am, 64))
        cdt = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": m / cdt, "unit": "elements/s", "cores": 1, "kind": "port",
                               "sample": f"first {m} elements, numpy oracle, 1 run of {cdt:.2f} s"}
    return res


def torch_same_algorithm_step(hidden, lm_head, tokens, old, adv, mask, weights, chunk=1024, eps=0.2):
    """The reference's own algorithm for this path, written with stock torch ops and run on the
    same GPU (src/art/local/train.py:111-151, 245-285): per chunk of positions a bf16 matmul
    against the transposed lm_head view, gather, logsumexp; then the clipped loss on the shifted
    tensors and autograd back to the hidden states.  The reference itself cannot be imported
    (its dependencies are absent), so this is a baseline of the method, not of its code."""
    import torch
    import torch.nn.functional as F

    shifted = lambda t, pad: F.pad(t[:, 1:], (0, 1), value=pad)
    hs = hidden.detach().unsqueeze(0).requires_grad_(True)             # [1, T, H]
    head_t = lm_head.t()                                               # [H, V] view of [V, H]
    ids = shifted(tokens.unsqueeze(0), 0)
    parts = []
    for h_c, id_c in zip(hs.split(chunk, 1), ids.split(chunk, 1)):
        logits = h_c @ head_t
        parts.append(logits.gather(-1, id_c.unsqueeze(-1)).squeeze(-1) - logits.logsumexp(-1))
    new = torch.cat(parts, 1)
    old_s = shifted(old.unsqueeze(0), 0.0)
    adv_s = shifted(adv.unsqueeze(0), 0.0)
    m = shifted(mask.unsqueeze(0), False).to(new.dtype)
    w = shifted(weights.unsqueeze(0), 0.0)
    old_s = torch.where(torch.isnan(old_s), new.detach(), old_s)
    ratio = torch.exp(new - old_s)
    pl = -torch.minimum(ratio * adv_s, ratio.clip(1 - eps, 1 + eps) * adv_s) * w * m
    loss = pl.sum() / (m.sum() + 1e-6)
    loss.backward()
    return loss.detach(), hs.grad


class GpuStateSampler:
    """Polls the amdgpu hwmon files (shader clock, socket power, power cap) from a thread
    while a burst of steps runs; sysfs reads only, no GPU runtime calls.  Fields that the
    box does not expose are left out."""

    def __init__(self, period_s=0.01):
        import glob
        self.period = period_s
        self.files = {}
        self.dpm_sclk = None
        for hw in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
            for key, names in (("sclk_mhz", ("freq1_input",)), ("power_w", ("power1_average", "power1_input")),
                               ("power_cap_w", ("power1_cap",))):
                for n in names:
                    p = os.path.join(hw, n)
                    if key not in self.files and os.path.exists(p):
                        self.files[key] = p
            if self.files:
                # the current shader clock is the starred line of pp_dpm_sclk ("1: 1710Mhz *")
                dpm = os.path.join(os.path.dirname(os.path.dirname(hw)), "pp_dpm_sclk")
                if "sclk_mhz" not in self.files and os.path.exists(dpm):
                    self.dpm_sclk = dpm
                break
        self.samples = {k: [] for k in self.files}
        if self.dpm_sclk:
            self.samples["sclk_mhz"] = []
        self._stop = False
        self._thread = None

    def _read(self):
        for k, p in self.files.items():
            try:
                with open(p) as f:
                    self.samples[k].append(float(f.read().strip()) / 1e6)  # Hz -> MHz, uW -> W
            except (OSError, ValueError):
                pass
        if self.dpm_sclk:
            try:
                with open(self.dpm_sclk) as f:
                    for line in f:
                        if "*" in line:
                            self.samples["sclk_mhz"].append(float(line.split(":")[1].lower().split("mhz")[0]))
            except (OSError, ValueError, IndexError):
                pass

    def _run(self):
        while not self._stop:
            self._read()
            time.sleep(self.period)

    def __enter__(self):
        import threading
        if self.files or self.dpm_sclk:
            self._thread = threading.Thread(target=self._run, daemon=True)
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        if self._thread is not None:
            self._thread.join()

    def summary(self):
        out = {}
        for k, v in self.samples.items():
            if v:
                v = sorted(v)
                out[k] = {"median": v[len(v) // 2], "min": v[0], "max": v[-1], "samples": len(v)}
        return out or None


def bench_ceiling(args, hidden=None, lm_head=None, seconds=0.6):
    """What the part sustains under its power limit, measured in this run, with the shader
    clock and socket power sampled under each load:
      mfma_only        MFMA 32x32x16 bf16 instructions alone on random operands (no LDS, no memory)
      hipblaslt        torch.matmul (hipBLASLt) on the forward shape of the fused step,
                       [chunk, H] x [H, V] with the bench's own hidden states and lm_head
      artk_gemm_nt     this library's plain GEMM (the shared main loop, bf16 store) on that shape
      stream_copy      a plain device copy (HBM read + write bytes per second)."""
    import torch

    from art_amd import ops

    dev = torch.device("cuda:0")
    if hidden is None:
        g = torch.Generator().manual_seed(1003)
        hidden = torch.randn(5632, 3584, generator=g).to(torch.bfloat16).to(dev)
        lm_head = (0.02 * torch.randn(152064, 3584, generator=g)).to(torch.bfloat16).to(dev)
    chunk = min(5632, hidden.shape[0])
    h = hidden[:chunk].contiguous()
    V, H = lm_head.shape
    out = {"shape": {"positions": chunk, "hidden": H, "vocab": V}}

    def run(fn, flop=None, nbytes=None):
        """Repeat fn for about `seconds`, HIP-event timed, with clock and power sampled meanwhile."""
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        reps = max(3, int(seconds * 1e3 / max(e0.elapsed_time(e1), 1e-3)))
        with GpuStateSampler() as sampler:
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        rec = {"ms": ms, "reps": reps}
        if flop is not None:
            rec["tflops"] = flop / (ms * 1e-3) / 1e12
            rec["frac_of_bf16_peak"] = rec["tflops"] / PEAK_BF16_TFLOPS
        if nbytes is not None:
            rec["gb_per_s"] = nbytes / (ms * 1e-3) / 1e9
        st = sampler.summary() or {}
        for k in ("sclk_mhz", "power_w"):
            if k in st:
                rec[k] = st[k]["median"]
        return rec

    operands = torch.randn(1 << 20).to(torch.bfloat16).to(dev)
    blocks = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.empty(blocks * 512, dtype=torch.float32, device=dev)
    iters = 40000
    flop = float(blocks) * 8 * iters * 32 * 32768.0
    out["mfma_only"] = run(lambda: ops.mfma_loop(operands, iters, blocks, sink), flop=flop)
    out["mfma_only_16x16x32"] = run(lambda: ops.mfma_loop(operands, iters, blocks, sink, shape="16x16x32"), flop=flop)
    gemm_flop = 2.0 * chunk * V * H
    w_t = lm_head.t()
    dst = torch.empty((chunk, V), dtype=torch.bfloat16, device=dev)
    out["hipblaslt"] = run(lambda: torch.matmul(h, w_t, out=dst), flop=gemm_flop)
    del dst
    out["artk_gemm_nt"] = run(lambda: ops.gemm_nt(lm_head, h), flop=gemm_flop)
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(3)
    dst = torch.empty_like(src)
    out["stream_copy"] = run(lambda: ops.stream_copy(src, dst), nbytes=2.0 * src.numel())
    del src, dst
    # LDS bytes per clock of a CU, reads alone and with the DMA writes of the GEMM's fill mixed in
    # (one 1 KiB buffer_load ... lds per 2 or 3 reads: the 4-wave and the 8-wave loop's ratio)
    lds = {}
    for name, waves, kind, rpd in (("ds_read_b128_4waves", 4, 1, 0), ("ds_read_b128_8waves", 8, 1, 0),
                                   ("ds_read_b64_tr_b16_8waves", 8, 2, 0), ("ds_read_b128_4waves_dma", 4, 1, 2),
                                   ("ds_read_b128_8waves_dma", 8, 1, 3), ("ds_read_b64_tr_b16_8waves_dma", 8, 2, 3)):
        ops.lds_probe(waves, kind, rpd, 200, blocks, dev)
        lds[name] = ops.lds_probe(waves, kind, rpd, 20000, blocks, dev)
    out["lds_bytes_per_clk_per_cu"] = lds
    if not args.no_secondary:
        # what each part of the main loop costs: the persistent plain GEMM on the same shape, bf16 output,
        # on the library's loops, on the MFMA 16x16x32 loops (4-wave with parts switched off, 8-wave) and on
        # 256 x 128 tiles with two work-groups per CU
        probe_out = torch.empty((chunk, V), dtype=torch.bfloat16, device=dev)
        cyc = torch.zeros(2 * blocks, dtype=torch.int64, device=dev)
        rows = (("8wave_32x32x16_group8", 0, 0, 8, False), ("8wave_32x32x16_group4", 0, 0, 4, False),
                ("8wave_32x32x16_group2", 0, 0, 2, False), ("8wave_32x32x16_group16", 0, 0, 16, False),
                ("8wave_32x32x16_first_wave_fills_group4", 5, 0, 4, False),
                ("8wave_32x32x16_first_wave_fills_all_early_group4", 5, 1, 4, False),
                ("4wave_32x32x16_group4", 1, 0, 4, False), ("4wave_16x16x32_group4", 2, 0, 4, False),
                ("4wave_16x16x32_group8", 2, 0, 8, False), ("8wave_16x16x32_group4", 3, 0, 4, False),
                ("two_workgroups_per_cu_256x128_group4", 4, 0, 4, False),
                ("4wave_16x16x32_all_fetches_hit_L2", 2, 0, 4, True),
                ("4wave_16x16x32_no_wait_no_barrier", 2, 2, 4, False), ("4wave_16x16x32_no_fill", 2, 1, 4, False),
                ("4wave_16x16x32_no_fill_no_barrier", 2, 3, 4, False),
                ("4wave_16x16x32_no_lds_reads", 2, 4, 4, False),
                ("4wave_16x16x32_mfma_and_stores_only", 2, 7, 4, False))
        table = {}
        for name, loop, abl, grp, same in rows:
            rec = run(lambda: ops.gemm_loop_probe(lm_head, h, loop=loop, ablate=abl, group=grp, same_tile=same,
                                                  out=probe_out, cycles=cyc), flop=gemm_flop)
            c = cyc.view(-1, 2).double().cpu()
            rec["core_ghz_in_kernel"] = float((c[:, 0].sum() / (c[:, 1].sum() * 10.0)).item())
            table[name] = rec
        out["main_loop_parts"] = table
    return out


def main():
    args = parse()
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        print("bench.py: this build runs on ONE GPU only (the path shards over tokens with no "
              "exchange, which is not built). Re-run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    if args.workload == "pack":
        print(json.dumps(bench_pack(args)))
        return

    import torch

    from art_amd import ops, synthetic

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    single = {"lora": bench_lora, "moe": bench_moe, "attn": bench_attn, "optim": bench_optim,
              "nf4": bench_nf4, "ceiling": bench_ceiling}
    if args.workload in single:
        res = single[args.workload](args)
        if args.workload == "ceiling":
            res = {"metric": "sustained ceilings of the part (MFMA-only loop, vendor GEMM, own GEMM, copy)",
                   "n_gpus": 1, "data": "synthetic", **res}
        print(json.dumps(res))
        return
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

    chunk = args.chunk_tokens or ops.DEFAULT_CHUNK_TOKENS  # 0 = library default
    ws = torch.empty(ops.grpo_fused_workspace_bytes(T, V, H, chunk), dtype=torch.uint8, device=dev)
    out = (torch.empty(5, dtype=torch.float32, device=dev),
           torch.empty(T, dtype=torch.float32, device=dev),
           torch.empty((T, H), dtype=torch.bfloat16, device=dev))

    def step(skip_inactive=False):
        ops.grpo_fused(hidden, lm_head, lm_head_t, tokens, old, adv, mask, weights, None, T, 0.8,
                       1.2, 0.0, chunk, workspace=ws, out=out, skip_inactive=skip_inactive)

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
    # The headline: exactly `steps` calls between two device synchronisations, nothing else
    # on the stream but one event per step (per-kernel timing is off here).
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(args.steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    step_ms = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    # Per-kernel durations from a second burst of the same steps with the library's HIP-event
    # brackets switched on (outside the headline's timed region).
    ops.profile_enable(True)
    t0 = time.perf_counter()
    for i in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt_profiled = time.perf_counter() - t0
    fwd_ms, fwd_n = ops.profile_collect(ops.PROF_LMHEAD_FWD)
    bwd_ms, bwd_n = ops.profile_collect(ops.PROF_DHIDDEN_GEMM)
    sm_ms, sm_n = ops.profile_collect(ops.PROF_TARGET_REF)
    ops.profile_enable(False)
    mask_count = int(out[0][3].item())
    # positions whose loss coefficient is non-zero (masked in, non-zero advantage, unclipped):
    # exactly the rows with a non-zero d_hidden row, which are the rows the backward GEMM runs
    t_active_dense = int((out[2] != 0).any(dim=1).sum().item())

    # Clock and power while the same step runs back to back (its own burst, outside the timing).
    with GpuStateSampler() as sampler:
        for _ in range(max(args.steps, 10)):
            step()
        torch.cuda.synchronize()
    gpu_state = sampler.summary()

    # Secondary figure (never `value`): the same batch with the projection restricted to the
    # positions that can contribute to the loss; same loss and gradient, less work.
    dt_skip = None
    if not args.no_secondary:
        for _ in range(args.warmup):
            step(True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step(True)
        torch.cuda.synchronize()
        dt_skip = time.perf_counter() - t0
        step()  # leave the dense results in `out`
        torch.cuda.synchronize()

    # Secondary figure: the reference's method in stock torch ops on this GPU.
    torch_ms = None
    if not args.no_secondary:
        targs = (hidden, lm_head, tokens, old, adv, mask, weights)
        t_loss, t_grad = torch_same_algorithm_step(*targs)   # warm-up, also a cross-check
        torch.cuda.synchronize()
        t_rel = ((t_grad[0].float() - out[2].float()).norm() / out[2].float().norm()).item()
        n_rep = 3
        t0 = time.perf_counter()
        for _ in range(n_rep):
            torch_same_algorithm_step(*targs)
        torch.cuda.synchronize()
        torch_ms = (time.perf_counter() - t0) / n_rep * 1e3
        torch_note = (f"bf16 matmul/gather/logsumexp per 1024 positions + autograd; d_hidden rel-L2 "
                      f"against the kernels {t_rel:.1e}; loss {float(t_loss):.6f}")
        del t_grad

    ms_per_step = dt / args.steps * 1e3
    tokens_per_s = T / (dt / args.steps)
    # rows whose loss coefficient is zero (non-assistant positions) have a zero d_hidden row
    # and are skipped by the backward: the algorithmic work counts them in the forward only
    t_active = int((out[2] != 0).any(dim=1).sum().item())
    alg_flops_step = 2.0 * T * V * H + 2.0 * t_active * V * H
    # dominant kernel: one launch covers `chunk` positions against the whole vocabulary
    fwd_launch_ms = fwd_ms / max(fwd_n, 1)
    launches_per_step = fwd_n / args.steps
    chunk = chunk or -(-T // int(launches_per_step))  # report the chunk the library chose (approximate)
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
        "ms_per_step_median": step_ms[len(step_ms) // 2],
        "ms_per_step_min": step_ms[0],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": case.name, "tokens": T, "hidden": H, "vocab": V,
                   "chunk_tokens": chunk, "mask_fraction": float(case.assistant_mask.float().mean()),
                   "mask_count": mask_count, "t_active": t_active},
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
            "traffic_source": TRAFFIC_SOURCE.get(args.workload),
            "launch_ms": fwd_launch_ms,
            "launch_ms_source": "HIP events around each launch in a second burst of the same steps "
                                f"({dt_profiled / args.steps * 1e3:.3f} ms per step with the events on)",
            "launches_per_step": launches_per_step,
        },
        "kernels": {
            "dhidden_gemm_kernel": {"launch_ms": bwd_launch_ms, "tflops": bwd_achieved,
                                    "frac": bwd_achieved / PEAK_BF16_TFLOPS},
            "target_ref_kernel": {"launch_ms": sm_ms / max(sm_n, 1)},
        },
    }
    assert t_active == t_active_dense
    if gpu_state:
        result["gpu_state_under_load"] = gpu_state
    if dt_skip is not None:
        result["skip_inactive"] = {"value": T / (dt_skip / args.steps), "unit": "tokens/s",
                                   "ms_per_step": dt_skip / args.steps * 1e3,
                                   "note": "flag ARTK_FUSED_SKIP_INACTIVE; batch tokens per second"}
    if torch_ms is not None:
        result["torch_gpu_same_algorithm"] = {"value": T / (torch_ms * 1e-3), "unit": "tokens/s",
                                              "ms_per_step": torch_ms, "note": torch_note}
    result["config"]["input_sha256"] = input_digests(case)
    if not args.no_cpu_baseline:
        result["cpu_baseline"], parity = cpu_baseline(case, args.cpu_sample_tokens, out[1], out[2], mask_count)
        if parity:
            result["parity_same_run"] = parity
    if args.workload == "c3" and not args.no_sub_records:
        # The other half of the headline metric (LoRA linear TFLOP/s, % of peak), the expert-LoRA
        # configuration and the measured ceilings of this part, as records of their own.
        gemm_inputs = (hidden, lm_head)
        del ws, out, lm_head_t
        result["ceiling"] = bench_ceiling(args, *gemm_inputs)
        del gemm_inputs, hidden, lm_head
        torch.cuda.empty_cache()
        result["lora"] = bench_lora(args)
        result["moe"] = bench_moe(args)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
