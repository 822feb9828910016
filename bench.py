#!/usr/bin/env python3
"""Benchmark of the MoE feed-forward path on one MI355X.

Default workload (the configuration the metric is quoted on): one MoE layer at
hidden 2048 / 512 experts / top-10 / intermediate 512 with IQ2_XXS expert
blocks, decode batch 1, seeded RMS-normalised tokens whose top-11 router logits
are at least 1e-3 apart.  A step is one token through the layer; inputs and
weights are resident in HBM before the timed region; every step uses another
token, hence other experts.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Prints one JSON line.  `value` is microseconds per layer per token (lower is
better).  `roofline` is for the kernel that moves the most bytes, timed live
with HIP events on the launch stream.  `cpu_baseline` times the CPU path (the reference's own
compiled C when oracle/_ref is present, else the oracle port) on a bounded
sample of the same tokens, single thread, and the same sample is used to check
the GPU results (ids exact, outputs within 1e-3 + 1e-4 relative).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

import picoforge_amd as pf  # noqa: E402
from picoforge_amd import abi, workloads  # noqa: E402

HBM_PEAK_GBPS = 8000.0

WORKLOADS = {
    "iq2xxs_decode": dict(type=abi.GGUF_IQ2_XXS, tokens=1, label="IQ2_XXS experts, decode batch 1"),
    "q4k_decode": dict(type=abi.GGUF_Q4_K, tokens=1, label="Q4_K experts, decode batch 1"),
    "q4k_verify4": dict(type=abi.GGUF_Q4_K, tokens=4, label="Q4_K experts, 4-token verify batch, ~50% expert overlap"),
}
STAGES = ["pf_k_dec_router (router logits)", "pf_k_dec_gate_up (routing, gate/up + SwiGLU, routed and shared)",
          "pf_k_dec_down (down products, routed and shared, combine)"]


def device_forward_sample(api, layer, x, tokens):
    """Runs the first sample batches through the device path and returns y, ids, weights."""
    outs = []
    for b in range(len(x)):
        _, y, ids, w = layer.forward(x[b].reshape(tokens, -1))
        outs.append((y, ids, w))
    return outs


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default="iq2xxs_decode", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-sample", type=int, default=None, help="tokens timed on the CPU path (default ~15 s of work)")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MIB",
                    help="also launch a plain copy kernel of this many MiB three times (byte-counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every box has one GPU); use --gpus 1")

    wl = WORKLOADS[args.workload]
    api = pf.load_product()
    hip = api.hip
    if hip.device_count() < 1:
        sys.exit("no HIP device: the benchmark runs the HIP path only")
    cfg = workloads.measured_config()
    tokens = wl["tokens"]
    t0 = time.time()
    weights = pf.LayerWeights.synthetic(cfg, wl["type"], seed=args.seed)
    n_inputs = max(1, min(args.steps, 10000))
    if tokens == 1:
        x, info = workloads.decode_tokens(weights, n_inputs, seed=args.seed)
        x = x.reshape(n_inputs, 1, cfg.hidden_size)
        unique = float(cfg.top_k)
    else:
        n_inputs = min(n_inputs, 2000)
        x, info = workloads.verify_batches(weights, n_inputs, seed=args.seed)
        unique = info["mean_unique_experts"]
    prep_s = time.time() - t0

    layer = pf.MoeLayer(api, cfg, weights, tokens)
    moe, work = layer.device_handles()     # the layer's HBM-resident tensors and scratch, for the timed loop
    d_x = hip.to_device(x)
    d_y = hip.to_device(np.zeros((tokens, cfg.hidden_size), dtype=np.float32))

    ms = C.c_float()
    hip.check(hip.moe_time_forwards(moe, work, d_x, n_inputs, d_y, tokens, args.warmup, C.byref(ms)), "warmup")
    hip.check(hip.synchronize(), "sync")
    wall0 = time.perf_counter()
    hip.check(hip.moe_time_forwards(moe, work, d_x, n_inputs, d_y, tokens, args.steps, C.byref(ms)), "timed loop")
    hip.check(hip.synchronize(), "sync")
    wall_ms = (time.perf_counter() - wall0) * 1e3
    ms_per_step = ms.value / args.steps
    us_per_token = ms_per_step * 1e3 / tokens
    err_word = hip.from_device(hip.work_error_word(work), (1,), np.uint32)[0]
    exact = C.c_uint32()
    hip.work_exact_rows(work, C.byref(exact))

    # Per-kernel durations inside the dependent chain: graph replays of the first 1, 2, 3
    # kernels of every forward, bracketed by HIP events on the launch stream; a kernel's
    # duration is the difference between consecutive replays (it includes the dispatch gap
    # before it, as a profiler's start-to-end time of a dependent kernel does).
    stage = (C.c_float * 4)()
    hip.check(hip.moe_profile_stages(moe, work, d_x, n_inputs, d_y, tokens, min(args.steps, 2000), stage), "stages")
    stage_us = [max(float(stage[j]) * 1e3, 1e-3) for j in range(3)]

    alg_bytes = workloads.algorithmic_bytes_per_token(wl["type"], unique_experts=unique)
    block, size = abi.BLOCK[wl["type"]]
    h, i, s_i = cfg.hidden_size, cfg.intermediate, cfg.shared_intermediate
    # algorithmic bytes per launch: what each kernel must read once
    stage_bytes = [(cfg.experts + 1) * h * 4,
                   unique * 2 * i * h // block * size + 2 * s_i * h // block * size,
                   unique * h * i // block * size + h * s_i // block * size]
    dom = int(np.argmax(stage_bytes))
    achieved = stage_bytes[dom] / (stage_us[dom] * 1e-6) / 1e9

    # CPU baseline and parity on a bounded sample of the same inputs
    ref = pf.load_reference()
    cpu_api, kind = (ref, "reference") if ref is not None else (pf.load_oracle(), "port")
    per_token_guess = 0.55 if wl["type"] == abi.GGUF_IQ2_XXS else 0.32
    sample = args.cpu_sample or max(1, int(15.0 / per_token_guess / tokens))
    sample = min(sample, n_inputs)
    with pf.MoeLayer(cpu_api, cfg, weights, tokens) as cpu:
        c0 = time.perf_counter()
        cpu_out = [cpu.forward(x[b].reshape(tokens, -1))[1:] for b in range(sample)]
        cpu_s = time.perf_counter() - c0
    gpu_out = device_forward_sample(api, layer, x[:sample], tokens)
    ids_equal = all((g[1] == c[1]).all() for g, c in zip(gpu_out, cpu_out))
    max_abs = max(float(np.abs(g[0] - c[0]).max()) for g, c in zip(gpu_out, cpu_out))
    within = all((np.abs(g[0] - c[0]) <= 1e-3 + 1e-4 * np.abs(c[0])).all() for g, c in zip(gpu_out, cpu_out))
    layer.close()
    if args.copy_probe:
        hip.check(hip.copy_probe(args.copy_probe << 20, 3), "copy probe")

    result = {
        "metric": "moe_decode_us_per_layer_token",
        "value": round(us_per_token, 3),
        "unit": "us/layer/token",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"one MoE layer, hidden 2048, 512 experts, top-10, intermediate 512, shared 512; "
                               f"{wl['label']}; {n_inputs} seeded inputs, top-11 logit margins >= 1e-3",
                   "tokens_per_step": tokens, "expert_format": {12: "Q4_K", 16: "IQ2_XXS"}[wl["type"]],
                   "unique_experts_per_step": unique, "inputs": info},
        "hbm_GBps_on_algorithmic_bytes": round(alg_bytes / (ms_per_step * 1e-3) / 1e9, 1),
        "algorithmic_bytes_per_step": int(alg_bytes),
        "tokens_per_s": round(tokens / (ms_per_step * 1e-3), 1),
        "roofline": {"bound": "hbm", "kernel": STAGES[dom], "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "bytes_per_launch": int(stage_bytes[dom]), "us_per_launch": round(stage_us[dom], 3)},
        "kernel_us": dict(zip(STAGES, [round(v, 3) for v in stage_us])),
        "kernel_bytes": dict(zip(STAGES, [int(b) for b in stage_bytes])),
        "cpu_baseline": {"value": round(cpu_s / (sample * tokens) * 1e6, 1), "unit": "us/layer/token", "cores": 1,
                         "kind": kind, "sample": f"first {sample} steps ({sample * tokens} tokens) of the same inputs, "
                                                   f"{cpu_s:.1f} s"},
        "parity_on_sample": {"ids_equal": bool(ids_equal), "within_1e-3_abs_1e-4_rel": bool(within),
                             "max_abs_err": max_abs, "error_word": int(err_word), "serial_order_reroutes": int(exact.value)},
        "wall_ms_timed_loop": round(wall_ms, 2), "prep_s": round(prep_s, 1),
    }
    print(json.dumps(result))
    if not (ids_equal and within and err_word == 0):
        sys.exit("parity check failed on the sample")


if __name__ == "__main__":
    main()
