#!/usr/bin/env python3
"""Benchmark of the MoE feed-forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Default (`--workload all`): one JSON line whose headline (`metric`, `value`, `roofline`,
`cpu_baseline`) is the Q4_K decode layer -- one token through one MoE layer at hidden 2048 / 512
experts / top-10 / intermediate 512 / shared 512 -- and whose `configs` object carries a record of
the same form for each further benchmark configuration: IQ2_XXS decode, the 4-token Q4_K verify
batch, the 1024-token Q4_K prefill chunk under a Zipf(1.1) router, and the 48-layer resident stack.
`--workload NAME` runs one configuration alone and prints its record as the line.

A step is one token batch through the layer (or, for the stack, one token through all layers);
inputs and weights are resident in HBM before the timed region; every step uses another seeded
input, hence other experts.  K steps are captured once into HIP graphs and replayed until at least
50 ms have been timed; `ms_per_step` is the median over the replays (p10 / p90 beside it), each
replay bracketed by HIP events on the launch stream.  `roofline` is for the kernel that moves the
most bytes: its duration is the difference between replays of the chain cut after it and before it
(events on the launch stream).  `cpu_baseline` times the CPU path (the reference's own compiled C
when oracle/_ref is present, else the oracle port) on a bounded sample of the same inputs, one
thread, and the same sample checks the GPU results (ids exact, outputs within 1e-3 + 1e-4 relative).

Further workloads: iq2xxs_prefill1024; q2profile_* / q4profile_* (the format mixes of real checkpoints)
and q2ckpt_* / q4ckpt_* (those mixes at the checkpoints' own widths: hidden 2560, intermediate and shared
640, the Q2_K down projection stored 768 wide); *_hc: the layer between its two hyper-connection steps.
"""
import argparse
import ctypes as C
import hashlib
import json
import math
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

import picoforge_amd as pf  # noqa: E402
from picoforge_amd import abi, workloads  # noqa: E402
from oracle.load import load_oracle, load_reference  # noqa: E402  (the cpu_baseline leg and its parity sample only)

FORMAT_LABEL = {12: "Q4_K", 16: "IQ2_XXS", "q2": "IQ2_XXS gate/up, Q2_K down, Q8_0 shared expert",
                "q4": "Q4_K gate/up, MXFP4 down, Q8_0 shared expert"}
HBM_PEAK_GBPS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
MIN_TIMED_MS = 50.0
CKPT_Q2, CKPT_Q4 = (2560, 512, 10, 640, 640, 768), (2560, 512, 10, 640, 640, 640)
PREFILL_LABEL = "1024-token prefill chunk, N(0,1) activations, Zipf(1.1) expert popularity"

WORKLOADS = {
    "q4k_decode": dict(type=abi.GGUF_Q4_K, tokens=1, steps=2000, warmup=200, label="Q4_K experts, decode batch 1"),
    "iq2xxs_decode": dict(type=abi.GGUF_IQ2_XXS, tokens=1, steps=2000, warmup=200, label="IQ2_XXS experts, decode batch 1"),
    "q4k_verify4": dict(type=abi.GGUF_Q4_K, tokens=4, steps=1000, warmup=100,
                        label="Q4_K experts, 4-token verify batch, ~50% expert overlap"),
    "q4k_verify8": dict(type=abi.GGUF_Q4_K, tokens=8, steps=500, warmup=50,
                        label="Q4_K experts, 8-token batch of the same process (each token about half of its neighbour's experts)"),
    "q4k_verify16": dict(type=abi.GGUF_Q4_K, tokens=16, steps=250, warmup=25,
                         label="Q4_K experts, 16-token batch of the same process: the longest the decode kernels take"),
    "q4k_prefill1024": dict(type=abi.GGUF_Q4_K, tokens=1024, steps=20, warmup=5, label="Q4_K experts, " + PREFILL_LABEL),
    "q4k_prefill2048": dict(type=abi.GGUF_Q4_K, tokens=2048, steps=20, warmup=5,
                            label="Q4_K experts, " + PREFILL_LABEL.replace("1024", "2048") + " (the chunk size of the 48-layer stack)"),
    "iq2xxs_prefill1024": dict(type=abi.GGUF_IQ2_XXS, tokens=1024, steps=20, warmup=5, label="IQ2_XXS experts, " + PREFILL_LABEL),
    "iq2xxs_decode_hc": dict(type=abi.GGUF_IQ2_XXS, tokens=1, steps=2000, warmup=200, hc=4,
                             label="IQ2_XXS experts, decode batch 1, between the HC read and add of 4 residual streams"),
    "q4k_decode_hc": dict(type=abi.GGUF_Q4_K, tokens=1, steps=2000, warmup=200, hc=4,
                          label="Q4_K experts, decode batch 1, between the HC read and add of 4 residual streams"),
    "q4k_prefill1024_hc": dict(type=abi.GGUF_Q4_K, tokens=1024, steps=20, warmup=5, hc=4,
                               label="Q4_K experts, 1024-token prefill chunk, between the HC read and add of 4 residual "
                                     "streams, Zipf(1.1) expert popularity"),
    "q2profile_decode": dict(type="q2", tokens=1, steps=2000, warmup=100, label="checkpoint profile Q2, decode batch 1"),
    "q4profile_decode": dict(type="q4", tokens=1, steps=2000, warmup=100, label="checkpoint profile Q4, decode batch 1"),
    "q2profile_prefill1024": dict(type="q2", tokens=1024, steps=20, warmup=5, label="checkpoint profile Q2, " + PREFILL_LABEL),
    "q4profile_prefill1024": dict(type="q4", tokens=1024, steps=20, warmup=5, label="checkpoint profile Q4, " + PREFILL_LABEL),
    "q2ckpt_decode": dict(type="q2", tokens=1, steps=2000, warmup=100, dims=CKPT_Q2,
                          label="checkpoint profile Q2 at the checkpoints' widths, decode batch 1"),
    "q4ckpt_decode": dict(type="q4", tokens=1, steps=2000, warmup=100, dims=CKPT_Q4,
                          label="checkpoint profile Q4 at the checkpoints' widths, decode batch 1"),
    "q2ckpt_prefill1024": dict(type="q2", tokens=1024, steps=20, warmup=5, dims=CKPT_Q2,
                               label="checkpoint profile Q2 at the checkpoints' widths, " + PREFILL_LABEL),
    "q4ckpt_prefill1024": dict(type="q4", tokens=1024, steps=20, warmup=5, dims=CKPT_Q4,
                               label="checkpoint profile Q4 at the checkpoints' widths, " + PREFILL_LABEL),
    "q2ckpt_decode_hc": dict(type="q2", tokens=1, steps=2000, warmup=100, hc=4, dims=CKPT_Q2,
                             label="checkpoint profile Q2 at the checkpoints' widths, decode batch 1, between the HC read and "
                                   "add of 4 residual streams"),
    "q2ckpt_prefill1024_hc": dict(type="q2", tokens=1024, steps=20, warmup=5, hc=4, dims=CKPT_Q2,
                                  label="checkpoint profile Q2 at the checkpoints' widths, 1024-token prefill chunk, between "
                                        "the HC read and add of 4 residual streams, Zipf(1.1) expert popularity"),
    "q4k_decode_streamed": dict(type=abi.GGUF_Q4_K, tokens=1, steps=512, warmup=0, streamed=448,
                                label="Q4_K experts, decode batch 1, routed experts streamed from a file through a pool of 448 "
                                      "slots for 512 experts"),
    "iq2xxs_decode_streamed": dict(type=abi.GGUF_IQ2_XXS, tokens=1, steps=512, warmup=0, streamed=448,
                                   label="IQ2_XXS experts, decode batch 1, routed experts streamed from a file through a pool of "
                                         "448 slots for 512 experts"),
    "q4k_stack48": dict(type=abi.GGUF_Q4_K, tokens=1, steps=100, warmup=10,
                        label="48 independent Q4_K layers resident in HBM, decode batch 1 and 2048-token prefill chunks, "
                              "uniform and Zipf(1.1) expert popularity"),
}
# what the kernels compute in (every product exact; the result differs from the reference's serial f32 sums by the
# rounding of the activations and by the order of the additions; observed error <= 1e-5 against a bar of 1e-3)
DTYPE_DECODE = "i32 dot products of 24-bit block-fixed-point activations with integer weight codes, f32 scales and sums"
DTYPE_PREFILL = "f16 matrix-core products of exact-integer weight operands with two-part f16 activations, f32 accumulation"
HEADLINE = "q4k_decode"
ALL_CONFIGS = ["iq2xxs_decode", "q4k_verify4", "q4k_prefill1024", "q4k_stack48"]

DECODE_STAGES = ["pf_k_dec_router (router logits)",
                 "pf_k_dec_gate_up (routing, gate/up + SwiGLU, routed and shared)",
                 "pf_k_dec_down (down products, routed and shared, combine)"]
ROUTED_DECODE_STAGES = ["pf_k_dec_router (router logits)",
                        "pf_k_dec_route (top-k of every token, serial-order re-routes)",
                        "pf_k_dec_gate_up_given (gate/up + SwiGLU of the experts it is given, routed and shared)",
                        "pf_k_dec_down (down products, routed and shared, combine)"]
FUSED_DECODE_STAGES = ["pf_k_dec_router (router logits)",
                       "pf_k_dec_fused (routing, gate/up + SwiGLU, activation lines through memory, down products, combine)"]
GENERAL_STAGES = ["pf_k_pre (router logits, shared gate/up + SwiGLU, shared gate)",
                  "routing (top-k, serial-order re-routes)",
                  "pf_k_gate_up (routed gate/up + SwiGLU)",
                  "pf_k_down_combine (routed and shared down products, combine)"]
PREFILL_STAGES = ["pf_k_rows_to_half + pf_k_pf_router (fp16 copy of x, router logits by FP32 MFMA)",
                  "routing + grouping (top-k, serial-order re-routes, histogram/scan/stable placement)",
                  "pf_k_pf_gemm<gate_up> (grouped gate/up + SwiGLU by FP16 MFMA, then fp16 copy of the activations)",
                  "pf_k_pf_gemm<down> + pf_k_pf_combine (grouped down by FP16 MFMA, slot-ordered combine)"]
# on the checkpoint profiles the Q8_0 / Q2_K / MXFP4 items of stages 3 and 4 run in pf_k_pf_gemm_plain


class Tools:
    """picoforge_amd/libpf_bench.so (csrc/pf_bench_tools.h): graph-replay timing on top of the shipped library."""

    def __init__(self):
        path = ROOT / "picoforge_amd" / "libpf_bench.so"
        if not path.exists():
            raise pf.LibraryMissing(f"{path} is not built: run make -C picoforge_amd/csrc")
        lib = C.CDLL(str(path), mode=C.RTLD_GLOBAL)
        vp, sz, P = C.c_void_p, C.c_size_t, C.POINTER
        lib.pf_bench_last_error.restype = C.c_char_p
        lib.pf_bench_plan_moe.argtypes = [P(vp), P(vp), sz, vp, sz, vp, sz, sz, sz, C.c_int, sz, P(vp)]
        lib.pf_bench_plan_hc.argtypes = [vp, vp, vp, vp, sz, vp, vp, sz, sz, sz, C.c_int, sz, P(vp)]
        lib.pf_bench_plan_run.argtypes = [vp, sz, P(C.c_float)]
        lib.pf_bench_plan_destroy.argtypes = [vp]
        lib.pf_bench_plan_destroy.restype = None
        lib.pf_bench_hc_time_step.argtypes = [C.c_int, vp, vp, vp, vp, sz, sz, sz, sz, vp, P(C.c_float)]
        lib.pf_bench_copy_probe.argtypes = [sz, sz]
        self.lib = lib

    def check(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what}: status {rc}: {self.lib.pf_bench_last_error().decode()}")

    def plan_moe(self, moes, works, d_x, n_inputs, d_y, y_blocks, tokens, forwards, hidden, kernel_limit=0):
        n = len(moes)
        plan = C.c_void_p()
        self.check(self.lib.pf_bench_plan_moe((C.c_void_p * n)(*moes), (C.c_void_p * n)(*works), n, d_x, n_inputs, d_y,
                                              y_blocks, tokens, forwards, kernel_limit, hidden, C.byref(plan)), "plan")
        return plan

    def plan_hc(self, moe, work, d_n, d_g, n_inputs, d_r, d_i, streams, tokens, forwards, fused, hidden):
        plan = C.c_void_p()
        self.check(self.lib.pf_bench_plan_hc(moe, work, d_n, d_g, n_inputs, d_r, d_i, streams, tokens, forwards, fused, hidden,
                                             C.byref(plan)), "hc plan")
        return plan

    def run(self, plan, repeats):
        ms = (C.c_float * repeats)()
        self.check(self.lib.pf_bench_plan_run(plan, repeats, ms), "plan run")
        return np.array(ms[:], dtype=np.float64)

    def destroy(self, plan):
        self.lib.pf_bench_plan_destroy(plan)

    def timed(self, plan, forwards, warmup):
        """Warm-up replays (at least `warmup` forwards), then replays until MIN_TIMED_MS are timed (at least 5).
        Returns ms per forward: median, p10, p90, the number of timed replays and the total timed ms."""
        self.run(plan, max(1, math.ceil(warmup / forwards)))
        first = self.run(plan, 3)
        est = max(float(np.median(first)), 1e-4)
        repeats = int(min(5000, max(5, math.ceil(MIN_TIMED_MS / est))))
        ms = self.run(plan, repeats)
        per = ms / forwards
        return {"median": float(np.median(per)), "p10": float(np.percentile(per, 10)), "p90": float(np.percentile(per, 90)),
                "replays": repeats, "timed_ms": float(ms.sum())}


def sources_digest():
    """Digest of the kernel sources: a traffic figure from a profile is only quoted for the kernels it was taken on."""
    h = hashlib.sha256()
    for path in sorted((ROOT / "picoforge_amd" / "csrc").glob("*.h*")):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    return h.hexdigest()[:12]


def measured_traffic(workload):
    """HBM bytes per launch of the workload's dominant kernel from profiles/traffic.json (rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE, scaled by the same counters on a plain copy of known size).  A counter cannot be
    read live, so the figure is quoted only while the kernel sources are the ones it was measured on."""
    path = ROOT / "profiles" / "traffic.json"
    if not path.exists():
        return None, None
    entry = json.loads(path.read_text()).get(workload)
    if not entry or WORKLOADS.get(workload, {}).get("custom_shape"):   # --dims: the table holds the workload's own shape
        return None, None
    source = {"profile": entry.get("profile"), "sources": entry.get("sources"), "kernel": entry.get("kernel")}
    if entry.get("sources") != sources_digest():
        return None, dict(source, stale=True)
    return entry["bytes"], source


def cpu_api_and_kind():
    ref = load_reference()
    return (ref, "reference") if ref is not None else (load_oracle(), "port")


def layer_config(wl):
    if wl.get("dims"):
        h, e, k, i, s_i, phys = wl["dims"]
        return abi.moe_config(h, e, k, i, s_i, down_physical=phys)
    return workloads.measured_config()


def unfiltered_decode(args, ctx, weights, layer, n_inputs, steps, warmup, filtered_us):
    """The one-token workload without the margin filter.  A token whose closest pair among the top-(k+1) router logits is
    nearer than the rounding noise of a parallel sum is routed again in the reference's serial order (by every workgroup
    of the token's launch).  Three figures: the drawn tokens as they come; a stream of such tokens only; and the mean
    the two imply at the share of such tokens among seeded tokens."""
    api, hip, tools = ctx
    cfg = weights.cfg
    moe, work = layer.device_handles()
    h = cfg.hidden_size
    d_y = hip.to_device(np.zeros((1, h), dtype=np.float32))

    def timed(x):
        d_x = hip.to_device(x.reshape(len(x), 1, h))
        hip.work_clear_status(work)
        plan = tools.plan_moe([moe], [work], d_x, len(x), d_y, 1, 1, len(x), h)
        tools.run(plan, 1)                       # one pass over the inputs: how many of them are routed again
        count = C.c_uint32()
        hip.work_exact_rows(work, C.byref(count))
        tools.destroy(plan)
        plan = tools.plan_moe([moe], [work], d_x, len(x), d_y, 1, 1, steps, h)
        t = tools.timed(plan, steps, warmup)
        tools.destroy(plan)
        hip.free(d_x)
        return t["median"] * 1e3, int(count.value)

    x_all, _ = workloads.decode_tokens(weights, n_inputs, seed=args.seed + 7, min_margin=0.0)
    all_us, all_flagged = timed(x_all)
    n_close = min(n_inputs, 16)
    x_close, info = workloads.decode_tokens(weights, n_close, seed=args.seed + 8, min_margin=0.0, max_margin=2e-5)
    close_us, close_flagged = timed(x_close)
    hip.work_clear_status(work)
    hip.free(d_y)
    share = info["kept_fraction"] * close_flagged / max(1, n_close)
    return {"as_drawn": {"value": round(all_us, 3), "inputs": int(len(x_all)), "routed_again": all_flagged},
            "close_tokens_only": {"value": round(close_us, 3), "inputs": n_close, "routed_again": close_flagged,
                                  "selection": "top-11 margin below 2e-5", "share_of_drawn_tokens": round(info["kept_fraction"], 5)},
            "expected_mean": {"value": round((1.0 - share) * filtered_us + share * close_us, 3), "share_routed_again": round(share, 5)},
            "unit": "us/layer/token"}


def run_layer(args, ctx, name, steps, warmup, cpu_seconds):
    """One MoE layer: decode batches or prefill chunks.  Returns the record."""
    api, hip, tools = ctx
    wl = WORKLOADS[name]
    cfg = layer_config(wl)
    tokens = wl["tokens"]
    chunk_inputs = tokens > 16          # a chunk under the Zipf router; shorter batches are correlated tokens
    t0 = time.time()
    weights = pf.LayerWeights.synthetic(cfg, wl["type"], seed=args.seed)
    if chunk_inputs:
        # Zipf(1.1) popularity profile, flattened (logit bias -1.1 * 0.18 * ln rank) so that the busiest
        # expert receives about 150 of the 1024 tokens, as the configuration states
        workloads.zipf_router(weights, seed=args.seed, temperature=0.18)
        n_inputs = max(1, min(steps, 4))
        x = np.stack([workloads.prefill_chunk(weights, tokens, seed=args.seed + b) for b in range(n_inputs)])
        load = workloads.expert_load(weights, x[0])
        unique = float(np.count_nonzero(load))
        info = {"active_experts_chunk0": int(unique), "max_tokens_per_expert": int(load.max()),
                "median_tokens_per_expert": float(np.median(load)), "chunks": n_inputs}
    elif tokens == 1:
        n_inputs = max(1, min(steps, 64))       # a plan replays one graph of 64 forwards: 64 inputs = 1.5 GB of weights touched, far beyond the caches
        x, info = workloads.decode_tokens(weights, n_inputs, seed=args.seed, min_margin=args.margin_window[0],
                                          max_margin=args.margin_window[1])
        x = x.reshape(n_inputs, 1, cfg.hidden_size)
        unique = float(cfg.top_k)
    else:
        n_inputs = max(1, min(steps, 64))
        x, info = workloads.verify_batches(weights, n_inputs, seed=args.seed, group=tokens)
        unique = info["mean_unique_experts"]
    prep_s = time.time() - t0

    layer = pf.MoeLayer(api, cfg, weights, tokens)
    moe, work = layer.device_handles()     # the layer's HBM-resident tensors and scratch, for the timed loop
    h = cfg.hidden_size
    d_x = hip.to_device(x)
    d_y = hip.to_device(np.zeros((tokens, h), dtype=np.float32))

    wall0 = time.perf_counter()
    plan = tools.plan_moe([moe], [work], d_x, n_inputs, d_y, 1, tokens, steps, h)
    timing = tools.timed(plan, steps, warmup)
    tools.destroy(plan)
    wall_ms = (time.perf_counter() - wall0) * 1e3
    ms_per_step = timing["median"]
    us_per_token = ms_per_step * 1e3 / tokens
    err_word = hip.from_device(hip.work_error_word(work), (1,), np.uint32)[0]
    exact, exact_full = C.c_uint32(), C.c_uint32()
    hip.work_exact_rows(work, C.byref(exact))
    hip.work_full_reroutes(work, C.byref(exact_full))

    # Per-kernel durations inside the dependent chain: the same plan with only the first 1, 2, ... kernel
    # groups of every forward; a group's duration is the difference between consecutive plans (it includes
    # the dispatch gap before it, as a profiler's start-to-end time of a dependent kernel does).
    family = hip.moe_kernel_family(moe, work, tokens)
    prefill = family == 2 or (family == 0 and chunk_inputs)   # accounted as a chunk: bytes of the grouped products, tokens per second
    names = {0: GENERAL_STAGES, 1: DECODE_STAGES, 2: PREFILL_STAGES}[family]
    if family == 1 and hip.moe_decode_launches(moe, work, tokens) == 2:
        names = FUSED_DECODE_STAGES
    if family == 1 and hip.moe_decode_launches(moe, work, tokens) == 4:
        names = ROUTED_DECODE_STAGES
    stage_us = [1e-3] * len(names)
    if not args.skip_stages:
        previous = 0.0
        n_fw = min(steps, 512)
        for j in range(len(names)):
            if j + 1 < len(names):
                plan = tools.plan_moe([moe], [work], d_x, n_inputs, d_y, 1, tokens, n_fw, h, kernel_limit=j + 1)
                t = tools.timed(plan, n_fw, min(warmup, n_fw))["median"]
                tools.destroy(plan)
            else:
                t = ms_per_step
            stage_us[j] = max((t - previous) * 1e3, 1e-3)
            previous = t

    lb = workloads.layer_bytes(wl["type"], cfg)
    i, s_i, k = cfg.intermediate, cfg.shared_intermediate, cfg.top_k
    extra = {}
    if tokens == 1 and args.margin_window == (1e-3, None) and name in ("q4k_decode", "iq2xxs_decode") and not wl.get("custom_shape") \
            and not under_tracer():   # a profiled run keeps to the plans it is there to look at
        extra["unfiltered_inputs"] = unfiltered_decode(args, ctx, weights, layer, n_inputs, steps, warmup, us_per_token)
    if prefill:
        # algorithmic bytes per launch: weights of the active experts once, activations once
        pairs = tokens * k
        stage_bytes = [tokens * h * 4 + (cfg.experts + 1) * h * 4 + tokens * h * 2,
                       tokens * cfg.experts * 4 + pairs * 16,
                       unique * lb["gate_up"] + lb["shared_gate_up"] + (pairs + tokens) * h * 2
                       + (pairs * i + tokens * s_i) * 4,
                       unique * lb["down"] + lb["shared_down"] + (pairs * i + tokens * s_i) * 2
                       + (pairs + tokens) * h * 4 + tokens * h * 4]
        alg_bytes = unique * (lb["gate_up"] + lb["down"]) + lb["shared_gate_up"] + lb["shared_down"] + lb["routers"] \
            + 2 * tokens * h * 4
        stage_flops = [2.0 * tokens * h * (cfg.experts + 1), 0.0, 2.0 * tokens * (k * 2 * h * i + 2 * h * s_i),
                       2.0 * tokens * (k * i * h + s_i * h)]
        flops = sum(stage_flops)
        extra = {"prefill_tokens_per_s": round(tokens / (ms_per_step * 1e-3), 1),
                 "flops_per_step": flops,
                 "mfma_frac_of_fp16_dense_peak": round(flops / (ms_per_step * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                 "stage_tflops": {names[j].split()[0]: round(stage_flops[j] / (stage_us[j] * 1e-6) / 1e12, 1)
                                  for j in (0, 2, 3)},
                 "binding_roofline": "hbm: about 80 flop per weight byte at this chunk size, below the MFMA ridge"}
    else:
        alg_bytes = workloads.algorithmic_bytes_per_token(wl["type"], unique_experts=unique, cfg=cfg)
        stage_bytes = [lb["routers"], unique * lb["gate_up"] + lb["shared_gate_up"],
                       unique * lb["down"] + lb["shared_down"]]
        if len(names) == 2:
            stage_bytes = [stage_bytes[0], stage_bytes[1] + stage_bytes[2]]
        if family == 1 and len(names) == 4:   # the routing launch reads the tokens' logits and their noise terms
            stage_bytes = [stage_bytes[0], tokens * cfg.experts * 8, stage_bytes[1], stage_bytes[2]]
        if family == 0:
            stage_bytes = [lb["routers"] + lb["shared_gate_up"], tokens * cfg.experts * 8, unique * lb["gate_up"],
                           unique * lb["down"] + lb["shared_down"]]
    dom = int(np.argmax(stage_bytes))
    achieved = stage_bytes[dom] / (stage_us[dom] * 1e-6) / 1e9

    # CPU baseline and parity on a bounded sample of the same inputs
    cpu_api, kind = cpu_api_and_kind()
    per_token_guess = 0.27 if wl["type"] in (abi.GGUF_IQ2_XXS, "q2") else 0.14
    if prefill:
        sample_tokens = min(tokens, args.cpu_sample or max(4, int(cpu_seconds / per_token_guess)))
        with pf.MoeLayer(cpu_api, cfg, weights, sample_tokens) as cpu:
            c0 = time.perf_counter()
            cpu_out = [cpu.forward(x[0][:sample_tokens])[1:]]
            cpu_s = time.perf_counter() - c0
        _, y, ids, w = layer.forward(x[0])
        gpu_out = [(y[:sample_tokens], ids[:sample_tokens], w[:sample_tokens])]
        sample_text = f"first {sample_tokens} tokens of chunk 0 (the CPU cost is linear in tokens), {cpu_s:.1f} s"
    else:
        sample = args.cpu_sample or max(1, int(cpu_seconds / per_token_guess / tokens))
        sample = min(sample, n_inputs)
        sample_tokens = sample * tokens
        with pf.MoeLayer(cpu_api, cfg, weights, tokens) as cpu:
            c0 = time.perf_counter()
            cpu_out = [cpu.forward(x[b].reshape(tokens, -1))[1:] for b in range(sample)]
            cpu_s = time.perf_counter() - c0
        gpu_out = [layer.forward(x[b].reshape(tokens, -1))[1:] for b in range(sample)]
        sample_text = f"first {sample} steps ({sample_tokens} tokens) of the same inputs, {cpu_s:.1f} s"
    ids_equal = all((g[1] == c[1]).all() for g, c in zip(gpu_out, cpu_out))
    max_abs = max(float(np.abs(g[0] - c[0]).max()) for g, c in zip(gpu_out, cpu_out))
    within = all((np.abs(g[0] - c[0]) <= 1e-3 + 1e-4 * np.abs(c[0])).all() for g, c in zip(gpu_out, cpu_out))
    layer.close()
    hip.free(d_x)
    hip.free(d_y)
    if args.copy_probe:
        tools.check(tools.lib.pf_bench_copy_probe(args.copy_probe << 20, 3), "copy probe")

    traffic, traffic_from = measured_traffic(name)
    margins = "; top-11 logit margins >= 1e-3" if not prefill else ""
    if tokens == 1 and args.margin_window != (1e-3, None):
        lo, hi = args.margin_window
        margins = f"; top-11 logit margins in [{lo:g}, {'inf' if hi is None else format(hi, 'g')})"
    whole = alg_bytes / (ms_per_step * 1e-3) / 1e9
    return {
        "metric": "moe_decode_us_per_layer_token" if not prefill else "moe_prefill_us_per_layer_token",
        "value": round(us_per_token, 3),
        "unit": "us/layer/token",
        "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 6),
        "ms_per_step_p10_p90": [round(timing["p10"], 6), round(timing["p90"], 6)],
        "timed_replays": timing["replays"], "timed_ms": round(timing["timed_ms"], 2),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": DTYPE_DECODE if not prefill else DTYPE_PREFILL,
        "data": "synthetic",
        "config": {"workload": f"one MoE layer, hidden {cfg.hidden_size}, {cfg.experts} experts, top-{cfg.top_k}, "
                               f"intermediate {cfg.intermediate}, shared {cfg.shared_intermediate}; "
                               f"{wl['label']}; {n_inputs} seeded inputs{margins}"
                               + ("; the inputs are cycled (drawn like the configuration's 10 000 tokens)" if tokens == 1 else ""),
                   "tokens_per_step": tokens, "expert_format": FORMAT_LABEL[wl["type"]],
                   "unique_experts_per_step": unique, "inputs": info},
        "hbm_GBps_on_algorithmic_bytes": round(whole, 1),
        "hbm_frac_whole_layer": round(whole / HBM_PEAK_GBPS, 4),
        "algorithmic_bytes_per_step": int(alg_bytes),
        "tokens_per_s": round(tokens / (ms_per_step * 1e-3), 1),
        "roofline": {"bound": "hbm", "kernel": names[dom], "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_from": traffic_from,
                     "bytes_per_launch": int(stage_bytes[dom]), "us_per_launch": round(stage_us[dom], 3)},
        "kernel_us": dict(zip(names, [round(v, 3) for v in stage_us])),
        "kernel_bytes": dict(zip(names, [int(b) for b in stage_bytes])),
        **extra,
        "cpu_baseline": {"value": round(cpu_s / sample_tokens * 1e6, 1), "unit": "us/layer/token", "cores": 1,
                         "kind": kind, "sample": sample_text},
        "parity_on_sample": {"ids_equal": bool(ids_equal), "within_1e-3_abs_1e-4_rel": bool(within),
                             "max_abs_err": max_abs, "error_word": int(err_word), "serial_order_reroutes": int(exact.value),
                             "of_those_all_logits_serially": int(exact_full.value)},
        "wall_ms_timed_loop": round(wall_ms, 2), "prep_s": round(prep_s, 1),
    }


def run_stack(args, ctx, steps, warmup, cpu_seconds):
    """A stack of independent layers, all resident: every token (or chunk) passes the layers in order, each
    layer with its own seeded input, hence its own routing.  The popularity bias sits in router column 0
    (workloads.zipf_router): inputs with coordinate 0 = 1 see Zipf(1.1) popularity, with 0 the plain router."""
    api, hip, tools = ctx
    cfg = workloads.measured_config()
    layers_n, chunk = args.layers, 2048
    t0 = time.time()
    layers, sample = [], None
    for l in range(layers_n):
        weights = pf.LayerWeights.synthetic(cfg, abi.GGUF_Q4_K, seed=args.seed * 1000 + l)
        workloads.zipf_router(weights, seed=args.seed * 1000 + l, temperature=0.18)
        layers.append(pf.MoeLayer(api, cfg, weights, chunk))
        if l == 0:
            sample = weights
        else:
            layers[-1].weights = None      # the library copied the bytes into HBM at create
    prep_s = time.time() - t0
    moes = [l.device_handles()[0] for l in layers]
    works = [l.device_handles()[1] for l in layers]
    resident = sum(hip.moe_bytes(m) for m in moes)
    synth = pf.Synth()
    h = cfg.hidden_size
    per_layer_tokens = 8
    dec = pf.rms_normalise(synth.normal((per_layer_tokens * layers_n, h), 77 + args.seed))
    pre = synth.normal((4 * chunk, h), 78 + args.seed)
    d_y = hip.to_device(np.zeros((chunk, h), dtype=np.float32))
    out, spread = {}, {}
    for name, coord in (("uniform", 0.0), ("zipf", 1.0)):
        dec[:, 0] = coord
        pre[:, 0] = coord
        d_dec, d_pre = hip.to_device(dec), hip.to_device(pre)
        plan = tools.plan_moe(moes, works, d_dec, len(dec), d_y, 1, 1, steps * layers_n, h)
        t = tools.timed(plan, steps, warmup)        # per token through the stack
        tools.destroy(plan)
        out[name + "_decode_us_per_token"] = t["median"] * 1e3
        spread[name + "_decode_us_p10_p90"] = [round(t["p10"] * 1e3, 2), round(t["p90"] * 1e3, 2)]
        chunks = 2
        plan = tools.plan_moe(moes, works, d_pre, 4, d_y, 1, chunk, chunks * layers_n, h)
        t = tools.timed(plan, chunks, 1)
        tools.destroy(plan)
        out[name + "_prefill_ms_per_chunk"] = t["median"]
        out[name + "_prefill_tokens_per_s"] = chunk / (t["median"] * 1e-3)
        hip.free(d_dec)
        hip.free(d_pre)
    errors = sum(int(hip.from_device(hip.work_error_word(w), (1,), np.uint32)[0]) for w in works)
    # parity and the CPU cost per layer-token on layer 0; the stack's CPU time is that times the layers
    cpu_api, kind = cpu_api_and_kind()
    n = args.cpu_sample or max(2, int(cpu_seconds / 0.14))
    xs = dec[:n].copy()
    with pf.MoeLayer(cpu_api, cfg, sample, n) as cpu:
        c0 = time.perf_counter()
        _, y0, ids0, _ = cpu.forward(xs)
        cpu_s = time.perf_counter() - c0
    _, y1, ids1, _ = layers[0].forward(xs)
    ids_equal = bool((ids0 == ids1).all())
    within = bool((np.abs(y1 - y0) <= 1e-3 + 1e-4 * np.abs(y0)).all())
    for l in layers:
        l.close()
    hip.free(d_y)
    if args.copy_probe:
        tools.check(tools.lib.pf_bench_copy_probe(args.copy_probe << 20, 3), "copy probe")
    us = out["uniform_decode_us_per_token"]
    alg = layers_n * workloads.algorithmic_bytes_per_token(abi.GGUF_Q4_K)
    per_layer, traffic_from = measured_traffic("q4k_stack48")   # the three decode kernels of one layer of a stack, cold caches
    return {
        "metric": "moe_stack_decode_us_per_token", "value": round(us, 2), "unit": "us/token (all layers)",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(us * 1e-3, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": DTYPE_DECODE, "data": "synthetic",
        "config": {"workload": f"{layers_n} independent MoE layers (hidden 2048, 512 experts, top-10, intermediate 512, "
                               f"shared 512, Q4_K), {resident / 1e9:.1f} GB resident in HBM; decode batch 1 and "
                               f"{chunk}-token prefill chunks; per-layer seeded inputs and routers",
                   "layers": layers_n, "tokens_per_step": 1},
        "us_per_layer_token": round(us / layers_n, 3),
        "hbm_GBps_on_algorithmic_bytes": round(alg / (us * 1e-6) / 1e9, 1),
        "algorithmic_bytes_per_step": int(alg),
        "roofline": {"bound": "hbm", "kernel": "whole stack: three decode kernels per layer", "achieved":
                     round(alg / (us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(alg / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                     "traffic": None if per_layer is None else int(per_layer) * layers_n, "traffic_from": traffic_from},
        "stack": {k: round(v, 3) for k, v in out.items()}, "stack_spread": spread,
        "cpu_baseline": {"value": round(cpu_s / n * 1e6 * layers_n, 1), "unit": "us/token (all layers)", "cores": 1,
                         "kind": kind, "sample": f"{n} tokens through layer 0 ({cpu_s:.1f} s), times {layers_n} layers: "
                                                 "an extrapolation, the CPU cost is linear in layers and tokens"},
        "parity_on_sample": {"ids_equal": ids_equal, "within_1e-3_abs_1e-4_rel": within, "error_word": errors},
        "prep_s": round(prep_s, 1),
    }


def run_hc(args, ctx, name, steps, warmup, cpu_seconds):
    """One layer between its two hyper-connection steps (src/qwen4_forward.c:362-367): per step a gated read
    of [tokens, streams, hidden] normed streams and gate logits, the MoE block, and the injection of the
    block's output into the [tokens, streams, hidden] residual.  Timed three ways on resident buffers: the
    chain with the injection folded into the block's last kernel (`value`), the chain with the injection as
    a kernel of its own, and the block alone on the same mixed rows."""
    api, hip, tools = ctx
    wl = WORKLOADS[name]
    cfg = layer_config(wl)
    tokens, streams, h = wl["tokens"], wl["hc"], cfg.hidden_size
    t0 = time.time()
    weights = pf.LayerWeights.synthetic(cfg, wl["type"], seed=args.seed)
    if tokens > 4:
        workloads.zipf_router(weights, seed=args.seed, temperature=0.18)
    n_inputs = max(1, min(steps, 4 if tokens > 4 else 64))
    rng = np.random.default_rng(args.seed)
    # streams whose gated mix has about unit RMS, as the block sees after the norm
    normed = (rng.standard_normal((n_inputs, tokens, streams, h)) * (2.0 * streams ** 0.5 / 1.12)).astype(np.float32)
    logits = rng.standard_normal((n_inputs, tokens, streams, h)).astype(np.float32)
    residual = rng.standard_normal((tokens, streams, h)).astype(np.float32)
    inject = rng.uniform(0.0, 2.0 / streams, (tokens, streams)).astype(np.float32)
    # the timed loop adds into one residual many thousands of times: weights scaled down so that it stays small
    inject_timed = inject * np.float32(1e-4)
    prep_s = time.time() - t0
    layer = pf.MoeLayer(api, cfg, weights, tokens)
    moe, work = layer.device_handles()
    d_n, d_g, d_i = hip.to_device(normed), hip.to_device(logits), hip.to_device(inject_timed)
    d_r = hip.to_device(residual)
    timed = {}
    for label, fused in (("fused", 1), ("separate_add", 0)):
        hip.check(hip.memcpy_h2d(d_r, residual.ctypes.data, residual.nbytes), "residual")
        plan = tools.plan_hc(moe, work, d_n, d_g, n_inputs, d_r, d_i, streams, tokens, steps, fused, h)
        timed[label] = tools.timed(plan, steps, warmup)
        tools.destroy(plan)
    err_word = int(hip.from_device(hip.work_error_word(work), (1,), np.uint32)[0])
    # the block alone on the mixed rows the read produces
    shape = abi.Qwen4HcShape(streams, h, 1, 1e-6)
    mixed = np.empty((n_inputs, tokens, h), dtype=np.float32)
    for b in range(n_inputs):
        st = api.hc.read(C.byref(shape), abi.f32_cube(normed[b]), abi.f32_cube(logits[b]), abi.f32_view(mixed[b]), None)
        assert st == abi.QW4_OK, st
    d_x = hip.to_device(mixed)
    d_y = hip.to_device(np.zeros((tokens, h), dtype=np.float32))
    plan = tools.plan_moe([moe], [work], d_x, n_inputs, d_y, 1, tokens, steps, h)
    block_ms = tools.timed(plan, steps, warmup)["median"]
    tools.destroy(plan)

    # the two hyper-connection kernels alone, HIP events on the launch stream around back-to-back launches
    # (the add runs with zero weights so that the residual stays put over the launches)
    d_zero = hip.to_device(np.zeros_like(inject))
    d_err = hip.to_device(np.zeros(64, dtype=np.uint32))
    kernel_us = {}
    n_launch = max(50, min(steps, 1000))
    ms = C.c_float()
    for which, kname in ((0, "pf_k_hc_read"), (1, "pf_k_hc_add")):
        for count in (10, n_launch):
            tools.check(tools.lib.pf_bench_hc_time_step(which, d_n if which == 0 else d_r, d_g, d_x if which == 0 else d_y,
                                                        d_zero, tokens, streams, h, count, d_err, C.byref(ms)), kname)
        kernel_us[kname] = ms.value * 1e3 / n_launch
    read_bytes = tokens * h * 4 * (2 * streams + 1)
    add_bytes = tokens * h * 4 * (2 * streams + 1) + tokens * streams * 4
    if args.copy_probe:
        tools.check(tools.lib.pf_bench_copy_probe(args.copy_probe << 20, 3), "copy probe")

    # parity on a bounded sample, stage by stage on identical inputs: CPU read against the device's mixed rows,
    # CPU block on those rows, CPU add of its output; the device's chained call against that residual
    cpu_api, kind = cpu_api_and_kind()
    per_token = 0.27 if wl["type"] in (abi.GGUF_IQ2_XXS, "q2") else 0.14
    sample = min(tokens, args.cpu_sample or max(2, int(cpu_seconds / per_token / 2)))
    steps_cpu = 1 if tokens > 1 else min(sample, n_inputs)
    rows = sample if tokens > 1 else 1
    ids_equal = within = read_close = True
    max_abs = 0.0
    cpu_s = 0.0
    with pf.MoeLayer(cpu_api, cfg, weights, rows) as cpu:
        for b in range(steps_cpu):
            n_b, g_b = normed[b][:rows], logits[b][:rows]
            want = residual[:rows].copy()
            c0 = time.perf_counter()
            _, ids_c, _ = cpu.forward_hc(n_b, g_b, want, inject[:rows], fused=False)
            cpu_s += time.perf_counter() - c0
            # the same chain with the CPU block fed the device's mixed rows (identical inputs to every stage)
            _, y_c, ids_m, _ = cpu.forward(mixed[b][:rows])
            want_m = residual[:rows].copy()
            cpu_api.hc.add(C.byref(shape), abi.f32_cube(want_m), abi.f32_view(y_c), abi.f32_view(inject[:rows]), None)
            got = residual.copy()
            _, ids_g, _ = layer.forward_hc(normed[b], logits[b], got, inject)
            ids_equal &= bool((ids_g[:rows] == ids_m).all())
            bound = np.abs(inject[:rows])[:, :, None] * (1e-3 + 1e-4 * np.abs(y_c)[:, None, :]) + 1e-6 * np.abs(want_m)
            within &= bool((np.abs(got[:rows] - want_m) <= bound).all())
            max_abs = max(max_abs, float(np.abs(got[:rows] - want_m).max()))
            read_close &= bool(np.allclose(want, want_m, atol=1e-5, rtol=1e-5))
    layer.close()
    sample_tokens = steps_cpu * rows
    ms_per_step = timed["fused"]["median"]
    hc_bytes = tokens * h * 4 * (2 * streams + 1) + tokens * h * 4 * 2 * streams   # read in/out, residual in/out
    traffic, traffic_from = measured_traffic(name)
    return {
        "metric": "moe_hc_block_us_per_layer_token", "value": round(ms_per_step * 1e3 / tokens, 3),
        "unit": "us/layer/token", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 6),
        "ms_per_step_p10_p90": [round(timed["fused"]["p10"], 6), round(timed["fused"]["p90"], 6)],
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if tokens <= 4 else "f16 products, f32 accumulation", "data": "synthetic",
        "config": {"workload": f"one MoE layer, hidden {cfg.hidden_size}, {cfg.experts} experts, top-{cfg.top_k}, "
                               f"intermediate {cfg.intermediate}, shared {cfg.shared_intermediate}; "
                               f"{wl['label']}; {n_inputs} seeded inputs",
                   "tokens_per_step": tokens, "streams": streams,
                   "expert_format": FORMAT_LABEL[wl["type"]]},
        "chain_us_per_step": {"read + block with the add folded in": round(timed["fused"]["median"] * 1e3, 3),
                              "read + block + add kernel": round(timed["separate_add"]["median"] * 1e3, 3),
                              "block alone": round(block_ms * 1e3, 3)},
        "hc_bytes_per_step": int(hc_bytes),
        "kernel_us": {k: round(v, 3) for k, v in kernel_us.items()},
        "kernel_bytes": {"pf_k_hc_read": int(read_bytes), "pf_k_hc_add": int(add_bytes)},
        "kernel_GBps": {"pf_k_hc_read": round(read_bytes / (kernel_us["pf_k_hc_read"] * 1e-6) / 1e9, 1),
                        "pf_k_hc_add": round(add_bytes / (kernel_us["pf_k_hc_add"] * 1e-6) / 1e9, 1)},
        "roofline": {"bound": "hbm", "kernel": "pf_k_hc_read (gated mix of the residual streams)",
                     "achieved": round(read_bytes / (kernel_us["pf_k_hc_read"] * 1e-6) / 1e9, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(read_bytes / (kernel_us["pf_k_hc_read"] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_from": traffic_from, "bytes_per_launch": int(read_bytes),
                     "us_per_launch": round(kernel_us["pf_k_hc_read"], 3)},
        "cpu_baseline": {"value": round(cpu_s / sample_tokens * 1e6, 1), "unit": "us/layer/token", "cores": 1,
                         "kind": kind, "sample": f"{sample_tokens} tokens of the same inputs through read, block and add, "
                                                 f"{cpu_s:.1f} s"},
        "parity_on_sample": {"ids_equal": ids_equal, "residual_within_block_tolerance_times_inject": within,
                             "cpu_read_vs_device_read_chain_close": read_close, "max_abs_err": max_abs,
                             "error_word": err_word},
        "prep_s": round(prep_s, 1),
    }


def run_streamed(args, ctx, name, steps, cpu_seconds):
    """A layer whose routed experts stay in a file (here: in the page cache of a file written just before) and reach the
    GPU through an expert pool with fewer slots than experts: per token the router and the routing (first device call),
    the pool's acquire (misses are read by the pool's reader threads and stored in the device layout), the expert kernels
    on the pool's slots (second device call), the release.  Wall time of the host call per token over a seeded token
    stream, after one pass that fills the pool; the same with a slot for every expert (no misses) beside it."""
    import tempfile
    api, hip, tools = ctx
    wl = WORKLOADS[name]
    cfg = workloads.measured_config()
    weights = pf.LayerWeights.synthetic(cfg, wl["type"], seed=args.seed)
    x, info = workloads.decode_tokens(weights, steps, seed=args.seed, min_margin=0.0)
    sizes = [weights.raw[j].size // cfg.experts for j in (1, 2, 3)]
    folder = tempfile.mkdtemp(prefix="pf_bench_")
    path = os.path.join(folder, "experts.bin")
    offsets, at = [], 4096
    with open(path, "wb") as f:
        f.write(bytes(4096))
        for j in (1, 2, 3):
            offsets.append(at)
            weights.raw[j].tofile(f)
            at += weights.raw[j].size
    fd = os.open(path, os.O_RDONLY)
    table = (abi.QW4ExpertLayer * 1)(abi.QW4ExpertLayer((C.c_uint64 * 3)(*offsets)))
    h, i = cfg.hidden_size, cfg.intermediate
    err, handle = abi.Qwen4Error(), C.c_void_p()
    struct = weights.without_routed_bytes()
    assert api.create_streamed(C.byref(cfg), C.byref(struct), C.byref(handle), C.byref(err)) == abi.QW4_OK, err.detail
    cpu_api, kind = cpu_api_and_kind()
    sample = args.cpu_sample or max(1, int(cpu_seconds / 0.14))
    with pf.MoeLayer(cpu_api, cfg, weights, 1) as cpu:
        c0 = time.perf_counter()
        want = [cpu.forward(x[b:b + 1])[1:] for b in range(sample)]
        cpu_s = time.perf_counter() - c0
    results, parity = {}, None
    with pf.MoeLayer(api, cfg, weights, 16, handle=handle) as layer:
        for slots in (wl["streamed"], cfg.experts):
            pool = api.pool_create(fd, table, 1, cfg.experts, (C.c_size_t * 3)(*sizes), slots)
            assert pool and api.pool_set_formats(pool, (C.c_uint32 * 3)(*weights.types[1:4]), (C.c_size_t * 3)(h, h, cfg.down_physical),
                                                 (C.c_size_t * 3)(i, i, h)) == 0
            y = np.zeros((1, h), np.float32)
            ids = np.zeros((1, cfg.top_k), np.uint32)
            w = np.zeros((1, cfg.top_k), np.float32)
            routes = abi.Qwen4MoeRoutes(abi.u32_view(ids), abi.f32_view(w))

            def forward(row):
                st = api.forward_streamed(layer.handle, pool, 0, abi.f32_view(row), abi.f32_view(y), C.byref(routes), layer.work,
                                          C.byref(layer.err))
                assert st == abi.QW4_OK, layer.err.detail

            for b in range(steps):                      # fills the pool
                forward(np.ascontiguousarray(x[b:b + 1]))
            before = api.pool_stats(pool)
            t0 = time.perf_counter()
            for b in range(steps):
                forward(np.ascontiguousarray(x[b:b + 1]))
            wall = time.perf_counter() - t0
            after = api.pool_stats(pool)
            misses = after.misses - before.misses
            results[slots] = {"us_per_token": round(wall / steps * 1e6, 1), "misses_per_token": round(misses / steps, 3),
                              "miss_rate_per_routed_expert": round(misses / (steps * cfg.top_k), 4),
                              "MB_read_per_token": round((after.bytes_read - before.bytes_read) / steps / 1e6, 3),
                              "acquire_us_per_token": round((after.acquire_ns - before.acquire_ns) / steps / 1e3, 1)}
            if parity is None:
                got = []
                for b in range(sample):
                    forward(np.ascontiguousarray(x[b:b + 1]))
                    got.append((y.copy(), ids.copy(), w.copy()))
                parity = {"ids_equal": bool(all((g[1] == c[1]).all() for g, c in zip(got, want))),
                          "within_1e-3_abs_1e-4_rel": bool(all((np.abs(g[0] - c[0]) <= 1e-3 + 1e-4 * np.abs(c[0])).all()
                                                               for g, c in zip(got, want))),
                          "max_abs_err": max(float(np.abs(g[0] - c[0]).max()) for g, c in zip(got, want)), "error_word": 0}
            api.pool_destroy(pool)
    os.close(fd)
    os.unlink(path)
    os.rmdir(folder)
    main = results[wl["streamed"]]
    per_miss = (main["us_per_token"] - results[cfg.experts]["us_per_token"]) / max(main["misses_per_token"], 1e-9)
    return {
        "metric": "moe_decode_us_per_layer_token", "value": main["us_per_token"], "unit": "us/layer/token (host call, wall clock)",
        "n_gpus": 1, "steps": steps, "warmup": steps, "ms_per_step": round(main["us_per_token"] * 1e-3, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": DTYPE_DECODE, "data": "synthetic",
        "config": {"workload": f"one MoE layer, hidden {cfg.hidden_size}, {cfg.experts} experts, top-{cfg.top_k}, intermediate "
                               f"{cfg.intermediate}, shared {cfg.shared_intermediate}; {wl['label']}; {steps} seeded tokens, each "
                               "routed to its own experts; the file is in the page cache (written just before)",
                   "tokens_per_step": 1, "expert_format": FORMAT_LABEL[wl["type"]], "pool_slots": wl["streamed"],
                   "readers": 8, "inputs": info},
        "pool": {str(k): v for k, v in results.items()},
        "us_per_missed_expert": round(per_miss, 1),
        "GBps_of_missed_experts": round(sum(sizes) / max(per_miss, 1e-9) / 1e3, 2),
        "roofline": {"bound": "hbm", "kernel": "not a kernel figure: the misses are bound by the file reads and the copies to the GPU",
                     "achieved": None, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": None, "traffic": None},
        "cpu_baseline": {"value": round(cpu_s / sample * 1e6, 1), "unit": "us/layer/token", "cores": 1, "kind": kind,
                         "sample": f"first {sample} tokens, every expert in memory, {cpu_s:.1f} s"},
        "parity_on_sample": parity,
    }


def run_one(args, ctx, name, cpu_seconds):
    wl = WORKLOADS[name]
    steps = args.steps if args.steps is not None else wl["steps"]
    warmup = args.warmup if args.warmup is not None else wl["warmup"]
    if wl.get("streamed"):
        return run_streamed(args, ctx, name, steps, cpu_seconds)
    if name == "q4k_stack48":
        return run_stack(args, ctx, min(steps, 200), warmup, cpu_seconds)
    if wl.get("hc"):
        return run_hc(args, ctx, name, steps, warmup, cpu_seconds)
    return run_layer(args, ctx, name, steps, warmup, cpu_seconds)


TRACED_GRAPH_NODES_LIMIT = 512


def under_tracer():
    """Whether a profiler's tracing library is loaded into this process (rocprofv3 preloads its tool library)."""
    preload = os.environ.get("LD_PRELOAD", "")
    return "rocprofiler" in preload or any(k.startswith("ROCPROF") for k in os.environ)


def parity_ok(record):
    p = record["parity_on_sample"]
    return all(v for v in p.values() if isinstance(v, bool)) and p.get("error_word", 0) == 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default="all", choices=["all"] + sorted(WORKLOADS))
    ap.add_argument("--cpu-sample", type=int, default=None, help="tokens timed on the CPU path (default: 10 s of work for "
                    "the headline, 3 s for each further configuration)")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--layers", type=int, default=48, help="layers of the q4k_stack48 workload")
    ap.add_argument("--no-stack", action="store_true", help="with --workload all: leave out the 48-layer stack")
    ap.add_argument("--skip-stages", action="store_true",
                    help="leave out the per-kernel timing by cut-off replays (kernel_us is then meaningless): for runs "
                         "under a profiler, which records the kernels' durations itself")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MIB",
                    help="also launch a plain copy kernel of this many MiB three times (byte-counter calibration)")
    ap.add_argument("--margin-window", default="1e-3,inf", metavar="LO,HI",
                    help="one-token decode workloads: keep the seeded tokens whose closest pair among the top-(k+1) router "
                         "logits is at least LO and less than HI apart (default 1e-3,inf: no token is routed again in "
                         "serial order; 0,inf: every drawn token; 0,2e-5: only tokens that are)")
    ap.add_argument("--dims", default=None, metavar="H,E,K,I,S,P",
                    help="with --workload NAME: the layer's shape instead of the workload's own (hidden, experts, top_k, "
                         "intermediate, shared intermediate, stored width of the down projection)")
    args = ap.parse_args()
    lo, hi = args.margin_window.split(",")
    args.margin_window = (float(lo), None if hi.strip() in ("inf", "") else float(hi))
    if args.dims:
        if args.workload == "all":
            sys.exit("--dims needs --workload NAME")
        dims = tuple(int(v) for v in args.dims.split(","))
        if len(dims) != 6:
            sys.exit("--dims takes six numbers: H,E,K,I,S,P")
        wl = WORKLOADS[args.workload]
        WORKLOADS[args.workload] = dict(wl, dims=dims, custom_shape=True, label=wl["label"] + " at the shape " + args.dims)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every box has one GPU); use --gpus 1")

    if under_tracer():
        # A profiled run has ended inside the tracer (a segmentation fault below a graph launch; cause unexplained) whenever
        # the graphs it had instantiated held 640 kernel nodes or more in all, and never with 500 or fewer: refuse such a run.
        names = [args.workload] if args.workload != "all" else [HEADLINE] + ALL_CONFIGS
        for name in names:
            steps = args.steps if args.steps is not None else WORKLOADS[name]["steps"]
            wl_tokens = WORKLOADS[name]["tokens"]
            per_forward = 10 if wl_tokens > 16 else (3 if wl_tokens < 3 else 4)
            forwards = min(steps, 64) + (steps % 64 if steps > 64 else 0)         # the 64-forward graph and the remainder's
            nodes = forwards * per_forward
            if name == "q4k_stack48":                                             # a token and two 2048-token chunks through every layer, on two inputs
                nodes = 2 * (steps * args.layers * 3 + 2 * args.layers * 10)
            elif WORKLOADS[name].get("hc"):
                nodes = forwards * (3 * per_forward + 3)                          # the chain with the add folded, with its own kernel, the block alone
            elif not args.skip_stages:
                nodes += min(steps, 64) * per_forward * 3 // 2                    # the plans of the first 1, 2, ... kernels
            if nodes > TRACED_GRAPH_NODES_LIMIT:
                sys.exit(f"under a profiler's tracer, {name} with --steps {steps} would instantiate graphs of about {nodes} kernel "
                         f"nodes; keep it to {TRACED_GRAPH_NODES_LIMIT} (--skip-stages, fewer steps, or a step count that is a multiple of 64)")
    api = pf.load_product()
    hip = api.hip
    if hip.device_count() < 1:
        sys.exit("no HIP device: the benchmark runs the HIP path only")
    ctx = (api, hip, Tools())
    if args.workload != "all":
        record = run_one(args, ctx, args.workload, 12.0)
        print(json.dumps(record))
        if not parity_ok(record):
            sys.exit("parity check failed on the sample")
        return
    record = run_one(args, ctx, HEADLINE, 10.0)
    record["configs"] = {}
    for name in ALL_CONFIGS:
        if name == "q4k_stack48" and args.no_stack:
            continue
        print(f"[bench] {name} ...", file=sys.stderr, flush=True)
        record["configs"][name] = run_one(args, ctx, name, 3.0)
    print(json.dumps(record))
    bad = [n for n, r in [(HEADLINE, record)] + list(record["configs"].items()) if not parity_ok(r)]
    if bad:
        sys.exit(f"parity check failed on the sample: {bad}")


if __name__ == "__main__":
    main()
