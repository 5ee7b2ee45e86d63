"""Benchmark of the hot path on one MI355X.

A step is one pass of the north-star chain over one batch of synthetic input resident in
HBM: gate-logits GEMM -> softmax / top-2 / capacity slots -> dispatch fused with the int8
codec, at 16384 tokens x model_dim 4096 x 8 experts, top-2, capacity_factor 1.25, bf16.
Prints ONE JSON line (see --help for the knobs).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def event_time_us(fn, iters, warm, rounds=5):
    """Average device time of one call: `iters` calls are enqueued back to back between one
    pair of HIP events (so the GPU never waits for the host), best and mean of `rounds`."""
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    per_call = []
    for _ in range(rounds):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        per_call.append(a.elapsed_time(b) * 1e3 / iters)
    per_call.sort()
    return sum(per_call) / len(per_call), per_call[len(per_call) // 2], per_call[0]


def cpu_baseline(T_sample, M, E, k, cf, x_bits, wg_bits, min_seconds):
    """The CPU oracle (single thread) on the first T_sample tokens of the same batch, repeated
    until `min_seconds` have passed."""
    import numpy as np
    import oracle
    xs = np.ascontiguousarray(x_bits[:T_sample])
    reps, t0 = 0, time.perf_counter()
    while True:
        logits = oracle.gate_logits(xs, wg_bits).astype(np.float32)
        scores = oracle.softmax(logits)
        idx, loc, gates, _ = oracle.route_topk(scores, k)
        C = oracle.capacity(T_sample, E, k, cf, 4)
        x32 = (xs.astype(np.uint32) << 16).view(np.float32)
        d = oracle.encode(x32, list(idx), list(loc), None, E, C)
        d_bits = (d.view(np.uint32) >> 16).astype(np.uint16)          # exact: values are bf16 already
        oracle.int8_compress(d_bits)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds:
            break
    return T_sample * reps / dt, dt, reps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--cpu-sample", type=int, default=16384, help="tokens given to the CPU baseline (0 = skip)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="minimum CPU-baseline run time")
    ap.add_argument("--copy-reference", action="store_true",
                    help="also run a plain 256 MiB device copy a few times (a kernel of known traffic, "
                         "to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings against)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU's share of the path; --gpus %d is not supported "
                 "(nothing here uses a second GPU)" % args.gpus)

    import numpy as np
    import torch
    from planmoe_amd import ops

    dev = "cuda:0"
    T, M, E, k, cf = 16384, 4096, 8, 2, 1.25
    C = ops.capacity(T, E, k, cf, 4)
    R = E * C
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, M, generator=g).bfloat16()
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16()
    xd, wd = x.to(dev), wg.to(dev)

    # the whole chain is one C-ABI call (three launches) writing into buffers allocated once
    plan = ops.ForwardInt8Plan(xd, wd, k, C, fp32_gate=True)

    def chain():
        return plan.run()

    if args.copy_reference:
        ref_src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        ref_dst = torch.empty_like(ref_src)
        for _ in range(5):
            ref_dst.copy_(ref_src)
        torch.cuda.synchronize()

    # timed region: EXACTLY --steps passes between two synchronisations
    for _ in range(args.warmup):
        chain()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        chain()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    tokens_per_s = T / (wall / args.steps)

    # device times (HIP events on the stream the kernels are launched on): the chain, and the
    # dominant kernel alone (dispatch + int8 on the routing the chain produced)
    chain()
    stages = {}
    stages["gate_route (gate GEMM + routing, 2 launches + offsets)"] = event_time_us(
        lambda: ops.gate_route(xd, wd, k, fp32_gate=True), 30, 5)
    stages["dispatch_int8_routed"] = event_time_us(plan.redispatch, 30, 5)
    chain_ev = event_time_us(chain, 30, 5)

    # algorithmic bytes: every input read once, every output written once
    chain_bytes = T * M * 2 + R * M + R * 2 * 2 + T * k * 12 + E * M * 2
    dom_bytes = T * M * 2 + R * M + R * 2 * 2 + T * k * 12         # last launch alone: x, codes, bias/scale, idx/rank/loc
    dom_avg_us = stages["dispatch_int8_routed"][0]
    achieved = dom_bytes / dom_avg_us / 1e3                        # GB/s

    out = {
        "metric": "MoE dispatch/combine+int8 codec tokens/s; achieved HBM GB/s vs peak (1 GPU)",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "config 2: gate GEMM + softmax/top-2/capacity slots + dispatch fused with int8 "
                               "compress, forward", "tokens": T, "model_dim": M, "experts": E, "top_k": k,
                   "capacity_factor": cf, "capacity": C},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     # HBM bytes per launch read from rocprofv3 FETCH_SIZE (x 2.0, the factor a device
                     # copy of known size shows for that counter) + WRITE_SIZE; see profiles/
                     "traffic": 306.0e6,
                     "kernel": "dispatch_int8_routed_kernel (last launch of the chain, timed alone)",
                     "algorithmic_bytes": dom_bytes, "avg_us": dom_avg_us},
        "chain": {"algorithmic_bytes": chain_bytes, "device_us_avg": chain_ev[0], "device_us_min": chain_ev[2],
                  "GBps": chain_bytes / chain_ev[0] / 1e3, "frac_of_hbm_peak": chain_bytes / chain_ev[0] / 1e3 / HBM_PEAK_GBS,
                  "stage_us_avg": {n: v[0] for n, v in stages.items()}},
    }
    if args.cpu_sample > 0:
        bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
        v, dt, reps = cpu_baseline(min(args.cpu_sample, T), M, E, k, cf, bits(x), bits(wg), args.cpu_seconds)
        out["cpu_baseline"] = {"value": v, "unit": "tokens/s", "cores": 1, "kind": "port",
                               "sample": "%d of the %d tokens x %d passes of the same chain through the CPU "
                                         "oracle (single thread, %.1f s)" % (min(args.cpu_sample, T), T, reps, dt),
                               "host_cores": os.cpu_count()}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
