"""Benchmark of the hot path on one MI355X.

A step is one pass of the north-star chain over one batch of synthetic input resident in
HBM: gate-logits GEMM -> softmax / top-2 / capacity slots -> dispatch fused with the int8
codec, at 16384 tokens x model_dim 4096 x 8 experts, top-2, capacity_factor 1.25, bf16, through
the one-launch entry point that reads the tokens once.
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


def cpu_baseline_oracle(T_sample, M, E, k, cf, x_bits, wg_bits, min_seconds):
    """The whole chain through the CPU oracle (one thread, scalar C) on the first T_sample tokens of
    the same batch, repeated until `min_seconds` have passed."""
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


def cpu_baseline(T_sample, M, E, k, cf, x, wg, min_seconds):
    """The reference's CPU path for the same chain on the first T_sample tokens of the same batch:
    torch-CPU ops with all of torch's intra-op threads for the gate (x.float() @ wg.float().T,
    top.py:21-26), softmax, top-k, one-hot masks, cumsum and gate normalisation
    (fast_dispatch.py:140-172) and for the int8 codec's ATen chain in bf16 (int8.cpp:10-16); the
    dispatch is the single-threaded C loop of custom_kernel.cpp:57-81 (the oracle's restatement; the
    reference has no OpenMP there) on fp32 data, cast back to bf16 as the dispatcher does
    (fast_dispatch.py:121-125).  Repeated until `min_seconds` have passed."""
    import numpy as np
    import torch
    import oracle
    xs, wf = x[:T_sample], wg.float()
    reps, t0 = 0, time.perf_counter()
    while True:
        logits = torch.nn.functional.linear(xs.float(), wf)
        scores = torch.softmax(logits, dim=1)
        top = torch.topk(scores, k, dim=1).indices
        masks = [torch.zeros_like(scores, dtype=torch.int64).scatter_(1, top[:, j:j + 1], 1) for j in range(k)]
        gates = [(scores * m).sum(1) for m in masks]
        locs, base = [], torch.zeros((1, E), dtype=torch.int64)
        for j in range(k):
            locs.append((((torch.cumsum(masks[j], 0) - 1) + base) * masks[j]).sum(1).to(torch.int32))
            base = base + masks[j].sum(0, keepdim=True)
        den = torch.clamp(sum(gates), min=torch.finfo(scores.dtype).eps)
        gates = [v / den for v in gates]
        C = oracle.capacity(T_sample, E, k, cf, 4)
        idx = [top[:, j].to(torch.int32).numpy() for j in range(k)]
        d = oracle.encode(xs.float().numpy(), idx, [l.numpy() for l in locs], None, E, C)
        db = torch.from_numpy(d).bfloat16().view(E, C, M)
        bias = torch.min(db, -1, keepdim=True).values
        scale = torch.max(db, -1, keepdim=True).values - bias
        codes = (((db - bias) / scale) * 255.0).to(torch.uint8)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds:
            break
    del codes
    return T_sample * reps / dt, dt, reps


def profile_traffic_bytes():
    """HBM bytes per launch of the one-launch chain as the committed rocprofv3 counter summary states
    them (a line 'traffic_bytes_per_launch = N' in profiles/forward_int8_single_config2_hbm_traffic.txt);
    None when the summary is not there.  Nothing is typed in here: a stale profile shows by its date."""
    path = os.path.join(ROOT, "profiles", "forward_int8_single_config2_hbm_traffic.txt")
    try:
        for line in open(path):
            if line.strip().startswith("traffic_bytes_per_launch"):
                return float(line.split("=")[1].split()[0])
    except OSError:
        pass
    return None


def kernel_table(only=None):
    """Every entry point at the full size of its workload (the five benchmark configurations): device time over
    back-to-back launches (HIP events) against the algorithmic bytes = inputs read once + outputs
    written once.  One line per entry point; an entry point may be several launches."""
    import torch
    from planmoe_amd import ops
    dev = "cuda:0"
    g = torch.Generator().manual_seed(0)
    rows = []
    scrub = torch.zeros((1 << 28,), dtype=torch.int32, device=dev)

    def add(name, cfg, nbytes, fn, iters=20):
        if only and only not in "%s [%s]" % (name, cfg):
            return
        # the calls are recorded into a HIP graph once and the graph is replayed: the Python
        # wrappers (output allocation + ctypes call) are slower than the short kernels
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(iters):
                fn()
        avg, med, best = event_time_us(graph.replay, 1, 1, rounds=5)
        del graph
        # cold: every call behind a pass over 1 GiB that leaves none of the call's operands in the
        # L2s or the 256 MB memory-side cache; one event pair per call (the scrub runs long enough
        # for the host to have the call enqueued before the device reaches it).  Two scrubs: one
        # that only reads (the caches hold clean lines of other data) and one that also writes
        # (they hold dirty lines, whose write-back then falls into the timed call).
        cold = []
        for scrub_fn in (lambda: torch.max(scrub), lambda: scrub.add_(1)):
            pairs = []
            for _ in range(7):
                scrub_fn()
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                fn()
                b.record()
                pairs.append((a, b))
            torch.cuda.synchronize()
            cold.append(sorted(a.elapsed_time(b) * 1e3 for a, b in pairs)[len(pairs) // 2])
        rows.append((name, cfg, nbytes, avg / iters, best / iters, cold[0], cold[1]))

    # configs 2 / 4: 16384 tokens x 4096, 8 experts, top-2, capacity_factor 1.25, bf16
    T, M, E, k = 16384, 4096, 8, 2
    C = ops.capacity(T, E, k, 1.25, 4); R = E * C
    x = torch.randn(T, M, generator=g).bfloat16().to(dev)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(dev)
    r = ops.gate_route(x, wg, k)
    idx, loc, gates = list(r["indices"]), list(r["locations"]), list(r["gates"])
    live = int(sum(((l >= 0) & (l < C)).sum() for l in loc))                 # token rows that reach a slot

    def kept(locs, cap):
        """Tokens with at least one slot: a dispatch has no use for the rows of the others."""
        hit = torch.zeros_like(locs[0], dtype=torch.bool)
        for l in locs:
            hit |= (l >= 0) & (l < cap)
        return int(hit.sum())
    xb, db, plane = T * M * 2, R * M * 2, T * k * 12
    add("gate_logits", "2", xb + E * M * 2 + T * E * 4, lambda: ops.gate_logits(x, wg, torch.float32))
    add("gate_route (gate + routing)", "2", xb + E * M * 2 + plane, lambda: ops.gate_route(x, wg, k))
    sc = torch.softmax(ops.gate_logits(x, wg, torch.float32), 1)
    add("route_topk (scores in)", "2", T * E * 4 + plane, lambda: ops.route_topk(sc, k))
    add("dispatch_fwd", "2", kept(loc, C) * M * 2 + db + plane, lambda: ops.dispatch_fwd(x, idx, loc, None, E, C))
    d = ops.dispatch_fwd(x, idx, loc, None, E, C)
    add("combine_fwd", "2", live * M * 2 + xb + plane, lambda: ops.combine_fwd(d, idx, loc, gates, T, C))
    add("bwd_gate", "2", live * M * 2 + xb + plane, lambda: ops.bwd_gate(x, d, idx, loc, C))
    add("int8_compress", "2", db + R * M + R * 4, lambda: ops.int8_compress(d))
    codes, b, s_ = ops.int8_compress(d)
    add("int8_decompress", "2", db + R * M + R * 4, lambda: ops.int8_decompress(codes, b, s_))
    add("combine_int8 (fused)", "2", live * M + R * 4 + xb + plane,
        lambda: ops.combine_int8(codes, b, s_, idx, loc, gates, T, C))
    add("dispatch_int8 (fused)", "2", xb + R * M + R * 4 + plane, lambda: ops.dispatch_int8(x, idx, loc, None, E, C))
    add("combine_bwd_int8 (fused)", "4", xb + live * M * 2 + R * M + R * 4 + plane + T * k * 4,
        lambda: ops.combine_bwd_int8(x, d, idx, loc, gates, E, C))
    dc = ops.int8_compress(d)
    add("combine_bwd_int8 (coded in)", "4", xb + live * M + R * M + 2 * R * 4 + plane + T * k * 4,
        lambda: ops.combine_bwd_int8(x, dc, idx, loc, gates, E, C))
    dxb = torch.randn(T, M, generator=g).bfloat16().to(dev)
    glog = (torch.randn(T, E, generator=g) * 0.01).to(dev)
    add("gate_dx_accumulate", "2", 2 * xb + T * E * 4 + E * M * 2, lambda: ops.gate_dx_accumulate(dxb, glog, wg))
    plan = ops.ForwardInt8Plan(x, wg, k, C, fp32_gate=True)
    add("forward_int8 (2 launches)", "2", xb + E * M * 2 + R * M + R * 4 + plane, plan.run)
    plan1 = ops.ForwardInt8Plan(x, wg, k, C, fp32_gate=True, single=True)
    add("forward_int8_single (1 launch)", "2", xb + E * M * 2 + R * M + R * 4 + plane, plan1.run)
    # the experts' first GEMM straight from the codes (hidden 4096): bound by the matrix cores, so
    # its line below the table is priced in flops; in the table it has its operand and result bytes
    Hf = 4096
    wk = (torch.randn(E, Hf, M, generator=g) * M ** -0.5).bfloat16().to(dev)
    fb = torch.zeros(E, Hf, dtype=torch.bfloat16, device=dev)
    fout = torch.empty(E, C, Hf, dtype=torch.bfloat16, device=dev)
    add("ffn_fc1_int8 (GEMM from codes)", "2", R * M + R * 4 + E * Hf * M * 2 + R * Hf * 2,
        lambda: ops.ffn_fc1_int8(codes.view(E, C, M), b.view(E, C, 1), s_.view(E, C, 1), wk, fb, out=fout), iters=5)
    wcs = ops.ffn_weight_colsum(wk)
    add("ffn_fc1_int8_affine (GEMM on codes)", "2", R * M + R * 4 + E * Hf * M * 2 + R * Hf * 2,
        lambda: ops.ffn_fc1_int8_affine(codes.view(E, C, M), b.view(E, C, 1), s_.view(E, C, 1), wk, wcs, fb, out=fout), iters=5)
    ffn_flops = 2.0 * R * M * Hf
    # the experts' GEMMs proper: the first one with bias + relu on the decompressed rows (planmoe_gemm_nt_bf16,
    # second operand k-major), and the transpose that brings an operand into that form
    xin = torch.randn(E, C, M, generator=g).bfloat16().to(dev)
    add("ffn_gemm_nt_bf16 (x @ W + b, relu)", "2", R * M * 2 + E * Hf * M * 2 + R * Hf * 2,
        lambda: ops.gemm_nt_bf16(xin, wk, fb, relu=True, out=fout), iters=5)
    # the same product with the weight as the experts store it ([E, in, out]: no transposed copy), and the
    # weight gradient x^T dy with both operands as they lie (Hf == M here, so the flops are the same)
    wst = wk.transpose(1, 2).contiguous()
    add("ffn_gemm_nn_bf16 (x @ W + b, relu)", "2", R * M * 2 + E * Hf * M * 2 + R * Hf * 2,
        lambda: ops.gemm_nn_bf16(xin, wst, fb, relu=True, out=fout), iters=5)
    dwout = torch.empty(E, M, Hf, dtype=torch.bfloat16, device=dev)
    add("ffn_gemm_tn_bf16 (dW = x^T @ dy)", "2", R * M * 2 + R * Hf * 2 + E * M * Hf * 2,
        lambda: ops.gemm_tn_bf16(xin, fout, out=dwout), iters=5)
    del wst, dwout
    add("ffn_transpose_bf16 [8, 5120, 4096]", "2", 2 * R * M * 2, lambda: ops.transpose_bf16(xin, 64), iters=5)
    del d, dc, codes, plan, plan1, wk, fout, xin

    # config 1: 8192 x 2048 fp32, 2 experts, top-2
    T1, M1, E1 = 8192, 2048, 2
    x1 = torch.randn(T1, M1, generator=g).to(dev)
    w1 = (torch.randn(E1, M1, generator=g) * M1 ** -0.5).to(dev)
    C1 = ops.capacity(T1, E1, 2, 1.0, 4)
    r1 = ops.gate_route(x1, w1, 2)
    i1, l1, g1 = list(r1["indices"]), list(r1["locations"]), list(r1["gates"])
    add("gate_route (gate + routing)", "1", T1 * M1 * 4 + T1 * 24, lambda: ops.gate_route(x1, w1, 2))
    add("dispatch_fwd", "1", kept(l1, C1) * M1 * 4 + E1 * C1 * M1 * 4, lambda: ops.dispatch_fwd(x1, i1, l1, None, E1, C1))
    d1 = ops.dispatch_fwd(x1, i1, l1, None, E1, C1)
    add("combine_fwd", "1", 3 * T1 * M1 * 4, lambda: ops.combine_fwd(d1, i1, l1, g1, T1, C1))
    del d1

    def chain1():
        r = ops.forward_plain(x1, w1, 2, C1)
        return ops.combine_fwd(r["dispatched"], list(r["indices"]), list(r["locations"]), list(r["gates"]), T1, C1)
    add("forward_plain (gate, routing, dispatch)", "1", T1 * M1 * 4 + E1 * C1 * M1 * 4 + T1 * 24, lambda: ops.forward_plain(x1, w1, 2, C1))
    # the config's whole chain: x read, the dispatched buffer written and read, y written
    add("chain: forward_plain, combine", "1", T1 * M1 * 4 + E1 * C1 * M1 * 4 + 2 * T1 * M1 * 4 + T1 * M1 * 4 + T1 * 24, chain1)

    # config 3: 32768 x 2048 bf16, 64 experts, top-1, skewed logits
    T3, M3, E3 = 32768, 2048, 64
    x3 = torch.randn(T3, M3, generator=g).bfloat16().to(dev)
    w3 = (torch.randn(E3, M3, generator=g) * M3 ** -0.5).bfloat16().to(dev)
    pz = torch.arange(1, E3 + 1, dtype=torch.float64) ** -1.2
    bias = torch.log(pz / pz.sum()).float().to(dev)
    C3 = ops.capacity(T3, E3, 1, 1.0, 4)
    add("gate_logits", "3", T3 * M3 * 2 + T3 * E3 * 4, lambda: ops.gate_logits(x3, w3, torch.float32))
    add("gate_route (gate + routing)", "3", T3 * M3 * 2 + T3 * 12, lambda: ops.gate_route(x3, w3, 1, logit_bias=bias))
    add("forward_int8 (chain)", "3", T3 * M3 * 2 + E3 * C3 * M3 + T3 * 12,
        lambda: ops.forward_int8(x3, w3, 1, C3, logit_bias=bias))
    r3 = ops.gate_route(x3, w3, 1, logit_bias=bias)
    i3, l3 = list(r3["indices"]), list(r3["locations"])
    add("dispatch_fwd", "3", kept(l3, C3) * M3 * 2 + E3 * C3 * M3 * 2 + T3 * 12, lambda: ops.dispatch_fwd(x3, i3, l3, None, E3, C3))

    # the config's chain as stated (no codec): x read by the gate, kept rows read again, the buffer written
    add("forward_plain (gate, routing, dispatch)", "3", T3 * M3 * 2 + E3 * C3 * M3 * 2 + T3 * 12,
        lambda: ops.forward_plain(x3, w3, 1, C3, logit_bias=bias))
    lg = ops.gate_logits(x3, w3, torch.float32)
    add("route_topk (logits in)", "3", T3 * E3 * 4 + T3 * 12, lambda: ops.route_topk(lg, 1, is_logits=True, logit_bias=bias))
    mask = (torch.rand(T3, E3, device=dev) < 0.1).to(torch.int32)
    add("cumsum_sub_one", "3", 2 * T3 * E3 * 4, lambda: ops.cumsum_sub_one(mask))

    # config 5: zfp rate 8 on a [16, 8192, 1024] fp32 buffer
    f = torch.randn(16 * 8192, 1024, generator=g).to(dev)
    nx, ny = 1024, 16 * 8192
    zb = f.numel() * 4 + f.numel()
    for dims in (2, 1):
        add("zfp_compress %d-D" % dims, "5", zb, lambda: ops.zfp_compress(f, nx, ny, dims), iters=5)
        st = ops.zfp_compress(f, nx, ny, dims)
        add("zfp_decompress %d-D" % dims, "5", zb, lambda: ops.zfp_decompress(st, nx, ny, dims), iters=5)

    # config 5's send side: 65536 tokens x 1024 fp32, 16 experts, top-2, capacity 8192, into the zfp stream
    T5, M5, E5, k5 = 65536, 1024, 16, 2
    C5 = ops.capacity(T5, E5, k5, 1.0, 4)
    x5 = torch.randn(T5, M5, generator=g).to(dev)
    r5 = ops.route_topk(torch.softmax(torch.randn(T5, E5, generator=g), 1).to(dev), k5)
    i5, l5 = list(r5["indices"]), list(r5["locations"])
    zs = ops.dispatch_zfp(x5, i5, l5, None, E5, C5)
    g5 = [t.float() for t in r5["gates"]]
    d5 = ops.zfp_decompress(zs, M5, E5 * C5, 2)
    add("dispatch_fwd", "5", kept(l5, C5) * M5 * 4 + E5 * C5 * M5 * 4, lambda: ops.dispatch_fwd(x5, i5, l5, None, E5, C5), iters=5)
    add("combine_fwd", "5", 3 * T5 * M5 * 4, lambda: ops.combine_fwd(d5, i5, l5, g5, T5, C5), iters=5)
    add("combine_zfp (fused)", "5", E5 * C5 * M5 + T5 * M5 * 4,
        lambda: ops.combine_zfp(zs, i5, l5, g5, T5, E5, C5, M5), iters=5)
    add("dispatch_zfp (fused)", "5", T5 * M5 * 4 + E5 * C5 * M5, lambda: ops.dispatch_zfp(x5, i5, l5, None, E5, C5, out=zs), iters=5)
    add("bwd_gate", "5", 3 * T5 * M5 * 4, lambda: ops.bwd_gate(x5, d5, i5, l5, C5), iters=5)
    add("bwd_gate_zfp (fused)", "5", E5 * C5 * M5 + T5 * M5 * 4, lambda: ops.bwd_gate_zfp(zs, x5, i5, l5, E5, C5), iters=5)

    # the same buffer through the lossless codec: as it is (no symbol repeats, nothing shrinks) and
    # with 30 % of the capacity slots empty (zero rows shrink to 44 bytes per 2048)
    for label, buf in (("dense", f), ("30% empty", f * (torch.rand(f.shape[0], 1, device=dev) >= 0.3))):
        buf = buf.contiguous()
        fo, do, fl, da = ops.lz_compress(buf)
        used = int(fo[-1]) + int(do[-1]) + 2 * fo.numel() * 4
        lws = torch.empty((ops.lib.planmoe_lz_workspace_bytes(buf.numel() * 4),), dtype=torch.uint8, device=dev)
        add("lz_compress %s" % label, "5", buf.numel() * 4 + used, lambda: ops.lz_compress(buf, workspace=lws), iters=5)
        out = torch.empty_like(buf)
        add("lz_decompress %s" % label, "5", buf.numel() * 4 + used, lambda: ops.lz_decompress(out, fo, do, fl, da), iters=5)

    print("%-36s %-4s %10s %9s %9s %8s %6s %10s %10s" % ("entry point", "cfg", "alg MB", "avg us", "best us", "GB/s", "frac",
                                                         "cold-r us", "cold-w us"))
    for name, cfg, nbytes, avg, best, cold_r, cold_w in rows:
        gbs = nbytes / avg / 1e3
        print("%-36s %-4s %10.1f %9.1f %9.1f %8.0f %6.2f %10.1f %10.1f" % (name, cfg, nbytes / 1e6, avg, best, gbs,
                                                                         gbs / HBM_PEAK_GBS, cold_r, cold_w))
        if name.startswith("ffn_fc1_int8") or name.startswith("ffn_gemm"):
            print("%-36s %-4s %10s %9s %9s %8.0f TFLOP/s = %.3f of the %.0f TFLOP/s dense bf16 MFMA peak" % (
                "  ^ as a GEMM", cfg, "", "", "", ffn_flops / avg / 1e6, ffn_flops / avg / 1e6 / 2500.0, 2500.0))


def cpu_stage_table(min_seconds=2.0):
    """The CPU oracle, one thread, stage by stage on bounded samples of the same workloads (the
    first `sample` tokens or rows; slot capacity recomputed for the sample): seconds per call and
    algorithmic bytes per second, to set beside the device table of --kernels."""
    import numpy as np
    import oracle
    rng = np.random.default_rng(0)
    rows = []

    def add(name, cfg, sample, nbytes, fn):
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= min_seconds:
                break
        rows.append((name, cfg, sample, nbytes, dt / reps))

    # configs 2 / 4 on 4096 of the 16384 tokens (bf16 data as the fp32 the reference computes in)
    T, M, E, k = 4096, 4096, 8, 2
    C = oracle.capacity(T, E, k, 1.25, 4); R = E * C
    xb = (rng.standard_normal((T, M), dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)
    wb = ((rng.standard_normal((E, M), dtype=np.float32) * M ** -0.5).view(np.uint32) >> 16).astype(np.uint16)
    x = (xb.astype(np.uint32) << 16).view(np.float32)
    logits = oracle.gate_logits(xb, wb).astype(np.float32)
    scores = oracle.softmax(logits)
    idx, loc, gates, _ = oracle.route_topk(scores, k)
    idx, loc, gates = list(idx), list(loc), list(gates)
    tok = "%d tokens" % T
    add("gate_logits", "2", tok, T * M * 2 + E * M * 2 + T * E * 4, lambda: oracle.gate_logits(xb, wb))
    add("softmax + route_topk", "2", tok, T * E * 4 + T * k * 12, lambda: oracle.route_topk(oracle.softmax(logits), k))
    add("dispatch_fwd (encode)", "2", tok, T * M * 2 + R * M * 2, lambda: oracle.encode(x, idx, loc, None, E, C))
    d = oracle.encode(x, idx, loc, None, E, C)
    add("combine_fwd (decode)", "2", tok, T * k * M * 2 + T * M * 2, lambda: oracle.decode(d, idx, loc, gates, T, C))
    add("bwd_gate", "2", tok, T * k * M * 2 + T * M * 2,
        lambda: [oracle.bwd_gate(idx[j], loc[j], x, d, C) for j in range(k)])
    db = (d.view(np.uint32) >> 16).astype(np.uint16)
    add("int8_compress", "2", tok, R * M * 2 + R * M, lambda: oracle.int8_compress(db))
    codes, bias, scale = oracle.int8_compress(db)
    add("int8_decompress", "2", tok, R * M * 2 + R * M, lambda: oracle.int8_decompress(codes, bias, scale))

    # config 3's routing: 64 experts, top-1
    T3, E3 = 8192, 64
    mask = (rng.random((T3, E3)) < 0.1).astype(np.int32)
    add("cumsum_sub_one", "3", "%d tokens" % T3, 2 * T3 * E3 * 4, lambda: oracle.cumsum_sub_one(mask))
    s3 = oracle.softmax(rng.standard_normal((T3, E3), dtype=np.float32))
    add("route_topk", "3", "%d tokens" % T3, T3 * E3 * 4 + T3 * 12, lambda: oracle.route_topk(s3, 1))

    # the routing as the reference's CPU path runs it: ATen ops on the CPU, multi-threaded by torch
    # (softmax, top-k, one-hot masks, cumsum, fast_dispatch.py:140-172 restated)
    import torch

    def torch_routing(lg, kk):
        sc = torch.softmax(lg, 1)
        top = torch.topk(sc, kk, dim=1).indices
        masks = [torch.zeros_like(sc, dtype=torch.int64).scatter_(1, top[:, j:j + 1], 1) for j in range(kk)]
        gs = [(sc * m).sum(1) for m in masks]
        locs, base = [], torch.zeros((1, sc.shape[1]), dtype=torch.int64)
        for j in range(kk):
            locs.append((((torch.cumsum(masks[j], 0) - 1) + base) * masks[j]).sum(1).to(torch.int32))
            base = base + masks[j].sum(0, keepdim=True)
        den = torch.clamp(sum(gs), min=torch.finfo(sc.dtype).eps)
        return top, locs, [v / den for v in gs]

    tl2 = torch.from_numpy(logits)
    add("routing, torch-CPU x%d thr" % torch.get_num_threads(), "2", tok, T * E * 4 + T * k * 12, lambda: torch_routing(tl2, k))
    tl3 = torch.from_numpy(rng.standard_normal((T3, E3), dtype=np.float32))
    add("routing, torch-CPU x%d thr" % torch.get_num_threads(), "3", "%d tokens" % T3, T3 * E3 * 4 + T3 * 12, lambda: torch_routing(tl3, 1))

    # config 5's codecs on 2048 of the 131072 slot rows
    R5, M5 = 2048, 1024
    f = rng.standard_normal((R5, M5), dtype=np.float32)
    rw = "%d rows" % R5
    for dims in (2, 1):
        add("zfp_compress %d-D" % dims, "5", rw, R5 * M5 * 5, lambda: oracle.zfp_compress(f, dims))
        st = oracle.zfp_compress(f, dims)
        add("zfp_decompress %d-D" % dims, "5", rw, R5 * M5 * 5, lambda: oracle.zfp_decompress(st, R5, M5, dims))
    f[rng.random(R5) < 0.3] = 0.0
    add("lz_compress 30% empty", "5", rw, R5 * M5 * 4, lambda: oracle.lz_compress(f))
    lz = oracle.lz_compress(f)
    add("lz_decompress 30% empty", "5", rw, R5 * M5 * 4, lambda: oracle.lz_decompress(*lz))

    print("CPU oracle, 1 thread of %d (%s)" % (os.cpu_count(), "bounded samples; GB/s of algorithmic bytes; the torch-CPU rows use torch's threads"))
    print("%-26s %-4s %-12s %10s %10s %8s" % ("stage", "cfg", "sample", "alg MB", "ms / call", "GB/s"))
    for name, cfg, sample, nbytes, sec in rows:
        print("%-26s %-4s %-12s %10.1f %10.2f %8.3f" % (name, cfg, sample, nbytes / 1e6, sec * 1e3, nbytes / sec / 1e9))


def layer_table():
    """moe_layer forward + backward with identity experts (the data path alone: gate, routing,
    encode, codec, comm copy, codec, decode and their backward passes) for every compressor,
    with the fused entry points and with the step-by-step pipeline of the reference's structure."""
    import torch
    import planmoe_amd
    from planmoe_amd import overlap
    dev = "cuda:0"

    class Identity(torch.nn.Module):
        def update(self, ctx):
            self.dummy = torch.nn.Parameter(torch.zeros(1))

        def forward(self, x, ctx):
            return x

    cases = [("2", 16384, 4096, 8, 2, 1.25, torch.bfloat16, "no"), ("2", 16384, 4096, 8, 2, 1.25, torch.bfloat16, "int8"),
             ("5", 65536, 1024, 16, 2, 1.0, torch.float32, "no"), ("5", 65536, 1024, 16, 2, 1.0, torch.float32, "zfp"),
             ("5", 65536, 1024, 16, 2, 1.0, torch.float32, "lz")]
    print("%-4s %-6s %-9s %14s %14s" % ("cfg", "codec", "dtype", "fused ms", "stepwise ms"))
    for cfg, T, M, E, k, cf, dtype, codec in cases:
        times = []
        for fused in (True, False):
            overlap.FUSE_INT8 = overlap.FUSE_GATE = overlap.FUSE_ZFP = fused
            layer = planmoe_amd.moe_layer({'type': 'top', 'k': k, 'capacity_factor': cf, 'fp32_gate': True}, M,
                                          experts={'type': 'custom', 'module': Identity(), 'count_per_node': E},
                                          seeds=(1, 2, 3), compress_name=codec).to(dev).to(dtype)
            x = torch.randn(T, M, generator=torch.Generator().manual_seed(0)).to(dtype).to(dev).requires_grad_(True)

            dy = torch.randn(T, M, generator=torch.Generator().manual_seed(1)).to(dtype).to(dev)
            one = torch.ones((), device=dev)

            def step():
                y = layer(x)
                # the gradient comes in ready-made, as from the layers above: no loss kernels in the timing
                torch.autograd.backward([y, y.l_aux], [dy, one.to(y.l_aux.dtype)])
                x.grad = None
            times.append(event_time_us(step, 5, 5, rounds=5)[1] / 1e3)      # median of the rounds
        overlap.FUSE_INT8 = overlap.FUSE_GATE = overlap.FUSE_ZFP = True
        print("%-4s %-6s %-9s %14.3f %14.3f" % (cfg, codec, str(dtype).replace("torch.", ""), times[0], times[1]))


def overlap_run(passes=6):
    """The reference's pipeline (one entry point per step) around identity experts with the comm
    step copying on the comm stream, at a2a_ffn_overlap_degree 1 and 2, forward only, config 2 with
    the int8 compressor.  Meant to be run under `rocprofv3 --kernel-trace --memory-copy-trace`: at
    degree 2 the copy of a chunk (comm stream) lies beside the compress of the next chunk."""
    import torch
    import planmoe_amd
    from planmoe_amd import overlap, compressor
    dev = "cuda:0"

    class Identity(torch.nn.Module):
        def update(self, ctx):
            self.dummy = torch.nn.Parameter(torch.zeros(1))

        def forward(self, x, ctx):
            return x

    T, M, E, k, cf = 16384, 4096, 8, 2, 1.25
    overlap.FUSE_INT8 = overlap.FUSE_GATE = overlap.FUSE_ZFP = False
    compressor.SINGLE_RANK_COMM_COPIES = True
    x = torch.randn(T, M, generator=torch.Generator().manual_seed(0)).bfloat16().to(dev)
    outs = []
    for degree in (1, 2):
        layer = planmoe_amd.moe_layer({'type': 'top', 'k': k, 'capacity_factor': cf, 'fp32_gate': True}, M,
                                      experts={'type': 'custom', 'module': Identity(), 'count_per_node': E},
                                      seeds=(1, 2, 3), compress_name="int8", a2a_ffn_overlap_degree=degree).to(dev).to(torch.bfloat16)
        scrub = torch.zeros((1 << 28,), dtype=torch.int32, device=dev)
        with torch.no_grad():
            def step():
                # two passes over 1 GiB first: while the GPU is busy with them the host enqueues the whole
                # layer, so that the trace shows what the streams allow and not how fast Python is
                torch.max(scrub), torch.max(scrub)
                return layer(x)
            avg, med, best = event_time_us(step, passes, 2, rounds=3)
            outs.append(step())
        torch.cuda.synchronize()
        print("a2a_ffn_overlap_degree %d: 2 GiB of reads + forward %.1f us (median of 3 rounds of %d passes)" % (degree, med, passes), flush=True)
    print("outputs of degree 2 equal to degree 1:", bool(torch.equal(outs[0], outs[1])))


def phase_table():
    """Wall-clock stamps of the phases of the one-launch forward kernel and of its ceiling kernel
    (modes 0 and 1), per work-group, from the measurement build of the library
    (make -C planmoe_amd/csrc libplanmoe_hip_trace.so: forward.hip with -DPM_FS_TRACE).  Config 2."""
    import ctypes
    import subprocess
    import numpy as np
    import torch
    from planmoe_amd import ops, _lib
    csrc = os.path.join(os.path.dirname(os.path.abspath(__file__)), "planmoe_amd", "csrc")
    path = os.path.join(csrc, "libplanmoe_hip_trace.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", csrc, "libplanmoe_hip_trace.so"])
    tl = ctypes.CDLL(path)
    dev = "cuda:0"
    T, M, E, k = 16384, 4096, 8, 2
    C = ops.capacity(T, E, k, 1.25, 4)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, M, generator=g).bfloat16().to(dev)
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(dev)
    plan = ops.ForwardInt8Plan(x, wg, k, C, fp32_gate=True, single=True)
    a = list(plan._args)
    fn, cf = tl.planmoe_forward_int8_single, tl.planmoe_forward_int8_single_ceiling
    fn.restype = cf.restype = ctypes.c_int
    fn.argtypes = _lib.SIGNATURES["planmoe_forward_int8_single"][1]
    cf.argtypes = _lib.SIGNATURES["planmoe_forward_int8_single_ceiling"][1]
    gave = torch.zeros((), dtype=torch.int32, device=dev)
    st = ops._stream(x)
    ceil = ops.ForwardCeiling(x, E, k, C)

    def trace(run):
        for _ in range(5):
            run()
        torch.cuda.synchronize()
        buf = np.zeros(1024 * 16, dtype=np.uint64)
        tl.planmoe_debug_fs_trace(buf.ctypes.data_as(ctypes.c_void_p))
        tr = buf.reshape(1024, 16)[:(T + 63) // 64, :16].astype(np.int64)
        return (tr - tr[:, 0].min()) / 100.0            # the stamps count a 100 MHz clock

    def real():
        assert fn(*a, 0, ops._ptr(gave), st) == 0

    res = {"forward_single": trace(real)}
    for mode in (0, 1):
        def run(mode=mode):
            assert cf(ops._ptr(x), T, M, E, k, C, ops._ptr(ceil.codes), ops._ptr(ceil.bias), ops._ptr(ceil.scale),
                      ops._ptr(ceil.planes), ops._ptr(ceil.ws), ceil.ws.numel(), mode, 0, ops._ptr(gave), st) == 0
        res["ceiling mode %d" % mode] = trace(run)
    names = {0: "first instruction", 1: "round 0 done", 2: "round 1 done", 3: "round 2 done", 4: "round 3 done + barrier",
             5: "histogram published", 7: "all groups seen", 8: "slot bases known", 9: "parked rows flushed (wave 0)",
             10: "register rounds in LDS", 11: "register rounds flushed", 12: "empty slots zeroed (end)"}
    print("microseconds since the first work-group's first instruction; thread 0 of each of the %d work-groups; median / max" % ((T + 63) // 64))
    print("%-30s" % "stamp" + "".join("%24s" % n for n in res))
    for i, n in names.items():
        print("%-30s" % n + "".join("%14.2f %9.2f" % (np.median(r[:, i]), r[:, i].max()) for r in res.values()))
    for n, r in res.items():
        print("%-16s published at (percentiles 0/10/50/90/100) %s | ended at %s" % (
            n, " ".join("%.1f" % np.percentile(r[:, 5], p) for p in (0, 10, 50, 90, 100)),
            " ".join("%.1f" % np.percentile(r[:, 12], p) for p in (0, 10, 50, 90, 100))))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-sample", type=int, default=16384, help="tokens given to the CPU baseline (0 = skip)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="minimum CPU-baseline run time")
    ap.add_argument("--copy-reference", action="store_true",
                    help="also run a plain 256 MiB device copy a few times (a kernel of known traffic, "
                         "to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings against)")
    ap.add_argument("--kernels", action="store_true",
                    help="instead of the JSON line, print a table of every entry point at full size "
                         "(device time, algorithmic bytes, fraction of the HBM peak)")
    ap.add_argument("--layer", action="store_true",
                    help="instead of the JSON line, time moe_layer forward + backward with identity experts for "
                         "every compressor, with and without the fused entry points")
    ap.add_argument("--overlap", action="store_true",
                    help="instead of the JSON line, run the step-by-step int8 pipeline with the comm copy on the "
                         "comm stream at a2a_ffn_overlap_degree 1 and 2 (to be traced with rocprofv3)")
    ap.add_argument("--cpu-stages", action="store_true",
                    help="instead of the JSON line, time the CPU oracle (one thread) stage by stage on bounded "
                         "samples of the same workloads; needs no GPU")
    ap.add_argument("--phases", action="store_true",
                    help="instead of the JSON line, print the phase stamps of the one-launch forward kernel and of its "
                         "ceiling kernel from the measurement build of the library")
    ap.add_argument("--only", default=None, help="with --kernels: only the lines whose 'name [config]' contains this, e.g. lz_ or [5]")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU's share of the path; --gpus %d is not supported "
                 "(nothing here uses a second GPU)" % args.gpus)
    if args.cpu_stages:
        import __graft_entry__
        __graft_entry__.ensure_built()
        cpu_stage_table()
        return
    if args.kernels or args.layer or args.overlap or args.phases:
        import __graft_entry__
        __graft_entry__.ensure_built()
        if args.phases:
            phase_table()
        elif args.kernels:
            kernel_table(args.only)
        elif args.layer:
            layer_table()
        else:
            overlap_run()
        return

    import __graft_entry__
    __graft_entry__.ensure_built()
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

    # the whole chain is one C-ABI call.  planmoe_forward_int8_single: one launch that reads x once
    # (the codes wait on chip until every work-group has published its expert histogram);
    # planmoe_forward_int8: two launches (gate + routing, then dispatch + int8), x read twice.
    # Outputs and workspace are allocated once.
    plan = ops.ForwardInt8Plan(xd, wd, k, C, fp32_gate=True, single=True)
    plan2 = ops.ForwardInt8Plan(xd, wd, k, C, fp32_gate=True, single=False)

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
    note = None
    if int(plan.gave_up) != 0:
        # what the layer does then: the pass again through the two launches (measured as the step, and said so)
        note = "a work-group of the one-launch kernel gave up waiting for the others: the step is planmoe_forward_int8 (two launches)"
        print("bench.py: " + note, file=sys.stderr)
        plan = plan2
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

    # algorithmic bytes: every input read once, every output written once
    chain_bytes = T * M * 2 + R * M + R * 2 * 2 + T * k * 12 + E * M * 2

    # device times (HIP events on the stream the kernels are launched on): the one-launch chain, the
    # two-launch chain and its two launches on their own
    chain_ev = event_time_us(chain, 30, 5)
    plan2.run()
    stages = {}
    stages["gate_route entry point (gate GEMM + routing; stand-alone it adds a small launch that finishes the slots)"] = event_time_us(
        lambda: ops.gate_route(xd, wd, k, fp32_gate=True), 30, 5)
    plan2.run()
    stages["dispatch_int8_routed (second launch of the two-launch chain, alone)"] = event_time_us(plan2.redispatch, 30, 5)
    chain2_ev = event_time_us(plan2.run, 30, 5)
    # the measuring stick: the chain's grid, loads, exchange and stores without its arithmetic (the
    # floor under this kernel's structure), and the same with nobody waiting at the exchange (the
    # floor under any arrangement of these loads and stores: what the dependency costs is the difference)
    # (a side measurement: whatever goes wrong with it leaves its fields empty, not the line unprinted)
    ceil_ev = {0: (None,), 1: (None,), 2: (None,)}
    try:
        ceiling = ops.ForwardCeiling(xd, E, k, C)
        got = {mode: event_time_us(lambda mode=mode: ceiling.run(mode), 30, 5) for mode in (0, 1, 2)}
        if int(ceiling.gave_up) == 0:
            ceil_ev = got
        else:
            print("bench.py: a work-group of the ceiling kernel gave up waiting for the others", file=sys.stderr)
    except Exception as ex:                                          # noqa: BLE001
        print("bench.py: the ceiling kernel was not measured: %s" % ex, file=sys.stderr)
    chain_ev_again = event_time_us(chain, 30, 5)
    frac_of_peak = lambda us: None if us is None else chain_bytes / us / 1e3 / HBM_PEAK_GBS

    # the chains with none of their operands in the L2s or the 256 MB memory-side cache: a reduction
    # over 1 GiB of other data before every call, one event pair per call, median of 9
    scrub = torch.zeros((1 << 28,), dtype=torch.int32, device=dev)

    def cold(fn):
        pairs = []
        for _ in range(9):
            torch.max(scrub)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            pairs.append((a, b))
        torch.cuda.synchronize()
        return sorted(a.elapsed_time(b) * 1e3 for a, b in pairs)[len(pairs) // 2]
    cold_us, cold2_us = cold(chain), cold(plan2.run)
    del scrub

    achieved = chain_bytes / chain_ev[0] / 1e3                     # GB/s, hot (back-to-back calls)
    traffic = profile_traffic_bytes()

    out = {
        "metric": "MoE dispatch/combine+int8 codec tokens/s; achieved HBM GB/s vs peak (1 GPU)",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "config 2: gate GEMM + softmax/top-2/capacity slots + dispatch fused with int8 "
                               "compress, forward", "tokens": T, "model_dim": M, "experts": E, "top_k": k,
                   "capacity_factor": cf, "capacity": C},
        # the whole chain (one launch) against its algorithmic bytes; hot = back-to-back calls on the
        # same buffers, cold = after a pass over 1 GiB of other data
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "kernel": "forward_single_kernel (the whole chain: planmoe_forward_int8_single, one launch)"
                               if note is None else "gate_route_kernel + dispatch_int8_routed_kernel (planmoe_forward_int8)",
                     "algorithmic_bytes": chain_bytes, "avg_us": chain_ev[0], "min_us": chain_ev[2],
                     "cold_us": cold_us, "cold_achieved": chain_bytes / cold_us / 1e3,
                     "cold_frac": chain_bytes / cold_us / 1e3 / HBM_PEAK_GBS,
                     "target_frac": 0.70, "target_met": achieved / HBM_PEAK_GBS >= 0.70,
                     # planmoe_forward_int8_single_ceiling in the same run: same grid, loads, exchange and
                     # stores, no arithmetic
                     "ceiling_us": ceil_ev[0][0], "ceiling_frac": frac_of_peak(ceil_ev[0][0]),
                     "ceiling_no_exchange_us": ceil_ev[1][0],
                     "ceiling_no_exchange_frac": frac_of_peak(ceil_ev[1][0]),
                     "ceiling_two_halves_us": ceil_ev[2][0],
                     "avg_us_after_ceilings": chain_ev_again[0]},
        "two_launch_chain": {"entry_point": "planmoe_forward_int8 (x read by both launches)",
                             "algorithmic_bytes": chain_bytes, "device_us_avg": chain2_ev[0],
                             "device_us_min": chain2_ev[2], "GBps": chain_bytes / chain2_ev[0] / 1e3,
                             "frac_of_hbm_peak": chain_bytes / chain2_ev[0] / 1e3 / HBM_PEAK_GBS,
                             "device_us_cold_caches": cold2_us,
                             "stage_us_avg": {n: v[0] for n, v in stages.items()}},
    }
    if note is not None:
        out["note"] = note
    if args.cpu_sample > 0:
        n = min(args.cpu_sample, T)
        v, dt, reps = cpu_baseline(n, M, E, k, cf, x, wg, args.cpu_seconds)
        out["cpu_baseline"] = {"value": v, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": "%d of the %d tokens x %d passes of the same chain on the host: torch-CPU ops "
                                         "(%d threads) for gate, softmax, top-k, one-hot, cumsum and the int8 chain, "
                                         "the single-threaded C loop for the dispatch (%.1f s)"
                                         % (n, T, reps, torch.get_num_threads(), dt),
                               "host_cores": os.cpu_count()}
        bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
        n1 = min(n, 4096)
        v1, dt1, reps1 = cpu_baseline_oracle(n1, M, E, k, cf, bits(x), bits(wg), min(args.cpu_seconds, 3.0))
        out["cpu_baseline"]["single_thread_oracle"] = {
            "value": v1, "unit": "tokens/s", "cores": 1,
            "sample": "%d tokens x %d passes through the scalar C oracle (%.1f s)" % (n1, reps1, dt1)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
