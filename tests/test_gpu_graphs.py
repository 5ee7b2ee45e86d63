"""Entry points recorded into a HIP graph and replayed: every replay, with new input values and
with eager work and synchronisations in between, must give what the eager call gives.  (None of
the entry points allocates or records a memset node; clearing is done by fill kernels.)"""
import numpy as np
import pytest
import torch

from planmoe_amd import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def replay_against_eager(make_inputs, run, outputs_of, rounds=3):
    """run(inputs) -> result object; outputs_of(result) -> list of tensors to compare."""
    static = make_inputs(0)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):                      # warm-up outside the capture
        for _ in range(2):
            run(static)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        held = run(static)
    for r in range(1, rounds + 1):
        fresh = make_inputs(r)
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outputs_of(held)]
        want = outputs_of(run(fresh))                  # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a.view(torch.uint8).reshape(-1), b.view(torch.uint8).reshape(-1)), r


def test_forward_chain_replays():
    T, M, E, k = 2048, 512, 8, 2
    C = ops.capacity(T, E, k, 1.25, 4)

    def make(seed):
        g = torch.Generator().manual_seed(seed)
        return [torch.randn(T, M, generator=g).bfloat16().to(DEV),
                (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)]

    def run(inp):
        return ops.forward_int8(inp[0], inp[1], k, C, want_counts=True)

    replay_against_eager(make, run, lambda o: [o["indices"], o["locations"], o["gates"], o["codes"], o["bias"],
                                               o["scale"], o["counts"], o["l_aux"].reshape(1)])


def test_forward_plain_and_the_expert_gemms_replay():
    T, M, E, k, H = 1024, 256, 4, 2, 128
    C = ops.capacity(T, E, k, 1.0, 4)                  # 512: a multiple of 64, so dW takes the direct form

    def make(seed):
        g = torch.Generator().manual_seed(20 + seed)
        return [torch.randn(T, M, generator=g).bfloat16().to(DEV),
                (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV),
                (torch.randn(E, M, H, generator=g) * M ** -0.5).bfloat16().to(DEV),
                torch.randn(E, H, generator=g).bfloat16().to(DEV)]

    def run(inp):
        out = ops.forward_plain(inp[0], inp[1], k, C, want_counts=True)
        d = out["dispatched"].view(E, C, M)
        h = ops.gemm_nn_bf16(d, inp[2], inp[3], relu=True)                       # [E, C, H]
        dw = ops.gemm_tn_bf16(d, h)                                              # [E, M, H]
        dx = ops.gemm_nt_bf16(h, inp[2])                                         # [E, C, M]
        return out, h, dw, dx

    replay_against_eager(make, run, lambda r: [r[0]["indices"], r[0]["locations"], r[0]["gates"], r[0]["dispatched"],
                                               r[0]["counts"], r[0]["l_aux"].reshape(1), r[1], r[2], r[3]])


def test_routing_and_sparse_kernels_replay():
    T, M, E, k = 1500, 256, 16, 2
    C = ops.capacity(T, E, k, 1.0, 4)

    def make(seed):
        g = torch.Generator().manual_seed(10 + seed)
        return [torch.randn(T, E, generator=g).to(DEV), torch.randn(T, M, generator=g).to(DEV)]

    def run(inp):
        r = ops.route_topk(inp[0], k, is_logits=True, want_counts=True)
        idx, loc, gates = list(r["indices"]), list(r["locations"]), list(r["gates"])
        d = ops.dispatch_fwd(inp[1], idx, loc, None, E, C)
        y = ops.combine_fwd(d, idx, loc, gates, T, C)
        codes, bias, scale = ops.dispatch_int8(inp[1], idx, loc, None, E, C)
        return [r["indices"], r["locations"], r["gates"], r["counts"], d, y, codes, bias, scale]

    replay_against_eager(make, run, lambda o: o)


def test_zfp_and_lz_entry_points_replay():
    T, M, E, k = 1024, 128, 8, 2
    C = ops.capacity(T, E, k, 1.0, 4)
    scores = torch.softmax(torch.randn(T, E, generator=torch.Generator().manual_seed(3)), 1).to(DEV)
    r = ops.route_topk(scores, k)
    idx, loc, gates = list(r["indices"]), list(r["locations"]), [g.float() for g in r["gates"]]

    def make(seed):
        g = torch.Generator().manual_seed(20 + seed)
        x = torch.randn(T, M, generator=g)
        x[torch.rand(T, generator=g) < 0.3] = 0.0
        return [x.to(DEV)]

    def run(inp):
        stream = ops.dispatch_zfp(inp[0], idx, loc, None, E, C)
        y = ops.combine_zfp(stream, idx, loc, gates, T, E, C, M)
        gg = ops.bwd_gate_zfp(stream, inp[0], idx, loc, E, C)
        lz = ops.lz_compress(inp[0])
        back = torch.empty_like(inp[0])
        ops.lz_decompress(back, *lz)
        return [stream, y, gg.contiguous(), *lz, back]

    replay_against_eager(make, run, lambda o: o)


def test_forward_chain_on_two_streams_at_once():
    """The chain keeps its routing state in a cached workspace: calls issued on two streams must not
    share it.  Two different batches, enqueued alternately on two streams without waiting, against
    the same calls made one after the other."""
    T, M, E, k = 4096, 512, 8, 2
    C = ops.capacity(T, E, k, 1.25, 4)
    g = torch.Generator().manual_seed(3)
    xs = [torch.randn(T, M, generator=g).bfloat16().to(DEV) for _ in range(2)]
    wg = (torch.randn(E, M, generator=g) * M ** -0.5).bfloat16().to(DEV)
    want = [ops.forward_int8(x, wg, k, C) for x in xs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [None, None]
    for _ in range(5):
        for i in (0, 1):
            with torch.cuda.stream(streams[i]):
                got[i] = ops.forward_int8(xs[i], wg, k, C)
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        for name in ("indices", "locations", "codes", "bias", "scale"):
            assert torch.equal(a[name].view(torch.uint8).reshape(-1), b[name].view(torch.uint8).reshape(-1)), name

