"""HIP graph capture of the ops: no entry point allocates, synchronises or records a memset, so a
captured sequence must replay to the same bits as eager execution, replay after replay, with eager
work and synchronisation in between."""
import pytest
import torch

from helpers import E4

pytestmark = pytest.mark.gpu
ops = torch.ops.hpu


def pipeline(x, w8, sw_inv):
    x8, sx_inv = torch.ops.mi355q.quantize_rows(x, E4)
    y = ops.fp8_gemm_v2(x8, False, w8, False, None, torch.bfloat16, sx_inv, sw_inv, None, False, [1, w8.shape[1]])
    y8, amax = ops.cast_to_fp8_v2(y, None, False, True, E4)          # amax: fill kernel + atomics inside the graph
    back = ops.cast_from_fp8(y8, None, torch.bfloat16)
    return y, y8, amax, back


def test_graph_replays_match_eager(dev):
    g = torch.Generator().manual_seed(12)
    M, K, N = 192, 512, 384
    w = (torch.randn(K, N, generator=g) * 0.05).bfloat16().to(dev)
    sw = 448.0 / w.abs().amax(dim=0).float()
    w8 = ops.cast_to_fp8_v2(w, sw, False, False, E4, [1, N])[0]
    sw_inv = (1.0 / sw).contiguous()
    x = torch.randn(M, K, generator=g).bfloat16().to(dev)
    static_x = x.clone()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # warm-up on the capture stream, as torch's graph recipe asks
        for _ in range(3):
            pipeline(static_x, w8, sw_inv)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = pipeline(static_x, w8, sw_inv)

    for rep in range(4):
        xin = torch.randn(M, K, generator=g).bfloat16().to(dev) * (rep + 1)
        static_x.copy_(xin)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        ref = pipeline(xin, w8, sw_inv)     # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, ref):
            assert torch.equal(a.view(torch.uint8) if a.dtype == E4 else a, b.view(torch.uint8) if b.dtype == E4 else b), rep


def test_graph_replays_of_a_ragged_product(dev):
    """A large product with ragged extents: the operator's zero-padded operand copies (torch's
    allocator, a fill kernel and a copy kernel) are part of the captured sequence."""
    g = torch.Generator().manual_seed(3)
    M, K, N = 333, 1001, 515
    w8 = torch.randint(-4, 5, (K, N), generator=g).float().to(E4).to(dev)
    static_a = torch.zeros(M, K, dtype=E4, device=dev)
    run = lambda a: ops.fp8_gemm_v2(a, False, w8, False, None, torch.float32)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            run(static_a)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = run(static_a)
    for rep in range(4):
        a = torch.randint(-4, 5, (M, K), generator=g).float()
        static_a.copy_(a.to(E4))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager = run(a.to(E4).to(dev))       # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, eager) and torch.equal(got.cpu(), a @ w8.cpu().float()), rep


def attention_like(q8, k8, sq, sk):
    """scores = q k^T in fp8, probabilities through softmax_fp8, their row sums through sum_fp8 (split: workspace)."""
    scores = ops.fp8_gemm_v2(q8, False, k8, True, None, torch.bfloat16, sq, sk, None, False)
    p8 = ops.softmax_fp8(scores, -1, 0.125, 256.0, None)
    return scores, p8, ops.sum_fp8(p8, [0, 1], False, torch.float), ops.sum_fp8(p8, [2], False, torch.bfloat16)


def test_graph_replays_of_the_reductions(dev):
    g = torch.Generator().manual_seed(13)
    B, L, D = 4, 256, 128
    k8 = torch.randn(B, L, D, generator=g).to(E4).to(dev)
    sq, sk = torch.tensor(0.5, device=dev), torch.tensor(0.25, device=dev)
    static_q = torch.randn(B, L, D, generator=g).to(E4).to(dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            attention_like(static_q, k8, sq, sk)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = attention_like(static_q, k8, sq, sk)
    for rep in range(4):
        q = (torch.randn(B, L, D, generator=g) * (rep + 1)).to(E4).to(dev)
        static_q.copy_(q)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        ref = attention_like(q, k8, sq, sk)
        torch.cuda.synchronize()
        for a, b in zip(got, ref):
            assert torch.equal(a.view(torch.uint8) if a.dtype == E4 else a, b.view(torch.uint8) if b.dtype == E4 else b), rep


def decode_step(q, k, v, x8, pk, s, z):
    """Attention for one query per head against a long cache (the keys split over workgroups, which meet through
    arrival counters in a workspace), a W4A8 product and a W4A16 product on the same weights (K split over
    workgroups, which meet the same way)."""
    o = ops.fp8_sdpa_recomp_fwd(q, k, v, None, 0.0, 128 ** -0.5, False, False, "None", None, None, None, None, None, None,
                                False, False, None, "left")[0]
    y = torch.ops.mi355q.w4a8_gemm(x8, pk, s, z, False, torch.bfloat16, None, None)
    y16 = torch.ops.mi355q.w4a16_gemm(x8.to(torch.bfloat16), pk, s, z, False, torch.bfloat16, None)
    return o, y, y16


def test_graph_replays_of_a_decode_step(dev):
    """The counters of the key split and of the W4A8 product's split over K live in a tensor of the graph's own while
    capturing (cleared by a fill kernel of the graph, so every replay starts from zero) and in the stream's kept
    workspace in eager runs: same bits either way, replay after replay, with eager calls in between."""
    g = torch.Generator().manual_seed(14)
    B, G, HG, S, D = 1, 2, 4, 4096, 128
    k = torch.randn(B, G, 1, S, D, generator=g).to(E4).to(dev)
    v = torch.randn(B, G, 1, S, D, generator=g).to(E4).to(dev)
    K, N = 4096, 512
    pk = torch.randint(-2 ** 31, 2 ** 31 - 1, (K, N // 8), generator=g, dtype=torch.int64).to(torch.int32).to(dev)
    s = (torch.rand(K // 128, N, generator=g) * 0.019 + 0.001).bfloat16().to(dev)
    z = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 128, N // 8), generator=g, dtype=torch.int64).to(torch.int32).to(dev)
    static_q = torch.randn(B, G, HG, 1, D, generator=g).to(E4).to(dev)
    static_x = torch.randn(8, K, generator=g).to(E4).to(dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            decode_step(static_q, k, v, static_x, pk, s, z)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = decode_step(static_q, k, v, static_x, pk, s, z)
    for rep in range(4):
        q = (torch.randn(B, G, HG, 1, D, generator=g) * (rep + 1)).to(E4).to(dev)
        x = torch.randn(8, K, generator=g).to(E4).to(dev)
        static_q.copy_(q)
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        ref = decode_step(q, k, v, x, pk, s, z)
        torch.cuda.synchronize()
        assert torch.equal(got[0], ref[0]), rep
        assert torch.equal(got[1], ref[1]), rep   # the same kernel and the same split over K, captured or not
        assert torch.equal(got[2], ref[2]), rep


def test_ops_follow_the_current_stream(oracle, dev):
    """Work is enqueued on torch's current stream (as the reference uses the current HPUStream,
    habana_eager/eager_exec.cpp:341), not on the default one: results are right when the inputs were
    produced on a side stream and nothing synchronises in between."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(512, 1024, generator=g).bfloat16()
    s = torch.tensor(2.5)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        xd = x.to(dev, non_blocking=True) * 1.0       # produced on the side stream
        y, amax = ops.cast_to_fp8_v2(xd, s.to(dev), False, True, E4)
        back = ops.cast_from_fp8(y, None, torch.bfloat16)
    side.synchronize()
    ref, ref_amax = oracle.c_cast_to_fp8(x, s, E4, True)
    assert torch.equal(y.cpu().view(torch.uint8), ref.view(torch.uint8))
    assert amax.cpu() == ref_amax
    assert torch.equal(back.cpu().float(), ref.float())
