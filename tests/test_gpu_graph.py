"""HIP-graph capture of the WOQ linear: every kernel family recorded once and replayed, each replay
checked against the eager result (the kernels are deterministic, so bit for bit), with eager work
and synchronizations between the replays."""
import pytest
import torch

from helpers import make_context

pytestmark = pytest.mark.gpu


def _synthetic():
    from ipex_amd.utils import synthetic

    return synthetic


# (label, M, K, N, G, lowp_mode, act_quant_mode[, cache_weight_for_large_batch])
CASES = [
    ("fp16-regime decode kernel", 1, 1024, 256, 128, 2, -1),
    ("dequantizing decode kernel", 16, 1024, 256, 32, 2, -1),
    ("dequantizing decode kernel, K shared by two workgroups", 16, 8192, 512, 128, 2, -1),
    ("4-bit prefill GEMM", 200, 1024, 512, 128, 2, -1),
    ("lowp INT8 prefill, scales per row", 200, 1024, 512, 128, 3, 6),
    ("lowp INT8 prefill, scales per row and K block", 130, 1024, 256, 128, 3, 7),
    ("lowp INT8 small batch", 8, 1024, 256, 128, 3, 6),
    ("prefill GEMM on the dense copy of the weight cache", 1536, 512, 7168, 128, 2, -1, True),
]


def test_graph_replays_match_eager(cuda):
    syn = _synthetic()
    ctxs, xs = [], []
    for i, (_, M, K, N, G, lowp, aq, *cache) in enumerate(CASES):
        case = syn.make_int4_case(60 + i, M, K, N, G, bias=(i % 2 == 0))
        ctxs.append(make_context(case, lowp, aq, cache=bool(cache)))
        xs.append(case["x"].cuda())
    static_x = [x.clone() for x in xs]

    def run_all():
        return [ctx.run(x) for ctx, x in zip(ctxs, static_x)]

    # warm-up on the capture stream (allocations of the op layer, e.g. the split-K counters)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        run_all()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    from ipex_amd import _lib
    assert _lib.last_kernel() == "woq_gemm_dense_kernel"  # the last case runs on the copy

    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        static_y = run_all()

    gen = torch.Generator(device="cpu").manual_seed(7)
    for rep in range(4):
        for sx, x in zip(static_x, xs):
            sx.copy_((torch.randn(x.shape, generator=gen) * (1.0 + rep)).to(x.dtype))
        g.replay()
        torch.cuda.synchronize()
        got = [y.clone() for y in static_y]
        # eager work between the replays, on the same inputs
        want = run_all()
        torch.cuda.synchronize()
        for (label, *_), a, b in zip(CASES, got, want):
            assert torch.equal(a, b), (label, rep)
        assert all(bool(torch.isfinite(y.float()).all()) for y in got)


def test_moe_layer_graph_replays_with_new_routing(cuda):
    """deepseek_moe_woq with its routing sorted on the device, captured once: the replays see new hidden states, new
    expert ids and new routing weights (written into the captured tensors) and must equal the eager results -- the
    captured launches have no shape that depends on the routing."""
    import ipex_amd  # noqa: F401
    from ipex_amd import _lib
    from test_gpu_module import _woq_module

    E, H, I, T, topk = 8, 256, 384, 6, 3
    mk = lambda k, n, s: _woq_module(ipex_amd, k, n, "INT4", 64, "BF16", bias=False, seed=s)._op_context
    gate, up, down = [mk(H, I, 700 + e) for e in range(E)], [mk(H, I, 720 + e) for e in range(E)], [mk(I, H, 740 + e) for e in range(E)]
    op = torch.ops.torch_ipex.deepseek_moe_woq
    gen = torch.Generator().manual_seed(3)

    def draw():
        hidden = torch.randn(T, H, generator=gen).to(torch.bfloat16)
        ids = torch.stack([torch.randperm(E, generator=gen)[:topk] for _ in range(T)])
        rw = torch.softmax(torch.randn(T, topk, generator=gen), -1).to(torch.bfloat16)
        return hidden, ids, rw

    static = [t.cuda() for t in draw()]
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        op(static[0], static[1], gate, up, down, static[2], False)  # builds the layer's pointer tables and buffers
        assert _lib.last_kernel() == "moe_combine_rows"
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        static_out = op(static[0], static[1], gate, up, down, static[2], False)
    for rep in range(4):
        new = draw()
        if rep == 2:
            new[1][:, 0] = 5  # every token to expert 5: one expert with six rows, the others with few or none
        for dst, src in zip(static, new):
            dst.copy_(src)
        g.replay()
        torch.cuda.synchronize()
        got = static_out.clone()
        want = op(*[t.cuda() for t in new[:2]], gate, up, down, new[2].cuda(), False)
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep
