"""woq_hip_linear_noalloc (the entry point that takes no workspace and allocates nothing) against
woq_hip_linear on the same inputs: same kernels, so the outputs must be bit-identical.  Every case
makes two calls in a row, the second on a smaller input, through the C ABI."""
import pytest
import torch

from helpers import make_context
from oracle import woq_oracle as O

pytestmark = pytest.mark.gpu


def _run_both(ctx, x, **kw):
    from ipex_amd import _kernels, _lib

    N, K = ctx.weight_shape_
    args = (x, ctx.at_weight_, ctx.weight_dtype_, N, K, *ctx.scales_list_, ctx.zeros_u8_, ctx.group_size_,
            ctx.bias_f32_, ctx.lowp_mode_, ctx.act_quant_mode_)
    want = _kernels.linear(*args, scale_zero_f16x2=ctx.scale_zero_f16x2_, **kw)
    k_want = _lib.last_kernel()
    got = _kernels.linear(*args, scale_zero_f16x2=ctx.scale_zero_f16x2_, noalloc=True, **kw)
    k_got = _lib.last_kernel()
    torch.cuda.synchronize()
    assert k_got == k_want, (k_got, k_want)
    assert torch.equal(got, want), (k_got, float((got.float() - want.float()).abs().max()))
    return k_got


def _synthetic():
    from ipex_amd.utils import synthetic

    return synthetic


@pytest.mark.parametrize("mode", [6, 7, 2])
def test_noalloc_lowp_int8_quantized_activations_in_resident_scratch(cuda, mode):
    """lowp INT8: the quantized activations and their scales live in the resident array; a prefill-sized
    call, then a decode-sized one that reuses the front of the same array."""
    big = _synthetic().make_int4_case(51, 150, 1024, 272, 128, bias=True, outliers=True)
    ctx = make_context(big, O.LOWP_INT8, mode)
    assert _run_both(ctx, big["x"].cuda()) == "woq_gemm_w4i8_kernel"
    assert _run_both(ctx, big["x"][:5].cuda()) == "woq_decode_w4i8_kernel"
    # and the fp32 accumulators
    _run_both(ctx, big["x"][:33].cuda(), out_fp32=True)


def test_noalloc_split_k_decode_and_prefill(cuda):
    """Long K and few output columns: the workgroups that share K meet in the resident scratch (partial
    tiles and counters); second call smaller.  Repeated calls stay bit-identical and leave the counters
    at zero for the next one."""
    case = _synthetic().make_int4_case(52, 16, 8192, 512, 128, bias=True)
    ctx = make_context(case, O.LOWP_BF16)
    assert _run_both(ctx, case["x"].cuda()) == "woq_decode_dq_kernel"
    assert _run_both(ctx, case["x"][:7].cuda()) == "woq_decode_dq_kernel"
    for _ in range(20):
        _run_both(ctx, case["x"].cuda())
    # prefill GEMM with 64 x 128 tiles sharing K, floating point and lowp INT8
    case = _synthetic().make_int4_case(53, 128, 8192, 256, 128, bias=True, outliers=True)
    assert _run_both(make_context(case, O.LOWP_BF16), case["x"].cuda()) == "woq_gemm_w4_kernel"
    ctx8 = make_context(case, O.LOWP_INT8, 6)
    assert _run_both(ctx8, case["x"].cuda()) == "woq_gemm_w4i8_kernel"
    assert _run_both(ctx8, case["x"][:70].cuda()) == "woq_gemm_w4i8_kernel"


def test_noalloc_plain_calls_and_rejections(cuda):
    from ipex_amd import _kernels

    case = _synthetic().make_int4_case(54, 4, 1024, 512, 128)
    ctx = make_context(case, O.LOWP_BF16)
    assert _run_both(ctx, case["x"].cuda()) == "woq_decode_kernel"
    assert _run_both(ctx, case["x"][:1].cuda()) == "woq_decode_m1_kernel"
    # beyond the resident scratch: rejected before anything is launched
    N, K = 64, 4096
    big = _synthetic().make_int4_case(55, 1, K, N, 128)
    ctx8 = make_context(big, O.LOWP_INT8, 6)
    x = torch.zeros(4096, K, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="resident scratch holds"):
        _kernels.linear(x, ctx8.at_weight_, 2, N, K, *ctx8.scales_list_, ctx8.zeros_u8_, 128, None, O.LOWP_INT8, 6,
                        noalloc=True)
    # a caller-side workspace is refused: the entry point exists for callers that have none
    from ipex_amd import _lib
    import ctypes

    p = _lib.LinearParams()
    p.struct_size = ctypes.sizeof(_lib.LinearParams)
    p.M, p.K, p.N = 1, K, N
    p.workspace, p.workspace_bytes = x.data_ptr(), 1024
    assert _lib.load().woq_hip_linear_noalloc(ctypes.byref(p)) != 0
    assert b"must be null" in _lib.load().woq_hip_last_error()


def test_noalloc_calls_captured_into_a_graph_replay_like_eager(cuda):
    """What the entry point is for: a split-K call (counters re-zeroed by a fill kernel, partial tiles in the
    resident scratch) and a lowp INT8 call (quantized activations there) recorded into one HIP graph after a
    warm-up call outside the capture, replayed several times on new inputs with eager work in between; every
    replay equals the eager woq_hip_linear result bit for bit."""
    from ipex_amd import _kernels, _lib

    syn = _synthetic()
    split = syn.make_int4_case(56, 16, 8192, 512, 128, bias=True)
    int8 = syn.make_int4_case(57, 150, 1024, 272, 128, bias=True, outliers=True)
    ctxs = [make_context(split, O.LOWP_BF16), make_context(int8, O.LOWP_INT8, 6)]
    xs = [split["x"].cuda(), int8["x"].cuda()]
    static_x = [x.clone() for x in xs]

    def call(ctx, x, noalloc):
        N, K = ctx.weight_shape_
        return _kernels.linear(x, ctx.at_weight_, ctx.weight_dtype_, N, K, *ctx.scales_list_, ctx.zeros_u8_,
                               ctx.group_size_, ctx.bias_f32_, ctx.lowp_mode_, ctx.act_quant_mode_,
                               scale_zero_f16x2=ctx.scale_zero_f16x2_, scale_zero_bf16=ctx.scale_zero_bf16_, noalloc=noalloc)

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        kernels = []
        for ctx, x in zip(ctxs, static_x):  # the warm-up: the scratch address of this device is looked up here
            call(ctx, x, True)
            kernels.append(_lib.last_kernel())
    assert kernels == ["woq_decode_dq_kernel", "woq_gemm_w4i8_kernel"]
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        static_y = [call(ctx, x, True) for ctx, x in zip(ctxs, static_x)]
    gen = torch.Generator(device="cpu").manual_seed(3)
    for rep in range(4):
        for sx, x in zip(static_x, xs):
            sx.copy_((torch.randn(x.shape, generator=gen) * (1.0 + rep)).to(x.dtype))
        g.replay()
        torch.cuda.synchronize()
        got = [y.clone() for y in static_y]
        want = [call(ctx, x, False) for ctx, x in zip(ctxs, static_x)]  # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b), rep
