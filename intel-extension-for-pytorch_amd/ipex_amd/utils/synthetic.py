"""Seeded synthetic inputs of the benchmark configurations (weights as a quantized checkpoint
would hold them: packed nibbles or int8, scales, zero points).  Everything is generated on the
CPU from ``torch.Generator().manual_seed(1000 * config + tensor_index)`` so that the GPU run and
the CPU checker see identical bits.
"""
import torch


def _gen(cfg, idx):
    return torch.Generator().manual_seed(1000 * cfg + idx)


def make_int4_case(cfg, M, K, N, group_size, outliers=False, bias=False, scale_dtype=torch.bfloat16):
    """bf16 activations ~ N(0,1) (optionally 1% of entries x20), uint4 weights uniform in 0..15
    packed two per byte along K, scales uniform in [0.005, 0.02] rounded to ``scale_dtype``,
    uint4 zero points per (N, K / group_size)."""
    x = torch.randn(M, K, generator=_gen(cfg, 0))
    if outliers:
        mask = torch.rand(M, K, generator=_gen(cfg, 5)) < 0.01
        x = torch.where(mask, x * 20, x)
    x = x.to(torch.bfloat16)
    q = torch.randint(0, 16, (N, K), dtype=torch.uint8, generator=_gen(cfg, 1))
    qweight = (q[:, 1::2] << 4).bitwise_or(q[:, ::2]).contiguous()
    KG = (K + group_size - 1) // group_size if group_size > 0 else 1
    scales = (0.005 + 0.015 * torch.rand(N, KG, generator=_gen(cfg, 2))).to(scale_dtype).float()
    zeros = torch.randint(0, 16, (N, KG), generator=_gen(cfg, 3)).float()
    if group_size <= 0:
        scales, zeros = scales.reshape(N), zeros.reshape(N)
    b = (0.02 * torch.randn(N, generator=_gen(cfg, 4))).to(torch.bfloat16) if bias else None
    return dict(x=x, qweight=qweight, scales=scales, zeros=zeros, bias=b, M=M, K=K, N=N,
                group_size=group_size, weight_dtype=2)


def make_nf4_case(cfg, M, K, N, group_size, bias=False, scale_dtype=torch.bfloat16):
    """NF4 weights: codes uniform in 0..15 packed like int4, absmax scales uniform in [0.02, 0.08],
    no zero points."""
    case = make_int4_case(cfg, M, K, N, group_size, bias=bias, scale_dtype=scale_dtype)
    case["scales"] = (case["scales"] * 4).to(scale_dtype).float()
    case["zeros"] = None
    case["weight_dtype"] = 3
    return case


def make_int8_case(cfg, M, K, N, bias=True, group_size=-1):
    """Symmetric int8 weights uniform in -127..127, fp32 scales uniform in [0.001, 0.01] per output
    channel (or per group of ``group_size`` input channels), bf16 bias ~ N(0, 0.02)."""
    x = torch.randn(M, K, generator=_gen(cfg, 0)).to(torch.bfloat16)
    qweight = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=_gen(cfg, 1))
    shape = (N,) if group_size <= 0 else (N, (K + group_size - 1) // group_size)
    scales = 0.001 + 0.009 * torch.rand(shape, generator=_gen(cfg, 2))
    b = (0.02 * torch.randn(N, generator=_gen(cfg, 4))).to(torch.bfloat16) if bias else None
    return dict(x=x, qweight=qweight, scales=scales, zeros=None, bias=b, M=M, K=K, N=N,
                group_size=group_size, weight_dtype=1)


def make_fp8_case(cfg, M, K, N, bias=True, group_size=-1, x_dtype=torch.bfloat16):
    """float8 e4m3fn weights: every byte except the two NaN codes, uniform (so all exponents and the
    subnormals occur), fp32 scales uniform in [0.0005, 0.002] per output channel (or per group of
    ``group_size`` input channels), no zero points, bias ~ N(0, 0.02)."""
    x = torch.randn(M, K, generator=_gen(cfg, 0)).to(x_dtype)
    code = torch.randint(0, 254, (N, K), dtype=torch.int16, generator=_gen(cfg, 1))
    code = code + (code >= 0x7F).to(torch.int16)  # skips 0x7F; 0xFF is out of range
    qweight = code.to(torch.uint8).view(torch.float8_e4m3fn)
    shape = (N,) if group_size <= 0 else (N, (K + group_size - 1) // group_size)
    scales = 0.0005 + 0.0015 * torch.rand(shape, generator=_gen(cfg, 2))
    b = (0.02 * torch.randn(N, generator=_gen(cfg, 4))).to(x_dtype) if bias else None
    return dict(x=x, qweight=qweight, scales=scales, zeros=None, bias=b, M=M, K=K, N=N,
                group_size=group_size, weight_dtype=4)
