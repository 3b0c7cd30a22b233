"""Shared test plumbing: numpy views of a synthetic case, error metrics."""
import numpy as np
import torch


def to_np_f32(t):
    return t.detach().float().cpu().numpy()


def case_np(case):
    """Numpy view of a case from ipex_amd.utils.synthetic for the oracle."""
    return dict(
        x=to_np_f32(case["x"]),
        qw=(case["qweight"].view(torch.uint8) if case["qweight"].dtype == torch.float8_e4m3fn else case["qweight"])
        .cpu()
        .numpy(),
        scales=to_np_f32(case["scales"]),
        zps=None if case["zeros"] is None else to_np_f32(case["zeros"]),
        bias=None if case["bias"] is None else to_np_f32(case["bias"]),
    )


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def max_abs(a, b):
    return float(np.max(np.abs(np.asarray(a, dtype=np.float64) - np.asarray(b, dtype=np.float64))))


def bf16_ulp_diff(a, b):
    """|difference| in bf16 ulps between two float32 arrays holding bf16 values."""
    ia = (np.asarray(a, dtype=np.float32).view(np.uint32) >> 16).astype(np.int64)
    ib = (np.asarray(b, dtype=np.float32).view(np.uint32) >> 16).astype(np.int64)
    # map sign-magnitude to a monotone integer line
    ia = np.where(ia & 0x8000, 0x8000 - ia, ia)
    ib = np.where(ib & 0x8000, 0x8000 - ib, ib)
    return np.abs(ia - ib)


def make_context(case, lowp_mode, act_quant_mode=-1, device="cuda", cache=False):
    from ipex_amd import ops

    return ops.WoqLinearOpContext(
        case["qweight"].to(device),
        case["weight_dtype"],
        [case["N"], case["K"]],
        case["scales"].to(device),
        None if case["zeros"] is None else case["zeros"].to(device),
        None if case["bias"] is None else case["bias"].to(device),
        None,
        None,
        case["group_size"],
        lowp_mode,
        act_quant_mode,
        cache,
    )


def make_torch_context(case, lowp_mode, act_quant_mode=-1, device="cuda", cache=False, g_idx=None):
    """The registered custom class (torch.classes.ipex_prepack.WoqLinearOpContext) for a synthetic case,
    made by the registered prepack operator."""
    import torch
    import ipex_amd  # noqa: F401

    return torch.ops.ipex_prepack.weight_only_qlinear_prepack(
        case["qweight"].to(device),
        case["weight_dtype"],
        [case["N"], case["K"]],
        case["scales"].to(device),
        None if case["zeros"] is None else case["zeros"].to(device),
        None if case["bias"] is None else case["bias"].to(device),
        g_idx,
        None,
        case["group_size"],
        lowp_mode,
        act_quant_mode,
        cache,
    )
