"""Weight quantization / dequantization helpers: they define the checkpoint format the
kernels consume.

Format (same as the reference, intel_extension_for_pytorch/quantization/_quantize_utils.py:864-1290):
  * INT4 / NF4: values 0..15, two per byte along K, element 2j in the low nibble of byte j and
    2j+1 in the high nibble; odd K is padded with one zero element.  Symmetric INT4 is stored
    shifted by +8.
  * INT8: int8, one per byte.
  * scales, zero points: fp32 [N] (per channel) or [N, ceil(K / group_size)] (per block);
    dequantized weight = (q - zero_point) * scale.
"""
from typing import Optional

import torch

from ._qconfig import WoqWeightDtype

NF4_QUANT_TABLE = [
    -1.0 - 1e-2,
    -0.8480964004993439,
    -0.6106329262256622,
    -0.4599952697753906,
    -0.33967943489551544,
    -0.23460740596055984,
    -0.13791173323988914,
    -0.045525018125772476,
    0.03979014977812767,
    0.1202552504837513,
    0.2035212516784668,
    0.2920137718319893,
    0.3893125355243683,
    0.5016634166240692,
    0.6427869200706482,
    0.8614784181118011,
]

NF4_DEQUANT_TABLE = [
    -1.0,
    -0.6961928009986877,
    -0.5250730514526367,
    -0.39491748809814453,
    -0.28444138169288635,
    -0.18477343022823334,
    -0.09105003625154495,
    0.0,
    0.07958029955625534,
    0.16093020141124725,
    0.24611230194568634,
    0.33791524171829224,
    0.44070982933044434,
    0.5626170039176941,
    0.7229568362236023,
    1.0,
]

NF4_TO_INT8_TABLE = [round(x * 127) for x in NF4_DEQUANT_TABLE]


def map_float_tensor_to_nf4(t, dtype=torch.uint8):
    """Values in [-1, 1] -> NF4 code: the largest i with t > NF4_QUANT_TABLE[i]."""
    out = torch.empty(t.shape, dtype=dtype, device=t.device)
    for i, edge in enumerate(NF4_QUANT_TABLE):
        out[t > edge] = i
    return out


def map_nf4_tensor_to_float(t, dtype=torch.float32):
    lut = torch.tensor(NF4_DEQUANT_TABLE, dtype=dtype, device=t.device)
    return lut[t.long()]


def map_nf4_tensor_to_int8(t, dtype=torch.float32):
    lut = torch.tensor(NF4_TO_INT8_TABLE, dtype=dtype, device=t.device)
    return lut[t.long()]


def is_4bit(dtype):
    return dtype in (WoqWeightDtype.INT4, WoqWeightDtype.NF4)


def is_sym_quant(dtype):
    return dtype in (WoqWeightDtype.NF4,)


def pack_nibbles(q):
    """uint8 values 0..15, [N, K] -> [N, ceil(K/2)] with the even element in the low nibble."""
    if q.size(-1) % 2:
        q = torch.nn.functional.pad(q, (0, 1), value=0)
    return (q[:, 1::2] << 4).bitwise_or(q[:, ::2].bitwise_and(0xF)).contiguous()


def unpack_nibbles(qt):
    """[N, Kb] bytes -> [N, 2 * Kb] uint8 values 0..15."""
    out = torch.empty(qt.shape[0], qt.shape[1] * 2, dtype=torch.uint8, device=qt.device)
    out[:, ::2] = qt.bitwise_and(0xF)
    out[:, 1::2] = qt.bitwise_right_shift(4)
    return out


def _qparams_from_minmax(mins, maxs, dtype, sym_quant):
    """Scale / zero point of one reduction (per row or per group) from its min and max, both
    already widened to include 0."""
    eps = torch.tensor([torch.finfo(torch.float32).eps], device=mins.device)
    zps = None
    absmax = torch.maximum(torch.abs(maxs), torch.abs(mins))
    if dtype == WoqWeightDtype.INT8:
        if sym_quant:
            scales = torch.max(absmax / 127, eps)
        else:
            scales = torch.max((maxs - mins) / 255, eps)
            zps = -torch.round(mins / scales) - 128
    elif dtype == WoqWeightDtype.INT4:
        if sym_quant:
            scales = torch.max(absmax / 7, eps)
        else:
            scales = torch.max((maxs - mins) / 15, eps)
            zps = -torch.round(mins / scales)
    else:  # NF4
        scales = torch.max(absmax, eps)
    return scales, zps


def _quantize_values(t, inv_scales, zps, dtype, sym_quant):
    """t * inv_scales (+ zero point), rounded and clamped to the storage range.  The
    multiplication by the reciprocal (rather than a division) is part of the format."""
    if dtype == WoqWeightDtype.INT8:
        shift = zps if zps is not None else 0
        return torch.clamp(torch.round(t * inv_scales) + shift, min=-128, max=127)
    if dtype == WoqWeightDtype.INT4:
        shift = zps if not sym_quant else 8
        return torch.clamp(torch.round(t * inv_scales) + shift, min=0, max=15)
    return map_float_tensor_to_nf4(t * inv_scales)


def quantize_per_channel(t: torch.Tensor, dtype, scales=None, zero_points=None, sym_quant=False):
    """Quantizes a [N, K] weight with one (scale, zero point) per output channel.

    Returns (qweight, scales [N], zero_points [N] or None)."""
    assert t.ndim == 2
    assert dtype in (WoqWeightDtype.INT8, WoqWeightDtype.INT4, WoqWeightDtype.NF4)
    assert not (dtype == WoqWeightDtype.NF4 and not sym_quant), "NF4 must be symmetric quant"
    if not (scales is not None and (sym_quant or zero_points is not None)):
        zero = torch.zeros(t.shape[0], dtype=t.dtype, device=t.device)
        mins = torch.minimum(t.min(dim=1)[0], zero)
        maxs = torch.maximum(t.max(dim=1)[0], zero)
        scales, zero_points = _qparams_from_minmax(mins, maxs, dtype, sym_quant)
    inv = 1 / scales.unsqueeze(1)
    zp = zero_points.unsqueeze(1) if zero_points is not None else None
    qt = _quantize_values(t, inv, zp, dtype, sym_quant)
    if dtype == WoqWeightDtype.INT8:
        return qt.to(torch.int8).contiguous(), scales, zero_points
    return pack_nibbles(qt.to(torch.uint8)), scales, zero_points


def quantize_per_block(input: torch.Tensor, dtype, group_size, scales=None, zero_points=None, sym_quant=False):
    """Quantizes a [N, K] weight in blocks of [1, group_size]; a trailing partial block gets its
    own parameters.  Returns (qweight, scales [N, Kc], zero_points [N, Kc] or None)."""
    assert input.dim() == 2, f"{__name__}: Expect input has 2 dimensions but got {input.dim()}"
    assert group_size > 0, f"{__name__}: Expect group_size > 0 but got {group_size}"
    assert dtype in (WoqWeightDtype.INT8, WoqWeightDtype.INT4, WoqWeightDtype.NF4)
    assert not (dtype == WoqWeightDtype.NF4 and not sym_quant), "NF4 must be symmetric quant"
    N, K = input.shape
    k_rem = K % group_size
    k_com = K - k_rem
    n_full = k_com // group_size
    body = input[:, :k_com].view(N, n_full, group_size)
    tail = input[:, k_com:].view(N, 1, k_rem) if k_rem else None

    if not (scales is not None and (sym_quant or zero_points is not None)):
        zero = torch.tensor([0], device=input.device)

        def minmax_params(blocks):
            mins = torch.minimum(blocks.min(dim=-1)[0], zero)
            maxs = torch.maximum(blocks.max(dim=-1)[0], zero)
            return _qparams_from_minmax(mins, maxs, dtype, sym_quant)

        scales, zero_points = minmax_params(body)
        if tail is not None:
            s_tail, z_tail = minmax_params(tail)
            scales = torch.cat([scales, s_tail], dim=-1)
            if not sym_quant:
                zero_points = torch.cat([zero_points, z_tail], dim=-1)

    def quant(blocks, s, z):
        zp = z.unsqueeze(-1) if z is not None else None
        return _quantize_values(blocks, 1 / s.unsqueeze(-1), zp, dtype, sym_quant)

    z_body = zero_points[:, :n_full] if not sym_quant else None
    qt = quant(body, scales[:, :n_full], z_body).view(N, k_com)
    if tail is not None:
        z_tail = zero_points[:, n_full:] if not sym_quant else None
        qt_tail = quant(tail, scales[:, n_full:], z_tail).view(N, k_rem)
        qt = torch.cat([qt, qt_tail], dim=1).contiguous()
    if is_4bit(dtype):
        return pack_nibbles(qt.to(torch.uint8).view(N, K)), scales, zero_points
    return qt.to(torch.int8).view(N, K).contiguous(), scales, zero_points


def _codes_to_float(qt, dtype, dequant_nf4_via_int8):
    if dtype == WoqWeightDtype.NF4:
        if dequant_nf4_via_int8:
            return map_nf4_tensor_to_int8(qt) / 127.0
        return map_nf4_tensor_to_float(qt)
    return qt.to(torch.float)


def dequantize_per_channel(
    qt: torch.Tensor, scales, zps: Optional[torch.Tensor], dtype, weight_shape=None, dequant_nf4_via_int8=False
):
    """Inverse of quantize_per_channel: (q - zero_point) * scale, fp32 [N, K]."""
    assert qt.ndim == 2
    assert dtype in (WoqWeightDtype.INT8, WoqWeightDtype.INT4, WoqWeightDtype.NF4)
    scales = scales.squeeze()
    if zps is None:
        zps = torch.zeros_like(scales)
        if dtype == WoqWeightDtype.INT4:
            zps += 8  # stored range [0, 15] stands for [-8, 7]
    else:
        zps = zps.squeeze()
    if is_4bit(dtype):
        qt = unpack_nibbles(qt)
    if dtype == WoqWeightDtype.NF4:
        t = _codes_to_float(qt, dtype, dequant_nf4_via_int8)
        if weight_shape is not None:
            t = t[: weight_shape[0], : weight_shape[1]].contiguous()
        return t * scales.unsqueeze(-1)
    t = (qt.to(torch.float) - zps.unsqueeze(-1)) * scales.unsqueeze(-1)
    if weight_shape is not None and is_4bit(dtype):
        t = t[: weight_shape[0], : weight_shape[1]].contiguous()
    return t


def dequantize_per_block(
    qt: torch.Tensor,
    scales,
    zps: Optional[torch.Tensor],
    dtype,
    group_size,
    weight_shape=None,
    dequant_nf4_via_int8=False,
):
    """Inverse of quantize_per_block: (q - zero_point) * scale per [1, group_size] block."""
    N = qt.size(0)
    K = qt.size(1) * 2 if is_4bit(dtype) else qt.size(1)
    if scales.dim() > 2:
        scales = scales.squeeze()
    if zps is None:
        zps = torch.zeros_like(scales)
        if dtype == WoqWeightDtype.INT4:
            zps += 8
    if zps.dim() > 2:
        zps = zps.squeeze()
    if is_4bit(dtype):
        qt = unpack_nibbles(qt)
    k_rem = K % group_size
    k_com = K - k_rem
    n_full = k_com // group_size

    def deq(codes, s, z):
        v = _codes_to_float(codes, dtype, dequant_nf4_via_int8)
        if dtype == WoqWeightDtype.NF4:
            return v * s.unsqueeze(-1)
        return (v - z.unsqueeze(-1)) * s.unsqueeze(-1)

    t = deq(qt[:, :k_com].view(N, n_full, group_size), scales[:, :n_full], zps[:, :n_full]).view(N, k_com)
    if k_rem:
        t_rem = deq(qt[:, k_com:].view(N, 1, k_rem), scales[:, n_full:], zps[:, n_full:]).view(N, k_rem)
        t = torch.cat([t, t_rem], dim=1)
    t = t.contiguous()
    if weight_shape is not None:
        t = t[: weight_shape[0], : weight_shape[1]].contiguous()
    return t
