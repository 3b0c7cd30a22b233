"""INT4 checkpoint layouts (AutoGPTQ / AutoAWQ) -> the plain format the prepack takes.

Closed forms follow the reference converters
(intel_extension_for_pytorch/nn/utils/_model_convert.py:62-257 and
csrc/cpu/aten/kernels/WoqUtilKrnl.cpp:109-218):

  GPTQ : qweight int32 [K/8, N], nibble i of word [j, n] is q[8j + i, n];
         scales [K/G, N]; qzeros int32 [K/G, N/8], nibble i of word [g, j] is zp[g, 8j + i] - 1
         (stored minus one, so one is added back and 16 wraps to 0).
  AWQ  : qweight int32 [K, N/8], nibble i of word [k, j] is q[k, 8j + AWQ_ORDER[i]];
         scales [K/G, N]; qzeros int32 [K/G, N/8] in the same nibble order, no offset.
  plain: uint8 [N, K/2], low nibble = even k; scales / zero points [N, K/G].
"""
import torch

AWQ_ORDER = [0, 2, 4, 6, 1, 3, 5, 7]
# column c of a group of 8 sits in nibble AWQ_NIBBLE_OF_COL[c]
AWQ_NIBBLE_OF_COL = [AWQ_ORDER.index(c) for c in range(8)]


def _unpack_int32_nibbles(t):
    """int32 [..., C] -> int32 [..., C, 8], nibble i in the last dim."""
    shifts = torch.arange(0, 32, 4, dtype=torch.int32, device=t.device)
    return (t.unsqueeze(-1) >> shifts) & 0xF


def _nibbles_to_plain(q_nk):
    """uint8 codes [N, K] -> plain packed [N, K/2]."""
    q_nk = q_nk.to(torch.uint8)
    if q_nk.shape[1] % 2:
        q_nk = torch.nn.functional.pad(q_nk, (0, 1), value=0)
    return (q_nk[:, 1::2] << 4).bitwise_or(q_nk[:, ::2]).contiguous()


def gptq_to_plain(qweight):
    """GPTQ int32 [K/8, N] -> plain uint8 [N, K/2]."""
    assert qweight.dtype == torch.int32 and qweight.dim() == 2
    k8, n = qweight.shape
    q = _unpack_int32_nibbles(qweight)  # [K/8, N, 8]
    q = q.permute(1, 0, 2).reshape(n, k8 * 8)
    return _nibbles_to_plain(q)


def awq_to_plain(qweight):
    """AWQ int32 [K, N/8] -> plain uint8 [N, K/2]."""
    assert qweight.dtype == torch.int32 and qweight.dim() == 2
    k, n8 = qweight.shape
    nib = _unpack_int32_nibbles(qweight)  # [K, N/8, 8] by nibble
    sel = torch.tensor(AWQ_NIBBLE_OF_COL, dtype=torch.long, device=qweight.device)
    q = nib.index_select(-1, sel).reshape(k, n8 * 8)  # [K, N] by column
    return _nibbles_to_plain(q.t())


def _convert_gptq_scales_qzeros(scales, qzeros, inplace=True):
    """GPTQ (n_groups, N) scales and (n_groups, N/8) packed zeros -> (N, n_groups) each; the
    zero points get the +1 the GPTQ packing removed, with 16 wrapping to 0."""
    scales = scales.t().contiguous()
    if qzeros is None:
        return scales, qzeros
    g, n8 = qzeros.shape
    zp = _unpack_int32_nibbles(qzeros).reshape(g, n8 * 8).t().contiguous().to(torch.int32)
    zp = zp + 1
    zp = torch.where(zp > 15, torch.zeros_like(zp), zp)
    return scales, zp


def _convert_awq_scales_qzeros(scales, qzeros, bits=4):
    """AWQ (n_groups, N) scales and (n_groups, N/8) packed zeros -> (N, n_groups) each."""
    assert bits == 4
    new_scales = scales.t().contiguous()
    g, n8 = qzeros.shape
    nib = _unpack_int32_nibbles(qzeros)
    sel = torch.tensor(AWQ_NIBBLE_OF_COL, dtype=torch.long, device=qzeros.device)
    zp = nib.index_select(-1, sel).reshape(g, n8 * 8).to(torch.int8)
    return new_scales, zp.t().contiguous()


def _convert_optimum_format_to_desired(qweight, scales, qzeros, inplace=True):
    """Optimum / GPTQ tensors -> qweight int32 [N, K/8] (still 8 nibbles per word along K, which
    is the plain byte layout when viewed as uint8), scales and zero points [N, n_groups]."""
    if qweight is None:
        return qweight, scales, qzeros
    assert qweight.shape[1] == scales.shape[1]
    qweight = qweight.t().contiguous()
    scales, zp = _convert_gptq_scales_qzeros(scales, qzeros, inplace)
    return qweight, scales, zp
