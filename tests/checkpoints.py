"""Synthetic low-precision checkpoints in the layouts the converters read (test plumbing): the tensors
AutoGPTQ / AutoAWQ / DeepSeek-FP8 / round-to-nearest checkpoints hold for one linear layer, built from known
codes so that the expected dequantized weight is known in closed form."""
import torch

AWQ_ORDER = [0, 2, 4, 6, 1, 3, 5, 7]


def _pack8(v, order=range(8)):
    """int64 [..., 8] nibbles -> int32 [...], nibble i of a word = v[..., order[i]]."""
    w = torch.zeros(v.shape[:-1], dtype=torch.int64)
    for i, o in enumerate(order):
        w |= v[..., o].to(torch.int64) << (4 * i)
    return (w - (w >= 2**31) * 2**32).to(torch.int32)


def gptq_layer(q, zp, scales):
    """q [N, K] codes, zp [N, KG], scales [N, KG] -> (qweight [K/8, N], scales [KG, N], qzeros [KG, N/8])."""
    N, K = q.shape
    qweight = _pack8(q.t().contiguous().view(K // 8, 8, N).permute(0, 2, 1))
    qzeros = _pack8(((zp - 1) % 16).t().contiguous().view(zp.shape[1], N // 8, 8))
    return qweight, scales.t().contiguous(), qzeros


def awq_layer(q, zp, scales):
    """-> (qweight [K, N/8], scales [KG, N], qzeros [KG, N/8]), AWQ nibble order, zero points as they are."""
    N, K = q.shape
    qweight = _pack8(q.t().contiguous().view(K, N // 8, 8), AWQ_ORDER)
    qzeros = _pack8(zp.t().contiguous().view(zp.shape[1], N // 8, 8), AWQ_ORDER)
    return qweight, scales.t().contiguous(), qzeros


def int4_dequant(q, zp, scales, G):
    g = torch.arange(q.shape[1]) // G
    return (q - zp[:, g]).float() * scales.float()[:, g]


def fp8_layer(w, block_n, block_k):
    """float weight [N, K] -> (float8 e4m3fn weight, weight_scale_inv [ceil(N / block_n), K / block_k]) with one
    scale per block (absmax / 448), and the dequantized weight."""
    N, K = w.shape
    nb = (N + block_n - 1) // block_n
    wp = torch.zeros(nb * block_n, K)
    wp[:N] = w
    blocks = wp.view(nb, block_n, K // block_k, block_k)
    scale = blocks.abs().amax(dim=(1, 3)) / 448.0
    q = (blocks / scale[:, None, :, None]).reshape(nb * block_n, K)[:N].to(torch.float8_e4m3fn)
    dq = (q.float().view(N, K // block_k, block_k) * torch.repeat_interleave(scale, block_n, 0)[:N, :, None]).view(N, K)
    return q, scale, dq
