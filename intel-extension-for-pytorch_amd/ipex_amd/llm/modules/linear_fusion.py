"""``ipex.llm.modules`` linear fusions over weight-only-quantized linears: the callers of the
fused ``torch.ops.torch_ipex.woq_linear_*`` operators
(intel_extension_for_pytorch/llm/modules/linear_fusion.py:55-400 for the public classes,
intel_extension_for_pytorch/transformers/models/cpu/fusions/linear_fusion.py:33-534 for what they
do with a WOQ linear).

A wrapped ``WeightOnlyQuantizedLinear`` runs the post-op inside the GEMM kernel's epilogue; any
other linear module takes the reference's fallback path, the unfused composition.
"""
import types

import torch
import torch.nn as nn

from ...nn.modules.weight_only_quantization import WeightOnlyQuantizedLinear


def _woq_handle(linear):
    """The prepacked-context handle of a WOQ linear, or None for any other module."""
    ctx = getattr(linear, "_op_context", None)
    if isinstance(linear, WeightOnlyQuantizedLinear) and ctx is not None:
        return ctx.get_data_handle()
    return None


class _LinearFusion(nn.Module):
    def __init__(self, linear):
        super().__init__()
        self.linear = linear


class LinearSilu(_LinearFusion):
    r"""``silu(linear(x))`` (linear_fusion.py:55-90; WOQ branch fusions/linear_fusion.py:52-62)."""

    def forward(self, x):
        h = _woq_handle(self.linear)
        if h is not None:
            return torch.ops.torch_ipex.woq_linear_silu(x, h)
        return nn.functional.silu(self.linear(x))


class LinearRelu(_LinearFusion):
    r"""``relu(linear(x))`` (linear_fusion.py:135-170)."""

    def forward(self, x):
        h = _woq_handle(self.linear)
        if h is not None:
            return torch.ops.torch_ipex.woq_linear_relu(x, h)
        return nn.functional.relu(self.linear(x))


class LinearGelu(_LinearFusion):
    r"""``gelu(linear(x))``, erf form (linear_fusion.py:211-246)."""

    def forward(self, x):
        h = _woq_handle(self.linear)
        if h is not None:
            return torch.ops.torch_ipex.woq_linear_gelu(x, h)
        return nn.functional.gelu(self.linear(x))


class LinearNewGelu(_LinearFusion):
    r"""``gelu(linear(x))``, tanh form (linear_fusion.py:173-208)."""

    def forward(self, x):
        h = _woq_handle(self.linear)
        if h is not None:
            return torch.ops.torch_ipex.woq_linear_new_gelu(x, h)
        return nn.functional.gelu(self.linear(x), approximate="tanh")


class LinearMul(_LinearFusion):
    r"""``linear(x) * y`` (linear_fusion.py:288-323)."""

    def forward(self, x, y):
        h = _woq_handle(self.linear)
        if h is not None:
            return torch.ops.torch_ipex.woq_linear_mul(x, h, [y])
        return self.linear(x) * y


class LinearAdd(_LinearFusion):
    r"""``linear(x) + y`` (linear_fusion.py:326-361)."""

    def forward(self, x, y):
        h = _woq_handle(self.linear)
        if h is not None:
            return torch.ops.torch_ipex.woq_linear_add(x, h, [y])
        return self.linear(x) + y


class LinearAddAdd(_LinearFusion):
    r"""``linear(x) + y + z`` (linear_fusion.py:364-400)."""

    def forward(self, x, y, z):
        h = _woq_handle(self.linear)
        if h is not None:
            return torch.ops.torch_ipex.woq_linear_add_add(x, h, [y, z])
        return self.linear(x) + y + z


class LinearSiluMul(_LinearFusion):
    r"""``silu(linear(x)) * y`` (linear_fusion.py:249-285): the silu is fused, the product is a
    separate elementwise op, as in the reference's WOQ branch (fusions/linear_fusion.py:519-531)."""

    def forward(self, x, y):
        h = _woq_handle(self.linear)
        if h is not None:
            return torch.ops.torch_ipex.woq_linear_silu(x, h) * y
        return nn.functional.silu(self.linear(x)) * y


class Linear2SiluMul(nn.Module):
    r"""``silu(linear_s(x)) * linear_m(x)``, the gated-MLP front half (linear_fusion.py:93-132):
    ``woq_linear_silu`` on the gate, then ``woq_linear_mul`` on the up projection with the gate as
    its multiplicand (fusions/linear_fusion.py:475-490)."""

    def __init__(self, linear_s, linear_m):
        super().__init__()
        self.linear_s = linear_s
        self.linear_m = linear_m

    def forward(self, x):
        hs, hm = _woq_handle(self.linear_s), _woq_handle(self.linear_m)
        if hs is not None and hm is not None:
            y = torch.ops.torch_ipex.woq_linear_silu(x, hs)
            return torch.ops.torch_ipex.woq_linear_mul(x, hm, [y])
        return nn.functional.silu(self.linear_s(x)) * self.linear_m(x)


class ConcatLinear(nn.Module):
    r"""Several linears over the same input (Q / K / V, gate / up) as one linear over the
    concatenated output channels; ``forward`` returns the tuple of the individual outputs
    (``_IPEXConcatLinearCPU``, fusions/linear_fusion.py:296-434).

    WOQ linears are merged when none carries ``g_idx`` and they agree in weight dtype, group size,
    symmetric / asymmetric scheme, lowp mode and act-quant mode.  The reference dequantizes every
    weight and quantizes the concatenation again with the concatenated scales and zero points
    (fusions/linear_fusion.py:356-416), which reproduces the stored codes; here the plain
    quantized weights (``to_public``) are concatenated as they are, so the merged linear gives
    bit for bit the outputs of the separate ones.  Anything else runs the linears one by one."""

    def __init__(self, linears):
        super().__init__()
        self.num_concat = len(linears)
        for i, lin in enumerate(linears):
            setattr(self, f"linear_{i}", lin)
        self.concat_linear = None
        self.split_sizes = None
        merged = self._merge_woq(list(linears))
        if merged is not None:
            self.concat_linear = merged
            self.split_sizes = [lin.out_features for lin in linears]
            for i in range(self.num_concat):
                delattr(self, f"linear_{i}")

    @staticmethod
    def _merge_woq(linears):
        if not linears or not all(_woq_handle(lin) is not None for lin in linears):
            return None
        first = linears[0]
        ctxs = [lin._op_context for lin in linears]
        if any(c.get_g_idx() is not None for c in ctxs):
            return None
        same = all(
            lin.dtype == first.dtype
            and lin.in_features == first.in_features
            and lin._group_size == first._group_size
            and lin._lowp_mode == first._lowp_mode
            and lin._act_quant_mode == first._act_quant_mode
            and lin._weight_qscheme == first._weight_qscheme
            and lin._cache_weight_for_large_batch == first._cache_weight_for_large_batch
            for lin in linears
        )
        if not same:
            return None
        qweight = torch.cat([c.to_public(c.get_weight()) for c in ctxs], 0)
        scales = torch.cat([c.get_scales() for c in ctxs], 0)
        zeros = [c.get_zero_points() for c in ctxs]
        zeros = torch.cat(zeros, 0) if zeros[0] is not None else None
        biases = [c.get_bias() for c in ctxs]
        if all(b is None for b in biases):
            bias = None
        else:  # a linear without bias contributes zeros
            bias = torch.cat(
                [b.float() if b is not None else torch.zeros(lin.out_features, device=qweight.device)
                 for b, lin in zip(biases, linears)], 0)
        shape = types.SimpleNamespace(
            in_features=first.in_features, out_features=sum(lin.out_features for lin in linears), bias=None
        )
        return WeightOnlyQuantizedLinear._init_cls(
            shape, first.dtype, qweight, scales, zeros, bias, None, first._group_size, first._lowp_mode,
            first._act_quant_mode, first._cache_weight_for_large_batch, False, device=qweight.device,
        )

    def forward(self, x):
        if self.concat_linear is not None:
            return tuple(torch.split(self.concat_linear(x), self.split_sizes, dim=-1))
        return tuple(getattr(self, f"linear_{i}")(x) for i in range(self.num_concat))
