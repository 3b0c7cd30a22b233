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


# ---------------------------------------------------------------------------------------------
# A whole model from a low-precision checkpoint (state dict + quantization config), the way
# ipex.llm.optimize(..., low_precision_checkpoint=...) does it
# (intel_extension_for_pytorch/utils/weight_only_quantization.py:22-376).
# ---------------------------------------------------------------------------------------------
# Where a checkpoint of each kind keeps a linear layer's tensors (keys under the layer's name).
GPTQ_LOWP_CHECKPOINT_CONFIG = {"name": "gptq", "weight_key": "qweight", "scale_key": "scales", "zero_point_key": "qzeros",
                               "bias_key": "bias", "g_idx_key": "g_idx", "desc_act": None}
AWQ_LOWP_CHECKPOINT_CONFIG = {"name": "awq", "weight_key": "qweight", "scale_key": "scales", "zero_point_key": "qzeros",
                              "bias_key": "bias"}
RTN_LOWP_CHECKPOINT_CONFIG = {"name": "rtn", "weight_key": "qweight", "scale_key": "scales", "zero_point_key": "qzeros",
                              "bias_key": "bias"}
# DeepSeek-V3 / R1: float8 e4m3fn weights with one scale per block of weight_block_size = [rows, columns]
FP8_LOWP_CHECKPOINT_CONFIG = {"name": "fp8", "weight_key": "weight", "scale_key": "weight_scale_inv",
                              "zero_point_key": "qzeros", "bias_key": "bias"}
# per-channel INT8 (meituan/DeepSeek-R1-Channel-INT8)
INT8_LOWP_CHECKPOINT_CONFIG = {"name": "int8", "weight_key": "weight", "scale_key": "weight_scale",
                               "zero_point_key": "qzeros", "bias_key": "bias"}


def _get_keys_from_config(checkpoint_config):
    get = checkpoint_config.get
    return (get("weight_key", "qweight"), get("scale_key", "scales"), get("zero_point_key", "qzeros"),
            get("bias_key", "bias"), get("g_idx_key", "g_idx"))


def _get_linear_parameters(attr_name, state_dict, checkpoint_config, quant_config):
    """The tensors of layer ``attr_name`` in the layouts from_float_and_qweight takes:
    (weight, scales, zero points, bias, group_size, g_idx, weight_format).  scales is None for a
    layer the checkpoint keeps in floating point (lm_head)."""
    from ..nn.modules.weight_only_quantization import WoqWeightFormat

    wk, sk, zk, bk, gk = _get_keys_from_config(checkpoint_config)
    qweight = state_dict.get(f"{attr_name}.{wk}")
    scales = state_dict.get(f"{attr_name}.{sk}")
    qzeros = state_dict.get(f"{attr_name}.{zk}")
    bias = state_dict.get(f"{attr_name}.{bk}")
    g_idx = state_dict.get(f"{attr_name}.{gk}")
    group_size, weight_format = -1, WoqWeightFormat.PLAIN_FORMAT
    if qweight is None:
        return state_dict.get(f"{attr_name}.weight"), scales, qzeros, bias, group_size, g_idx, weight_format
    method = quant_config["quant_method"]
    if method == "gptq":
        # qweight [K / 8, N] int32, scales [K / G, N], qzeros [K / G, N / 8] int32
        K = qweight.size(0) * 8
        if scales is not None:
            assert scales.dim() == 2, "Unexpected scales tensor dimension"
            if scales.size(-1) != 1:
                group_size = K // scales.size(0)
                assert group_size > 0
                group_size = 2 ** (group_size - 1).bit_length()  # next power of two
        if checkpoint_config.get("desc_act") is False:
            g_idx = None
        if g_idx is not None and group_size > 0:
            # an identity or all-zero g_idx is no act-order
            if torch.equal(g_idx.to(torch.int64).cpu(), torch.arange(K) // group_size) or not bool(g_idx.any()):
                g_idx = None
        if g_idx is not None:
            # act-order shuffles input channels: that needs the plain layout
            qweight, scales, qzeros = _convert_optimum_format_to_desired(qweight, scales, qzeros)
        else:
            scales, qzeros = _convert_gptq_scales_qzeros(scales, qzeros)
            weight_format = WoqWeightFormat.GPTQ_FORMAT
    elif method == "awq":
        if scales is not None:
            assert qweight.size(0) % scales.size(0) == 0, "Uneven group sizes are not supported"
            group_size = qweight.size(0) // scales.size(0)
            scales, qzeros = _convert_awq_scales_qzeros(scales, qzeros)
            weight_format = WoqWeightFormat.AWQ_FORMAT
            g_idx = None
    elif method == "fp8":
        if scales is not None:
            block_n, block_k = quant_config["weight_block_size"]
            assert qweight.size(1) % block_k == 0, f"Weight size is not divisible by {block_k}, got {qweight.shape}"
            if scales.size(0) != qweight.size(0):
                assert (qweight.size(0) + block_n - 1) // block_n == scales.size(0), (
                    f"WOQ FP8 got misaligned shapes of weight and scales: {qweight.shape}, {scales.shape}, "
                    f"blocks = {[block_n, block_k]}"
                )
                # one scale per block of rows -> one per row
                scales = torch.repeat_interleave(scales, block_n, 0)[: qweight.size(0)].contiguous()
            group_size = block_k
    elif method == "rtn":
        # 8 bits: qweight [K / 4, N] int32 (four int8 along K), scales [K / G, N] or [1, N],
        # qzeros [K / G, N / 4] or [1, N / 4] int32 holding uint8 zero points minus one
        assert quant_config.get("bits", 8) == 8, "rtn checkpoints are read with 8-bit weights"
        assert scales.shape[0] == qzeros.shape[0]
        if scales.shape[0] == 1:
            scales = scales.squeeze(0)
            qzeros = qzeros.squeeze(0).contiguous().view(torch.uint8)
        else:
            group_size = qweight.size(0) * 4 // scales.size(0)
            scales = scales.t().contiguous()
            qzeros = qzeros.contiguous().view(torch.uint8).t().contiguous()
        qzeros = (qzeros + 1).view(torch.int8)  # uint8 arithmetic: 255 wraps to 0
        g_idx = None
        qweight = qweight.t().contiguous().view(torch.int8)
    return qweight, scales, qzeros, bias, group_size, g_idx, weight_format


def _convert_woq_with_low_precision_checkpoint(model, qconfig_mapping, low_precision_checkpoint, quant_config,
                                               inplace=True):
    """Replaces every nn.Linear of ``model`` whose tensors the checkpoint holds in quantized form by a
    WeightOnlyQuantizedLinear built from them (GPTQ / AWQ INT4, DeepSeek block-wise FP8, round-to-nearest
    and per-channel INT8); layers the checkpoint keeps in floating point (lm_head) and every other
    parameter are loaded as they are.  ``quant_config``: {"quant_method": "gptq" | "awq" | "fp8" | "rtn" |
    "int8", "group_size": optional override, "desc_act", "weight_block_size", "bits"}."""
    import copy

    from ..nn.modules.weight_only_quantization import WeightOnlyQuantizedLinear
    from ..quantization import WoqWeightDtype

    assert isinstance(low_precision_checkpoint, dict), "low_precision_checkpoint should be a state_dict"
    method = quant_config["quant_method"]
    group_size_override = quant_config.get("group_size")
    target = WoqWeightDtype.INT4
    if method == "gptq":
        config = dict(GPTQ_LOWP_CHECKPOINT_CONFIG)
        if "desc_act" in quant_config:
            config["desc_act"] = quant_config.get("desc_act")
    elif method == "awq":
        config = AWQ_LOWP_CHECKPOINT_CONFIG
    elif method == "fp8":
        config, target = FP8_LOWP_CHECKPOINT_CONFIG, WoqWeightDtype.FP8
    elif method == "rtn":
        config, target = RTN_LOWP_CHECKPOINT_CONFIG, WoqWeightDtype.INT8
    elif method == "int8":
        config, target = INT8_LOWP_CHECKPOINT_CONFIG, WoqWeightDtype.INT8
    else:
        raise AssertionError(f"{method} is not supported, quantization_method choice in [`gptq`, `awq`, `fp8`].")
    state_dict = low_precision_checkpoint
    wk, sk, *_ = _get_keys_from_config(config)
    assert any(k.endswith("." + wk) for k in state_dict) and any(k.endswith("." + sk) for k in state_dict), (
        "Error: Format of checkpoint and config do not match"
    )
    global_qconfig = getattr(qconfig_mapping, "global_qconfig", qconfig_mapping)

    def convert(mod, attr_name):
        if isinstance(mod, torch.nn.Linear):
            mod.qconfig = global_qconfig
            weight, scales, qzeros, bias, group_size, g_idx, w_format = _get_linear_parameters(
                attr_name, state_dict, config, quant_config)
            if group_size_override is not None:
                group_size = group_size_override
            if scales is None:  # kept in floating point by the checkpoint
                if weight is not None and weight.dtype in (torch.float, torch.bfloat16, torch.half):
                    mod.weight = torch.nn.Parameter(weight)
                    if isinstance(getattr(mod, "bias", None), torch.nn.Parameter) and bias is not None:
                        mod.bias = torch.nn.Parameter(bias)
                return mod
            return WeightOnlyQuantizedLinear.from_float_and_qweight(
                mod, weight, target, scales, qzeros, bias, group_size=group_size, g_idx=g_idx, weight_format=w_format)
        if isinstance(getattr(mod, "weight", None), torch.nn.Parameter):
            mod.weight = torch.nn.Parameter(state_dict.get(attr_name + ".weight", mod.weight.data))
            if isinstance(getattr(mod, "bias", None), torch.nn.Parameter):
                mod.bias = torch.nn.Parameter(state_dict.get(attr_name + ".bias", mod.bias.data))
            if hasattr(mod, "e_score_correction_bias"):  # DeepSeek-V3 router
                mod.e_score_correction_bias = torch.nn.Parameter(
                    state_dict.get(attr_name + ".e_score_correction_bias", mod.e_score_correction_bias.data))
            return mod
        for name, child in mod.named_children():
            setattr(mod, name, convert(child, f"{attr_name}.{name}" if attr_name else name))
        return mod

    return convert(model if inplace else copy.deepcopy(model), "")
