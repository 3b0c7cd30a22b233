"""ctypes binding of libwoq_hip.so (the C ABI declared in include/woq_hip.h).

The library is looked up in-tree (``<package root>/lib/libwoq_hip.so``).  There is no
CPU implementation behind these wrappers: if the library is missing, loading raises.
"""
import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libwoq_hip.so")

# weight dtype / lowp mode / fusion codes of the C ABI
DTYPE_INT8, DTYPE_INT4, DTYPE_NF4, DTYPE_FP8 = 1, 2, 3, 4
DTYPES_8BIT = (DTYPE_INT8, DTYPE_FP8)
MOE_ROUTE_MAX = 2048  # WOQ_HIP_MOE_ROUTE_MAX
LOWP_NONE, LOWP_FP16, LOWP_BF16, LOWP_INT8 = 0, 1, 2, 3
ACT_FP32, ACT_FP16, ACT_BF16 = 0, 1, 2
FUSE_NONE, FUSE_GELU_ERF, FUSE_GELU_TANH, FUSE_RELU, FUSE_SILU = 0x0, 0x1, 0x2, 0x3, 0x4
FUSE_ADD, FUSE_ADD_ADD, FUSE_MUL = 0x10, 0x20, 0x30
TILE_N, TILE_BYTES, TILE_K_INT4, TILE_K_INT8 = 16, 1024, 128, 64

EXPORTS = [
    "woq_hip_last_error",
    "woq_hip_abi_version",
    "woq_hip_small_batch_threshold",
    "woq_hip_weight_cache_batch_threshold",
    "woq_hip_dense_weight_bytes",
    "woq_hip_dense_weight",
    "woq_hip_last_kernel",
    "woq_hip_padded_n",
    "woq_hip_padded_k",
    "woq_hip_packed_weight_bytes",
    "woq_hip_pack_weight",
    "woq_hip_unpack_weight",
    "woq_hip_pack_qparams",
    "woq_hip_unpack_int4_zeros",
    "woq_hip_dynamic_quant",
    "woq_hip_linear_workspace_bytes",
    "woq_hip_linear_split_k_workspace_bytes",
    "woq_hip_linear_auto_split_k_workspace_bytes",
    "woq_hip_int8_block_k",
    "woq_hip_linear",
    "woq_hip_linear_noalloc",
    "woq_hip_dequant_weight",
    "woq_hip_convert_activations",
    "woq_hip_shuffle_activations",
    "woq_hip_shuffle_int4_weight",
    "woq_hip_moe_gather_rows",
    "woq_hip_moe_scale_add_rows",
    "woq_hip_moe_route",
    "woq_hip_linear_grouped",
    "woq_hip_moe_combine_rows",
]


class LinearParams(ctypes.Structure):
    """Mirror of ``woq_hip_linear_params``."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("x", ctypes.c_void_p),
        ("x_dtype", ctypes.c_int32),
        ("M", ctypes.c_int64),
        ("K", ctypes.c_int64),
        ("N", ctypes.c_int64),
        ("qweight", ctypes.c_void_p),
        ("weight_dtype", ctypes.c_int32),
        ("scales_f32", ctypes.c_void_p),
        ("scales_f16", ctypes.c_void_p),
        ("scales_bf16", ctypes.c_void_p),
        ("zeros_u8", ctypes.c_void_p),
        ("scale_zero_f16x2", ctypes.c_void_p),
        ("scale_zero_bf16", ctypes.c_void_p),
        ("dense_bf16", ctypes.c_void_p),
        ("group_size", ctypes.c_int64),
        ("bias", ctypes.c_void_p),
        ("lowp_mode", ctypes.c_int32),
        ("act_quant_mode", ctypes.c_int32),
        ("fusion", ctypes.c_int32),
        ("others", ctypes.c_void_p * 2),
        ("out", ctypes.c_void_p),
        ("out_dtype", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_int64),
        ("split_k_counters", ctypes.c_void_p),
        ("debug_block_sums", ctypes.c_void_p),
        ("force_kernel", ctypes.c_int32),
        ("stream", ctypes.c_void_p),
    ]


_lib = None
_lock = threading.Lock()


def load():
    """Loads the shared library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with "
                "`python intel-extension-for-pytorch_amd/csrc/build.py` (needs hipcc); "
                "there is no CPU fallback for the WOQ linear kernels."
            )
        lib = ctypes.CDLL(LIB_PATH)
        i32, i64, vp = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p
        lib.woq_hip_last_error.restype = ctypes.c_char_p
        lib.woq_hip_last_error.argtypes = []
        lib.woq_hip_abi_version.restype = i32
        lib.woq_hip_small_batch_threshold.restype = i32
        lib.woq_hip_small_batch_threshold.argtypes = []
        lib.woq_hip_weight_cache_batch_threshold.restype = i32
        lib.woq_hip_weight_cache_batch_threshold.argtypes = []
        lib.woq_hip_dense_weight_bytes.restype = i64
        lib.woq_hip_dense_weight_bytes.argtypes = [ctypes.c_int32, i64, i64]
        lib.woq_hip_dense_weight.restype = i32
        lib.woq_hip_dense_weight.argtypes = [vp, ctypes.c_int32, i64, i64, vp, vp, i64, vp, vp]
        lib.woq_hip_last_kernel.restype = ctypes.c_char_p
        lib.woq_hip_last_kernel.argtypes = []
        lib.woq_hip_padded_n.restype = i64
        lib.woq_hip_padded_n.argtypes = [i64]
        lib.woq_hip_padded_k.restype = i64
        lib.woq_hip_padded_k.argtypes = [i32, i64]
        lib.woq_hip_packed_weight_bytes.restype = i64
        lib.woq_hip_packed_weight_bytes.argtypes = [i32, i64, i64]
        lib.woq_hip_pack_weight.restype = i32
        lib.woq_hip_pack_weight.argtypes = [vp, i32, i64, i64, vp, vp]
        lib.woq_hip_unpack_weight.restype = i32
        lib.woq_hip_unpack_weight.argtypes = [vp, i32, i64, i64, vp, vp]
        lib.woq_hip_pack_qparams.restype = i32
        lib.woq_hip_pack_qparams.argtypes = [vp, vp, i32, i64, i64, vp, vp, vp, vp, vp, vp, vp]
        lib.woq_hip_unpack_int4_zeros.restype = i32
        lib.woq_hip_unpack_int4_zeros.argtypes = [vp, i64, i64, i64, vp, vp]
        lib.woq_hip_dynamic_quant.restype = i32
        lib.woq_hip_dynamic_quant.argtypes = [vp, i32, i64, i64, i64, i32, vp, vp, vp, vp]
        lib.woq_hip_linear_workspace_bytes.restype = i64
        lib.woq_hip_linear_workspace_bytes.argtypes = [i64, i64, ctypes.c_int32, ctypes.c_int32, i64]
        lib.woq_hip_linear_split_k_workspace_bytes.restype = i64
        lib.woq_hip_linear_split_k_workspace_bytes.argtypes = [i64, i64]
        lib.woq_hip_linear_auto_split_k_workspace_bytes.restype = i64
        lib.woq_hip_linear_auto_split_k_workspace_bytes.argtypes = [i64, i64, i64, i32]
        lib.woq_hip_int8_block_k.restype = i64
        lib.woq_hip_int8_block_k.argtypes = [i64, i64]
        lib.woq_hip_linear.restype = i32
        lib.woq_hip_linear.argtypes = [ctypes.POINTER(LinearParams)]
        lib.woq_hip_linear_noalloc.restype = i32
        lib.woq_hip_linear_noalloc.argtypes = [ctypes.POINTER(LinearParams)]
        lib.woq_hip_dequant_weight.restype = i32
        lib.woq_hip_dequant_weight.argtypes = [vp, i32, i64, i64, vp, vp, i64, vp, i32, vp]
        lib.woq_hip_convert_activations.restype = i32
        lib.woq_hip_convert_activations.argtypes = [vp, i32, vp, i32, i64, vp]
        lib.woq_hip_shuffle_activations.restype = i32
        lib.woq_hip_shuffle_activations.argtypes = [vp, i32, i64, i64, vp, vp, vp]
        lib.woq_hip_shuffle_int4_weight.restype = i32
        lib.woq_hip_shuffle_int4_weight.argtypes = [vp, i64, i64, vp, vp, vp]
        lib.woq_hip_moe_gather_rows.restype = i32
        lib.woq_hip_moe_gather_rows.argtypes = [vp, i32, i64, i64, vp, i64, vp, vp]
        lib.woq_hip_moe_scale_add_rows.restype = i32
        lib.woq_hip_moe_scale_add_rows.argtypes = [vp, i32, i64, i64, vp, vp, i64, vp, vp, i64, vp]
        lib.woq_hip_moe_route.restype = i32
        lib.woq_hip_moe_route.argtypes = [vp, i64, i64, i64, i64, i64, i32, i64, vp, vp, vp, vp, vp]
        lib.woq_hip_linear_grouped.restype = i32
        lib.woq_hip_linear_grouped.argtypes = [ctypes.POINTER(LinearParams), vp, i64]
        lib.woq_hip_moe_combine_rows.restype = i32
        lib.woq_hip_moe_combine_rows.argtypes = [vp, i32, i64, i64, vp, vp, i64, vp, vp, i32, vp]
        if lib.woq_hip_abi_version() != 3:
            raise RuntimeError("libwoq_hip.so has an unexpected ABI version")
        _lib = lib
    return _lib


TORCH_LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libwoq_torch.so")
_torch_binding_loaded = False


def load_torch_binding():
    """Loads libwoq_torch.so, whose static initialisers register the ``torch_ipex`` / ``ipex_prepack``
    operators and the ``ipex_prepack.WoqLinearOpContext`` custom class; raises if it has not been built."""
    global _torch_binding_loaded
    if _torch_binding_loaded:
        return
    load()  # libwoq_hip.so first: the binding links against it
    with _lock:
        if _torch_binding_loaded:
            return
        if not os.path.exists(TORCH_LIB_PATH):
            raise RuntimeError(
                f"{TORCH_LIB_PATH} is missing: build it with "
                "`python intel-extension-for-pytorch_amd/csrc/build.py` (needs hipcc and g++); "
                "there is no Python or CPU fallback for the WOQ linear operators."
            )
        import torch

        torch.ops.load_library(TORCH_LIB_PATH)
        _torch_binding_loaded = True


def last_kernel():
    """Name of the kernel this thread launched last through the library."""
    return load().woq_hip_last_kernel().decode("ascii")


def check(rc, what):
    if rc != 0:
        msg = load().woq_hip_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what}: {msg}")
