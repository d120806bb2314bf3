"""ctypes binding of libek_hip.so (the C ABI declared in include/ek_hip.h).

This is the Python spelling of the stub a Rust maintainer would write with
``extern "C"``: structs and prototypes only, no arithmetic.  Loading fails
loudly when the shared library has not been built; there is no fallback.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libek_hip.so")

EK_OK, EK_INVALID_INPUT, EK_EXPERT_NOT_FOUND, EK_WEIGHT_NOT_FOUND, EK_OOM, EK_HIP_ERROR, EK_INTERNAL = range(7)
EK_BF16, EK_F16, EK_F32, EK_I8, EK_F8E4M3 = range(5)
EK_HOST, EK_DEVICE = 0, 1
EK_SCALE_NONE, EK_SCALE_PER_CHANNEL, EK_SCALE_BLOCK128 = 0, 1, 2

STATUS_NAMES = ["EK_OK", "EK_INVALID_INPUT", "EK_EXPERT_NOT_FOUND", "EK_WEIGHT_NOT_FOUND", "EK_OOM",
                "EK_HIP_ERROR", "EK_INTERNAL"]


class ek_cfg(ctypes.Structure):
    _fields_ = [("hidden", ctypes.c_int64), ("inter", ctypes.c_int64), ("n_experts", ctypes.c_int32),
                ("top_k", ctypes.c_int32), ("act_dtype", ctypes.c_int32), ("w_dtype", ctypes.c_int32),
                ("max_tokens", ctypes.c_int64), ("device_id", ctypes.c_int32), ("flags", ctypes.c_int32)]


class ek_weight_desc(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("rows", ctypes.c_int64), ("cols", ctypes.c_int64),
                ("dtype", ctypes.c_int32), ("mem", ctypes.c_int32), ("scale", ctypes.c_void_p),
                ("scale_dtype", ctypes.c_int32), ("scale_kind", ctypes.c_int32)]


class ek_route_out(ctypes.Structure):
    _fields_ = [("counts", ctypes.c_void_p), ("offsets", ctypes.c_void_p), ("perm", ctypes.c_void_p),
                ("inv_perm", ctypes.c_void_p), ("expert_out", ctypes.c_void_p)]


class ek_stats(ctypes.Structure):
    _fields_ = [("forward_calls", ctypes.c_int64), ("tokens", ctypes.c_int64), ("pairs", ctypes.c_int64),
                ("expert_forward_calls", ctypes.c_int64), ("last_forward_us", ctypes.c_double),
                ("kernel_us", ctypes.c_double * 4), ("profiled_calls", ctypes.c_int64)]


class ek_tensor_view(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("shape", ctypes.c_int64 * 4), ("rank", ctypes.c_int32),
                ("dtype", ctypes.c_int32), ("nbytes", ctypes.c_int64)]


class ek_histogram(ctypes.Structure):
    _fields_ = [("le", ctypes.c_double * 10), ("cumulative", ctypes.c_int64 * 11), ("sum", ctypes.c_double),
                ("count", ctypes.c_int64)]


class ek_batcher_stats(ctypes.Structure):
    _fields_ = [("calls", ctypes.c_int64), ("batches", ctypes.c_int64), ("largest_batch", ctypes.c_int64)]


class ek_peaks(ctypes.Structure):
    _fields_ = [("copy_gbps", ctypes.c_double), ("read_nt_gbps", ctypes.c_double), ("mfma_bf16_tflops", ctypes.c_double),
                ("mfma_bf16_random_tflops", ctypes.c_double), ("mfma_bf16_dequant_tflops", ctypes.c_double)]


class ek_router_cfg(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("renorm", ctypes.c_int32), ("n_group", ctypes.c_int32),
                ("topk_group", ctypes.c_int32), ("routed_scaling", ctypes.c_float), ("flags", ctypes.c_int32),
                ("logits_dtype", ctypes.c_int32), ("w_dtype", ctypes.c_int32), ("bias", ctypes.c_void_p)]


(EK_ROUTER_SOFTMAX_TOPK, EK_ROUTER_TOPK_RAW, EK_ROUTER_TOPK_SOFTMAX, EK_ROUTER_TOPK_SIGMOID,
 EK_ROUTER_SIGMOID_GROUP) = range(5)
EK_ROUTER_MASK_NEG_INF = 1
EK_SHARED_EXPERT = -1
EK_CFG_BLOCK_SCALES = 1
EK_STATIC_SCRATCH_BYTES = 32 << 20

_P = ctypes.c_void_p
_PP = ctypes.POINTER(ctypes.c_void_p)
_I32, _I64 = ctypes.c_int32, ctypes.c_int64
_DESC = ctypes.POINTER(ek_weight_desc)
_SZ = ctypes.c_size_t
_VIEW = ctypes.POINTER(ek_tensor_view)
_STRS = ctypes.POINTER(ctypes.c_char_p)

# name -> (restype, argtypes); every symbol include/ek_hip.h declares
PROTOTYPES = {
    "ek_backend_name": (ctypes.c_char_p, []),
    "ek_last_error": (ctypes.c_char_p, []),
    "ek_device_count": (_I32, []),
    "ek_layer_create": (_I32, [ctypes.POINTER(ek_cfg), _PP]),
    "ek_layer_destroy": (_I32, [_P]),
    "ek_layer_set_expert": (_I32, [_P, _I32, _DESC, _DESC, _DESC]),
    "ek_layer_remove_expert": (_I32, [_P, _I32]),
    "ek_layer_has_expert": (_I32, [_P, _I32, ctypes.POINTER(_I32)]),
    "ek_layer_forward": (_I32, [_P, _P, _P, _P, _I32, _I64, _P, ctypes.POINTER(ek_route_out), _I32, _P]),
    "ek_layer_forward_static": (_I32, [_P, _P, _P, _P, _I32, _I64, _P, ctypes.POINTER(ek_route_out), _P]),
    "ek_layer_pack": (_I32, [_P, _P, _I64, ctypes.POINTER(ek_route_out), _P, _P, _I32, _P]),
    "ek_layer_expert_forward": (_I32, [_P, _I32, _P, _I64, _P, _I32, _P]),
    "ek_layer_describe": (_I32, [_P, ctypes.POINTER(_I64), ctypes.POINTER(_I64), ctypes.POINTER(_I32),
                                 ctypes.POINTER(_I32), ctypes.POINTER(_I32)]),
    "ek_layer_experts_forward": (_I32, [_P, _I32, ctypes.POINTER(_I32), _PP, ctypes.POINTER(_I64), _PP, _I32, _P]),
    "ek_expert_id_parse": (_I32, [ctypes.c_char_p, ctypes.POINTER(_I32), ctypes.POINTER(_I32)]),
    "ek_expert_id_format": (_I32, [ctypes.c_char_p, _I32, _I32, ctypes.c_char_p, _SZ]),
    "ek_safetensors_find": (_I32, [_P, _SZ, ctypes.c_char_p, _VIEW]),
    "ek_safetensors_find_suffix": (_I32, [_P, _SZ, _STRS, _I32, _VIEW]),
    "ek_safetensors_size": (_SZ, [ctypes.c_char_p, _I32, _I32, ctypes.POINTER(_I64)]),
    "ek_safetensors_emit": (_I32, [ctypes.c_char_p, _I32, _I32, ctypes.POINTER(_I64), _P, _P, _SZ,
                                   ctypes.POINTER(_SZ)]),
    "ek_layer_set_expert_safetensors": (_I32, [_P, _I32, _P, _SZ]),
    "ek_worker_forward": (_I32, [_P, ctypes.c_char_p, _P, _SZ, _P, _SZ, ctypes.POINTER(_SZ)]),
    "ek_worker_forward_batch": (_I32, [_P, _I32, _STRS, _PP, ctypes.POINTER(_SZ), _PP, ctypes.POINTER(_SZ),
                                       ctypes.POINTER(_SZ)]),
    "ek_batcher_create": (_I32, [_P, _I64, _I32, _PP]),
    "ek_batcher_forward": (_I32, [_P, ctypes.c_char_p, _P, _SZ, _P, _SZ, ctypes.POINTER(_SZ)]),
    "ek_batcher_get_stats": (_I32, [_P, ctypes.POINTER(ek_batcher_stats)]),
    "ek_batcher_destroy": (_I32, [_P]),
    "ek_layer_route": (_I32, [_P, _P, ctypes.POINTER(ek_router_cfg), _I64, _P, _P, _I32, _P]),
    "ek_layer_forward_logits": (_I32, [_P, _P, _P, ctypes.POINTER(ek_router_cfg), _I64, _P, _P, _P,
                                       ctypes.POINTER(ek_route_out), _I32, _P]),
    "ek_layer_get_activation": (_I32, [_P, ctypes.POINTER(_I64)]),
    "ek_layer_get_forward_histogram": (_I32, [_P, ctypes.POINTER(ek_histogram)]),
    "ek_layer_profile": (_I32, [_P, _I32]),
    "ek_layer_get_stats": (_I32, [_P, ctypes.POINTER(ek_stats)]),
    "ek_measure_peaks": (_I32, [_I32, ctypes.POINTER(ek_peaks)]),
    "ek_chain_create": (_I32, [_PP, _I32, _PP]),
    "ek_chain_forward": (_I32, [_P, _P, _P, _P, _I32, _I64, _P, _I32, _P]),
    "ek_chain_destroy": (_I32, [_P]),
    "ek_expert_create": (_I32, [ctypes.POINTER(ek_cfg), _I64, _DESC, _DESC, _DESC, _PP]),
    "ek_expert_forward": (_I32, [_P, _P, _I64, _P, _I32, _P]),
    "ek_expert_shape": (_I32, [_P, ctypes.POINTER(_I64), ctypes.POINTER(_I64)]),
    "ek_expert_destroy": (_I32, [_P]),
}

_LIB = None


def load() -> ctypes.CDLL:
    """dlopen libek_hip.so and attach prototypes.  Raises if it is not built."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C expert-kit_amd/csrc` "
                "(or __graft_entry__.build()); there is no non-HIP fallback")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _LIB = lib
    return _LIB


class EKError(RuntimeError):
    """Mirrors ek_base::error::EKError for this path (ek-base/src/error.rs:12-72)."""

    def __init__(self, status: int, message: str):
        super().__init__(f"{STATUS_NAMES[status] if 0 <= status < len(STATUS_NAMES) else status}: {message}")
        self.status = status
        self.message = message


def check(status: int) -> None:
    if status != EK_OK:
        raise EKError(status, load().ek_last_error().decode("utf-8", "replace"))
