"""ek_hip: Python host mirror of Expert Kit's worker-side expert interface over libek_hip.so."""
from ._capi import (EK_BF16, EK_DEVICE, EK_EXPERT_NOT_FOUND, EK_F16, EK_F32, EK_HIP_ERROR, EK_HOST, EK_I8,
                    EK_INTERNAL, EK_INVALID_INPUT, EK_OK, EK_OOM, EK_WEIGHT_NOT_FOUND, EKError, LIB_PATH, load)
from .backend import (EKInstance, ExpertBackend, ExpertWeight, HipBatcher, HipChain, HipFFN, HipLayer, RouterConfig,
                      RouteTables)

__all__ = ["EKInstance", "ExpertBackend", "ExpertWeight", "HipBatcher", "HipChain", "HipFFN", "HipLayer", "RouterConfig", "RouteTables", "EKError", "load",
           "LIB_PATH"]
