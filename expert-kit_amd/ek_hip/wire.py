"""Wire-format helpers over the C ABI: expert ids and one-tensor safetensors blobs.

Mirrors ExpertKey (ek-db/src/safetensor/mod.rs:57-90) and TchTensor::serialize /
SafeTensors::deserialize as the worker uses them (worker/core.rs:52-53, 61).
Parsing and emitting are done by the library, not here.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Sequence, Tuple

import torch

from . import _capi as C

_TORCH_OF = {C.EK_BF16: torch.bfloat16, C.EK_F16: torch.float16, C.EK_F32: torch.float32, C.EK_I8: torch.int8,
             C.EK_F8E4M3: torch.float8_e4m3fn}
_EK_OF = {v: k for k, v in _TORCH_OF.items()}


@dataclass(frozen=True)
class ExpertKey:
    model: str
    layer: int
    expert: int

    @classmethod
    def from_expert_id(cls, expert_id: str) -> "ExpertKey":
        layer, expert = ctypes.c_int32(), ctypes.c_int32()
        C.check(C.load().ek_expert_id_parse(expert_id.encode(), ctypes.byref(layer), ctypes.byref(expert)))
        return cls(expert_id.split("/l")[0], layer.value, expert.value)

    def as_object_key(self) -> str:
        buf = ctypes.create_string_buffer(len(self.model) + 32)
        C.check(C.load().ek_expert_id_format(self.model.encode(), self.layer, self.expert, buf, len(buf)))
        return buf.value.decode()


def find(blob: bytes, name: str) -> torch.Tensor:
    """Tensor `name` of a safetensors blob (a copy)."""
    view = C.ek_tensor_view()
    C.check(C.load().ek_safetensors_find(blob, len(blob), name.encode(), ctypes.byref(view)))
    return _tensor_of(view)


def find_suffix(blob: bytes, suffixes: Sequence[str]) -> torch.Tensor:
    view = C.ek_tensor_view()
    arr = (ctypes.c_char_p * len(suffixes))(*[s.encode() for s in suffixes])
    C.check(C.load().ek_safetensors_find_suffix(blob, len(blob), arr, len(suffixes), ctypes.byref(view)))
    return _tensor_of(view)


def _tensor_of(view: "C.ek_tensor_view") -> torch.Tensor:
    shape: Tuple[int, ...] = tuple(view.shape[i] for i in range(view.rank))
    raw = ctypes.string_at(view.data, view.nbytes) if view.nbytes else b""
    t = torch.frombuffer(bytearray(raw), dtype=torch.uint8) if raw else torch.empty(0, dtype=torch.uint8)
    return t.view(_TORCH_OF[view.dtype]).reshape(shape)


def emit(name: str, t: torch.Tensor) -> bytes:
    """One-tensor safetensors blob, byte for byte what safetensors::serialize writes."""
    t = t.contiguous().cpu()
    dt = _EK_OF[t.dtype]
    shape = (ctypes.c_int64 * max(t.dim(), 1))(*t.shape)
    lib = C.load()
    size = lib.ek_safetensors_size(name.encode(), dt, t.dim(), shape)
    if size == 0:
        raise C.EKError(C.EK_INVALID_INPUT, "tensor cannot be described in a safetensors header")
    out = ctypes.create_string_buffer(size)
    written = ctypes.c_size_t()
    C.check(lib.ek_safetensors_emit(name.encode(), dt, t.dim(), shape, ctypes.c_void_p(t.data_ptr()), out, size,
                                    ctypes.byref(written)))
    return out.raw[:written.value]
