"""Host-side mirror of the reference's worker-side expert interface, over the C ABI.

Names, argument meaning and error behaviour follow the Rust items they stand
for, so the parity tests read like the reference's own:

  EKInstance     ek-computation/src/x.rs:27-32
  ExpertWeight   ek-computation/src/ffn/meta.rs:10-23, loader :56-75
  HipFFN         a third implementation of trait Expert<T> (ffn/meta.rs:30-39),
                 next to TorchFFN (ffn/expert_torch.rs:94-128)
  ExpertBackend  ek-computation/src/ffn/mod.rs:17-53
  HipLayer       the worker's ExpertDB for one layer (worker/manager.rs:14-88)
                 plus the fused pack -> FFN -> combine call

Everything here is plumbing: torch supplies buffers and streams, all
arithmetic happens inside libek_hip.so.
"""
from __future__ import annotations

import contextlib
import ctypes
from dataclasses import dataclass
from typing import Dict, Optional, Sequence

import torch

from . import _capi as C

_DT = {torch.bfloat16: C.EK_BF16, torch.float16: C.EK_F16, torch.float32: C.EK_F32, torch.int8: C.EK_I8,
       torch.float8_e4m3fn: C.EK_F8E4M3}


def _mem(t: torch.Tensor) -> int:
    return C.EK_DEVICE if t.is_cuda else C.EK_HOST


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_NO_CTX = contextlib.nullcontext()


def _alloc_on(stream):
    """Context in which the outputs of an enqueue-only call are allocated: the caller's stream.  torch's
    caching allocator hands a freed block to the next request on the stream it was allocated on without
    waiting for other streams, so a result allocated on the current stream, written by kernels on
    `stream` and dropped by the caller before they ran could be handed out again under those kernels."""
    return torch.cuda.stream(stream) if isinstance(stream, torch.cuda.Stream) else _NO_CTX


def _stream_ptr(stream) -> ctypes.c_void_p:
    if stream is None:
        return ctypes.c_void_p(0)
    return ctypes.c_void_p(stream.cuda_stream if hasattr(stream, "cuda_stream") else int(stream))


@dataclass
class EKInstance:
    hidden: int
    intermediate: int
    backend: str = "hip"


@dataclass
class ExpertWeight:
    """up/gate [I,H], down [H,I]; *_scale: per-output-channel scales for int8."""
    up_w: torch.Tensor
    gate_w: torch.Tensor
    down_w: torch.Tensor
    up_scale: Optional[torch.Tensor] = None
    gate_scale: Optional[torch.Tensor] = None
    down_scale: Optional[torch.Tensor] = None

    @staticmethod
    def _lookup_suffix(tensors: Dict[str, torch.Tensor], suffixes: Sequence[str]):
        for name in sorted(tensors):
            if any(name.endswith(s) for s in suffixes):
                return tensors[name]
        return None

    @classmethod
    def from_safetensor(cls, tensors: Dict[str, torch.Tensor]) -> "ExpertWeight":
        """Suffix lookup of ffn/meta.rs:56-75 (w1 = up, w2 = down, w3 = gate)."""
        up = cls._lookup_suffix(tensors, ["w1.weight", "up_proj.weight"])
        if up is None:
            raise C.EKError(C.EK_WEIGHT_NOT_FOUND, "w1/up_w")
        down = cls._lookup_suffix(tensors, ["w2.weight", "down_proj.weight"])
        if down is None:
            raise C.EKError(C.EK_WEIGHT_NOT_FOUND, "w2/down_w")
        gate = cls._lookup_suffix(tensors, ["w3.weight", "gate_proj.weight"])
        if gate is None:
            raise C.EKError(C.EK_WEIGHT_NOT_FOUND, "w3/gate_w")
        return cls(up_w=up, gate_w=gate, down_w=down,
                   up_scale=cls._lookup_suffix(tensors, ["w1.weight_scale", "up_proj.weight_scale",
                                                         "w1.weight_scale_inv", "up_proj.weight_scale_inv"]),
                   gate_scale=cls._lookup_suffix(tensors, ["w3.weight_scale", "gate_proj.weight_scale",
                                                           "w3.weight_scale_inv", "gate_proj.weight_scale_inv"]),
                   down_scale=cls._lookup_suffix(tensors, ["w2.weight_scale", "down_proj.weight_scale",
                                                           "w2.weight_scale_inv", "down_proj.weight_scale_inv"]))

    @classmethod
    def from_rand_linear(cls, hidden: int, intermediate: int, dtype=torch.bfloat16, device="cpu"):
        """ffn/meta.rs:77-89."""
        return cls(up_w=torch.rand(intermediate, hidden, device=device).to(dtype),
                   gate_w=torch.rand(intermediate, hidden, device=device).to(dtype),
                   down_w=torch.rand(hidden, intermediate, device=device).to(dtype))


def _desc(w: Optional[torch.Tensor], scale: Optional[torch.Tensor]):
    """Builds an ek_weight_desc; returns (desc or None, keepalive)."""
    if w is None:
        return None, ()
    w = w.contiguous()
    d = C.ek_weight_desc()
    d.ptr = w.data_ptr()
    d.rows, d.cols = w.shape
    d.dtype = _DT[w.dtype]
    d.mem = _mem(w)
    keep = [w]
    if scale is not None:
        scale = scale.contiguous()
        if scale.is_cuda != w.is_cuda:
            scale = scale.to(w.device)
        d.scale = scale.data_ptr()
        d.scale_dtype = _DT[scale.dtype]
        # [rows] = per output channel; [rows/128, cols/128] = the checkpoint's weight_scale_inv blocks
        d.scale_kind = C.EK_SCALE_PER_CHANNEL if scale.dim() == 1 else C.EK_SCALE_BLOCK128
        keep.append(scale)
    else:
        d.scale = None
        d.scale_dtype = C.EK_F32
        d.scale_kind = C.EK_SCALE_NONE
    return d, keep


@dataclass
class RouterConfig:
    """Which of the reference shims' routers to run in front of pack (ek_router_cfg)."""
    kind: int = C.EK_ROUTER_SOFTMAX_TOPK
    renorm: bool = True              # norm_topk_prob
    n_group: int = 1
    topk_group: int = 1
    routed_scaling: float = 1.0
    mask_neg_inf: bool = False
    w_dtype: Optional[torch.dtype] = None    # None: the layer's activation dtype
    bias: Optional[torch.Tensor] = None      # e_score_correction_bias [E] fp32


@dataclass
class RouteTables:
    counts: torch.Tensor
    offsets: torch.Tensor
    perm: torch.Tensor
    inv_perm: torch.Tensor


class HipLayer:
    """The experts of one MoE layer, resident in HBM, with the fused layer call."""

    def __init__(self, hidden: int, inter: int, n_experts: int, top_k: int, act_dtype=torch.bfloat16,
                 w_dtype=None, max_tokens: int = 1024, device_id: int = 0, block_scales: bool = False):
        """w_dtype: None (= act_dtype), torch.int8 (one scale per output channel; with block_scales the
        int8 tensors of a Block-INT8 checkpoint kept with their 128x128 scales) or torch.float8_e4m3fn
        (an FP8 checkpoint's tensors kept with their 128x128 scales)."""
        self._lib = C.load()
        self.cfg = C.ek_cfg(hidden=hidden, inter=inter, n_experts=n_experts, top_k=top_k,
                            act_dtype=_DT[act_dtype], w_dtype=_DT[w_dtype or act_dtype],
                            max_tokens=max_tokens, device_id=device_id,
                            flags=C.EK_CFG_BLOCK_SCALES if block_scales else 0)
        self.act_dtype = act_dtype
        self._h = ctypes.c_void_p()
        C.check(self._lib.ek_layer_create(ctypes.byref(self.cfg), ctypes.byref(self._h)))

    # -- ExpertDB ---------------------------------------------------------
    def set_expert(self, e: int, weight: ExpertWeight) -> None:
        up, k1 = _desc(weight.up_w, weight.up_scale)
        gate, k2 = _desc(weight.gate_w, weight.gate_scale)
        down, k3 = _desc(weight.down_w, weight.down_scale)
        ref = lambda d: ctypes.byref(d) if d is not None else None
        C.check(self._lib.ek_layer_set_expert(self._h, e, ref(up), ref(gate), ref(down)))
        del k1, k2, k3

    def set_shared_expert(self, weight: ExpertWeight) -> None:
        """DeepSeek's always-on shared expert (deepseek_v3/model.py:57-61,152) as one more segment."""
        self.set_expert(C.EK_SHARED_EXPERT, weight)

    def remove_expert(self, e: int) -> None:
        C.check(self._lib.ek_layer_remove_expert(self._h, e))

    def has_expert(self, e: int) -> bool:
        out = ctypes.c_int32(0)
        C.check(self._lib.ek_layer_has_expert(self._h, e, ctypes.byref(out)))
        return bool(out.value)

    # -- compute ----------------------------------------------------------
    def _route(self, T: int, device, expert_out: Optional[torch.Tensor] = None):
        E, K = self.cfg.n_experts, self.cfg.top_k
        rt = RouteTables(torch.empty(E, dtype=torch.int32, device=device),
                         torch.empty(E + 1, dtype=torch.int32, device=device),
                         torch.empty(T * K, dtype=torch.int32, device=device),
                         torch.empty(T * K, dtype=torch.int32, device=device))
        ro = C.ek_route_out(rt.counts.data_ptr(), rt.offsets.data_ptr(), rt.perm.data_ptr(),
                            rt.inv_perm.data_ptr(), 0 if expert_out is None else expert_out.data_ptr())
        return rt, ro

    def forward(self, x: torch.Tensor, ids: torch.Tensor, w: torch.Tensor, return_route: bool = False,
                stream=None, out: Optional[torch.Tensor] = None, expert_out: Optional[torch.Tensor] = None):
        """y[T,H] = sum_k w[t,k] * expert_{ids[t,k]}(x[t]); see ek_layer_forward.
        expert_out (with return_route): a [T*K, H] tensor beside x that receives every pair's expert
        output in packed order (ek_route_out.expert_out)."""
        assert x.dim() == 2 and ids.dim() == 2 and w.shape == ids.shape
        x, ids, w = x.contiguous(), ids.contiguous(), w.contiguous()
        assert ids.dtype == torch.int32 and x.dtype == self.act_dtype
        assert x.is_cuda == ids.is_cuda == w.is_cuda
        T = x.shape[0]
        if expert_out is not None:
            assert return_route and expert_out.is_contiguous() and expert_out.dtype == x.dtype
            assert expert_out.is_cuda == x.is_cuda and tuple(expert_out.shape) == (ids.numel(), x.shape[1])
        with (_alloc_on(stream) if out is None or return_route else _NO_CTX):
            y = out if out is not None else torch.empty_like(x)
            rt, ro = self._route(T, x.device, expert_out) if return_route else (None, None)
        C.check(self._lib.ek_layer_forward(self._h, _ptr(x), _ptr(ids), _ptr(w), _DT[w.dtype], T, _ptr(y),
                                           ctypes.byref(ro) if ro is not None else None, _mem(x),
                                           _stream_ptr(stream)))
        return (y, rt) if return_route else y

    def forward_static(self, x: torch.Tensor, ids: torch.Tensor, w: torch.Tensor, return_route: bool = False,
                       stream=None, out: Optional[torch.Tensor] = None):
        """ek_layer_forward_static: the same call with its workspace in the library's static device
        array (no allocation inside the call); device tensors only.  `out` (and the routing tables,
        which this wrapper allocates before the call) are the caller's."""
        assert x.is_cuda and ids.is_cuda and w.is_cuda and x.dim() == 2 and w.shape == ids.shape
        assert x.is_contiguous() and ids.is_contiguous() and w.is_contiguous()
        assert ids.dtype == torch.int32 and x.dtype == self.act_dtype
        T = x.shape[0]
        with (_alloc_on(stream) if out is None or return_route else _NO_CTX):
            y = out if out is not None else torch.empty_like(x)
            rt, ro = self._route(T, x.device) if return_route else (None, None)
        C.check(self._lib.ek_layer_forward_static(self._h, _ptr(x), _ptr(ids), _ptr(w), _DT[w.dtype], T, _ptr(y),
                                                  ctypes.byref(ro) if ro is not None else None,
                                                  _stream_ptr(stream)))
        return (y, rt) if return_route else y

    def pack(self, ids: torch.Tensor, x: Optional[torch.Tensor] = None, stream=None):
        """Routing tables (and the gathered rows Xp if x is given)."""
        ids = ids.contiguous()
        T = ids.shape[0]
        with _alloc_on(stream):
            rt, ro = self._route(T, ids.device)
            xp = None
            if x is not None:
                x = x.contiguous()
                xp = torch.empty(T * self.cfg.top_k, x.shape[1], dtype=x.dtype, device=x.device)
        C.check(self._lib.ek_layer_pack(self._h, _ptr(ids), T, ctypes.byref(ro), _ptr(x), _ptr(xp),
                                        _mem(ids), _stream_ptr(stream)))
        return (rt, xp) if x is not None else rt

    def expert_forward(self, e: int, x: torch.Tensor, stream=None) -> torch.Tensor:
        assert x.dim() == 2, "input must be rank 2 (ffn/mod.rs:45)"
        with _alloc_on(stream):
            x = x.contiguous()
            out = torch.empty_like(x)
        C.check(self._lib.ek_layer_expert_forward(self._h, e, _ptr(x), x.shape[0], _ptr(out), _mem(x),
                                                  _stream_ptr(stream)))
        return out

    def _router_cfg(self, r: RouterConfig, logits: torch.Tensor):
        cfg = C.ek_router_cfg(kind=r.kind, renorm=int(r.renorm), n_group=r.n_group, topk_group=r.topk_group,
                              routed_scaling=r.routed_scaling,
                              flags=C.EK_ROUTER_MASK_NEG_INF if r.mask_neg_inf else 0,
                              logits_dtype=_DT[logits.dtype], w_dtype=_DT[r.w_dtype or self.act_dtype])
        bias = None
        if r.bias is not None:
            bias = r.bias.to(device=logits.device, dtype=torch.float32).contiguous()
            cfg.bias = bias.data_ptr()
        return cfg, bias

    def route(self, logits: torch.Tensor, router: RouterConfig, stream=None):
        """logits [T,E] -> (ids [T,K] int32, w [T,K])."""
        logits = logits.contiguous()
        T, K = logits.shape[0], self.cfg.top_k
        cfg, keep = self._router_cfg(router, logits)
        with _alloc_on(stream):
            ids = torch.empty(T, K, dtype=torch.int32, device=logits.device)
            w = torch.empty(T, K, dtype=router.w_dtype or self.act_dtype, device=logits.device)
        C.check(self._lib.ek_layer_route(self._h, _ptr(logits), ctypes.byref(cfg), T, _ptr(ids), _ptr(w),
                                         _mem(logits), _stream_ptr(stream)))
        del keep
        return ids, w

    def forward_logits(self, x: torch.Tensor, logits: torch.Tensor, router: RouterConfig, stream=None):
        """Router + layer in one call; returns (y, ids, w)."""
        x, logits = x.contiguous(), logits.contiguous()
        T, K = x.shape[0], self.cfg.top_k
        assert logits.shape[0] == T and _mem(x) == _mem(logits)
        cfg, keep = self._router_cfg(router, logits)
        with _alloc_on(stream):
            y = torch.empty_like(x)
            ids = torch.empty(T, K, dtype=torch.int32, device=x.device)
            w = torch.empty(T, K, dtype=router.w_dtype or self.act_dtype, device=x.device)
        C.check(self._lib.ek_layer_forward_logits(self._h, _ptr(x), _ptr(logits), ctypes.byref(cfg), T, _ptr(y),
                                                  _ptr(ids), _ptr(w), None, _mem(x), _stream_ptr(stream)))
        del keep
        return y, ids, w

    def experts_forward(self, experts: Sequence[int], xs: Sequence[torch.Tensor], stream=None):
        """Several per-expert calls as one grouped launch; xs[i] is [n_i, H]."""
        n = len(experts)
        assert n == len(xs)
        with _alloc_on(stream):
            xs = [x.contiguous() for x in xs]
            outs = [torch.empty_like(x) for x in xs]
        mem = _mem(xs[0]) if n else C.EK_HOST
        assert all(_mem(x) == mem for x in xs)
        ex = (ctypes.c_int32 * n)(*experts)
        rows = (ctypes.c_int64 * n)(*[x.shape[0] for x in xs])
        xp = (ctypes.c_void_p * n)(*[x.data_ptr() for x in xs])
        op = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
        C.check(self._lib.ek_layer_experts_forward(self._h, n, ex, xp, rows, op, mem, _stream_ptr(stream)))
        return outs

    def set_expert_safetensors(self, e: int, blob: bytes) -> None:
        """ExpertBackend::build from the bytes ek-db serves for one expert (ffn/mod.rs:27-34)."""
        C.check(self._lib.ek_layer_set_expert_safetensors(self._h, e, blob, len(blob)))

    def worker_forward(self, expert_id: str, req: bytes) -> bytes:
        """EKInstanceGate::forward on wire bytes (worker/core.rs:47-74)."""
        return self.worker_forward_batch([expert_id], [req])[0]

    def worker_forward_batch(self, expert_ids: Sequence[str], reqs: Sequence[bytes]):
        n = len(expert_ids)
        assert n == len(reqs)
        # a response is never larger than its request: same tensor name, dtype and shape
        caps = [len(r) + 64 for r in reqs]
        bufs = [ctypes.create_string_buffer(c) for c in caps]
        ids = (ctypes.c_char_p * n)(*[i.encode() for i in expert_ids])
        rp = (ctypes.c_void_p * n)(*[ctypes.cast(ctypes.c_char_p(r), ctypes.c_void_p).value for r in reqs])
        rl = (ctypes.c_size_t * n)(*[len(r) for r in reqs])
        op = (ctypes.c_void_p * n)(*[ctypes.addressof(b) for b in bufs])
        oc = (ctypes.c_size_t * n)(*caps)
        ol = (ctypes.c_size_t * n)()
        C.check(self._lib.ek_worker_forward_batch(self._h, n, ids, rp, rl, op, oc, ol))
        return [bufs[i].raw[:ol[i]] for i in range(n)]

    def activation(self) -> torch.Tensor:
        """worker_expert_activation: rows given to each expert so far (metrics.rs:56-62)."""
        out = (ctypes.c_int64 * self.cfg.n_experts)()
        C.check(self._lib.ek_layer_get_activation(self._h, out))
        return torch.tensor(list(out), dtype=torch.int64)

    def forward_histogram(self) -> dict:
        """worker_forward: durations of blocking compute calls in the reference's buckets."""
        h = C.ek_histogram()
        C.check(self._lib.ek_layer_get_forward_histogram(self._h, ctypes.byref(h)))
        return {"le": list(h.le), "cumulative": list(h.cumulative), "sum": h.sum, "count": h.count}

    def profile(self, enable) -> None:
        """True / 1: per-phase events on every call; n > 1: on every n-th call; False / 0: off."""
        C.check(self._lib.ek_layer_profile(self._h, int(enable)))

    def stats(self) -> dict:
        s = C.ek_stats()
        C.check(self._lib.ek_layer_get_stats(self._h, ctypes.byref(s)))
        d = {f: getattr(s, f) for f, _ in s._fields_}
        d["kernel_us"] = list(s.kernel_us)
        return d

    def close(self) -> None:
        if getattr(self, "_h", None) is not None and self._h.value:
            self._lib.ek_layer_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class HipChain:
    """L consecutive MoE layers (x_{l+1} = y_l) launched as one HIP graph."""

    def __init__(self, layers: Sequence[HipLayer]):
        self._lib = C.load()
        self.layers = list(layers)
        arr = (ctypes.c_void_p * len(self.layers))(*[l._h.value for l in self.layers])
        self._h = ctypes.c_void_p()
        C.check(self._lib.ek_chain_create(arr, len(self.layers), ctypes.byref(self._h)))

    def forward(self, x: torch.Tensor, ids: torch.Tensor, w: torch.Tensor, use_graph: bool = True, stream=None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """ids, w: [L, T, K] on the device."""
        assert x.is_cuda and ids.is_cuda and w.is_cuda and ids.dtype == torch.int32
        assert x.is_contiguous() and ids.is_contiguous() and w.is_contiguous()
        assert ids.dim() == 3 and ids.shape[0] == len(self.layers) and w.shape == ids.shape
        with (_alloc_on(stream) if out is None else _NO_CTX):
            y = out if out is not None else torch.empty_like(x)
        C.check(self._lib.ek_chain_forward(self._h, _ptr(x), _ptr(ids), _ptr(w), _DT[w.dtype], x.shape[0], _ptr(y),
                                           int(use_graph), _stream_ptr(stream)))
        return y

    def close(self) -> None:
        if getattr(self, "_h", None) is not None and self._h.value:
            self._lib.ek_chain_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class HipBatcher:
    """Collector of concurrent per-expert requests (one Forward RPC per expert and task,
    worker/server.rs:39-63): `forward` may be called from many threads at once; the calls in
    flight together are answered by one grouped launch."""

    def __init__(self, layer: HipLayer, max_wait_us: int = 0, max_calls: int = 256):
        self._lib = C.load()
        self.layer = layer
        self._h = ctypes.c_void_p()
        C.check(self._lib.ek_batcher_create(layer._h, max_wait_us, max_calls, ctypes.byref(self._h)))

    def forward(self, expert_id: str, req: bytes) -> bytes:
        cap = len(req) + 64                     # a response is never larger than its request
        buf = ctypes.create_string_buffer(cap)
        n = ctypes.c_size_t()
        C.check(self._lib.ek_batcher_forward(self._h, expert_id.encode(), req, len(req), buf, cap, ctypes.byref(n)))
        return buf.raw[:n.value]

    def stats(self) -> dict:
        st = C.ek_batcher_stats()
        C.check(self._lib.ek_batcher_get_stats(self._h, ctypes.byref(st)))
        return {"calls": st.calls, "batches": st.batches, "largest_batch": st.largest_batch}

    def close(self) -> None:
        if getattr(self, "_h", None) is not None and self._h.value:
            C.check(self._lib.ek_batcher_destroy(self._h))
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class HipFFN:
    """One expert behind trait Expert<T> (ffn/meta.rs:30-39)."""

    def __init__(self, handle, lib, instance: EKInstance, act_dtype, device: str):
        self._h, self._lib, self._instance, self._act_dtype, self._device = handle, lib, instance, act_dtype, device

    @classmethod
    def construct(cls, x: EKInstance, weight: ExpertWeight, act_dtype=torch.bfloat16, max_rows: int = 4096,
                  device_id: int = 0) -> "HipFFN":
        lib = C.load()
        per_channel_i8 = (weight.up_w is not None and weight.up_w.dtype == torch.int8
                          and weight.up_scale is not None and weight.up_scale.dim() == 1)
        w_dtype = torch.int8 if per_channel_i8 else act_dtype
        cfg = C.ek_cfg(hidden=x.hidden, inter=x.intermediate, n_experts=1, top_k=1, act_dtype=_DT[act_dtype],
                       w_dtype=_DT[w_dtype], max_tokens=max_rows, device_id=device_id, flags=0)
        up, k1 = _desc(weight.up_w, weight.up_scale)
        gate, k2 = _desc(weight.gate_w, weight.gate_scale)
        down, k3 = _desc(weight.down_w, weight.down_scale)
        ref = lambda d: ctypes.byref(d) if d is not None else None
        h = ctypes.c_void_p()
        C.check(lib.ek_expert_create(ctypes.byref(cfg), max_rows, ref(up), ref(gate), ref(down), ctypes.byref(h)))
        del k1, k2, k3
        return cls(h, lib, x, act_dtype, f"cuda:{device_id}")

    def backend(self) -> str:
        return self._lib.ek_backend_name().decode()

    def shape(self):
        hidden, inter = ctypes.c_int64(), ctypes.c_int64()
        C.check(self._lib.ek_expert_shape(self._h, ctypes.byref(hidden), ctypes.byref(inter)))
        return hidden.value, inter.value

    def rand_input(self, batch: int) -> torch.Tensor:
        return torch.rand(batch, self._instance.hidden).to(self._act_dtype)

    def forward(self, x: torch.Tensor, stream=None) -> torch.Tensor:
        with _alloc_on(stream):
            x = x.contiguous()
            out = torch.empty_like(x)
        C.check(self._lib.ek_expert_forward(self._h, _ptr(x), x.shape[0], _ptr(out), _mem(x), _stream_ptr(stream)))
        return out

    def close(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            self._lib.ek_expert_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class ExpertBackend:
    """enum ExpertBackend { Torch, OnnxF32 } + the new Hip variant (ffn/mod.rs:17-53)."""

    def __init__(self, exp: HipFFN):
        self.exp = exp

    @classmethod
    def build(cls, instance: EKInstance, tensors: Dict[str, torch.Tensor], **kw) -> "ExpertBackend":
        if instance.backend != "hip":
            raise NotImplementedError(f"backend {instance.backend!r} (x.rs:18-24 knows torch/ort; this library adds hip)")
        weight = ExpertWeight.from_safetensor(tensors)
        return cls(HipFFN.construct(instance, weight, **kw))

    def forward(self, view: torch.Tensor) -> torch.Tensor:
        assert view.dim() == 2  # ffn/mod.rs:45
        return self.exp.forward(view)
