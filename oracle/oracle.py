"""CPU oracle for the Expert Kit routed-expert path -- TEST INFRASTRUCTURE ONLY.

Two independent statements of the reference's arithmetic live here:

* thin ctypes wrappers over ``ek_oracle.c`` (scalar C, double accumulation,
  explicit round-to-nearest-even at the reference's rounding points), and
* ``torch_*`` functions that evaluate the same op sequence with the
  container's libtorch CPU kernels -- the library family the reference itself
  calls through ``tch`` (ek-computation/src/ffn/expert_torch.rs:80-85).

Only tests, the smoke check and the benchmark's ``cpu_baseline`` leg may import
this module; the shipped library never does.

Tensors cross this API as CPU ``torch.Tensor`` objects (bf16 / fp16 / fp32 for
activations and weights, int32 for routing tables).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

BF16, F16, F32 = 0, 1, 2
_DT = {torch.bfloat16: BF16, torch.float16: F16, torch.float32: F32}


def build() -> str:
    """Compile ek_oracle.c into libek_oracle.so (always recompiles)."""
    subprocess.check_call(["make", "-B", "-C", _HERE, "libek_oracle.so"], stdout=subprocess.DEVNULL)
    return os.path.join(_HERE, "libek_oracle.so")


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libek_oracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
        _LIB.eko_bf16_to_f32.restype = ctypes.c_float
        _LIB.eko_f16_to_f32.restype = ctypes.c_float
        _LIB.eko_f32_to_bf16.restype = ctypes.c_uint16
        _LIB.eko_f32_to_f16.restype = ctypes.c_uint16
        _LIB.eko_f32_to_bf16.argtypes = [ctypes.c_float]
        _LIB.eko_f32_to_f16.argtypes = [ctypes.c_float]
        _LIB.eko_bf16_to_f32.argtypes = [ctypes.c_uint16]
        _LIB.eko_f16_to_f32.argtypes = [ctypes.c_uint16]
    return _LIB


def _p(t: torch.Tensor | None):
    if t is None:
        return ctypes.c_void_p(0)
    assert t.device.type == "cpu" and t.is_contiguous(), "oracle takes contiguous CPU tensors"
    return ctypes.c_void_p(t.data_ptr())


def _i64(v):
    return ctypes.c_int64(int(v))


def _ptr_array(ts):
    arr = (ctypes.c_void_p * len(ts))()
    for i, t in enumerate(ts):
        arr[i] = None if t is None else t.data_ptr()
    return arr


# ----------------------------------------------------------------- C oracle


def router(logits: torch.Tensor, k: int, renorm: bool = True, w_dtype=torch.float32):
    """softmax(fp32) -> top-k -> renormalise -> cast (qwen3_moe.py:161-169)."""
    logits = logits.contiguous().float()
    T, E = logits.shape
    ids = torch.empty(T, k, dtype=torch.int32)
    w = torch.empty(T, k, dtype=w_dtype)
    rc = lib().eko_router_softmax_topk(_p(logits), _i64(T), E, k, int(renorm), _p(ids), _p(w), _DT[w_dtype])
    if rc:
        raise ValueError(f"eko_router_softmax_topk rc={rc}")
    return ids, w


def expf(x: torch.Tensor) -> torch.Tensor:
    """eko_expf element by element (the IEEE-operations-only exp the routers use)."""
    L = lib()
    L.eko_expf.restype = ctypes.c_float
    L.eko_expf.argtypes = [ctypes.c_float]
    return torch.tensor([L.eko_expf(float(v)) for v in x.flatten().tolist()], dtype=torch.float32).reshape(x.shape)


def silu_forms(g: torch.Tensor):
    """silu of fp32 gate values, element by element, in the form the HIP kernels evaluate (eko_expf_wide)
    and in the form eko_ffn evaluates (libm's expf): gate / (1 + exp(-gate)) both times."""
    L = lib()
    for f in (L.eko_silu_kernel_form, L.eko_silu_libm_form):
        f.restype = ctypes.c_float
        f.argtypes = [ctypes.c_float]
    v = g.flatten().tolist()
    a = torch.tensor([L.eko_silu_kernel_form(float(t)) for t in v], dtype=torch.float32).reshape(g.shape)
    b = torch.tensor([L.eko_silu_libm_form(float(t)) for t in v], dtype=torch.float32).reshape(g.shape)
    return a, b


def route(kind: int, logits: torch.Tensor, k: int, renorm: bool = True, w_dtype=torch.float32, bias=None,
          n_group: int = 1, topk_group: int = 1, mask_neg_inf: bool = False, routed_scaling: float = 1.0):
    """The reference shims' routers (see eko_route): kind 0 Qwen3, 1-3 the vLLM shims, 4 DeepSeek-V3."""
    logits = logits.contiguous()
    T, E = logits.shape
    ids = torch.empty(T, k, dtype=torch.int32)
    w = torch.empty(T, k, dtype=w_dtype)
    if bias is not None:
        bias = bias.contiguous().float()
    rc = lib().eko_route(kind, _p(logits), _DT[logits.dtype], _p(bias), _i64(T), E, k, int(renorm), n_group,
                         topk_group, int(mask_neg_inf), ctypes.c_float(routed_scaling), _p(ids), _p(w),
                         _DT[w_dtype])
    if rc:
        raise ValueError(f"eko_route rc={rc}")
    return ids, w


def pack(ids: torch.Tensor, n_experts: int):
    """Group (token, slot) pairs by expert (controller/executor.rs:283-304).

    Returns (counts[E], offsets[E+1], perm[P], inv_perm[P]) as int32 tensors.
    """
    flat = ids.reshape(-1).to(torch.int32).contiguous()
    P = flat.numel()
    counts = torch.empty(n_experts, dtype=torch.int32)
    offsets = torch.empty(n_experts + 1, dtype=torch.int32)
    perm = torch.empty(P, dtype=torch.int32)
    inv = torch.empty(P, dtype=torch.int32)
    rc = lib().eko_pack(_p(flat), _i64(P), n_experts, _p(counts), _p(offsets), _p(perm), _p(inv))
    if rc:
        raise ValueError(f"eko_pack rc={rc}: expert id out of range")
    return counts, offsets, perm, inv


def gather(x: torch.Tensor, perm: torch.Tensor, k: int) -> torch.Tensor:
    """Xp[j] = x[perm[j] // K] (controller/executor.rs:112-133)."""
    x = x.contiguous()
    P = perm.numel()
    xp = torch.empty(P, x.shape[1], dtype=x.dtype)
    lib().eko_gather(_p(x), _i64(x.shape[1]), x.element_size(), _p(perm.contiguous()), _i64(P), k, _p(xp))
    return xp


def scatter(yp: torch.Tensor, perm: torch.Tensor, T: int, k: int) -> torch.Tensor:
    """Y[t,k] = Yp[j] with perm[j] = t*K+k (controller/executor.rs:203-252)."""
    yp = yp.contiguous()
    H = yp.shape[1]
    y3 = torch.empty(T, k, H, dtype=yp.dtype)
    lib().eko_scatter(_p(yp), _i64(H), yp.element_size(), _p(perm.contiguous()), _i64(perm.numel()), _p(y3))
    return y3


def dequant_channel(q: torch.Tensor, scale: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    """W[n,:] = rne_dtype(f32(q[n,:]) * f32(scale[n])); q int8 [N,C], scale bf16 [N]."""
    q = q.contiguous()
    scale = scale.contiguous()
    assert q.dtype == torch.int8 and scale.dtype == torch.bfloat16
    N, C = q.shape
    w = torch.empty(N, C, dtype=dtype)
    lib().eko_dequant_channel(_p(q), _p(scale), _i64(N), _i64(C), _DT[dtype], _p(w))
    return w


def dequant_block(q: torch.Tensor, s: torch.Tensor, block: int = 128) -> torch.Tensor:
    """Block-scaled dequant (ffn/expert_torch.rs:24-53); q any dtype, s fp32."""
    qf = q.float().contiguous()
    s = s.float().contiguous()
    N, C = qf.shape
    w = torch.empty(N, C, dtype=torch.bfloat16)
    lib().eko_dequant_block(_p(qf), _p(s), _i64(N), _i64(C), _i64(block), _p(w))
    return w


def fp8_e4m3fn_to_f32(b: torch.Tensor) -> torch.Tensor:
    """Bytes of an fp8 e4m3fn tensor (uint8 or float8_e4m3fn) -> fp32 values (backend/mod.rs:13)."""
    raw = b.contiguous().view(torch.uint8)
    out = torch.empty(raw.shape, dtype=torch.float32)
    lib().eko_fp8_e4m3fn_to_f32(_p(raw), _i64(raw.numel()), _p(out))
    return out


def ffn(x, w_up, w_gate, w_down, mode: int = 0, return_h: bool = False):
    """One expert SwiGLU FFN (ffn/expert_torch.rs:80-85).

    mode 0: reference rounding points, result in x.dtype.
    mode 1: ideal (double, unrounded), result fp32.
    mode 2: as mode 0 with the last storage rounding left out, result fp32.
    mode 3: as mode 0 with every dot product accumulated in fp32 in index order.
    """
    dt = _DT[x.dtype]
    assert w_up.dtype == x.dtype and w_gate.dtype == x.dtype and w_down.dtype == x.dtype
    x = x.contiguous()
    n, H = x.shape
    I = w_up.shape[0]
    assert tuple(w_up.shape) == (I, H) and tuple(w_gate.shape) == (I, H) and tuple(w_down.shape) == (H, I)
    out = torch.empty(n, H, dtype=x.dtype if mode in (0, 3) else torch.float32)
    h = torch.empty(n, I, dtype=torch.float32 if mode == 1 else x.dtype) if return_h else None
    lib().eko_ffn(_p(x), _i64(n), _i64(H), _i64(I), _p(w_up.contiguous()), _p(w_gate.contiguous()),
                  _p(w_down.contiguous()), dt, mode, _p(out), _p(h))
    return (out, h) if return_h else out


def combine(y3: torch.Tensor, w: torch.Tensor, round_out: bool = True) -> torch.Tensor:
    """y[t] = sum_k w[t,k] * Y[t,k] (qwen3_moe.py:102-104; deepseek_v3/model.py:97-103).

    round_out=False returns the fp32 sum before its storage rounding."""
    y3 = y3.contiguous()
    w = w.contiguous()
    T, K, H = y3.shape
    y = torch.empty(T, H, dtype=y3.dtype if round_out else torch.float32)
    lib().eko_combine(_p(y3), _p(w), _i64(T), K, _i64(H), _DT[y3.dtype], _DT[w.dtype], int(round_out), _p(y))
    return y


def layer_forward(x, ids, w, w_up, w_gate, w_down, mode: int = 0, return_y3: bool = False):
    """Whole layer, Expert Kit form.  w_* are lists of E tensors (None allowed).

    Returns (y, counts, offsets, perm, inv_perm); y is x.dtype (mode 0; mode 3, the same with
    fp32 accumulation in index order) or fp32 (mode 1 ideal; mode 2 reference-rounded except
    for y's own storage rounding).
    With return_y3 the [T,K,H] tensor before the weighted sum is appended.
    """
    x = x.contiguous()
    T, H = x.shape
    K = ids.shape[1]
    E = len(w_up)
    I = next(t for t in w_up if t is not None).shape[0]
    ids = ids.to(torch.int32).contiguous()
    w = w.contiguous()
    P = T * K
    y = torch.empty(T, H, dtype=x.dtype if mode in (0, 3) else torch.float32)
    counts = torch.empty(E, dtype=torch.int32)
    offsets = torch.empty(E + 1, dtype=torch.int32)
    perm = torch.empty(P, dtype=torch.int32)
    inv = torch.empty(P, dtype=torch.int32)
    y3 = torch.empty(T, K, H, dtype=torch.float32 if mode == 1 else x.dtype) if return_y3 else None
    wu = [None if t is None else t.contiguous() for t in w_up]
    wg = [None if t is None else t.contiguous() for t in w_gate]
    wd = [None if t is None else t.contiguous() for t in w_down]
    rc = lib().eko_layer_forward(_p(x), _p(ids), _p(w), _i64(T), K, E, _i64(H), _i64(I), _ptr_array(wu),
                                 _ptr_array(wg), _ptr_array(wd), _DT[x.dtype], _DT[w.dtype], mode, _p(y),
                                 _p(counts), _p(offsets), _p(perm), _p(inv), _p(y3))
    if rc:
        raise ValueError(f"eko_layer_forward rc={rc}")
    return (y, counts, offsets, perm, inv, y3) if return_y3 else (y, counts, offsets, perm, inv)


def add_shared(y_routed: torch.Tensor, x: torch.Tensor, w_up, w_gate, w_down, rounded: bool = True):
    """hidden_states + shared_experts(residuals) (deepseek_v3/model.py:57-61,152): the routed result
    and the shared MLP's output are both tensors of the activation dtype; their sum is formed in
    fp32 and (rounded=True) stored in the activation dtype."""
    assert y_routed.dtype == x.dtype
    y_shared = ffn(x, w_up, w_gate, w_down, mode=0)
    total = y_routed.float() + y_shared.float()
    return total.to(x.dtype) if rounded else total


def layer_loop_form(x, ids, w, w_up, w_gate, w_down):
    """Whole layer, stock per-expert loop + index_add_ (qwen3_moe.py:115-151)."""
    x = x.contiguous()
    T, H = x.shape
    K = ids.shape[1]
    E = len(w_up)
    I = next(t for t in w_up if t is not None).shape[0]
    ids = ids.to(torch.int32).contiguous()
    y = torch.empty(T, H, dtype=x.dtype)
    wu = [None if t is None else t.contiguous() for t in w_up]
    wg = [None if t is None else t.contiguous() for t in w_gate]
    wd = [None if t is None else t.contiguous() for t in w_down]
    rc = lib().eko_layer_loop_form(_p(x), _p(ids), _p(w.contiguous()), _i64(T), K, E, _i64(H), _i64(I),
                                   _ptr_array(wu), _ptr_array(wg), _ptr_array(wd), _DT[x.dtype],
                                   _DT[w.dtype], _p(y))
    if rc:
        raise ValueError(f"eko_layer_loop_form rc={rc}")
    return y


# ------------------------------------------------------------ libtorch twin


def torch_router(logits: torch.Tensor, k: int, renorm: bool = True, w_dtype=torch.float32):
    """The router exactly as qwen3_moe.py:161-169 spells it."""
    rw = torch.nn.functional.softmax(logits, dim=1, dtype=torch.float)
    rw, sel = torch.topk(rw, k, dim=-1)
    if renorm:
        rw = rw / rw.sum(dim=-1, keepdim=True)
    return sel.to(torch.int32), rw.to(w_dtype)


def torch_route(kind: int, logits: torch.Tensor, k: int, renorm: bool = True, w_dtype=torch.float32, bias=None,
                n_group: int = 1, topk_group: int = 1, mask_neg_inf: bool = False, routed_scaling: float = 1.0):
    """The same routers in torch primitives, written after the reference's lines (kinds 0-3) and
    after the published DeepseekV3TopkRouter.forward (kind 4)."""
    if kind == 0:      # qwen3_moe.py:161-169
        p = torch.softmax(logits, dim=1, dtype=torch.float)
        w, ids = torch.topk(p, k, dim=-1)
        if renorm:
            w = w / w.sum(dim=-1, keepdim=True)
        return ids.to(torch.int32), w.to(w_dtype)
    if kind in (1, 2, 3):   # grpc_expert.py:120-121, deepseek_v2.py:123-130
        w, ids = torch.topk(logits, k, dim=-1)
        if kind == 2:
            w = torch.softmax(w, dim=-1)
        elif kind == 3:
            w = torch.sigmoid(w)
        return ids.to(torch.int32), w.to(w_dtype)
    T, E = logits.shape
    scores = logits.float().sigmoid()
    choice = scores + bias if bias is not None else scores.clone()
    group_scores = choice.view(T, n_group, E // n_group).topk(2, dim=-1)[0].sum(dim=-1)
    group_idx = torch.topk(group_scores, k=topk_group, dim=-1, sorted=False)[1]
    group_mask = torch.zeros_like(group_scores)
    group_mask.scatter_(1, group_idx, 1)
    score_mask = group_mask.unsqueeze(-1).expand(T, n_group, E // n_group).reshape(T, E)
    choice = choice.masked_fill(~score_mask.bool(), float("-inf") if mask_neg_inf else 0.0)
    ids = torch.topk(choice, k=k, dim=-1, sorted=True)[1]
    w = scores.gather(1, ids)
    if renorm:
        w = w / (w.sum(dim=-1, keepdim=True) + 1e-20)
    return ids.to(torch.int32), (w * routed_scaling).to(w_dtype)


def torch_dequant_channel(q: torch.Tensor, scale: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    """rne(f32(q) * f32(scale[n])) with libtorch ops: what a CPU backend holds
    after load_module's cast to its compute dtype (ffn/expert_torch.rs:61-78)."""
    if q.dtype != torch.int8:
        return q.cpu()
    return (q.cpu().float() * scale.cpu().float().unsqueeze(1)).to(dtype)


def torch_ffn(x, w_up, w_gate, w_down):
    """The four libtorch ops of ffn/expert_torch.rs:81-84, in that order."""
    up = x.matmul(w_up.transpose(0, 1))
    gate = x.matmul(w_gate.transpose(0, 1))
    hidden = up * torch.nn.functional.silu(gate)
    return hidden.matmul(w_down.transpose(0, 1))


def torch_layer_forward(x, ids, w, w_up, w_gate, w_down, experts=None):
    """Reference-equivalent CPU backend for one layer.

    For each active expert in ascending id: index_select its rows, run the four
    ops, place the rows in [T,K,H]; then sum(w.unsqueeze(-1) * Y, dim=1)
    (qwen3_moe.py:102-104).  ``experts`` restricts the loop to a subset (used
    for bounded CPU-baseline samples); rows of other experts stay zero.
    Returns (y, pairs_done).
    """
    T, H = x.shape
    K = ids.shape[1]
    flat = ids.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=len(w_up))
    y3 = torch.zeros(T * K, H, dtype=x.dtype)
    pos = 0
    done = 0
    for e in range(len(w_up)):
        n = int(counts[e])
        if n and (experts is None or e in experts):
            pairs = order[pos:pos + n]
            xe = x.index_select(0, pairs // K)
            y3[pairs] = torch_ffn(xe, w_up[e], w_gate[e], w_down[e])
            done += n
        pos += n
    y = torch.sum(w.unsqueeze(-1) * y3.view(T, K, H), dim=1)
    return y.to(x.dtype), done


# ------------------------------------------------------------- brute forces


def brute_pack(ids: torch.Tensor, n_experts: int):
    """O(P*E) statement of the grouping, independent of eko_pack."""
    flat = [int(v) for v in ids.reshape(-1)]
    perm = []
    counts = []
    for e in range(n_experts):
        mine = [p for p, v in enumerate(flat) if v == e]
        counts.append(len(mine))
        perm.extend(mine)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    inv = np.empty(len(flat), dtype=np.int32)
    inv[np.asarray(perm, dtype=np.int64)] = np.arange(len(flat), dtype=np.int32)
    return (torch.tensor(counts, dtype=torch.int32), torch.from_numpy(offsets),
            torch.tensor(perm, dtype=torch.int32), torch.from_numpy(inv))
