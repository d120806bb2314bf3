"""Writes the golden vectors of tests/golden/ (run from the repository root:
`python tests/golden/make_golden.py`).

The reference's own fixtures for this path are Git-LFS pointers without content, so
these vectors are produced by the CPU oracle (oracle/ek_oracle.c) at the moment it is
pinned by tests/test_oracle_*.py, and frozen: the oracle, its libtorch twin and the
HIP path are all compared against the same stored bytes from then on.  Every case is
small (a few hundred KiB): inputs, routing tables, the [T,K,H] expert outputs and the
combined result, all stored with safetensors.
"""
import os
import sys

import torch
from safetensors.torch import save_file

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path[:0] = [ROOT, os.path.join(ROOT, "expert-kit_amd")]
from oracle import oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

# name: (H, I, E, K, T, activation dtype, one-byte weights: False | True (int8 per channel) | "fp8" (e4m3fn
#        with 128x128 block scales), gate weights kept in fp32)
CASES = {
    "layer_bf16": (128, 64, 6, 2, 37, torch.bfloat16, False, False),
    "layer_f16_w32": (64, 128, 5, 3, 29, torch.float16, False, True),
    "layer_w8a16": (128, 128, 4, 2, 33, torch.bfloat16, True, False),
    "layer_fp8_block": (256, 128, 3, 2, 35, torch.bfloat16, "fp8", False),
}


def make_case(name):
    H, I, E, K, T, dt, w8, w_f32 = CASES[name]
    g = torch.Generator().manual_seed(sum(name.encode()))
    out = {}
    x = torch.randn(T, H, generator=g).to(dt)
    logits = torch.randn(T, E, generator=g)
    logits[:, E - 1] = -30.0                      # one expert never chosen: an empty segment
    ids, w = oracle.route(0, logits, K, True, w_dtype=torch.float32 if w_f32 else dt)
    wu, wg, wd = [], [], []
    for e in range(E):
        if w8 == "fp8":
            q = [(torch.randn(s, generator=g) * 110).clamp(-448, 448).to(torch.float8_e4m3fn) for s in ((I, H), (I, H), (H, I))]
            sc = [torch.rand((r + 127) // 128, (c + 127) // 128, generator=g) * 3e-4 + 5e-5 for r, c in ((I, H), (I, H), (H, I))]
            for m, (qq, ss) in zip(("up", "gate", "down"), zip(q, sc)):
                out[f"e{e}.{m}_q"], out[f"e{e}.{m}_scale"] = qq, ss
            deq = [oracle.dequant_block(oracle.fp8_e4m3fn_to_f32(qq), ss) for qq, ss in zip(q, sc)]
        elif w8:
            q = [torch.randint(-127, 128, s, generator=g, dtype=torch.int8) for s in ((I, H), (I, H), (H, I))]
            sc = [(torch.rand(n, generator=g) * 3e-3 + 1e-3).to(torch.bfloat16) for n in (I, I, H)]
            for m, (qq, ss) in zip(("up", "gate", "down"), zip(q, sc)):
                out[f"e{e}.{m}_q"], out[f"e{e}.{m}_scale"] = qq, ss
            deq = [oracle.dequant_channel(qq, ss, dt) for qq, ss in zip(q, sc)]
        else:
            deq = [(torch.randn(s, generator=g) * 0.08).to(dt) for s in ((I, H), (I, H), (H, I))]
        for m, t in zip(("up", "gate", "down"), deq):
            out[f"e{e}.{m}_w"] = t                # for int8: the dequantised weights the FFN must see
        wu.append(deq[0]); wg.append(deq[1]); wd.append(deq[2])
    y, counts, offsets, perm, inv, y3 = oracle.layer_forward(x, ids, w, wu, wg, wd, mode=0, return_y3=True)
    y_before_rounding = oracle.layer_forward(x, ids, w, wu, wg, wd, mode=2)[0]
    out.update(x=x, logits=logits, ids=ids, w=w, counts=counts, offsets=offsets, perm=perm, inv_perm=inv,
               xp=oracle.gather(x, perm, K), y3=y3, y=y, y_before_rounding=y_before_rounding)
    return out


def make_router_case():
    g = torch.Generator().manual_seed(77)
    T, E, K = 48, 64, 6
    logits = torch.randn(T, E, generator=g) * 1.5
    bias = torch.randn(E, generator=g) * 0.2
    out = {"logits": logits, "bias": bias}
    for kind in range(4):
        ids, w = oracle.route(kind, logits, K, True)
        out[f"kind{kind}.ids"], out[f"kind{kind}.w"] = ids, w
    for tag, neg in (("zero", False), ("neginf", True)):
        ids, w = oracle.route(4, logits, K, True, bias=bias, n_group=8, topk_group=3, mask_neg_inf=neg,
                              routed_scaling=2.5)
        out[f"kind4_{tag}.ids"], out[f"kind4_{tag}.w"] = ids, w
    return out


if __name__ == "__main__":
    for name in CASES:
        save_file({k: v.contiguous() for k, v in make_case(name).items()}, os.path.join(HERE, name + ".safetensors"))
    save_file(make_router_case(), os.path.join(HERE, "router.safetensors"))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".safetensors"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
