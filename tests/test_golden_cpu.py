"""The committed golden vectors (tests/golden/*.safetensors, written by make_golden.py) against
the oracle as it is now, against independent restatements, and against what the arithmetic fixes.
The reference's own fixtures for this path are Git-LFS pointers without content; these vectors
are the frozen stand-in that every implementation here is compared with."""
import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
LAYER_CASES = ["layer_bf16", "layer_f16_w32", "layer_w8a16", "layer_fp8_block"]


def load_case(name):
    t = load_file(os.path.join(HERE, name + ".safetensors"))
    E = 1 + max(int(k.split(".")[0][1:]) for k in t if k[0] == "e" and k[1].isdigit())
    wu, wg, wd = ([t[f"e{e}.{m}_w"] for e in range(E)] for m in ("up", "gate", "down"))
    return t, E, wu, wg, wd


def bits(a):
    return a.contiguous().view(torch.int16 if a.element_size() == 2 else torch.int32)


@pytest.mark.parametrize("name", LAYER_CASES)
def test_oracle_reproduces_the_vectors(oracle, name):
    t, E, wu, wg, wd = load_case(name)
    K = t["ids"].shape[1]
    ids, w = oracle.route(0, t["logits"], K, True, w_dtype=t["w"].dtype)
    assert torch.equal(ids, t["ids"]) and torch.equal(bits(w), bits(t["w"]))
    y, counts, offsets, perm, inv, y3 = oracle.layer_forward(t["x"], ids, w, wu, wg, wd, mode=0, return_y3=True)
    for got, key in ((counts, "counts"), (offsets, "offsets"), (perm, "perm"), (inv, "inv_perm")):
        assert torch.equal(got, t[key]), key
    assert torch.equal(bits(y3), bits(t["y3"])) and torch.equal(bits(y), bits(t["y"]))
    assert torch.equal(bits(oracle.gather(t["x"], perm, K)), bits(t["xp"]))
    assert int(t["counts"][E - 1]) == 0                     # the case holds an empty segment
    if name in ("layer_w8a16", "layer_fp8_block"):
        for e in range(E):
            for m in ("up", "gate", "down"):
                q, sc = t[f"e{e}.{m}_q"], t[f"e{e}.{m}_scale"]
                deq = oracle.dequant_channel(q, sc, torch.bfloat16) if name == "layer_w8a16" else \
                    oracle.dequant_block(oracle.fp8_e4m3fn_to_f32(q), sc)
                assert torch.equal(bits(deq), bits(t[f"e{e}.{m}_w"]))


@pytest.mark.parametrize("name", LAYER_CASES)
def test_vectors_against_independent_forms(oracle, name):
    t, E, wu, wg, wd = load_case(name)
    T, K = t["ids"].shape
    dt = t["x"].dtype
    # grouping: O(P*E) brute force
    for got, key in zip(oracle.brute_pack(t["ids"], E), ("counts", "offsets", "perm", "inv_perm")):
        assert torch.equal(got, t[key]), key
    # gather: plain indexing
    assert torch.equal(bits(t["x"][(t["perm"].long() // K)]), bits(t["xp"]))
    # FFN: float64 closed form of expert_torch.rs:81-84 (no intermediate rounding) per (token, slot)
    x64 = t["x"].double()
    y3 = t["y3"].double()
    ideal = torch.empty_like(y3)
    for tok in range(T):
        for k in range(K):
            e = int(t["ids"][tok, k])
            up, gate = wu[e].double() @ x64[tok], wg[e].double() @ x64[tok]
            ideal[tok, k] = wd[e].double() @ (up * gate / (1 + torch.exp(-gate)))
    rms = float(ideal.pow(2).mean().sqrt())
    err = float((y3 - ideal).abs().max()) / rms
    err_rms = float((y3 - ideal).pow(2).mean().sqrt()) / rms
    print(f"{name}: stored y3 vs float64 closed form: max|err|/rms = {err:.2e}, rms(err)/rms = {err_rms:.2e}")
    # five roundings to the 16-bit type (a bf16 ulp at 4 sigma is 3e-2 x rms); a wrong operand gives O(1)
    assert err < (1e-1 if dt == torch.bfloat16 else 1.25e-2)
    assert err_rms < (1e-2 if dt == torch.bfloat16 else 1.25e-3)
    # combine: float64 weighted sum of the stored y3, one rounding
    y64 = (t["w"].double().unsqueeze(-1) * y3).sum(1)
    ulp = 2.0 ** (-8 if dt == torch.bfloat16 else -11)
    mag = (t["w"].double().unsqueeze(-1) * y3).abs().sum(1)      # products are rounded one by one, then the sum
    assert bool(((t["y"].double() - y64).abs() <= 2 * ulp * mag + 1e-12).all())
    assert bool(((t["y_before_rounding"].double() - t["y"].double()).abs() <= ulp * t["y"].double().abs() + 1e-12).all())
    # libtorch running the reference's op sequence
    ty, done = oracle.torch_layer_forward(t["x"], t["ids"], t["w"], wu, wg, wd)
    assert done == T * K
    same = float((bits(ty) == bits(t["y"])).float().mean())
    print(f"{name}: libtorch twin bit-identical on {same:.4f} of the outputs")
    assert same > 0.9
    assert float((ty.double() - t["y"].double()).abs().max()) <= 2e-2 * rms
    # int8: the stored dequantised weights are the exact product rounded once
    if name == "layer_w8a16":
        q, s = t["e1.down_q"], t["e1.down_scale"]
        exact = (q.double() * s.double().unsqueeze(1))
        assert torch.equal(bits(exact.float().to(torch.bfloat16)), bits(t["e1.down_w"]))
    # fp8 with block scales: libtorch's widening, the fp32 product w8a16_activate forms
    # (expert_torch.rs:45-52), one rounding; the down matrix [256,128] spans two row blocks
    if name == "layer_fp8_block":
        q, s = t["e1.down_q"], t["e1.down_scale"]
        assert tuple(s.shape) == (2, 1) and q.dtype == torch.float8_e4m3fn
        full = s.repeat_interleave(128, 0).repeat_interleave(128, 1)
        assert torch.equal(bits((q.float() * full).to(torch.bfloat16)), bits(t["e1.down_w"]))


def test_router_vectors(oracle):
    t = load_file(os.path.join(HERE, "router.safetensors"))
    logits, bias = t["logits"], t["bias"]
    K = t["kind0.ids"].shape[1]
    for kind in range(4):
        ids, w = oracle.route(kind, logits, K, True)
        assert torch.equal(ids, t[f"kind{kind}.ids"]) and torch.equal(bits(w), bits(t[f"kind{kind}.w"]))
        t_ids, t_w = oracle.torch_route(kind, logits, K, True)
        assert torch.equal(t_ids, t[f"kind{kind}.ids"])
        assert float((t_w - t[f"kind{kind}.w"]).abs().max()) < 1e-6 * max(1.0, float(t_w.abs().max()))
    for tag, neg in (("zero", False), ("neginf", True)):
        kw = dict(bias=bias, n_group=8, topk_group=3, mask_neg_inf=neg, routed_scaling=2.5)
        ids, w = oracle.route(4, logits, K, True, **kw)
        assert torch.equal(ids, t[f"kind4_{tag}.ids"]) and torch.equal(bits(w), bits(t[f"kind4_{tag}.w"]))
        t_ids, t_w = oracle.torch_route(4, logits, K, True, **kw)
        assert torch.equal(t_ids.sort(1)[0], t[f"kind4_{tag}.ids"].sort(1)[0])
        assert abs(float(t[f"kind4_{tag}.w"].sum(1).mean()) - 2.5) < 1e-5      # renormalised, then scaled
    # every chosen expert of kind 4 lies in one of at most topk_group = 3 groups of 8
    groups = (t["kind4_zero.ids"] // 8)
    assert max(len(set(r.tolist())) for r in groups) <= 3
