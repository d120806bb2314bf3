"""The HIP path against the committed golden vectors (tests/golden/, see make_golden.py):
routing tables, gather and router ids bit-exact; outputs within the layer gate of
test_gpu_parity.py measured from the stored reference."""
import os

import pytest
import torch
from safetensors.torch import load_file

from test_golden_cpu import HERE, LAYER_CASES, bits, load_case
from test_gpu_parity import layer_gate

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", LAYER_CASES)
@pytest.mark.parametrize("mem", ["device", "host"])
def test_layer_matches_golden(ek, cuda, name, mem):
    t, E, wu, wg, wd = load_case(name)
    T, K = t["ids"].shape
    H, I = t["x"].shape[1], wu[0].shape[0]
    dt = t["x"].dtype
    w8 = name in ("layer_w8a16", "layer_fp8_block")          # one-byte weights with their scales, as stored
    w_dtype = torch.float8_e4m3fn if name == "layer_fp8_block" else torch.int8 if w8 else dt
    layer = ek.HipLayer(H, I, E, K, act_dtype=dt, w_dtype=w_dtype, max_tokens=64)
    for e in range(E):
        if w8:
            layer.set_expert(e, ek.ExpertWeight(up_w=t[f"e{e}.up_q"], gate_w=t[f"e{e}.gate_q"], down_w=t[f"e{e}.down_q"],
                                                up_scale=t[f"e{e}.up_scale"], gate_scale=t[f"e{e}.gate_scale"],
                                                down_scale=t[f"e{e}.down_scale"]))
        else:
            layer.set_expert(e, ek.ExpertWeight(up_w=wu[e], gate_w=wg[e], down_w=wd[e]))
    mv = (lambda a: a.to(cuda)) if mem == "device" else (lambda a: a)
    # router -> the stored ids and gate weights
    ids, w = layer.route(mv(t["logits"]), ek.RouterConfig(kind=0, w_dtype=t["w"].dtype))
    assert torch.equal(ids.cpu(), t["ids"])
    if t["w"].dtype == torch.float32:
        assert float(((w.cpu() - t["w"]).abs() / t["w"]).max()) < 4e-6
    else:
        assert int((bits(w.cpu()).int() - bits(t["w"]).int()).abs().max()) <= 1
    # pack + gather
    rt, xp = layer.pack(mv(t["ids"]), mv(t["x"]))
    for got, key in ((rt.counts, "counts"), (rt.offsets, "offsets"), (rt.perm, "perm"), (rt.inv_perm, "inv_perm")):
        assert torch.equal(got.cpu(), t[key]), key
    assert torch.equal(bits(xp.cpu()), bits(t["xp"]))
    # whole layer with the stored gate weights
    y = layer.forward(mv(t["x"]), mv(t["ids"]), mv(t["w"]))
    layer_gate(y, t["y_before_rounding"], t["y3"], t["w"], f"golden {name} ({mem})")
    same = float((bits(y.cpu()) == bits(t["y"])).float().mean())
    print(f"golden {name} ({mem}): bit-identical to the stored y on {same:.4f}", flush=True)
    assert same > 0.9
    layer.close()


def test_routers_match_golden(ek, cuda):
    t = load_file(os.path.join(HERE, "router.safetensors"))
    logits, bias = t["logits"], t["bias"]
    T, E = logits.shape
    K = t["kind0.ids"].shape[1]
    layer = ek.HipLayer(128, 128, E, K, max_tokens=64)
    for kind in range(4):
        ids, w = layer.route(logits.to(cuda), ek.RouterConfig(kind=kind, w_dtype=torch.float32))
        assert torch.equal(ids.cpu(), t[f"kind{kind}.ids"])
        if kind == 0:
            assert float(((w.cpu() - t["kind0.w"]).abs() / t["kind0.w"]).max()) < 4e-6
        else:
            assert torch.equal(bits(w.cpu()), bits(t[f"kind{kind}.w"]))
    for tag, neg in (("zero", False), ("neginf", True)):
        r = ek.RouterConfig(kind=4, bias=bias, n_group=8, topk_group=3, mask_neg_inf=neg, routed_scaling=2.5,
                            w_dtype=torch.float32)
        ids, w = layer.route(logits.to(cuda), r)
        assert torch.equal(ids.cpu(), t[f"kind4_{tag}.ids"])
        assert torch.equal(bits(w.cpu()), bits(t[f"kind4_{tag}.w"]))
    layer.close()
