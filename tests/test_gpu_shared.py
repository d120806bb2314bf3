"""DeepSeek's shared expert as an always-on segment of the grouped launch.

Bars: (1) composition, bit-exact: the fused result equals round(y_routed + y_shared) where
y_routed is the same layer's result without the shared expert and y_shared the same weights'
output through the per-expert entry point (same kernels, same cut of the T rows);
(2) against the oracle: 2e-2 * rms of the reference plus the storage quanta of the two
16-bit summands and of the result.
"""
import pytest
import torch

from ek_hip import _capi as C
from ek_hip import workloads as wl
from test_gpu_parity import TOL, oracle_weights, ulp_of

pytestmark = pytest.mark.gpu

H, I, E, K = 256, 192, 8, 2


def build(ek, dt, w8, max_tokens=512, inter_shared=I):
    work = wl.Workload("shared", H, I, E + 1, K, 1, dt, w8=w8)
    ws = {e: wl.make_expert(work, e, std=0.05) for e in range(E)}
    # index E: the shared one, moe_intermediate_size * n_shared_experts channels wide
    ws[E] = wl.make_expert(wl.Workload("shared", H, inter_shared, E + 1, K, 1, dt, w8=w8), E, std=0.05)
    layer = ek.HipLayer(H, I, E, K, act_dtype=dt, w_dtype=torch.int8 if w8 else dt, max_tokens=max_tokens)
    for e in range(E):
        layer.set_expert(e, ws[e])
    return layer, ws


def routing(T, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32).reshape(T, K)
    w = torch.rand(T, K, generator=g) + 0.1
    return x, ids, w / w.sum(-1, keepdim=True)


@pytest.mark.parametrize("n_shared", [1, 2])
@pytest.mark.parametrize("dt,w8", [(torch.bfloat16, False), (torch.float16, False), (torch.bfloat16, True)])
def test_shared_expert_segment(ek, oracle, cuda, dt, w8, n_shared):
    """n_shared = 2: a shared expert of moe_intermediate_size * n_shared_experts channels
    (expertkit_torch/models/deepseek_v3/model.py:57-61; DeepSeek-V2-Lite has two): other shapes than
    the routed experts', so launches, work lists and an intermediate buffer of its own."""
    layer, ws = build(ek, dt, w8, inter_shared=I * n_shared)
    single = ek.HipLayer(H, I * n_shared, 1, 1, act_dtype=dt, w_dtype=torch.int8 if w8 else dt, max_tokens=512)
    single.set_expert(0, ws[E])
    wu, wg, wd = oracle_weights(oracle, ws, E + 1, dt)
    for T in (1, 16, 17, 33, 64, 65, 100, 130, 256, 257, 300):
        x, ids, w = routing(T, 40 + T)
        x, w = x.to(dt), w.to(dt)
        assert not layer.has_expert(C.EK_SHARED_EXPERT)
        y_plain = layer.forward(x.to(cuda), ids.to(cuda), w.to(cuda))
        layer.set_shared_expert(ws[E])
        assert layer.has_expert(C.EK_SHARED_EXPERT)
        y = layer.forward(x.to(cuda), ids.to(cuda), w.to(cuda))
        # (1) composition: the same expert as the only routed one with gate weight 1 is cut like the
        # shared segment (a per-expert call of this size may be cut for the other kernel family)
        # (up to 64 tokens the shared segment is a run of 16-row streaming items, up to 256 a run
        # of 64-row ones, which is how a lone per-expert call of that size is cut too)
        if T <= 64:
            y_sh = torch.cat(single.experts_forward([0] * ((T + 15) // 16), list(x.to(cuda).split(16))))
        elif T <= 256:
            y_sh = single.expert_forward(0, x.to(cuda))
        else:
            y_sh = single.forward(x.to(cuda), torch.zeros(T, 1, dtype=torch.int32, device=cuda),
                                  torch.ones(T, 1, dtype=dt, device=cuda))
        want = (y_plain.float() + y_sh.float()).to(dt)
        assert torch.equal(y.view(torch.int16), want.view(torch.int16)), T
        assert not torch.equal(y, y_plain)
        # host-memory call takes the same path
        assert torch.equal(layer.forward(x, ids, w).view(torch.int16), y.cpu().view(torch.int16))
        # (2) oracle
        y_r = oracle.layer_forward(x, ids, w, wu[:E], wg[:E], wd[:E], mode=0)[0]
        ref32 = oracle.add_shared(y_r, x, wu[E], wg[E], wd[E], rounded=False)
        y_s = ref32 - y_r.float()
        rms = float(ref32.pow(2).mean().sqrt())
        err = (y.float().cpu() - ref32).abs()
        quanta = 0.5 * ulp_of(ref32, dt) * 1.0001 + ulp_of(y_r.float(), dt) + ulp_of(y_s, dt)
        worst = float(err.max()) / rms
        over = float((err > TOL * rms).float().mean())
        print(f"shared x{n_shared} {dt} w8={w8} T={T}: max|err|/rms = {worst:.3e}, elements over 2e-2*rms: {over:.2e}", flush=True)
        assert bool((err <= TOL * rms + quanta).all()), worst
        assert over <= 1e-4 or T * H * over <= 2      # tiny outputs: allow two elements
        layer.remove_expert(C.EK_SHARED_EXPERT)
        again = layer.forward(x.to(cuda), ids.to(cuda), w.to(cuda))
        assert torch.equal(again.view(torch.int16), y_plain.view(torch.int16))
    assert layer.activation().shape == (E,)                    # the shared expert is not a routed expert
    with pytest.raises(ek.EKError) as ei:
        layer.remove_expert(C.EK_SHARED_EXPERT)
    assert ei.value.status == C.EK_EXPERT_NOT_FOUND
    layer.close()
    single.close()


def test_shared_expert_in_a_chain(ek, cuda):
    dt, L, T = torch.float16, 3, 90
    layers = []
    for l in range(L):
        work = wl.Workload("shared-chain", H, I, E + 1, K, 1, dt)
        layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=128)
        for e in range(E):
            layer.set_expert(e, wl.make_expert(work, e, layer=l, std=0.08))
        if l != 1:                                              # layers 0 and 2 have one, layer 1 does not
            layer.set_shared_expert(wl.make_expert(work, E, layer=l, std=0.08))
        layers.append(layer)
    x, _, _ = routing(T, 7)
    x = x.to(dt).to(cuda)
    ids = torch.stack([routing(T, 100 + l)[1] for l in range(L)]).to(cuda)
    w = torch.stack([routing(T, 100 + l)[2] for l in range(L)]).to(dt).to(cuda)
    step = x
    for l in range(L):
        step = layers[l].forward(step, ids[l], w[l])
    chain = ek.HipChain(layers)
    eager = chain.forward(x, ids, w, use_graph=False)
    assert torch.equal(eager.view(torch.int16), step.view(torch.int16))
    for rep in range(3):
        got = chain.forward(x, ids, w, use_graph=True)
        assert torch.equal(got.view(torch.int16), step.view(torch.int16)), rep
        torch.cuda.synchronize()
    # loading a shared expert into layer 1 changes the launches: the graph must be captured again
    work = wl.Workload("shared-chain", H, I, E + 1, K, 1, dt)
    layers[1].set_shared_expert(wl.make_expert(work, E, layer=1, std=0.08))
    step2 = x
    for l in range(L):
        step2 = layers[l].forward(step2, ids[l], w[l])
    assert not torch.equal(step2, step)
    for rep in range(2):
        got = chain.forward(x, ids, w, use_graph=True)
        assert torch.equal(got.view(torch.int16), step2.view(torch.int16)), rep
    chain.close()
    for layer in layers:
        layer.close()


def test_shared_expert_of_another_width_at_a_model_shape(ek, oracle, cuda):
    """DeepSeek-V2-Lite's sizes: hidden 2048, moe_intermediate_size 1408, two shared experts, i.e. a
    shared expert of 2816 channels beside routed experts of 1408 (neither a multiple of the tile
    kernel's 256-channel blocks); the static-workspace entry point and a chain take the same path."""
    dt, Hm, Im, Em, Km = torch.bfloat16, 2048, 1408, 4, 2
    work = wl.Workload("v2lite", Hm, Im, Em, Km, 1, dt)
    ws = {e: wl.make_expert(work, e, std=0.03) for e in range(Em)}
    shared = wl.make_expert(wl.Workload("v2lite", Hm, 2 * Im, 1, 1, 1, dt), Em, std=0.03)
    layer = ek.HipLayer(Hm, Im, Em, Km, act_dtype=dt, max_tokens=320)
    for e in range(Em):
        layer.set_expert(e, ws[e])
    wu, wg, wd = oracle_weights(oracle, {**ws, Em: shared}, Em + 1, dt)
    for T in (24, 130, 300):
        g = torch.Generator().manual_seed(T)
        x = torch.randn(T, Hm, generator=g).to(dt)
        ids = torch.stack([torch.randperm(Em, generator=g)[:Km] for _ in range(T)]).to(torch.int32)
        w = torch.rand(T, Km, generator=g) + 0.1
        w = (w / w.sum(-1, keepdim=True)).to(dt)
        y_plain = layer.forward(x.to(cuda), ids.to(cuda), w.to(cuda))
        layer.set_shared_expert(shared)
        y = layer.forward(x.to(cuda), ids.to(cuda), w.to(cuda))
        assert torch.equal(layer.forward(x.to(cuda), ids.to(cuda), w.to(cuda)).view(torch.int16), y.view(torch.int16))
        assert torch.equal(layer.forward_static(x.to(cuda), ids.to(cuda), w.to(cuda)).view(torch.int16), y.view(torch.int16))
        rows = torch.arange(0, T, max(1, T // 12))[:12]                 # the oracle recomputes a dozen tokens
        y_r = oracle.layer_forward(x[rows], ids[rows], w[rows], wu[:Em], wg[:Em], wd[:Em], mode=0)[0]
        ref32 = oracle.add_shared(y_r, x[rows], wu[Em], wg[Em], wd[Em], rounded=False)
        y_s = ref32 - y_r.float()
        rms = float(ref32.pow(2).mean().sqrt())
        err = (y[rows.to(cuda)].float().cpu() - ref32).abs()
        quanta = 0.5 * ulp_of(ref32, dt) * 1.0001 + ulp_of(y_r.float(), dt) + ulp_of(y_s, dt)
        print(f"shared 2816 beside 1408, T={T}: max|err|/rms = {float(err.max()) / rms:.3e}", flush=True)
        assert bool((err <= TOL * rms + quanta).all())
        assert float((y.float() - y_plain.float()).abs().max()) > 0
        layer.remove_expert(C.EK_SHARED_EXPERT)
    # a shape the kernels cannot take is refused with the sizes in the message
    bad = wl.make_expert(wl.Workload("bad", Hm, 1000, 1, 1, 1, dt), 0)
    with pytest.raises(ek.EKError) as ei:
        layer.set_shared_expert(bad)
    assert ei.value.status == C.EK_INVALID_INPUT and "1000" in ei.value.message
    layer.close()


def test_shared_expert_of_another_width_in_a_chain(ek, cuda):
    dt, L, T = torch.float16, 2, 90
    layers = []
    for l in range(L):
        work = wl.Workload("shared-chain", H, I, E + 1, K, 1, dt)
        layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=128)
        for e in range(E):
            layer.set_expert(e, wl.make_expert(work, e, layer=l, std=0.08))
        layer.set_shared_expert(wl.make_expert(wl.Workload("sc", H, 2 * I, 1, 1, 1, dt), E, layer=l, std=0.08))
        layers.append(layer)
    x, _, _ = routing(T, 7)
    x = x.to(dt).to(cuda)
    ids = torch.stack([routing(T, 100 + l)[1] for l in range(L)]).to(cuda)
    w = torch.stack([routing(T, 100 + l)[2] for l in range(L)]).to(dt).to(cuda)
    step = x
    for l in range(L):
        step = layers[l].forward(step, ids[l], w[l])
    chain = ek.HipChain(layers)
    assert torch.equal(chain.forward(x, ids, w, use_graph=False).view(torch.int16), step.view(torch.int16))
    for rep in range(3):
        got = chain.forward(x, ids, w, use_graph=True)
        assert torch.equal(got.view(torch.int16), step.view(torch.int16)), rep
        torch.cuda.synchronize()
    # a shared expert of the routed experts' width in layer 0 instead: other launches, the graph is captured again
    layers[0].set_shared_expert(wl.make_expert(wl.Workload("sc", H, I, 1, 1, 1, dt), E, layer=0, std=0.08))
    step2 = x
    for l in range(L):
        step2 = layers[l].forward(step2, ids[l], w[l])
    assert not torch.equal(step2, step)
    for rep in range(2):
        got = chain.forward(x, ids, w, use_graph=True)
        assert torch.equal(got.view(torch.int16), step2.view(torch.int16)), rep
    chain.close()
    for layer in layers:
        layer.close()
