"""Chains of MoE layers launched as one HIP graph (the ragged continuous-batching
configuration): chain == the same layers called one by one, every graph replay ==
the eager chain bit for bit, plus size-independent properties at the full shape."""
import pytest
import torch

from ek_hip import workloads as wl

pytestmark = pytest.mark.gpu


def build_chain(ek, w, cuda, device="cpu", std=0.02):
    w = wl.resolve(w)
    layers, weights = [], []
    for l in range(w.n_layers):
        layer = ek.HipLayer(w.hidden, w.inter, w.n_experts, w.top_k, act_dtype=w.act_dtype,
                            w_dtype=torch.int8 if w.w8 else w.act_dtype, max_tokens=w.tokens)
        ws = {}
        for e in range(w.n_experts):
            ws[e] = wl.make_expert(w, e, layer=l, device=device, std=std)
            layer.set_expert(e, ws[e])
        layers.append(layer)
        weights.append(ws)
    routing = [wl.make_routing(w, layer=l) for l in range(w.n_layers)]
    ids = torch.stack([r[0] for r in routing]).to(cuda)
    gw = torch.stack([r[1] for r in routing]).to(cuda)
    return w, layers, weights, ids, gw


def bits(t):
    return t.cpu().view(torch.int16)


def test_chain_small_vs_layers_and_oracle(ek, oracle, cuda):
    w0 = wl.Workload("ragged_x3", 256, 128, 16, 4, 0, torch.float16, zipf_s=1.2, n_layers=3, ragged=True)
    lens = [1] * 10 + [70, 33]
    w0 = wl.Workload(**{**w0.__dict__, "tokens": sum(lens)})
    # weight std 0.08 keeps the activation scale near 1 from layer to layer at this shape
    w, layers, weights, ids, gw = build_chain(ek, w0, cuda, std=0.08)
    x = wl.make_x(w)
    xd = x.to(cuda)
    chain = ek.HipChain(layers)
    y_eager = chain.forward(xd, ids, gw, use_graph=False)
    # the same layers, one ek_layer_forward each
    cur = xd
    for l, layer in enumerate(layers):
        cur = layer.forward(cur, ids[l].contiguous(), gw[l].contiguous())
    assert torch.equal(bits(y_eager), bits(cur))
    # oracle chain (each layer fed with the oracle's own previous output)
    ref = x
    for l in range(w.n_layers):
        wu = [weights[l][e].up_w for e in range(w.n_experts)]
        wg = [weights[l][e].gate_w for e in range(w.n_experts)]
        wd = [weights[l][e].down_w for e in range(w.n_experts)]
        mode = 2 if l == w.n_layers - 1 else 0
        ref = oracle.layer_forward(ref, ids[l].cpu(), gw[l].cpu(), wu, wg, wd, mode=mode)[0]
    rms = float(ref.pow(2).mean().sqrt())
    err = float((y_eager.float().cpu() - ref).abs().max()) / rms
    print(f"3-layer chain vs oracle chain: max|err|/rms = {err:.3e}", flush=True)
    assert err <= 3e-2          # three layers of storage-rounding flips compound; single layers are gated at 2e-2
    # graph replays, with eager work and synchronisation in between
    for rep in range(4):
        y_graph = chain.forward(xd, ids, gw, use_graph=True)
        assert torch.equal(bits(y_graph), bits(y_eager)), f"replay {rep}"
        scratch = layers[rep % len(layers)].forward(xd, ids[0].contiguous(), gw[0].contiguous())
        torch.cuda.synchronize()
        assert scratch.shape == xd.shape
    # new inputs in the same buffers: the graph reads them at replay time
    xd.copy_(torch.randn_like(xd))
    ids.copy_(torch.stack([wl.make_routing(w, layer=10 + l)[0] for l in range(w.n_layers)]).to(cuda))
    y_eager2 = chain.forward(xd, ids, gw, use_graph=False)
    y_graph2 = chain.forward(xd, ids, gw, use_graph=True)
    assert torch.equal(bits(y_graph2), bits(y_eager2))
    assert not torch.equal(bits(y_graph2), bits(y_eager))
    chain.close()
    for layer in layers:
        layer.close()


def test_chain_with_a_layer_used_twice(ek, cuda):
    """A chain may name one layer object more than once (tied weights).  Its workspace is then used
    by two steps of the chain, so the chain must not run those steps' routing ahead of their turn
    (it does for chains of distinct layers); eager and graph results equal the layer-by-layer calls."""
    w0 = wl.Workload("ragged_x3", 256, 128, 16, 4, 0, torch.float16, zipf_s=1.2, n_layers=3, ragged=True)
    w0 = wl.Workload(**{**w0.__dict__, "tokens": 90})
    w, layers, weights, ids, gw = build_chain(ek, w0, cuda, std=0.08)
    order = [layers[0], layers[1], layers[0]]
    xd = wl.make_x(w).to(cuda)
    cur = xd
    for l, layer in enumerate(order):
        cur = layer.forward(cur, ids[l].contiguous(), gw[l].contiguous())
    chain = ek.HipChain(order)
    assert torch.equal(bits(chain.forward(xd, ids, gw, use_graph=False)), bits(cur))
    for rep in range(3):
        assert torch.equal(bits(chain.forward(xd, ids, gw, use_graph=True)), bits(cur)), f"replay {rep}"
        torch.cuda.synchronize()
    chain.close()
    for layer in layers:
        layer.close()


def test_chain_c5_full_shape_properties(ek, cuda):
    """Qwen3 shape, 128 experts, top-8, 4 layers, 48 requests (40 decode + 8 prefill chunks):
    too large for the oracle, so the chain is checked through properties that do not
    depend on size."""
    w, layers, _, ids, gw = build_chain(ek, wl.C5, cuda, device="cuda")
    assert w.tokens == sum(wl.request_lengths()) and int(wl.request_offsets()[-1]) == w.tokens
    xd = wl.make_x(w).to(cuda)
    chain = ek.HipChain(layers)
    y_eager = chain.forward(xd, ids, gw, use_graph=False)
    assert bool(torch.isfinite(y_eager.float()).all())
    for rep in range(3):                                    # replays == eager, bit for bit
        y_graph = chain.forward(xd, ids, gw, use_graph=True)
        assert torch.equal(bits(y_graph), bits(y_eager)), f"replay {rep}"
        layers[0].pack(ids[0].contiguous())
        torch.cuda.synchronize()
    cur = xd                                                # == one call per layer
    for l, layer in enumerate(layers):
        cur = layer.forward(cur, ids[l].contiguous(), gw[l].contiguous())
    assert torch.equal(bits(cur), bits(y_eager))
    # with the benchmark's N(0, 0.02) weights the activations shrink from layer to layer
    # (x_{l+1} = y_l) and reach fp16's subnormals by the last one, so value properties
    # are checked on the first two layers
    chain2 = ek.HipChain(layers[:2])
    ids2, gw2 = ids[:2].contiguous(), gw[:2].contiguous()
    y2 = chain2.forward(xd, ids2, gw2, use_graph=True)
    assert float(y2.float().abs().max()) > 1e-3
    # the last layer is linear in its gate weights; doubling them is exact in fp16 except
    # where a product w*Y falls into the subnormal range (quantum 2^-24 per term), which can
    # also flip the final rounding by one ulp
    gw_dbl = gw2.clone()
    gw_dbl[-1] = gw_dbl[-1] * 2
    y_dbl = chain2.forward(xd, ids2, gw_dbl, use_graph=False)
    ulp = torch.exp2(torch.floor(torch.log2((2 * y2.float()).abs().clamp_min(2.0 ** -14))) - 10)
    assert bool(((y_dbl.float() - 2 * y2.float()).abs() <= ulp + w.top_k * 2.0 ** -23).all())
    assert float((bits(y_dbl) == bits(y2 * 2)).float().mean()) > 0.9
    chain2.close()
    # x = 0 -> y = 0 through every layer
    assert not chain.forward(torch.zeros_like(xd), ids, gw, use_graph=False).float().any()
    # a token's result does not depend on what else is in the batch: first request alone
    n0 = 1
    y_first = layers[0].forward(xd[:n0].contiguous(), ids[0, :n0].contiguous(), gw[0, :n0].contiguous())
    y_all = layers[0].forward(xd, ids[0].contiguous(), gw[0].contiguous())
    assert float((y_first.float() - y_all[:n0].float()).abs().max()) <= 2e-2 * float(y_all.float().pow(2).mean().sqrt())
    chain.close()
    for layer in layers:
        layer.close()


@pytest.mark.parametrize("T,shared", [(8, False), (48, False), (100, True), (300, False)])
def test_layer_call_in_the_callers_graph(ek, cuda, T, shared):
    """A caller that captures ek_layer_forward on its own stream (the library forks its side
    stream inside the capture and joins it again; no memset nodes, no allocation, no
    synchronisation): every replay, with eager work of the same layer between the replays,
    gives the eager call's bits.  T spans the regimes: streaming items only, both kernel
    families side by side, a shared expert's segment in a launch of its own, tiles."""
    dt, H, I, E, K = torch.float16, 256, 128, 8, 2
    w = wl.Workload("cap", H, I, E + 1, K, T, dt)
    layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=T)
    for e in range(E):
        layer.set_expert(e, wl.make_expert(w, e, std=0.05))
    if shared:
        layer.set_shared_expert(wl.make_expert(w, E, std=0.05))
    g = torch.Generator().manual_seed(T)
    x = torch.randn(T, H, generator=g).to(dt).to(cuda)
    p = torch.tensor([6.0] + [1.0] * (E - 1))                       # one hot expert: long and short segments
    ids = torch.stack([torch.multinomial(p, K, generator=g) for _ in range(T)]).to(torch.int32).to(cuda)
    gw = torch.rand(T, K, generator=g) + 0.1
    gw = (gw / gw.sum(-1, keepdim=True)).to(dt).to(cuda)
    y_eager = layer.forward(x, ids, gw).clone()
    y = torch.empty_like(x)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        layer.forward(x, ids, gw, stream=side, out=y)               # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            layer.forward(x, ids, gw, stream=torch.cuda.current_stream(), out=y)
    torch.cuda.synchronize()
    for rep in range(3):
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(bits(y), bits(y_eager)), f"replay {rep}"
        other = layer.forward(x.flip(0).contiguous(), ids, gw)      # eager work on the same workspace
        torch.cuda.synchronize()
        assert other.shape == x.shape
    layer.close()

