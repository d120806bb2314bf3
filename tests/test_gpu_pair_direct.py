"""Decode calls of one or two tokens run without pack and combine kernels: every pair is a one-row
item taken straight from the ids, and stage 2 adds a token's pairs in k order itself (the
worker's expert call per pair, ek-computation/src/ffn/expert_torch.rs:80-85, followed by the shim's
weighted sum, qwen3_moe.py:102-104).  A call that asks for its routing tables takes the ordinary
path (pack, lists, combine kernel); the two must give the same bits, the same error codes and the
same activation counters.  Held to the oracle as every layer call is."""
import pytest
import torch

from ek_hip import _capi as C
from ek_hip import workloads as wl
from test_gpu_block_scaled import KINDS, make_expert as make_block_expert, ref_weights
from test_gpu_parity import layer_gate, oracle_weights

pytestmark = pytest.mark.gpu


def build(ek, oracle, kind, dt, H, I, E, K, max_tokens=8):
    """A layer of weight kind `kind` with four distinct experts repeated over E slots, and the
    reference's weights of every slot."""
    if kind in KINDS:
        layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=max_tokens, **KINDS[kind])
        ws = [make_block_expert(ek, H, I, 10 + e, kind) for e in range(4)]
        ref_w = [ref_weights(oracle, ew, dt) for ew in ws]
    else:
        w = wl.Workload("t", H, I, E, K, max_tokens, dt, w8=kind == "i8")
        layer = ek.HipLayer(H, I, E, K, act_dtype=dt, w_dtype=torch.int8 if w.w8 else dt, max_tokens=max_tokens)
        ws = [wl.make_expert(w, 10 + e, std=0.05) for e in range(4)]
        cols = oracle_weights(oracle, dict(enumerate(ws)), 4, dt)
        ref_w = [tuple(c[i] for c in cols) for i in range(4)]
    for e in range(E):
        layer.set_expert(e, ws[e % 4])
    wu, wg, wd = zip(*[ref_w[e % 4] for e in range(E)])
    return layer, (list(wu), list(wg), list(wd))


def same_bits(a, b):
    return torch.equal(a.cpu().view(torch.int16), b.cpu().view(torch.int16))


@pytest.mark.parametrize("kind", ["w16", "i8", "fp8", "int8"])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,K", [(1, 8), (2, 8), (1, 1), (2, 2), (2, 6), (3, 5), (1, 7)])
def test_pair_direct_equals_the_tabled_call(ek, oracle, cuda, kind, dt, T, K):
    H, I, E = 384 if kind == "w16" else 512, 192 if kind == "w16" else 384, 12
    layer, (wu, wg, wd) = build(ek, oracle, kind, dt, H, I, E, K)
    g = torch.Generator().manual_seed(100 * T + K)
    x = torch.randn(T, H, generator=g).to(dt)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32).reshape(T, K)
    gw = torch.rand(T, K, generator=g) + 0.1
    gw = (gw / gw.sum(-1, keepdim=True)).to(dt)
    for w in (gw, gw.float()):                               # gate weights of the activation type, and fp32
        y = layer.forward(x.to(cuda), ids.to(cuda), w.to(cuda))
        y_t, rt = layer.forward(x.to(cuda), ids.to(cuda), w.to(cuda), return_route=True)
        assert same_bits(y, y_t), "pair-direct call differs from the call through pack and combine"
        assert same_bits(layer.forward(x, ids, w), y)        # host memory
        assert same_bits(layer.forward_static(x.to(cuda), ids.to(cuda), w.to(cuda)), y)
        ref, _, _, _, _, y3 = oracle.layer_forward(x, ids, w, wu, wg, wd, mode=2, return_y3=True)
        layer_gate(y, ref, y3, w, f"pair-direct {kind} {dt} T={T} K={K} w={w.dtype}")
    layer.close()


def test_repeated_experts_and_repeated_calls(ek, oracle, cuda):
    """One expert named twice by a token, and by both tokens; the call repeated on a stream."""
    dt = torch.bfloat16
    layer, (wu, wg, wd) = build(ek, oracle, "i8", dt, 512, 256, 6, 4)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 512, generator=g).to(dt)
    ids = torch.tensor([[3, 3, 1, 0], [3, 5, 5, 5]], dtype=torch.int32)
    gw = torch.tensor([[0.4, 0.3, 0.2, 0.1], [0.25, 0.25, 0.25, 0.25]]).to(dt)
    xd, idd, gwd = x.to(cuda), ids.to(cuda), gw.to(cuda)
    y = layer.forward(xd, idd, gwd)
    y_t, rt = layer.forward(xd, idd, gwd, return_route=True)
    assert same_bits(y, y_t)
    ref, _, _, _, _, y3 = oracle.layer_forward(x, ids, gw, wu, wg, wd, mode=2, return_y3=True)
    layer_gate(y, ref, y3, gw, "pair-direct, repeated experts")
    s = torch.cuda.Stream()
    out = torch.empty_like(xd)
    for _ in range(20):
        layer.forward(xd, idd, gwd, stream=s, out=out)
    s.synchronize()
    assert same_bits(out, y)
    layer.close()


def test_bookkeeping_matches_the_tabled_call(ek, cuda):
    """Error codes, activation counters and the call statistics of a pair-direct call are those of the
    call through the pack kernel; a failed call leaves the next one clean."""
    dt = torch.bfloat16
    w = wl.Workload("t", 128, 64, 8, 2, 2, dt)
    layer = ek.HipLayer(128, 64, 8, 2, act_dtype=dt, w_dtype=dt, max_tokens=4)
    ws = {e: wl.make_expert(w, e) for e in range(4)}
    for e, ew in ws.items():
        layer.set_expert(e, ew)
    x = torch.randn(2, 128).to(dt).to(cuda)
    gw = torch.full((2, 2), 0.5).to(dt).to(cuda)
    ok = torch.tensor([[0, 1], [2, 1]], dtype=torch.int32, device=cuda)
    y0 = layer.forward(x, ok, gw)
    assert layer.activation().tolist() == [1, 2, 1, 0, 0, 0, 0, 0]
    layer.forward(x, ok, gw, return_route=True)
    assert layer.activation().tolist() == [2, 4, 2, 0, 0, 0, 0, 0]
    for bad, status in ((7, C.EK_EXPERT_NOT_FOUND), (8, C.EK_INVALID_INPUT), (-1, C.EK_INVALID_INPUT),
                        (1 << 20, C.EK_INVALID_INPUT), (-(1 << 31), C.EK_INVALID_INPUT)):
        ids = ok.clone()
        ids[1, 0] = bad
        for tabled in (False, True):
            with pytest.raises(ek.EKError) as ei:
                layer.forward(x, ids, gw, return_route=tabled)
            assert ei.value.status == status, (bad, tabled)
        assert same_bits(layer.forward(x, ok, gw), y0)
    # a pair without an expert adds nothing: the other pairs' sum is the call's output either way
    ids = ok.clone()
    ids[0, 1] = 100
    y_bad = torch.empty_like(x)
    s = torch.cuda.Stream()
    layer.forward(x, ids, gw, stream=s, out=y_bad)            # enqueue-only: the error word is not read
    s.synchronize()
    ids_ok = ok.clone()
    gw0 = gw.clone()
    gw0[0, 1] = 0.0
    y_ref = layer.forward(x, ids_ok, gw0)                     # the same sum with a zero weight for that pair
    assert same_bits(y_bad[1:], y_ref[1:])
    assert torch.allclose(y_bad[0].float(), y_ref[0].float(), atol=0, rtol=0)
    st = layer.stats()
    assert st["tokens"] == st["forward_calls"] * 2
    layer.close()


def test_pair_direct_call_in_the_callers_graph(ek, cuda):
    """The two launches of a one-token call captured into a graph of the caller's and replayed with
    other inputs in the same buffers."""
    dt = torch.bfloat16
    w = wl.Workload("t", 256, 128, 16, 4, 1, dt)
    layer = ek.HipLayer(256, 128, 16, 4, act_dtype=dt, w_dtype=dt, max_tokens=2)
    for e in range(16):
        layer.set_expert(e, wl.make_expert(w, e))
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, 256, generator=g).to(dt).to(cuda)
    ids = torch.tensor([[1, 5, 9, 13]], dtype=torch.int32, device=cuda)
    gw = torch.tensor([[0.4, 0.3, 0.2, 0.1]]).to(dt).to(cuda)
    y = torch.empty_like(x)
    s = torch.cuda.Stream()
    layer.forward(x, ids, gw, stream=s, out=y)
    s.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        with torch.cuda.graph(graph, stream=s, capture_error_mode="global"):
            layer.forward(x, ids, gw, stream=torch.cuda.current_stream(), out=y)
    for trial in range(3):
        x.copy_(torch.randn(1, 256, generator=g).to(dt))
        ids.copy_(torch.randperm(16, generator=g)[:4].to(torch.int32).reshape(1, 4))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want, _ = layer.forward(x, ids, gw, return_route=True)
        assert same_bits(y, want), trial
    del graph
    layer.close()


def test_wider_top_k_and_more_pairs_take_the_ordinary_path(ek, oracle, cuda):
    """top-k above eight and calls of more than sixteen pairs are not pair-direct; they still agree with
    the tabled call (nothing else to tell them apart from outside)."""
    dt = torch.float16
    for T, K in ((1, 12), (3, 8), (5, 4)):
        layer, (wu, wg, wd) = build(ek, oracle, "w16", dt, 256, 128, 16, K)
        g = torch.Generator().manual_seed(K)
        x = torch.randn(T, 256, generator=g).to(dt).to(cuda)
        ids = torch.stack([torch.randperm(16, generator=g)[:K] for _ in range(T)]).to(torch.int32).to(cuda)
        gw = torch.full((T, K), 1.0 / K).to(dt).to(cuda)
        y = layer.forward(x, ids, gw)
        y_t, _ = layer.forward(x, ids, gw, return_route=True)
        assert same_bits(y, y_t)
        layer.close()


@pytest.mark.parametrize("T", [1, 2, 4])
def test_chain_of_few_pairs(ek, cuda, T):
    """A chain's layer calls of one or two tokens are pair-direct as well (4 tokens x top-4 = 16 pairs is
    the last size that is): eager and replayed graph give the bits of the layers called one by one
    through pack and combine, also after new inputs arrive in the same buffers."""
    from test_gpu_chain import build_chain, bits
    w0 = wl.Workload("decode_x3", 256, 128, 16, 4, T, torch.float16, zipf_s=1.2, n_layers=3)
    w, layers, weights, ids, gw = build_chain(ek, w0, cuda, std=0.08)
    xd = wl.make_x(w).to(cuda)
    chain = ek.HipChain(layers)

    def one_by_one():
        cur = xd
        for l, layer in enumerate(layers):
            cur, _ = layer.forward(cur, ids[l].contiguous(), gw[l].contiguous(), return_route=True)
        return cur

    for trial in range(2):
        want = one_by_one()
        assert torch.equal(bits(chain.forward(xd, ids, gw, use_graph=False)), bits(want)), trial
        for rep in range(3):
            assert torch.equal(bits(chain.forward(xd, ids, gw, use_graph=True)), bits(want)), (trial, rep)
            layers[rep % 3].forward(xd, ids[0].contiguous(), gw[0].contiguous())
            torch.cuda.synchronize()
        xd.copy_(torch.randn_like(xd))
        ids.copy_(torch.stack([wl.make_routing(w, layer=10 + l)[0] for l in range(w.n_layers)]).to(cuda))
    chain.close()
    for layer in layers:
        layer.close()


@pytest.mark.parametrize("kind", ["w16", "i8", "fp8", "int8"])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,K", [(1, 8), (2, 8), (2, 3), (5, 1)])
def test_pair_direct_with_a_shared_expert(ek, oracle, cuda, kind, dt, T, K):
    """A shared expert of the routed experts' shape (deepseek_v3/model.py:57-61,152) is one more wave
    of stage 2's workgroups: its rounded output joins the rounded weighted sum, as in the call through
    pack and combine, whose bits the call must give; held to the oracle by test_gpu_shared.py's bound."""
    from test_gpu_parity import TOL, ulp_of
    H, I, E = 384 if kind == "w16" else 512, 192 if kind == "w16" else 384, 12
    layer, (wu, wg, wd) = build(ek, oracle, kind, dt, H, I, E, K)
    # the shared expert: the weights of slot 3 (build's fourth distinct expert)
    if kind in KINDS:
        shared_w = make_block_expert(ek, H, I, 13, kind)
    else:
        shared_w = wl.make_expert(wl.Workload("t", H, I, E, K, 8, dt, w8=kind == "i8"), 13, std=0.05)
    g = torch.Generator().manual_seed(7 * T + K)
    x = torch.randn(T, H, generator=g).to(dt)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32).reshape(T, K)
    gw = torch.rand(T, K, generator=g) + 0.1
    gw = (gw / gw.sum(-1, keepdim=True)).to(dt)
    y_plain = layer.forward(x.to(cuda), ids.to(cuda), gw.to(cuda))
    layer.set_shared_expert(shared_w)
    for w in (gw, gw.float()):
        y = layer.forward(x.to(cuda), ids.to(cuda), w.to(cuda))
        y_t, _ = layer.forward(x.to(cuda), ids.to(cuda), w.to(cuda), return_route=True)
        assert same_bits(y, y_t), "pair-direct call differs from the call through pack and combine"
        assert same_bits(layer.forward(x, ids, w), y)
        assert same_bits(layer.forward_static(x.to(cuda), ids.to(cuda), w.to(cuda)), y)
    assert not same_bits(y, y_plain)
    y = layer.forward(x.to(cuda), ids.to(cuda), gw.to(cuda))
    y_r = oracle.layer_forward(x, ids, gw, wu, wg, wd, mode=0)[0]
    ref32 = oracle.add_shared(y_r, x, wu[3], wg[3], wd[3], rounded=False)
    y_s = ref32 - y_r.float()
    rms = float(ref32.pow(2).mean().sqrt())
    err = (y.float().cpu() - ref32).abs()
    quanta = 0.5 * ulp_of(ref32, dt) * 1.0001 + ulp_of(y_r.float(), dt) + ulp_of(y_s, dt)
    assert bool((err <= TOL * rms + quanta).all()), float(err.max()) / rms
    layer.remove_expert(C.EK_SHARED_EXPERT)
    assert same_bits(layer.forward(x.to(cuda), ids.to(cuda), gw.to(cuda)), y_plain)
    layer.close()
