"""ek_layer_forward_static: the layer call whose workspace is the library's static device array
(for callers that cannot allocate device memory), held to ek_layer_forward through the C ABI:
bit-identical outputs and routing tables on two calls in a row, the second with a smaller
input (the array keeps the first call's contents), on a caller's stream and blocking, with
several layers sharing the GPU's one array, a refusal for calls that do not fit, and the property
itself: free device memory unchanged over the calls, and the call accepted inside a stream capture
that refuses allocating runtime calls."""
import pytest
import torch

from ek_hip import workloads as wl

pytestmark = pytest.mark.gpu


def bits(t):
    return t.contiguous().view(torch.int16)


def build(ek, w, max_tokens):
    layer = ek.HipLayer(w.hidden, w.inter, w.n_experts, w.top_k, act_dtype=w.act_dtype,
                        w_dtype=torch.int8 if w.w8 else w.act_dtype, max_tokens=max_tokens)
    for e in range(w.n_experts):
        layer.set_expert(e, wl.make_expert(w, e, std=0.05))
    return layer


def inputs(w, T, seed, dev):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, w.hidden, generator=g).to(w.act_dtype)
    ids = torch.stack([torch.randperm(w.n_experts, generator=g)[:w.top_k] for _ in range(max(T, 1))])[:T].to(torch.int32)
    if T > 64:                                     # a hot expert: 128-row tiles and a remainder beside streaming items
        ids[: T // 2, 0] = 3
        ids[: T // 2, 1] = torch.where(ids[: T // 2, 1] == 3, 4, ids[: T // 2, 1])
        for k in range(2, w.top_k):
            clash = ids[: T // 2, k] == 3
            ids[: T // 2, k] = torch.where(clash, (5 + k) % w.n_experts, ids[: T // 2, k])
    gw = torch.rand(T, w.top_k, generator=g).to(w.act_dtype)
    return x.to(dev), ids.to(dev), gw.to(dev)


@pytest.mark.parametrize("w8", [False, True])
def test_static_call_matches_the_allocating_call(ek, cuda, w8):
    w = wl.Workload("static", 512, 256, 16, 4, 1, torch.bfloat16, w8=w8)
    layer = build(ek, w, 600)
    stream = torch.cuda.Stream()
    for T, seed in ((600, 1), (37, 2), (600, 3), (0, 4), (5, 5)):     # large, then smaller, ...
        print(f"static call w8={w8} T={T}", flush=True)
        x, ids, gw = inputs(w, T, seed, cuda)
        want, rt = layer.forward(x, ids, gw, return_route=True)
        got, rs = layer.forward_static(x, ids, gw, return_route=True)                # blocking
        assert torch.equal(bits(got), bits(want)), T
        for a, b in zip((rs.counts, rs.offsets, rs.perm, rs.inv_perm), (rt.counts, rt.offsets, rt.perm, rt.inv_perm)):
            assert torch.equal(a, b), T
        out = torch.zeros_like(x)
        torch.cuda.synchronize()
        layer.forward_static(x, ids, gw, stream=stream, out=out)                     # enqueue only
        stream.synchronize()
        assert torch.equal(bits(out), bits(want)), T
    layer.close()


def test_static_calls_of_two_layers_share_the_array(ek, cuda):
    """Two layers of different shapes, calls alternating on two streams: the library orders them
    on the device, so each result equals the layer's own allocating call."""
    wa = wl.Workload("a", 256, 128, 8, 2, 1, torch.float16)
    wb = wl.Workload("b", 512, 256, 16, 4, 1, torch.bfloat16, w8=True)
    la, lb = build(ek, wa, 300), build(ek, wb, 300)
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    ins_a, ins_b = inputs(wa, 300, 11, cuda), inputs(wb, 150, 12, cuda)
    want_a, want_b = la.forward(*ins_a), lb.forward(*ins_b)
    outs = []
    torch.cuda.synchronize()
    for i in range(6):
        oa, ob = torch.zeros_like(ins_a[0]), torch.zeros_like(ins_b[0])
        la.forward_static(*ins_a, stream=sa, out=oa)
        lb.forward_static(*ins_b, stream=sb, out=ob)
        outs.append((oa, ob))
    torch.cuda.synchronize()
    for i, (oa, ob) in enumerate(outs):
        assert torch.equal(bits(oa), bits(want_a)), i
        assert torch.equal(bits(ob), bits(want_b)), i
    la.close(); lb.close()


def test_static_call_refuses_what_does_not_fit(ek, cuda):
    from ek_hip import _capi as C
    w = wl.Workload("big", 2048, 1024, 8, 8, 1, torch.bfloat16)
    layer = ek.HipLayer(w.hidden, w.inter, w.n_experts, w.top_k, act_dtype=w.act_dtype, max_tokens=4096)
    layer.set_expert(0, wl.make_expert(w, 0))
    T = 4096                      # (T*K + T) * (H + I) * 2 bytes = 226 MB of intermediates alone
    x = torch.zeros(T, w.hidden, dtype=w.act_dtype, device=cuda)
    ids = torch.zeros(T, w.top_k, dtype=torch.int32, device=cuda)
    gw = torch.ones(T, w.top_k, dtype=w.act_dtype, device=cuda)
    with pytest.raises(ek.EKError) as ei:
        layer.forward_static(x, ids, gw)
    assert ei.value.status == C.EK_INVALID_INPUT and "static scratch" in ei.value.message
    # an unloaded expert is reported like ek_layer_forward reports it
    with pytest.raises(ek.EKError) as ei:
        layer.forward_static(x[:4], ids[:4] + 1, gw[:4])
    assert ei.value.status == C.EK_EXPERT_NOT_FOUND
    y = layer.forward_static(x[:4], ids[:4], gw[:4])
    assert y.shape == (4, w.hidden) and not y.float().any()
    layer.close()
    # a layer whose sizes need padding stages rows in allocated buffers: refused
    small = ek.HipLayer(16, 8, 2, 1, max_tokens=4)
    with pytest.raises(ek.EKError) as ei:
        small.forward_static(torch.zeros(2, 16, dtype=torch.bfloat16, device=cuda),
                             torch.zeros(2, 1, dtype=torch.int32, device=cuda),
                             torch.ones(2, 1, dtype=torch.bfloat16, device=cuda))
    assert ei.value.status == C.EK_INVALID_INPUT
    small.close()


def test_static_call_allocates_nothing(ek, cuda):
    """The property itself, observed two ways.  (1) Free device memory (hipMemGetInfo) is the same
    before and after calls whose output tensor is the caller's.  (2) The call is made while the
    caller's stream is under capture in the mode that refuses every allocating runtime call: the
    capture ends without an error, and the graph replays to the allocating call's bits, twice, with
    a smaller eager static call (which leaves its own contents in the shared array) in between."""
    w = wl.Workload("static", 512, 256, 16, 4, 1, torch.bfloat16, w8=True)
    layer = build(ek, w, 300)
    x, ids, gw = inputs(w, 300, 21, cuda)            # a hot expert's tiles beside streaming items
    xs, idss, gws = inputs(w, 23, 22, cuda)
    want, want_small = layer.forward(x, ids, gw), layer.forward(xs, idss, gws)
    y, ysmall = torch.empty_like(x), torch.empty_like(xs)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    layer.forward_static(x, ids, gw, stream=side, out=y)          # first use of this stream (its side stream is picked)
    side.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        layer.forward_static(x, ids, gw, stream=side, out=y)
        layer.forward_static(xs, idss, gws, stream=side, out=ysmall)
    side.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "a static call changed the free device memory"
    assert torch.equal(bits(y), bits(want)) and torch.equal(bits(ysmall), bits(want_small))

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side, capture_error_mode="global"):
            layer.forward_static(x, ids, gw, stream=torch.cuda.current_stream(), out=y)
    torch.cuda.synchronize()
    for rep in range(2):
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(bits(y), bits(want)), f"replay {rep}"
        layer.forward_static(xs, idss, gws, out=ysmall)           # eager, blocking, smaller: same array
        assert torch.equal(bits(ysmall), bits(want_small)), f"after replay {rep}"
    layer.close()
