"""Router kernels against the oracle's routers, through the C ABI.

Bars: expert ids bit-exact.  Gate weights bit-exact for every router whose sums run over
the K chosen values (kinds 1-4: the kernel adds them in the oracle's order, and exp is
built from IEEE operations only on both sides); for the softmax over all E experts (kind
0) the kernel adds E exponentials as a tree and the oracle one after another, so fp32
weights agree to 4e-6 relative (a one-after-another fp32 sum of 256 terms is itself only good
to about that) and 16-bit weights to one unit in the last place.
"""
import pytest
import torch

from ek_hip import _capi as C
from ek_hip import workloads as wl
from test_gpu_parity import layer_gate

pytestmark = pytest.mark.gpu


def router_layer(ek, E, K, dt=torch.bfloat16, max_tokens=8192):
    # no experts are loaded: routing alone does not touch weights
    return ek.HipLayer(128, 128, E, K, act_dtype=dt, max_tokens=max_tokens)


def logits_of(T, E, seed, zipf=0.0):
    g = torch.Generator().manual_seed(seed)
    lg = torch.randn(T, E, generator=g)
    if zipf:
        rank = torch.randperm(E, generator=g) + 1
        lg = lg - zipf * torch.log(rank.float())
    return lg


def ulps(a, b):
    """distance in representable 16-bit values (same-sign finite inputs)"""
    return (a.view(torch.int16).int() - b.view(torch.int16).int()).abs().max().item()


@pytest.mark.parametrize("T,E,K,zipf", [(64, 16, 2, 0.0), (256, 128, 8, 1.0), (128, 256, 8, 0.0), (8192, 256, 8, 0.8),
                                        (33, 100, 7, 0.0), (5, 1024, 64, 0.0), (3, 1, 1, 0.0)])
@pytest.mark.parametrize("renorm", [True, False])
def test_softmax_topk(ek, oracle, cuda, T, E, K, zipf, renorm):
    layer = router_layer(ek, E, K)
    lg = logits_of(T, E, 3000, zipf)
    o_ids, o_w = oracle.route(0, lg, K, renorm)
    r = ek.RouterConfig(kind=C.EK_ROUTER_SOFTMAX_TOPK, renorm=renorm, w_dtype=torch.float32)
    ids, w = layer.route(lg.to(cuda), r)
    assert torch.equal(ids.cpu(), o_ids)
    rel = float(((w.cpu() - o_w).abs() / o_w).max())
    print(f"T={T} E={E} K={K}: max relative weight difference {rel:.2e}", flush=True)
    assert rel < 4e-6
    for dt in (torch.bfloat16, torch.float16):
        lay = router_layer(ek, E, K, dt)
        ids16, w16 = lay.route(lg.to(cuda), ek.RouterConfig(kind=0, renorm=renorm))
        assert torch.equal(ids16.cpu(), o_ids) and w16.dtype == dt
        assert ulps(w16.cpu(), o_w.to(dt)) <= 1
        lay.close()
    # host-memory call: same kernel behind a staging copy
    h_ids, h_w = layer.route(lg, r)
    assert torch.equal(h_ids, ids.cpu()) and torch.equal(h_w, w.cpu())
    layer.close()


@pytest.mark.parametrize("kind", [1, 2, 3])
@pytest.mark.parametrize("ldt", [torch.float32, torch.bfloat16, torch.float16])
def test_topk_on_logits_routers(ek, oracle, cuda, kind, ldt):
    T, E, K = 300, 160, 6
    layer = router_layer(ek, E, K)
    lg = logits_of(T, E, 7).to(ldt)          # 16-bit logits hold many exact ties: the tie rule is exercised
    o_ids, o_w = oracle.route(kind, lg, K, w_dtype=torch.float32)
    ids, w = layer.route(lg.to(cuda), ek.RouterConfig(kind=kind, w_dtype=torch.float32))
    assert torch.equal(ids.cpu(), o_ids)
    assert torch.equal(w.cpu(), o_w)
    o_w16 = oracle.route(kind, lg, K, w_dtype=torch.bfloat16)[1]
    w16 = layer.route(lg.to(cuda), ek.RouterConfig(kind=kind))[1]
    assert torch.equal(w16.cpu().view(torch.int16), o_w16.view(torch.int16))
    layer.close()


@pytest.mark.parametrize("T,E,K,ng,tg", [(128, 256, 8, 8, 4), (8192, 256, 8, 8, 4), (50, 64, 6, 4, 2), (9, 1024, 8, 64, 3),
                                         (7, 16, 4, 2, 2)])
@pytest.mark.parametrize("renorm,neg_inf,with_bias", [(True, False, True), (False, True, True), (True, True, False)])
def test_group_limited_sigmoid_router(ek, oracle, cuda, T, E, K, ng, tg, renorm, neg_inf, with_bias):
    layer = router_layer(ek, E, K)
    g = torch.Generator().manual_seed(31)
    lg = logits_of(T, E, 3001) * 1.5
    bias = (torch.randn(E, generator=g) * 0.3 - (0.6 if not neg_inf else 0.0)) if with_bias else None
    kw = dict(renorm=renorm, n_group=ng, topk_group=tg, mask_neg_inf=neg_inf, routed_scaling=2.5)
    o_ids, o_w = oracle.route(4, lg, K, bias=bias, w_dtype=torch.float32, **kw)
    r = ek.RouterConfig(kind=C.EK_ROUTER_SIGMOID_GROUP, bias=bias, w_dtype=torch.float32, **kw)
    ids, w = layer.route(lg.to(cuda), r)
    assert torch.equal(ids.cpu(), o_ids)
    assert torch.equal(w.cpu(), o_w)
    h_ids, h_w = layer.route(lg, r)           # host call: bias staged too
    assert torch.equal(h_ids, o_ids) and torch.equal(h_w, o_w)
    layer.close()


def test_hand_cases_and_ties(ek, cuda):
    layer = router_layer(ek, 8, 2)
    lg = torch.tensor([[3.0, -3.0, 2.0, 1.9, 2.5, -4.0, -0.2, -0.2]])
    r = ek.RouterConfig(kind=4, renorm=False, n_group=4, topk_group=2, w_dtype=torch.float32)
    ids, w = layer.route(lg.to(cuda), r)
    assert ids.tolist() == [[0, 2]]           # expert 4 would win a plain top-2 but sits in a dropped group
    assert w[0].tolist() == pytest.approx([0.9525741, 0.8807971], rel=1e-6)
    r.bias = torch.tensor([0.0, 0, 0, 0, 0, 0, 0.9, 0.9])
    ids, w = layer.route(lg.to(cuda), r)
    assert ids.tolist() == [[6, 7]]
    assert w[0].tolist() == pytest.approx([0.450166, 0.450166], rel=1e-5)     # unbiased scores
    layer.close()
    layer = router_layer(ek, 6, 4)
    lg = torch.tensor([[1.0, 2.0, 2.0, 0.5, 2.0, 1.0]])
    for kind in (0, 1, 2, 3):
        assert layer.route(lg.to(cuda), ek.RouterConfig(kind=kind))[0].tolist() == [[1, 2, 4, 0]]
    assert layer.route(lg[:0].to(cuda), ek.RouterConfig(kind=0))[0].shape == (0, 4)
    layer.close()


@pytest.mark.parametrize("dt,w8", [(torch.bfloat16, False), (torch.float16, False), (torch.bfloat16, True)])
def test_forward_logits_is_route_then_forward(ek, oracle, cuda, dt, w8):
    H, I, E, K, T = 256, 192, 16, 4, 200
    layer = ek.HipLayer(H, I, E, K, act_dtype=dt, w_dtype=torch.int8 if w8 else dt, max_tokens=256)
    work = wl.Workload("router", H, I, E, K, T, dt, w8=w8)
    experts = [wl.make_expert(work, e, std=0.05) for e in range(E)]
    for e, ew in enumerate(experts):
        layer.set_expert(e, ew)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, H, generator=g).to(dt)
    lg = logits_of(T, E, 9)
    for r in (ek.RouterConfig(kind=0), ek.RouterConfig(kind=0, w_dtype=torch.float32),
              ek.RouterConfig(kind=4, n_group=4, topk_group=2, routed_scaling=2.5, w_dtype=torch.float32,
                              bias=torch.randn(E, generator=g) * 0.1)):
        y, ids, w = layer.forward_logits(x.to(cuda), lg.to(cuda), r)
        ids2, w2 = layer.route(lg.to(cuda), r)
        assert torch.equal(ids, ids2) and torch.equal(w.view(torch.uint8), w2.view(torch.uint8))
        y2 = layer.forward(x.to(cuda), ids2, w2)
        assert torch.equal(y.view(torch.int16), y2.view(torch.int16))
        hy, hids, hw = layer.forward_logits(x, lg, r)        # host-memory call
        assert torch.equal(hids, ids.cpu()) and torch.equal(hy.view(torch.int16), y.cpu().view(torch.int16))
        assert float(y.float().abs().max()) > 0
    # and against the oracle end to end for the Qwen3 router in the activation dtype
    o_ids, o_w = oracle.route(0, lg, K, True, w_dtype=dt)
    y, ids, w = layer.forward_logits(x.to(cuda), lg.to(cuda), ek.RouterConfig(kind=0))
    assert torch.equal(ids.cpu(), o_ids)
    if w8:
        ws = [oracle.dequant_channel(getattr(ew, m + "_w"), getattr(ew, m + "_scale"), dt) for ew in experts
              for m in ("up", "gate", "down")]
        wu, wg, wd = ws[0::3], ws[1::3], ws[2::3]
    else:
        wu, wg, wd = [e.up_w for e in experts], [e.gate_w for e in experts], [e.down_w for e in experts]
    out = oracle.layer_forward(x, ids.cpu(), w.cpu(), wu, wg, wd, mode=2, return_y3=True)
    # (measured: bf16 1.34e-2, fp16 1.7e-3, bf16 with int8 weights whose scales make |W| reach 0.5 1.25e-2)
    layer_gate(y, out[0], out[5], w.cpu(), f"forward_logits {dt} w8={w8}")
    layer.close()


def test_router_errors(ek, cuda):
    layer = router_layer(ek, 64, 8)
    lg = torch.zeros(4, 64, device=cuda)

    def status(**kw):
        with pytest.raises(ek.EKError) as ei:
            layer.route(kw.pop("logits", lg), ek.RouterConfig(**kw))
        return ei.value.status

    assert status(kind=7) == C.EK_INVALID_INPUT
    assert status(kind=4, n_group=5, topk_group=1) == C.EK_INVALID_INPUT            # 5 does not divide 64
    assert status(kind=4, n_group=64, topk_group=8) == C.EK_INVALID_INPUT           # groups of one expert
    assert status(kind=4, n_group=8, topk_group=9) == C.EK_INVALID_INPUT
    assert status(kind=4, n_group=16, topk_group=1) == C.EK_INVALID_INPUT           # 4 experts kept < K = 8
    assert status(kind=0, bias=torch.zeros(64)) == C.EK_INVALID_INPUT               # bias without kind 4
    assert status(kind=0, w_dtype=torch.float16) == C.EK_INVALID_INPUT              # neither act dtype nor f32
    assert status(kind=0, logits=torch.zeros(9000, 64, device=cuda)) == C.EK_INVALID_INPUT   # T > max_tokens
    layer.close()
    big = ek.HipLayer(128, 128, 128, 65, max_tokens=4)
    with pytest.raises(ek.EKError) as ei:
        big.route(torch.zeros(2, 128, device=cuda), ek.RouterConfig(kind=0))
    assert ei.value.status == C.EK_INVALID_INPUT                                     # top_k > 64
    big.close()
