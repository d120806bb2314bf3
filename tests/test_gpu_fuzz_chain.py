"""Twelve seeded draws of a chain of two to five layers: weight kind, activation type, sizes, expert
count, top-k, token count, uniform or skewed routing, with or without shared experts, and sometimes
one layer object named twice.  The eager chain and three replays of its graph must give the bits of
the same layers called one after the other.  EKSEED=n draws another twelve."""
import os
import pytest
import torch
from ek_hip import workloads as wl
from test_gpu_chain import build_chain, bits
pytestmark = pytest.mark.gpu
SEED = int(os.environ.get("EKSEED", "0"))

@pytest.mark.parametrize("case", range(12))
def test_fuzz(ek, cuda, case):
    g = torch.Generator().manual_seed(SEED * 1000 + case + 31337)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    w8 = bool(r(0, 1))
    dt = [torch.bfloat16, torch.float16][r(0, 1)]
    step = 128 if w8 else 64
    H, I = step * r(1, 6), step * r(1, 4)
    E, K, L = r(2, 32), r(1, 4), r(2, 5)
    K = min(K, E)
    T = [r(1, 16), r(17, 200), r(201, 1500)][r(0, 2)]
    shared = r(0, 3) == 0
    tied = r(0, 3) == 0
    print(f"fuzz-chain seed={SEED} case={case} w8={w8} dt={dt} H={H} I={I} E={E} K={K} L={L} T={T} shared={shared} tied={tied}", flush=True)
    w0 = wl.Workload("fz", H, I, E, K, T, dt, w8=w8, zipf_s=[0.0, 1.2][r(0, 1)], n_layers=L)
    w, layers, weights, ids, gw = build_chain(ek, w0, cuda, std=0.08)
    if shared:
        for l, layer in enumerate(layers):
            layer.set_shared_expert(wl.make_expert(w, 900 + l, std=0.05))
    order = list(layers)
    if tied:
        order[-1] = order[0]
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
