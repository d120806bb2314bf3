"""Twenty seeded draws of a layer with a shared expert (deepseek_v3/model.py:57-61,152: every token
once, added to the rounded routed sum): weight kind, activation type, sizes, expert count, top-k and
1 to 1500 tokens, so that the shared segment is met as 16-row streaming items, as 64-row ones on the
side stream and as tiles, beside every mix of routed segments; in half of the draws the shared
expert is two or three times as wide as the routed ones (launches of its own).  Held to the oracle's layer plus
add_shared by test_gpu_shared.py's bound, and to the same call on host tensors.
EKSEED=n draws another twenty."""
import os
import pytest
import torch
from ek_hip import _capi as C
from ek_hip import workloads as wl
from test_gpu_block_scaled import KINDS, make_expert as make_block_expert, ref_weights
from test_gpu_parity import TOL, oracle_weights, ulp_of
pytestmark = pytest.mark.gpu
SEED = int(os.environ.get("EKSEED", "0"))

@pytest.mark.parametrize("case", range(20))
def test_fuzz(ek, oracle, cuda, case):
    g = torch.Generator().manual_seed(SEED * 1000 + case + 4242)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    kind = ["w16", "i8", "fp8", "int8"][r(0, 3)]
    dt = [torch.bfloat16, torch.float16][r(0, 1)]
    step = 64 if kind == "w16" else 128
    H, I = step * r(1, 8), step * r(1, 5)
    E, K = r(2, 24), r(1, 4)
    K = min(K, E)
    T = [r(1, 16), r(17, 64), r(65, 256), r(257, 1500)][r(0, 3)]
    n_shared = [1, 1, 2, 3][r(0, 3)]      # the shared expert has moe_intermediate_size * n_shared_experts channels
    print(f"fuzz-shared seed={SEED} case={case} kind={kind} dt={dt} H={H} I={I} x{n_shared} E={E} K={K} T={T}", flush=True)
    if kind in KINDS:
        layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=T, **KINDS[kind])
        ws = [make_block_expert(ek, H, I * (n_shared if e == 4 else 1), 100 * case + e, kind) for e in range(5)]
        ref_w = [ref_weights(oracle, ew, dt) for ew in ws]
    else:
        w = wl.Workload("t", H, I, E, K, T, dt, w8=kind == "i8")
        layer = ek.HipLayer(H, I, E, K, act_dtype=dt, w_dtype=torch.int8 if w.w8 else dt, max_tokens=T)
        ws = [wl.make_expert(w, 100 * case + e, std=0.05) for e in range(4)]
        ws.append(wl.make_expert(wl.Workload("t", H, I * n_shared, E, K, T, dt, w8=w.w8), 100 * case + 4, std=0.05))
        cols = oracle_weights(oracle, dict(enumerate(ws)), 5, dt)
        ref_w = [tuple(c[i] for c in cols) for i in range(5)]
    for e in range(E):
        layer.set_expert(e, ws[e % 4])
    layer.set_shared_expert(ws[4])
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32).reshape(T, K)
    gw = torch.rand(T, K, generator=g) + 0.1
    gw = (gw / gw.sum(-1, keepdim=True)).to(dt)
    x = torch.randn(T, H, generator=g).to(dt)
    wu, wg, wd = zip(*[ref_w[e % 4] for e in range(E)])
    y = layer.forward(x.to(cuda), ids.to(cuda), gw.to(cuda))
    y_r = oracle.layer_forward(x, ids, gw, list(wu), list(wg), list(wd), mode=0)[0]
    ref32 = oracle.add_shared(y_r, x, *ref_w[4], rounded=False)
    y_s = ref32 - y_r.float()
    rms = float(ref32.pow(2).mean().sqrt())
    err = (y.float().cpu() - ref32).abs()
    quanta = 0.5 * ulp_of(ref32, dt) * 1.0001 + ulp_of(y_r.float(), dt) + ulp_of(y_s, dt)
    worst = float(err.max()) / rms
    over = float((err > TOL * rms).float().mean())
    print(f"fuzz-shared {case}: max|err|/rms = {worst:.3e}, over 2e-2*rms: {over:.2e}", flush=True)
    assert bool((err <= TOL * rms + quanta).all()), worst
    assert over <= 1e-4 or T * H * over <= 2
    assert torch.equal(layer.forward(x, ids, gw).view(torch.int16), y.cpu().view(torch.int16))
    layer.close()
