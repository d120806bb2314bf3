"""Whole-layer parity at full size: EVERY output row of the benchmark configurations, not a sample.

The library's call (pack -> grouped FFN -> combine over all experts at once) is held to the
reference's own procedure evaluated on the host by libtorch, the library the reference calls:
one expert at a time (ek-computation/src/controller/executor.rs:141-195 sends one request per
expert; ffn/expert_torch.rs:61-78 holds the weights cast to the compute type, :81-84 are the four
ops), results scattered into [T, K, H] (executor.rs:203-252), weighted sum over k
(expertkit_torch/models/qwen3_moe.py:102-104).  Weights are streamed through the host one expert
at a time.  A fault tied to one tile index, one XCD's share of a work list or one position of the
load pipeline moves whole rows x channel blocks far outside the gate and cannot hide.

Anchors: the host evaluation itself is held to the scalar C oracle on sampled tokens (bit for bit
but for single-ulp differences of accumulation order).
"""
import time

import pytest
import torch

import parity_report
from ek_hip import workloads as wl
from test_gpu_parity import TOL, load_layer, ulp_of

pytestmark = pytest.mark.gpu


def host_weights(oracle, ew, dt):
    """What load_module holds for one expert: 16-bit tensors on the host (int8 dequantised with
    libtorch ops: fp32 product, one rounding)."""
    if ew.up_w.dtype == torch.int8:
        return tuple(oracle.torch_dequant_channel(q.cpu(), s.cpu(), dt) for q, s in
                     ((ew.up_w, ew.up_scale), (ew.gate_w, ew.gate_scale), (ew.down_w, ew.down_scale)))
    return ew.up_w.cpu(), ew.gate_w.cpu(), ew.down_w.cpu()


def reference_layers(oracle, cases, ws, n_experts, dt):
    """cases: list of (x, ids, gw) on the host sharing one set of experts.  Returns per case the
    reference's y [T, H] and Y [T, K, H]; every expert's weights are brought to the host once."""
    y3 = [torch.zeros(ids.numel(), x.shape[1], dtype=dt) for x, ids, _ in cases]
    order = [torch.argsort(ids.reshape(-1).long(), stable=True) for _, ids, _ in cases]
    counts = [torch.bincount(ids.reshape(-1).long(), minlength=n_experts) for _, ids, _ in cases]
    offs = [torch.cat([torch.zeros(1, dtype=torch.long), c.cumsum(0)]) for c in counts]
    for e in range(n_experts):
        if not any(int(c[e]) for c in counts):
            continue
        wu, wg, wd = host_weights(oracle, ws[e], dt)
        for i, (x, ids, _) in enumerate(cases):
            n = int(counts[i][e])
            if n:
                pairs = order[i][int(offs[i][e]):int(offs[i][e]) + n]
                y3[i][pairs] = oracle.torch_ffn(x.index_select(0, pairs // ids.shape[1]), wu, wg, wd)
    out = []
    for i, (x, ids, gw) in enumerate(cases):
        T, K = ids.shape
        Y = y3[i].view(T, K, -1)
        out.append((torch.sum(gw.unsqueeze(-1) * Y, dim=1).to(dt), Y))
    return out


def classify_excess(name, y, y_ref, Y, yp, inv_perm, over, gw):
    """The sharp statement behind the envelope, element by element.  Every output further than
    2e-2 * rms from libtorch's value is either (a) within one ulp of the output type from it (two
    16-bit outputs on either side of a rounding boundary), or (b) the weighted sum of expert outputs
    Y[t, k, c] of which some were stored as another 16-bit value than libtorch's (accumulation order
    decided a rounding inside that expert), and those differences account for it:
        |y - y_ref| <= ulp(y_ref) + sum_k (|w_k| |Y_k - Y_ref_k| + [Y_k != Y_ref_k] ulp(w_k Y_ref_k))
    (the reference rounds each product w_k Y_k to the 16-bit type before the sum; a product of a
    different Y may round to the other side).  Each differing stored expert output is in turn
    within 2e-2 * rms(Y) of libtorch's plus half an ulp of its own for either side's storage.
    Y of the library's call: rows of its packed expert outputs `yp` (ek_route_out.expert_out),
    found through inv_perm."""
    T, K, H = Y.shape
    tc = over.nonzero()                                        # [n, 2] token, channel
    if tc.numel() == 0:
        print(f"{name}: no output over 2e-2 * rms", flush=True)
        return 0, 0
    t, c = tc[:, 0], tc[:, 1]
    err = (y.float() - y_ref.float()).abs()[t, c]
    u_out = ulp_of(y_ref, y.dtype)[t, c]
    one_ulp = err <= u_out * 1.0001
    rows = inv_perm.view(T, K)[t].long()                        # [n, K] packed rows of the token's pairs
    mine = yp[rows.to(yp.device), c.to(yp.device).unsqueeze(1)].cpu().float()      # [n, K]
    theirs = Y[t, :, c].float()                                 # [n, K]
    w = gw.float()[t]                                           # [n, K]
    d = (mine - theirs).abs()
    carried = (w.abs() * d + (d > 0).float() * ulp_of(w * theirs, y.dtype)).sum(dim=1)
    accounted = err <= (u_out + carried) * 1.0001
    rms_Y = float(Y.float().pow(2).mean().sqrt())
    inside = (d <= TOL * rms_Y + ulp_of(theirs, y.dtype) * 1.0001).all(dim=1)
    a, b = int(one_ulp.sum()), int((accounted & inside & ~one_ulp).sum())
    rest = ~(one_ulp | (accounted & inside))
    for i in rest.nonzero().flatten().tolist()[:20]:
        print(f"   unexplained [{int(t[i])}, {int(c[i])}]: |y - y_ref| = {float(err[i] / u_out[i]):.2f} output ulps; "
              f"expert outputs off by {[float(v) for v in d[i].tolist()]}; gate weights {[round(float(v), 3) for v in w[i].tolist()]}", flush=True)
    print(f"{name}: {tc.shape[0]} outputs over 2e-2 * rms: {a} within one output ulp of libtorch's value, "
          f"{b} more accounted for by stored expert outputs that differ (each within the one-expert gate), "
          f"{int(rest.sum())} unexplained", flush=True)
    assert not bool(rest.any()), (f"{name}: output [{int(t[rest][0])}, {int(c[rest][0])}] is over the plain bound, further "
                                  f"than one ulp from libtorch's, and the stored expert outputs do not account for it")
    return a, b


def hold_to_reference(name, y, y_ref, Y, gw, yp=None, inv_perm=None):
    """Both sides are 16-bit outputs.  Every element: within 2e-2 * rms plus the storage quanta (one
    ulp of y: half for each side's storage rounding; one ulp of the largest gate-weighted term);
    all but 5e-4 of them within the plain 2e-2 * rms; nine in ten bit-identical; and every element
    over the plain bound explained one by one (classify_excess)."""
    y, y_ref = y.cpu(), y_ref.cpu()
    rms = float(y_ref.float().pow(2).mean().sqrt())
    err = (y.float() - y_ref.float()).abs()
    quanta = ulp_of(y_ref, y.dtype) + ulp_of((gw.float().unsqueeze(-1) * Y.float()).abs().amax(dim=1), y.dtype)
    worst = float(err.max()) / rms
    over = float((err > TOL * rms).float().mean())
    same = float((y.view(torch.int16) == y_ref.view(torch.int16)).float().mean())
    parity_report.record(f"{name} every row vs the reference's procedure on libtorch", worst, over, err.numel(), False,
                         float(ulp_of(y_ref, y.dtype).max()) * 0.5 / rms)
    print(f"{name}: {err.numel()} outputs, max|err|/rms = {worst:.3e}, over 2e-2*rms: {over:.2e}, bit-identical: {same:.4f}", flush=True)
    bad = err > TOL * rms + quanta
    assert not bool(bad.any()), f"{name}: {int(bad.sum())} outputs outside the gate, first at {torch.nonzero(bad)[0].tolist()}"
    if yp is not None:
        classify_excess(name, y, y_ref, Y, yp, inv_perm.cpu(), err > TOL * rms, gw.float())
    # two stored 16-bit outputs one ulp apart are further than 2e-2 * rms from each other beyond ~3 sigma:
    # the share over the plain bound is a share of the one-ulp differences (measured 1.3e-4 for c4)
    assert over <= 5e-4 and same > 0.9, (over, same)


def anchor_to_oracle(oracle, name, y_ref, case, ws, n_experts, dt):
    """The host evaluation against the scalar oracle's fully rounded form on sampled tokens."""
    from oracle import sampled
    x, ids, gw = case
    tokens = sampled.choose_tokens(ids, n_experts)
    r = sampled.check(y_ref[tokens], x[tokens], ids[tokens], gw[tokens], n_experts, lambda e: ws[e])
    rounded = r["ref"].to(dt)
    same = float((y_ref[tokens].view(torch.int16) == rounded.view(torch.int16)).float().mean())
    print(f"{name}: libtorch vs the C oracle on tokens {tokens}: bit-identical {same:.4f}, max|err|/rms {r['max_err_over_rms']:.3e}", flush=True)
    assert same > 0.95
    quanta = 0.5 * ulp_of(r["ref"], dt) * 1.0001 + ulp_of((gw[tokens].float().unsqueeze(-1) * r["y3"].float()).abs().amax(dim=1), dt)
    rms = float(r["ref"].pow(2).mean().sqrt())
    assert bool(((y_ref[tokens].float() - r["ref"]).abs() <= TOL * rms + quanta).all())


@pytest.mark.parametrize("names", [("c4", "c3"), ("c2", "c5")])
def test_every_output_row_at_full_size(ek, oracle, cuda, names):
    """c4 + c3 share the 256 DeepSeek-V3 W8A16 experts (8192 prefill tokens, 128 decode tokens);
    c2 + the first layer of c5 share the 128 Qwen3 fp16 experts (256 decode tokens, the ragged
    5052-token mix)."""
    wls = [wl.resolve(wl.CONFIGS[n]) for n in names]
    big = max(wls, key=lambda w: w.tokens)
    dt = big.act_dtype
    t0 = time.time()
    print(f"{names}: building {big.n_experts} experts on the GPU", flush=True)
    layer, ws = load_layer(ek, big, device="cuda")
    cases, ys, yps, inv_perms = [], [], [], []
    for w in wls:
        x = wl.make_x(w)
        ids, gw = wl.make_routing(w)
        cases.append((x, ids, gw))
        yp = torch.empty(ids.numel(), w.hidden, dtype=dt, device=cuda)     # every pair's expert output, packed order
        y, rt = layer.forward(x.to(cuda), ids.to(cuda), gw.to(cuda), return_route=True, expert_out=yp)
        assert torch.equal(layer.forward(x.to(cuda), ids.to(cuda), gw.to(cuda)), y)
        ys.append(y.cpu())
        yps.append(yp)
        inv_perms.append(rt.inv_perm.cpu())
    print(f"{names}: GPU calls done at {time.time() - t0:.1f} s; the reference's procedure on the host ...", flush=True)
    refs = reference_layers(oracle, cases, ws, big.n_experts, dt)
    print(f"{names}: host evaluation done at {time.time() - t0:.1f} s", flush=True)
    for name, w, case, y, (y_ref, Y), yp, inv_perm in zip(names, wls, cases, ys, refs, yps, inv_perms):
        hold_to_reference(name, y, y_ref, Y, case[2], yp, inv_perm)
        anchor_to_oracle(oracle, name, y_ref, case, ws, w.n_experts, dt)
    print(f"{names}: done at {time.time() - t0:.1f} s", flush=True)
    layer.close()
