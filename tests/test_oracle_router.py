"""Pins the oracle's routers (eko_route) without the GPU.

Checkers, none of which shares code with the oracle:
  * libm / float64 for eko_expf (the IEEE-operations-only exp the routers use);
  * torch primitives written after the reference's lines (oracle.torch_route);
  * transformers' own DeepseekV3TopkRouter (installed package, third party to the
    reference) fed with an identity gate so that its logits are the test's logits;
  * hand-worked tiny cases chosen so that a plausible mistake (group limit ignored,
    biased scores used as weights, wrong mask value, wrong tie order) changes the answer.
"""
import math
import types

import numpy as np
import pytest
import torch

from ek_hip import workloads as wl


def ulp32(v):
    return np.spacing(np.abs(np.float32(v)))


def test_expf_within_two_ulp_and_clamped(oracle):
    g = torch.Generator().manual_seed(1)
    xs = torch.cat([torch.linspace(-87, 88, 4001), torch.randn(4000, generator=g) * 4,
                    torch.tensor([0.0, -0.0, 1.0, -1.0, 0.5 * math.log(2), -0.5 * math.log(2), 1e-8, -1e-8,
                                  -87.0, 88.0])]).float()
    got = oracle.expf(xs).numpy().astype(np.float64)
    want = np.exp(xs.numpy().astype(np.float64))
    err = np.abs(got - want) / ulp32(want.astype(np.float32)).astype(np.float64)
    print("eko_expf max error: %.3f ulp" % err.max())
    assert err.max() <= 2.0
    assert float(oracle.expf(torch.tensor([0.0]))[0]) == 1.0
    # clamped outside the range of normal results; never inf, zero or subnormal
    lo, hi = oracle.expf(torch.tensor([-1000.0, 1000.0])).tolist()
    assert lo == float(oracle.expf(torch.tensor([-87.0]))[0]) and lo >= 2.0 ** -126
    assert hi == float(oracle.expf(torch.tensor([88.0]))[0]) and math.isfinite(hi)
    # monotone where the routers use it most (differences to the row maximum)
    fine = torch.linspace(-12, 0, 20001).float()
    assert bool((oracle.expf(fine).diff() >= 0).all())


def seeded_logits(w, layer=0):
    g = torch.Generator().manual_seed(3000 + layer)
    logits = torch.randn(w.tokens, w.n_experts, generator=g)
    b = wl.expert_bias(w)
    return logits + b if b is not None else logits


@pytest.mark.parametrize("cfg", ["c1", "c2", "c3"])
@pytest.mark.parametrize("renorm", [True, False])
def test_softmax_topk_matches_reference_lines(oracle, cfg, renorm):
    w = wl.CONFIGS[cfg]
    logits = seeded_logits(w)
    ids, gw = oracle.route(0, logits, w.top_k, renorm)
    t_ids, t_w = oracle.torch_route(0, logits, w.top_k, renorm)
    assert torch.equal(ids, t_ids)
    assert float(((gw - t_w).abs() / t_w).max()) < 1e-6
    # the workloads' own router (libm exp, choice made on the probabilities)
    o_ids, o_w = oracle.router(logits, w.top_k, renorm)
    assert torch.equal(ids, o_ids)
    assert float(((gw - o_w).abs() / o_w).max()) < 1e-6
    if renorm:
        assert float((gw.sum(-1) - 1).abs().max()) < 1e-6
    # cast to the activation dtype as qwen3_moe.py:169 does: at most one rounding step apart
    for dt in (torch.bfloat16, torch.float16):
        c_w = oracle.route(0, logits, w.top_k, renorm, w_dtype=dt)[1]
        assert torch.equal(c_w, gw.to(dt))


@pytest.mark.parametrize("kind", [1, 2, 3])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16, torch.float16])
def test_vllm_shim_routers(oracle, kind, dt):
    g = torch.Generator().manual_seed(11)
    # distinct values even after rounding to 16 bits: a shuffled grid
    T, E, K = 64, 64, 6
    base = torch.linspace(-4, 4, E)
    logits = torch.stack([base[torch.randperm(E, generator=g)] for _ in range(T)]).to(dt)
    assert all(len(set(r.tolist())) == E for r in logits.float())
    ids, gw = oracle.route(kind, logits, K, w_dtype=torch.float32)
    t_ids, t_w = oracle.torch_route(kind, logits.float(), K)
    assert torch.equal(ids, t_ids)
    if kind == 1:
        assert torch.equal(gw, t_w)
    else:
        assert float(((gw - t_w).abs() / t_w).max()) < 1e-6


def ds_router(E, K, n_group, topk_group, renorm, scaling, bias):
    """transformers' DeepseekV3TopkRouter with an identity gate: router_logits == its input."""
    from transformers.models.deepseek_v3.modeling_deepseek_v3 import DeepseekV3TopkRouter
    cfg = types.SimpleNamespace(num_experts_per_tok=K, num_local_experts=E, n_routed_experts=E, hidden_size=E,
                                routed_scaling_factor=scaling, n_group=n_group, topk_group=topk_group,
                                norm_topk_prob=renorm)
    r = DeepseekV3TopkRouter(cfg)
    with torch.no_grad():
        r.weight.copy_(torch.eye(E))
        r.e_score_correction_bias.copy_(bias)
    return r


@pytest.mark.parametrize("renorm", [True, False])
def test_group_limited_router_matches_transformers(oracle, renorm):
    """ds-tiny / DeepSeek-V3 parameters (ek-db/resources/ds-tiny/config.json:26-48)."""
    E, K, n_group, topk_group, scaling, T = 256, 8, 8, 4, 2.5, 512
    g = torch.Generator().manual_seed(21)
    logits = torch.randn(T, E, generator=g) * 1.5
    bias = torch.randn(E, generator=g) * 0.1
    ids, gw = oracle.route(4, logits, K, renorm, bias=bias, n_group=n_group, topk_group=topk_group,
                           mask_neg_inf=True, routed_scaling=scaling)
    r = ds_router(E, K, n_group, topk_group, renorm, scaling, bias)
    with torch.no_grad():
        out = r(logits)
    t_logits, t_w, t_ids = out if len(out) == 3 else (logits, out[1], out[0])
    assert torch.equal(t_logits, logits)          # the identity gate did what it should
    # transformers leaves the order inside a token open (sorted=False): compare as sets
    order_o, order_t = ids.long().argsort(dim=1), t_ids.argsort(dim=1)
    s_ids, s_w = ids.long().gather(1, order_o), gw.gather(1, order_o)
    st_ids, st_w = t_ids.gather(1, order_t), t_w.gather(1, order_t)
    same = (s_ids == st_ids).all(dim=1)
    # torch's sigmoid and eko_sigmoidf differ by an ulp or two: a token may differ only where the
    # K-th and (K+1)-th choice values are that close
    choice = torch.sigmoid(logits) + bias
    for t in (~same).nonzero().flatten().tolist():
        only = set(s_ids[t].tolist()) ^ set(st_ids[t].tolist())
        vals = choice[t, sorted(only)]
        assert float(vals.max() - vals.min()) < 1e-6, t
    assert float(same.float().mean()) > 0.99
    assert float(((s_w - st_w).abs() / st_w)[same].max()) < 2e-6
    # the same against the torch-primitive form, whose order is ours (descending choice value)
    p_ids, p_w = oracle.torch_route(4, logits, K, renorm, bias=bias, n_group=n_group, topk_group=topk_group,
                                    mask_neg_inf=True, routed_scaling=scaling)
    rows = (ids == p_ids).all(dim=1)
    assert float(rows.float().mean()) > 0.99
    assert float(((gw - p_w).abs() / p_w)[rows].max()) < 2e-6


def sig(v):
    return 1.0 / (1.0 + math.exp(-v))


def test_group_limit_hand_case(oracle):
    """E = 8 in 4 groups of 2, keep 2 groups, K = 2.
    logits: group 0 = {3.0, -3.0}, group 1 = {2.0, 1.9}, group 2 = {2.5, -4.0}, group 3 = {-.2, -.2}.
    Group scores (sum of both members' sigmoid): g0 1.000, g1 1.751, g2 0.942, g3 0.900.
    Kept: g1 and g0.  Plain top-2 would pick experts 0 and 4; the group limit excludes
    expert 4 (group 2), so the answer is experts 0 and 2."""
    logits = torch.tensor([[3.0, -3.0, 2.0, 1.9, 2.5, -4.0, -0.2, -0.2]])
    ids, gw = oracle.route(4, logits, 2, False, n_group=4, topk_group=2, routed_scaling=1.0)
    assert ids.tolist() == [[0, 2]]
    assert gw[0].tolist() == pytest.approx([sig(3.0), sig(2.0)], rel=1e-6)
    # renormalised and scaled
    _, gw = oracle.route(4, logits, 2, True, n_group=4, topk_group=2, routed_scaling=2.5)
    tot = sig(3.0) + sig(2.0)
    assert gw[0].tolist() == pytest.approx([2.5 * sig(3.0) / tot, 2.5 * sig(2.0) / tot], rel=1e-6)


def test_bias_steers_the_choice_but_not_the_weights(oracle):
    logits = torch.tensor([[3.0, -3.0, 2.0, 1.9, 2.5, -4.0, 0.0, 0.0]])
    bias = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.9, 0.9])   # lifts group 3 to 2.8
    ids, gw = oracle.route(4, logits, 2, False, bias=bias, n_group=4, topk_group=2, routed_scaling=1.0)
    # kept groups: g3 (2.8) and g1 (1.751); choice values: e6 = e7 = 1.4, e2 = 0.881, e3 = 0.870
    assert ids.tolist() == [[6, 7]]
    assert gw[0].tolist() == pytest.approx([0.5, 0.5], rel=1e-6)       # sigmoid(0), not 1.4


def test_mask_value_matters_for_negative_choice_values(oracle):
    """With a negative bias every kept expert's choice value is below 0, so the 0.0 that the
    masked experts carry in transformers 4.51.3 wins (lowest indices first); -inf does not."""
    logits = torch.tensor([[3.0, -3.0, 2.0, 1.9, 2.5, -4.0, -0.2, -0.2]])
    bias = torch.full((8,), -2.0)
    z_ids, _ = oracle.route(4, logits, 2, False, bias=bias, n_group=4, topk_group=2)
    n_ids, _ = oracle.route(4, logits, 2, False, bias=bias, n_group=4, topk_group=2, mask_neg_inf=True)
    # kept groups g1 (-2.25) and g0 (-3.0, above g2's -3.06 and g3's -3.1); masked: experts 4..7
    assert z_ids.tolist() == [[4, 5]]
    assert n_ids.tolist() == [[0, 2]]
    t_ids, _ = oracle.torch_route(4, logits, 2, False, bias=bias, n_group=4, topk_group=2)
    assert set(t_ids[0].tolist()) <= {4, 5, 6, 7}     # torch picks any two of the equal zeros


@pytest.mark.parametrize("kind", [0, 1, 2, 3])
def test_equal_logits_go_to_the_lower_index(oracle, kind):
    logits = torch.tensor([[1.0, 2.0, 2.0, 0.5, 2.0, 1.0]])
    ids, _ = oracle.route(kind, logits, 4)
    assert ids.tolist() == [[1, 2, 4, 0]]


def test_bad_arguments(oracle):
    logits = torch.zeros(2, 8)
    for kw in (dict(n_group=3, topk_group=1), dict(n_group=8, topk_group=1), dict(n_group=4, topk_group=5),
               dict(n_group=4, topk_group=1)):      # 1 group of 2 cannot supply K = 3
        with pytest.raises(ValueError):
            oracle.route(4, logits, 3, **kw)
    with pytest.raises(ValueError):
        oracle.route(0, logits, 9)
