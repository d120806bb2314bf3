"""Pins eko_ffn / dequant / combine / whole-layer forms against closed forms
(fp64 numpy), special cases and the libtorch evaluation of the same ops."""
import numpy as np
import pytest
import torch

DT = [torch.bfloat16, torch.float16]


def _rand_expert(g, H, I, dt, scale=0.05):
    mk = lambda r, c: (torch.randn(r, c, generator=g) * scale).to(dt)
    return mk(I, H), mk(I, H), mk(H, I)


def _np64(t):
    return t.float().numpy().astype(np.float64)


def _ideal_np(x, wu, wg, wd):
    up = _np64(x) @ _np64(wu).T            # transposed operand or swapped up/gate would fail here
    gate = _np64(x) @ _np64(wg).T
    h = up * (gate / (1.0 + np.exp(-gate)))
    return h @ _np64(wd).T, h


@pytest.mark.parametrize("dt", DT)
def test_ffn_ideal_vs_numpy(oracle, dt):
    g = torch.Generator().manual_seed(11)
    n, H, I = 5, 48, 80                     # H != I catches a transposed weight
    x = torch.randn(n, H, generator=g).to(dt)
    wu, wg, wd = _rand_expert(g, H, I, dt, 0.2)
    out, h = oracle.ffn(x, wu, wg, wd, mode=1, return_h=True)
    ref, href = _ideal_np(x, wu, wg, wd)
    np.testing.assert_allclose(h.numpy(), href, rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(out.numpy(), ref, rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("dt", DT)
def test_ffn_rounded_vs_libtorch(oracle, dt):
    """Same op sequence through libtorch CPU (what the reference calls via tch).
    The only freedom left is the fp32 accumulation order inside the GEMMs, so
    results agree to within one storage ulp almost everywhere."""
    g = torch.Generator().manual_seed(12)
    n, H, I = 7, 256, 192
    x = torch.randn(n, H, generator=g).to(dt)
    wu, wg, wd = _rand_expert(g, H, I, dt)
    got, h = oracle.ffn(x, wu, wg, wd, mode=0, return_h=True)
    ref = oracle.torch_ffn(x, wu, wg, wd)
    href = (x @ wu.T) * torch.nn.functional.silu(x @ wg.T)
    eps = 2.0 ** (-8 if dt == torch.bfloat16 else -11)
    for a, b in ((h, href), (got, ref)):
        a, b = a.float(), b.float()
        tol = 2 * eps * b.abs() + 2 * eps * b.abs().mean()
        assert bool(((a - b).abs() <= tol).all())
        assert float((a == b).float().mean()) > 0.9
    rms = ref.float().pow(2).mean().sqrt()
    assert float((got.float() - ref.float()).abs().max()) <= 2e-2 * float(rms)


@pytest.mark.parametrize("dt", DT)
def test_ffn_special_cases(oracle, dt):
    g = torch.Generator().manual_seed(13)
    n, H, I = 4, 64, 32
    x = torch.randn(n, H, generator=g).to(dt)
    wu, wg, wd = _rand_expert(g, H, I, dt)
    z = lambda t: torch.zeros_like(t)
    assert not oracle.ffn(z(x), wu, wg, wd).float().any()            # x = 0
    assert not oracle.ffn(x, wu, z(wg), wd).float().any()            # silu(0) = 0
    assert not oracle.ffn(x, z(wu), wg, wd).float().any()
    full = oracle.ffn(x, wu, wg, wd)
    for r in range(n):                                               # rows are independent
        one = oracle.ffn(x[r:r + 1], wu, wg, wd)
        assert torch.equal(one.view(torch.int16), full[r:r + 1].view(torch.int16))
    a = oracle.ffn(x, wu, wg, wd, mode=1)
    b = oracle.ffn(x, wu, wg, (wd.float() * 2).to(dt), mode=1)        # linear in W_down (x2 is exact)
    np.testing.assert_allclose(b.numpy(), 2 * a.numpy(), rtol=1e-6, atol=1e-9)
    # silu at a known point: gate = 1 -> 1/(1+e^-1)
    xe = torch.zeros(1, H, dtype=dt); xe[0, 0] = 1
    wu1 = z(wu); wu1[:, 0] = 1
    wg1 = z(wg); wg1[:, 0] = 1
    wd1 = z(wd); wd1[0, 0] = 1
    o = oracle.ffn(xe, wu1, wg1, wd1, mode=1)
    assert abs(float(o[0, 0]) - 1.0 / (1.0 + np.exp(-1.0))) < 1e-6


def test_dequant_channel(oracle):
    g = torch.Generator().manual_seed(14)
    q = torch.randint(-127, 128, (48, 96), generator=g, dtype=torch.int8)
    s = (torch.rand(48, generator=g) * 3e-3 + 1e-3).to(torch.bfloat16)
    got = oracle.dequant_channel(q, s)
    exact = q.numpy().astype(np.float64) * s.float().numpy().astype(np.float64)[:, None]
    ref = torch.from_numpy(exact).to(torch.bfloat16)     # product is exact in fp64 -> single rounding
    assert torch.equal(got.view(torch.int16), ref.view(torch.int16))
    assert torch.equal(got.view(torch.int16), oracle.torch_dequant_channel(q, s).view(torch.int16))
    assert float((got.float()[3] / s.float()[3] - q[3].float()).abs().max()) < 0.6   # right row gets right scale


def test_dequant_block_vs_reshape_form(oracle):
    """w8a16_activate spelled with the reference's own reshape/permute sequence
    (ffn/expert_torch.rs:24-53) in libtorch, against the per-element closed form."""
    g = torch.Generator().manual_seed(15)
    B, m, n = 128, 3, 2
    x = torch.randint(-127, 128, (m * B, n * B), generator=g, dtype=torch.int8)
    s = torch.rand(m, n, generator=g) * 1e-2
    l = x.reshape(m, B, n, B).permute(0, 2, 1, 3).reshape(m, n, B * B).to(torch.float)
    ref = (l * s.reshape(m, n, 1)).to(torch.bfloat16).reshape(m, n, B, B).permute(0, 2, 1, 3).reshape(x.shape)
    got = oracle.dequant_block(x, s, B)
    assert torch.equal(got.view(torch.int16), ref.contiguous().view(torch.int16))


@pytest.mark.parametrize("dt", DT)
@pytest.mark.parametrize("w_f32", [False, True])
def test_combine_vs_libtorch(oracle, dt, w_f32):
    g = torch.Generator().manual_seed(16)
    T, K, H = 9, 8, 40
    y3 = torch.randn(T, K, H, generator=g).to(dt)
    w = torch.rand(T, K, generator=g)
    w = (w / w.sum(-1, keepdim=True)).to(torch.float32 if w_f32 else dt)
    got = oracle.combine(y3, w)
    ref = torch.sum(w.unsqueeze(-1) * y3, dim=1).to(dt)       # qwen3_moe.py:103-104
    diff = (got.float() - ref.float()).abs()
    eps = 2.0 ** (-8 if dt == torch.bfloat16 else -11)
    assert bool((diff <= eps * ref.float().abs() + 1e-6).all())
    assert float((got.float() == ref.float()).float().mean()) > 0.97
    # K = 1, w = 1 -> identity
    one = oracle.combine(y3[:, :1].contiguous(), torch.ones(T, 1, dtype=w.dtype))
    assert torch.equal(one.view(torch.int16), y3[:, 0].contiguous().view(torch.int16))


@pytest.mark.parametrize("dt", DT)
def test_layer_forms_agree(oracle, dt):
    """EK form (pack/gather/ffn/scatter/combine) == stock loop form (index_add_)
    up to storage rounding, and == ideal form within the parity tolerance."""
    g = torch.Generator().manual_seed(17)
    T, K, E, H, I = 24, 3, 6, 64, 32
    x = torch.randn(T, H, generator=g).to(dt)
    logits = torch.randn(T, E, generator=g)
    ids, w = oracle.torch_router(logits, K, True, dt)
    ws = [_rand_expert(g, H, I, dt, 0.1) for _ in range(E)]
    wu, wg, wd = [list(t) for t in zip(*ws)]
    y, counts, offsets, perm, inv = oracle.layer_forward(x, ids, w, wu, wg, wd, mode=0)
    y_loop = oracle.layer_loop_form(x, ids, w, wu, wg, wd)
    y_ideal = oracle.layer_forward(x, ids, w, wu, wg, wd, mode=1)[0]
    y_torch, done = oracle.torch_layer_forward(x, ids, w, wu, wg, wd)
    assert done == T * K
    rms = float(y_ideal.pow(2).mean().sqrt())
    # storage roundings alone (5 per element, bf16 eps 2^-8) put the rounded forms
    # a few 1e-2 x RMS from the unrounded one in max norm; among themselves they
    # differ only by accumulation order and the order of the final sum
    for other in (y_loop, y_torch, y):
        assert float((other.float() - y_ideal).abs().max()) <= 5e-2 * rms
    assert float((y.float() - y_torch.float()).abs().max()) <= 1e-2 * rms
    assert float((y.float() - y_loop.float()).abs().max()) <= 2e-2 * rms
    ref = oracle.brute_pack(ids, E)
    for a, b in zip((counts, offsets, perm, inv), ref):
        assert torch.equal(a, b)
    # an expert nobody selects may have no weights; a selected one must
    unused = [e for e in range(E) if int(counts[e]) == 0]
    used = int(ids[0, 0])
    wu2 = list(wu); wu2[used] = None
    with pytest.raises(ValueError):
        oracle.layer_forward(x, ids, w, wu2, wg, wd)
    for e in unused:
        wu3, wg3, wd3 = list(wu), list(wg), list(wd)
        wu3[e] = wg3[e] = wd3[e] = None
        y3 = oracle.layer_forward(x, ids, w, wu3, wg3, wd3)[0]
        assert torch.equal(y3.view(torch.int16), y.view(torch.int16))


def test_router_vs_libtorch(oracle):
    g = torch.Generator().manual_seed(18)
    logits = torch.randn(200, 64, generator=g)
    ids, w = oracle.router(logits, 8, True, torch.float32)
    rid, rw = oracle.torch_router(logits, 8, True, torch.float32)
    assert torch.equal(ids, rid)                      # descending weight, distinct experts
    np.testing.assert_allclose(w.numpy(), rw.numpy(), rtol=1e-5)
    np.testing.assert_allclose(w.sum(-1).numpy(), 1.0, rtol=1e-5)
    ids2, w2 = oracle.router(logits, 8, False, torch.bfloat16)
    p = torch.softmax(logits, 1)
    assert torch.equal(w2.view(torch.int16), torch.gather(p, 1, ids2.long()).to(torch.bfloat16).view(torch.int16)) or \
        float((w2.float() - torch.gather(p, 1, ids2.long())).abs().max()) < 1e-3
    # tie rule: equal logits -> lower index first
    tid, _ = oracle.router(torch.zeros(1, 5), 2)
    assert tid.tolist() == [[0, 1]]


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_silu_form_of_the_kernels_equals_the_libm_form_for_every_16bit_gate(oracle, dt):
    """The HIP kernels evaluate silu(gate) = gate / (1 + exp(-gate)) with an exp made of IEEE fma / mul / add
    only (restated as eko_expf_wide); eko_ffn, the oracle, uses libm's expf.  The two exps differ in the last
    fp32 bit now and then; after the storage rounding of silu(gate) to the activation type they agree for
    every one of the 65536 gate values of that type, so the choice of exp cannot show in a parity figure."""
    pat = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dt)
    g = pat.float()
    fin = torch.isfinite(g)
    a, b = oracle.silu_forms(g[fin])
    assert (a != b).sum() < 2000                       # they are different routines ...
    ra, rb = a.to(dt), b.to(dt)
    assert torch.equal(ra.view(torch.int16), rb.view(torch.int16))   # ... with the same rounded results
    # overflow side: exp(88.5) is finite, exp(89) is not
    lo, hi = oracle.silu_forms(torch.tensor([-88.5, -89.0, -1e30, 89.0, 1e30]))
    assert torch.equal(lo, hi) and lo[0] < 0 and lo[1] == 0 and lo[3] == 89.0
