"""Why the parity gates are shaped as they are, shown on the CPU with the reference's own arithmetic.

The stated tolerance is max|y - y_ref| <= 2e-2 * rms(y_ref).  The GPU tests assert it as it stands
wherever it holds, against y_ref = the oracle's reference-rounded form before its last storage
rounding (mode 2).  Where they do not, they assert the bound plus storage quanta of the 16-bit
tensors the reference materialises.  These tests show, without any GPU code, that faithful CPU
evaluations of the reference's op sequence (ek-computation/src/ffn/expert_torch.rs:81-84 and
qwen3_moe.py:102-104: the oracle's correctly rounded mode 0, its fp32-accumulating mode 3, and
the libtorch kernels the reference itself calls) already lie outside the plain bound, by exactly
those quanta:

  * against the fp32-accumulate "ideal" form (mode 1) the reference exceeds the bound on the
    benchmark's own tiny configuration: that form is reported, never gated;
  * against mode 2 the correctly rounded reference output is up to half an output ulp away,
    which beyond 4 sigma is more than 2e-2 * rms in bf16;
  * two evaluations that differ only in fp32 accumulation order store a few intermediates one
    ulp apart; where such a flip meets a large gate-weighted term the output moves by more than
    the bound plus half an ulp.
"""
import torch

import parity_report  # noqa: F401  (keeps the test directory importable the same way as the GPU tests)
from ek_hip import workloads as wl

TOL = 2e-2


def ulp_of(v: torch.Tensor, dtype) -> torch.Tensor:
    bits = 7 if dtype == torch.bfloat16 else 10
    return torch.exp2(torch.floor(torch.log2(v.float().abs().clamp_min(1e-30))) - bits)


def build(oracle, w, seed=0, std=0.02):
    ws = [wl.make_expert(w, e, layer=seed, std=std) for e in range(w.n_experts)]
    dt = w.act_dtype
    if w.w8:
        wu = [oracle.dequant_channel(e.up_w, e.up_scale, dt) for e in ws]
        wg = [oracle.dequant_channel(e.gate_w, e.gate_scale, dt) for e in ws]
        wd = [oracle.dequant_channel(e.down_w, e.down_scale, dt) for e in ws]
    else:
        wu, wg, wd = [e.up_w for e in ws], [e.gate_w for e in ws], [e.down_w for e in ws]
    return wu, wg, wd


def test_fp32_ideal_form_cannot_be_the_gate(oracle):
    """C1 (the configuration the reference's CPU backend runs): the reference's arithmetic,
    evaluated by libtorch and by the oracle's mode 0, is further than 2e-2 * rms from the
    unrounded fp32/fp64 form, because it stores up, gate, silu(gate) and their product in bf16."""
    w = wl.C1
    wu, wg, wd = build(oracle, w)
    x = wl.make_x(w)
    ids, gw = wl.make_routing(w)
    ideal = oracle.layer_forward(x, ids, gw, wu, wg, wd, mode=1)[0]
    rms = float(ideal.pow(2).mean().sqrt())
    twin, _ = oracle.torch_layer_forward(x, ids, gw, wu, wg, wd)
    rounded = oracle.layer_forward(x, ids, gw, wu, wg, wd, mode=0)[0]
    for name, y in (("libtorch", twin), ("oracle mode 0", rounded)):
        worst = float((y.float() - ideal).abs().max()) / rms
        print(f"c1 {name} vs ideal: max|err|/rms = {worst:.3e}")
        assert worst > TOL, (name, worst)
        assert worst < 3 * TOL


def test_last_storage_rounding_alone_exceeds_the_plain_bound(oracle):
    """Segment lengths 0..hundreds, bf16, top-2: the correctly rounded reference output (mode 0)
    against the same value before its storage rounding (mode 2).  Nothing but one rounding to
    bf16 separates the two, and the largest element's half ulp is more than 2e-2 * rms."""
    w = wl.Workload("ragged", 256, 128, 24, 2, 400, torch.bfloat16, zipf_s=2.0)
    wu, wg, wd = build(oracle, w)
    x = wl.make_x(w)
    ids, gw = wl.make_routing(w)
    ref = oracle.layer_forward(x, ids, gw, wu, wg, wd, mode=2)[0]
    rounded = oracle.layer_forward(x, ids, gw, wu, wg, wd, mode=0)[0]
    assert torch.equal(rounded, ref.to(torch.bfloat16))          # (that is all mode 0 adds)
    rms = float(ref.pow(2).mean().sqrt())
    err = (rounded.float() - ref).abs()
    worst = float(err.max()) / rms
    print(f"ragged: rounded reference vs its unrounded value: max|err|/rms = {worst:.3e}")
    assert worst > TOL
    assert bool((err <= 0.5 * ulp_of(ref, torch.bfloat16) * 1.0001).all())
    # the libtorch evaluation of the same ops sits at the same distance
    twin, _ = oracle.torch_layer_forward(x, ids, gw, wu, wg, wd)
    assert float((twin.float() - ref).abs().max()) / rms > TOL


def test_mode3_is_fp32_accumulation_in_index_order(oracle):
    """Pins the oracle's mode 3 on a tiny case: numpy float32 running sums, term by term."""
    import numpy as np
    g = torch.Generator().manual_seed(3)
    n, H, I = 3, 24, 16
    x = torch.randn(n, H, generator=g).to(torch.bfloat16)
    wu, wg = (torch.randn(I, H, generator=g) * 0.3).to(torch.bfloat16), (torch.randn(I, H, generator=g) * 0.3).to(torch.bfloat16)
    wd = (torch.randn(H, I, generator=g) * 0.3).to(torch.bfloat16)
    got = oracle.ffn(x, wu, wg, wd, mode=3)
    rb = lambda v: torch.tensor(float(v)).to(torch.bfloat16).float().item()      # round to bf16, back to python

    def dot32(a, b):
        acc = np.float32(0.0)
        for p, q in zip(a, b):
            acc = np.float32(acc + np.float32(np.float32(p) * np.float32(q)))
        return acc

    xf, uf, gf, df = x.float().numpy(), wu.float().numpy(), wg.float().numpy(), wd.float().numpy()
    h = np.zeros((n, I), dtype=np.float32)
    for r in range(n):
        for c in range(I):
            up, gate = rb(dot32(xf[r], uf[c])), rb(dot32(xf[r], gf[c]))
            sg = rb(np.float32(gate) / (np.float32(1.0) + np.exp(np.float32(-gate), dtype=np.float32)))
            h[r, c] = rb(np.float32(up) * np.float32(sg))
    want = torch.tensor([[rb(dot32(h[r], df[c])) for c in range(H)] for r in range(n)])
    same = float((got.float() == want).float().mean())
    assert same >= 0.97, same       # (expf may differ from numpy's exp in the last place for an element or two)
    assert float((got.float() - want).abs().max()) <= float(ulp_of(want, torch.bfloat16).max())


def test_accumulation_order_moves_outputs_by_more_than_half_an_ulp(oracle):
    """The reference's op sequence on libtorch (the kernels the reference itself runs), on a small
    W8A16 top-2 layer over several seeds: every evaluation must stay inside the wide gate
    (2e-2 * rms + half an ulp of y + one ulp of the largest gate-weighted term); most seeds exceed
    the plain bound; and in at least one the libtorch result leaves 2e-2 * rms + half an ulp --
    an intermediate was stored one ulp away from where the oracle's accumulation order puts it.
    The oracle's own fp32 sequential order (mode 3) is held to the wide gate too."""
    w = wl.Workload("w8_top2", 256, 128, 6, 2, 400, torch.bfloat16, w8=True)
    dt = w.act_dtype
    over_plain = over_half = 0
    for seed in range(12):
        wu, wg, wd = build(oracle, w, seed=seed, std=0.05)
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(w.tokens, w.hidden, generator=g).to(dt)
        ids, gw = oracle.route(0, torch.randn(w.tokens, w.n_experts, generator=g), w.top_k, True, w_dtype=dt)
        ref, _, _, _, _, y3 = oracle.layer_forward(x, ids, gw, wu, wg, wd, mode=2, return_y3=True)
        rms = float(ref.pow(2).mean().sqrt())
        half = 0.5 * ulp_of(ref, dt) * 1.0001
        flip = ulp_of((gw.float().unsqueeze(-1) * y3.float()).abs().amax(dim=1), dt)
        twin, _ = oracle.torch_layer_forward(x, ids, gw, wu, wg, wd)
        seq = oracle.layer_forward(x, ids, gw, wu, wg, wd, mode=3)[0]
        for name, y in (("libtorch", twin), ("mode 3", seq)):
            err = (y.float() - ref).abs()
            assert bool((err <= TOL * rms + half + flip).all()), (seed, name)
            assert float((err > TOL * rms).float().mean()) <= 1e-4, (seed, name)
        err = (twin.float() - ref).abs()
        over_plain += not bool((err <= TOL * rms).all())
        over_half += not bool((err <= TOL * rms + half).all())
        print(f"seed {seed}: libtorch vs y_ref max|err|/rms = {float(err.max()) / rms:.3e}")
    assert over_plain >= 6, over_plain
    assert over_half >= 1, "no seed showed a flipped intermediate at a large term"


def test_a_tie_in_a_hidden_activation_moves_one_ffn_output_by_two_ulps(oracle):
    """One expert's FFN alone (fp8 weights with block scales, 896 -> 512 -> 896, a case the seeded
    fuzz of per-expert calls drew: EKSEED=8, case 23, row 1106, output channel 175).  The gate
    pre-activation of hidden channel 350 is 1.37890641: 1.6e-7 above the midpoint of the bf16
    neighbours 1.375 and 1.3828125.  The oracle's double sum and a sequential fp32 sum store
    1.3828125; an fp32 sum kept as eight interleaved partial sums, as legitimate an evaluation of
    x.matmul(w3.T) (ffn/expert_torch.rs:82), lands on the midpoint and stores 1.375.  silu and the
    product with `up` turn that one ulp into two ulps of h, that hidden channel carries 92 % of
    the output, and the output moves by 2.9e-2 * rms: past 2e-2 * rms plus half an output ulp,
    the one-expert gate of the GPU tests.  Nothing in it is an error; the GPU kernels' MFMA
    order lands on the 1.375 side."""
    import ek_hip
    from test_gpu_block_scaled import make_expert as make_block_expert, ref_weights
    dt, H, I, case, row, col, j = torch.bfloat16, 896, 512, 23, 1106, 175, 350
    g = torch.Generator().manual_seed(8 * 1000 + case + 77)
    draws = [int(torch.randint(lo, hi + 1, (1,), generator=g)) for lo, hi in ((0, 3), (0, 1), (1, 10), (1, 6))]
    assert draws == [2, 0, 7, 4]                      # fp8, bf16, 7 x 128, 4 x 128: the generator stream of the fuzz
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    sizes = [[r(1, 16), r(17, 64), r(65, 200)][r(0, 2)] for _ in range(r(1, 6))] + [[r(200, 900), r(900, 2600)][r(0, 1)]]
    assert sizes == [171, 3, 1898]
    ws = [make_block_expert(ek_hip, H, I, 100 * case + e, "fp8") for e in range(4)]
    xs = [torch.randn(n, H, generator=g).to(dt) for n in sizes]
    es = [r(0, 3) for _ in sizes]
    wu, wg, wd = ref_weights(oracle, ws[es[-1]], dt)
    x = xs[-1][1024:1152]                              # the 128-row work item that holds the row
    ref = oracle.ffn(x, wu, wg, wd, mode=2)
    rms = float(ref.pow(2).mean().sqrt())
    xr = x[row - 1024].float()

    def interleaved8(w_row):                           # eight running fp32 sums over k mod 8, then added in order
        parts = torch.zeros(8, dtype=torch.float32)
        for k in range(0, H, 8):
            parts = parts + w_row[k:k + 8] * xr[k:k + 8]
        tot = torch.zeros((), dtype=torch.float32)
        for p in parts:
            tot = tot + p
        return tot

    seq = torch.zeros((), dtype=torch.float32)
    for k in range(H):
        seq = seq + wg[j].float()[k] * xr[k]
    alt = interleaved8(wg[j].float())
    assert abs(float(seq) - float(alt)) < 1e-6 and float(alt) == 1.37890625
    assert float(seq.to(dt)) == 1.3828125 and float(alt.to(dt)) == 1.375

    def out_with(gate_b):                              # the reference's rounding points from the stored gate value on
        up_b = (wu.double() @ xr.double()).float().to(dt)
        gates = (wg.double() @ xr.double()).float().to(dt)
        gates[j] = gate_b
        silu_b = torch.nn.functional.silu(gates.float()).to(dt)
        h = (up_b.float() * silu_b.float()).to(dt)
        return float(h.double() @ wd[col].double())

    a, b = out_with(1.3828125), out_with(1.375)
    assert abs(a - float(ref[row - 1024, col])) < 1e-6             # the oracle's side of the tie
    stored = float(torch.tensor(b).to(dt))                          # what an implementation on that side writes
    moved = abs(stored - float(ref[row - 1024, col]))
    half_ulp = 0.5 * float(ulp_of(ref[row - 1024, col], dt))
    print(f"tie in gate[{j}]: output {a:.6f} -> {b:.6f}, stored {stored:.6f}: {moved / rms:.3e} x rms, "
          f"{moved / (2 * half_ulp):.2f} output ulps from y_ref")
    assert stored == -0.359375                                      # the value the GPU kernels write
    assert moved > TOL * rms + half_ulp
    assert moved < 1.6 * TOL * rms
