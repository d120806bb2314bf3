"""The tile kernel's register-streamed form for 17..64-row segments (run_mid in csrc/ek_ffn_tile.hip).

A launch whose tile items fill the chip (items x channel blocks >= workgroups launched) serves its
32- and 64-row items with weights loaded straight into registers, when the contraction is a
multiple of 256 elements (128 with 16-bit weights) and at least twice that long; every other launch
brings them in through LDS.  Both forms add the same products in the same order, so they must give
the same bits.  Here 256 experts get 17..64 rows each (top-1 routing, gate weight 1: the combine
multiplies by exactly 1), which fills the chip in both stages; the rows of a few experts routed
alone are a launch of a dozen items, which takes the LDS form.  The oracle holds the gate on the
same rows (arithmetic of ek-computation/src/ffn/expert_torch.rs:81-84).
"""
import pytest
import torch

from ek_hip import workloads as wl
from test_gpu_block_scaled import KINDS, make_expert as make_block_expert, ref_weights
from test_gpu_parity import check_vs_rounded, ffn_gate, oracle_weights

pytestmark = pytest.mark.gpu

E = 256
ROWS = [17, 24, 31, 32, 33, 40, 48, 57, 63, 64]     # both item classes, full and ragged
DISTINCT = 8                                         # weight sets; expert e holds set e % 8
ALONE = list(range(10)) + [137, 254, 255]            # every row count once; first and last XCD share

CASES = [
    # kind, activation type, hidden, inter
    ("i8", torch.bfloat16, 512, 512),       # both contractions exactly two windows of four steps
    ("i8", torch.float16, 1024, 768),
    ("i8", torch.bfloat16, 512, 640),       # stage 2: 10 steps, not a multiple of four -> LDS form there
    ("fp8", torch.bfloat16, 512, 512),
    ("fp8", torch.float16, 768, 512),
    ("int8", torch.bfloat16, 512, 768),     # int8 with 128 x 128 block scales
    ("w16", torch.float16, 256, 512),       # 16-bit weights: windows of two steps
    ("w16", torch.bfloat16, 512, 384),
]


def build(ek, oracle, kind, dt, H, I, max_rows=64):
    if kind in KINDS:
        layer = ek.HipLayer(H, I, E, 1, act_dtype=dt, max_tokens=E * max_rows, **KINDS[kind])
        ws = [make_block_expert(ek, H, I, 500 + i, kind) for i in range(DISTINCT)]
        ref = [ref_weights(oracle, ew, dt) for ew in ws]
    else:
        w = wl.Workload("t", H, I, E, 1, 0, dt, w8=kind == "i8")
        layer = ek.HipLayer(H, I, E, 1, act_dtype=dt, w_dtype=torch.int8 if w.w8 else dt, max_tokens=E * max_rows)
        ws = [wl.make_expert(w, i) for i in range(DISTINCT)]
        if kind == "w16":    # larger than the benchmark's weights: silu off its linear part
            ws = [ek.ExpertWeight(ew.up_w * 4, ew.gate_w * 4, ew.down_w * 4) for ew in ws]
        cols = oracle_weights(oracle, dict(enumerate(ws)), DISTINCT, dt)
        ref = [tuple(c[i] for c in cols) for i in range(DISTINCT)]
    for e in range(E):
        layer.set_expert(e, ws[e % DISTINCT])
    return layer, ref


@pytest.mark.parametrize("kind,dt,H,I", CASES)
def test_short_tiles_of_a_full_launch(ek, oracle, cuda, kind, dt, H, I):
    print(f"short tiles kind={kind} dt={dt} H={H} I={I}", flush=True)
    layer, ref = build(ek, oracle, kind, dt, H, I)
    g = torch.Generator().manual_seed(H + I)
    owner = torch.cat([torch.full((ROWS[e % len(ROWS)],), e, dtype=torch.int32) for e in range(E)])
    owner = owner[torch.randperm(owner.numel(), generator=g)]
    T = owner.numel()
    x = torch.randn(T, H, generator=g).to(dt)
    xd, ids = x.to(cuda), owner.view(T, 1).to(cuda)
    ones = torch.ones(T, 1, dtype=dt, device=cuda)
    y = layer.forward(xd, ids, ones)
    assert torch.equal(layer.forward(xd, ids, ones).view(torch.int16), y.view(torch.int16))

    # the same rows in a launch of a dozen items
    pick = torch.isin(owner, torch.tensor(ALONE, dtype=torch.int32)).nonzero().flatten().to(cuda)
    alone = layer.forward(xd[pick], ids[pick], ones[pick])
    assert torch.equal(alone.view(torch.int16), y[pick].view(torch.int16))

    # and against the oracle, expert by expert (rows in token order, as the pack step keeps them)
    for e in ALONE:
        rows = (owner == e).nonzero().flatten()
        assert rows.numel() == ROWS[e % len(ROWS)]
        want = oracle.ffn(x[rows], *ref[e % DISTINCT], mode=2)
        got = y[rows.to(cuda)]
        ffn_gate(got, want, f"short tiles {kind} dt={dt} H={H} I={I} e={e}")
        assert check_vs_rounded(got, want) > 0.9
    layer.close()


# ---- launches that hold 128-row items as well ----------------------------------------------------
# The register-streamed form follows the 128-row class in the same workgroups, so what the long
# tiles leave in LDS (their last stage, their epilogue scratch) and what the short tiles bring in
# (window buffers, block-scale rows) must not meet.  Channel counts that are not a multiple of a
# workgroup's span (256 hidden channels in stage 1, 512 output channels in stage 2) leave waves with
# no channels of their own: those skip the epilogue and reach the next class first.
MIXED_ROWS = [20, 40, 64, 130, 200, 300, 17, 129, 33, 192]
MIXED_ALONE = list(range(10)) + [131, 255]
MIXED_CASES = [
    # kind, activation type, hidden, inter
    ("i8", torch.bfloat16, 768, 640),       # stage 1: waves past the last channel, register-streamed
    ("i8", torch.float16, 768, 512),        # stage 2: waves past the last channel, register-streamed
    ("fp8", torch.bfloat16, 768, 640),
    ("fp8", torch.float16, 768, 512),
    ("int8", torch.bfloat16, 768, 640),
    ("int8", torch.bfloat16, 768, 512),
    ("fp8", torch.bfloat16, 1536, 1408),    # DeepSeek-V2-Lite's intermediate size
    ("w16", torch.float16, 768, 384),
    ("w16", torch.bfloat16, 768, 640),
]


@pytest.mark.parametrize("kind,dt,H,I", MIXED_CASES)
def test_long_and_short_tiles_in_one_full_launch(ek, oracle, cuda, kind, dt, H, I):
    print(f"mixed tiles kind={kind} dt={dt} H={H} I={I}", flush=True)
    layer, ref = build(ek, oracle, kind, dt, H, I, max_rows=max(MIXED_ROWS))
    g = torch.Generator().manual_seed(3 * H + I)
    owner = torch.cat([torch.full((MIXED_ROWS[e % len(MIXED_ROWS)],), e, dtype=torch.int32) for e in range(E)])
    owner = owner[torch.randperm(owner.numel(), generator=g)]
    T = owner.numel()
    x = torch.randn(T, H, generator=g).to(dt)
    xd, ids = x.to(cuda), owner.view(T, 1).to(cuda)
    ones = torch.ones(T, 1, dtype=dt, device=cuda)
    y = layer.forward(xd, ids, ones)
    for _ in range(3):     # a race shows as a run that differs
        assert torch.equal(layer.forward(xd, ids, ones).view(torch.int16), y.view(torch.int16))

    # the same rows in a launch of a dozen experts: its short items come in through LDS
    pick = torch.isin(owner, torch.tensor(MIXED_ALONE, dtype=torch.int32)).nonzero().flatten().to(cuda)
    alone = layer.forward(xd[pick], ids[pick], ones[pick])
    assert torch.equal(alone.view(torch.int16), y[pick].view(torch.int16))
    # every expert holds one of eight weight sets: experts e and e + 8k with the same row count see
    # different neighbours in the launch and must agree with a launch of their own rows all the same
    for e in (8, 57, 122, 203, 250):
        rows = (owner == e).nonzero().flatten().to(cuda)
        own = layer.forward(xd[rows], ids[rows], ones[rows])
        assert torch.equal(own.view(torch.int16), y[rows].view(torch.int16)), f"expert {e}"

    for e in MIXED_ALONE[: 6 if H * I > 1 << 20 else len(MIXED_ALONE)]:
        rows = (owner == e).nonzero().flatten()
        assert rows.numel() == MIXED_ROWS[e % len(MIXED_ROWS)]
        want = oracle.ffn(x[rows], *ref[e % DISTINCT], mode=2)
        got = y[rows.to(cuda)]
        ffn_gate(got, want, f"mixed tiles {kind} dt={dt} H={H} I={I} e={e}")
        assert check_vs_rounded(got, want) > 0.9
    layer.close()
