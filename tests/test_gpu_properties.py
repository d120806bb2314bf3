"""Properties of the routed-expert path that hold at any size, checked at the benchmark's full sizes.

In the reference a token's result depends on that token's row, its expert ids and its gate weights
only: pairs are grouped per expert (ek-computation/src/controller/executor.rs:283-299), an expert
works row by row (ffn/expert_torch.rs:81-84) and the sum runs over the token's own K rows
(expertkit_torch/models/qwen3_moe.py:102-104).  Here a row's neighbours in its expert's segment
decide which tile or streaming item it lands in and at which position, so these properties hold
bit for bit only if no kernel lets one row's data reach another's result:

  * reordering the tokens of a call reorders its output rows and changes nothing else;
  * a call split in two gives the two halves of the whole call's output;
  * renaming the experts (ids and weights permuted alike) changes nothing.

Comparisons are exact (bit patterns) for every token whose pairs are served by the same kernel
family in both calls (the weight-streaming kernel takes the last <= 16 rows of a segment, the MFMA
tile kernel the rest; the two add in different orders), on the 8192-token DeepSeek-V3 W8A16
prefill call and on the Qwen3 fp16 decode call with skewed routing, where segments of every class
occur.
"""
import pytest
import torch

from ek_hip import workloads as wl
from test_gpu_parity import load_layer

pytestmark = pytest.mark.gpu


def bits(t):
    return t.contiguous().view(torch.int16)


def streamed_pairs(ids: torch.Tensor, E: int) -> torch.Tensor:
    """[T, K] bool: the pair is served by the weight-streaming kernel (it sits in the last
    count % 128 rows of its expert's segment and these are at most 16), the others by the MFMA tile
    kernel.  Pairs are grouped stably (executor.rs:283-299): a pair's rank in its segment is the
    number of earlier pairs of the same expert."""
    flat = ids.flatten().long().cpu()
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=E)
    offsets = torch.cat([torch.zeros(1, dtype=torch.long), counts.cumsum(0)])
    rank = torch.empty_like(flat)
    rank[order] = torch.arange(flat.numel()) - offsets[flat[order]]
    rem = counts % 128
    tail = torch.where((rem > 0) & (rem <= 16), rem, torch.zeros_like(rem))
    return (rank >= (counts - tail)[flat]).view(ids.shape)


def hold_rows(y_a, y_b, fam_a, fam_b, what):
    """Rows whose K pairs are served by the same kernel family in both calls must agree bit for bit;
    the others differ in accumulation order only: nine in ten of their elements equal, the rest close."""
    same_family = (fam_a == fam_b).all(dim=1).to(y_a.device)
    assert float(same_family.float().mean()) > 0.5, "the comparison would be vacuous"
    assert torch.equal(bits(y_a[same_family]), bits(y_b[same_family])), f"{what} changed the result of a token whose pairs stayed in their kernels"
    moved = ~same_family
    if bool(moved.any()):
        a, b = y_a[moved].float(), y_b[moved].float()
        eq = float((bits(y_a[moved]) == bits(y_b[moved])).float().mean())
        rms = float(b.pow(2).mean().sqrt())
        print(f"{what}: {int(moved.sum())} tokens had a pair move between the kernels: {eq:.4f} of their elements identical, "
              f"max difference {float((a - b).abs().max()) / rms:.2e} x rms", flush=True)
        assert eq > 0.9 and float((a - b).abs().max()) <= 4e-2 * rms


@pytest.mark.parametrize("name", ["c4", "c2"])
def test_token_order_and_call_split_do_not_matter(ek, cuda, name):
    w = wl.resolve(wl.CONFIGS[name])
    E = w.n_experts
    print(f"{name}: building {E} experts on the GPU", flush=True)
    layer, _ = load_layer(ek, w, device="cuda")
    x = wl.make_x(w).to(cuda)
    ids, gw = wl.make_routing(w)
    fam = streamed_pairs(ids, E)
    ids, gw = ids.to(cuda), gw.to(cuda)
    y = layer.forward(x, ids, gw)
    assert float(y.float().abs().max()) > 0

    g = torch.Generator().manual_seed(11)
    perm = torch.randperm(w.tokens, generator=g)
    pd = perm.to(cuda)
    y_perm = layer.forward(x[pd].contiguous(), ids[pd].contiguous(), gw[pd].contiguous())
    hold_rows(y_perm, y[pd], streamed_pairs(ids.cpu()[perm], E), fam[perm], f"{name}: reordering the tokens")

    # the call split at an odd place: every expert's segment is cut differently in the two parts
    cut = w.tokens * 5 // 13
    y_a = layer.forward(x[:cut].contiguous(), ids[:cut].contiguous(), gw[:cut].contiguous())
    y_b = layer.forward(x[cut:].contiguous(), ids[cut:].contiguous(), gw[cut:].contiguous())
    fam_split = torch.cat([streamed_pairs(ids[:cut].cpu(), E), streamed_pairs(ids[cut:].cpu(), E)])
    hold_rows(torch.cat([y_a, y_b]), y, fam_split, fam, f"{name}: splitting the call")
    layer.close()


def test_expert_names_do_not_matter(ek, cuda):
    """Experts renamed by a permutation p (expert e's weights loaded as expert p[e], ids mapped through
    p): same tokens, same pairs, other segment order in the packed buffers and other work lists."""
    w = wl.Workload("rename", 1024, 512, 32, 4, 1500, torch.bfloat16, w8=True, zipf_s=1.0)
    layer, ws = load_layer(ek, w, device="cuda")
    x = wl.make_x(w).to(cuda)
    ids, gw = wl.make_routing(w)
    y = layer.forward(x, ids.to(cuda), gw.to(cuda))
    p = torch.randperm(w.n_experts, generator=torch.Generator().manual_seed(5))
    renamed = ek.HipLayer(w.hidden, w.inter, w.n_experts, w.top_k, act_dtype=w.act_dtype, w_dtype=torch.int8,
                          max_tokens=w.tokens)
    for e in range(w.n_experts):
        renamed.set_expert(int(p[e]), ws[e])
    ids_r = p[ids.long()].to(torch.int32)
    y_r = renamed.forward(x, ids_r.to(cuda), gw.to(cuda))
    assert torch.equal(bits(y_r), bits(y))       # (every segment keeps its length and its rows' order: same kernels, other places)
    layer.close(); renamed.close()
