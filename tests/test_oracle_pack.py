"""Pins eko_pack / gather / scatter: brute force on every case, plus the
invariants a stable group-by must satisfy (a dropped pair, an unstable order or
an off-by-one offset fails at least one)."""
import pytest
import torch

from ek_hip import workloads as wl


def check_invariants(ids, E, counts, offsets, perm, inv):
    flat = ids.reshape(-1).long()
    P = flat.numel()
    assert int(offsets[0]) == 0 and int(offsets[E]) == P
    assert torch.equal(counts.long(), torch.bincount(flat, minlength=E))
    assert torch.equal(offsets[1:].long() - offsets[:-1].long(), counts.long())
    assert torch.equal(torch.sort(perm.long()).values, torch.arange(P))
    if P:
        assert torch.equal(inv.long()[perm.long()], torch.arange(P))
    for e in range(E):
        seg = perm[int(offsets[e]):int(offsets[e + 1])].long()
        assert bool((flat[seg] == e).all())
        assert bool((seg[1:] > seg[:-1]).all()), "arrival order (t,k ascending) must be kept"


CASES = [(0, 1, 4), (1, 1, 1), (1, 2, 2), (5, 2, 3), (64, 2, 16), (33, 8, 128), (257, 8, 256), (1000, 4, 7)]


@pytest.mark.parametrize("T,K,E", CASES)
def test_pack_vs_brute_force(oracle, T, K, E):
    g = torch.Generator().manual_seed(T * 131 + K * 7 + E)
    ids = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32)
    got = oracle.pack(ids, E)
    ref = oracle.brute_pack(ids, E)
    for a, b in zip(got, ref):
        assert torch.equal(a, b)
    check_invariants(ids, E, *got)


def test_pack_degenerate(oracle):
    ids = torch.full((50, 4), 3, dtype=torch.int32)          # everything to one expert
    c, o, p, i = oracle.pack(ids, 8)
    assert torch.equal(p, torch.arange(200, dtype=torch.int32)) and int(c[3]) == 200
    with pytest.raises(ValueError):
        oracle.pack(torch.tensor([[0, 9]], dtype=torch.int32), 8)
    with pytest.raises(ValueError):
        oracle.pack(torch.tensor([[-1, 0]], dtype=torch.int32), 8)


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c5"])
def test_pack_on_benchmark_routing(oracle, name):
    w = wl.resolve(wl.CONFIGS[name])
    ids, _ = wl.make_routing(w)
    got = oracle.pack(ids, w.n_experts)
    check_invariants(ids, w.n_experts, *got)
    # top-k never repeats an expert within a token
    assert all(len(set(r)) == w.top_k for r in ids[:64].tolist())


def test_gather_scatter(oracle):
    g = torch.Generator().manual_seed(3)
    T, K, E, H = 37, 3, 5, 16
    ids = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    _, _, perm, inv = oracle.pack(ids, E)
    xp = oracle.gather(x, perm, K)
    assert torch.equal(xp.view(torch.int16), x[(perm // K).long()].view(torch.int16))
    y3 = oracle.scatter(xp, perm, T, K)                       # scatter o gather = broadcast of x over K
    assert torch.equal(y3.view(torch.int16), x.unsqueeze(1).expand(T, K, H).contiguous().view(torch.int16))
    assert torch.equal(y3.reshape(T * K, H)[perm.long()].view(torch.int16), xp.view(torch.int16))
