"""Counters behind the reference's worker metrics (metrics.rs:46-62): per-expert activation
counts must equal, exactly, the rows each expert was given (bincount of the routed ids for the
fused calls, n for per-expert calls); the forward histogram must hold one observation per
blocking compute call, cumulative over the reference's buckets."""
import pytest
import torch
from safetensors.torch import save as st_save

from ek_hip import workloads as wl

pytestmark = pytest.mark.gpu


def test_activation_counts_and_forward_histogram(ek, cuda):
    H, I, E, K, T = 256, 192, 12, 3, 150
    dt = torch.bfloat16
    layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=256)
    work = wl.Workload("obs", H, I, E, K, T, dt)
    for e in range(E):
        layer.set_expert(e, wl.make_expert(work, e, std=0.05))
    assert layer.activation().tolist() == [0] * E
    g = torch.Generator().manual_seed(1)
    x = torch.randn(T, H, generator=g).to(dt)
    lg = torch.randn(T, E, generator=g)
    want = torch.zeros(E, dtype=torch.int64)
    calls = 0

    ids, w = layer.route(lg.to(cuda), ek.RouterConfig(kind=0))
    assert layer.activation().tolist() == [0] * E           # routing alone gives no expert any rows
    layer.pack(ids)
    assert layer.activation().tolist() == [0] * E
    for _ in range(3):                                       # fused call, device tensors
        layer.forward(x.to(cuda), ids, w)
        want += torch.bincount(ids.cpu().flatten().long(), minlength=E)
        calls += 1
    layer.forward(x[:7], ids[:7].cpu(), w[:7].cpu())         # fused call, host tensors
    want += torch.bincount(ids[:7].cpu().flatten().long(), minlength=E)
    calls += 1
    layer.forward_logits(x.to(cuda), lg.to(cuda), ek.RouterConfig(kind=0))
    want += torch.bincount(ids.cpu().flatten().long(), minlength=E)
    calls += 1
    assert layer.activation().tolist() == want.tolist()

    layer.expert_forward(4, x[:9])                           # per-expert contract: += sequences.len()
    want[4] += 9
    calls += 1
    layer.experts_forward([1, 1, 7], [x[:2], x[:5], x[:130]])
    want[1] += 7
    want[7] += 130
    calls += 3
    layer.worker_forward("m/l0-e11", st_save({"data": x[:20]}))
    want[11] += 20
    calls += 1
    assert layer.activation().tolist() == want.tolist()

    s = torch.cuda.Stream()                                  # enqueue-only call: counted, not timed
    with torch.cuda.stream(s):
        layer.forward(x.to(cuda), ids, w, stream=s)
    s.synchronize()
    want += torch.bincount(ids.cpu().flatten().long(), minlength=E)
    assert layer.activation().tolist() == want.tolist()

    h = layer.forward_histogram()
    assert h["le"] == [4000.0 * i for i in range(10)]
    assert h["count"] == calls and h["cumulative"][10] == calls
    assert all(a <= b for a, b in zip(h["cumulative"], h["cumulative"][1:]))
    assert h["cumulative"][0] == 0 and h["sum"] > 0          # nothing takes 0 us
    assert h["cumulative"][9] >= calls - 1                   # these calls take far less than 36 ms
    layer.close()


def test_chain_counts_every_layer(ek, cuda):
    H, I, E, K, T, L = 128, 128, 8, 2, 40, 3
    dt = torch.float16
    work = wl.Workload("obs-chain", H, I, E, K, T, dt)
    layers = []
    for l in range(L):
        layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=64)
        for e in range(E):
            layer.set_expert(e, wl.make_expert(work, e, layer=l, std=0.08))
        layers.append(layer)
    chain = ek.HipChain(layers)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(T, H, generator=g).to(dt).to(cuda)
    ids = torch.randint(0, E, (L, T, K), generator=g, dtype=torch.int32)
    # top-k ids of one token are distinct in the reference; keep that property
    ids[:, :, 1] = (ids[:, :, 0] + 1 + ids[:, :, 1] % (E - 1)) % E
    w = torch.rand(L, T, K, generator=g).to(dt)
    reps = 4
    for _ in range(reps):
        chain.forward(x, ids.to(cuda), w.to(cuda), use_graph=True)     # replays of one captured graph
    for l in range(L):
        want = reps * torch.bincount(ids[l].flatten().long(), minlength=E)
        assert layers[l].activation().tolist() == want.tolist()
    chain.close()
    for layer in layers:
        layer.close()


def test_phase_timing_every_call_and_sampled(ek, cuda):
    """ek_layer_profile(1) records the four phases of every fused call, ek_layer_profile(n) of every
    n-th call beginning with the first (the PerfTimer checkpoints of the reference stand behind it:
    ek-base/src/utils.rs:4-45); turning it off or on again clears what was accumulated; results
    do not depend on it."""
    H, I, E, K, T = 256, 128, 8, 2, 64
    dt = torch.bfloat16
    layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=T)
    work = wl.Workload("phases", H, I, E, K, T, dt)
    for e in range(E):
        layer.set_expert(e, wl.make_expert(work, e, std=0.05))
    x = wl.make_x(work).to(cuda)
    ids, gw = wl.make_routing(work)
    ids, gw = ids.to(cuda), gw.to(cuda)
    y0 = layer.forward(x, ids, gw)
    assert layer.stats()["profiled_calls"] == 0
    stream = torch.cuda.Stream()
    for every, calls, want in ((1, 6, 6), (4, 10, 3), (3, 3, 1), (True, 2, 2)):
        layer.profile(every)
        for i in range(calls):
            y = layer.forward(x, ids, gw, stream=stream if i % 2 else None)
            stream.synchronize()
            assert torch.equal(y.view(torch.int16), y0.view(torch.int16))
        st = layer.stats()
        assert st["profiled_calls"] == want, (every, st["profiled_calls"])
        assert all(v > 0 for v in st["kernel_us"]) and sum(st["kernel_us"]) < 1e6 * want
        layer.profile(False)
        assert layer.stats()["profiled_calls"] == 0 and sum(layer.stats()["kernel_us"]) == 0
    layer.close()


def test_measured_peaks_are_ordered_and_below_the_published_ones(ek, cuda):
    """ek_measure_peaks: the device's own ceilings.  Each is below the published peak, the MFMA loop
    slows down when its operands toggle and again when the int8 conversion runs beside it."""
    import ctypes
    from ek_hip import _capi as C
    pk = C.ek_peaks()
    C.check(C.load().ek_measure_peaks(0, ctypes.byref(pk)))
    assert 2000.0 < pk.copy_gbps < 8000.0
    assert 4000.0 < pk.read_nt_gbps < 8000.0
    assert 1000.0 < pk.mfma_bf16_dequant_tflops < pk.mfma_bf16_random_tflops <= pk.mfma_bf16_tflops * 1.02
    assert pk.mfma_bf16_tflops < 2500.0 * 1.02
    assert C.load().ek_measure_peaks(0, None) == C.EK_INVALID_INPUT
