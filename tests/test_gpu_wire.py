"""The worker contract on wire bytes (safetensors in, safetensors out) and the micro-batcher.

Bars: a wire call is the per-expert entry point plus a codec, so its payload must be
bit-identical to ek_layer_expert_forward on the same rows; a batch of calls (one grouped
launch) must be bit-identical to the same calls made one by one.  The per-expert entry
point itself is gated against the oracle in test_gpu_parity.py.  Blobs are produced and
read back with the `safetensors` package, the implementation the reference links.
"""
import pytest
import torch
from safetensors.torch import load as st_load
from safetensors.torch import save as st_save

from ek_hip import workloads as wl

pytestmark = pytest.mark.gpu

H, I, E = 256, 192, 6


def bits(t):
    return t.contiguous().cpu().view(torch.int16)


def make_layer(ek, dt, w8=False, max_tokens=1024, n_loaded=E):
    layer = ek.HipLayer(H, I, E, 1, act_dtype=dt, w_dtype=torch.int8 if w8 else dt, max_tokens=max_tokens)
    w = wl.Workload("wire", H, I, E, 1, 1, dt, w8=w8)
    for e in range(n_loaded):
        layer.set_expert(e, wl.make_expert(w, e, layer=0, device="cpu", std=0.05))
    return layer


def x_rows(n, dt, seed):
    return torch.randn(n, H, generator=torch.Generator().manual_seed(seed)).to(dt)


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w8", [False, True])
def test_worker_forward_equals_expert_forward(ek, dt, w8):
    layer = make_layer(ek, dt, w8)
    for n, e in [(1, 0), (16, 1), (17, 2), (64, 3), (65, 4), (300, 5), (0, 0)]:
        x = x_rows(n, dt, 100 + n)
        resp = layer.worker_forward(f"wire-model/l0-e{e}", st_save({"data": x}))
        got = st_load(resp)["data"]               # a blob the reference's reader accepts
        assert got.dtype == dt and tuple(got.shape) == (n, H)
        want = layer.expert_forward(e, x)
        assert torch.equal(bits(got), bits(want)), (n, e)
        if n:
            assert float(want.float().abs().max()) > 0
    layer.close()


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("w8", [False, True])
def test_batch_equals_individual_calls(ek, dt, w8):
    layer = make_layer(ek, dt, w8)
    # every size class, empty calls, repeated experts, calls in no particular expert order (the batch is
    # small enough that its longer calls are cut for the streaming kernel, as they are alone)
    calls = [(3, 5), (0, 0), (1, 1), (5, 16), (2, 17), (3, 32), (4, 33), (0, 64), (1, 65), (5, 129), (0, 7), (0, 0)]
    ids = [f"m/l3-e{e}" for e, _ in calls]
    xs = [x_rows(n, dt, 200 + i) for i, (_, n) in enumerate(calls)]
    resps = layer.worker_forward_batch(ids, [st_save({"data": x}) for x in xs])
    outs = layer.experts_forward([e for e, _ in calls], xs)
    for (e, n), x, resp, out in zip(calls, xs, resps, outs):
        want = layer.expert_forward(e, x)
        got = st_load(resp)["data"]
        assert tuple(got.shape) == (n, H)
        assert torch.equal(bits(got), bits(want)), (e, n)
        assert torch.equal(bits(out), bits(want)), (e, n)
    # device-resident tensors through the same entry point
    dev = layer.experts_forward([e for e, _ in calls], [x.cuda() for x in xs])
    for out, d in zip(outs, dev):
        assert d.is_cuda and torch.equal(bits(out), bits(d))
    # device rows that do not start on a 16-byte boundary take the copy-by-copy route: same bits
    shifted = []
    for x in xs:
        flat = torch.empty(x.numel() + 1, dtype=dt, device="cuda")
        flat[1:] = x.reshape(-1).cuda()
        shifted.append(flat[1:].view(x.shape))
    assert any(t.data_ptr() % 16 for t in shifted if t.numel())
    for out, d in zip(outs, layer.experts_forward([e for e, _ in calls], shifted)):
        assert torch.equal(bits(out), bits(d))
    assert layer.stats()["expert_forward_calls"] >= 4 * len(calls)
    # a batch with enough rows for the tile kernel: its long calls take the other kernel family than
    # they take alone, so the results agree as two evaluations of the same product do, not bit for bit
    big = [(2, 128), (4, 300), (1, 200), (3, 9)]
    xs = [x_rows(n, dt, 900 + i).cuda() for i, (_, n) in enumerate(big)]
    outs = layer.experts_forward([e for e, _ in big], xs)
    for (e, n), x, out in zip(big, xs, outs):
        want = layer.expert_forward(e, x).float()
        rms = float(want.pow(2).mean().sqrt())
        assert float((out.float() - want).abs().max()) <= 2e-2 * rms, (e, n)
        if n <= 16:
            assert torch.equal(bits(out), bits(layer.expert_forward(e, x)))
    layer.close()


def test_batch_is_one_grouped_launch_per_stage(ek):
    """The point of the micro-batcher: E concurrent decode requests cost two kernel launches,
    not 2*E, so the batch must not be slower than the calls made one by one."""
    import time
    dt = torch.bfloat16
    layer = make_layer(ek, dt)
    xs = [x_rows(4, dt, 300 + e).cuda() for e in range(E)]
    ex = list(range(E))
    for _ in range(3):
        layer.experts_forward(ex, xs)
        [layer.expert_forward(e, x) for e, x in zip(ex, xs)]
    def best_of(fn, reps=5, n=20):          # wall clock of n calls with the device drained, best of reps
        best = float("inf")
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                fn()
            torch.cuda.synchronize()
            best = min(best, time.perf_counter() - t0)
        return best

    t_batch = best_of(lambda: layer.experts_forward(ex, xs))
    t_single = best_of(lambda: [layer.expert_forward(e, x) for e, x in zip(ex, xs)])
    print(f"batch of {E}: {t_batch / 20 * 1e6:.0f} us, one by one: {t_single / 20 * 1e6:.0f} us", flush=True)
    assert t_batch < 1.25 * t_single
    layer.close()


def test_wire_errors(ek):
    from ek_hip import _capi as C
    dt = torch.bfloat16
    layer = make_layer(ek, dt, n_loaded=2)
    ok = st_save({"data": x_rows(4, dt, 1)})

    def status(expert_id, blob):
        with pytest.raises(ek.EKError) as ei:
            layer.worker_forward(expert_id, blob)
        return ei.value.status

    assert status("m/l0-e1x", ok) == C.EK_INVALID_INPUT                     # malformed id
    assert status(f"m/l0-e{E}", ok) == C.EK_EXPERT_NOT_FOUND                # id beyond the layer
    assert status("m/l0-e3", ok) == C.EK_EXPERT_NOT_FOUND                   # not loaded
    assert status("m/l0-e0", ok[:-3]) == C.EK_INVALID_INPUT                 # truncated blob
    assert status("m/l0-e0", st_save({"x": x_rows(4, dt, 1)})) == C.EK_WEIGHT_NOT_FOUND   # no tensor "data"
    assert status("m/l0-e0", st_save({"data": x_rows(4, torch.float16, 1)})) == C.EK_INVALID_INPUT
    assert status("m/l0-e0", st_save({"data": torch.zeros(4, H + 64, dtype=dt)})) == C.EK_INVALID_INPUT
    assert status("m/l0-e0", st_save({"data": torch.zeros(2, 2, H, dtype=dt)})) == C.EK_INVALID_INPUT
    assert status("m/l0-e0", st_save({"data": torch.zeros(2000, H, dtype=dt)})) == C.EK_INVALID_INPUT  # > capacity
    # a failed call leaves the layer usable
    x = x_rows(4, dt, 1)
    assert torch.equal(bits(st_load(layer.worker_forward("m/l0-e1", ok))["data"]), bits(layer.expert_forward(1, x)))
    layer.close()


@pytest.mark.parametrize("kind", ["bf16", "f32", "fp8_block", "int8_block", "int8_channel"])
def test_set_expert_from_blob(ek, kind):
    """ek-db's expert blob (transformer.rs:248-300) loaded by suffix, scales picked up by name."""
    from ek_hip import _capi as C
    dt = torch.bfloat16
    g = torch.Generator().manual_seed(9)
    w8 = kind == "int8_channel"
    names = {"up": "model.layers.3.mlp.experts.7.up_proj.weight", "gate": "model.layers.3.mlp.experts.7.gate_proj.weight",
             "down": "model.layers.3.mlp.experts.7.down_proj.weight"}
    if kind == "f32":
        names = {"up": "experts.7.w1.weight", "gate": "experts.7.w3.weight", "down": "experts.7.w2.weight"}
    shapes = {"up": (I, H), "gate": (I, H), "down": (H, I)}

    def weight(r, c):
        if kind in ("bf16", "f32"):
            return (torch.randn(r, c, generator=g) * 0.05).to(torch.bfloat16 if kind == "bf16" else torch.float32)
        if kind == "fp8_block":
            return (torch.randn(r, c, generator=g) * 40).to(torch.float8_e4m3fn)
        return torch.randint(-127, 128, (r, c), generator=g, dtype=torch.int8)

    def scale(r, c):
        if kind.endswith("_block"):
            return torch.rand((r + 127) // 128, (c + 127) // 128, generator=g) * 2e-3 + 5e-4
        if kind == "int8_channel":
            return torch.rand(r, generator=g) * 2e-3 + 5e-4
        return None

    tensors, kw = {}, {}
    for m, (r, c) in shapes.items():
        tensors[names[m]] = weight(r, c)
        kw[f"{m}_w"] = tensors[names[m]]
        sc = scale(r, c)
        if sc is not None:
            tensors[names[m] + ("_scale_inv" if kind.endswith("_block") else "_scale")] = sc
            kw[f"{m}_scale"] = sc
    a = ek.HipLayer(H, I, 2, 1, act_dtype=dt, w_dtype=torch.int8 if w8 else dt, max_tokens=64)
    a.set_expert(0, ek.ExpertWeight(**kw))                    # descriptors built by the caller
    a.set_expert_safetensors(1, st_save(tensors))             # the same tensors found in the blob
    x = x_rows(40, dt, 5)
    y0, y1 = a.expert_forward(0, x), a.expert_forward(1, x)
    assert float(y0.float().abs().max()) > 0
    assert torch.equal(bits(y0), bits(y1))
    # a blob that lacks one matrix: ExpertWeightNotFound("w2/down_w") (ffn/meta.rs:60-61)
    del tensors[names["down"]]
    with pytest.raises(ek.EKError) as ei:
        a.set_expert_safetensors(1, st_save(tensors))
    assert ei.value.status == C.EK_WEIGHT_NOT_FOUND and "w2/down_w" in ei.value.message
    assert a.has_expert(1)                                     # the failed load did not evict the old weights
    assert torch.equal(bits(a.expert_forward(1, x)), bits(y1))
    a.close()
