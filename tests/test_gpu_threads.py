"""Thread safety of the C ABI.  The reference's worker runs forwards from a 48-thread tokio pool
(ek-cli/src/main.rs:92), takes its gate with read() so that they overlap (worker/server.rs:64) and
loads experts concurrently with them (worker/state.rs:186).  Here: many host threads call the same
layer handle (ctypes drops the GIL during a call), each checks its own results bit-for-bit against
what a single thread computed, while another thread keeps replacing and removing an expert that
none of them uses."""
import threading

import pytest
import torch
from safetensors.torch import load as st_load
from safetensors.torch import save as st_save

from ek_hip import workloads as wl

pytestmark = pytest.mark.gpu


def test_concurrent_calls_on_one_layer(ek, cuda):
    H, I, E, K = 256, 192, 8, 2
    dt = torch.bfloat16
    layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=256)
    work = wl.Workload("threads", H, I, E, K, 1, dt)
    experts = [wl.make_expert(work, e, std=0.05) for e in range(E)]
    for e in range(E - 1):                      # expert E-1 belongs to the loader thread
        layer.set_expert(e, experts[e])
    n_threads, iters = 12, 25

    def inputs(t):
        g = torch.Generator().manual_seed(100 + t)
        n = 5 + 13 * t
        x = torch.randn(n, H, generator=g).to(dt)
        ids = torch.stack([torch.randperm(E - 1, generator=g)[:K] for _ in range(n)]).to(torch.int32)
        w = torch.rand(n, K, generator=g).to(dt)
        return x, ids, w

    want = []
    for t in range(n_threads):                  # single-threaded answers first
        x, ids, w = inputs(t)
        want.append((layer.forward(x, ids, w), layer.expert_forward(t % (E - 1), x),
                     layer.worker_forward(f"m/l0-e{t % (E - 1)}", st_save({"data": x}))))
    errors, stop = [], threading.Event()

    def worker(t):
        try:
            x, ids, w = inputs(t)
            xd, idd, wd = (x.to(cuda), ids.to(cuda), w.to(cuda)) if t % 2 else (x, ids, w)
            for _ in range(iters):
                y = layer.forward(xd, idd, wd)
                if not torch.equal(y.cpu().view(torch.int16), want[t][0].view(torch.int16)):
                    raise AssertionError(f"thread {t}: forward differs")
                ye = layer.expert_forward(t % (E - 1), xd)
                if not torch.equal(ye.cpu().view(torch.int16), want[t][1].view(torch.int16)):
                    raise AssertionError(f"thread {t}: expert_forward differs")
                blob = layer.worker_forward(f"m/l0-e{t % (E - 1)}", st_save({"data": x}))
                if blob != want[t][2] or st_load(blob)["data"].shape != x.shape:
                    raise AssertionError(f"thread {t}: wire forward differs")
        except Exception as ex:                 # noqa: BLE001 - reported by the main thread
            errors.append(ex)

    def loader():
        try:
            while not stop.is_set():
                layer.set_expert(E - 1, experts[E - 1])
                assert layer.has_expert(E - 1)
                layer.set_expert(E - 1, experts[0])          # replace in place
                layer.remove_expert(E - 1)
        except Exception as ex:                 # noqa: BLE001
            errors.append(ex)

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(n_threads)]
    lt = threading.Thread(target=loader)
    lt.start()
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    stop.set()
    lt.join(timeout=30)
    assert not any(th.is_alive() for th in threads) and not lt.is_alive()
    assert not errors, errors[:3]
    st = layer.stats()
    assert st["forward_calls"] >= n_threads * (iters + 1)
    assert int(layer.activation().sum()) > 0
    layer.close()


def test_concurrent_layers_do_not_interfere(ek, cuda):
    """One handle per thread (the per-expert HipFFN shape): no shared workspace at all."""
    H, I = 128, 128
    dt = torch.float16
    n_threads, iters = 8, 20
    work = wl.Workload("threads2", H, I, n_threads, 1, 1, dt)
    ffns = [ek.HipFFN.construct(ek.EKInstance(H, I), wl.make_expert(work, t, std=0.08), act_dtype=dt, max_rows=128)
            for t in range(n_threads)]
    xs = [torch.randn(20 + 9 * t, H, generator=torch.Generator().manual_seed(t)).to(dt).to(cuda) for t in range(n_threads)]
    want = [f.forward(x).cpu() for f, x in zip(ffns, xs)]
    errors = []

    def worker(t):
        try:
            for _ in range(iters):
                if not torch.equal(ffns[t].forward(xs[t]).cpu().view(torch.int16), want[t].view(torch.int16)):
                    raise AssertionError(f"thread {t}")
        except Exception as ex:                 # noqa: BLE001
            errors.append(ex)

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(n_threads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not any(th.is_alive() for th in threads)
    assert not errors, errors[:3]
    for f in ffns:
        f.close()


def test_enqueue_only_calls_on_two_streams(ek, cuda):
    """Calls that only enqueue (device pointers and a caller's stream) return while their kernels
    still use the layer's one workspace.  Two host threads, each with a stream of its own, keep
    enqueuing calls with different inputs on the same layer while a third makes blocking calls on
    host tensors (the library's own stream): every result must be bit-equal to the answer the
    same call gives alone.  Without an ordering between the streams the routing tables and
    intermediates of one call would be overwritten under the kernels of another."""
    H, I, E, K = 1024, 512, 16, 4
    dt = torch.bfloat16
    layer = ek.HipLayer(H, I, E, K, act_dtype=dt, max_tokens=700)
    work = wl.Workload("streams", H, I, E, K, 1, dt)
    for e in range(E):
        layer.set_expert(e, wl.make_expert(work, e, std=0.05))
    iters = 12

    def inputs(t):
        g = torch.Generator().manual_seed(900 + t)
        n = [650, 37, 300][t]                      # tiles and streaming items; a decode-sized call; in between
        x = torch.randn(n, H, generator=g).to(dt)
        ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(n)]).to(torch.int32)
        w = torch.rand(n, K, generator=g).to(dt)
        return x, ids, w

    ins = [inputs(t) for t in range(3)]
    want = [layer.forward(*i) for i in ins]                      # serial answers (blocking, host tensors)
    errors = []

    def enqueuer(t):
        try:
            stream = torch.cuda.Stream()
            x, ids, w = (v.to(cuda) for v in ins[t])
            outs = [torch.zeros_like(x) for _ in range(iters)]
            torch.cuda.synchronize()
            for i in range(iters):
                layer.forward(x, ids, w, stream=stream, out=outs[i])
                if i % 4 == 3:
                    layer.expert_forward(t, x[:20].contiguous(), stream=stream)   # another user of the workspace
            stream.synchronize()
            for i in range(iters):
                if not torch.equal(outs[i].cpu().view(torch.int16), want[t].view(torch.int16)):
                    raise AssertionError(f"stream {t}, call {i}: differs from the serial answer")
        except Exception as ex:                 # noqa: BLE001 - reported by the main thread
            errors.append(ex)

    def blocker():
        try:
            for i in range(iters):
                y = layer.forward(*ins[2])
                if not torch.equal(y.view(torch.int16), want[2].view(torch.int16)):
                    raise AssertionError(f"blocking host call {i}: differs from the serial answer")
        except Exception as ex:                 # noqa: BLE001
            errors.append(ex)

    threads = [threading.Thread(target=enqueuer, args=(0,)), threading.Thread(target=enqueuer, args=(1,)),
               threading.Thread(target=blocker)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not any(th.is_alive() for th in threads)
    assert not errors, errors[:3]
    layer.close()
