"""The worker-side collector: concurrent per-expert requests answered by grouped launches.

Bar: what a caller gets through the batcher is bit-identical to ek_worker_forward on the same
request (requests of at most 16 rows take the same kernel form alone or batched), whatever
the other threads are doing; a request that fails does not fail its neighbours.
"""
import threading

import pytest
import torch
from safetensors.torch import load as st_load
from safetensors.torch import save as st_save

from test_gpu_wire import E, H, bits, make_layer, x_rows

pytestmark = pytest.mark.gpu


def run_threads(n, fn):
    errs, gate = [], threading.Barrier(n)

    def body(i):
        try:
            gate.wait()
            fn(i)
        except BaseException as ex:          # noqa: BLE001 - reported to the test below
            errs.append((i, ex))

    ts = [threading.Thread(target=body, args=(i,)) for i in range(n)]
    for t in ts:
        t.start()
    for t in ts:
        t.join(120)
    assert not any(t.is_alive() for t in ts), "a caller never returned"
    return errs


@pytest.mark.parametrize("dt,w8", [(torch.bfloat16, False), (torch.float16, True)])
def test_concurrent_callers_share_launches(ek, dt, w8):
    layer = make_layer(ek, dt, w8)
    n_threads, rounds = 24, 6
    reqs = {(i, r): (f"m/l0-e{(i * 7 + r) % E}", st_save({"data": x_rows(1 + (i + r) % 16, dt, 1000 + 31 * i + r)}))
            for i in range(n_threads) for r in range(rounds)}
    want = {k: layer.worker_forward(eid, req) for k, (eid, req) in reqs.items()}
    batcher = ek.HipBatcher(layer, max_wait_us=2000, max_calls=64)
    got = {}

    def caller(i):
        for r in range(rounds):
            got[(i, r)] = batcher.forward(*reqs[(i, r)])

    assert run_threads(n_threads, caller) == []
    for k in reqs:
        assert got[k] == want[k], k                       # whole response blob, header included
    st = batcher.stats()
    assert st["calls"] == n_threads * rounds
    assert st["batches"] < st["calls"] and st["largest_batch"] > 1, st
    print("batcher:", st, flush=True)
    batcher.close()
    layer.close()


def test_no_window_and_single_slot(ek):
    dt = torch.bfloat16
    layer = make_layer(ek, dt)
    req = st_save({"data": x_rows(5, dt, 1)})
    want = layer.worker_forward("m/l0-e2", req)
    for wait, cap in ((0, 64), (500, 1)):
        b = ek.HipBatcher(layer, max_wait_us=wait, max_calls=cap)
        out = []
        assert run_threads(8, lambda i: out.append(b.forward("m/l0-e2", req))) == []
        assert len(out) == 8 and all(o == want for o in out)
        st = b.stats()
        assert st["calls"] == 8 and (cap != 1 or (st["batches"] == 8 and st["largest_batch"] == 1))
        assert b.forward("m/l0-e2", req) == want          # a lone caller leads a batch of one
        b.close()
    layer.close()


def test_a_bad_request_fails_alone(ek):
    dt = torch.bfloat16
    layer = make_layer(ek, dt, n_loaded=E - 1)            # expert E-1 is not loaded
    good = st_save({"data": x_rows(3, dt, 2)})
    want = layer.worker_forward("m/l0-e1", good)
    bad = {1: ("m/l0-e1", good[:40]),                                        # truncated blob
           4: (f"m/l0-e{E - 1}", good),                                      # expert not loaded
           6: ("m/l0-e1", st_save({"data": x_rows(3, dt, 2).float()})),      # wrong dtype
           9: ("nonsense", good)}                                            # malformed expert id
    b = ek.HipBatcher(layer, max_wait_us=5000, max_calls=64)
    res = {}

    def caller(i):
        eid, req = bad.get(i, ("m/l0-e1", good))
        try:
            res[i] = b.forward(eid, req)
        except ek.EKError as ex:
            res[i] = ex

    assert run_threads(12, caller) == []
    for i in range(12):
        if i in bad:
            assert isinstance(res[i], ek.EKError) and str(res[i]), i
        else:
            assert res[i] == want, i
    assert res[4].status == ek.EK_EXPERT_NOT_FOUND
    assert all(res[i].status == ek.EK_INVALID_INPUT for i in (1, 6, 9))
    assert st_load(res[0])["data"].shape == (3, H)
    b.close()
    with pytest.raises(ek.EKError):
        ek.HipBatcher(layer, max_wait_us=-1)
    layer.close()
