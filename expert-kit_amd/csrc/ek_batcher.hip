// Micro-batcher in front of the per-expert worker contract.
//
// The controller fires one Forward RPC per active expert concurrently
// (ek-computation/src/controller/executor.rs:141-195) and the worker serves each
// on its own task with Expert::forward (worker/core.rs:47-74).  Served one by
// one, E decode requests cost 2*E kernel launches and E synchronisations on one
// GPU queue.  Here the concurrent callers meet: the first caller to arrive
// leads, optionally lingers for a short window while others join, and runs
// everyone's request as ONE grouped launch (ek_worker_forward_batch); callers
// that arrive while a batch is running queue up and form the next batch, the
// first of them leading it.  Every caller gets its own status and error text.
// Host code only.
#include "../../include/ek_hip.h"

#include <algorithm>
#include <chrono>
#include <condition_variable>
#include <deque>
#include <mutex>
#include <string>
#include <vector>

namespace ek { void set_last_error(const char *msg); }   // the thread's ek_last_error() text

namespace {

struct Slot {
    const char *expert_id;
    const void *req;
    size_t req_len;
    void *resp;
    size_t resp_cap;
    size_t resp_len = 0;
    ek_status st = EK_OK;
    std::string err;
    bool done = false;
    bool lead = false;
    bool oom = false;       // failed without room for an error text
};

}  // namespace

struct ek_batcher {
    ek_layer *layer = nullptr;
    int64_t max_wait_us = 0;
    int32_t max_calls = 0;
    std::mutex mu;
    std::condition_variable cv_arrive;   // a caller joined the queue (wakes a lingering leader)
    std::condition_variable cv_done;     // a batch finished, or leadership was handed over
    std::deque<Slot *> pending;          // arrival order; a leader is always at the front
    bool active = false;                 // a leader is collecting or running
    ek_batcher_stats stats{};
};

static void run_batch(ek_batcher *b, std::vector<Slot *> &batch)
{
    const int32_t n = (int32_t)batch.size();
    std::vector<const char *> ids(n);
    std::vector<const void *> reqs(n);
    std::vector<size_t> lens(n), caps(n), outl(n);
    std::vector<void *> resps(n);
    for (int i = 0; i < n; ++i) {
        ids[i] = batch[i]->expert_id;
        reqs[i] = batch[i]->req;
        lens[i] = batch[i]->req_len;
        resps[i] = batch[i]->resp;
        caps[i] = batch[i]->resp_cap;
    }
    ek_status st = ek_worker_forward_batch(b->layer, n, ids.data(), reqs.data(), lens.data(), resps.data(),
                                           caps.data(), outl.data());
    if (st == EK_OK) {
        for (int i = 0; i < n; ++i) batch[i]->resp_len = outl[i];
        return;
    }
    if (n == 1) {
        batch[0]->st = st;
        batch[0]->err = ek_last_error();
        return;
    }
    // One request spoiled the launch (malformed bytes, an expert that is not loaded, rows beyond
    // the layer's capacity once added up): each caller gets the answer its own request earns.
    for (int i = 0; i < n; ++i) {
        Slot *s = batch[i];
        s->st = ek_worker_forward(b->layer, s->expert_id, s->req, s->req_len, s->resp, s->resp_cap, &s->resp_len);
        if (s->st != EK_OK) s->err = ek_last_error();
    }
}

extern "C" {

ek_status ek_batcher_create(ek_layer *layer, int64_t max_wait_us, int32_t max_calls, ek_batcher **out)
{
    if (!layer || !out) { ek::set_last_error("NULL argument"); return EK_INVALID_INPUT; }
    if (max_wait_us < 0 || max_wait_us > 1000000 || max_calls < 1) {
        ek::set_last_error("max_wait_us must be in [0, 1000000] and max_calls at least 1");
        return EK_INVALID_INPUT;
    }
    try {
        ek_batcher *b = new ek_batcher;
        b->layer = layer;
        b->max_wait_us = max_wait_us;
        b->max_calls = max_calls;
        *out = b;
        return EK_OK;
    } catch (...) {
        ek::set_last_error("out of host memory");
        return EK_OOM;
    }
}

ek_status ek_batcher_forward(ek_batcher *b, const char *expert_id, const void *req, size_t req_len, void *resp,
                             size_t resp_cap, size_t *resp_len)
{
    if (!b || !expert_id || !req || !resp || !resp_len) { ek::set_last_error("NULL argument"); return EK_INVALID_INPUT; }
    Slot me;
    me.expert_id = expert_id; me.req = req; me.req_len = req_len; me.resp = resp; me.resp_cap = resp_cap;
    std::unique_lock<std::mutex> lk(b->mu);
    try {
        b->pending.push_back(&me);
    } catch (...) {
        ek::set_last_error("out of host memory");
        return EK_OOM;
    }
    b->stats.calls += 1;
    if (b->active) {
        b->cv_arrive.notify_one();
        b->cv_done.wait(lk, [&] { return me.done || me.lead; });
    } else {
        b->active = true;
        me.lead = true;
    }
    if (!me.done) {
        // leading: this slot is at the front of the queue
        if (b->max_wait_us > 0 && (int32_t)b->pending.size() < b->max_calls)
            b->cv_arrive.wait_for(lk, std::chrono::microseconds(b->max_wait_us),
                                  [&] { return (int32_t)b->pending.size() >= b->max_calls; });
        std::vector<Slot *> batch;
        bool ran = false;
        try {
            const size_t n = std::min<size_t>(b->pending.size(), (size_t)b->max_calls);
            batch.assign(b->pending.begin(), b->pending.begin() + (std::ptrdiff_t)n);
            b->pending.erase(b->pending.begin(), b->pending.begin() + (std::ptrdiff_t)n);
            b->stats.batches += 1;
            if ((int64_t)n > b->stats.largest_batch) b->stats.largest_batch = (int64_t)n;
            lk.unlock();
            run_batch(b, batch);
            ran = true;
        } catch (...) {
            // host memory ran out while the batch was cut or run: nobody may be left waiting
        }
        if (!lk.owns_lock()) lk.lock();
        if (!ran) {
            if (batch.empty()) {              // never cut: this caller fails alone and the queue moves on
                b->pending.pop_front();
                me.st = EK_OOM;
                me.oom = true;
                me.done = true;
            }
            for (Slot *s : batch) { s->st = EK_OOM; s->oom = true; }
        }
        for (Slot *s : batch) s->done = true;
        if (!b->pending.empty()) b->pending.front()->lead = true;   // the next batch has its leader
        else b->active = false;
        b->cv_done.notify_all();
    }
    lk.unlock();
    if (me.oom) ek::set_last_error("out of host memory");
    else if (me.st != EK_OK) ek::set_last_error(me.err.c_str());
    else *resp_len = me.resp_len;
    return me.st;
}

ek_status ek_batcher_get_stats(ek_batcher *b, ek_batcher_stats *out)
{
    if (!b || !out) { ek::set_last_error("NULL argument"); return EK_INVALID_INPUT; }
    std::lock_guard<std::mutex> lk(b->mu);
    *out = b->stats;
    return EK_OK;
}

ek_status ek_batcher_destroy(ek_batcher *b)
{
    if (!b) return EK_OK;
    {
        std::lock_guard<std::mutex> lk(b->mu);
        if (b->active || !b->pending.empty()) {
            ek::set_last_error("calls are still in flight");
            return EK_INVALID_INPUT;
        }
    }
    delete b;
    return EK_OK;
}

}  // extern "C"
