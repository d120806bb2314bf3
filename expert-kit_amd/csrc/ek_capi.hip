// C-ABI host layer of libek_hip.so (see include/ek_hip.h for the contract).
#include "../../include/ek_hip.h"
#include "ek_internal.h"

#include <algorithm>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <memory>
#include <new>
#include <string>
#include <vector>

namespace {

thread_local std::string g_last_error;

}  // namespace

namespace ek {
void set_last_error(const char *msg) { g_last_error = msg ? msg : ""; }
}  // namespace ek

namespace {

ek_status fail(ek_status st, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return st;
}

ek_status hip_fail(hipError_t e, const char *what)
{
    (void)hipGetLastError();   // clear the sticky error
    return fail(e == hipErrorOutOfMemory ? EK_OOM : EK_HIP_ERROR, "%s: %s", what,
                hipGetErrorString(e));
}

#define EK_HIP(call)                                                  \
    do {                                                              \
        hipError_t _e = (call);                                       \
        if (_e != hipSuccess) return hip_fail(_e, #call);             \
    } while (0)

#define EK_TRY(call)                                                  \
    do {                                                              \
        ek_status _s = (call);                                        \
        if (_s != EK_OK) return _s;                                   \
    } while (0)

// Makes `dev` current for the scope and restores the caller's device.
struct DeviceGuard {
    int prev = -1;
    bool ok = false;
    explicit DeviceGuard(int dev)
    {
        if (hipGetDevice(&prev) != hipSuccess) { (void)hipGetLastError(); prev = -1; }
        ok = hipSetDevice(dev) == hipSuccess;
        if (!ok) (void)hipGetLastError();
    }
    ~DeviceGuard()
    {
        if (prev >= 0 && ok) (void)hipSetDevice(prev);
    }
};

int64_t elem_size(int dt)
{
    switch (dt) {
    case EK_BF16: case EK_F16: return 2;
    case EK_F32: return 4;
    case EK_I8: case EK_F8E4M3: return 1;
    default: return 0;
    }
}

}  // namespace

// Device memory one layer call works in besides its inputs and outputs: routing tables, work
// lists and the two packed intermediates.  Every call writes what it reads (nothing has to start
// at zero).  A layer owns one; ek_layer_forward_static carves one out of a static device array.
struct Workspace {
    int32_t *counts = nullptr, *offsets = nullptr, *perm = nullptr, *inv_perm = nullptr;
    int32_t *row_token = nullptr, *block_hist = nullptr, *err = nullptr;
    void *h = nullptr, *yp = nullptr;
    ek::WorkLists lists{};                   // device work lists (see ek_internal.h)
    int64_t list_cap[ek::kNumLists] = {0, 0, 0, 0};
    // a list of its own for a shared expert's segment cut into wide streaming items
    ek::WorkItem *wide_items = nullptr;
    int32_t *wide_count = nullptr;           // [kNumLists], only [kListStream] is used
    // a shared expert whose intermediate size is not the routed experts': lists of its own (its
    // launches have other shapes) and its own intermediate buffer [T, shared_inter]
    ek::WorkLists slists{};
    int64_t slist_cap[ek::kNumLists] = {0, 0, 0, 0};
    void *hs = nullptr;
};
// capacities of a shared segment's own lists for at most T rows (see launch_segment_lists)
inline int64_t shared_list_cap(int l, int64_t T)
{
    return l == ek::kListStream ? T / 16 + 2 : l == ek::kListT128 ? T / 128 + 2 : 1;
}

struct ek_layer {
    ek_cfg cfg{};             // as the kernels see it: hidden and inter rounded up to what they need
    // The caller's hidden and inter.  A layer whose sizes are not multiples of the kernels' 64
    // (the reference's toy configurations, e.g. ds-tiny: hidden 16, intermediate 8) runs on
    // zero-padded weights and on zero-padded copies of the activation rows: `padded`.
    int64_t user_hidden = 0, user_inter = 0;
    bool padded = false;
    int act = 0;        // 0 bf16, 1 f16
    bool w8 = false;          // one-byte weights (int8 per channel or fp8 per block)
    int wmode = 0;            // ek::WeightMode
    int64_t Pmax = 0;
    hipStream_t stream = nullptr;
    std::mutex mu;       // serialises users of the workspace and the slab table
    std::mutex load_mu;  // serialises weight ingestion

    std::vector<void *> expert_mem;          // one allocation per loaded expert
    std::vector<ek::ExpertSlab> h_slabs;
    ek::ExpertSlab *d_slabs = nullptr;

    Workspace ws;                            // the layer's own, allocated at creation
    // Calls that only enqueue return, and drop `mu`, while their kernels still use the workspace
    // (and the side stream with its fork / join events).  ev_ws marks the end of the last such
    // call; the next user of the workspace, on whatever stream, waits for it on the device first.
    hipEvent_t ev_ws = nullptr;
    bool ws_busy = false;                    // ev_ws has been recorded and not been waited out by a host synchronisation
    int32_t *h_err = nullptr;                // pinned: [0] the error word of a finished call; [1] the number of tile
                                             // items the last pack cut, stored by its kernel (see enqueue_ffn)
    int32_t *d_tile_items = nullptr;         // the device's address of h_err[1] (nullptr: the word stays 0)
    // host-built work lists (ek_layer_experts_forward): pinned image of the device lists,
    // reused once ev_items says the previous copy has been consumed
    uint8_t *h_items = nullptr;
    uint8_t *d_items = nullptr;              // the device's address of h_items (nullptr: asynchronous copies instead)
    hipEvent_t ev_items = nullptr;
    ek::RowCopy *h_segs = nullptr;           // pinned: the row-copy tables of a batched device-memory call, in then out
    ek::RowCopy *d_segs = nullptr;           // the device's address of h_segs
    int64_t segs_cap = 0;                    // entries per table

    // staging for host-memory callers (allocated on first use)
    void *st_x = nullptr, *st_w = nullptr, *st_y = nullptr, *st_xp = nullptr;
    // pinned bounce buffers for their small transfers (see h2d / d2h)
    char *pin_in = nullptr, *pin_out = nullptr;
    size_t pin_cap = 0, pin_in_used = 0, pin_out_used = 0;
    struct PendingOut { void *dst; const char *src; size_t bytes; };
    std::vector<PendingOut> pin_pending;
    int32_t *st_ids = nullptr;
    // router outputs and staging (allocated on first use)
    int32_t *rt_ids = nullptr;
    void *rt_w = nullptr, *st_logits = nullptr;
    float *st_bias = nullptr;
    void *st_raw = nullptr;                  // raw weight bytes during ingestion
    size_t st_raw_bytes = 0;
    hipStream_t load_stream = nullptr;
    // the two FFN kernel families work on disjoint items, so their chains run side by side
    hipStream_t side_stream = nullptr;
    hipEvent_t ev_fork = nullptr, ev_join = nullptr;
    hipEvent_t ev_sfork = nullptr, ev_sjoin = nullptr;   // around the launches of a shared expert of another width
    int64_t shared_inter = 0;                // that shared expert's intermediate size (0: none loaded, or the routed experts')
    size_t hs_bytes = 0;
    // Streams that share a hardware queue run their kernels one after the other (the runtime
    // spreads streams over a few queues in turn), which would undo the fork: the side stream
    // comes from a pool, and for every caller's stream the library finds once, by timing an idle
    // kernel alone and beside itself, a pool member whose kernels do run beside that stream's.
    static constexpr int kSidePool = 3;
    hipStream_t side_pool[kSidePool] = {nullptr, nullptr, nullptr};
    hipEvent_t ev_probe[4] = {nullptr, nullptr, nullptr, nullptr};
    std::vector<std::pair<hipStream_t, hipStream_t>> side_for;   // caller's stream -> pool member

    ek_stats stats{};
    std::mutex stats_mu;
    // worker_expert_activation: pairs per expert, summed by the pack kernel on the device
    // (fused calls) and on the host (per-expert calls)
    uint64_t *d_activation = nullptr;
    std::vector<int64_t> h_activation;
    ek_histogram forward_hist{};             // worker_forward: blocking compute calls, microseconds

    // per-phase event timing (ek_layer_profile)
    bool profiling = false;
    int profile_every = 1;                   // record the events of every n-th call only
    int64_t profile_tick = 0;
    std::vector<hipEvent_t> events;          // 5 per recorded call
    size_t events_used = 0;
};

struct ek_expert {
    ek_layer *layer = nullptr;
};

struct ek_chain {
    std::vector<ek_layer *> layers;
    void *act[2] = {nullptr, nullptr};       // ping-pong activations [max_tokens, H]
    void *act_in = nullptr;                  // hidden size padded: the caller's rows at the kernels' row size
    int32_t *d_err = nullptr;                // [L] per-layer routing error words, gathered
    int32_t *h_err = nullptr;                // pinned
    hipStream_t stream = nullptr;
    // Every layer's ids are the caller's, known when the call starts: the routing halves of layers
    // 1 .. L-1 (pack and work lists, ~50 us each on a stream where they wait their turn) run on
    // route_stream from the start of the call, beside layer 0's kernels; layer l waits for
    // ev_routed[l].  Only when the layers are L different objects (each has its own workspace).
    hipStream_t route_stream = nullptr;
    hipEvent_t ev_begin = nullptr;
    std::vector<hipEvent_t> ev_routed;
    bool distinct = false;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    // key of the captured graph
    const void *k_x = nullptr, *k_ids = nullptr, *k_w = nullptr;
    void *k_y = nullptr;
    int64_t k_T = -1;
    int32_t k_wdt = -1;
    std::vector<int64_t> k_shared;           // per layer when captured: -1 no shared expert, 0 one of the routed experts'
                                             // shape, else its own intermediate size (launches and buffers of its own)
    std::mutex mu;
};

namespace {

// A shared expert's segment (one row per token) is cut by the number of tokens T:
// up to kSharedStreamRows into 16-row streaming items in the routed pairs' list, up to
// kSharedWideRows into streaming items of up to ek::kWideRows rows with a launch of their own
// beside the others, beyond that into tiles like any segment (see enqueue_forward).
constexpr int64_t kSharedStreamRows = 64, kSharedWideRows = 256;
constexpr int64_t kSharedWideItems = kSharedWideRows / ek::kWideRows;

ek_status static_scratch_setup(int dev);   // (defined with ek_layer_forward_static's scratch array)

ek_status dev_alloc(void **p, size_t bytes, const char *what)
{
    hipError_t e = hipMalloc(p, bytes ? bytes : 16);
    if (e != hipSuccess) {
        *p = nullptr;
        (void)hipGetLastError();
        return fail(e == hipErrorOutOfMemory ? EK_OOM : EK_HIP_ERROR, "hipMalloc(%s, %zu bytes): %s",
                    what, bytes, hipGetErrorString(e));
    }
    return EK_OK;
}

void free_layer(ek_layer *L)
{
    if (!L) return;
    (void)hipDeviceSynchronize();
    for (void *p : L->expert_mem) if (p) (void)hipFree(p);
    void *bufs[] = {L->d_slabs, L->ws.counts, L->ws.offsets, L->ws.perm, L->ws.inv_perm, L->ws.row_token,
                    L->ws.block_hist, L->ws.err, L->ws.h, L->ws.yp, L->st_x, L->st_w, L->st_y, L->st_xp,
                    L->d_activation, L->st_ids, L->st_raw, L->rt_ids, L->rt_w, L->st_logits, L->st_bias, L->ws.lists.count, L->ws.lists.items[0], L->ws.lists.items[1],
                    L->ws.lists.items[2], L->ws.lists.items[3], L->ws.wide_items, L->ws.wide_count,
                    L->ws.slists.count, L->ws.slists.items[0], L->ws.slists.items[1], L->ws.slists.items[2],
                    L->ws.slists.items[3], L->ws.hs};
    for (void *p : bufs) if (p) (void)hipFree(p);
    for (hipEvent_t ev : L->events) (void)hipEventDestroy(ev);
    if (L->h_err) (void)hipHostFree(L->h_err);
    if (L->h_items) (void)hipHostFree(L->h_items);
    if (L->pin_in) (void)hipHostFree(L->pin_in);
    if (L->pin_out) (void)hipHostFree(L->pin_out);
    if (L->ev_items) (void)hipEventDestroy(L->ev_items);
    if (L->h_segs) (void)hipHostFree(L->h_segs);
    if (L->stream) (void)hipStreamDestroy(L->stream);
    if (L->load_stream) (void)hipStreamDestroy(L->load_stream);
    if (L->side_stream) (void)hipStreamDestroy(L->side_stream);
    if (L->ev_sfork) (void)hipEventDestroy(L->ev_sfork);
    if (L->ev_sjoin) (void)hipEventDestroy(L->ev_sjoin);
    if (L->ev_fork) (void)hipEventDestroy(L->ev_fork);
    if (L->ev_join) (void)hipEventDestroy(L->ev_join);
    for (hipStream_t ps : L->side_pool) if (ps && ps != L->side_stream) (void)hipStreamDestroy(ps);
    for (hipEvent_t ev : L->ev_probe) if (ev) (void)hipEventDestroy(ev);
    if (L->ev_ws) (void)hipEventDestroy(L->ev_ws);
    delete L;
}

ek_status validate_cfg(const ek_cfg *c)
{
    if (!c) return fail(EK_INVALID_INPUT, "cfg is NULL");
    if (c->act_dtype != EK_BF16 && c->act_dtype != EK_F16)
        return fail(EK_INVALID_INPUT, "act_dtype must be EK_BF16 or EK_F16 (got %d)", c->act_dtype);
    if (c->w_dtype != c->act_dtype && c->w_dtype != EK_I8 && c->w_dtype != EK_F8E4M3)
        return fail(EK_INVALID_INPUT, "w_dtype must equal act_dtype or be EK_I8 or EK_F8E4M3 (got %d)", c->w_dtype);
    if (c->flags & ~EK_CFG_BLOCK_SCALES) return fail(EK_INVALID_INPUT, "unknown flags 0x%x", c->flags);
    if ((c->flags & EK_CFG_BLOCK_SCALES) && c->w_dtype != EK_I8 && c->w_dtype != EK_F8E4M3)
        return fail(EK_INVALID_INPUT, "EK_CFG_BLOCK_SCALES needs w_dtype EK_I8 or EK_F8E4M3");
    if ((c->w_dtype == EK_F8E4M3 || (c->flags & EK_CFG_BLOCK_SCALES)) && (c->hidden > 8192 || c->inter > 8192))
        return fail(EK_INVALID_INPUT, "block-scaled layers hold at most 64 scale blocks per row: hidden and "
                    "inter must not exceed 8192");
    // (the kernels want multiples of 64, at least 128 with one-byte weights: create_layer rounds up
    // and pads; rows of x and y are moved 16 bytes at a time)
    if (c->hidden < 8 || c->hidden % 8 || c->inter < 1)
        return fail(EK_INVALID_INPUT, "hidden (%lld) must be a positive multiple of 8 and inter (%lld) positive",
                    (long long)c->hidden, (long long)c->inter);
    if (c->n_experts < 1 || c->n_experts > ek::kMaxExperts)
        return fail(EK_INVALID_INPUT, "n_experts must be in [1, %d] (got %d)", ek::kMaxExperts,
                    c->n_experts);
    if (c->top_k < 1 || c->top_k > c->n_experts)
        return fail(EK_INVALID_INPUT, "top_k must be in [1, n_experts] (got %d)", c->top_k);
    if (c->max_tokens < 1 || c->max_tokens * (int64_t)c->top_k >= (1ll << 31))
        return fail(EK_INVALID_INPUT, "max_tokens * top_k must be in [1, 2^31) (max_tokens %lld)",
                    (long long)c->max_tokens);
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess) { (void)hipGetLastError(); ndev = 0; }
    if (c->device_id < 0 || c->device_id >= ndev)
        return fail(EK_HIP_ERROR, "device_id %d not available (%d HIP devices visible)", c->device_id,
                    ndev);
    return EK_OK;
}

ek_status create_layer(const ek_cfg *cfg, int64_t pmax, ek_layer **out)
{
    ek_layer *L = new (std::nothrow) ek_layer();
    if (!L) return fail(EK_OOM, "host allocation failed");
    L->cfg = *cfg;
    L->user_hidden = cfg->hidden;
    L->user_inter = cfg->inter;
    {
        const bool one_byte = cfg->w_dtype == EK_I8 || cfg->w_dtype == EK_F8E4M3;
        auto up = [&](int64_t v) { return std::max<int64_t>((v + 63) / 64 * 64, one_byte ? 128 : 64); };
        L->cfg.hidden = up(cfg->hidden);
        L->cfg.inter = up(cfg->inter);
        L->padded = L->cfg.hidden != cfg->hidden || L->cfg.inter != cfg->inter;
        cfg = &L->cfg;                            // from here on: the kernels' sizes
    }
    L->act = cfg->act_dtype == EK_BF16 ? 0 : 1;
    L->w8 = cfg->w_dtype == EK_I8 || cfg->w_dtype == EK_F8E4M3;
    L->wmode = cfg->w_dtype == EK_I8 ? ((cfg->flags & EK_CFG_BLOCK_SCALES) ? ek::kWI8Block : ek::kWI8)
               : cfg->w_dtype == EK_F8E4M3 ? ek::kWF8Block : ek::kW16;
    L->Pmax = pmax;
    const int E = cfg->n_experts;
    // slot E of the tables is the shared expert; its segment (one row per token) follows the
    // P routed rows in the packed buffers
    const int64_t rows_max = pmax + cfg->max_tokens;
    L->expert_mem.assign(E + 1, nullptr);
    L->h_slabs.assign(E + 1, ek::ExpertSlab{nullptr, nullptr, nullptr, nullptr, nullptr});
    const int64_t nblocks = (pmax + ek::kPackChunk - 1) / ek::kPackChunk;
    ek_status st = EK_OK;
    auto A = [&](void **p, size_t bytes, const char *what) {
        if (st == EK_OK) st = dev_alloc(p, bytes, what);
    };
    A((void **)&L->d_slabs, sizeof(ek::ExpertSlab) * (E + 1), "slab table");
    A((void **)&L->ws.counts, sizeof(int32_t) * E, "counts");
    A((void **)&L->ws.offsets, sizeof(int32_t) * (E + 1), "offsets");
    A((void **)&L->ws.perm, sizeof(int32_t) * pmax, "perm");
    A((void **)&L->ws.inv_perm, sizeof(int32_t) * pmax, "inv_perm");
    A((void **)&L->ws.row_token, sizeof(int32_t) * rows_max, "row_token");
    A((void **)&L->ws.block_hist, sizeof(int32_t) * nblocks * E, "block_hist");
    A((void **)&L->ws.err, sizeof(int32_t) * 4, "err");
    A((void **)&L->d_activation, sizeof(uint64_t) * E, "activation counters");
    L->h_activation.assign(E, 0);
    for (int i = 0; i < 10; ++i) L->forward_hist.le[i] = 4000.0 * i;   // the reference's buckets (metrics.rs:51)
    A(&L->ws.h, (size_t)rows_max * cfg->inter * 2, "h");
    A(&L->ws.yp, (size_t)rows_max * cfg->hidden * 2, "yp");
    A((void **)&L->ws.lists.count, sizeof(int32_t) * ek::kNumLists, "work list counts");
    A((void **)&L->ws.wide_items, sizeof(ek::WorkItem) * kSharedWideItems, "shared expert's work list");
    A((void **)&L->ws.wide_count, sizeof(int32_t) * ek::kNumLists, "shared expert's work list count");
    A((void **)&L->ws.slists.count, sizeof(int32_t) * ek::kNumLists, "shared expert's work list counts");
    for (int l = 0; l < ek::kNumLists; ++l) {
        L->ws.slist_cap[l] = shared_list_cap(l, cfg->max_tokens);
        A((void **)&L->ws.slists.items[l], sizeof(ek::WorkItem) * L->ws.slist_cap[l], "shared expert's work list");
    }
    for (int l = 0; l < ek::kNumLists; ++l) {
        // A layer call's lists hold at most one remainder item per expert (list_capacity); a grouped
        // launch of per-expert calls may name an expert many times, each call a segment of its own,
        // so this workspace's lists are sized by rows alone: rows_max / 17 items of 17..32 rows, and
        // so on (16 bytes an item).  The streaming list also takes the wide cut's items (see
        // wide_cut_pays: fewer than 128 tile items of at most 128 rows become at most two streaming
        // items each) and is bounded by what one launch's grid can number.
        const int64_t min_rows[ek::kNumLists] = {1, 17, 33, 65};
        int64_t cap = rows_max / min_rows[l] + (l == ek::kListStream ? 264 : 1);
        if (l == ek::kListStream && cap > 65535) cap = 65535;
        if (cap < ek::list_capacity(l, rows_max, E + 1) + 1) cap = ek::list_capacity(l, rows_max, E + 1) + 1;
        L->ws.list_cap[l] = cap;
        A((void **)&L->ws.lists.items[l], sizeof(ek::WorkItem) * cap, "work list");
    }
    if (st == EK_OK) {
        hipError_t e = hipMemset(L->d_slabs, 0, sizeof(ek::ExpertSlab) * (E + 1));
        if (e == hipSuccess) e = hipMemset(L->ws.err, 0, sizeof(int32_t) * 4);
        if (e == hipSuccess) e = hipMemset(L->d_activation, 0, sizeof(uint64_t) * E);
        if (e == hipSuccess) e = hipMemset(L->ws.lists.count, 0, sizeof(int32_t) * ek::kNumLists);
        if (e == hipSuccess) e = hipMemset(L->ws.wide_count, 0, sizeof(int32_t) * ek::kNumLists);
        if (e == hipSuccess) e = hipHostMalloc((void **)&L->h_err, sizeof(int32_t) * 4, hipHostMallocDefault);
        if (e == hipSuccess) {
            memset(L->h_err, 0, sizeof(int32_t) * 4);
            void *dp = nullptr;
            if (hipHostGetDevicePointer(&dp, L->h_err + 1, 0) == hipSuccess) L->d_tile_items = (int32_t *)dp;
            else (void)hipGetLastError();
        }
        if (e == hipSuccess) e = hipStreamCreateWithFlags(&L->stream, hipStreamNonBlocking);
        if (e == hipSuccess) e = hipStreamCreateWithFlags(&L->load_stream, hipStreamNonBlocking);
        if (e == hipSuccess) e = hipStreamCreateWithFlags(&L->side_stream, hipStreamNonBlocking);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&L->ev_sfork, hipEventDisableTiming);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&L->ev_sjoin, hipEventDisableTiming);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&L->ev_fork, hipEventDisableTiming);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&L->ev_join, hipEventDisableTiming);
        L->side_pool[0] = L->side_stream;
        for (int i = 1; i < ek_layer::kSidePool && e == hipSuccess; ++i)
            e = hipStreamCreateWithFlags(&L->side_pool[i], hipStreamNonBlocking);
        for (int i = 0; i < 4 && e == hipSuccess; ++i) e = hipEventCreate(&L->ev_probe[i]);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&L->ev_ws, hipEventDisableTiming);
        if (e != hipSuccess) st = hip_fail(e, "layer setup");
    }
    if (st == EK_OK) st = static_scratch_setup(cfg->device_id);
    if (st != EK_OK) {
        std::string keep = g_last_error;
        free_layer(L);
        g_last_error = keep;
        return st;
    }
    *out = L;
    return EK_OK;
}

// table slot of a public expert index; EK_SHARED_EXPERT names the shared expert
ek_status expert_slot(ek_layer *L, int32_t expert, int32_t *slot)
{
    if (expert == EK_SHARED_EXPERT) { *slot = L->cfg.n_experts; return EK_OK; }
    if (expert < 0 || expert >= L->cfg.n_experts)
        return fail(EK_INVALID_INPUT, "expert %d outside [0, %d)", expert, L->cfg.n_experts);
    *slot = expert;
    return EK_OK;
}

ek_status check_desc(const ek_weight_desc *d, const char *name, int64_t rows, int64_t cols, int wmode)
{
    const bool w8 = wmode == ek::kWI8;
    if (!d || !d->ptr) return fail(EK_WEIGHT_NOT_FOUND, "%s weight is missing", name);
    if (d->rows != rows || d->cols != cols)
        return fail(EK_INVALID_INPUT, "%s weight is [%lld,%lld], expected [%lld,%lld]", name,
                    (long long)d->rows, (long long)d->cols, (long long)rows, (long long)cols);
    if (d->mem != EK_HOST && d->mem != EK_DEVICE)
        return fail(EK_INVALID_INPUT, "%s weight: bad mem %d", name, d->mem);
    if (ek::block_scaled(wmode)) {
        // kept as stored: the checkpoint's bytes and its 128 x 128 scale blocks
        const int want = wmode == ek::kWF8Block ? EK_F8E4M3 : EK_I8;
        if (d->dtype != want)
            return fail(EK_INVALID_INPUT, "%s weight must be of the layer's w_dtype %d (got %d)", name, want, d->dtype);
        if (d->scale_kind != EK_SCALE_BLOCK128)
            return fail(EK_INVALID_INPUT, "%s weight: a block-scaled layer needs EK_SCALE_BLOCK128", name);
        if (!d->scale) return fail(EK_WEIGHT_NOT_FOUND, "%s block scale is missing", name);
        if (d->scale_dtype != EK_BF16 && d->scale_dtype != EK_F32 && d->scale_dtype != EK_F16)
            return fail(EK_INVALID_INPUT, "%s scale: bad dtype %d", name, d->scale_dtype);
    } else if (w8) {
        if (d->dtype != EK_I8)
            return fail(EK_INVALID_INPUT, "%s weight must be EK_I8 for an int8 layer (got %d)", name,
                        d->dtype);
        if (d->scale_kind != EK_SCALE_PER_CHANNEL)
            return fail(EK_INVALID_INPUT, "%s weight: int8 needs EK_SCALE_PER_CHANNEL", name);
        if (!d->scale) return fail(EK_WEIGHT_NOT_FOUND, "%s scale is missing", name);
        if (d->scale_dtype != EK_BF16 && d->scale_dtype != EK_F32 && d->scale_dtype != EK_F16)
            return fail(EK_INVALID_INPUT, "%s scale: bad dtype %d", name, d->scale_dtype);
    } else if (d->scale_kind == EK_SCALE_BLOCK128) {
        // block-scaled checkpoint tensors are dequantised to the 16-bit type at load
        if (d->dtype != EK_I8 && d->dtype != EK_F8E4M3 && d->dtype != EK_BF16 && d->dtype != EK_F16 &&
            d->dtype != EK_F32)
            return fail(EK_INVALID_INPUT, "%s weight: bad dtype %d", name, d->dtype);
        if (!d->scale) return fail(EK_WEIGHT_NOT_FOUND, "%s block scale is missing", name);
        if (d->scale_dtype != EK_BF16 && d->scale_dtype != EK_F32 && d->scale_dtype != EK_F16)
            return fail(EK_INVALID_INPUT, "%s scale: bad dtype %d", name, d->scale_dtype);
    } else {
        if (d->dtype != EK_BF16 && d->dtype != EK_F16 && d->dtype != EK_F32)
            return fail(EK_INVALID_INPUT, "%s weight: dtype %d cannot be cast to the layer's 16-bit type "
                        "without block scales", name, d->dtype);
        if (d->scale_kind != EK_SCALE_NONE)
            return fail(EK_INVALID_INPUT, "%s weight: per-channel scales need an EK_I8 layer", name);
    }
    return EK_OK;
}

// bytes of a descriptor's scale tensor (0 if it has none)
size_t scale_bytes(const ek_weight_desc *d)
{
    if (d->scale_kind == EK_SCALE_PER_CHANNEL) return (size_t)d->rows * elem_size(d->scale_dtype);
    if (d->scale_kind == EK_SCALE_BLOCK128)
        return (size_t)((d->rows + 127) / 128) * ((d->cols + 127) / 128) * elem_size(d->scale_dtype);
    return 0;
}

// Brings `bytes` of (host or device) source to a device address usable by the
// tiling kernels.  Host sources go through the layer's raw staging buffer.
ek_status stage_raw(ek_layer *L, const void *src, int mem, size_t bytes, size_t stage_off,
                    const void **dev)
{
    if (mem == EK_DEVICE) { *dev = src; return EK_OK; }
    EK_HIP(hipMemcpyAsync((char *)L->st_raw + stage_off, src, bytes, hipMemcpyHostToDevice,
                          L->load_stream));
    *dev = (char *)L->st_raw + stage_off;
    return EK_OK;
}

// inter_e: the expert's intermediate size (the layer's; a shared expert may have another)
ek_status set_expert_locked(ek_layer *L, int32_t e, const ek_weight_desc *up,
                            const ek_weight_desc *gate, const ek_weight_desc *down, int64_t inter_e = 0)
{
    const int64_t H = L->cfg.hidden, I = inter_e > 0 ? inter_e : L->cfg.inter;
    EK_TRY(check_desc(up, "up", I, H, L->wmode));
    EK_TRY(check_desc(gate, "gate", I, H, L->wmode));
    EK_TRY(check_desc(down, "down", H, I, L->wmode));
    const size_t wsz = L->w8 ? 1 : 2;
    const size_t mat_bytes = (size_t)H * I * wsz;
    const bool blocks = ek::block_scaled(L->wmode);
    // scales kept beside the weights: one per output channel (int8) or per 128 x 128 block (fp8)
    const size_t nb_ih = (size_t)((I + 127) / 128) * (size_t)((H + 127) / 128);
    const size_t s_upgate = blocks ? nb_ih : (size_t)I, s_dn = blocks ? nb_ih : (size_t)H;
    const size_t scale_floats = L->w8 ? 2 * s_upgate + s_dn : 0;
    const size_t total = 3 * mat_bytes + scale_floats * sizeof(float);

    // staging for host sources: three raw matrices (+ scales) back to back
    const ek_weight_desc *ds[3] = {up, gate, down};
    size_t need = 0;
    for (auto d : ds) {
        if (d->mem == EK_HOST) {
            need += (size_t)d->rows * d->cols * elem_size(d->dtype);
            need = (need + 255) & ~(size_t)255;
            need += (scale_bytes(d) + 255) & ~(size_t)255;
        }
    }
    if (need > L->st_raw_bytes) {
        EK_HIP(hipStreamSynchronize(L->load_stream));
        if (L->st_raw) (void)hipFree(L->st_raw);
        L->st_raw = nullptr; L->st_raw_bytes = 0;
        EK_TRY(dev_alloc(&L->st_raw, need, "weight staging"));
        L->st_raw_bytes = need;
    }

    // device-resident sources may still be being written on the caller's streams
    if (up->mem == EK_DEVICE || gate->mem == EK_DEVICE || down->mem == EK_DEVICE)
        EK_HIP(hipDeviceSynchronize());

    void *mem = nullptr;
    EK_TRY(dev_alloc(&mem, total, "expert weights"));
    uint8_t *base = (uint8_t *)mem;
    ek::ExpertSlab slab;
    slab.upgate = base;
    slab.down = base + 2 * mat_bytes;
    float *sc = (float *)(base + 3 * mat_bytes);
    slab.s_up = L->w8 ? sc : nullptr;
    slab.s_gate = L->w8 ? sc + s_upgate : nullptr;
    slab.s_down = L->w8 ? sc + 2 * s_upgate : nullptr;

    ek_status st = EK_OK;
    size_t off = 0;
    const int dst_dt = L->w8 ? L->cfg.w_dtype : L->cfg.act_dtype;
    float *sdst[3] = {sc, sc + s_upgate, sc + 2 * s_upgate};
    uint8_t *wdst[3] = {base, base, base + 2 * mat_bytes};
    const int mi[3] = {0, 1, 0}, nmat[3] = {2, 2, 1};
    for (int i = 0; i < 3 && st == EK_OK; ++i) {
        const ek_weight_desc *d = ds[i];
        const void *src = nullptr;
        const size_t bytes = (size_t)d->rows * d->cols * elem_size(d->dtype);
        st = stage_raw(L, d->ptr, d->mem, bytes, off, &src);
        if (d->mem == EK_HOST) off = (off + bytes + 255) & ~(size_t)255;
        if (st != EK_OK) break;
        const void *ssrc = nullptr;
        const size_t sbytes = scale_bytes(d);
        if (sbytes) {
            st = stage_raw(L, d->scale, d->mem, sbytes, off, &ssrc);
            if (d->mem == EK_HOST) off = (off + sbytes + 255) & ~(size_t)255;
            if (st != EK_OK) break;
        }
        ek::launch_tile_weights(src, d->dtype, d->rows, d->cols, wdst[i], dst_dt, mi[i], nmat[i],
                                d->scale_kind == EK_SCALE_BLOCK128 && !blocks ? ssrc : nullptr, d->scale_dtype,
                                L->load_stream);
        if (L->w8)
            ek::launch_scales_to_f32(ssrc, d->scale_dtype, blocks ? (int64_t)(i == 2 ? s_dn : s_upgate) : d->rows,
                                     sdst[i], L->load_stream);
    }
    if (st == EK_OK) {
        hipError_t e = hipGetLastError();
        if (e == hipSuccess) e = hipStreamSynchronize(L->load_stream);
        if (e != hipSuccess) st = hip_fail(e, "weight tiling");
    }
    if (st != EK_OK) { (void)hipFree(mem); return st; }

    // publish: swap the slab entry under the forward lock; free any old copy
    void *old = nullptr;
    {
        std::lock_guard<std::mutex> lk(L->mu);
        old = L->expert_mem[e];
        if (old) (void)hipDeviceSynchronize();   // drain work that may read the old copy
        hipError_t er = hipMemcpy(L->d_slabs + e, &slab, sizeof slab, hipMemcpyHostToDevice);
        if (er != hipSuccess) {
            // the table still names the old copy (if any): keep it, drop the new one
            (void)hipFree(mem);
            return hip_fail(er, "slab table update");
        }
        L->expert_mem[e] = mem;
        L->h_slabs[e] = slab;
        if (e == L->cfg.n_experts) L->shared_inter = I != L->cfg.inter ? I : 0;
    }
    if (old) (void)hipFree(old);
    return EK_OK;
}

// A shared expert whose intermediate size is not the routed experts' (DeepSeek's shared_experts has
// moe_intermediate_size * n_shared_experts channels: expertkit_torch/models/deepseek_v3/model.py:57-61):
// its size must suit the kernels as the layer's own does, and the layer's workspace gets an
// intermediate buffer of that width.
ek_status prepare_shared_width(ek_layer *L, const ek_weight_desc *up, int64_t *inter_e)
{
    *inter_e = 0;
    if (!up || up->rows == L->cfg.inter) return EK_OK;
    const int64_t Is = up->rows;
    if (L->padded)
        return fail(EK_INVALID_INPUT, "a shared expert of another intermediate size (%lld) needs a layer whose hidden and "
                    "inter are multiples of 64 (128 with one-byte weights)", (long long)Is);
    if (Is < (L->w8 ? 128 : 64) || Is % 64)
        return fail(EK_INVALID_INPUT, "the shared expert's intermediate size (%lld) must be a multiple of 64, at least %d",
                    (long long)Is, L->w8 ? 128 : 64);
    if (ek::block_scaled(L->wmode) && Is > 8192)
        return fail(EK_INVALID_INPUT, "block-scaled layers hold at most 64 scale blocks per row: the shared expert's "
                    "intermediate size (%lld) must not exceed 8192", (long long)Is);
    const size_t need = (size_t)L->cfg.max_tokens * Is * 2;
    std::lock_guard<std::mutex> lk(L->mu);
    if (need > L->hs_bytes) {
        EK_HIP(hipDeviceSynchronize());
        if (L->ws.hs) (void)hipFree(L->ws.hs);
        L->ws.hs = nullptr; L->hs_bytes = 0;
        EK_TRY(dev_alloc(&L->ws.hs, need, "shared expert's intermediate rows"));
        L->hs_bytes = need;
    }
    *inter_e = Is;
    return EK_OK;
}

// A padded layer's weights: zero-padded device copies of the caller's matrices (and scales) in
// the kernels' sizes, handed to set_expert_locked as device sources.  Padded channels have
// weight 0 (and scale 0), padded contraction elements meet the zero columns of the staged rows.
ek_status set_expert_padded(ek_layer *L, int32_t e, const ek_weight_desc *up, const ek_weight_desc *gate,
                            const ek_weight_desc *down)
{
    const int64_t UH = L->user_hidden, UI = L->user_inter, H = L->cfg.hidden, I = L->cfg.inter;
    EK_TRY(check_desc(up, "up", UI, UH, L->wmode));
    EK_TRY(check_desc(gate, "gate", UI, UH, L->wmode));
    EK_TRY(check_desc(down, "down", UH, UI, L->wmode));
    const ek_weight_desc *src[3] = {up, gate, down};
    const int64_t pr[3] = {I, I, H}, pc[3] = {H, H, I};
    ek_weight_desc padded[3];
    std::vector<void *> tmp;
    ek_status st = EK_OK;
    for (int i = 0; i < 3 && st == EK_OK; ++i) {
        const ek_weight_desc *d = src[i];
        const hipMemcpyKind kind = d->mem == EK_HOST ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice;
        padded[i] = *d;
        padded[i].rows = pr[i];
        padded[i].cols = pc[i];
        padded[i].mem = EK_DEVICE;
        const size_t es = (size_t)elem_size(d->dtype);
        void *w = nullptr;
        st = dev_alloc(&w, (size_t)pr[i] * pc[i] * es, "padded weights");
        if (st != EK_OK) break;
        tmp.push_back(w);
        padded[i].ptr = w;
        hipError_t er = hipMemsetAsync(w, 0, (size_t)pr[i] * pc[i] * es, L->load_stream);
        if (er == hipSuccess)
            er = hipMemcpy2DAsync(w, (size_t)pc[i] * es, d->ptr, (size_t)d->cols * es, (size_t)d->cols * es,
                                  (size_t)d->rows, kind, L->load_stream);
        if (er == hipSuccess && d->scale_kind != EK_SCALE_NONE && d->scale) {
            const size_t ses = (size_t)elem_size(d->scale_dtype);
            const bool per_channel = d->scale_kind == EK_SCALE_PER_CHANNEL;
            // per channel: one row of `rows` scales; per block: a [ceil(rows/128), ceil(cols/128)] grid
            const size_t ur = per_channel ? 1 : (size_t)(d->rows + 127) / 128, uc = per_channel ? (size_t)d->rows : (size_t)(d->cols + 127) / 128;
            const size_t qr = per_channel ? 1 : (size_t)(pr[i] + 127) / 128, qc = per_channel ? (size_t)pr[i] : (size_t)(pc[i] + 127) / 128;
            void *sc = nullptr;
            st = dev_alloc(&sc, qr * qc * ses, "padded scales");
            if (st != EK_OK) break;
            tmp.push_back(sc);
            padded[i].scale = sc;
            er = hipMemsetAsync(sc, 0, qr * qc * ses, L->load_stream);
            if (er == hipSuccess)
                er = hipMemcpy2DAsync(sc, qc * ses, d->scale, uc * ses, uc * ses, ur, kind, L->load_stream);
        }
        if (er != hipSuccess) st = hip_fail(er, "padding the weights");
    }
    if (st == EK_OK) st = set_expert_locked(L, e, &padded[0], &padded[1], &padded[2]);   // (waits for the copies)
    std::string keep = g_last_error;
    (void)hipStreamSynchronize(L->load_stream);
    for (void *p : tmp) (void)hipFree(p);
    g_last_error = keep;
    return st;
}

// One use of a layer's workspace on stream s; the caller holds L->mu for the scope.
// begin(): the stream waits (on the device) for the last enqueue-only call that used the
// workspace.  At the end of the scope the stream's position is recorded as that call's end,
// unless synced() says the host has waited for the stream, after which nothing is pending.
// A stream under capture by the caller is left alone both ways (a captured wait on an event
// recorded outside the capture is not allowed): replays of such a graph use the workspace like
// the call they record, and ordering them against other calls on the layer is the caller's part.
struct WorkspaceUse {
    hipEvent_t ev;
    bool *busy;
    hipStream_t s;
    bool capturing = false, host_synced = false;
    WorkspaceUse(ek_layer *layer, hipStream_t stream) : ev(layer->ev_ws), busy(&layer->ws_busy), s(stream) {}
    WorkspaceUse(hipEvent_t event, bool *busy_flag, hipStream_t stream) : ev(event), busy(busy_flag), s(stream) {}
    ek_status begin()
    {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cs) != hipSuccess) { (void)hipGetLastError(); cs = hipStreamCaptureStatusNone; }
        capturing = cs != hipStreamCaptureStatusNone;
        if (!capturing && *busy) EK_HIP(hipStreamWaitEvent(s, ev, 0));
        return EK_OK;
    }
    void device_idle() { *busy = false; }          // after a hipDeviceSynchronize
    void synced() { host_synced = true; }          // after a hipStreamSynchronize(s) that followed begin()
    ~WorkspaceUse()
    {
        if (capturing) return;
        if (host_synced) { *busy = false; return; }
        if (hipEventRecord(ev, s) == hipSuccess) *busy = true;
        else (void)hipGetLastError();
    }
};

// ---- ek_layer_forward_static: the workspace of a layer call in a static device array ----------
// Callers that must not allocate (code under HIP graph capture, serving loops, harnesses that
// forbid hipMalloc) get a layer call whose workspace is this array instead of memory from
// hipMalloc.  Every GPU the library runs on holds its own copy of the array, at its own address,
// until the process ends; the array's name is only a host-side handle, so host code takes the
// device address once per device (static_scratch_setup, with that device current) and passes
// that address, never the name, to kernels.
constexpr size_t kStaticScratchBytes = EK_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
struct StaticScratch {
    unsigned char *ptr = nullptr;            // this device's address of `scratch`
    hipEvent_t ev = nullptr;                 // end of the last enqueue-only call that used it
    bool busy = false;
    std::mutex mu;                           // one call at a time carves and enqueues
};
StaticScratch g_static[kMaxDevices];
std::mutex g_static_setup_mu;

// Once per device, with that device current (called by ek_layer_create): address and event.
ek_status static_scratch_setup(int dev)
{
    if (dev < 0 || dev >= kMaxDevices) return EK_OK;   // such a device gets no static entry point
    std::lock_guard<std::mutex> lk(g_static_setup_mu);
    StaticScratch &S = g_static[dev];
    if (S.ptr) return EK_OK;
    void *p = nullptr;
    EK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p || ((uintptr_t)p & 255)) return fail(EK_INTERNAL, "static scratch array at %p is not 256-byte aligned", p);
    EK_HIP(hipEventCreateWithFlags(&S.ev, hipEventDisableTiming));
    S.ptr = (unsigned char *)p;
    return EK_OK;
}

// Lays a workspace for T tokens of layer L out in `base` (capacity `cap` bytes).  Returns the bytes
// needed; W is valid only if they fit.
size_t carve_workspace(const ek_layer *L, int64_t T, unsigned char *base, size_t cap, Workspace *W)
{
    const int64_t E = L->cfg.n_experts, K = L->cfg.top_k, P = T * K, rows = P + T;
    const int64_t nblocks = (P + ek::kPackChunk - 1) / ek::kPackChunk;
    size_t off = 0;
    auto take = [&](size_t bytes) -> void * {
        void *p = base + off;
        off += (bytes + 255) & ~(size_t)255;
        return off <= cap ? p : nullptr;
    };
    W->counts = (int32_t *)take(sizeof(int32_t) * E);
    W->offsets = (int32_t *)take(sizeof(int32_t) * (E + 1));
    W->perm = (int32_t *)take(sizeof(int32_t) * P);
    W->inv_perm = (int32_t *)take(sizeof(int32_t) * P);
    W->row_token = (int32_t *)take(sizeof(int32_t) * rows);
    W->block_hist = (int32_t *)take(sizeof(int32_t) * nblocks * E);
    W->err = (int32_t *)take(sizeof(int32_t) * 4);
    W->lists.count = (int32_t *)take(sizeof(int32_t) * ek::kNumLists);
    W->wide_items = (ek::WorkItem *)take(sizeof(ek::WorkItem) * kSharedWideItems);
    W->wide_count = (int32_t *)take(sizeof(int32_t) * ek::kNumLists);
    for (int l = 0; l < ek::kNumLists; ++l) {
        W->list_cap[l] = ek::list_capacity(l, rows, E + 1) + (l == ek::kListStream ? 264 : 1);
        W->lists.items[l] = (ek::WorkItem *)take(sizeof(ek::WorkItem) * (size_t)W->list_cap[l]);
    }
    W->slists.count = (int32_t *)take(sizeof(int32_t) * ek::kNumLists);
    for (int l = 0; l < ek::kNumLists; ++l) {
        W->slist_cap[l] = shared_list_cap(l, T);
        W->slists.items[l] = (ek::WorkItem *)take(sizeof(ek::WorkItem) * (size_t)W->slist_cap[l]);
    }
    W->h = take((size_t)rows * L->cfg.inter * 2);
    W->yp = take((size_t)rows * L->cfg.hidden * 2);
    W->hs = L->shared_inter ? take((size_t)T * L->shared_inter * 2) : nullptr;
    return off;
}

struct Timer {
    std::chrono::steady_clock::time_point t0 = std::chrono::steady_clock::now();
    double us() const
    {
        return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
    }
};

// one observation of the worker_forward histogram; the caller holds stats_mu
void observe_forward(ek_layer *L, double us)
{
    ek_histogram &h = L->forward_hist;
    for (int i = 0; i < 10; ++i) if (us <= h.le[i]) h.cumulative[i] += 1;
    h.cumulative[10] += 1;
    h.count += 1;
    h.sum += us;
}

ek_status ensure_io_staging(ek_layer *L)
{
    if (L->st_x) return EK_OK;
    const int64_t T = L->cfg.max_tokens, K = L->cfg.top_k, H = L->cfg.hidden;
    // st_x / st_y also serve ek_layer_expert_forward, whose n may reach Pmax
    const int64_t rows = L->Pmax > T ? L->Pmax : T;
    EK_TRY(dev_alloc(&L->st_x, (size_t)rows * H * 2, "x staging"));
    if (L->padded) {                                   // the padding columns stay zero from here on
        EK_HIP(hipMemset(L->st_x, 0, (size_t)rows * H * 2));
        EK_HIP(hipDeviceSynchronize());
    }
    EK_TRY(dev_alloc(&L->st_y, (size_t)rows * H * 2, "y staging"));
    EK_TRY(dev_alloc(&L->st_w, (size_t)T * K * 4, "gate-weight staging"));
    EK_TRY(dev_alloc((void **)&L->st_ids, (size_t)T * K * 4, "ids staging"));
    return EK_OK;
}

// Host <-> device copies of blocking host-memory calls.  A pageable hipMemcpyAsync of tens to
// hundreds of KiB costs 20-75 us here; the same bytes through pinned memory (a CPU memcpy and
// a DMA the stream can queue) 10-20 us; alone the two forms meet between 1 and 4 MiB, inside
// a call the staged form still wins at 1.8 MiB (DeepSeek-V3 decode layer call with host
// tensors: 2.67 -> 2.01 ms; measured on the MI355X box).  So transfers up to kBounceMax go
// through a pinned bounce buffer while it has room; results are copied out of it once the
// stream has been waited for (bounce_flush).  One call at a time uses the buffers:
// host-memory calls hold the layer's lock and end with a synchronisation.
// The buffers start at 2 MiB each; the first call that wants more makes them kBounceCapMax.
constexpr size_t kBounceMax = 4u << 20, kBounceCapMin = 2u << 20, kBounceCapMax = 16u << 20;

ek_status bounce_begin(ek_layer *L, hipStream_t s, size_t want = 0)
{
    if (L->pin_in_used || L->pin_out_used || !L->pin_pending.empty()) {
        // a call that failed half way left transfers behind: let them finish, drop their results
        EK_HIP(hipStreamSynchronize(s));
        L->pin_pending.clear();
        L->pin_in_used = L->pin_out_used = 0;
    }
    size_t cap = L->pin_cap ? L->pin_cap : kBounceCapMin;
    if (cap < want) cap = kBounceCapMax;
    if (cap != L->pin_cap) {
        // nothing is in flight here: host-memory calls end with a synchronisation
        if (L->pin_in) (void)hipHostFree(L->pin_in);
        if (L->pin_out) (void)hipHostFree(L->pin_out);
        L->pin_in = L->pin_out = nullptr;
        L->pin_cap = 0;
        EK_HIP(hipHostMalloc((void **)&L->pin_in, cap, hipHostMallocDefault));
        EK_HIP(hipHostMalloc((void **)&L->pin_out, cap, hipHostMallocDefault));
        L->pin_cap = cap;
    }
    return EK_OK;
}

ek_status h2d(ek_layer *L, void *dst, const void *src, size_t bytes, hipStream_t s)
{
    if (bytes == 0) return EK_OK;
    if (L->pin_in && bytes <= kBounceMax && L->pin_in_used + bytes <= L->pin_cap) {
        char *p = L->pin_in + L->pin_in_used;
        memcpy(p, src, bytes);
        L->pin_in_used += (bytes + 63) & ~(size_t)63;
        EK_HIP(hipMemcpyAsync(dst, p, bytes, hipMemcpyHostToDevice, s));
    } else {
        EK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s));
    }
    return EK_OK;
}

ek_status d2h(ek_layer *L, void *dst, const void *src, size_t bytes, hipStream_t s)
{
    if (bytes == 0) return EK_OK;
    if (L->pin_out && bytes <= kBounceMax && L->pin_out_used + bytes <= L->pin_cap) {
        char *p = L->pin_out + L->pin_out_used;
        L->pin_out_used += (bytes + 63) & ~(size_t)63;
        EK_HIP(hipMemcpyAsync(p, src, bytes, hipMemcpyDeviceToHost, s));
        L->pin_pending.push_back({dst, p, bytes});
    } else {
        EK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s));
    }
    return EK_OK;
}

// Rows of a padded layer: n rows of the caller's hidden size between the caller's buffer
// (host or device, rows back to back) and a staging buffer whose rows have the kernels'
// hidden size (its padding columns are zero and are never written).
ek_status rows_in(ek_layer *L, void *staged, const void *src, int64_t n, int mem, hipStream_t s)
{
    if (n <= 0) return EK_OK;
    const size_t w = (size_t)L->user_hidden * 2;
    EK_HIP(hipMemcpy2DAsync(staged, (size_t)L->cfg.hidden * 2, src, w, w, (size_t)n,
                            mem == EK_HOST ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice, s));
    return EK_OK;
}

ek_status rows_out(ek_layer *L, void *dst, const void *staged, int64_t n, int mem, hipStream_t s)
{
    if (n <= 0) return EK_OK;
    const size_t w = (size_t)L->user_hidden * 2;
    EK_HIP(hipMemcpy2DAsync(dst, w, staged, (size_t)L->cfg.hidden * 2, w, (size_t)n,
                            mem == EK_HOST ? hipMemcpyDeviceToHost : hipMemcpyDeviceToDevice, s));
    return EK_OK;
}

// after the stream has been waited for
void bounce_flush(ek_layer *L)
{
    for (const auto &p : L->pin_pending) memcpy(p.dst, p.src, p.bytes);
    L->pin_pending.clear();
    L->pin_in_used = L->pin_out_used = 0;
}

ek_status err_to_status(int32_t err)
{
    if (err & 1) return fail(EK_INVALID_INPUT, "expert id outside [0, n_experts)");
    if (err & 2) return fail(EK_EXPERT_NOT_FOUND, "a pair was routed to an expert that is not loaded");
    return EK_OK;
}

ek_status copy_route_out(ek_layer *L, const Workspace &W, const ek_route_out *r, int64_t P, int mem, hipStream_t s,
                         bool experts_ran = true)
{
    if (!r) return EK_OK;
    if (r->expert_out && !experts_ran)
        return fail(EK_INVALID_INPUT, "ek_route_out.expert_out: this call runs no experts");
    const int E = L->cfg.n_experts;
    auto out = [&](void *dst, const void *src, size_t bytes) -> ek_status {
        if (mem == EK_HOST) return d2h(L, dst, src, bytes, s);
        EK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s));
        return EK_OK;
    };
    if (r->counts) EK_TRY(out(r->counts, W.counts, sizeof(int32_t) * E));
    if (r->offsets) EK_TRY(out(r->offsets, W.offsets, sizeof(int32_t) * (E + 1)));
    if (P > 0 && r->perm) EK_TRY(out(r->perm, W.perm, sizeof(int32_t) * P));
    if (P > 0 && r->inv_perm) EK_TRY(out(r->inv_perm, W.inv_perm, sizeof(int32_t) * P));
    if (P > 0 && r->expert_out) {
        if (L->padded) EK_TRY(rows_out(L, r->expert_out, W.yp, P, mem, s));    // the caller's hidden size
        else EK_TRY(out(r->expert_out, W.yp, (size_t)P * L->cfg.hidden * 2));
    }
    return EK_OK;
}

ek::PackArgs pack_args(ek_layer *L, const Workspace &W, const int32_t *ids, int64_t P, bool check_loaded)
{
    ek::PackArgs a;
    a.ids = ids;
    a.P = P;
    a.E = L->cfg.n_experts;
    a.K = L->cfg.top_k;
    a.nblocks = (int32_t)((P + ek::kPackChunk - 1) / ek::kPackChunk);
    a.slabs = check_loaded ? L->d_slabs : nullptr;
    a.block_hist = W.block_hist;
    a.counts = W.counts;
    a.offsets = W.offsets;
    a.perm = W.perm;
    a.inv_perm = W.inv_perm;
    a.row_token = W.row_token;
    a.err = W.err;
    a.activation = check_loaded ? L->d_activation : nullptr;
    a.tile_items_host = check_loaded ? L->d_tile_items : nullptr;
    if (check_loaded) a.lists = W.lists;
    else a.lists = ek::WorkLists{{nullptr, nullptr, nullptr, nullptr}, nullptr};
    return a;
}

// The side stream to fork to from stream s (the caller holds L->mu).  Decided once per caller's
// stream: an idle kernel of ~100 us is timed alone on s, then on s and on a pool member at once;
// the first member beside which the pair takes clearly less than twice the time runs its kernels
// beside s's.  This first use waits for s on the host (a few hundred microseconds).  A stream under
// capture is not probed (a graph's branches are not bound to the streams they were recorded on).
hipStream_t pick_side_stream(ek_layer *L, hipStream_t s)
{
    for (const auto &p : L->side_for) if (p.first == s) return p.second;
    // (the choice is remembered per handle; a stream that was destroyed and another created at the same
    // address inherits it: either choice is correct, a poor one costs the overlap only)
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &cs) != hipSuccess) { (void)hipGetLastError(); return L->side_stream; }
    if (cs != hipStreamCaptureStatusNone) return L->side_stream;
    hipStream_t chosen = L->side_stream;
    constexpr int kIters = 200;            // ~200k cycles: far above launch jitter
    hipEvent_t *ev = L->ev_probe;
    bool ok = hipEventRecord(ev[0], s) == hipSuccess;
    if (ok) { ek::launch_idle(kIters, s); ok = hipEventRecord(ev[1], s) == hipSuccess; }
    float alone = 0.f;
    if (ok) ok = hipEventSynchronize(ev[1]) == hipSuccess && hipEventElapsedTime(&alone, ev[0], ev[1]) == hipSuccess;
    for (int i = 0; i < ek_layer::kSidePool && ok; ++i) {
        hipStream_t c = L->side_pool[i];
        if (c == s) continue;
        ok = hipEventRecord(ev[0], s) == hipSuccess && hipStreamWaitEvent(c, ev[0], 0) == hipSuccess;
        if (!ok) break;
        ek::launch_idle(kIters, s);
        ek::launch_idle(kIters, c);
        ok = hipEventRecord(ev[2], c) == hipSuccess && hipStreamWaitEvent(s, ev[2], 0) == hipSuccess &&
             hipEventRecord(ev[3], s) == hipSuccess && hipEventSynchronize(ev[3]) == hipSuccess;
        float both = 0.f;
        if (ok) ok = hipEventElapsedTime(&both, ev[0], ev[3]) == hipSuccess;
        if (ok && both < 1.6f * alone) { chosen = c; break; }
    }
    if (!ok) (void)hipGetLastError();
    if (L->side_for.size() >= 64) L->side_for.erase(L->side_for.begin());   // (streams come and go)
    L->side_for.emplace_back(s, chosen);
    return chosen;
}

// Both FFN stages over the work lists in W.lists: x [*, H] (rows picked through
// `rows`, or packed order when nullptr) -> W.h -> out [P, H].  P and E bound the
// list lengths (grid sizes); ev, if set, receives the stage boundary event.
// wide_items > 0: the lists hold that many weight-streaming items of up to kWideRows rows and
// nothing else (the per-expert entry points' cut for calls that would leave the tile kernel
// most of the chip idle).
// extra_stream: streaming items the lists hold beyond what P rows over E experts can give (a
// shared segment cut into 16-row items).
// shared_wide: W.wide_items holds that many streaming items of up to kWideRows rows (a shared
// segment); they get launches of their own on the side stream, beside the others.
// exact: the lists' lengths when the caller built them on the host (the grids then fit them,
// an empty list gets no launch, and the two chains run side by side exactly when both have work).
ek_status enqueue_ffn(ek_layer *L, const Workspace &W, const void *x, const int32_t *rows, void *out, int64_t P, int64_t E,
                      hipStream_t s, hipEvent_t *ev, int64_t wide_items = 0, int64_t extra_stream = 0,
                      int64_t shared_wide = 0, const int64_t *exact = nullptr, int64_t known_tile_items = -1)
{
    const int64_t H = L->cfg.hidden, I = L->cfg.inter;
    ek::FfnArgs a1;
    a1.x = x; a1.x_stride = H; a1.rows = rows; a1.slabs = L->d_slabs; a1.out = W.h; a1.out_stride = I;
    a1.N = (int32_t)I; a1.Kdim = (int32_t)H; a1.lists = W.lists;
    ek::FfnArgs a2 = a1;
    a2.x = W.h; a2.x_stride = I; a2.rows = nullptr; a2.out = out; a2.out_stride = H;
    a2.N = (int32_t)H; a2.Kdim = (int32_t)I;
    int64_t cap[ek::kNumLists];
    for (int l = 0; l < ek::kNumLists; ++l) {
        cap[l] = ek::list_capacity(l, P, E) + (l == ek::kListStream ? extra_stream : 0);
        if (exact) cap[l] = exact[l];          // the caller built the lists on the host
        if (cap[l] > W.list_cap[l]) cap[l] = W.list_cap[l];
        if (cap[l] < 0) cap[l] = 0;
    }
    if (wide_items > 0) {
        EK_HIP(ek::launch_ffn_stream(a1, 1, L->act, L->wmode, wide_items, true, false, s));
        if (ev) EK_HIP(hipEventRecord(ev[2], s));
        EK_HIP(ek::launch_ffn_stream(a2, 2, L->act, L->wmode, wide_items, true, false, s));
        return EK_OK;
    }
    // Two independent chains: the weight-streaming kernel (items of <= 16 rows) and the
    // MFMA tile kernel (longer items) touch disjoint rows of h and out, and run side by side:
    // the streaming chain is forked to the side stream and joined before returning.  The tile
    // chain stays on s: a tile workgroup takes a whole CU (registers and LDS), so its persistent
    // workgroups should claim as many CUs as they have tiles at once and leave the others to the
    // streaming kernel, instead of waiting for streaming workgroups to drain CU by CU.  Which kernel
    // the device starts first is decided by the queues, not by the order of the launches: the
    // kernel on s follows the pack kernel in its own queue at once, the one on the side stream
    // only when the fork's event has crossed to the other queue, ~6 us later (Qwen3 fp16 decode at
    // 256 tokens, enqueue-only calls: tile kernel second 128 us and 0.216 ms per call, first 88 us
    // and 0.201 ms).  With tiles for all 256 CUs the two run in turn.
    // Measured on MI355X against running both in order: Qwen3 fp16 (E 128, K 8) 512 / 1024 /
    // 2048 / 4096 / 16384 tokens -7 / -11 / -2 / -1 / 0 %, the ragged 4-layer chain -4.8 %;
    // DeepSeek-V3 int8 (E 128) -2 / -5 / -3 / 0 / 0 %; with its 16-bit weights (E 64) -7 / -4 /
    // +3 / -1 / +1 %: with experts of that size, beyond 128 pairs per expert, the long streaming
    // kernel takes from the tiles what the overlap returns.
    // Up to 4 pairs per expert the tile lists are empty unless the routing is skewed: then a hot
    // expert's 17+ rows are a tile that keeps a handful of CUs busy for a whole contraction, after
    // the streaming kernel in the same stream (DeepSeek-V3 int8, 32 / 64 / 128 tokens, Zipf 1.0:
    // 493 / 587 / 813 us in order, 391 / 521 / 748 us side by side), while with no tiles the
    // fork/join costs 10-20 us for nothing.  Skew persists from one call to the next, so the last
    // pack's tile count, which its kernel left in pinned memory, decides; it may be a call or two
    // old, and either choice computes the same bits.
    const bool have_stream = cap[ek::kListStream] > 0;
    const bool few_rows = P <= 4 * E;      // streaming items of about four rows or fewer: see launch_ffn_stream
    const bool have_tiles = cap[ek::kListT32] + cap[ek::kListT64] + cap[ek::kListT128] > 0;
    const bool small_expert = 3 * H * I * (L->w8 ? 1 : 2) <= (16ll << 20);
    const bool tiles_lately = exact ? true : ((volatile int32_t *)L->h_err)[1] > 0;   // (exact: have_tiles says it)
    // Above 4 pairs per expert tiles are the rule; but when the last call cut none at all, this one's
    // tile launches will most likely find empty lists too, and the fork's event records and waits are
    // host time (~30 us of a 57 us call of 64 tokens on 16 small experts).  Not under capture: what is
    // recorded there is replayed for other routings, and the sizes decide alone.
    bool capturing = false;
    if (P > 4 * E && !tiles_lately) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cs) != hipSuccess) (void)hipGetLastError();
        capturing = cs != hipStreamCaptureStatusNone;
    }
    const bool fork = have_stream && have_tiles &&
                      (P > 4 * E ? (P <= 128 * E || small_expert) && (tiles_lately || capturing) : tiles_lately);
    hipStream_t s_stream = s, s_tiles = s;
    hipStream_t side = nullptr;
    if (fork || shared_wide > 0) {
        side = pick_side_stream(L, s);
        EK_HIP(hipEventRecord(L->ev_fork, s));
        EK_HIP(hipStreamWaitEvent(side, L->ev_fork, 0));
    }
    if (fork) s_stream = side;
    // The per-expert entry points know how many tile items their lists hold.  When those would put a
    // tile on at most half of the CUs, the narrow form of the tile kernel (half the channels per
    // workgroup, twice the workgroups) shortens the call: one tile's walk over the whole contraction is
    // what such a call waits for (one DeepSeek-V3 int8 expert, 1024 rows: 225 -> 157 us; Qwen3 fp16,
    // 2048 / 4096 rows: 97 -> 79 / 100 -> 76 us).  With more tiles the wide form's fewer reads of the
    // activation tile win (DeepSeek-V3, 4096 rows: 350 against 412 us), and a layer call's streaming
    // chain runs on the CUs the tiles leave free, so that narrower tiles there only move time from
    // one chain to the other (Qwen3 decode, 256 tokens: 0.195 against 0.199 ms).  Same bits either way.
    if (exact) known_tile_items = exact[ek::kListT32] + exact[ek::kListT64] + exact[ek::kListT128];
    for (int stage = 1; stage <= 2; ++stage) {
        const ek::FfnArgs &a = stage == 1 ? a1 : a2;
        const bool tiles_first = fork;
        const int64_t wgs_per_item = (a.N + ek::tile_channels(stage, false) - 1) / ek::tile_channels(stage, false);
        // (the narrow form runs three stages deep also with 16-bit weights, i.e. starts a tile with the
        // loads of its first two steps: a contraction of one 64-element step has no second one, and
        // the load would read past the last row of x and past the expert's last weight chunk)
        const bool narrow = known_tile_items > 0 && known_tile_items * wgs_per_item <= 128 && a.Kdim >= 128;
        if (tiles_first && have_tiles) EK_HIP(ek::launch_ffn_tile(a, stage, L->act, L->wmode, cap, narrow, s_tiles));
        if (have_stream) EK_HIP(ek::launch_ffn_stream(a, stage, L->act, L->wmode, cap[ek::kListStream], false, few_rows, s_stream));
        if (shared_wide > 0) {
            ek::FfnArgs aw = a;                  // the same stage over the shared segment's own list
            aw.lists.items[ek::kListStream] = W.wide_items;
            aw.lists.count = W.wide_count;
            EK_HIP(ek::launch_ffn_stream(aw, stage, L->act, L->wmode, shared_wide, true, false, side));
        }
        if (!tiles_first && have_tiles) EK_HIP(ek::launch_ffn_tile(a, stage, L->act, L->wmode, cap, narrow, s_tiles));
        if (stage == 1 && ev) EK_HIP(hipEventRecord(ev[2], s));
    }
    if (fork || shared_wide > 0) {
        EK_HIP(hipEventRecord(L->ev_join, side));
        EK_HIP(hipStreamWaitEvent(s, L->ev_join, 0));
    }
    return EK_OK;
}

// How a call's shared-expert segment (if the layer has one) is cut.
struct SharedCut {
    bool shared, streamed, wide;
    bool own;        // another intermediate size than the routed experts': lists, launches and buffer of its own
};
SharedCut shared_cut(const ek_layer *L, int64_t T)
{
    SharedCut c;
    c.shared = L->expert_mem[L->cfg.n_experts] != nullptr && T > 0;
    c.streamed = c.shared && T <= kSharedStreamRows;
    c.wide = c.shared && !c.streamed && T <= kSharedWideRows;
    c.own = c.shared && L->shared_inter != 0;
    return c;
}

// The routing half of a layer call on stream s: pack, and the shared expert's segment appended to
// its work lists.  It reads nothing but the ids, so a chain may run it ahead of the layer's turn.
ek_status enqueue_route(ek_layer *L, const Workspace &W, const int32_t *ids, int64_t T, hipStream_t s)
{
    const int E = L->cfg.n_experts;
    const int64_t P = T * L->cfg.top_k;
    ek::launch_pack(pack_args(L, W, ids, P, true), s);
    const SharedCut sc = shared_cut(L, T);
    if (sc.own) {
        ek::launch_segment_lists(W.slists, E, (int32_t)P, (int32_t)T, W.row_token, sc.streamed ? 1 : sc.wide ? 2 : 0, s);
    } else if (sc.wide) {
        ek::WorkLists own = W.lists;
        own.items[ek::kListStream] = W.wide_items;
        own.count = W.wide_count;
        ek::launch_append_segment(own, E, (int32_t)P, (int32_t)T, W.row_token, 2, s);
    } else if (sc.shared) {
        ek::launch_append_segment(W.lists, E, (int32_t)P, (int32_t)T, W.row_token, sc.streamed ? 1 : 0, s);
    }
    EK_HIP(hipGetLastError());
    return EK_OK;
}

// A shared expert of another intermediate size: both stages over its own lists (W.slists: rows
// P .. P+T-1 of the packed order, token t at row P + t), with its own shapes, on the side stream
// beside the routed pairs' launches; the caller's stream waits for L->ev_sjoin before the combine.
// The intermediate rows live in W.hs [T, shared_inter]: the kernels index rows by packed position,
// so they get the address row P would have if the buffer started at row 0.
ek_status enqueue_shared_own(ek_layer *L, const Workspace &W, const void *x, int64_t P, int64_t T, const SharedCut &sc,
                             hipStream_t s)
{
    const int64_t H = L->cfg.hidden, Is = L->shared_inter;
    if (!W.hs) return fail(EK_INTERNAL, "no intermediate buffer for the shared expert");
    hipStream_t side = pick_side_stream(L, s);
    EK_HIP(hipEventRecord(L->ev_sfork, s));
    EK_HIP(hipStreamWaitEvent(side, L->ev_sfork, 0));
    ek::FfnArgs a1;
    a1.x = x; a1.x_stride = H; a1.rows = W.row_token; a1.slabs = L->d_slabs;
    a1.out = (char *)W.hs - (size_t)P * Is * 2; a1.out_stride = Is;
    a1.N = (int32_t)Is; a1.Kdim = (int32_t)H; a1.lists = W.slists;
    ek::FfnArgs a2 = a1;
    a2.x = a1.out; a2.x_stride = Is; a2.rows = nullptr; a2.out = W.yp; a2.out_stride = H;
    a2.N = (int32_t)H; a2.Kdim = (int32_t)Is;
    int64_t cap[ek::kNumLists];
    for (int l = 0; l < ek::kNumLists; ++l) cap[l] = std::min<int64_t>(shared_list_cap(l, T), W.slist_cap[l]);
    for (int stage = 1; stage <= 2; ++stage) {
        const ek::FfnArgs &a = stage == 1 ? a1 : a2;
        if (sc.streamed) {
            EK_HIP(ek::launch_ffn_stream(a, stage, L->act, L->wmode, (T + 15) / 16, false, T <= 4, side));
        } else if (sc.wide) {
            EK_HIP(ek::launch_ffn_stream(a, stage, L->act, L->wmode, (T + ek::kWideRows - 1) / ek::kWideRows, true, false, side));
        } else {
            cap[ek::kListStream] = 1;        // the usual cut leaves at most one item of <= 16 rows
            EK_HIP(ek::launch_ffn_tile(a, stage, L->act, L->wmode, cap, false, side));
            EK_HIP(ek::launch_ffn_stream(a, stage, L->act, L->wmode, 1, false, false, side));
        }
    }
    EK_HIP(hipEventRecord(L->ev_sjoin, side));
    return EK_OK;
}

// pack -> stage 1 -> stage 2 -> combine on stream s; all pointers are device.
// routed: enqueue_route for these ids has been enqueued already (s waits for it).
// before_combine: called between the FFN launches and the combine (a chain enqueues the later
// layers' routing halves and waits for the next layer's there: the wait costs nothing at that
// point, and the next layer's first kernel then depends on nothing but this layer's combine in
// its own queue).
// Most pairs of a call that runs pair-direct (launch_ffn_pairs).  Every pair streams its expert's
// weights on its own, so tokens that share an expert read it twice, and stage 2's one wave per pair
// walks the whole contraction where the ordinary launch of so few items slices it.  Measured on
// MI355X, DeepSeek-V3 int8 layer (256 experts, top-8), enqueue-only calls: 1 token 75.3 -> 62.4 us
// (352 MB: 5.6 TB/s, 71 % of the 8 TB/s peak, over the whole call), 2 tokens 131.7 -> 121-127 us,
// 4 tokens 220 -> 231 us, 8 tokens 366 -> 437 us.
constexpr int64_t kPairDirectPairs = 16;
bool pair_direct_fits(const ek_layer *L, int64_t T)
{
    const int64_t P = T * L->cfg.top_k;
    const SharedCut sc = shared_cut(L, T);          // a shared expert of the routed experts' shape is one more wave
    return P > 0 && P <= kPairDirectPairs && L->cfg.top_k <= ek::kPairDirectMaxK && (!sc.shared || !sc.own);
}

// want_tables: the caller reads the call's routing tables or packed expert outputs afterwards.
ek_status enqueue_forward(ek_layer *L, const Workspace &W, const void *x, const int32_t *ids, const void *w, int w_f32,
                          int64_t T, void *y, hipStream_t s, bool routed = false,
                          const std::function<ek_status()> *before_combine = nullptr, bool want_tables = true)
{
    const int64_t H = L->cfg.hidden;
    const int E = L->cfg.n_experts, K = L->cfg.top_k;
    const int64_t P = T * K;
    hipEvent_t *ev = nullptr;
    if (L->profiling && L->profile_tick++ % L->profile_every == 0 && L->events_used + 5 <= L->events.size()) {
        ev = L->events.data() + L->events_used;
        L->events_used += 5;
    }
    if (ev) EK_HIP(hipEventRecord(ev[0], s));
    // A decode call of one or two tokens: its few pairs run as one-row items straight from the ids,
    // and stage 2 adds a token's pairs itself: two kernels instead of four (no pack, no combine;
    // DeepSeek-V3 int8 layer on MI355X, 1 / 2 tokens: see kPairDirectPairs).  Same bits.
    if (!routed && !want_tables && pair_direct_fits(L, T)) {
        ek::FfnArgs a1;
        a1.x = x; a1.x_stride = H; a1.rows = nullptr; a1.slabs = L->d_slabs; a1.out = W.h; a1.out_stride = L->cfg.inter;
        a1.N = (int32_t)L->cfg.inter; a1.Kdim = (int32_t)H; a1.lists = W.lists;
        a1.pair_ids = ids; a1.pair_K = K; a1.pair_P = (int32_t)P; a1.n_experts = E;
        a1.pair_shared = shared_cut(L, T).shared ? 1 : 0;
        a1.pair_err = W.err; a1.pair_activation = L->d_activation; a1.pair_tile_items_host = L->d_tile_items;
        ek::FfnArgs a2 = a1;
        a2.x = W.h; a2.x_stride = L->cfg.inter; a2.out = nullptr; a2.out_stride = H;
        a2.N = (int32_t)H; a2.Kdim = (int32_t)L->cfg.inter;
        a2.pair_w = w; a2.pair_w_f32 = w_f32; a2.pair_y = y;
        if (ev) EK_HIP(hipEventRecord(ev[1], s));
        EK_HIP(ek::launch_ffn_pairs(a1, 1, L->act, L->wmode, s));
        if (ev) EK_HIP(hipEventRecord(ev[2], s));
        EK_HIP(ek::launch_ffn_pairs(a2, 2, L->act, L->wmode, s));
        if (ev) EK_HIP(hipEventRecord(ev[3], s));
        if (before_combine) EK_TRY((*before_combine)());
        if (ev) EK_HIP(hipEventRecord(ev[4], s));
        return EK_OK;
    }
    if (!routed) EK_TRY(enqueue_route(L, W, ids, T, s));
    // the shared expert is one more segment: every token once, rows P .. P+T-1 of the packed buffers.
    // As tiles a decode-sized shared segment would occupy 8 to 14 CUs for the length of the whole
    // contraction.  Up to kSharedStreamRows tokens it is cut into 16-row streaming items
    // (measured on the DeepSeek-V3 shape at 64 tokens: 1.62 ms against 1.76 ms as a tile); each
    // item re-reads the expert's weights, so beyond that it is cut into items of up to 64 rows,
    // which the streaming kernel's wide form takes in a launch of its own.
    const SharedCut sc = shared_cut(L, T);
    const bool shared = sc.shared, shared_streamed = sc.streamed && !sc.own, shared_wide = sc.wide && !sc.own;
    if (ev) EK_HIP(hipEventRecord(ev[1], s));
    if (P > 0 && sc.own) EK_TRY(enqueue_shared_own(L, W, x, P, T, sc, s));     // on the side stream, joined before the combine
    if (P > 0) {
        const bool in_lists = shared && !shared_wide && !sc.own;   // the shared segment's items sit in the routed pairs' lists
        EK_TRY(enqueue_ffn(L, W, x, W.row_token, W.yp, in_lists ? P + T : P, in_lists ? E + 1 : E, s, ev, 0,
                           shared_streamed ? (T + 15) / 16 : 0,
                           shared_wide ? (T + ek::kWideRows - 1) / ek::kWideRows : 0));
        if (sc.own) EK_HIP(hipStreamWaitEvent(s, L->ev_sjoin, 0));
        if (ev) EK_HIP(hipEventRecord(ev[3], s));
        if (before_combine) EK_TRY((*before_combine)());
        ek::CombineArgs c;
        c.yp = W.yp; c.inv_perm = W.inv_perm; c.w = w; c.y = y; c.T = T; c.K = K; c.H = H;
        c.act = L->act; c.w_f32 = w_f32;
        c.shared = shared ? (const char *)W.yp + (size_t)P * H * 2 : nullptr;
        ek::launch_combine(c, s);
    } else {
        if (ev) {
            EK_HIP(hipEventRecord(ev[2], s));
            EK_HIP(hipEventRecord(ev[3], s));
        }
        if (before_combine) EK_TRY((*before_combine)());
    }
    if (ev) EK_HIP(hipEventRecord(ev[4], s));
    EK_HIP(hipGetLastError());
    return EK_OK;
}

ek_status finish_blocking(ek_layer *L, const Workspace &W, hipStream_t s)
{
    EK_HIP(hipMemcpyAsync(L->h_err, W.err, sizeof(int32_t), hipMemcpyDeviceToHost, s));
    EK_HIP(hipStreamSynchronize(s));
    bounce_flush(L);
    return err_to_status(L->h_err[0]);
}

}  // namespace

// ------------------------------------------------------------------ C ABI

#define EK_GUARDED(...)                                               \
    try {                                                             \
        __VA_ARGS__                                                   \
    } catch (const std::bad_alloc &) {                                \
        return fail(EK_OOM, "host allocation failed");                \
    } catch (const std::exception &ex) {                              \
        return fail(EK_INTERNAL, "exception: %s", ex.what());         \
    } catch (...) {                                                   \
        return fail(EK_INTERNAL, "unknown exception");                \
    }

extern "C" {

const char *ek_backend_name(void) { return "hip"; }

const char *ek_last_error(void) { return g_last_error.c_str(); }

int32_t ek_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return 0; }
    return n;
}

ek_status ek_layer_create(const ek_cfg *cfg, ek_layer **out)
{
    EK_GUARDED(
        if (!out) return fail(EK_INVALID_INPUT, "out is NULL");
        *out = nullptr;
        EK_TRY(validate_cfg(cfg));
        DeviceGuard dg(cfg->device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", cfg->device_id);
        return create_layer(cfg, cfg->max_tokens * (int64_t)cfg->top_k, out);
    )
}

ek_status ek_layer_destroy(ek_layer *layer)
{
    EK_GUARDED(
        if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
        DeviceGuard dg(layer->cfg.device_id);
        {
            // wait for users of the workspace
            std::lock_guard<std::mutex> l1(layer->load_mu);
            std::lock_guard<std::mutex> l2(layer->mu);
        }
        free_layer(layer);
        return EK_OK;
    )
}

ek_status ek_layer_set_expert(ek_layer *layer, int32_t expert, const ek_weight_desc *up,
                              const ek_weight_desc *gate, const ek_weight_desc *down)
{
    EK_GUARDED(
        if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
        EK_TRY(expert_slot(layer, expert, &expert));
        DeviceGuard dg(layer->cfg.device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", layer->cfg.device_id);
        std::lock_guard<std::mutex> lk(layer->load_mu);
        if (layer->padded) {
            if (!up || !gate || !down) return fail(EK_WEIGHT_NOT_FOUND, "a weight matrix is missing");
            return set_expert_padded(layer, expert, up, gate, down);
        }
        int64_t inter_e = 0;
        if (expert == layer->cfg.n_experts) EK_TRY(prepare_shared_width(layer, up, &inter_e));
        return set_expert_locked(layer, expert, up, gate, down, inter_e);
    )
}

ek_status ek_layer_remove_expert(ek_layer *layer, int32_t expert)
{
    EK_GUARDED(
        if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
        EK_TRY(expert_slot(layer, expert, &expert));
        DeviceGuard dg(layer->cfg.device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", layer->cfg.device_id);
        std::lock_guard<std::mutex> lk0(layer->load_mu);
        void *old = nullptr;
        {
            std::lock_guard<std::mutex> lk(layer->mu);
            old = layer->expert_mem[expert];
            if (!old) return fail(EK_EXPERT_NOT_FOUND, "expert %d is not loaded", expert);
            EK_HIP(hipDeviceSynchronize());
            layer->expert_mem[expert] = nullptr;
            if (expert == layer->cfg.n_experts) layer->shared_inter = 0;
            layer->h_slabs[expert] = ek::ExpertSlab{nullptr, nullptr, nullptr, nullptr, nullptr};
            EK_HIP(hipMemcpy(layer->d_slabs + expert, &layer->h_slabs[expert], sizeof(ek::ExpertSlab),
                             hipMemcpyHostToDevice));
        }
        (void)hipFree(old);
        return EK_OK;
    )
}

ek_status ek_layer_has_expert(ek_layer *layer, int32_t expert, int32_t *loaded)
{
    EK_GUARDED(
        if (!layer || !loaded) return fail(EK_INVALID_INPUT, "NULL argument");
        EK_TRY(expert_slot(layer, expert, &expert));
        std::lock_guard<std::mutex> lk(layer->mu);
        *loaded = layer->expert_mem[expert] != nullptr;
        return EK_OK;
    )
}

ek_status ek_layer_forward(ek_layer *layer, const void *x, const int32_t *ids, const void *w,
                           int32_t w_dtype, int64_t T, void *y, const ek_route_out *route,
                           int32_t mem, void *stream)
{
    EK_GUARDED(
        if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
        if (T < 0 || T > layer->cfg.max_tokens)
            return fail(EK_INVALID_INPUT, "T = %lld outside [0, max_tokens = %lld]", (long long)T,
                        (long long)layer->cfg.max_tokens);
        if (mem != EK_HOST && mem != EK_DEVICE) return fail(EK_INVALID_INPUT, "bad mem %d", mem);
        if (w_dtype != layer->cfg.act_dtype && w_dtype != EK_F32)
            return fail(EK_INVALID_INPUT, "w_dtype must be the activation dtype or EK_F32 (got %d)",
                        w_dtype);
        if (T > 0 && (!x || !ids || !w || !y)) return fail(EK_INVALID_INPUT, "NULL tensor pointer");
        if (mem == EK_HOST && stream)
            return fail(EK_INVALID_INPUT, "host-memory calls are blocking: stream must be NULL");
        DeviceGuard dg(layer->cfg.device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", layer->cfg.device_id);
        Timer tm;
        const int64_t H = layer->cfg.hidden, K = layer->cfg.top_k, P = T * K;
        const int w_f32 = w_dtype == EK_F32;
        std::lock_guard<std::mutex> lk(layer->mu);
        hipStream_t s = stream ? (hipStream_t)stream : layer->stream;
        WorkspaceUse use(layer, s);
        EK_TRY(use.begin());
        ek_status st = EK_OK;
        // a blocking call on device buffers sees everything submitted before it
        if (mem == EK_DEVICE && !stream) { EK_HIP(hipDeviceSynchronize()); use.device_idle(); }
        if (layer->padded) {
            EK_TRY(ensure_io_staging(layer));
            const int32_t *d_ids = ids;
            const void *d_w = w;
            if (mem == EK_HOST && T > 0) {
                EK_HIP(hipMemcpyAsync(layer->st_ids, ids, (size_t)P * 4, hipMemcpyHostToDevice, s));
                EK_HIP(hipMemcpyAsync(layer->st_w, w, (size_t)P * (w_f32 ? 4 : 2), hipMemcpyHostToDevice, s));
                d_ids = layer->st_ids;
                d_w = layer->st_w;
            }
            EK_TRY(rows_in(layer, layer->st_x, x, T, mem, s));
            EK_TRY(enqueue_forward(layer, layer->ws, layer->st_x, d_ids, d_w, w_f32, T, layer->st_y, s, false, nullptr, route != nullptr));
            EK_TRY(rows_out(layer, y, layer->st_y, T, mem, s));
            EK_TRY(copy_route_out(layer, layer->ws, route, P, mem, s));
            if (!stream) { st = finish_blocking(layer, layer->ws, s); use.synced(); }
        } else if (mem == EK_DEVICE) {
            EK_TRY(enqueue_forward(layer, layer->ws, x, ids, w, w_f32, T, y, s, false, nullptr, route != nullptr));
            EK_TRY(copy_route_out(layer, layer->ws, route, P, mem, s));
            if (!stream) { st = finish_blocking(layer, layer->ws, s); use.synced(); }
        } else {
            EK_TRY(ensure_io_staging(layer));
            EK_TRY(bounce_begin(layer, s, (size_t)T * H * 2 + (size_t)P * 8));
            if (T > 0) {
                EK_TRY(h2d(layer, layer->st_x, x, (size_t)T * H * 2, s));
                EK_TRY(h2d(layer, layer->st_ids, ids, (size_t)P * 4, s));
                EK_TRY(h2d(layer, layer->st_w, w, (size_t)P * (w_f32 ? 4 : 2), s));
            }
            EK_TRY(enqueue_forward(layer, layer->ws, layer->st_x, layer->st_ids, layer->st_w, w_f32, T,
                                   layer->st_y, s, false, nullptr, route != nullptr));
            if (T > 0) EK_TRY(d2h(layer, y, layer->st_y, (size_t)T * H * 2, s));
            EK_TRY(copy_route_out(layer, layer->ws, route, P, mem, s));
            st = finish_blocking(layer, layer->ws, s);
            use.synced();
        }
        {
            std::lock_guard<std::mutex> sl(layer->stats_mu);
            layer->stats.forward_calls += 1;
            layer->stats.tokens += T;
            layer->stats.pairs += P;
            if (!stream) { layer->stats.last_forward_us = tm.us(); observe_forward(layer, layer->stats.last_forward_us); }
        }
        return st;
    )
}

ek_status ek_layer_forward_static(ek_layer *layer, const void *x, const int32_t *ids, const void *w,
                                  int32_t w_dtype, int64_t T, void *y, const ek_route_out *route, void *stream)
{
    EK_GUARDED(
        if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
        if (T < 0 || T > layer->cfg.max_tokens)
            return fail(EK_INVALID_INPUT, "T = %lld outside [0, max_tokens = %lld]", (long long)T,
                        (long long)layer->cfg.max_tokens);
        if (w_dtype != layer->cfg.act_dtype && w_dtype != EK_F32)
            return fail(EK_INVALID_INPUT, "w_dtype must be the activation dtype or EK_F32 (got %d)", w_dtype);
        if (T > 0 && (!x || !ids || !w || !y)) return fail(EK_INVALID_INPUT, "NULL tensor pointer");
        if (layer->padded)
            return fail(EK_INVALID_INPUT, "ek_layer_forward_static: hidden and inter must be multiples of 64 (128 with "
                        "one-byte weights); padded layers stage their rows in allocated buffers");
        const int dev = layer->cfg.device_id;
        if (dev < 0 || dev >= kMaxDevices || !g_static[dev].ptr)
            return fail(EK_INTERNAL, "no static scratch on device %d", dev);
        StaticScratch &S = g_static[dev];
        Workspace W;
        const size_t need = carve_workspace(layer, T, S.ptr, kStaticScratchBytes, &W);
        if (need > kStaticScratchBytes)
            return fail(EK_INVALID_INPUT, "ek_layer_forward_static: T = %lld needs %zu bytes of workspace, the static "
                        "scratch holds %zu; use ek_layer_forward", (long long)T, need, kStaticScratchBytes);
        DeviceGuard dg(dev);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", dev);
        Timer tm;
        const int64_t P = T * layer->cfg.top_k;
        const int w_f32 = w_dtype == EK_F32;
        std::lock_guard<std::mutex> lk(layer->mu);      // the layer's side stream, events and slab table
        std::lock_guard<std::mutex> sk(S.mu);           // the device's scratch array
        hipStream_t s = stream ? (hipStream_t)stream : layer->stream;
        WorkspaceUse use(layer, s);
        EK_TRY(use.begin());
        WorkspaceUse use_scratch(S.ev, &S.busy, s);
        EK_TRY(use_scratch.begin());
        ek_status st = EK_OK;
        // a blocking call sees everything submitted before it (waiting allocates nothing)
        if (!stream) EK_HIP(hipDeviceSynchronize());
        EK_TRY(enqueue_forward(layer, W, x, ids, w, w_f32, T, y, s, false, nullptr, route != nullptr));
        EK_TRY(copy_route_out(layer, W, route, P, EK_DEVICE, s));
        if (!stream) {
            st = finish_blocking(layer, W, s);
            use.synced();
            use_scratch.synced();
        }
        {
            std::lock_guard<std::mutex> sl(layer->stats_mu);
            layer->stats.forward_calls += 1;
            layer->stats.tokens += T;
            layer->stats.pairs += P;
            if (!stream) { layer->stats.last_forward_us = tm.us(); observe_forward(layer, layer->stats.last_forward_us); }
        }
        return st;
    )
}

ek_status ek_layer_pack(ek_layer *layer, const int32_t *ids, int64_t T, const ek_route_out *route,
                        const void *x, void *xp, int32_t mem, void *stream)
{
    EK_GUARDED(
        if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
        if (T < 0 || T > layer->cfg.max_tokens)
            return fail(EK_INVALID_INPUT, "T = %lld outside [0, max_tokens = %lld]", (long long)T,
                        (long long)layer->cfg.max_tokens);
        if (mem != EK_HOST && mem != EK_DEVICE) return fail(EK_INVALID_INPUT, "bad mem %d", mem);
        if (T > 0 && !ids) return fail(EK_INVALID_INPUT, "ids is NULL");
        if (xp && !x) return fail(EK_INVALID_INPUT, "xp requested but x is NULL");
        if (mem == EK_HOST && stream)
            return fail(EK_INVALID_INPUT, "host-memory calls are blocking: stream must be NULL");
        DeviceGuard dg(layer->cfg.device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", layer->cfg.device_id);
        const int64_t H = layer->user_hidden, K = layer->cfg.top_k, P = T * K;   // rows are gathered as the caller has them
        std::lock_guard<std::mutex> lk(layer->mu);
        hipStream_t s = stream ? (hipStream_t)stream : layer->stream;
        WorkspaceUse use(layer, s);
        EK_TRY(use.begin());
        if (mem == EK_DEVICE && !stream) { EK_HIP(hipDeviceSynchronize()); use.device_idle(); }
        const int32_t *d_ids = ids;
        const void *d_x = x;
        void *d_xp = xp;
        if (mem == EK_HOST) {
            EK_TRY(ensure_io_staging(layer));
            EK_TRY(bounce_begin(layer, s, (size_t)P * H * 2 + (size_t)P * 8));
            if (P > 0) EK_TRY(h2d(layer, layer->st_ids, ids, (size_t)P * 4, s));
            d_ids = layer->st_ids;
            if (xp && T > 0) {
                EK_TRY(h2d(layer, layer->st_x, x, (size_t)T * H * 2, s));
                d_x = layer->st_x;
                d_xp = layer->ws.yp;   // [Pmax, H] scratch of the right size
            }
        }
        ek::launch_pack(pack_args(layer, layer->ws, d_ids, P, false), s);
        if (xp) ek::launch_gather(d_x, layer->ws.row_token, P, H * 2, d_xp, s);
        EK_HIP(hipGetLastError());
        if (mem == EK_HOST && xp && P > 0) EK_TRY(d2h(layer, xp, d_xp, (size_t)P * H * 2, s));
        // the rows went into the staging buffer back to back: give a padded layer its zero columns back
        if (layer->padded && mem == EK_HOST && xp && T > 0) EK_HIP(hipMemsetAsync(layer->st_x, 0, (size_t)T * H * 2, s));
        EK_TRY(copy_route_out(layer, layer->ws, route, P, mem, s, false));
        if (!stream) { use.synced(); return finish_blocking(layer, layer->ws, s); }
        return EK_OK;
    )
}

ek_status ek_layer_expert_forward(ek_layer *layer, int32_t expert, const void *x, int64_t n,
                                  void *out, int32_t mem, void *stream)
{
    EK_GUARDED(
        if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
        if (expert < 0 || expert >= layer->cfg.n_experts)
            return fail(EK_INVALID_INPUT, "expert %d outside [0, %d)", expert, layer->cfg.n_experts);
        if (n < 0 || n > layer->Pmax)
            return fail(EK_INVALID_INPUT, "n = %lld outside [0, %lld]", (long long)n,
                        (long long)layer->Pmax);
        if (mem != EK_HOST && mem != EK_DEVICE) return fail(EK_INVALID_INPUT, "bad mem %d", mem);
        if (n > 0 && (!x || !out)) return fail(EK_INVALID_INPUT, "NULL tensor pointer");
        if (mem == EK_HOST && stream)
            return fail(EK_INVALID_INPUT, "host-memory calls are blocking: stream must be NULL");
        DeviceGuard dg(layer->cfg.device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", layer->cfg.device_id);
        const int64_t H = layer->cfg.hidden;
        Timer tm;
        std::lock_guard<std::mutex> lk(layer->mu);
        if (!layer->expert_mem[expert])
            return fail(EK_EXPERT_NOT_FOUND, "expert %d is not loaded", expert);
        hipStream_t s = stream ? (hipStream_t)stream : layer->stream;
        WorkspaceUse use(layer, s);
        EK_TRY(use.begin());
        if (mem == EK_DEVICE && !stream) { EK_HIP(hipDeviceSynchronize()); use.device_idle(); }
        if (n > 0) {
            const void *d_x = x;
            void *d_out = out;
            if (layer->padded) {
                EK_TRY(ensure_io_staging(layer));
                EK_TRY(rows_in(layer, layer->st_x, x, n, mem, s));
                d_x = layer->st_x;
                d_out = layer->st_y;
            } else if (mem == EK_HOST) {
                EK_TRY(ensure_io_staging(layer));
                EK_TRY(bounce_begin(layer, s, (size_t)n * H * 2));
                EK_TRY(h2d(layer, layer->st_x, x, (size_t)n * H * 2, s));
                d_x = layer->st_x;
                d_out = layer->st_y;
            }
            // the ordinary cut's tile items: full 128-row tiles and a remainder of more than 16 rows
            const int64_t wide_items = (n + ek::kWideRows - 1) / ek::kWideRows;
            const bool wide = ek::wide_cut_pays((n >> 7) + ((n & 127) > 16), n, H, layer->cfg.inter) &&
                              wide_items <= layer->ws.list_cap[ek::kListStream];
            ek::launch_single_lists(layer->ws.lists, expert, (int32_t)n, wide, s);
            EK_TRY(enqueue_ffn(layer, layer->ws, d_x, nullptr, d_out, n, 1, s, nullptr, wide ? wide_items : 0, 0, 0, nullptr,
                               wide ? 0 : (n >> 7) + ((n & 127) > 16)));
            if (layer->padded) EK_TRY(rows_out(layer, out, layer->st_y, n, mem, s));
            else if (mem == EK_HOST) EK_TRY(d2h(layer, out, layer->st_y, (size_t)n * H * 2, s));
        }
        if (!stream) {
            EK_HIP(hipStreamSynchronize(s));
            use.synced();
            bounce_flush(layer);
        }
        {
            std::lock_guard<std::mutex> sl(layer->stats_mu);
            layer->stats.expert_forward_calls += 1;
            layer->h_activation[expert] += n;
            if (!stream) observe_forward(layer, tm.us());
        }
        return EK_OK;
    )
}

ek_status ek_layer_describe(ek_layer *layer, int64_t *hidden, int64_t *inter, int32_t *n_experts,
                            int32_t *top_k, int32_t *act_dtype)
{
    if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
    if (hidden) *hidden = layer->user_hidden;
    if (inter) *inter = layer->user_inter;
    if (n_experts) *n_experts = layer->cfg.n_experts;
    if (top_k) *top_k = layer->cfg.top_k;
    if (act_dtype) *act_dtype = layer->cfg.act_dtype;
    return EK_OK;
}

ek_status ek_layer_experts_forward(ek_layer *layer, int32_t n_calls, const int32_t *experts,
                                   const void *const *xs, const int64_t *rows, void *const *outs,
                                   int32_t mem, void *stream)
{
    EK_GUARDED(
        if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
        if (n_calls < 0) return fail(EK_INVALID_INPUT, "n_calls is negative");
        if (n_calls > 0 && (!experts || !xs || !rows || !outs)) return fail(EK_INVALID_INPUT, "NULL argument");
        if (mem != EK_HOST && mem != EK_DEVICE) return fail(EK_INVALID_INPUT, "bad mem %d", mem);
        if (mem == EK_HOST && stream)
            return fail(EK_INVALID_INPUT, "host-memory calls are blocking: stream must be NULL");
        const int64_t H = layer->cfg.hidden;
        int64_t P = 0;
        for (int i = 0; i < n_calls; ++i) {
            if (experts[i] < 0 || experts[i] >= layer->cfg.n_experts)
                return fail(EK_INVALID_INPUT, "call %d: expert %d outside [0, %d)", i, experts[i],
                            layer->cfg.n_experts);
            if (rows[i] < 0 || rows[i] > layer->Pmax - P)
                return fail(EK_INVALID_INPUT, "call %d: rows exceed the layer's capacity of %lld", i,
                            (long long)layer->Pmax);
            if (rows[i] > 0 && (!xs[i] || !outs[i])) return fail(EK_INVALID_INPUT, "call %d: NULL tensor pointer", i);
            P += rows[i];
        }
        DeviceGuard dg(layer->cfg.device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", layer->cfg.device_id);
        Timer tm;
        std::lock_guard<std::mutex> lk(layer->mu);
        for (int i = 0; i < n_calls; ++i)
            if (!layer->expert_mem[experts[i]])
                return fail(EK_EXPERT_NOT_FOUND, "expert %d is not loaded", experts[i]);
        hipStream_t s = stream ? (hipStream_t)stream : layer->stream;
        WorkspaceUse use(layer, s);
        EK_TRY(use.begin());
        if (mem == EK_DEVICE && !stream) { EK_HIP(hipDeviceSynchronize()); use.device_idle(); }
        if (P > 0) {
            // Work lists cut on the host exactly as the pack kernels cut them: a call is one
            // segment (ek_internal.h, "work lists").
            std::vector<ek::WorkItem> items[ek::kNumLists];
            int64_t row0 = 0, tile_items = 0, wide_items = 0, short_items = 0;
            for (int i = 0; i < n_calls; ++i) {
                tile_items += (rows[i] >> 7) + ((rows[i] & 127) > 16);
                wide_items += (rows[i] + ek::kWideRows - 1) / ek::kWideRows;
                short_items += (rows[i] & 127) > 0 && (rows[i] & 127) <= 16;
            }
            // The wide cut spares a batch the tile kernel's long, nearly empty launch.  When the batch
            // also has many short requests, their streaming chain (one pass over an expert's weights
            // each, ~6.5 TB/s) runs beside the tile chain and covers it, and the short items are
            // served faster by the sliced streaming form than by the wide one (64 DeepSeek-V3 int8
            // requests from host memory, 4 rows each but one of 40 / four of 100: 995 / 1500 us cut wide,
            // 890 / 1325 us as tiles beside streams).
            const int wb = layer->w8 ? 1 : 2;
            const double cover_us = (double)short_items * 3.0 * (double)H * (double)layer->cfg.inter * wb / 6.5e6;
            const double tiled_us = ek::tile_call_us(H, layer->cfg.inter);
            const bool wide = ek::wide_cut_pays(tile_items, P, H, layer->cfg.inter) && cover_us < 0.5 * tiled_us &&
                              wide_items <= layer->ws.list_cap[ek::kListStream];
            for (int i = 0; i < n_calls; ++i) {
                const int32_t n = (int32_t)rows[i], full = n >> 7, r = n & 127;
                if (wide) {
                    for (int32_t r0 = 0; r0 < n; r0 += ek::kWideRows)
                        items[ek::kListStream].push_back(
                            ek::WorkItem{experts[i], (int32_t)row0 + r0, std::min<int32_t>(ek::kWideRows, n - r0), 0});
                    row0 += n;
                    continue;
                }
                for (int32_t t = 0; t < full; ++t)
                    items[ek::kListT128].push_back(ek::WorkItem{experts[i], (int32_t)row0 + t * 128, 128, 0});
                const ek::WorkItem rem{experts[i], (int32_t)row0 + full * 128, r, 0};
                if (r > 64) items[ek::kListT128].push_back(rem);
                else if (r > 32) items[ek::kListT64].push_back(rem);
                else if (r > 16) items[ek::kListT32].push_back(rem);
                else if (r > 0) items[ek::kListStream].push_back(rem);
                row0 += n;
            }
            // pinned block: the lists' lengths (16 bytes), the table of the copy kernel that takes them to the
            // device, then the lists
            size_t off[ek::kNumLists + 1];
            off[0] = 256;
            static_assert(16 + sizeof(ek::RowCopy) * (ek::kNumLists + 1) <= 256, "list-copy table");
            for (int l = 0; l < ek::kNumLists; ++l) {
                if ((int64_t)items[l].size() > layer->ws.list_cap[l])
                    return fail(EK_INVALID_INPUT, "too many calls for one launch (work list %d holds %lld items)", l,
                                (long long)layer->ws.list_cap[l]);
                off[l + 1] = off[l] + sizeof(ek::WorkItem) * (size_t)layer->ws.list_cap[l];
            }
            if (!layer->h_items) {
                EK_HIP(hipHostMalloc((void **)&layer->h_items, off[ek::kNumLists], hipHostMallocDefault));
                EK_HIP(hipEventCreateWithFlags(&layer->ev_items, hipEventDisableTiming));
                void *dp = nullptr;
                if (hipHostGetDevicePointer(&dp, layer->h_items, 0) != hipSuccess) { (void)hipGetLastError(); dp = nullptr; }
                layer->d_items = (uint8_t *)dp;
            } else {
                EK_HIP(hipEventSynchronize(layer->ev_items));
            }
            // One copy kernel reads the lists and their lengths where they lie in pinned memory, instead of up to
            // five asynchronous copies (8 DeepSeek-V3 int8 requests of one row: 84.5 -> 83.4 us per call).
            int32_t *cnt = (int32_t *)layer->h_items;
            ek::RowCopy *tab = (ek::RowCopy *)(layer->h_items + 16);
            int n_tab = 0;
            static_assert(sizeof(ek::WorkItem) == 16 && sizeof(int32_t) * ek::kNumLists == 16, "whole 16-byte units");
            for (int l = 0; l < ek::kNumLists; ++l) {
                cnt[l] = (int32_t)items[l].size();
                if (!cnt[l]) continue;
                const size_t bytes = sizeof(ek::WorkItem) * items[l].size();
                memcpy(layer->h_items + off[l], items[l].data(), bytes);
                if (layer->d_items)
                    tab[n_tab++] = ek::RowCopy{layer->d_items + off[l], (uint8_t *)layer->ws.lists.items[l], 0, 0, 1, (int32_t)bytes};
                else
                    EK_HIP(hipMemcpyAsync(layer->ws.lists.items[l], layer->h_items + off[l], bytes, hipMemcpyHostToDevice, s));
            }
            if (layer->d_items) {
                tab[n_tab++] = ek::RowCopy{layer->d_items, (uint8_t *)layer->ws.lists.count, 0, 0, 1, 16};
                ek::launch_rows_copy((const ek::RowCopy *)(layer->d_items + 16), n_tab, s);
                EK_HIP(hipGetLastError());
            } else {
                EK_HIP(hipMemcpyAsync(layer->ws.lists.count, cnt, sizeof(int32_t) * ek::kNumLists, hipMemcpyHostToDevice, s));
            }
            EK_HIP(hipEventRecord(layer->ev_items, s));
            EK_TRY(ensure_io_staging(layer));
            // Many small host requests: their rows are gathered in pinned memory and cross the
            // bus as one transfer each way (an asynchronous copy costs ~5 us of host time per
            // call, as much as the memcpy of a decode-sized request).
            const size_t all_bytes = (size_t)P * H * 2;
            bool one_transfer = false;
            if (mem == EK_HOST && !layer->padded) {
                EK_TRY(bounce_begin(layer, s, all_bytes));
                one_transfer = n_calls > 1 && all_bytes <= layer->pin_cap;
            }
            if (one_transfer) {
                row0 = 0;
                for (int i = 0; i < n_calls; ++i) {
                    if (rows[i]) memcpy(layer->pin_in + row0 * H * 2, xs[i], (size_t)rows[i] * H * 2);
                    row0 += rows[i];
                }
                layer->pin_in_used = all_bytes;
                EK_HIP(hipMemcpyAsync(layer->st_x, layer->pin_in, all_bytes, hipMemcpyHostToDevice, s));
            }
            // Device-memory requests: one copy kernel each way over a table of the requests' rows
            // (64 requests: 128 asynchronous copies cost ~500 us of host time, more than the kernels).
            bool table = mem == EK_DEVICE && n_calls > 1;
            for (int i = 0; i < n_calls && table; ++i)
                table = (((uintptr_t)xs[i] | (uintptr_t)outs[i]) & 15) == 0 || rows[i] == 0;
            if (table && layer->segs_cap < n_calls) {
                EK_HIP(hipEventSynchronize(layer->ev_items));      // (the previous tables have been read)
                if (layer->h_segs) { (void)hipHostFree(layer->h_segs); layer->h_segs = nullptr; layer->segs_cap = 0; }
                const int64_t cap_new = n_calls < 1024 ? 1024 : 2 * (int64_t)n_calls;
                EK_HIP(hipHostMalloc((void **)&layer->h_segs, sizeof(ek::RowCopy) * 2 * (size_t)cap_new, hipHostMallocDefault));
                void *dp = nullptr;
                if (hipHostGetDevicePointer(&dp, layer->h_segs, 0) != hipSuccess) { (void)hipGetLastError(); table = false; }
                layer->d_segs = (ek::RowCopy *)dp;
                layer->segs_cap = table ? cap_new : 0;
            }
            if (table) {
                const int64_t uw = layer->user_hidden * 2;          // bytes of a caller's row
                row0 = 0;
                for (int i = 0; i < n_calls; ++i) {
                    layer->h_segs[i] = ek::RowCopy{(const uint8_t *)xs[i], (uint8_t *)layer->st_x + row0 * H * 2, uw, H * 2,
                                                   (int32_t)rows[i], (int32_t)uw};
                    layer->h_segs[layer->segs_cap + i] = ek::RowCopy{(const uint8_t *)layer->st_y + row0 * H * 2, (uint8_t *)outs[i],
                                                                     H * 2, uw, (int32_t)rows[i], (int32_t)uw};
                    row0 += rows[i];
                }
                ek::launch_rows_copy(layer->d_segs, n_calls, s);
            }
            row0 = 0;
            for (int i = 0; i < n_calls && !one_transfer && !table; ++i) {
                if (layer->padded)
                    EK_TRY(rows_in(layer, (char *)layer->st_x + row0 * H * 2, xs[i], rows[i], mem, s));
                else if (rows[i] && mem == EK_HOST)
                    EK_TRY(h2d(layer, (char *)layer->st_x + row0 * H * 2, xs[i], (size_t)rows[i] * H * 2, s));
                else if (rows[i])
                    EK_HIP(hipMemcpyAsync((char *)layer->st_x + row0 * H * 2, xs[i], (size_t)rows[i] * H * 2,
                                          hipMemcpyDeviceToDevice, s));
                row0 += rows[i];
            }
            int64_t exact[ek::kNumLists];
            for (int l = 0; l < ek::kNumLists; ++l) exact[l] = (int64_t)items[l].size();
            EK_TRY(enqueue_ffn(layer, layer->ws, layer->st_x, nullptr, layer->st_y, P, n_calls, s, nullptr, wide ? wide_items : 0, 0, 0,
                               wide ? nullptr : exact));
            EK_HIP(hipGetLastError());
            row0 = 0;
            if (one_transfer) {
                EK_HIP(hipMemcpyAsync(layer->pin_out, layer->st_y, all_bytes, hipMemcpyDeviceToHost, s));
                layer->pin_out_used = all_bytes;
                for (int i = 0; i < n_calls; ++i) {
                    if (rows[i]) layer->pin_pending.push_back({outs[i], layer->pin_out + row0 * H * 2, (size_t)rows[i] * H * 2});
                    row0 += rows[i];
                }
            }
            if (table) {
                ek::launch_rows_copy(layer->d_segs + layer->segs_cap, n_calls, s);
                EK_HIP(hipGetLastError());
                EK_HIP(hipEventRecord(layer->ev_items, s));         // the tables are free again after this
            }
            for (int i = 0; i < n_calls && !one_transfer && !table; ++i) {
                if (layer->padded)
                    EK_TRY(rows_out(layer, outs[i], (char *)layer->st_y + row0 * H * 2, rows[i], mem, s));
                else if (rows[i] && mem == EK_HOST)
                    EK_TRY(d2h(layer, outs[i], (char *)layer->st_y + row0 * H * 2, (size_t)rows[i] * H * 2, s));
                else if (rows[i])
                    EK_HIP(hipMemcpyAsync(outs[i], (char *)layer->st_y + row0 * H * 2, (size_t)rows[i] * H * 2,
                                          hipMemcpyDeviceToDevice, s));
                row0 += rows[i];
            }
        }
        if (!stream) {
            EK_HIP(hipStreamSynchronize(s));
            use.synced();
            bounce_flush(layer);
        }
        {
            std::lock_guard<std::mutex> sl(layer->stats_mu);
            layer->stats.expert_forward_calls += n_calls;
            for (int i = 0; i < n_calls; ++i) layer->h_activation[experts[i]] += rows[i];
            // the reference observes one duration per request; the requests of a batch share this one
            if (!stream) { const double us = tm.us(); for (int i = 0; i < n_calls; ++i) observe_forward(layer, us); }
        }
        return EK_OK;
    )
}

ek_status ek_layer_get_activation(ek_layer *layer, int64_t *counts)
{
    EK_GUARDED(
        if (!layer || !counts) return fail(EK_INVALID_INPUT, "NULL argument");
        DeviceGuard dg(layer->cfg.device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", layer->cfg.device_id);
        const int E = layer->cfg.n_experts;
        std::lock_guard<std::mutex> lk(layer->mu);
        EK_HIP(hipDeviceSynchronize());   // calls enqueued on caller streams count once they have run
        std::vector<uint64_t> dev(E);
        EK_HIP(hipMemcpy(dev.data(), layer->d_activation, sizeof(uint64_t) * E, hipMemcpyDeviceToHost));
        std::lock_guard<std::mutex> sl(layer->stats_mu);
        for (int e = 0; e < E; ++e) counts[e] = (int64_t)dev[e] + layer->h_activation[e];
        return EK_OK;
    )
}

ek_status ek_layer_get_forward_histogram(ek_layer *layer, ek_histogram *out)
{
    EK_GUARDED(
        if (!layer || !out) return fail(EK_INVALID_INPUT, "NULL argument");
        std::lock_guard<std::mutex> sl(layer->stats_mu);
        *out = layer->forward_hist;
        return EK_OK;
    )
}

ek_status ek_layer_profile(ek_layer *layer, int32_t enable)
{
    EK_GUARDED(
        if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
        DeviceGuard dg(layer->cfg.device_id);
        std::lock_guard<std::mutex> lk(layer->mu);
        if (enable && layer->events.empty()) {
            layer->events.reserve(5 * 1024);
            for (int i = 0; i < 5 * 1024; ++i) {
                hipEvent_t ev;
                EK_HIP(hipEventCreate(&ev));
                layer->events.push_back(ev);
            }
        }
        if (layer->events_used) EK_HIP(hipEventSynchronize(layer->events[layer->events_used - 1]));
        layer->events_used = 0;
        layer->profiling = enable != 0;
        layer->profile_every = enable > 1 ? enable : 1;
        layer->profile_tick = 0;
        std::lock_guard<std::mutex> sl(layer->stats_mu);
        for (double &v : layer->stats.kernel_us) v = 0.0;
        layer->stats.profiled_calls = 0;
        return EK_OK;
    )
}

ek_status ek_layer_get_stats(ek_layer *layer, ek_stats *out)
{
    EK_GUARDED(
        if (!layer || !out) return fail(EK_INVALID_INPUT, "NULL argument");
        DeviceGuard dg(layer->cfg.device_id);
        std::lock_guard<std::mutex> lk(layer->mu);
        std::lock_guard<std::mutex> sl(layer->stats_mu);
        for (size_t i = 0; i + 5 <= layer->events_used; i += 5) {
            hipEvent_t *ev = layer->events.data() + i;
            EK_HIP(hipEventSynchronize(ev[4]));
            for (int k = 0; k < 4; ++k) {
                float ms = 0.f;
                EK_HIP(hipEventElapsedTime(&ms, ev[k], ev[k + 1]));
                layer->stats.kernel_us[k] += 1e3 * ms;
            }
            layer->stats.profiled_calls += 1;
        }
        layer->events_used = 0;
        *out = layer->stats;
        return EK_OK;
    )
}

static void free_chain(ek_chain *c)
{
    if (!c) return;
    (void)hipDeviceSynchronize();
    if (c->exec) (void)hipGraphExecDestroy(c->exec);
    if (c->graph) (void)hipGraphDestroy(c->graph);
    if (c->act[0]) (void)hipFree(c->act[0]);
    if (c->act[1]) (void)hipFree(c->act[1]);
    if (c->act_in) (void)hipFree(c->act_in);
    if (c->d_err) (void)hipFree(c->d_err);
    if (c->h_err) (void)hipHostFree(c->h_err);
    if (c->stream) (void)hipStreamDestroy(c->stream);
    if (c->route_stream) (void)hipStreamDestroy(c->route_stream);
    if (c->ev_begin) (void)hipEventDestroy(c->ev_begin);
    for (hipEvent_t e : c->ev_routed) if (e) (void)hipEventDestroy(e);
    delete c;
}

ek_status ek_chain_create(ek_layer *const *layers, int32_t n_layers, ek_chain **out)
{
    EK_GUARDED(
        if (!out) return fail(EK_INVALID_INPUT, "out is NULL");
        *out = nullptr;
        if (!layers || n_layers < 1 || n_layers > 1024)
            return fail(EK_INVALID_INPUT, "n_layers must be in [1, 1024]");
        for (int i = 0; i < n_layers; ++i) {
            if (!layers[i]) return fail(EK_INVALID_INPUT, "layer %d is NULL", i);
            const ek_cfg &a = layers[0]->cfg, &b = layers[i]->cfg;
            // (equal padded sizes too: layers with one-byte weights pad a small hidden size further)
            if (a.hidden != b.hidden || layers[0]->user_hidden != layers[i]->user_hidden || a.top_k != b.top_k || a.act_dtype != b.act_dtype ||
                a.device_id != b.device_id || a.max_tokens != b.max_tokens)
                return fail(EK_INVALID_INPUT, "layer %d differs from layer 0 in hidden / top_k / "
                            "act_dtype / device / max_tokens", i);
        }
        DeviceGuard dg(layers[0]->cfg.device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", layers[0]->cfg.device_id);
        ek_chain *c = new (std::nothrow) ek_chain();
        if (!c) return fail(EK_OOM, "host allocation failed");
        c->layers.assign(layers, layers + n_layers);
        const size_t act_bytes = (size_t)layers[0]->cfg.max_tokens * layers[0]->cfg.hidden * 2;
        ek_status st = dev_alloc(&c->act[0], act_bytes, "chain activations");
        if (st == EK_OK) st = dev_alloc(&c->act[1], act_bytes, "chain activations");
        if (st == EK_OK && layers[0]->cfg.hidden != layers[0]->user_hidden) {
            // the padding columns of the first layer's input are zero and stay so; every layer writes
            // zeros into those of its output (its padded output channels have zero weights)
            st = dev_alloc(&c->act_in, act_bytes, "chain input");
            if (st == EK_OK && hipMemset(c->act_in, 0, act_bytes) != hipSuccess) st = fail(EK_HIP_ERROR, "hipMemset failed");
            if (st == EK_OK && hipDeviceSynchronize() != hipSuccess) st = fail(EK_HIP_ERROR, "hipDeviceSynchronize failed");
        }
        if (st == EK_OK) st = dev_alloc((void **)&c->d_err, sizeof(int32_t) * n_layers, "chain errors");
        if (st == EK_OK) {
            hipError_t e = hipHostMalloc((void **)&c->h_err, sizeof(int32_t) * n_layers, hipHostMallocDefault);
            if (e == hipSuccess) e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
            std::vector<ek_layer *> uniq(c->layers);
            std::sort(uniq.begin(), uniq.end());
            c->distinct = std::adjacent_find(uniq.begin(), uniq.end()) == uniq.end();
            if (c->distinct && n_layers > 1) {
                if (e == hipSuccess) e = hipStreamCreateWithFlags(&c->route_stream, hipStreamNonBlocking);
                if (e == hipSuccess) e = hipEventCreateWithFlags(&c->ev_begin, hipEventDisableTiming);
                c->ev_routed.assign(n_layers, nullptr);
                for (int i = 1; i < n_layers && e == hipSuccess; ++i)
                    e = hipEventCreateWithFlags(&c->ev_routed[i], hipEventDisableTiming);
            }
            if (e != hipSuccess) st = hip_fail(e, "chain setup");
        }
        if (st != EK_OK) {
            std::string keep = g_last_error;
            free_chain(c);
            g_last_error = keep;
            return st;
        }
        *out = c;
        return EK_OK;
    )
}

// All layer calls of the chain on stream s (eager or under capture).
static ek_status enqueue_chain(ek_chain *c, const void *x, const int32_t *ids, const void *w, int w_f32,
                               int64_t T, void *y, hipStream_t s)
{
    const int L = (int)c->layers.size();
    const int64_t K = c->layers[0]->cfg.top_k;
    const size_t w_es = w_f32 ? 4 : 2;
    const void *in = x;
    if (c->act_in) {
        EK_TRY(rows_in(c->layers[0], c->act_in, x, T, EK_DEVICE, s));
        in = c->act_in;
    }
    // (a chain of a few pairs per layer has no routing halves to run ahead: its layer calls are
    // pair-direct, two kernels each)
    bool pair_direct = true;
    for (int l = 0; l < L; ++l) pair_direct = pair_direct && pair_direct_fits(c->layers[l], T);
    const bool ahead = c->route_stream != nullptr && T > 0 && !pair_direct;
    if (ahead) {
        // layer 0's routing half first, alone
        EK_TRY(enqueue_route(c->layers[0], c->layers[0]->ws, ids, T, s));
        EK_HIP(hipEventRecord(c->ev_begin, s));
    }
    for (int l = 0; l < L; ++l) {
        void *outp = l == L - 1 && !c->act_in ? y : c->act[l & 1];
        ek_layer *ly = c->layers[l];
        // Between layer l's FFN launches and its combine: (l = 0) the other layers' routing halves go
        // to their own stream behind layer 0's, where they run in what layer 0's kernels leave free
        // of the chip (enqueued after layer 0's FFN kernels, so that under capture the tile kernel
        // stays the first successor of layer 0's pack and follows it in its queue); then s
        // waits for layer l + 1's.
        const std::function<ek_status()> mid = [&]() -> ek_status {
            if (l == 0) {
                EK_HIP(hipStreamWaitEvent(c->route_stream, c->ev_begin, 0));
                for (int m = 1; m < L; ++m) {
                    EK_TRY(enqueue_route(c->layers[m], c->layers[m]->ws, ids + (size_t)m * T * K, T, c->route_stream));
                    EK_HIP(hipEventRecord(c->ev_routed[m], c->route_stream));
                }
            }
            if (l + 1 < L) EK_HIP(hipStreamWaitEvent(s, c->ev_routed[l + 1], 0));
            return EK_OK;
        };
        const bool prof = ly->profiling;
        ly->profiling = false;               // no event records inside a chain (capture-safe)
        ek_status st = enqueue_forward(ly, ly->ws, in, ids + (size_t)l * T * K,
                                       (const char *)w + (size_t)l * T * K * w_es, w_f32, T, outp, s, ahead,
                                       ahead ? &mid : nullptr, !pair_direct);
        ly->profiling = prof;
        EK_TRY(st);
        // collect the layer's error word with a copy kernel-free D2D memcpy node
        EK_HIP(hipMemcpyAsync(c->d_err + l, ly->ws.err, sizeof(int32_t), hipMemcpyDeviceToDevice, s));
        in = outp;
    }
    if (c->act_in) EK_TRY(rows_out(c->layers[0], y, in, T, EK_DEVICE, s));
    return EK_OK;
}

ek_status ek_chain_forward(ek_chain *chain, const void *x, const int32_t *ids, const void *w,
                           int32_t w_dtype, int64_t T, void *y, int32_t use_graph, void *stream)
{
    EK_GUARDED(
        if (!chain) return fail(EK_INVALID_INPUT, "chain is NULL");
        ek_layer *l0 = chain->layers[0];
        if (T < 0 || T > l0->cfg.max_tokens)
            return fail(EK_INVALID_INPUT, "T = %lld outside [0, max_tokens = %lld]", (long long)T,
                        (long long)l0->cfg.max_tokens);
        if (w_dtype != l0->cfg.act_dtype && w_dtype != EK_F32)
            return fail(EK_INVALID_INPUT, "w_dtype must be the activation dtype or EK_F32 (got %d)", w_dtype);
        if (T > 0 && (!x || !ids || !w || !y)) return fail(EK_INVALID_INPUT, "NULL tensor pointer");
        DeviceGuard dg(l0->cfg.device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", l0->cfg.device_id);
        std::lock_guard<std::mutex> ck(chain->mu);
        // every layer's workspace is ours for the call; locked in address order so that chains
        // that share layers cannot deadlock each other
        std::vector<ek_layer *> order(chain->layers);
        std::sort(order.begin(), order.end());
        order.erase(std::unique(order.begin(), order.end()), order.end());
        std::vector<std::unique_lock<std::mutex>> locks;
        for (ek_layer *ly : order) locks.emplace_back(ly->mu);
        hipStream_t s = stream ? (hipStream_t)stream : chain->stream;
        // every layer's workspace is used on s: eagerly, or by the replay of the graph
        std::vector<std::unique_ptr<WorkspaceUse>> uses;
        for (ek_layer *ly : order) {
            uses.emplace_back(new WorkspaceUse(ly, s));
            EK_TRY(uses.back()->begin());
        }
        const int w_f32 = w_dtype == EK_F32;
        const int L = (int)chain->layers.size();
        if (!stream) { EK_HIP(hipDeviceSynchronize()); for (auto &u : uses) u->device_idle(); }
        if (!use_graph) {
            EK_TRY(enqueue_chain(chain, x, ids, w, w_f32, T, y, s));
        } else {
            // a shared expert adds launches to its layer: part of the key
            std::vector<int64_t> shared(L);
            for (int l = 0; l < L; ++l)
                shared[l] = chain->layers[l]->expert_mem[chain->layers[l]->cfg.n_experts] != nullptr
                                ? chain->layers[l]->shared_inter : -1;
            const bool same = chain->exec && chain->k_x == x && chain->k_ids == ids && chain->k_w == w &&
                              chain->k_y == y && chain->k_T == T && chain->k_wdt == w_dtype &&
                              chain->k_shared == shared;
            if (!same) {
                if (chain->exec) { (void)hipGraphExecDestroy(chain->exec); chain->exec = nullptr; }
                if (chain->graph) { (void)hipGraphDestroy(chain->graph); chain->graph = nullptr; }
                // capture on the chain's own stream, never on the caller's
                EK_HIP(hipStreamBeginCapture(chain->stream, hipStreamCaptureModeThreadLocal));
                ek_status st = enqueue_chain(chain, x, ids, w, w_f32, T, y, chain->stream);
                hipGraph_t g = nullptr;
                hipError_t e = hipStreamEndCapture(chain->stream, &g);
                if (st != EK_OK) { if (g) (void)hipGraphDestroy(g); return st; }
                if (e != hipSuccess) return hip_fail(e, "hipStreamEndCapture");
                chain->graph = g;
                EK_HIP(hipGraphInstantiate(&chain->exec, g, nullptr, nullptr, 0));
                chain->k_x = x; chain->k_ids = ids; chain->k_w = w; chain->k_y = y;
                chain->k_T = T; chain->k_wdt = w_dtype; chain->k_shared = shared;
            }
            EK_HIP(hipGraphLaunch(chain->exec, s));
        }
        for (ek_layer *ly : chain->layers) {
            std::lock_guard<std::mutex> sl(ly->stats_mu);
            ly->stats.forward_calls += 1;
            ly->stats.tokens += T;
            ly->stats.pairs += T * ly->cfg.top_k;
        }
        if (!stream) {
            EK_HIP(hipMemcpyAsync(chain->h_err, chain->d_err, sizeof(int32_t) * L, hipMemcpyDeviceToHost, s));
            EK_HIP(hipStreamSynchronize(s));
            for (auto &u : uses) u->synced();
            int32_t err = 0;
            for (int l = 0; l < L; ++l) err |= chain->h_err[l];
            return err_to_status(err);
        }
        return EK_OK;
    )
}

ek_status ek_chain_destroy(ek_chain *chain)
{
    EK_GUARDED(
        if (!chain) return fail(EK_INVALID_INPUT, "chain is NULL");
        DeviceGuard dg(chain->layers[0]->cfg.device_id);
        { std::lock_guard<std::mutex> ck(chain->mu); }
        free_chain(chain);
        return EK_OK;
    )
}

ek_status ek_expert_create(const ek_cfg *cfg, int64_t max_rows, const ek_weight_desc *up,
                           const ek_weight_desc *gate, const ek_weight_desc *down, ek_expert **out)
{
    EK_GUARDED(
        if (!out) return fail(EK_INVALID_INPUT, "out is NULL");
        *out = nullptr;
        if (!cfg) return fail(EK_INVALID_INPUT, "cfg is NULL");
        ek_cfg c = *cfg;
        c.n_experts = 1;
        c.top_k = 1;
        c.max_tokens = max_rows;
        EK_TRY(validate_cfg(&c));
        DeviceGuard dg(c.device_id);
        if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", c.device_id);
        ek_layer *L = nullptr;
        EK_TRY(create_layer(&c, max_rows, &L));
        ek_status st;
        {
            std::lock_guard<std::mutex> lk(L->load_mu);
            if (L->padded && (!up || !gate || !down)) st = fail(EK_WEIGHT_NOT_FOUND, "a weight matrix is missing");
            else st = L->padded ? set_expert_padded(L, 0, up, gate, down) : set_expert_locked(L, 0, up, gate, down);
        }
        if (st != EK_OK) {
            std::string keep = g_last_error;
            free_layer(L);
            g_last_error = keep;
            return st;
        }
        ek_expert *x = new (std::nothrow) ek_expert();
        if (!x) { free_layer(L); return fail(EK_OOM, "host allocation failed"); }
        x->layer = L;
        *out = x;
        return EK_OK;
    )
}

ek_status ek_expert_forward(ek_expert *expert, const void *x, int64_t n, void *out, int32_t mem,
                            void *stream)
{
    if (!expert || !expert->layer) return fail(EK_INVALID_INPUT, "expert is NULL");
    return ek_layer_expert_forward(expert->layer, 0, x, n, out, mem, stream);
}

ek_status ek_expert_shape(ek_expert *expert, int64_t *hidden, int64_t *inter)
{
    if (!expert || !expert->layer || !hidden || !inter) return fail(EK_INVALID_INPUT, "NULL argument");
    *hidden = expert->layer->user_hidden;
    *inter = expert->layer->user_inter;
    return EK_OK;
}

ek_status ek_expert_destroy(ek_expert *expert)
{
    EK_GUARDED(
        if (!expert) return fail(EK_INVALID_INPUT, "expert is NULL");
        ek_status st = expert->layer ? ek_layer_destroy(expert->layer) : EK_OK;
        delete expert;
        return st;
    )
}

}  // extern "C"

namespace {

ek_status check_router(ek_layer *L, const ek_router_cfg *r)
{
    if (!r) return fail(EK_INVALID_INPUT, "router cfg is NULL");
    const int E = L->cfg.n_experts, K = L->cfg.top_k;
    if (r->kind < EK_ROUTER_SOFTMAX_TOPK || r->kind > EK_ROUTER_SIGMOID_GROUP)
        return fail(EK_INVALID_INPUT, "unknown router kind %d", r->kind);
    if (r->logits_dtype != EK_BF16 && r->logits_dtype != EK_F16 && r->logits_dtype != EK_F32)
        return fail(EK_INVALID_INPUT, "logits_dtype must be EK_BF16, EK_F16 or EK_F32 (got %d)", r->logits_dtype);
    if (r->w_dtype != L->cfg.act_dtype && r->w_dtype != EK_F32)
        return fail(EK_INVALID_INPUT, "router w_dtype must be the activation dtype or EK_F32 (got %d)", r->w_dtype);
    if (K > 64) return fail(EK_INVALID_INPUT, "the router kernel takes top_k <= 64 (layer has %d)", K);
    if (r->kind == EK_ROUTER_SIGMOID_GROUP) {
        if (r->n_group < 1 || r->n_group > 64 || E % r->n_group)
            return fail(EK_INVALID_INPUT, "n_group = %d must divide n_experts = %d and be in [1, 64]", r->n_group, E);
        const int G = E / r->n_group;
        if (G < 2) return fail(EK_INVALID_INPUT, "groups of %d expert(s): the group score needs two", G);
        if (r->topk_group < 1 || r->topk_group > r->n_group || (int64_t)r->topk_group * G < K)
            return fail(EK_INVALID_INPUT, "topk_group = %d must be in [1, n_group] and keep at least top_k experts",
                        r->topk_group);
        if (!(r->routed_scaling == r->routed_scaling)) return fail(EK_INVALID_INPUT, "routed_scaling is NaN");
    } else if (r->bias) {
        return fail(EK_INVALID_INPUT, "a correction bias belongs to EK_ROUTER_SIGMOID_GROUP only");
    }
    return EK_OK;
}

ek_status ensure_router_ws(ek_layer *L, bool host)
{
    const int64_t T = L->cfg.max_tokens, K = L->cfg.top_k, E = L->cfg.n_experts;
    if (!L->rt_ids) {
        EK_TRY(dev_alloc((void **)&L->rt_ids, (size_t)T * K * 4, "router ids"));
        EK_TRY(dev_alloc(&L->rt_w, (size_t)T * K * 4, "router weights"));
    }
    if (host && !L->st_logits) {
        EK_TRY(dev_alloc(&L->st_logits, (size_t)T * E * 4, "logits staging"));
        EK_TRY(dev_alloc((void **)&L->st_bias, (size_t)E * 4, "bias staging"));
    }
    return EK_OK;
}

// router on stream s; logits / bias are device addresses
ek_status enqueue_router(ek_layer *L, const ek_router_cfg *r, const void *logits, const float *bias, int64_t T,
                         int32_t *ids, void *w, hipStream_t s)
{
    ek::RouterArgs a;
    a.logits = logits; a.logits_dt = r->logits_dtype; a.bias = bias; a.T = T;
    a.E = L->cfg.n_experts; a.K = L->cfg.top_k; a.kind = r->kind; a.renorm = r->renorm;
    a.n_group = r->n_group; a.topk_group = r->topk_group;
    a.mask_neg_inf = (r->flags & EK_ROUTER_MASK_NEG_INF) != 0;
    a.routed_scaling = r->routed_scaling; a.ids = ids; a.w = w; a.w_dt = r->w_dtype;
    EK_HIP(ek::launch_router(a, s));
    return EK_OK;
}

// shared body of ek_layer_route (x == y == nullptr) and ek_layer_forward_logits
ek_status route_and_forward(ek_layer *layer, const void *x, const void *logits, const ek_router_cfg *rcfg,
                            int64_t T, void *y, int32_t *ids_out, void *w_out, const ek_route_out *route,
                            int32_t mem, void *stream, bool forward)
{
    if (!layer) return fail(EK_INVALID_INPUT, "layer is NULL");
    EK_TRY(check_router(layer, rcfg));
    if (T < 0 || T > layer->cfg.max_tokens)
        return fail(EK_INVALID_INPUT, "T = %lld outside [0, max_tokens = %lld]", (long long)T,
                    (long long)layer->cfg.max_tokens);
    if (mem != EK_HOST && mem != EK_DEVICE) return fail(EK_INVALID_INPUT, "bad mem %d", mem);
    if (T > 0 && (!logits || (forward && (!x || !y)) || (!forward && (!ids_out || !w_out))))
        return fail(EK_INVALID_INPUT, "NULL tensor pointer");
    if (mem == EK_HOST && stream)
        return fail(EK_INVALID_INPUT, "host-memory calls are blocking: stream must be NULL");
    DeviceGuard dg(layer->cfg.device_id);
    if (!dg.ok) return fail(EK_HIP_ERROR, "hipSetDevice(%d) failed", layer->cfg.device_id);
    Timer tm;
    const int64_t H = layer->cfg.hidden, K = layer->cfg.top_k, E = layer->cfg.n_experts, P = T * K;
    const int w_f32 = rcfg->w_dtype == EK_F32;
    const size_t w_bytes = (size_t)P * (w_f32 ? 4 : 2);
    const size_t l_bytes = (size_t)T * E * (rcfg->logits_dtype == EK_F32 ? 4 : 2);
    std::lock_guard<std::mutex> lk(layer->mu);
    hipStream_t s = stream ? (hipStream_t)stream : layer->stream;
    WorkspaceUse use(layer, s);
    EK_TRY(use.begin());
    if (mem == EK_DEVICE && !stream) { EK_HIP(hipDeviceSynchronize()); use.device_idle(); }
    EK_TRY(ensure_router_ws(layer, mem == EK_HOST));
    const void *d_logits = logits, *d_x = x;
    const float *d_bias = (const float *)rcfg->bias;
    void *d_y = y;
    if (mem == EK_HOST) {
        if (forward) EK_TRY(ensure_io_staging(layer));
        EK_TRY(bounce_begin(layer, s, l_bytes + (size_t)T * H * 2 + (size_t)E * 4));
        if (T > 0) {
            EK_TRY(h2d(layer, layer->st_logits, logits, l_bytes, s));
            if (forward && !layer->padded) EK_TRY(h2d(layer, layer->st_x, x, (size_t)T * H * 2, s));
        }
        if (rcfg->bias) {
            EK_TRY(h2d(layer, layer->st_bias, rcfg->bias, (size_t)E * 4, s));
            d_bias = layer->st_bias;
        }
        d_logits = layer->st_logits;
        d_x = layer->st_x;
        d_y = layer->st_y;
    }
    if (forward && layer->padded) {
        EK_TRY(ensure_io_staging(layer));
        EK_TRY(rows_in(layer, layer->st_x, x, T, mem, s));
        d_x = layer->st_x;
        d_y = layer->st_y;
    }
    EK_TRY(enqueue_router(layer, rcfg, d_logits, d_bias, T, layer->rt_ids, layer->rt_w, s));
    auto give = [&](void *dst, const void *src, size_t bytes) -> ek_status {
        if (mem == EK_HOST) return d2h(layer, dst, src, bytes, s);
        EK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s));
        return EK_OK;
    };
    if (P > 0 && ids_out) EK_TRY(give(ids_out, layer->rt_ids, (size_t)P * 4));
    if (P > 0 && w_out) EK_TRY(give(w_out, layer->rt_w, w_bytes));
    ek_status st = EK_OK;
    if (forward) {
        EK_TRY(enqueue_forward(layer, layer->ws, d_x, layer->rt_ids, layer->rt_w, w_f32, T, d_y, s, false, nullptr, route != nullptr));
        if (layer->padded) EK_TRY(rows_out(layer, y, layer->st_y, T, mem, s));
        else if (mem == EK_HOST && T > 0) EK_TRY(d2h(layer, y, layer->st_y, (size_t)T * H * 2, s));
        EK_TRY(copy_route_out(layer, layer->ws, route, P, mem, s));
        if (!stream) { st = finish_blocking(layer, layer->ws, s); use.synced(); }
        std::lock_guard<std::mutex> sl(layer->stats_mu);
        layer->stats.forward_calls += 1;
        layer->stats.tokens += T;
        layer->stats.pairs += P;
        if (!stream) { layer->stats.last_forward_us = tm.us(); observe_forward(layer, layer->stats.last_forward_us); }
    } else if (!stream) {
        EK_HIP(hipStreamSynchronize(s));
        use.synced();
        bounce_flush(layer);
    }
    return st;
}

}  // namespace

extern "C" {

ek_status ek_layer_route(ek_layer *layer, const void *logits, const ek_router_cfg *router, int64_t T,
                         int32_t *ids, void *w, int32_t mem, void *stream)
{
    EK_GUARDED(return route_and_forward(layer, nullptr, logits, router, T, nullptr, ids, w, nullptr, mem, stream, false);)
}

ek_status ek_layer_forward_logits(ek_layer *layer, const void *x, const void *logits, const ek_router_cfg *router,
                                  int64_t T, void *y, int32_t *ids, void *w, const ek_route_out *route,
                                  int32_t mem, void *stream)
{
    EK_GUARDED(return route_and_forward(layer, x, logits, router, T, y, ids, w, route, mem, stream, true);)
}

}  // extern "C"
