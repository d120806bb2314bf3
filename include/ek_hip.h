/*
 * ek_hip.h -- C ABI of libek_hip.so, an MI355X (gfx950) expert-computation
 * backend for Expert Kit.
 *
 * The reference has no FFI on this path: the seam is the Rust trait
 * `Expert<T>` (ek-computation/src/ffn/meta.rs:30-39), the dispatch enum
 * `ExpertBackend` (ek-computation/src/ffn/mod.rs:17-53) and the worker's
 * registry `ExpertDB` (ek-computation/src/worker/manager.rs:14-88).  Every
 * entry point below names the reference item it stands behind, so that a Rust
 * `HipFFN` can implement the trait with `extern "C"` calls only.
 *
 * Conventions
 *  - plain C types only; handles are opaque and never dereferenced by callers;
 *  - every function returns ek_status and never throws, aborts or unwinds;
 *    ek_last_error() gives a thread-local message for the last failure;
 *  - tensors are row-major and contiguous; `mem` says whether the pointers of
 *    a call are host (EK_HOST) or device (EK_DEVICE) addresses;
 *  - the caller owns every input/output buffer, the library owns weights and
 *    workspace; weight bytes are copied (and re-tiled) by set_expert, so the
 *    source buffer may be released as soon as the call returns;
 *  - `stream` is a hipStream_t passed as void*.  NULL means "run on the
 *    library's own stream and return after the work has completed".  With a
 *    non-NULL stream and device pointers the call only enqueues work.  One
 *    exception: the first call that forks work to a side stream on a stream
 *    the layer has not seen before waits for that stream once on the host (a
 *    few hundred microseconds: it times an idle kernel alone and beside itself
 *    to find a side stream whose kernels really run beside the caller's);
 *    the choice is remembered per stream handle;
 *  - all entry points may be called from any thread.  A layer has one
 *    workspace (routing tables, work lists, packed intermediates).  Host code
 *    that uses it runs under the layer's lock; on the device, every call makes
 *    its stream wait for the end of the last enqueue-only call on the layer
 *    (an event recorded when that call returned), so calls on different
 *    streams run one after another in the order they were made and never
 *    overlap in the workspace.  Exception: a call made while `stream` is under
 *    capture by the caller neither waits for nor records that event; replays
 *    of the captured graph use the workspace like the call they record, and
 *    ordering them against other work on the same layer is the caller's part.
 */
#ifndef EK_HIP_H
#define EK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Mirrors the variants of EKError that this path can raise
 * (ek-base/src/error.rs:12-72). */
typedef enum ek_status {
    EK_OK = 0,
    EK_INVALID_INPUT = 1,    /* EKError::InvalidInput: bad shape / dtype / pointer / id */
    EK_EXPERT_NOT_FOUND = 2, /* EKError::ExpertNotFound: pair routed to an unloaded expert */
    EK_WEIGHT_NOT_FOUND = 3, /* EKError::ExpertWeightNotFound: missing up/gate/down or scale */
    EK_OOM = 4,              /* device or host allocation failed */
    EK_HIP_ERROR = 5,        /* a HIP runtime call failed */
    EK_INTERNAL = 6          /* anything else (caught exception, broken invariant) */
} ek_status;

/* Element types (ek-computation/src/backend/mod.rs:7-16 and
 * backend/torch/tch_safetensors.rs:12-46 list the reference's). */
typedef enum ek_dtype {
    EK_BF16 = 0,
    EK_F16 = 1,
    EK_F32 = 2,
    EK_I8 = 3,
    EK_F8E4M3 = 4 /* OCP e4m3fn, DType::Float8e4m3fn (backend/mod.rs:13): a source type of
                     block-scaled tensors, and the type an fp8 layer keeps them in (ek_cfg.w_dtype) */
} ek_dtype;

typedef enum ek_mem { EK_HOST = 0, EK_DEVICE = 1 } ek_mem;

typedef enum ek_scale_kind {
    EK_SCALE_NONE = 0,
    EK_SCALE_PER_CHANNEL = 1, /* one scale per output row: W[n,:] = q[n,:] * scale[n] */
    /* one scale per 128x128 block, scale [ceil(rows/128), ceil(cols/128)] (the
     * `weight_scale_inv` tensors of DeepSeek Block-INT8 / FP8 checkpoints).  The weights are
     * dequantised once at load to the layer's 16-bit type, exactly as w8a16_activate does
     * (ffn/expert_torch.rs:24-53): W[r,c] = rne(f32(q[r,c]) * s[r/128, c/128]) -- for a layer
     * whose w_dtype is its act_dtype.  A layer whose w_dtype is EK_F8E4M3 takes EK_F8E4M3
     * tensors with these scales only, keeps both as they are and applies the same formula in
     * the kernels. */
    EK_SCALE_BLOCK128 = 2
} ek_scale_kind;

/* Stands for EKInstance{hidden, intermediate, backend} (ek-computation/src/x.rs:27-32)
 * plus the inference settings it is filled from (ek-base/src/config.rs:26-31). */
typedef struct ek_cfg {
    int64_t hidden;     /* H: a positive multiple of 8.  The kernels take multiples of 64 (at least 128
                           with one-byte weights); other sizes (the reference's toy models: ds-tiny has
                           hidden 16, intermediate 8) are served zero-padded: the weights once at load,
                           every call's rows through the layer's staging buffers, also for device
                           memory (a chain stages its first input and last output only).  Same results. */
    int64_t inter;      /* I  (moe_intermediate_size): any positive size, padded likewise */
    int32_t n_experts;  /* E  experts owned by one layer object */
    int32_t top_k;      /* K  slots per token */
    int32_t act_dtype;  /* ek_dtype of x, y and the gate weights: EK_BF16 or EK_F16 */
    int32_t w_dtype;    /* ek_dtype weights are kept in: act_dtype; EK_I8 (W8A16, one scale per
                           output channel); or EK_F8E4M3: the checkpoint's fp8 bytes with their
                           128x128 block scales, dequantised in the kernels with the arithmetic
                           of w8a16_activate (ffn/expert_torch.rs:24-53) -- half the HBM bytes of
                           dequantising at load; hidden, inter <= 8192 */
    int64_t max_tokens; /* largest T a forward call will pass */
    int32_t device_id;  /* HIP device ordinal */
    int32_t flags;      /* 0, or EK_CFG_BLOCK_SCALES */
} ek_cfg;
/* With w_dtype EK_I8: the weights are the int8 tensors of a Block-INT8 checkpoint, kept with
 * their 128x128 block scales like the fp8 form (EK_F8E4M3 implies it). */
#define EK_CFG_BLOCK_SCALES 1

/* One weight matrix of ExpertWeight<T> (ek-computation/src/ffn/meta.rs:10-23),
 * row-major [rows = out_features, cols = in_features] as HF nn.Linear stores
 * it.  For EK_I8 weights `scale` holds `rows` per-output-channel scales. */
typedef struct ek_weight_desc {
    const void *ptr;
    int64_t rows;
    int64_t cols;
    int32_t dtype;       /* EK_BF16 / EK_F16 / EK_F32 (cast on load, as
                            TorchFFN::load_module does, ffn/expert_torch.rs:61-78), EK_I8, or
                            EK_F8E4M3 (block-scaled only) */
    int32_t mem;         /* ek_mem of ptr and scale */
    const void *scale;   /* NULL unless scale_kind != EK_SCALE_NONE */
    int32_t scale_dtype; /* EK_BF16, EK_F16 or EK_F32 */
    int32_t scale_kind;  /* ek_scale_kind */
} ek_weight_desc;

/* Optional routing tables of a forward call: the dense form of
 * NaiveExecutor::pending_egress (ek-computation/src/controller/executor.rs:54,283-299).
 * Any pointer may be NULL.  Memory space = the call's `mem`. */
typedef struct ek_route_out {
    int32_t *counts;   /* [E]   pairs per expert */
    int32_t *offsets;  /* [E+1] exclusive scan of counts */
    int32_t *perm;     /* [T*K] packed position -> flat pair index t*K+k */
    int32_t *inv_perm; /* [T*K] flat pair index -> packed position */
    void *expert_out;  /* [T*K, hidden] every pair's expert output before the weighted sum, in packed
                        * order (row j belongs to pair perm[j]; activation dtype): the rows
                        * NaiveExecutor::scatter places into [T, K, H] (executor.rs:203-252).  Calls
                        * that run the experts only (not ek_layer_pack). */
} ek_route_out;

/* Counters the worker shell feeds into its Prometheus series
 * (ek-computation/src/metrics.rs:47-71; worker/server.rs:39-63). */
typedef struct ek_stats {
    int64_t forward_calls;
    int64_t tokens;
    int64_t pairs;
    int64_t expert_forward_calls;
    double last_forward_us; /* host wall time of the last blocking forward */
    /* filled only while profiling is on (ek_layer_profile): device time between
     * HIP events recorded around the four phases of ek_layer_forward, summed
     * over profiled_calls calls.  [0] pack, [1] up/gate + SwiGLU, [2] down, [3] combine */
    double kernel_us[4];
    int64_t profiled_calls;
} ek_stats;

typedef struct ek_layer ek_layer;
typedef struct ek_expert ek_expert;

/* Expert::backend() (ffn/meta.rs:34): returns "hip". */
const char *ek_backend_name(void);

/* Thread-local text of the last error raised on the calling thread. */
const char *ek_last_error(void);

/* Number of visible HIP devices (0 if none); never fails. */
int32_t ek_device_count(void);

/* ---- layer object: the E experts of one MoE layer, resident in HBM --------
 * Stands for the worker's ExpertDB (worker/manager.rs:14-88) restricted to one
 * layer: insert = set_expert, remove = remove_expert, has/loaded = has_expert. */
ek_status ek_layer_create(const ek_cfg *cfg, ek_layer **out);
ek_status ek_layer_destroy(ek_layer *layer);

/* Expert index that names the layer's shared expert in ek_layer_set_expert /
 * remove_expert / has_expert / set_expert_safetensors.  DeepSeek-V3 adds
 * shared_experts(x) to the routed result for every token
 * (expertkit_torch/models/deepseek_v3/model.py:57-61,152); the reference runs
 * it on the attention side.  Once loaded here it is one more segment of the
 * grouped launch (all T tokens, gate weight 1) and ek_layer_forward returns
 * round(routed + shared) in the activation dtype.  Its intermediate size may
 * differ from the routed experts' (moe_intermediate_size * n_shared_experts:
 * DeepSeek-V2-Lite has two shared experts): a multiple of 64, at least 128 with
 * one-byte weights; its segment then gets launches of its own beside the routed
 * pairs'.  (A layer whose own sizes need padding takes a shared expert of the
 * routed experts' shape only.) */
#define EK_SHARED_EXPERT (-1)

/* ExpertDB::insert after ExpertBackend::build (ffn/mod.rs:23-36;
 * worker/x.rs:13-34): copies the three matrices to HBM in the kernels' tiled
 * layout, casting to cfg.w_dtype.  Shapes must be up,gate [I,H], down [H,I].
 * A NULL descriptor or NULL data pointer gives EK_WEIGHT_NOT_FOUND
 * (ExpertWeight::from_safetensor, ffn/meta.rs:56-75). */
ek_status ek_layer_set_expert(ek_layer *layer, int32_t expert, const ek_weight_desc *up,
                              const ek_weight_desc *gate, const ek_weight_desc *down);

/* ExpertDB::remove (worker/manager.rs:69-72). */
ek_status ek_layer_remove_expert(ek_layer *layer, int32_t expert);

/* ExpertDB::has (worker/manager.rs:52-55): *loaded = 1 or 0. */
ek_status ek_layer_has_expert(ek_layer *layer, int32_t expert, int32_t *loaded);

/* Whole layer in one call: what today is spread over
 * break_down_to_egress + assemble_seq_tensors (controller/executor.rs:283-299,112-133),
 * one EKInstanceGate::forward per expert (worker/core.rs:47-74 ->
 * ffn/expert_torch.rs:80-85), the collection loop + output
 * (controller/executor.rs:203-252) and the weighted sum (qwen3_moe.py:102-104).
 *   x   [T,H] act_dtype        ids [T,K] int32 in [0,E)
 *   w   [T,K] w_dtype: act_dtype (Qwen3 shim) or EK_F32 (DeepSeek shim)
 *   y   [T,H] act_dtype        route: optional routing tables (may be NULL)
 * T == 0 is legal and does nothing.  An id outside [0,E) gives
 * EK_INVALID_INPUT, a pair routed to an unloaded expert EK_EXPERT_NOT_FOUND
 * (both reported by blocking calls; y is then unspecified).
 * With device pointers and a stream the call only enqueues (kernels, and events
 * on a side stream of the library's that it forks from and joins to `stream`):
 * it may be captured into the caller's HIP graph, whose grids depend on T only.
 * A call of at most 16 pairs (one or two tokens at top-8) that asks for no
 * routing tables (route == NULL), on a layer with top-k <= 8 (a shared expert
 * of the routed experts' width included), is two kernel launches: no pack and no combine kernel (same results,
 * same errors, same activation counts). */
ek_status ek_layer_forward(ek_layer *layer, const void *x, const int32_t *ids, const void *w,
                           int32_t w_dtype, int64_t T, void *y, const ek_route_out *route,
                           int32_t mem, void *stream);

/* ek_layer_forward for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
 * the reference.  Same arguments, results (bit for bit) and errors as ek_layer_forward with
 * device pointers, but the call's workspace (routing tables, work lists, the packed
 * intermediates h [P+T, I] and y' [P+T, H]) is laid out in a static device array of
 * EK_STATIC_SCRATCH_BYTES that each GPU holds until the process ends, and the call runs no
 * hipMalloc / hipFree or other allocating routine.  A call whose workspace does not fit
 * (roughly (T*K + T) * (H + I) * 2 bytes plus tables; DeepSeek-V3 shape: up to 192 tokens of
 * top-8) fails with EK_INVALID_INPUT and a message that gives the bytes needed.  x, ids, w, y
 * and route are device pointers; hidden and inter must be multiples of 64 (128 with one-byte
 * weights).  All layers on a GPU share that GPU's array, which keeps the last call's contents
 * (every call writes what it reads; nothing needs clearing): the library orders calls through
 * this entry point on one GPU one after another on the device (as it does for a layer's own
 * workspace), except calls made while `stream` is under capture -- replays of such graphs that
 * overlap on one GPU race. */
#define EK_STATIC_SCRATCH_BYTES (32u << 20)
ek_status ek_layer_forward_static(ek_layer *layer, const void *x, const int32_t *ids, const void *w,
                                  int32_t w_dtype, int64_t T, void *y, const ek_route_out *route,
                                  void *stream);

/* Routing only: the pack step of ek_layer_forward, plus (if xp != NULL) the
 * gather Xp[j,:] = x[perm[j]/K,:] of assemble_seq_tensors
 * (controller/executor.rs:112-133).  x may be NULL when xp is NULL. */
ek_status ek_layer_pack(ek_layer *layer, const int32_t *ids, int64_t T, const ek_route_out *route,
                        const void *x, void *xp, int32_t mem, void *stream);

/* One expert, one call: ExpertBackend::forward -> Expert::forward
 * (ffn/mod.rs:39-53; ffn/meta.rs:37) as EKInstanceGate::forward uses it
 * (worker/core.rs:55-59).  x [n,H] -> out [n,H], both act_dtype.  n may
 * exceed cfg.max_tokens * top_k only if it still fits the workspace. */
ek_status ek_layer_expert_forward(ek_layer *layer, int32_t expert, const void *x, int64_t n,
                                  void *out, int32_t mem, void *stream);

/* Geometry of a layer handle (what EKInstance carries: x.rs:27-32). Any out pointer may be NULL. */
ek_status ek_layer_describe(ek_layer *layer, int64_t *hidden, int64_t *inter, int32_t *n_experts,
                            int32_t *top_k, int32_t *act_dtype);

/* Several per-expert calls as ONE grouped launch.  The controller fires one
 * ForwardReq per expert concurrently (controller/executor.rs:141-195) and the
 * worker answers each with Expert::forward (worker/core.rs:55-59); a worker
 * that collects the concurrent requests hands them over together:
 *   call i: xs[i] [rows[i], H] -> outs[i] [rows[i], H], expert experts[i].
 * A row's result depends only on the row, the expert and the kernel family its
 * call is cut for: calls of at most 16 rows always take the weight-streaming
 * kernel and give the same bits alone or batched; longer calls take it too when
 * the whole launch is small (a lone expert with up to a few hundred rows), the
 * MFMA tile kernel otherwise, and the two differ in accumulation order (both
 * within the parity tolerance).
 * The same expert may appear more than once, any number of times; sum(rows) is
 * bounded like n of ek_layer_expert_forward (and one launch takes at most 65535
 * calls of up to 16 rows).  All pointers of one call share `mem`. */
ek_status ek_layer_experts_forward(ek_layer *layer, int32_t n_calls, const int32_t *experts,
                                   const void *const *xs, const int64_t *rows, void *const *outs,
                                   int32_t mem, void *stream);

/* ---- wire format of the worker contract ---------------------------------------
 * Expert ids are "{model}/l{layer}-e{expert}": ExpertKey::from_expert_id and
 * as_object_key (ek-db/src/safetensor/mod.rs:57-90).  Tensors travel as
 * safetensors blobs: 8-byte little-endian header length, a JSON header
 * {name: {dtype, shape, data_offsets}}, raw data. */
ek_status ek_expert_id_parse(const char *id, int32_t *layer, int32_t *expert);
ek_status ek_expert_id_format(const char *model, int32_t layer, int32_t expert, char *out, size_t cap);

typedef struct ek_tensor_view {
    const void *data;  /* points into the blob */
    int64_t shape[4];  /* unused dimensions are 1 */
    int32_t rank;
    int32_t dtype;     /* ek_dtype */
    int64_t nbytes;
} ek_tensor_view;

/* SafeTensors::deserialize + tensor(name) (worker/core.rs:52-53).  A name that is
 * absent gives EK_WEIGHT_NOT_FOUND, a malformed blob or a dtype outside ek_dtype
 * EK_INVALID_INPUT. */
ek_status ek_safetensors_find(const void *blob, size_t len, const char *name, ek_tensor_view *out);
/* First tensor (header order) whose name ends with one of the suffixes:
 * FromSafeTensor::lookup_suffix (backend/torch/mod.rs:138-152). */
ek_status ek_safetensors_find_suffix(const void *blob, size_t len, const char *const *suffixes,
                                     int32_t n_suffixes, ek_tensor_view *out);
/* Size and bytes of a one-tensor blob: TchTensor::serialize
 * (backend/torch/mod.rs:115-117).  ek_safetensors_size returns 0 for a bad description. */
size_t ek_safetensors_size(const char *name, int32_t dtype, int32_t rank, const int64_t *shape);
ek_status ek_safetensors_emit(const char *name, int32_t dtype, int32_t rank, const int64_t *shape,
                              const void *data, void *out, size_t cap, size_t *written);

/* Loads one expert from the blob ek-db serves for it (transformer.rs:248-300):
 * ExpertWeight::from_safetensor (ffn/meta.rs:56-75) picks up / down / gate by
 * the suffixes w1|up_proj, w2|down_proj, w3|gate_proj ".weight"; a tensor named
 * "<weight>_scale_inv" (or "<weight>_scale") beside a weight is taken as its
 * scale: [rows] per channel, [rows/128, cols/128] per block.  Then as
 * ek_layer_set_expert. */
ek_status ek_layer_set_expert_safetensors(ek_layer *layer, int32_t expert, const void *blob, size_t len);

/* EKInstanceGate::forward (worker/core.rs:47-74) on wire bytes: req is a
 * safetensors blob with tensor "data" [n, H] of the layer's act dtype,
 * expert_id the request's sequences[0].experts[0]; resp receives the blob of
 * the result [n, H] (resp_len bytes; ek_safetensors_size gives the capacity
 * to provide).  The layer part of the id is not checked: the handle is the
 * layer. */
ek_status ek_worker_forward(ek_layer *layer, const char *expert_id, const void *req, size_t req_len,
                            void *resp, size_t resp_cap, size_t *resp_len);
/* The same for n_calls requests collected by the worker, as one grouped launch
 * (ek_layer_experts_forward). */
ek_status ek_worker_forward_batch(ek_layer *layer, int32_t n_calls, const char *const *expert_ids,
                                  const void *const *reqs, const size_t *req_lens, void *const *resps,
                                  const size_t *resp_caps, size_t *resp_lens);

/* The worker-side collector for the above.  The reference serves each Forward
 * RPC on its own task (worker/server.rs:39-63 -> worker/core.rs:47-74) and the
 * controller has one in flight per active expert (controller/executor.rs:
 * 141-195).  ek_batcher_forward has ek_worker_forward's contract and may be
 * called from any number of threads: callers that are in flight together are
 * answered by one grouped launch.  The first caller to arrive leads: it waits
 * up to max_wait_us for others to join (0: takes what is there), runs up to
 * max_calls requests as one ek_worker_forward_batch and hands every caller its
 * own status (a request that fails does not fail its neighbours; the error
 * text is the caller's ek_last_error()).  Callers arriving while a batch runs
 * form the next one.  The layer must outlive the batcher; destroy fails while
 * calls are in flight. */
typedef struct ek_batcher ek_batcher;
typedef struct {
    int64_t calls;          /* requests answered */
    int64_t batches;        /* grouped launches they were answered by */
    int64_t largest_batch;
} ek_batcher_stats;
ek_status ek_batcher_create(ek_layer *layer, int64_t max_wait_us, int32_t max_calls, ek_batcher **out);
ek_status ek_batcher_forward(ek_batcher *batcher, const char *expert_id, const void *req, size_t req_len,
                             void *resp, size_t resp_cap, size_t *resp_len);
ek_status ek_batcher_get_stats(ek_batcher *batcher, ek_batcher_stats *out);
ek_status ek_batcher_destroy(ek_batcher *batcher);

/* Turns per-phase HIP-event timing of ek_layer_forward on (1: every call; n > 1: every n-th
 * call, the first included -- five event records cost a decode-sized call ~15 us of gaps on
 * the device, sampling keeps a timed loop close to its unobserved speed) or off (0) and
 * clears the accumulated kernel_us.  Stands for the PerfTimer checkpoints of
 * the reference (ek-base/src/utils.rs:4-45; controller/executor.rs:136,201,228).
 * At most 1024 calls are recorded between two ek_layer_get_stats calls. */
ek_status ek_layer_profile(ek_layer *layer, int32_t enable);

/* worker_expert_activation (metrics.rs:56-62; incremented by the number of
 * sequences of each request, worker/server.rs:39-45): counts[e] = rows expert e
 * has been given since the layer was created, over all compute entry points.
 * The fused calls add the pack step's counts[] on the device.  counts: [E], host. */
ek_status ek_layer_get_activation(ek_layer *layer, int64_t *counts);

/* worker_forward (metrics.rs:46-54; observed in microseconds per request,
 * worker/server.rs:55-63): durations of the blocking compute calls, in the
 * reference's buckets le = 0, 4000, ..., 36000 us.  cumulative[i] counts
 * observations <= le[i], cumulative[10] all of them (+Inf), as Prometheus does. */
typedef struct ek_histogram {
    double le[10];
    int64_t cumulative[11];
    double sum;
    int64_t count;
} ek_histogram;
ek_status ek_layer_get_forward_histogram(ek_layer *layer, ek_histogram *out);

/* Ceilings measured on the device itself, for roofline lines next to the published peaks: a
 * plain device copy (bytes read + written per second), a read-only stream with non-temporal
 * loads (how the weight-streaming kernel reads expert weights) and a register-only bf16 MFMA
 * loop, once on constant operands and once on operands with random signs, exponents and
 * mantissas that change from one MFMA to the next (the clock under the chip's power limit, and
 * with it the rate a matrix product of real data can reach, depends on the bits that toggle).
 * No counterpart in the reference (its ek-benchmark times whole calls only,
 * ek-benchmark/src/bench.rs:36-52).  Allocates 8 GiB for the duration of the call; takes about a
 * second. */
typedef struct ek_peaks {
    double copy_gbps;        /* GB/s, read + write */
    double read_nt_gbps;     /* GB/s */
    double mfma_bf16_tflops; /* TFLOP/s, dense, fp32 accumulate, constant operands */
    double mfma_bf16_random_tflops; /* the same loop on random operands */
    double mfma_bf16_dequant_tflops; /* ... with the W8A16 tile path's conversions beside every MFMA
                                        (5 vector instructions per MFMA, operands in registers) */
} ek_peaks;
ek_status ek_measure_peaks(int32_t device_id, ek_peaks *out);

/* Snapshot of the layer's counters (waits for recorded events to complete). */
ek_status ek_layer_get_stats(ek_layer *layer, ek_stats *out);

/* ---- routers: logits -> (ids, gate weights), fused in front of pack ----------
 * Every choice is "larger value first, lower expert index on equal values"
 * (torch.topk leaves the order of equal values open). */
typedef enum ek_router_kind {
    EK_ROUTER_SOFTMAX_TOPK = 0,  /* softmax_fp32 over E, top-K, w /= sum(w) if renorm, cast:
                                    expertkit_torch/models/qwen3_moe.py:161-169 */
    EK_ROUTER_TOPK_RAW = 1,      /* top-K of the logits, w = the logits:
                                    expertkit_vllm/experts/grpc_expert.py:120-121 */
    EK_ROUTER_TOPK_SOFTMAX = 2,  /* top-K of the logits, softmax over the K:
                                    expertkit_vllm/models/deepseek_v2.py:123-128 */
    EK_ROUTER_TOPK_SIGMOID = 3,  /* top-K of the logits, sigmoid of the K: deepseek_v2.py:123-130 */
    EK_ROUTER_SIGMOID_GROUP = 4  /* DeepSeek-V3 group-limited routing, called by the reference at
                                    expertkit_torch/models/deepseek_v3/model.py:142 (the routine
                                    itself is transformers' DeepseekV3TopkRouter; parameters in
                                    ek-db/resources/ds-tiny/config.json:26-48): s = sigmoid(logits);
                                    c = s + bias; group score = sum of the group's two largest c;
                                    keep the topk_group best groups; top-K of c inside them;
                                    w = s[ids]; if renorm w /= sum(w) + 1e-20; w *= routed_scaling */
} ek_router_kind;

/* experts outside the kept groups compete with -inf (newer transformers) instead of 0.0 */
#define EK_ROUTER_MASK_NEG_INF 1

typedef struct ek_router_cfg {
    int32_t kind;         /* ek_router_kind */
    int32_t renorm;       /* norm_topk_prob (kinds 0 and 4) */
    int32_t n_group;      /* kind 4 */
    int32_t topk_group;   /* kind 4 */
    float routed_scaling; /* kind 4 */
    int32_t flags;        /* EK_ROUTER_* */
    int32_t logits_dtype; /* EK_F32, EK_BF16 or EK_F16 */
    int32_t w_dtype;      /* type of the gate weights produced: the layer's act dtype or EK_F32 */
    const void *bias;     /* kind 4: e_score_correction_bias [E] fp32 (same memory kind as the
                             call's tensors) or NULL */
} ek_router_cfg;

/* Router only: logits [T,E] -> ids [T,K] int32, w [T,K] of router->w_dtype. */
ek_status ek_layer_route(ek_layer *layer, const void *logits, const ek_router_cfg *router, int64_t T,
                         int32_t *ids, void *w, int32_t mem, void *stream);
/* ek_layer_forward that takes logits instead of (ids, w): router, pack, FFN and
 * combine are enqueued back to back.  ids / w (optional) receive what the router chose.
 * The result is bit-identical to ek_layer_route followed by ek_layer_forward. */
ek_status ek_layer_forward_logits(ek_layer *layer, const void *x, const void *logits,
                                  const ek_router_cfg *router, int64_t T, void *y, int32_t *ids, void *w,
                                  const ek_route_out *route, int32_t mem, void *stream);

/* ---- chain of layers: consecutive MoE layers launched as one HIP graph ------
 * The reference issues one ForwardReq per MoE layer from the attention side
 * (qwen3_moe.py:89-104 is entered once per decoder layer); a chain runs L
 * layer calls back to back on the device, x_{l+1} = y_l, with no host
 * round trip: the calls are captured once into a hipGraph (grids depend only
 * on T; segment lengths are read from device memory) and replayed.
 *   layers [L]: same hidden / top_k / act_dtype / device; each keeps its own
 *               experts and workspace and must outlive the chain
 *   ids [L,T,K] int32, w [L,T,K] w_dtype, x [T,H] -> y [T,H]; device pointers.
 * All L layers' ids are the caller's and known when the call starts, so when the
 * layers are L different objects the pack steps of layers 1 .. L-1 run on a
 * stream of their own beside layer 0's kernels instead of between two layers
 * (a layer named twice shares one workspace between its steps: no running ahead).
 * use_graph = 0 runs the same launches eagerly (the reference for graph tests).
 * A graph is re-captured when T, a pointer or w_dtype changes.  stream as in
 * ek_layer_forward (NULL = blocking on the library's stream); routing errors
 * are reported by blocking calls. */
typedef struct ek_chain ek_chain;
ek_status ek_chain_create(ek_layer *const *layers, int32_t n_layers, ek_chain **out);
ek_status ek_chain_forward(ek_chain *chain, const void *x, const int32_t *ids, const void *w,
                           int32_t w_dtype, int64_t T, void *y, int32_t use_graph, void *stream);
ek_status ek_chain_destroy(ek_chain *chain);

/* ---- single expert object: the literal shape of trait Expert<T> ----------
 * construct (ffn/meta.rs:38), forward (:37), shape (:35).  Implemented as a
 * one-expert layer; max_rows bounds n of forward. */
ek_status ek_expert_create(const ek_cfg *cfg, int64_t max_rows, const ek_weight_desc *up,
                           const ek_weight_desc *gate, const ek_weight_desc *down,
                           ek_expert **out);
ek_status ek_expert_forward(ek_expert *expert, const void *x, int64_t n, void *out, int32_t mem,
                            void *stream);
ek_status ek_expert_shape(ek_expert *expert, int64_t *hidden, int64_t *inter);
ek_status ek_expert_destroy(ek_expert *expert);

#ifdef __cplusplus
}
#endif
#endif /* EK_HIP_H */
