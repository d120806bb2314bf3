/* A worker shell in miniature, in plain C over the C ABI: E threads, each serving the Forward
 * requests of one expert of a layer as the reference's gRPC handler does
 * (ek-computation/src/worker/server.rs:39-63 -> worker/core.rs:47-74), for one "layer step"
 * at a time: all threads are released together, each answers one request, the step ends
 * when the last answer is back (what the controller waits for, controller/executor.rs:
 * 203-252).  Prints the mean wall time of a step when the requests are served one by one
 * (ek_worker_forward), through the collector (ek_batcher_forward) and as one explicit batch.
 *
 *   make -C expert-kit_amd/csrc examples
 *   expert-kit_amd/examples/worker_threads [experts rows hidden inter rounds]
 */
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "../../include/ek_hip.h"

#define CHECK(call)                                                                         \
    do {                                                                                    \
        ek_status st_ = (call);                                                             \
        if (st_ != EK_OK) {                                                                 \
            fprintf(stderr, "%s:%d: status %d: %s\n", __FILE__, __LINE__, (int)st_, ek_last_error()); \
            exit(1);                                                                        \
        }                                                                                   \
    } while (0)

static double now_us(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return ts.tv_sec * 1e6 + ts.tv_nsec * 1e-3;
}

static uint32_t rng_state = 12345u;
static uint32_t rng(void) { rng_state = rng_state * 1664525u + 1013904223u; return rng_state >> 8; }

typedef struct {
    ek_layer *layer;
    ek_batcher *batcher;      /* NULL: ek_worker_forward */
    char id[64];
    void *req, *resp;
    size_t req_len, resp_cap;
    int rounds;
    pthread_barrier_t *gate;
} Caller;

static void *serve(void *arg)
{
    Caller *c = (Caller *)arg;
    for (int r = 0; r < c->rounds; ++r) {
        size_t n = 0;
        pthread_barrier_wait(c->gate);
        if (c->batcher) CHECK(ek_batcher_forward(c->batcher, c->id, c->req, c->req_len, c->resp, c->resp_cap, &n));
        else CHECK(ek_worker_forward(c->layer, c->id, c->req, c->req_len, c->resp, c->resp_cap, &n));
        pthread_barrier_wait(c->gate);
    }
    return NULL;
}

static double run_steps(Caller *callers, int n, int rounds, ek_layer *layer, ek_batcher *batcher)
{
    pthread_barrier_t gate;
    pthread_barrier_init(&gate, NULL, (unsigned)n + 1);
    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)n);
    const int warm = 3;
    for (int i = 0; i < n; ++i) {
        callers[i].layer = layer;
        callers[i].batcher = batcher;
        callers[i].rounds = rounds + warm;
        callers[i].gate = &gate;
        pthread_create(&th[i], NULL, serve, &callers[i]);
    }
    double total = 0;
    for (int r = 0; r < rounds + warm; ++r) {
        pthread_barrier_wait(&gate);
        const double t0 = now_us();
        pthread_barrier_wait(&gate);
        if (r >= warm) total += now_us() - t0;
    }
    for (int i = 0; i < n; ++i) pthread_join(th[i], NULL);
    pthread_barrier_destroy(&gate);
    free(th);
    return total / rounds;
}

int main(int argc, char **argv)
{
    const int E = argc > 1 ? atoi(argv[1]) : 16, rows = argc > 2 ? atoi(argv[2]) : 4;
    const int64_t H = argc > 3 ? atoll(argv[3]) : 7168, I = argc > 4 ? atoll(argv[4]) : 2048;
    const int rounds = argc > 5 ? atoi(argv[5]) : 50;
    if (E < 1 || E > 1024 || rows < 1 || rounds < 1) { fprintf(stderr, "bad arguments\n"); return 1; }
    if (ek_device_count() < 1) { fprintf(stderr, "no HIP device\n"); return 1; }

    ek_cfg cfg;
    memset(&cfg, 0, sizeof cfg);
    cfg.hidden = H; cfg.inter = I; cfg.n_experts = E; cfg.top_k = 1;
    cfg.act_dtype = EK_BF16; cfg.w_dtype = EK_I8; cfg.max_tokens = (int64_t)E * rows;
    ek_layer *layer;
    CHECK(ek_layer_create(&cfg, &layer));

    /* int8 weights with per-output-channel fp32 scales (the W8A16 form of the DeepSeek-V3 shape) */
    int8_t *q = (int8_t *)malloc((size_t)H * I);
    float *s = (float *)malloc(sizeof(float) * (size_t)(H > I ? H : I));
    for (int64_t i = 0; i < (H > I ? H : I); ++i) s[i] = 1e-3f + 3e-3f * (float)(rng() & 1023) / 1024.f;
    for (int e = 0; e < E; ++e) {
        for (int64_t i = 0; i < H * I; ++i) q[i] = (int8_t)((int)(rng() % 255) - 127);
        ek_weight_desc up = {q, I, H, EK_I8, EK_HOST, s, EK_F32, EK_SCALE_PER_CHANNEL};
        ek_weight_desc down = {q, H, I, EK_I8, EK_HOST, s, EK_F32, EK_SCALE_PER_CHANNEL};
        CHECK(ek_layer_set_expert(layer, e, &up, &up, &down));
    }

    /* one request per expert: safetensors {"data": [rows, H] bf16} */
    const int64_t shape[2] = {rows, H};
    const size_t blob = ek_safetensors_size("data", EK_BF16, 2, shape);
    uint16_t *x = (uint16_t *)malloc((size_t)rows * H * 2);
    Caller *callers = (Caller *)calloc((size_t)E, sizeof(Caller));
    for (int e = 0; e < E; ++e) {
        for (int64_t i = 0; i < rows * H; ++i) x[i] = (uint16_t)(0x3c00u + (rng() & 0x1ff) + ((rng() & 1) << 15));
        callers[e].req = malloc(blob);
        callers[e].resp = malloc(blob);
        callers[e].resp_cap = blob;
        CHECK(ek_safetensors_emit("data", EK_BF16, 2, shape, x, callers[e].req, blob, &callers[e].req_len));
        CHECK(ek_expert_id_format("model", 0, e, callers[e].id, sizeof callers[e].id));
    }

    printf("%d experts, one %d-row request each, hidden %lld, intermediate %lld, int8 weights; mean of %d steps\n", E, rows,
           (long long)H, (long long)I, rounds);
    printf("  %-44s %9.1f us per step\n", "ek_worker_forward, one thread per request", run_steps(callers, E, rounds, layer, NULL));
    const int waits[3] = {0, 20, 100};
    for (int w = 0; w < 3; ++w) {
        ek_batcher *b;
        ek_batcher_stats bs;
        char label[96];
        CHECK(ek_batcher_create(layer, waits[w], 256, &b));
        const double us = run_steps(callers, E, rounds, layer, b);
        CHECK(ek_batcher_get_stats(b, &bs));
        snprintf(label, sizeof label, "ek_batcher_forward, window %d us", waits[w]);
        printf("  %-44s %9.1f us per step   (%lld requests in %lld launches, largest %lld)\n", label, us,
               (long long)bs.calls, (long long)bs.batches, (long long)bs.largest_batch);
        CHECK(ek_batcher_destroy(b));
    }
    {
        const char **ids = (const char **)malloc(sizeof(char *) * (size_t)E);
        const void **reqs = (const void **)malloc(sizeof(void *) * (size_t)E);
        void **resps = (void **)malloc(sizeof(void *) * (size_t)E);
        size_t *lens = (size_t *)malloc(sizeof(size_t) * (size_t)E), *caps = (size_t *)malloc(sizeof(size_t) * (size_t)E),
               *outl = (size_t *)malloc(sizeof(size_t) * (size_t)E);
        for (int e = 0; e < E; ++e) {
            ids[e] = callers[e].id; reqs[e] = callers[e].req; resps[e] = callers[e].resp;
            lens[e] = callers[e].req_len; caps[e] = blob;
        }
        for (int r = 0; r < 3; ++r) CHECK(ek_worker_forward_batch(layer, E, ids, reqs, lens, resps, caps, outl));
        const double t0 = now_us();
        for (int r = 0; r < rounds; ++r) CHECK(ek_worker_forward_batch(layer, E, ids, reqs, lens, resps, caps, outl));
        printf("  %-44s %9.1f us per step\n", "ek_worker_forward_batch, one caller", (now_us() - t0) / rounds);
    }
    CHECK(ek_layer_destroy(layer));
    return 0;
}
