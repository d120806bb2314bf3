/*
 * ek_oracle.c -- CPU restatement of the Expert Kit routed-expert path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this file; it exists so that the HIP path can be checked against an
 * independent, slow, obviously-correct statement of the reference's algorithm.
 *
 * Each function cites the reference source it follows (paths are relative to
 * the expert-kit/expert-kit tree).
 *
 * Pinning status.  The reference's own fixtures for this path
 * (ek-computation/resources/qwen3-l0e1.*.safetensors,
 * w8a16active-l0q_a_proj.safetensors) are Git-LFS pointers without content,
 * so no function here is pinned by reference-held data ("parity unpinned" in
 * that sense).  Every function is instead pinned by tests/test_oracle_*.py
 * against brute force, closed forms, invariants and an independent libtorch
 * evaluation of the same op sequence.
 *
 * Plain C99 + optional OpenMP.  Floating-point storage types (bf16, fp16) are
 * handled as uint16 bit patterns with explicit round-to-nearest-even.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define EKO_BF16 0
#define EKO_F16 1
#define EKO_F32 2

/* ---------------------------------------------------------------- dtypes */

static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

static inline uint16_t f32_to_bf16(float f)
{
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    u += 0x7fffu + ((u >> 16) & 1u); /* round to nearest, ties to even */
    return (uint16_t)(u >> 16);
}

static inline float f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline uint16_t f32_to_f16(float f)
{
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);      /* NaN */
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);     /* >= 65520 -> inf */
    if (a < 0x33000001u) return sign;                           /* <= 2^-25 -> 0 (tie to even) */
    if (a < 0x38800000u) {
        /* subnormal half: multiples of 2^-24; nearbyintf rounds ties to even
         * in the default rounding mode and the scaling is exact */
        float r = nearbyintf(bits_f32(a) * 16777216.0f);
        return (uint16_t)(sign | (uint16_t)r);
    }
    uint32_t r = a + 0xfffu + ((a >> 13) & 1u); /* RNE on the 13 dropped bits */
    return (uint16_t)(sign | (uint16_t)((r - 0x38000000u) >> 13));
}

static inline float load_act(const void *p, int64_t i, int dt)
{
    switch (dt) {
    case EKO_BF16: return bf16_to_f32(((const uint16_t *)p)[i]);
    case EKO_F16: return f16_to_f32(((const uint16_t *)p)[i]);
    default: return ((const float *)p)[i];
    }
}

/* round a float to the storage type and return it widened back to float */
static inline float round_act(float v, int dt)
{
    switch (dt) {
    case EKO_BF16: return bf16_to_f32(f32_to_bf16(v));
    case EKO_F16: return f16_to_f32(f32_to_f16(v));
    default: return v;
    }
}

static inline void store_act(void *p, int64_t i, float v, int dt)
{
    switch (dt) {
    case EKO_BF16: ((uint16_t *)p)[i] = f32_to_bf16(v); break;
    case EKO_F16: ((uint16_t *)p)[i] = f32_to_f16(v); break;
    default: ((float *)p)[i] = v; break;
    }
}

static inline int act_size(int dt) { return dt == EKO_F32 ? 4 : 2; }

/* exported scalar conversions so tests can pin the rounding helpers */
uint16_t eko_f32_to_bf16(float f) { return f32_to_bf16(f); }
float eko_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }
uint16_t eko_f32_to_f16(float f) { return f32_to_f16(f); }
float eko_f16_to_f32(uint16_t h) { return f16_to_f32(h); }

/* ---------------------------------------------------------------- router */

/*
 * Router: softmax in fp32 over experts, top-k, renormalise, cast to the
 * activation dtype.
 * Follows ek-integration/expertkit_torch/expertkit_torch/models/qwen3_moe.py:161-169.
 * Tie rule: the lower expert index wins (ties have probability ~0 for
 * continuous logits; the rule is fixed so that the result is a function).
 * logits [T,E] f32 -> ids [T,K] int32, w [T,K] in w_dt (EKO_F32 keeps fp32,
 * which is the DeepSeek shim's behaviour, deepseek_v3/model.py:97-103).
 */
int eko_router_softmax_topk(const float *logits, int64_t T, int E, int K, int renorm,
                            int32_t *ids, void *w, int w_dt)
{
    if (K > E || K <= 0) return -1;
    float *p = (float *)malloc(sizeof(float) * (size_t)E);
    char *used = (char *)malloc((size_t)E);
    if (!p || !used) { free(p); free(used); return -2; }
    for (int64_t t = 0; t < T; ++t) {
        const float *l = logits + t * E;
        float m = l[0];
        for (int e = 1; e < E; ++e) if (l[e] > m) m = l[e];
        float s = 0.f;
        for (int e = 0; e < E; ++e) { p[e] = expf(l[e] - m); s += p[e]; }
        for (int e = 0; e < E; ++e) p[e] = p[e] / s;
        memset(used, 0, (size_t)E);
        float ws = 0.f;
        for (int k = 0; k < K; ++k) {
            int best = -1;
            for (int e = 0; e < E; ++e)
                if (!used[e] && (best < 0 || p[e] > p[best])) best = e;
            used[best] = 1;
            ids[t * K + k] = best;
            ws += p[best];
        }
        for (int k = 0; k < K; ++k) {
            float v = p[ids[t * K + k]];
            if (renorm) v = v / ws;
            store_act(w, t * K + k, v, w_dt);
        }
    }
    free(p); free(used);
    return 0;
}

/*
 * exp(x) built from IEEE-754 single operations only (fused multiply-add,
 * multiply, add, round-to-nearest-even), so that any conforming machine gives
 * the same bits: Cody-Waite reduction by ln 2, the degree-5 polynomial of
 * Cephes' expf, scaling by an exponent-field constant.  The argument is
 * clamped to [-87, 88], where the result is a normal number.  Within 2 ulp of
 * the exact value (pinned against libm in tests/test_oracle_router.py).
 * Compile with -ffp-contract=off: the unfused operations must stay unfused.
 */
float eko_expf(float x)
{
    x = x < -87.0f ? -87.0f : (x > 88.0f ? 88.0f : x);
    const float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    const float y = fmaf(r * r, p, r) + 1.0f;
    return y * bits_f32((uint32_t)((int32_t)n + 127) << 23);
}
float eko_sigmoidf(float x) { return 1.0f / (1.0f + eko_expf(-x)); }

/*
 * The same routine with the argument clamped to [-87, 89] and the scaling done by ldexpf, so
 * that it overflows to +inf beyond 88.72 as libm's expf does: the form the HIP kernels' SwiGLU
 * epilogue evaluates (expert-kit_amd/csrc/ek_mfma.h), restated here so that a CPU test can hold
 * gate / (1 + exp(-gate)) built on it against the same expression built on libm for every 16-bit
 * gate value.  Test support: eko_ffn itself uses libm's expf.
 */
float eko_expf_wide(float x)
{
    x = x < -87.0f ? -87.0f : (x > 89.0f ? 89.0f : x);
    const float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    const float y = fmaf(r * r, p, r) + 1.0f;
    return ldexpf(y, (int)n);
}
/* silu as the kernels form it (their exp, eko_expf_wide's operations one for one, and a correctly
 * rounded IEEE division) and as eko_ffn forms it (libm), for one fp32 gate value; that the two agree
 * after the storage rounding for every 16-bit gate is held on the CPU, and that the kernels return
 * this value for every gate by the GPU test over all gate values */
float eko_silu_kernel_form(float g) { return g / (1.0f + eko_expf_wide(-g)); }
float eko_silu_libm_form(float g) { return g / (1.0f + expf(-g)); }

/* larger value first, lower index on equal values */
static int pick_best(const float *v, const char *used, int n)
{
    int best = -1;
    for (int e = 0; e < n; ++e)
        if (!used[e] && (best < 0 || v[e] > v[best])) best = e;
    return best;
}

/*
 * The routers of the reference's model shims, one token at a time.
 *   kind 0  softmax_fp32 over E, top-K, optional renormalisation, cast
 *           (expertkit_torch/models/qwen3_moe.py:161-169).  The choice is made on
 *           the logits: softmax is monotone, so this is the choice torch.topk
 *           makes on the probabilities wherever those are distinct.
 *   kind 1  top-K of the raw logits, weights = the logits
 *           (expertkit_vllm/experts/grpc_expert.py:120-121)
 *   kind 2  top-K of the logits, softmax over the K (expertkit_vllm/models/deepseek_v2.py:123-128)
 *   kind 3  top-K of the logits, sigmoid of the K   (deepseek_v2.py:123-130)
 *   kind 4  DeepSeek-V3 group-limited routing.  The reference calls it at
 *           expertkit_torch/models/deepseek_v3/model.py:142; the routine is
 *           transformers' DeepseekV3TopkRouter.forward (third party, pinned by the
 *           reference at transformers==4.51.3, not part of the reference tree):
 *             s = sigmoid(logits); c = s + bias;
 *             group score = sum of the two largest c of the group;
 *             keep the topk_group best groups; c of every other expert := 0
 *             (-inf in newer transformers: mask_neg_inf); ids = top-K of c;
 *             w = s[ids]; if renorm: w /= sum(w) + 1e-20; w *= routed_scaling.
 * exp and sigmoid are eko_expf / eko_sigmoidf.  Sums run over k (or e) ascending.
 * logits [T,E] of logits_dt; bias [E] f32 or NULL; ids [T,K] int32; w [T,K] of w_dt.
 */
int eko_route(int kind, const void *logits, int logits_dt, const float *bias, int64_t T, int E, int K,
              int renorm, int n_group, int topk_group, int mask_neg_inf, float routed_scaling,
              int32_t *ids, void *w, int w_dt)
{
    if (K > E || K <= 0 || kind < 0 || kind > 4) return -1;
    if (kind == 4 && (n_group < 1 || E % n_group || E / n_group < 2 || topk_group < 1 || topk_group > n_group ||
                      (int64_t)topk_group * (E / n_group) < K))
        return -1;
    float *v = (float *)malloc(sizeof(float) * (size_t)E);      /* the value the choice is made on */
    float *sc = (float *)malloc(sizeof(float) * (size_t)E);     /* kind 4: unbiased scores */
    float *wk = (float *)malloc(sizeof(float) * (size_t)K);
    float *gs = (float *)malloc(sizeof(float) * (size_t)(n_group > 0 ? n_group : 1));
    char *used = (char *)malloc((size_t)E);
    char *gkeep = (char *)malloc((size_t)(n_group > 0 ? n_group : 1));
    if (!v || !sc || !wk || !gs || !used || !gkeep) { free(v); free(sc); free(wk); free(gs); free(used); free(gkeep); return -2; }
    for (int64_t t = 0; t < T; ++t) {
        for (int e = 0; e < E; ++e) v[e] = load_act(logits, t * E + e, logits_dt);
        float m = 0.f, s = 1.f;
        if (kind == 0) {
            m = v[0];
            for (int e = 1; e < E; ++e) if (v[e] > m) m = v[e];
            s = 0.f;
            for (int e = 0; e < E; ++e) s += eko_expf(v[e] - m);
        } else if (kind == 4) {
            const int G = E / n_group;
            for (int e = 0; e < E; ++e) {
                sc[e] = eko_sigmoidf(v[e]);
                v[e] = bias ? sc[e] + bias[e] : sc[e];
            }
            for (int g = 0; g < n_group; ++g) {
                float b0 = -INFINITY, b1 = -INFINITY;
                for (int i = 0; i < G; ++i) {
                    const float c = v[g * G + i];
                    if (c > b0) { b1 = b0; b0 = c; }
                    else if (c > b1) b1 = c;
                }
                gs[g] = b0 + b1;
            }
            memset(used, 0, (size_t)n_group);
            memset(gkeep, 0, (size_t)n_group);
            for (int k = 0; k < topk_group; ++k) {
                const int g = pick_best(gs, used, n_group);
                used[g] = 1;
                gkeep[g] = 1;
            }
            for (int e = 0; e < E; ++e)
                if (!gkeep[e / G]) v[e] = mask_neg_inf ? -INFINITY : 0.f;
        }
        memset(used, 0, (size_t)E);
        for (int k = 0; k < K; ++k) {
            const int best = pick_best(v, used, E);
            used[best] = 1;
            ids[t * K + k] = best;
        }
        for (int k = 0; k < K; ++k) {
            const float l = v[ids[t * K + k]];
            switch (kind) {
            case 0: wk[k] = eko_expf(l - m) / s; break;
            case 1: wk[k] = l; break;
            case 2: wk[k] = eko_expf(l - v[ids[t * K]]); break;
            case 3: wk[k] = eko_sigmoidf(l); break;
            default: wk[k] = sc[ids[t * K + k]]; break;
            }
        }
        if (kind == 2 || ((kind == 0 || kind == 4) && renorm)) {
            float tot = 0.f;
            for (int k = 0; k < K; ++k) tot += wk[k];
            if (kind == 4) tot += 1e-20f;
            for (int k = 0; k < K; ++k) wk[k] = wk[k] / tot;
        }
        for (int k = 0; k < K; ++k) store_act(w, t * K + k, kind == 4 ? wk[k] * routed_scaling : wk[k], w_dt);
    }
    free(v); free(sc); free(wk); free(gs); free(used); free(gkeep);
    return 0;
}

/* ------------------------------------------------------------------ pack */

/*
 * Group (token, slot) pairs by expert.
 * Follows NaiveExecutor::break_down_to_egress / add_seq
 * (ek-computation/src/controller/executor.rs:283-304): for each sequence
 * (token) in order and each of its experts in slot order, the pair is pushed
 * onto that expert's list.  The lists are then laid out one after another in
 * ascending integer expert id (the reference iterates a BTreeMap keyed by the
 * id *string*; the visiting order of experts does not influence any result
 * because every pair's output returns to its own (token, slot) cell,
 * executor.rs:214-225).
 *
 * ids [P] (P = T*K, flat index p = t*K + k), values in [0,E).
 * counts [E], offsets [E+1] (exclusive scan), perm [P] (packed position ->
 * flat pair index), inv_perm [P] (flat pair index -> packed position).
 * Returns 0, or -1 if an id is out of range.
 */
int eko_pack(const int32_t *ids, int64_t P, int E, int32_t *counts, int32_t *offsets,
             int32_t *perm, int32_t *inv_perm)
{
    /* literal restatement: growable per-expert lists with push_back */
    int32_t **list = (int32_t **)calloc((size_t)E, sizeof(int32_t *));
    int32_t *len = (int32_t *)calloc((size_t)E, sizeof(int32_t));
    int32_t *cap = (int32_t *)calloc((size_t)E, sizeof(int32_t));
    int rc = 0;
    for (int64_t p = 0; p < P; ++p) {
        int32_t e = ids[p];
        if (e < 0 || e >= E) { rc = -1; goto done; }
        if (len[e] == cap[e]) {
            cap[e] = cap[e] ? cap[e] * 2 : 4;
            list[e] = (int32_t *)realloc(list[e], sizeof(int32_t) * (size_t)cap[e]);
        }
        list[e][len[e]++] = (int32_t)p;
    }
    {
        int32_t pos = 0;
        for (int e = 0; e < E; ++e) {
            counts[e] = len[e];
            offsets[e] = pos;
            for (int32_t j = 0; j < len[e]; ++j) {
                perm[pos] = list[e][j];
                inv_perm[list[e][j]] = pos;
                ++pos;
            }
        }
        offsets[E] = pos;
    }
done:
    for (int e = 0; e < E; ++e) free(list[e]);
    free(list); free(len); free(cap);
    return rc;
}

/*
 * Gather token rows into packed order.
 * Follows NaiveExecutor::assemble_seq_tensors (executor.rs:112-133):
 * X_e = stack([x[t] for (t,k) in list_e]).  Pure byte copy.
 */
void eko_gather(const void *x, int64_t H, int elem_size, const int32_t *perm, int64_t P, int K,
                void *xp)
{
    size_t row = (size_t)H * (size_t)elem_size;
    for (int64_t j = 0; j < P; ++j)
        memcpy((char *)xp + (size_t)j * row, (const char *)x + (size_t)(perm[j] / K) * row, row);
}

/*
 * Scatter packed expert outputs back to [T,K,H].
 * Follows the collection loop of inner_execute (executor.rs:203-226) and
 * output (executor.rs:235-252): Y[t,k,:] = out_e[j,:] where (t,k) is the j-th
 * entry of expert e's list.  Pure byte copy.
 */
void eko_scatter(const void *yp, int64_t H, int elem_size, const int32_t *perm, int64_t P, void *y)
{
    size_t row = (size_t)H * (size_t)elem_size;
    for (int64_t j = 0; j < P; ++j)
        memcpy((char *)y + (size_t)perm[j] * row, (const char *)yp + (size_t)j * row, row);
}

/* --------------------------------------------------------------- dequant */

/*
 * Per-output-channel W8A16 dequantisation (the benchmark's definition):
 * W[n,c] = rne_dt( f32(q[n,c]) * f32(scale[n]) ), scale given as bf16 bits,
 * dt = bf16 (the definition) or fp16 (its analogue for fp16 activations).
 * The product of an int8 and a bf16 has at most 15 significant bits, so it is
 * exact in fp32 and the only rounding is the final one.
 */
void eko_dequant_channel(const int8_t *q, const uint16_t *scale_bf16, int64_t N, int64_t C,
                         int dt, uint16_t *w)
{
    for (int64_t n = 0; n < N; ++n) {
        float s = bf16_to_f32(scale_bf16[n]);
        for (int64_t c = 0; c < C; ++c)
            store_act(w, n * C + c, (float)q[n * C + c] * s, dt);
    }
}

/*
 * Block-scaled dequantisation as the reference has it.
 * Follows w8a16_activate (ek-computation/src/ffn/expert_torch.rs:24-53) for
 * row counts that are multiples of the block size (the reference's padding
 * branch is only reached otherwise): W[r,c] = bf16( f32(q[r,c]) * s[r/B, c/B] ).
 * q is given as fp32 values (the reference converts any stored kind to Float
 * first, expert_torch.rs:39,45); s [ceil(N/B), ceil(C/B)] fp32.
 */
void eko_dequant_block(const float *q, const float *s, int64_t N, int64_t C, int64_t B,
                       uint16_t *w_bf16)
{
    int64_t sc = (C + B - 1) / B;
    for (int64_t r = 0; r < N; ++r)
        for (int64_t c = 0; c < C; ++c)
            w_bf16[r * C + c] = f32_to_bf16(q[r * C + c] * s[(r / B) * sc + (c / B)]);
}

/*
 * OCP fp8 e4m3fn -> fp32: the element type of DeepSeek FP8 checkpoint tensors,
 * DType::Float8e4m3fn of the reference (ek-computation/src/backend/mod.rs:13), which
 * w8a16_activate converts with to_kind(Float) before scaling (expert_torch.rs:39).
 * 1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities; 0x7f / 0xff are NaN;
 * exponent 0 holds subnormals m/8 * 2^-6.
 */
void eko_fp8_e4m3fn_to_f32(const uint8_t *b, int64_t n, float *out)
{
    for (int64_t i = 0; i < n; ++i) {
        const int s = b[i] >> 7, e = (b[i] >> 3) & 15, m = b[i] & 7;
        float v;
        if (e == 15 && m == 7) v = NAN;
        else if (e == 0) v = ldexpf((float)m, -9);
        else v = ldexpf((float)(8 + m), e - 10);
        out[i] = s ? -v : v;
    }
}

/* ------------------------------------------------------------------- FFN */

static inline double silu_d(double v) { return v / (1.0 + exp(-v)); }

/*
 * One expert's SwiGLU FFN.
 * Follows TorchFFN::load_module's closure (ek-computation/src/ffn/expert_torch.rs:80-85)
 * with the weight naming of ffn/meta.rs:58-63 (w1 = up_proj, w3 = gate_proj,
 * w2 = down_proj), weights row-major [out_features, in_features]:
 *     up   = x . W_up^T          (:81)
 *     gate = x . W_gate^T        (:82)
 *     h    = up * silu(gate)     (:83)
 *     out  = h . W_down^T        (:84)
 *
 * mode 0 ("reference-rounded"): every named tensor above, and silu(gate), is
 * materialised in the activation dtype `dt` (round to nearest even), as
 * libtorch does for bf16/fp16 tensors; each dot product is accumulated in
 * double and rounded once to fp32 before the storage rounding, standing for
 * "fp32 accumulation in unspecified order".  silu is evaluated in fp32 from
 * the rounded gate.
 * mode 1 ("ideal"): no intermediate rounding; everything in double, the
 * result written as fp32 regardless of dt.
 * mode 2 ("reference-rounded, last rounding left out"): as mode 0, but `out`
 * is written as fp32 before its storage rounding.  A bf16 ulp at 4-5 sigma of
 * the output distribution is up to 3.5e-2 x RMS, so a max-norm gate against
 * the rounded output would be decided by 1-ulp coin flips of the last
 * rounding; this mode gives the value those flips are taken around.
 * mode 3 ("reference-rounded, fp32 accumulation in index order"): as mode 0, but
 * each dot product is accumulated in fp32, one term after the other, the way a
 * scalar fp32 backend would: a second legitimate evaluation order of the same
 * reference ops, used by the tests to show how far two faithful evaluations
 * of the reference lie apart.
 *
 * x [n,H] (dt), w_* 16-bit of type dt (or fp32 if dt==EKO_F32).
 * out: dt in modes 0 and 3, fp32 in modes 1 and 2.  h_out (optional, may be NULL):
 * [n,I], dt in modes 0, 2 and 3, fp32 in mode 1.
 */
void eko_ffn(const void *x, int64_t n, int64_t H, int64_t I, const void *w_up, const void *w_gate,
             const void *w_down, int dt, int mode, void *out, void *h_out)
{
    float *xf = (float *)malloc(sizeof(float) * (size_t)(n * H + 1));
    double *h = (double *)malloc(sizeof(double) * (size_t)(n * I + 1));
    for (int64_t i = 0; i < n * H; ++i) xf[i] = load_act(x, i, dt);

#pragma omp parallel for schedule(static)
    for (int64_t c = 0; c < I; ++c) {
        for (int64_t r = 0; r < n; ++r) {
            double au = 0.0, ag = 0.0;
            const float *xr = xf + r * H;
            if (mode == 3) {
                float fu = 0.0f, fg = 0.0f;
                for (int64_t k = 0; k < H; ++k) {
                    fu += xr[k] * load_act(w_up, c * H + k, dt);
                    fg += xr[k] * load_act(w_gate, c * H + k, dt);
                }
                au = (double)fu;
                ag = (double)fg;
            } else {
                for (int64_t k = 0; k < H; ++k) {
                    au += (double)xr[k] * (double)load_act(w_up, c * H + k, dt);
                    ag += (double)xr[k] * (double)load_act(w_gate, c * H + k, dt);
                }
            }
            if (mode != 1) {
                float up = round_act((float)au, dt);
                float gate = round_act((float)ag, dt);
                float sg = round_act(gate / (1.0f + expf(-gate)), dt);
                h[r * I + c] = (double)round_act(up * sg, dt);
            } else {
                h[r * I + c] = au * silu_d(ag);
            }
        }
    }
    if (h_out) {
        for (int64_t i = 0; i < n * I; ++i) {
            if (mode != 1) store_act(h_out, i, (float)h[i], dt);
            else ((float *)h_out)[i] = (float)h[i];
        }
    }
#pragma omp parallel for schedule(static)
    for (int64_t c = 0; c < H; ++c) {
        for (int64_t r = 0; r < n; ++r) {
            double a = 0.0;
            const double *hr = h + r * I;
            if (mode == 3) {
                float fa = 0.0f;
                for (int64_t k = 0; k < I; ++k) fa += (float)hr[k] * load_act(w_down, c * I + k, dt);
                a = (double)fa;
            } else {
                for (int64_t k = 0; k < I; ++k) a += hr[k] * (double)load_act(w_down, c * I + k, dt);
            }
            if (mode == 0 || mode == 3) store_act(out, r * H + c, (float)a, dt);
            else ((float *)out)[r * H + c] = (float)a;
        }
    }
    free(xf); free(h);
}

/* --------------------------------------------------------------- combine */

/*
 * Gate-weighted sum over the top-k slots.
 * Follows ek_forward (qwen3_moe.py:102-104): the outputs arrive as [T,K,H] in
 * the activation dtype; `expanded_weights * outputs` is an elementwise tensor
 * in the promoted dtype of the two operands, and torch.sum(dim=1) reduces it
 * with fp32 accumulation, k ascending, and rounds once.
 *   w_dt == dt      (Qwen3 shim, weights already cast, qwen3_moe.py:169):
 *                   product rounded to dt, then summed.
 *   w_dt == EKO_F32 (DeepSeek shim, deepseek_v3/model.py:97-103): product and
 *                   sum stay fp32, one rounding to dt at the end.
 * y3 [T,K,H] (dt), w [T,K] (w_dt) -> y [T,H]: dt if round_out, else the fp32
 * sum before its storage rounding.
 */
void eko_combine(const void *y3, const void *w, int64_t T, int K, int64_t H, int dt, int w_dt,
                 int round_out, void *y)
{
    for (int64_t t = 0; t < T; ++t)
        for (int64_t c = 0; c < H; ++c) {
            float acc = 0.f;
            for (int k = 0; k < K; ++k) {
                float wv = load_act(w, t * K + k, w_dt);
                float yv = load_act(y3, (t * K + k) * H + c, dt);
                float p = wv * yv;
                if (w_dt != EKO_F32) p = round_act(p, dt);
                acc += p;
            }
            if (round_out) store_act(y, t * H + c, acc, dt);
            else ((float *)y)[t * H + c] = acc;
        }
}

/* ------------------------------------------------------- whole layer (EK) */

/*
 * One MoE layer the way Expert Kit runs it: pack -> gather -> per-expert FFN
 * -> scatter -> combine (call stack: executor.rs:283-299, :112-133,
 * worker/core.rs:47-74 -> ffn/mod.rs:39-53 -> expert_torch.rs:80-85,
 * executor.rs:203-252, qwen3_moe.py:102-104).
 *
 * weights: arrays of E pointers (NULL allowed for experts that receive no
 * pair); mode as in eko_ffn.  In mode 1 the combine is done in double and y is
 * written as fp32 [T,H]; in modes 0 and 3 y has dtype dt; in mode 2 every tensor of
 * the reference is rounded as in mode 0 except y itself, written as fp32.
 * route outputs (counts, offsets, perm, inv_perm) may each be NULL.
 * y3_o (may be NULL): the [T,K,H] tensor the controller hands back before the
 * weighted sum (dt in modes 0 and 2, fp32 in mode 1).
 * Returns 0; -1 bad id; -3 pair routed to an expert without weights.
 */
int eko_layer_forward(const void *x, const int32_t *ids, const void *w, int64_t T, int K, int E,
                      int64_t H, int64_t I, const void *const *w_up, const void *const *w_gate,
                      const void *const *w_down, int dt, int w_dt, int mode, void *y,
                      int32_t *counts_o, int32_t *offsets_o, int32_t *perm_o, int32_t *inv_o,
                      void *y3_o)
{
    int64_t P = T * K;
    int es = act_size(dt);
    int32_t *counts = (int32_t *)malloc(sizeof(int32_t) * (size_t)(E + 1));
    int32_t *offsets = (int32_t *)malloc(sizeof(int32_t) * (size_t)(E + 2));
    int32_t *perm = (int32_t *)malloc(sizeof(int32_t) * (size_t)(P + 1));
    int32_t *inv = (int32_t *)malloc(sizeof(int32_t) * (size_t)(P + 1));
    int rc = eko_pack(ids, P, E, counts, offsets, perm, inv);
    if (rc) { free(counts); free(offsets); free(perm); free(inv); return rc; }

    int ffn_mode = mode == 1 ? 1 : (mode == 3 ? 3 : 0);
    int oes = ffn_mode == 1 ? 4 : es;
    char *xp = (char *)malloc((size_t)(P * H + 1) * (size_t)es);
    char *yp = (char *)malloc((size_t)(P * H + 1) * (size_t)oes);
    char *y3 = (char *)malloc((size_t)(P * H + 1) * (size_t)oes);
    eko_gather(x, H, es, perm, P, K, xp);
    for (int e = 0; e < E && rc == 0; ++e) {
        if (!counts[e]) continue;
        if (!w_up[e] || !w_gate[e] || !w_down[e]) { rc = -3; break; }
        eko_ffn(xp + (size_t)offsets[e] * (size_t)H * (size_t)es, counts[e], H, I, w_up[e],
                w_gate[e], w_down[e], dt, ffn_mode, yp + (size_t)offsets[e] * (size_t)H * (size_t)oes,
                NULL);
    }
    if (rc == 0) {
        eko_scatter(yp, H, oes, perm, P, y3);
        if (mode != 1) {
            eko_combine(y3, w, T, K, H, dt, w_dt, mode == 0 || mode == 3, y);
        } else {
            for (int64_t t = 0; t < T; ++t)
                for (int64_t c = 0; c < H; ++c) {
                    double acc = 0.0;
                    for (int k = 0; k < K; ++k)
                        acc += (double)load_act(w, t * K + k, w_dt) *
                               (double)((float *)y3)[(t * K + k) * H + c];
                    ((float *)y)[t * H + c] = (float)acc;
                }
        }
        if (y3_o) memcpy(y3_o, y3, (size_t)(P * H) * (size_t)oes);
        if (counts_o) memcpy(counts_o, counts, sizeof(int32_t) * (size_t)E);
        if (offsets_o) memcpy(offsets_o, offsets, sizeof(int32_t) * (size_t)(E + 1));
        if (perm_o) memcpy(perm_o, perm, sizeof(int32_t) * (size_t)P);
        if (inv_o) memcpy(inv_o, inv, sizeof(int32_t) * (size_t)P);
    }
    free(counts); free(offsets); free(perm); free(inv); free(xp); free(yp); free(y3);
    return rc;
}

/* ---------------------------------------- whole layer (stock loop form) */

/*
 * The model's own (non-EK) MoE loop, an independent statement of the same
 * layer.  Follows normal_forward (qwen3_moe.py:115-151): for each expert in
 * ascending index, rows that selected it (token ascending) go through the
 * expert, are multiplied by their gate weight (product in dt), and are added
 * into a zero-initialised [T,H] buffer of dtype dt with index_add_, i.e. one
 * storage rounding per (expert, token) addition.
 * Only mode-0 rounding is provided; y [T,H] dtype dt.
 */
int eko_layer_loop_form(const void *x, const int32_t *ids, const void *w, int64_t T, int K, int E,
                        int64_t H, int64_t I, const void *const *w_up, const void *const *w_gate,
                        const void *const *w_down, int dt, int w_dt, void *y)
{
    int es = act_size(dt);
    float *acc = (float *)calloc((size_t)(T * H + 1), sizeof(float));
    char *xr = (char *)malloc((size_t)(T * H + 1) * (size_t)es);
    char *yr = (char *)malloc((size_t)(T * H + 1) * (size_t)es);
    int64_t *tok = (int64_t *)malloc(sizeof(int64_t) * (size_t)(T + 1));
    int *slot = (int *)malloc(sizeof(int) * (size_t)(T + 1));
    int rc = 0;
    for (int e = 0; e < E; ++e) {
        int64_t n = 0;
        for (int64_t t = 0; t < T; ++t)
            for (int k = 0; k < K; ++k)
                if (ids[t * K + k] == e) { tok[n] = t; slot[n] = k; ++n; break; }
        if (!n) continue;
        if (!w_up[e]) { rc = -3; break; }
        for (int64_t j = 0; j < n; ++j)
            memcpy(xr + (size_t)j * (size_t)H * (size_t)es,
                   (const char *)x + (size_t)tok[j] * (size_t)H * (size_t)es,
                   (size_t)H * (size_t)es);
        eko_ffn(xr, n, H, I, w_up[e], w_gate[e], w_down[e], dt, 0, yr, NULL);
        for (int64_t j = 0; j < n; ++j) {
            float wv = load_act(w, tok[j] * K + slot[j], w_dt);
            for (int64_t c = 0; c < H; ++c) {
                float p = load_act(yr, j * H + c, dt) * wv;
                if (w_dt != EKO_F32) p = round_act(p, dt);
                float *a = acc + tok[j] * H + c;
                *a = round_act(*a + round_act(p, dt), dt);
            }
        }
    }
    for (int64_t i = 0; i < T * H; ++i) store_act(y, i, acc[i], dt);
    free(acc); free(xr); free(yr); free(tok); free(slot);
    return rc;
}
