// Router kernels: logits [T,E] -> (ids [T,K], gate weights [T,K]), in front of pack.
//
//   kind 0  softmax over E, top-K, optional renormalisation, cast
//           (expertkit_torch/models/qwen3_moe.py:161-169)
//   kind 1  top-K of the raw logits, weights = the logits (expertkit_vllm/experts/grpc_expert.py:120-121)
//   kind 2  top-K of the logits, softmax over the K      (expertkit_vllm/models/deepseek_v2.py:123-128)
//   kind 3  top-K of the logits, sigmoid of the K        (expertkit_vllm/models/deepseek_v2.py:123-130)
//   kind 4  DeepSeek-V3 group-limited routing: sigmoid scores, + correction bias for the choice
//           only, groups ranked by the sum of their two best, top-K inside the best groups,
//           weights = unbiased scores / (sum + 1e-20) * routed_scaling_factor.  The reference
//           calls transformers' DeepseekV3TopkRouter for it (deepseek_v3/model.py:142).
//
// Every choice is "larger value first, lower index on equal values", so the result is a function
// of the input.  One wavefront per token: lane l holds experts l, l+64, ... in registers; each of
// the K picks is one wave-wide arg-max.  HBM-bound: T*E logits in, T*K pairs out.
#include "ek_internal.h"

namespace ek {

// exp(x) from IEEE operations only (fma, mul, add, round-to-nearest-even), so that the host
// restatement of this file's arithmetic gives the same bits.  Cody-Waite reduction by ln 2 and the
// degree-5 Cephes polynomial; the argument is clamped to the range whose result is a normal number.
__device__ __forceinline__ float exp_ieee(float x)
{
    x = x < -87.0f ? -87.0f : (x > 88.0f ? 88.0f : x);
    const float n = __builtin_rintf(x * 1.44269504088896341f);
    float r = __builtin_fmaf(n, -0.693359375f, x);
    r = __builtin_fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    const float y = __builtin_fmaf(r * r, p, r) + 1.0f;
    return y * __builtin_bit_cast(float, (uint32_t)((int32_t)n + 127) << 23);
}
__device__ __forceinline__ float sigmoid_ieee(float x) { return 1.0f / (1.0f + exp_ieee(-x)); }

struct Pick { float v; int32_t i; };
// b goes before a?
__device__ __forceinline__ bool before(const Pick &b, const Pick &a)
{
    return b.i >= 0 && (a.i < 0 || b.v > a.v || (b.v == a.v && b.i < a.i));
}
__device__ __forceinline__ Pick wave_best(Pick p)
{
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        Pick o;
        o.v = __shfl_xor(p.v, d);
        o.i = __shfl_xor(p.i, d);
        if (before(o, p)) p = o;
    }
    return p;
}

__device__ __forceinline__ float load_logit(const void *p, int dt, int64_t i)
{
    if (dt == 0) return (float)((const __bf16 *)p)[i];
    if (dt == 1) return (float)((const _Float16 *)p)[i];
    return ((const float *)p)[i];
}
__device__ __forceinline__ void store_w(void *p, int dt, int64_t i, float v)
{
    if (dt == 0) ((__bf16 *)p)[i] = (__bf16)v;
    else if (dt == 1) ((_Float16 *)p)[i] = (_Float16)v;
    else ((float *)p)[i] = v;
}

constexpr int kRouterWaves = 4;     // tokens per workgroup
constexpr int kRouterSlots = 16;    // experts per lane: E <= 1024

__global__ __launch_bounds__(kRouterWaves * 64) void router_kernel(RouterArgs a)
{
    extern __shared__ float lds[];   // kind 4: [waves][2][E] choice values, then scores
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t t = (int64_t)blockIdx.x * kRouterWaves + wave;
    if (t >= a.T) return;   // whole waves leave; there is no workgroup barrier below
    const int E = a.E, K = a.K;
    float v[kRouterSlots];          // the value the choice is made on
    float sc[kRouterSlots];         // kind 4: unbiased score
#pragma unroll
    for (int j = 0; j < kRouterSlots; ++j) {
        const int e = j * 64 + lane;
        v[j] = e < E ? load_logit(a.logits, a.logits_dt, t * E + e) : 0.f;
        sc[j] = 0.f;
    }
    float m = 0.f, s = 1.f;
    if (a.kind == 0) {
        // softmax statistics over all experts
        float lm = -__builtin_inff();
#pragma unroll
        for (int j = 0; j < kRouterSlots; ++j) if (j * 64 + lane < E && v[j] > lm) lm = v[j];
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) { const float o = __shfl_xor(lm, d); lm = o > lm ? o : lm; }
        m = lm;
        float ls = 0.f;
#pragma unroll
        for (int j = 0; j < kRouterSlots; ++j) if (j * 64 + lane < E) ls += exp_ieee(v[j] - m);
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) ls += __shfl_xor(ls, d);
        s = ls;
    } else if (a.kind == 4) {
        float *cv = lds + (size_t)wave * 2 * E, *sv = cv + E;
        const int G = E / a.n_group;
#pragma unroll
        for (int j = 0; j < kRouterSlots; ++j) {
            const int e = j * 64 + lane;
            if (e < E) {
                sc[j] = sigmoid_ieee(v[j]);
                v[j] = a.bias ? sc[j] + a.bias[e] : sc[j];
                cv[e] = v[j];
                sv[e] = sc[j];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // lane g ranks group g by the sum of its two best choice values
        Pick gp{0.f, -1};
        if (lane < a.n_group) {
            float b0 = -__builtin_inff(), b1 = -__builtin_inff();
            for (int i = 0; i < G; ++i) {
                const float c = cv[lane * G + i];
                if (c > b0) { b1 = b0; b0 = c; }
                else if (c > b1) b1 = c;
            }
            gp = Pick{b0 + b1, lane};
        }
        uint64_t keep = 0;
        for (int k = 0; k < a.topk_group; ++k) {
            const Pick w = wave_best(gp);
            keep |= 1ull << w.i;
            if (lane == w.i) gp.i = -1;
        }
        const float masked = a.mask_neg_inf ? -__builtin_inff() : 0.f;
#pragma unroll
        for (int j = 0; j < kRouterSlots; ++j) {
            const int e = j * 64 + lane;
            if (e < E && !((keep >> (e / G)) & 1ull)) v[j] = masked;
        }
    }
    // K picks; lane k keeps pick k
    uint32_t taken = 0;
    Pick mine{0.f, -1};
    for (int k = 0; k < K; ++k) {
        Pick p{0.f, -1};
#pragma unroll
        for (int j = 0; j < kRouterSlots; ++j) {
            const int e = j * 64 + lane;
            if (e < E && !((taken >> j) & 1u) && (p.i < 0 || v[j] > p.v)) p = Pick{v[j], e};
        }
        const Pick w = wave_best(p);
        if ((w.i & 63) == lane) taken |= 1u << (w.i >> 6);
        if (lane == k) mine = w;
    }
    // weights
    float wv = 0.f;
    if (a.kind == 0) {
        wv = exp_ieee(mine.v - m) / s;
    } else if (a.kind == 1) {
        wv = mine.v;
    } else if (a.kind == 2) {
        const float top = __shfl(mine.v, 0);
        wv = exp_ieee(mine.v - top);
    } else if (a.kind == 3) {
        wv = sigmoid_ieee(mine.v);
    } else {
        const float *sv = lds + (size_t)wave * 2 * E + E;
        wv = lane < K ? sv[mine.i] : 0.f;
    }
    const bool norm = a.kind == 2 || ((a.kind == 0 || a.kind == 4) && a.renorm);
    if (norm) {
        float tot = 0.f;
        for (int k = 0; k < K; ++k) tot += __shfl(wv, k);   // k ascending, as a sequential sum
        if (a.kind == 4) tot += 1e-20f;
        wv = wv / tot;
    }
    if (a.kind == 4) wv = wv * a.routed_scaling;
    if (lane < K) {
        a.ids[t * K + lane] = mine.i;
        store_w(a.w, a.w_dt, t * K + lane, wv);
    }
}

hipError_t launch_router(const RouterArgs &a, hipStream_t s)
{
    if (a.T <= 0) return hipSuccess;
    const size_t lds = a.kind == 4 ? sizeof(float) * 2 * (size_t)a.E * kRouterWaves : 0;
    hipLaunchKernelGGL(router_kernel, dim3((unsigned)((a.T + kRouterWaves - 1) / kRouterWaves)),
                       dim3(kRouterWaves * 64), lds, s, a);
    return hipGetLastError();
}

}  // namespace ek
