// Weighted scatter-combine and weight ingestion kernels (HBM-bound copies).
#include "ek_internal.h"

namespace ek {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// y[t, :] = sum_k w[t,k] * Yp[inv_perm[t*K + k], :], k ascending.
// Follows the shim's weighted sum (qwen3_moe.py:102-104): the product tensor
// has the promoted dtype of its operands, torch.sum accumulates in fp32 and
// rounds once.  WF32 = gate weights kept in fp32 (deepseek_v3/model.py:97-103),
// so the product is not rounded.  The scatter back to [T,K,H]
// (controller/executor.rs:203-252) is folded into the indexed read.
// Fixed summation order, no atomics: bit-reproducible.
template <typename T, bool WF32>
__global__ __launch_bounds__(256) void combine_kernel(CombineArgs a)
{
    typedef T V8 __attribute__((ext_vector_type(8)));
    const int64_t t = blockIdx.x;
    const int64_t c = ((int64_t)blockIdx.y * 256 + threadIdx.x) * 8;
    if (c >= a.H) return;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    // The rows of up to 8 slots are requested together, then added in slot order.  Every load is
    // unconditional (slots past K and pairs without a row re-read a valid address and are left out
    // of the sum): conditional loads became a chain of branches in which each load waited for the
    // one before it.  The rows are read once: non-temporal loads.  (8192 tokens of the
    // DeepSeek-V3 layer on MI355X: 235 us with the branches, 216 with non-temporal loads alone.)
    for (int k0 = 0; k0 < a.K; k0 += 8) {
        int32_t pos[8];
        float wv[8];
        bool valid[8];
        V8 v[8];
        if ((a.K & 7) == 0) {
            // eight positions and eight gate weights as whole vectors (the addresses are the same for
            // every lane: two to four scalar loads in flight together)
            typedef int32_t I4 __attribute__((ext_vector_type(4)));
            typedef float F4 __attribute__((ext_vector_type(4)));
            typedef T T8 __attribute__((ext_vector_type(8)));
            const I4 *ip = (const I4 *)(a.inv_perm + t * a.K + k0);
            const I4 p0 = ip[0], p1 = ip[1];
            if constexpr (WF32) {
                const F4 *wp = (const F4 *)((const float *)a.w + t * a.K + k0);
                const F4 w0 = wp[0], w1 = wp[1];
#pragma unroll
                for (int j = 0; j < 4; ++j) { wv[j] = w0[j]; wv[4 + j] = w1[j]; }
            } else {
                const T8 w8 = *(const T8 *)((const T *)a.w + t * a.K + k0);
#pragma unroll
                for (int j = 0; j < 8; ++j) wv[j] = (float)w8[j];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) { pos[j] = p0[j]; pos[4 + j] = p1[j]; }
#pragma unroll
            for (int j = 0; j < 8; ++j) valid[j] = pos[j] >= 0;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int k = min(k0 + j, a.K - 1);
                pos[j] = a.inv_perm[t * a.K + k];
                wv[j] = WF32 ? ((const float *)a.w)[t * a.K + k] : (float)((const T *)a.w)[t * a.K + k];
                valid[j] = k0 + j < a.K && pos[j] >= 0;
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
            v[j] = __builtin_nontemporal_load((const V8 *)((const T *)a.yp + (int64_t)max(pos[j], 0) * a.H + c));
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (!valid[j]) continue;       // (the same for every lane)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float p = wv[j] * (float)v[j][i];
                if (!WF32) p = (float)(T)p;
                acc[i] = acc[i] + p;
            }
        }
    }
    V8 o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (T)acc[i];
    if (a.shared) {
        // hidden_states + shared_experts(residuals), both in the activation dtype
        // (deepseek_v3/model.py:152)
        const V8 sh = *(const V8 *)((const T *)a.shared + t * a.H + c);
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (T)((float)o[i] + (float)sh[i]);
    }
    *(V8 *)((T *)a.y + t * a.H + c) = o;
}

void launch_combine(const CombineArgs &a, hipStream_t s)
{
    if (a.T <= 0) return;
    dim3 grid((unsigned)a.T, (unsigned)((a.H / 8 + 255) / 256));
    if (a.act == 0) {
        if (a.w_f32) hipLaunchKernelGGL((combine_kernel<__bf16, true>), grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL((combine_kernel<__bf16, false>), grid, dim3(256), 0, s, a);
    } else {
        if (a.w_f32) hipLaunchKernelGGL((combine_kernel<_Float16, true>), grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL((combine_kernel<_Float16, false>), grid, dim3(256), 0, s, a);
    }
}

// ---- batched row copies -------------------------------------------------------

__global__ __launch_bounds__(256) void rows_copy_kernel(const RowCopy *segs)
{
    const RowCopy c = segs[blockIdx.x];
    const int per_row = c.row_bytes >> 4;
    const int64_t units = (int64_t)c.rows * per_row;
    for (int64_t u = (int64_t)blockIdx.y * 256 + threadIdx.x; u < units; u += (int64_t)gridDim.y * 256) {
        const int64_t r = u / per_row, k = u - r * per_row;
        *(uint4 *)(c.dst + r * c.dst_pitch + k * 16) = *(const uint4 *)(c.src + r * c.src_pitch + k * 16);
    }
}

void launch_rows_copy(const RowCopy *segs, int n, hipStream_t s)
{
    if (n <= 0) return;
    hipLaunchKernelGGL(rows_copy_kernel, dim3((unsigned)n, 8), dim3(256), 0, s, segs);
}

// ---- weight ingestion ---------------------------------------------------------

// OCP fp8 e4m3fn -> fp32 (no infinities; 0x7f / 0xff are NaN)
__device__ __forceinline__ float f8e4m3_to_f32(uint8_t b)
{
    const uint32_t sign = (uint32_t)(b & 0x80u) << 24;
    const uint32_t exp = (b >> 3) & 0xfu, man = b & 0x7u;
    float v;
    if (exp == 0) v = (float)man * 0.001953125f;                          // subnormal: man * 2^-9
    else if (exp == 15 && man == 7) v = __builtin_nanf("");
    else v = __builtin_bit_cast(float, ((exp + 120u) << 23) | (man << 20));
    return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) | sign);
}

__device__ __forceinline__ float load_src(const void *src, int dt, int64_t i)
{
    switch (dt) {
    case 0: return (float)((const __bf16 *)src)[i];
    case 1: return (float)((const _Float16 *)src)[i];
    case 3: return (float)((const int8_t *)src)[i];
    case 4: return f8e4m3_to_f32(((const uint8_t *)src)[i]);
    default: return ((const float *)src)[i];
    }
}

// One thread writes one lane's 16 bytes of one chunk.
// scale (optional): one factor per 128x128 block, [ceil(N/128), ceil(K/128)]; the product is
// formed in fp32 and rounded once, as w8a16_activate does (ffn/expert_torch.rs:45-52).
template <typename T>
__global__ __launch_bounds__(256) void tile_weights16_kernel(const void *src, int src_dt, int64_t N,
                                                            int64_t K, uint8_t *dst, int m, int nmat,
                                                            const void *scale, int scale_dt)
{
    typedef T V8 __attribute__((ext_vector_type(8)));
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t KT = K / 32, total = (N / 16) * KT * 64;
    if (idx >= total) return;
    const int l = idx & 63;
    const int64_t chunk = idx >> 6, nt = chunk / KT, kt = chunk % KT;
    const int64_t row = nt * 16 + (l & 15), col = kt * 32 + (l >> 4) * 8;
    V8 v;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float f = load_src(src, src_dt, row * K + col + i);
        if (scale) f = f * load_src(scale, scale_dt, (row >> 7) * ((K + 127) >> 7) + ((col + i) >> 7));
        v[i] = (T)f;
    }
    *(V8 *)(dst + (chunk * nmat + m) * kChunkBytes + l * 16) = v;
}

// flip: int8 is stored offset-binary (q ^ 0x80, see dequant_u8x4); fp8 bytes are kept as they are
__global__ __launch_bounds__(256) void tile_weights8_kernel(const uint8_t *src, int64_t N, int64_t K,
                                                           uint8_t *dst, int m, int nmat, uint32_t flip)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t KT = K / 64, total = (N / 16) * KT * 64;
    if (idx >= total) return;
    const int l = idx & 63;
    const int64_t chunk = idx >> 6, nt = chunk / KT, kt = chunk % KT;
    const int64_t row = nt * 16 + (l & 15), col = kt * 64 + (l >> 4) * 16;
    uint4 v = *(const uint4 *)(src + row * K + col);
    v.x ^= flip; v.y ^= flip; v.z ^= flip; v.w ^= flip;
    *(uint4 *)(dst + (chunk * nmat + m) * kChunkBytes + l * 16) = v;
}

void launch_tile_weights(const void *src, int src_dtype, int64_t N, int64_t K, uint8_t *dst,
                         int dst_dtype, int m, int nmat, const void *block_scale, int scale_dtype,
                         hipStream_t s)
{
    if (dst_dtype == 3 || dst_dtype == 4) {      // EK_I8, EK_F8E4M3: one byte per weight, kept as stored
        const int64_t total = (N / 16) * (K / 64) * 64;
        hipLaunchKernelGGL(tile_weights8_kernel, dim3((total + 255) / 256), dim3(256), 0, s,
                           (const uint8_t *)src, N, K, dst, m, nmat, dst_dtype == 3 ? 0x80808080u : 0u);
    } else {
        const int64_t total = (N / 16) * (K / 32) * 64;
        if (dst_dtype == 0)
            hipLaunchKernelGGL(tile_weights16_kernel<__bf16>, dim3((total + 255) / 256), dim3(256), 0,
                               s, src, src_dtype, N, K, dst, m, nmat, block_scale, scale_dtype);
        else
            hipLaunchKernelGGL(tile_weights16_kernel<_Float16>, dim3((total + 255) / 256), dim3(256),
                               0, s, src, src_dtype, N, K, dst, m, nmat, block_scale, scale_dtype);
    }
}

__global__ void scales_to_f32_kernel(const void *src, int dt, int64_t n, float *dst)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = load_src(src, dt, i);
}

void launch_scales_to_f32(const void *src, int src_dtype, int64_t n, float *dst, hipStream_t s)
{
    hipLaunchKernelGGL(scales_to_f32_kernel, dim3((n + 255) / 256), dim3(256), 0, s, src, src_dtype,
                       n, dst);
}

// A kernel that does nothing for a fixed time (one wave, `iters` sleeps of about 1000 cycles):
// the host times it alone and beside a copy of itself on another stream to learn whether the two
// streams can run kernels side by side (streams that share a hardware queue cannot).
__global__ void idle_kernel(int iters)
{
    for (int i = 0; i < iters; ++i) __builtin_amdgcn_s_sleep(16);
}

void launch_idle(int iters, hipStream_t s)
{
    hipLaunchKernelGGL(idle_kernel, dim3(1), dim3(64), 0, s, iters);
}

}  // namespace ek
