// Measured ceilings of the device the library runs on, for the benchmark's roofline lines:
// a plain copy, a read-only stream with non-temporal loads (the form the weight-streaming
// kernel reads expert weights in) and a register-only MFMA loop (bf16, 32x32x16).  Published
// peaks are what roofline fractions are quoted against; these say how much of them any kernel can
// reach on this very box.
#include "../../include/ek_hip.h"
#include "ek_mfma.h"

#include <algorithm>
#include <vector>

namespace ek { void set_last_error(const char *msg); }

namespace {

// dst[i] = src[i], 16 bytes per lane and load; a workgroup moves 16 KiB per step (4 loads in
// flight per lane, each a contiguous 4 KiB across the workgroup)
__global__ __launch_bounds__(256) void peak_copy_kernel(const uint4 *src, uint4 *dst, size_t n16)
{
    constexpr int D = 4;
    const size_t stride = (size_t)gridDim.x * 256 * D;
    for (size_t i = (size_t)blockIdx.x * 256 * D + threadIdx.x; i + (D - 1) * 256 < n16; i += stride) {
        uint4 v[D];
#pragma unroll
        for (int d = 0; d < D; ++d) v[d] = src[i + d * 256];
#pragma unroll
        for (int d = 0; d < D; ++d) dst[i + d * 256] = v[d];
    }
}

// reads n16 x 16 bytes once with non-temporal loads, 8 in flight per lane (32 KiB per workgroup
// and step); the xor of what was read is stored only if it has a value no input produces, so the
// loads cannot be dropped
__global__ __launch_bounds__(256) void peak_read_kernel(const uint4 *src, size_t n16, uint32_t *sink)
{
    constexpr int D = 8;
    const size_t stride = (size_t)gridDim.x * 256 * D;
    uint32_t acc = 0;
    for (size_t i = (size_t)blockIdx.x * 256 * D + threadIdx.x; i + (D - 1) * 256 < n16; i += stride) {
        uint4 v[D];
#pragma unroll
        for (int d = 0; d < D; ++d) v[d] = ek::ldg16_once(src + i + d * 256);
#pragma unroll
        for (int d = 0; d < D; ++d) acc ^= v[d].x ^ v[d].y ^ v[d].z ^ v[d].w;
    }
    if (acc == 0x9e3779b9u) *sink = acc;     // the buffer is zero-filled: never true
}

// iters x 8 independent MFMA 32x32x16 bf16 per wave on register operands: 8 accumulators keep the
// matrix pipe of a SIMD busy from one wave; two waves per SIMD as the tile kernel runs
__global__ __launch_bounds__(512, 1) void peak_mfma_kernel(int iters, float *sink)
{
    using V8 = ek::bf16x8;
    ek::f32x16 acc[8];
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;
    ek::u32x4 raw = {0x3f803f80u + threadIdx.x, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
    const V8 va = __builtin_bit_cast(V8, raw), vb = va;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int a = 0; a < 8; ++a) acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, vb, acc[a], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int a = 0; a < 8; ++a) s += acc[a][0];
    if (s == -1.f) *sink = s;                // sums of positive products: never true
}

// The same loop on operands with random signs, exponents and mantissas that change from one MFMA to
// the next, as a matrix product's do: the chip's power limit sets the clock, and the power an MFMA
// draws grows with the bits that toggle on its operand buses, so this is the rate real data can reach.
__global__ __launch_bounds__(512, 1) void peak_mfma_random_kernel(int iters, float *sink)
{
    using V8 = ek::bf16x8;
    ek::f32x16 acc[8];
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;
    V8 va[4], vb[4];
    uint32_t h = (blockIdx.x * 512u + threadIdx.x) * 0x9e3779b9u + 0x7f4a7c15u;
    auto next = [&]() -> uint32_t {
        h ^= h << 13; h ^= h >> 17; h ^= h << 5;
        // two bf16 values in [0.5, 2) with random signs
        return (h & 0x80ff80ffu) | 0x3f003f00u;
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        ek::u32x4 ra = {next(), next(), next(), next()}, rb = {next(), next(), next(), next()};
        va[i] = __builtin_bit_cast(V8, ra);
        vb[i] = __builtin_bit_cast(V8, rb);
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int a = 0; a < 8; ++a)
            acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[a & 3], vb[(a >> 1) & 3], acc[a], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int a = 0; a < 8; ++a) s += acc[a][0];
    if (s == 1.2345678e33f) *sink = s;       // sums of at most 2.6e6 products below 4: never true
}

// The random-operand loop with the tile kernel's conversion work beside every MFMA: per MFMA half
// a dword of offset-binary int8 goes through dequant_u8x4 (4 conversions, 4 fused multiply-adds, 2
// packed roundings per dword: 5 vector instructions per MFMA, what a 128-row tile of one-byte
// weights needs) and becomes part of a later A operand.  Operands never leave the registers: the
// ceiling of the W8A16 tile path before any byte is moved.
__global__ __launch_bounds__(512, 1) void peak_mfma_dequant_kernel(int iters, float *sink)
{
    using V8 = ek::bf16x8;
    ek::f32x16 acc[8];
#pragma unroll
    for (int a = 0; a < 8; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;
    uint32_t h = (blockIdx.x * 512u + threadIdx.x) * 0x9e3779b9u + 0x7f4a7c15u;
    auto next = [&]() -> uint32_t {
        h ^= h << 13; h ^= h >> 17; h ^= h << 5;
        return h;
    };
    V8 vb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        ek::u32x4 rb;
#pragma unroll
        for (int d = 0; d < 4; ++d) rb[d] = (next() & 0x80ff80ffu) | 0x3f003f00u;
        vb[i] = __builtin_bit_cast(V8, rb);
    }
    uint32_t wq[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) wq[i] = next();
    const float s = 0.0123f + 1e-6f * (float)(threadIdx.x & 31), c = -128.f * s;
    ek::u32x4 va[2];
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        const ek::u32x2 lo = ek::dequant_u8x4<__bf16>(next(), s, c), hi = ek::dequant_u8x4<__bf16>(next(), s, c);
        va[g] = ek::u32x4{lo[0], lo[1], hi[0], hi[1]};
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int a = 0; a < 8; ++a) {
            acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(V8, va[a & 1]), vb[(a >> 1) & 3], acc[a], 0, 0, 0);
            if ((a & 1) == 1) {
                // one dword per two MFMAs: the bytes change with the iteration
                const int d = a >> 1;
                const ek::u32x2 v = ek::dequant_u8x4<__bf16>(wq[d] + (uint32_t)it * 0x01030507u, s, c);
                va[d & 1][(d >> 1) * 2] = v[0];
                va[d & 1][(d >> 1) * 2 + 1] = v[1];
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float t = 0.f;
#pragma unroll
    for (int a = 0; a < 8; ++a) t += acc[a][0];
    if (t == 1.2345678e33f) *sink = t;       // never true for sums of this size
}

double median(std::vector<float> v)
{
    std::sort(v.begin(), v.end());
    return v[v.size() / 2];
}

}  // namespace

extern "C" ek_status ek_measure_peaks(int32_t device_id, ek_peaks *out)
{
    if (!out) { ek::set_last_error("out is NULL"); return EK_INVALID_INPUT; }
    *out = ek_peaks{0.0, 0.0, 0.0, 0.0, 0.0};
    int prev = -1;
    (void)hipGetDevice(&prev);
    if (hipSetDevice(device_id) != hipSuccess) {
        (void)hipGetLastError();
        ek::set_last_error("hipSetDevice failed");
        return EK_HIP_ERROR;
    }
    const size_t bytes = (size_t)4 << 30;   // well beyond the 256 MiB last-level cache
    void *a = nullptr, *b = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipStream_t s = nullptr;
    hipError_t e = hipMalloc(&a, bytes);
    if (e == hipSuccess) e = hipMalloc(&b, bytes);
    if (e == hipSuccess) e = hipMemset(a, 0, bytes);
    if (e == hipSuccess) e = hipMemset(b, 0, bytes);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    const size_t n16 = bytes / 16;
    auto timed = [&](auto launch, int reps) -> double {
        std::vector<float> ms;
        for (int r = 0; r < reps + 2 && e == hipSuccess; ++r) {
            e = hipEventRecord(e0, s);
            launch();
            if (e == hipSuccess) e = hipGetLastError();
            if (e == hipSuccess) e = hipEventRecord(e1, s);
            if (e == hipSuccess) e = hipEventSynchronize(e1);
            float t = 0.f;
            if (e == hipSuccess) e = hipEventElapsedTime(&t, e0, e1);
            if (r >= 2) ms.push_back(t);      // two warm-ups
        }
        return ms.empty() ? 0.0 : median(ms) * 1e-3;
    };
    if (e == hipSuccess) {
        const double t = timed([&] { hipLaunchKernelGGL(peak_copy_kernel, dim3(8192), dim3(256), 0, s, (const uint4 *)a, (uint4 *)b, n16); }, 9);
        if (t > 0) out->copy_gbps = 2.0 * (double)bytes / t / 1e9;
    }
    if (e == hipSuccess) {
        const double t = timed([&] { hipLaunchKernelGGL(peak_read_kernel, dim3(8192), dim3(256), 0, s, (const uint4 *)a, n16, (uint32_t *)b); }, 9);
        if (t > 0) out->read_nt_gbps = (double)bytes / t / 1e9;
    }
    if (e == hipSuccess) {
        int cus = 256;
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, device_id) == hipSuccess) cus = prop.multiProcessorCount;
        else (void)hipGetLastError();
        const int iters = 20000;
        const double t = timed([&] { hipLaunchKernelGGL(peak_mfma_kernel, dim3(cus), dim3(512), 0, s, iters, (float *)b); }, 5);
        // per workgroup: 8 waves x iters x 8 MFMAs x 2 * 32 * 32 * 16 flop
        if (t > 0) out->mfma_bf16_tflops = (double)cus * 8.0 * iters * 8.0 * 32768.0 / t / 1e12;
        const double tr = timed([&] { hipLaunchKernelGGL(peak_mfma_random_kernel, dim3(cus), dim3(512), 0, s, iters, (float *)b); }, 5);
        if (tr > 0) out->mfma_bf16_random_tflops = (double)cus * 8.0 * iters * 8.0 * 32768.0 / tr / 1e12;
        const double td = timed([&] { hipLaunchKernelGGL(peak_mfma_dequant_kernel, dim3(cus), dim3(512), 0, s, iters, (float *)b); }, 5);
        if (td > 0) out->mfma_bf16_dequant_tflops = (double)cus * 8.0 * iters * 8.0 * 32768.0 / td / 1e12;
    }
    if (s) (void)hipStreamDestroy(s);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (a) (void)hipFree(a);
    if (b) (void)hipFree(b);
    if (prev >= 0) (void)hipSetDevice(prev);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        ek::set_last_error(hipGetErrorString(e));
        return e == hipErrorOutOfMemory ? EK_OOM : EK_HIP_ERROR;
    }
    return EK_OK;
}
