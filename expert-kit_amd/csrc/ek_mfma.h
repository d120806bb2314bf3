// MFMA operand types and the shared W8A16 dequantisation / SwiGLU epilogue.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ek {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <typename T> struct Act;
template <> struct Act<__bf16> {
    using V8 = bf16x8;
    static __device__ __forceinline__ f32x4 mfma(V8 a, V8 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x16 mfma32(V8 a, V8 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Act<_Float16> {
    using V8 = f16x8;
    static __device__ __forceinline__ f32x4 mfma(V8 a, V8 b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x16 mfma32(V8 a, V8 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// 16-byte load through the global (not flat) path.  Pointers that come out of
// a struct in memory have no known address space, and a flat load also ties
// up the LDS counter that the fragment reads wait on.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ldg16(const void *p)
{
    typedef const __attribute__((address_space(1))) u32x4 *gptr;
    const u32x4 v = *(gptr)(uintptr_t)p;
    return __builtin_bit_cast(uint4, v);
}

// The same for bytes that are read once (expert weights in the weight-streaming kernel): a
// non-temporal load.  A plain read-only kernel reaches 7.0-7.1 TB/s with it on MI355X against
// 6.2-6.3 TB/s with ordinary loads (the lines are not kept in the caches on their way in).
__device__ __forceinline__ uint4 ldg16_once(const void *p)
{
    typedef const __attribute__((address_space(1))) u32x4 *gptr;
    const u32x4 v = __builtin_nontemporal_load((gptr)(uintptr_t)p);
    return __builtin_bit_cast(uint4, v);
}

template <typename T> __device__ __forceinline__ float rnd(float v) { return (float)(T)v; }

// Two fp32 values -> one dword holding their round-to-nearest-even 16-bit forms
// (v_cvt_pk_bf16_f32 / v_cvt_pkrtz is not used: rtz would differ from the CPU cast).
template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2<__bf16>(float lo, float hi)
{
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
template <> __device__ __forceinline__ uint32_t pack2<_Float16>(float lo, float hi)
{
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}

// 4 offset-binary bytes (one dword) of one output channel -> 4 dequantised weights
// rne_T((u - 128) * s) as two packed dwords; c = -128 * s
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
template <typename T> __device__ __forceinline__ u32x2 dequant_u8x4(uint32_t w, float s, float c)
{
    u32x2 r;
    r[0] = pack2<T>(__builtin_fmaf((float)(w & 0xffu), s, c), __builtin_fmaf((float)((w >> 8) & 0xffu), s, c));
    r[1] = pack2<T>(__builtin_fmaf((float)((w >> 16) & 0xffu), s, c), __builtin_fmaf((float)(w >> 24), s, c));
    return r;
}

// 8 offset-binary bytes (two dwords) of one output channel -> 8 dequantised
// weights rne_T((u - 128) * s); c = -128 * s
template <typename T>
__device__ __forceinline__ typename Act<T>::V8 dequant_u8x8(uint32_t lo, uint32_t hi, float s, float c)
{
    u32x4 r;
    r[0] = pack2<T>(__builtin_fmaf((float)(lo & 0xffu), s, c), __builtin_fmaf((float)((lo >> 8) & 0xffu), s, c));
    r[1] = pack2<T>(__builtin_fmaf((float)((lo >> 16) & 0xffu), s, c), __builtin_fmaf((float)(lo >> 24), s, c));
    r[2] = pack2<T>(__builtin_fmaf((float)(hi & 0xffu), s, c), __builtin_fmaf((float)((hi >> 8) & 0xffu), s, c));
    r[3] = pack2<T>(__builtin_fmaf((float)((hi >> 16) & 0xffu), s, c), __builtin_fmaf((float)(hi >> 24), s, c));
    return __builtin_bit_cast(typename Act<T>::V8, r);
}

// The same for OCP fp8 (e4m3fn) bytes with a block scale: rne_T(f32(b) * s), the arithmetic of
// the reference's w8a16_activate (ek-computation/src/ffn/expert_torch.rs:24-53).
// v_cvt_f32_fp8 converts one selected byte exactly (checked for all 256 values on gfx950).
template <typename T> __device__ __forceinline__ u32x2 dequant_f8x4(uint32_t w, float s)
{
    u32x2 r;
    r[0] = pack2<T>(__builtin_amdgcn_cvt_f32_fp8(w, 0) * s, __builtin_amdgcn_cvt_f32_fp8(w, 1) * s);
    r[1] = pack2<T>(__builtin_amdgcn_cvt_f32_fp8(w, 2) * s, __builtin_amdgcn_cvt_f32_fp8(w, 3) * s);
    return r;
}
template <typename T>
__device__ __forceinline__ typename Act<T>::V8 dequant_f8x8(uint32_t lo, uint32_t hi, float s)
{
    const u32x2 a = dequant_f8x4<T>(lo, s), b = dequant_f8x4<T>(hi, s);
    const u32x4 r = {a[0], a[1], b[0], b[1]};
    return __builtin_bit_cast(typename Act<T>::V8, r);
}

// exp(x) from IEEE-754 single operations only (fused multiply-add, multiply, add, all rounded to
// nearest even): Cody-Waite reduction by ln 2, the degree-5 polynomial of Cephes' expf, scaling by
// 2^n (ldexp: exact, overflows to +inf, never rounds for the arguments kept).  The argument is
// clamped to [-87, 89]: down there the result is still a normal number, up there it has
// overflowed to +inf as expf does beyond 88.72.  Within 2 ulp of the exact value, and the same
// bits on any conforming machine, so a CPU restatement of these lines reproduces the kernels'
// silu exactly.
__device__ __forceinline__ float expf_ieee(float x)
{
    x = __builtin_amdgcn_fmed3f(x, -87.0f, 89.0f);
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
    return __builtin_ldexpf(y, (int)n);
}

// SwiGLU with the reference's storage roundings: up, gate, silu(gate) and the
// product are each a materialised tensor of the activation dtype
// (ek-computation/src/ffn/expert_torch.rs:81-83).
template <typename T> __device__ __forceinline__ T swiglu_rounded(float acc_up, float acc_gate)
{
    const float up = rnd<T>(acc_up);
    const float gate = rnd<T>(acc_gate);
    // silu in fp32 as a CPU backend forms it: gate / (1 + exp(-gate)) with a 2-ulp exp and a
    // correctly rounded division, then the storage rounding (held for every one of the 65536 gate
    // values of either 16-bit type by a test that feeds all of them through both kernel families).
    // The hardware's exp2 and reciprocal (1 ulp each) would be a quarter of the instructions and
    // cost the tile kernel 1 % less time (7 % at contractions as short as Qwen3's), but move about
    // one element of h in 10^4 by one 16-bit ulp, which showed in the layer's output as
    // outliers of up to 2.7e-2 x RMS against the reference-rounded result where libtorch's own
    // evaluation stays at 1.2e-2 (DeepSeek-V3 decode, sampled tokens); with this form the
    // kernels score what libtorch scores on the same tokens.  (A reciprocal with one residual
    // correction in place of the division was tried: the reciprocal of 1 + e^87.5 and beyond is
    // a denormal, which v_rcp_f32 flushes, and three bf16 gate values came out as 0.)
    const float sg = rnd<T>(gate / (1.0f + expf_ieee(-gate)));
    return (T)(up * sg);
}

}  // namespace ek
