// Ragged grouped SwiGLU FFN, weight-streaming kernel (work items of <= 16 rows).
//
// Computes, per expert segment, the four ops of TorchFFN's closure
// (ek-computation/src/ffn/expert_torch.rs:81-84):
//   stage 1:  h   = (x . W_up^T) * silu(x . W_gate^T)
//   stage 2:  out = h . W_down^T
// with the reference's storage roundings (up, gate, silu(gate), h and out are
// each rounded to the activation dtype) and fp32 accumulation on MFMA.
//
// Regime: a handful of rows per expert, so the kernel is bound by streaming
// every active expert's weights from HBM exactly once.  One wavefront owns NG
// groups of 16 output channels and walks the whole contraction:
//   - weights are the MFMA "A" operand (16 channels x 32 k), fetched with one
//     16-byte load per lane straight from the chunked HBM layout (no LDS);
//   - the <= 16 activation rows of the segment are the "B" operand (32 k x 16
//     rows), re-read from L2 by every wave;
//   - D loads deep software prefetch keeps >= D KiB per wave in flight
//     (measured best on MI355X: one channel tile of up+gate per wave, 8 deep,
//     for stage 1; two channel tiles, 8 deep, for stage 2).
// int8 weights are dequantised in registers to exactly the tensor a CPU backend
// would hold, W[n,k] = rne_16bit(f32(q[n,k]) * f32(scale[n])): they are stored
// offset-binary (u = q + 128) so v_cvt_f32_ubyteN converts them, one
// fma(u, s, -128 s) per element gives the exact fp32 product q*s (16
// significant bits), and v_cvt_pk_bf16_f32 rounds two of them to nearest even.
// Each lane owns one output channel of the A operand, so s is a lane scalar.
#include "ek_internal.h"
#include "ek_mfma.h"

namespace ek {

template <typename T, bool W8, int NMAT, int NG, int D>
__global__ __launch_bounds__(256) void ffn_stream_kernel(FfnArgs a)
{
    using V8 = typename Act<T>::V8;
    constexpr int KE = W8 ? 64 : 32;   // contraction elements per chunk
    constexpr int XV = W8 ? 2 : 1;     // 16-byte activation loads per chunk per lane
    constexpr int NW = NMAT * NG;      // weight chunks per k step per wave

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if ((int)blockIdx.y >= a.lists.count[kListStream]) return;
    const WorkItem item = a.lists.items[kListStream][blockIdx.y];
    const int e = item.expert, seg0 = item.row0, n = item.nrows;
    const int NT = a.N >> 4;
    const int nt0 = (blockIdx.x * 4 + wave) * NG;
    if (nt0 >= NT) return;
    const ExpertSlab slab = a.slabs[e];
    const uint8_t *wmat = NMAT == 2 ? slab.upgate : slab.down;
    if (wmat == nullptr) return;   // expert not loaded: pack has flagged the call
    const int KT = a.Kdim / KE;
    const int j = lane & 15, g = lane >> 4;

    const uint8_t *wp[NG];
#pragma unroll
    for (int gi = 0; gi < NG; ++gi)
        wp[gi] = wmat + (int64_t)(nt0 + gi) * KT * (NMAT * kChunkBytes) + lane * 16;

    // per-lane dequantisation constants: the lane's channel of each A operand
    float ws[NW], wc[NW];
#pragma unroll
    for (int gi = 0; gi < NG; ++gi)
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            float sv = 1.f;
            if constexpr (W8) {
                const int ch = (nt0 + gi) * 16 + j;
                sv = NMAT == 2 ? (m == 0 ? slab.s_up[ch] : slab.s_gate[ch]) : slab.s_down[ch];
            }
            ws[gi * NMAT + m] = sv;
            wc[gi * NMAT + m] = -128.f * sv;
        }

    {
        constexpr int r0 = 0;   // items hold at most 16 rows
        const int jr = min(r0 + j, n - 1);   // lanes past the segment re-read its last row
        const int64_t row = a.rows ? (int64_t)a.rows[seg0 + jr] : (int64_t)(seg0 + jr);
        const T *xp = (const T *)a.x + row * a.x_stride + g * (KE / 4);

        f32x4 acc[NMAT][NG];
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) acc[m][gi] = (f32x4){0.f, 0.f, 0.f, 0.f};

        uint4 wq[D][NW];
        uint4 xq[D][XV];
#pragma unroll
        for (int d = 0; d < D; ++d) {
#pragma unroll
            for (int gi = 0; gi < NG; ++gi)
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
                    wq[d][gi * NMAT + m] = ldg16(wp[gi] + (int64_t)(d * NMAT + m) * kChunkBytes);
#pragma unroll
            for (int v = 0; v < XV; ++v) xq[d][v] = ldg16(xp + d * KE + v * 8);
        }

        for (int kt0 = 0; kt0 < KT; kt0 += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const int kt = kt0 + d;
                // consume slot d
                if constexpr (W8) {
                    const V8 x0 = __builtin_bit_cast(V8, xq[d][0]);
                    const V8 x1 = __builtin_bit_cast(V8, xq[d][1]);
#pragma unroll
                    for (int gi = 0; gi < NG; ++gi)
#pragma unroll
                        for (int m = 0; m < NMAT; ++m) {
                            const uint4 q = wq[d][gi * NMAT + m];
                            const float sv = ws[gi * NMAT + m], cv = wc[gi * NMAT + m];
                            acc[m][gi] = Act<T>::mfma(dequant_u8x8<T>(q.x, q.y, sv, cv), x0, acc[m][gi]);
                            acc[m][gi] = Act<T>::mfma(dequant_u8x8<T>(q.z, q.w, sv, cv), x1, acc[m][gi]);
                        }
                } else {
                    const V8 x0 = __builtin_bit_cast(V8, xq[d][0]);
#pragma unroll
                    for (int gi = 0; gi < NG; ++gi)
#pragma unroll
                        for (int m = 0; m < NMAT; ++m)
                            acc[m][gi] = Act<T>::mfma(__builtin_bit_cast(V8, wq[d][gi * NMAT + m]),
                                                      x0, acc[m][gi]);
                }
                // refill slot d with chunk kt + D
                if (kt + D < KT) {
#pragma unroll
                    for (int gi = 0; gi < NG; ++gi)
#pragma unroll
                        for (int m = 0; m < NMAT; ++m)
                            wq[d][gi * NMAT + m] =
                                ldg16(wp[gi] + (int64_t)((kt + D) * NMAT + m) * kChunkBytes);
#pragma unroll
                    for (int v = 0; v < XV; ++v)
                        xq[d][v] = ldg16(xp + (int64_t)(kt + D) * KE + v * 8);
                }
            }
        }

        // epilogue: lane (g, j) holds channels nt*16 + 4g + r (r = 0..3) of row r0 + j
        if (r0 + j < n) {
            T *orow = (T *)a.out + (int64_t)(seg0 + r0 + j) * a.out_stride;
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                const int ch = (nt0 + gi) * 16 + 4 * g;
                typedef T T4 __attribute__((ext_vector_type(4)));
                T4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if constexpr (NMAT == 2) {
                        o[r] = swiglu_rounded<T>(acc[0][gi][r], acc[1][gi][r]);
                    } else {
                        o[r] = (T)acc[0][gi][r];
                    }
                }
                *(uint2 *)(orow + ch) = __builtin_bit_cast(uint2, o);
            }
        }
    }
}

// Tuned on MI355X at the DeepSeek-V3 shape (see the profiles): channel tiles per wave (NG)
// and prefetch depth in k steps (D) per stage.
#ifndef EK_TUNE_S1_NG
#define EK_TUNE_S1_NG 1
#endif
#ifndef EK_TUNE_S1_D
#define EK_TUNE_S1_D 8
#endif
#ifndef EK_TUNE_S2_NG
#define EK_TUNE_S2_NG 2
#endif
#ifndef EK_TUNE_S2_D
#define EK_TUNE_S2_D 8
#endif

template <typename T, bool W8, int NMAT, int NG, int D>
static hipError_t launch_d(const FfnArgs &a, int32_t nseg, hipStream_t s)
{
    constexpr int KE = W8 ? 64 : 32;
    const int KT = a.Kdim / KE;
    const int NT = a.N / 16;
    if constexpr (D > 1) {
        if (KT % D != 0) return launch_d<T, W8, NMAT, NG, D / 2>(a, nseg, s);
    }
    dim3 grid((NT + 4 * NG - 1) / (4 * NG), nseg);
    hipLaunchKernelGGL((ffn_stream_kernel<T, W8, NMAT, NG, D>), grid, dim3(256), 0, s, a);
    return hipGetLastError();
}

template <typename T, bool W8, int NMAT>
static hipError_t launch_g(const FfnArgs &a, int32_t nseg, hipStream_t s)
{
    constexpr int NG = NMAT == 2 ? EK_TUNE_S1_NG : EK_TUNE_S2_NG;
    constexpr int D = NMAT == 2 ? EK_TUNE_S1_D : EK_TUNE_S2_D;
    const int NT = a.N / 16;
    if (NT % NG == 0) return launch_d<T, W8, NMAT, NG, D>(a, nseg, s);
    if (NT % 2 == 0) return launch_d<T, W8, NMAT, 2, D>(a, nseg, s);
    return launch_d<T, W8, NMAT, 1, D>(a, nseg, s);
}

hipError_t launch_ffn_stream(const FfnArgs &a, int stage, int act, bool w8, int64_t max_items,
                             hipStream_t s)
{
    const int32_t n_segments = (int32_t)max_items;
    if (n_segments <= 0) return hipSuccess;
    if (act == 0) {
        if (w8) return stage == 1 ? launch_g<__bf16, true, 2>(a, n_segments, s)
                                  : launch_g<__bf16, true, 1>(a, n_segments, s);
        return stage == 1 ? launch_g<__bf16, false, 2>(a, n_segments, s)
                          : launch_g<__bf16, false, 1>(a, n_segments, s);
    }
    if (w8) return stage == 1 ? launch_g<_Float16, true, 2>(a, n_segments, s)
                              : launch_g<_Float16, true, 1>(a, n_segments, s);
    return stage == 1 ? launch_g<_Float16, false, 2>(a, n_segments, s)
                      : launch_g<_Float16, false, 1>(a, n_segments, s);
}

}  // namespace ek
