// Ragged grouped SwiGLU FFN, weight-streaming kernel (work items of <= 16 rows; <= 64 rows
// in launches the host has cut wide).
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
//
// Accumulation order (the same bits whichever way a launch is shaped): the contraction is
// cut into kSlices slices of whole chunks, [KT*w/8, KT*(w+1)/8); a slice is summed by the
// MFMAs in k order into a zeroed accumulator and the slice sums are added in slice order.
// SK = 1: one wave walks all slices.  SK = 8: eight waves of one workgroup take one slice
// each and the first adds their sums, through LDS, in the same order -- used when a launch
// has too few (item, channel tile) pairs to keep the chip's memory system busy (a lone
// expert, a tiny layer), where eight times the waves mean eight times the loads in flight.
//
// RS = 4 (always with SK = 8): items of up to 64 rows, four 16-row B operands per weight
// chunk.  A lone expert with a few dozen to a few hundred rows would give the tile kernel a
// handful of workgroups; here its weights are still streamed (and dequantised) once per 64
// rows by a full grid.  Each 16-row fragment sees the MFMA sequence it would see as an item
// of its own, so a row's result does not depend on RS either.
#include "ek_internal.h"
#include "ek_mfma.h"

namespace ek {

constexpr int kSlices = 8;

constexpr int kMaxScaleBlocks = 64;   // 128-wide scale blocks along the contraction: K <= 8192

// What the pack kernel would have stored of a pair-direct call's bookkeeping; one wave.
__device__ __forceinline__ void pair_bookkeeping(const FfnArgs &a, int lane)
{
    const int32_t id = lane < a.pair_P ? a.pair_ids[lane] : 0;
    const bool bad = lane < a.pair_P && (uint32_t)id >= (uint32_t)a.n_experts;
    const bool ok = lane < a.pair_P && !bad;
    const bool unloaded = ok && a.slabs[id].upgate == nullptr;
    const uint64_t any_bad = __ballot(bad), any_unloaded = __ballot(unloaded);
    if (ok && a.pair_activation) atomicAdd((unsigned long long *)&a.pair_activation[id], 1ull);
    if (lane == 0) {
        a.pair_err[0] = (any_bad ? 1 : 0) | (any_unloaded ? 2 : 0);
        if (a.pair_tile_items_host) *a.pair_tile_items_host = 0;
    }
}

// The first wave of a pair-direct stage-2 workgroup adds the token's weighted expert outputs in k
// order (the arithmetic of combine_kernel) and stores the token's channels of this workgroup.
template <typename T, int NCH>
__device__ __forceinline__ void pair_combine(const FfnArgs &a, const float (*prod)[NCH], const int32_t *valid, int64_t t,
                                             int ch0, int lane)
{
    if (lane >= NCH) return;
    float acc = 0.f;
    for (int k = 0; k < a.pair_K; ++k)
        if (valid[k]) acc = acc + prod[k][lane];
    T o = (T)acc;
    // the shared expert's row (wave pair_K) joins after the sum's rounding
    if (a.pair_shared && valid[a.pair_K]) o = (T)((float)o + prod[a.pair_K][lane]);
    ((T *)a.pair_y)[t * a.N + ch0 + lane] = o;
}

// PD = 0: items from the work list.  PD = 1: pair-direct stage 1 (blockIdx.y is the pair).  PD = 2:
// pair-direct stage 2 (blockIdx.y is the token, wave k of the workgroup takes its k-th pair and walks
// the whole contraction, SK = 1; the weighted sum over k replaces the store of the rows).
template <typename T, int WM, int NMAT, int NG, int D, int SK, int RS, int PD = 0>
__global__ __launch_bounds__(PD == 2 ? 64 * (kPairDirectMaxK + 1) : SK == 1 ? 256 : 64 * kSlices) void ffn_stream_kernel(FfnArgs a)
{
    static_assert(PD == 0 || RS == 1, "pair-direct items hold one row");
    static_assert(PD != 1 || (NMAT == 2 && SK == kSlices), "pair-direct stage 1 is a sliced launch");
    static_assert(PD != 2 || (NMAT == 1 && SK == 1), "pair-direct stage 2: one wave per pair");
    constexpr bool W8 = WM != kW16;    // one-byte weights: 64 contraction elements per chunk
    static_assert(SK == 1 || SK == kSlices, "one wave per launch shape or one wave per slice");
    static_assert(RS == 1 || SK == kSlices, "wide items only in the sliced form");
    using V8 = typename Act<T>::V8;
    constexpr int KE = W8 ? 64 : 32;   // contraction elements per chunk
    constexpr int XV = W8 ? 2 : 1;     // 16-byte activation loads per chunk per lane
    constexpr int NW = NMAT * NG;      // weight chunks per k step per wave

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int e, seg0, n;
    [[maybe_unused]] bool live = true;      // PD = 2: this wave's pair has an expert to run
    if constexpr (PD == 0) {
        if ((int)blockIdx.y >= a.lists.count[kListStream]) return;
        const WorkItem item = a.lists.items[kListStream][blockIdx.y];
        e = item.expert; seg0 = item.row0; n = item.nrows;
    } else {
        if (PD == 1 && blockIdx.x == 0 && blockIdx.y == 0 && wave == 0) pair_bookkeeping(a, lane);
        // items past the pairs (stage 1) and wave pair_K (stage 2) are the tokens' rows of the shared expert
        const bool shared_row = PD == 1 ? (int)blockIdx.y >= a.pair_P : wave == a.pair_K;
        seg0 = PD == 1 ? (int)blockIdx.y : shared_row ? a.pair_P + (int)blockIdx.y : (int)blockIdx.y * a.pair_K + wave;
        n = 1;
        e = shared_row ? a.n_experts : a.pair_ids[seg0];
        live = shared_row || (uint32_t)e < (uint32_t)a.n_experts;
        if (!live) e = 0;
    }
    const int NT = a.N >> 4;
    const int nt0 = SK == 1 && PD != 2 ? (blockIdx.x * (blockDim.x >> 6) + wave) * NG : blockIdx.x * NG;
    if (nt0 >= NT) return;             // SK = 8, PD = 2: the same for every wave of the workgroup
    const ExpertSlab slab = a.slabs[e];
    const uint8_t *wmat = NMAT == 2 ? slab.upgate : slab.down;
    [[maybe_unused]] __shared__ float pd_prod[PD == 2 ? kPairDirectMaxK + 1 : 1][PD == 2 ? NG * 16 : 1];
    [[maybe_unused]] __shared__ int32_t pd_valid[PD == 2 ? kPairDirectMaxK + 1 : 1];
    if constexpr (PD == 2) {
        live = live && wmat != nullptr;
        if (!live) {
            // nothing to add for this pair; the workgroup's sum still needs this wave at its barrier
            if (lane == 0) pd_valid[wave] = 0;
            __syncthreads();
            if (wave == 0) pair_combine<T, NG * 16>(a, pd_prod, pd_valid, blockIdx.y, nt0 * 16, lane);
            return;
        }
    } else {
        if (!live || wmat == nullptr) return;   // expert not loaded: the call has been flagged
    }
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
            if constexpr (WM == kWI8) {
                const int ch = (nt0 + gi) * 16 + j;
                sv = NMAT == 2 ? (m == 0 ? slab.s_up[ch] : slab.s_gate[ch]) : slab.s_down[ch];
            }
            ws[gi * NMAT + m] = sv;
            wc[gi * NMAT + m] = -128.f * sv;
        }

    // Block scales: the wave's 16 channels lie in one 128-row block, so the scale of a chunk is
    // one number per 128 contraction elements: the wave keeps its rows of the scale matrices in
    // LDS (lane b holds block b) and reads one back per chunk.
    __shared__ float srow[block_scaled(WM) ? (PD == 2 ? kPairDirectMaxK + 1 : SK == 1 ? 4 : kSlices) : 1][block_scaled(WM) ? NW : 1]
                         [block_scaled(WM) ? kMaxScaleBlocks : 1];
    if constexpr (block_scaled(WM)) {
        const int KB = (a.Kdim + 127) >> 7;
#pragma unroll
        for (int gi = 0; gi < NG; ++gi)
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const float *smat = NMAT == 2 ? (m == 0 ? slab.s_up : slab.s_gate) : slab.s_down;
                if (lane < KB) srow[wave][gi * NMAT + m][lane] = smat[(int64_t)(((nt0 + gi) * 16) >> 7) * KB + lane];
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }

    const int nfr = RS == 1 ? 1 : (n + 15) >> 4;   // 16-row fragments that hold rows
    const T *xp[RS];
#pragma unroll
    for (int rs = 0; rs < RS; ++rs) {
        const int jr = min(rs * 16 + j, n - 1);   // lanes past the segment re-read its last row
        const int64_t row = PD == 1 ? (int64_t)(seg0 >= a.pair_P ? seg0 - a.pair_P : seg0 / a.pair_K)
                            : a.rows ? (int64_t)a.rows[seg0 + jr] : (int64_t)(seg0 + jr);
        xp[rs] = (const T *)a.x + row * a.x_stride + g * (KE / 4);
    }

    f32x4 acc[RS][NMAT][NG], tot[RS][NMAT][NG];
#pragma unroll
    for (int rs = 0; rs < RS; ++rs)
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                acc[rs][m][gi] = (f32x4){0.f, 0.f, 0.f, 0.f};
                tot[rs][m][gi] = (f32x4){0.f, 0.f, 0.f, 0.f};
            }
    // this wave's chunks and, for SK = 1, the end of the slice it is in
    const int kbeg = SK == 1 ? 0 : KT * wave / kSlices, kend = SK == 1 ? KT : KT * (wave + 1) / kSlices;
    int sl = 0, kb = KT / kSlices;
    if constexpr (SK == 1) {
        while (kb == 0) { ++sl; kb = KT * (sl + 1) / kSlices; }   // empty leading slices (KT < 8)
    }

    uint4 wq[D][NW];
    uint4 xq[D][RS][XV];
    auto fetch = [&](int d, int kt) {
#pragma unroll
        for (int gi = 0; gi < NG; ++gi)
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
            {
                // items of up to 16 rows: an expert's weights are read by one item (routed pairs) or a
                // few; wide items come several to an expert and find them in the caches
                const uint8_t *src = wp[gi] + (int64_t)(kt * NMAT + m) * kChunkBytes;
                wq[d][gi * NMAT + m] = RS == 1 ? ldg16_once(src) : ldg16(src);
            }
#pragma unroll
        for (int rs = 0; rs < RS; ++rs)
            if (RS == 1 || rs < nfr) {
#pragma unroll
                for (int v = 0; v < XV; ++v) xq[d][rs][v] = ldg16(xp[rs] + (int64_t)kt * KE + v * 8);
            }
    };
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (SK == 1 || kbeg + d < kend) fetch(d, kbeg + d);

    for (int kt0 = kbeg; kt0 < kend; kt0 += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int kt = kt0 + d;
            if (SK != 1 && kt >= kend) break;      // SK = 1: KT is a multiple of D
            // consume slot d
#pragma unroll
            for (int gi = 0; gi < NG; ++gi)
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    const uint4 q = wq[d][gi * NMAT + m];
                    if constexpr (W8) {
                        V8 w0, w1;
                        if constexpr (WM == kWI8) {
                            const float sv = ws[gi * NMAT + m], cv = wc[gi * NMAT + m];
                            w0 = dequant_u8x8<T>(q.x, q.y, sv, cv);
                            w1 = dequant_u8x8<T>(q.z, q.w, sv, cv);
                        } else if constexpr (WM == kWF8Block) {
                            const float sv = srow[wave][gi * NMAT + m][kt >> 1];
                            w0 = dequant_f8x8<T>(q.x, q.y, sv);
                            w1 = dequant_f8x8<T>(q.z, q.w, sv);
                        } else {
                            const float sv = srow[wave][gi * NMAT + m][kt >> 1], cv = -128.f * sv;
                            w0 = dequant_u8x8<T>(q.x, q.y, sv, cv);
                            w1 = dequant_u8x8<T>(q.z, q.w, sv, cv);
                        }
#pragma unroll
                        for (int rs = 0; rs < RS; ++rs)
                            if (RS == 1 || rs < nfr) {
                                acc[rs][m][gi] = Act<T>::mfma(w0, __builtin_bit_cast(V8, xq[d][rs][0]), acc[rs][m][gi]);
                                acc[rs][m][gi] = Act<T>::mfma(w1, __builtin_bit_cast(V8, xq[d][rs][1]), acc[rs][m][gi]);
                            }
                    } else {
                        const V8 w0 = __builtin_bit_cast(V8, q);
#pragma unroll
                        for (int rs = 0; rs < RS; ++rs)
                            if (RS == 1 || rs < nfr)
                                acc[rs][m][gi] = Act<T>::mfma(w0, __builtin_bit_cast(V8, xq[d][rs][0]), acc[rs][m][gi]);
                    }
                }
            if constexpr (SK == 1) {
                if (kt + 1 == kb) {                // a slice ends: its sum joins the total
#pragma unroll
                    for (int m = 0; m < NMAT; ++m)
#pragma unroll
                        for (int gi = 0; gi < NG; ++gi) {
                            tot[0][m][gi] += acc[0][m][gi];
                            acc[0][m][gi] = (f32x4){0.f, 0.f, 0.f, 0.f};
                        }
                    do { ++sl; kb = KT * (sl + 1) / kSlices; } while (kb == kt + 1 && sl < kSlices - 1);
                }
            }
            // refill slot d with chunk kt + D
            if (kt + D < kend) fetch(d, kt + D);
        }
    }

    if constexpr (SK != 1) {
        // slice sums meet in LDS; the first wave adds them in slice order
        __shared__ f32x4 red[kSlices][RS * NMAT * NG][64];
#pragma unroll
        for (int rs = 0; rs < RS; ++rs)
            if (RS == 1 || rs < nfr) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int gi = 0; gi < NG; ++gi) red[wave][(rs * NMAT + m) * NG + gi][lane] = acc[rs][m][gi];
            }
        __syncthreads();
        if (wave != 0) return;
        for (int w = 0; w < kSlices; ++w)
#pragma unroll
            for (int rs = 0; rs < RS; ++rs)
                if (RS == 1 || rs < nfr) {
#pragma unroll
                    for (int m = 0; m < NMAT; ++m)
#pragma unroll
                        for (int gi = 0; gi < NG; ++gi) tot[rs][m][gi] += red[w][(rs * NMAT + m) * NG + gi][lane];
                }
    }

    if constexpr (PD == 2) {
        // lanes (g, 0) hold the pair's row: its rounded outputs times the gate weight, as the
        // combine kernel forms them, meet in LDS
        const bool shared_row = wave == a.pair_K;
        const int wi = shared_row ? 0 : seg0;
        const float wv = a.pair_w_f32 ? ((const float *)a.pair_w)[wi] : (float)((const T *)a.pair_w)[wi];
        if (j == 0) {
#pragma unroll
            for (int gi = 0; gi < NG; ++gi)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float pr = (float)(T)tot[0][0][gi][r];
                    if (!shared_row) {
                        pr = wv * pr;
                        if (!a.pair_w_f32) pr = (float)(T)pr;
                    }
                    pd_prod[wave][gi * 16 + 4 * g + r] = pr;
                }
        }
        if (lane == 0) pd_valid[wave] = 1;
        __syncthreads();
        if (wave == 0) pair_combine<T, NG * 16>(a, pd_prod, pd_valid, blockIdx.y, nt0 * 16, lane);
        return;
    }
    // epilogue: lane (g, j) holds channels nt*16 + 4g + r (r = 0..3) of row rs*16 + j
#pragma unroll
    for (int rs = 0; rs < RS; ++rs) {
        if (rs * 16 + j >= n) continue;
        T *orow = (T *)a.out + (int64_t)(seg0 + rs * 16 + j) * a.out_stride;
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            const int ch = (nt0 + gi) * 16 + 4 * g;
            typedef T T4 __attribute__((ext_vector_type(4)));
            T4 o;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if constexpr (NMAT == 2) {
                    o[r] = swiglu_rounded<T>(tot[rs][0][gi][r], tot[rs][1][gi][r]);
                } else {
                    o[r] = (T)tot[rs][0][gi][r];
                }
            }
            *(uint2 *)(orow + ch) = __builtin_bit_cast(uint2, o);
        }
    }
}

// Channel tiles per wave and prefetch depth in k steps, per stage: stage 1 one tile eight steps
// deep, stage 2 two tiles four deep (the fastest of the shapes measured on MI355X at the
// DeepSeek-V3 shape).
constexpr int kStage1Tiles = 1, kStage1Depth = 8, kStage2Tiles = 2, kStage2Depth = 4;

template <typename T, int WM, int NMAT, int NG, int D>
static hipError_t launch_d(const FfnArgs &a, int32_t nseg, hipStream_t s)
{
    constexpr int KE = WM != kW16 ? 64 : 32;
    const int KT = a.Kdim / KE;
    const int NT = a.N / 16;
    if constexpr (D > 1) {
        if (KT % D != 0) return launch_d<T, WM, NMAT, NG, D / 2>(a, nseg, s);
    }
    // waves per workgroup: a workgroup's slot is free again when its slowest wave ends; stage 2's
    // short contraction (waves that live for a few dozen steps) does better with two than with
    // four (DeepSeek-V3 decode layer on MI355X: 569 -> 556 us), stage 1 the other way round
    constexpr int WPB = NMAT == 2 ? 4 : 2;
    dim3 grid((NT + WPB * NG - 1) / (WPB * NG), nseg);
    hipLaunchKernelGGL((ffn_stream_kernel<T, WM, NMAT, NG, D, 1, 1>), grid, dim3(64 * WPB), 0, s, a);
    return hipGetLastError();
}

// The sliced form (eight waves of a workgroup take one slice of the contraction each) against the
// one-wave form (one wave walks the whole contraction, four or two waves of a workgroup take
// neighbouring channel groups of one item and share its rows in the CU's cache).  Same bits
// either way.  Measured on MI355X, enqueue-only layer calls, stage kernel times:
//  * 16-bit weights: sliced is as fast or faster at every size tried (DeepSeek-V3 shape, 64 experts,
//    4 / 64 tokens: stage 1 242 -> 222 / 555 -> 546 us, stage 2 118 -> 115 / 287 -> 279 us; Qwen3 shape,
//    uniform routing, 4 / 64 / 256 tokens: stage 1 38 -> 35 / 127 -> 123 / 101 -> 97 us).
//  * one-byte weights hold twice the contraction per chunk, and the prefetch slots of the depth that
//    serves the one-wave form leave room for one sliced workgroup per CU only (164 registers): two
//    slots deep three fit, and stage 1 of the DeepSeek-V3 int8 layer goes from 47.3 to 39.4 us at
//    1 token, 242 -> 230 at 8, 681 -> 669 at 32, 1075 -> 1061 at 128.  From 8 rows per expert on the
//    one-wave form is ahead again (256 tokens: 1157 against 1172 us): every (item, channel group)
//    reads the item's rows from L2, and neighbouring channel groups in one workgroup share them.
//    Stage 2 (two channel tiles per wave, two slots deep) gains up to 4 tokens (27.4 -> 23.4 us at
//    1, 43.7 -> 42.0 at 2) and loses from 8 on (136 -> 141 us at 8, 224 -> 241 at 16, behind a sliced
//    stage 1).
constexpr int64_t kSliceStage2Below = 8192;   // (item, channel group) pairs, one-byte weights
// Below this many (item, channel group) pairs the one-wave form leaves most of the chip's memory
// system idle whatever the rows per item (a lone expert, a tiny layer).
constexpr int64_t kSplitBelow = 1536;

// few_rows: the launch's items hold about four rows or fewer on average.
template <typename T, int WM, int NMAT>
static hipError_t launch_g(const FfnArgs &a, int32_t nseg, bool wide, bool few_rows, hipStream_t s)
{
    constexpr bool W8 = WM != kW16;
    constexpr int NG = NMAT == 2 ? kStage1Tiles : kStage2Tiles;
    constexpr int D = NMAT == 2 ? kStage1Depth : kStage2Depth;
    const int NT = a.N / 16;
    if (wide) {
        // four activation fragments per prefetch slot: shallower, the eight slices make up for it
        constexpr int DW = W8 ? 2 : 4;
        // Channel tiles per workgroup: every workgroup reads its item's rows in full, so more
        // tiles per workgroup mean fewer readers of the rows; a short list wants the workgroups
        // instead.  Measured on MI355X, one DeepSeek-V3 expert: two instead of one (stage 1)
        // pays from three items on, four instead of two (stage 2) from two items on (256 rows:
        // 88 against 121 us for both stages, 64 rows: 68 us either way).
        constexpr int NG_FEW = NMAT == 2 ? 1 : 2, NG_MANY = 2 * NG_FEW;
        const bool many = nseg >= (NMAT == 2 ? 3 : 2);
        if (many && NT % NG_MANY == 0)
            hipLaunchKernelGGL((ffn_stream_kernel<T, WM, NMAT, NG_MANY, DW, kSlices, 4>), dim3(NT / NG_MANY, nseg),
                               dim3(64 * kSlices), 0, s, a);
        else if (NT % NG_FEW == 0)
            hipLaunchKernelGGL((ffn_stream_kernel<T, WM, NMAT, NG_FEW, DW, kSlices, 4>), dim3(NT / NG_FEW, nseg),
                               dim3(64 * kSlices), 0, s, a);
        else
            hipLaunchKernelGGL((ffn_stream_kernel<T, WM, NMAT, 1, DW, kSlices, 4>), dim3(NT, nseg),
                               dim3(64 * kSlices), 0, s, a);
        return hipGetLastError();
    }
    if (NT % NG == 0) {
        // prefetch slots of the sliced form: a slice is an eighth of the contraction
        constexpr int DS = W8 ? 2 : D;
        const int64_t groups = (int64_t)nseg * (NT / NG);
        const bool sliced = !W8 ? true : NMAT == 2 ? few_rows || groups < kSplitBelow : groups < kSliceStage2Below;
        if (sliced) {
            hipLaunchKernelGGL((ffn_stream_kernel<T, WM, NMAT, NG, DS, kSlices, 1>), dim3(NT / NG, nseg),
                               dim3(64 * kSlices), 0, s, a);
            return hipGetLastError();
        }
        return launch_d<T, WM, NMAT, NG, D>(a, nseg, s);
    }
    if (NT % 2 == 0) return launch_d<T, WM, NMAT, 2, D>(a, nseg, s);
    return launch_d<T, WM, NMAT, 1, D>(a, nseg, s);
}

template <typename T>
static hipError_t launch_w(const FfnArgs &a, int stage, int wmode, int32_t n_segments, bool wide, bool few_rows,
                           hipStream_t s)
{
    switch (wmode) {
    case kWI8:
        return stage == 1 ? launch_g<T, kWI8, 2>(a, n_segments, wide, few_rows, s) : launch_g<T, kWI8, 1>(a, n_segments, wide, few_rows, s);
    case kWF8Block:
        return stage == 1 ? launch_g<T, kWF8Block, 2>(a, n_segments, wide, few_rows, s)
                          : launch_g<T, kWF8Block, 1>(a, n_segments, wide, few_rows, s);
    case kWI8Block:
        return stage == 1 ? launch_g<T, kWI8Block, 2>(a, n_segments, wide, few_rows, s)
                          : launch_g<T, kWI8Block, 1>(a, n_segments, wide, few_rows, s);
    default:
        return stage == 1 ? launch_g<T, kW16, 2>(a, n_segments, wide, few_rows, s) : launch_g<T, kW16, 1>(a, n_segments, wide, few_rows, s);
    }
}

template <typename T, int WM>
static hipError_t launch_pairs_w(const FfnArgs &a, int stage, hipStream_t s)
{
    constexpr bool W8 = WM != kW16;
    const int NT = a.N / 16;
    const int KT = a.Kdim / (W8 ? 64 : 32);
    if (stage == 1) {
        // the sliced form of the ordinary launch, one item per pair
        constexpr int DS = W8 ? 2 : kStage1Depth;
        const int T1 = a.pair_P / a.pair_K;
        hipLaunchKernelGGL((ffn_stream_kernel<T, WM, 2, 1, DS, kSlices, 1, 1>), dim3(NT, a.pair_P + (a.pair_shared ? T1 : 0)),
                           dim3(64 * kSlices), 0, s, a);
        return hipGetLastError();
    }
    const dim3 block(64 * (a.pair_K + (a.pair_shared ? 1 : 0)));
    const int T_ = a.pair_P / a.pair_K;
    constexpr int NG = kStage2Tiles, D = kStage2Depth;
    if (NT % NG == 0 && KT % D == 0)
        hipLaunchKernelGGL((ffn_stream_kernel<T, WM, 1, NG, D, 1, 1, 2>), dim3(NT / NG, T_), block, 0, s, a);
    else if (NT % NG == 0 && KT % 2 == 0)      // (the one-wave loop takes contractions of whole prefetch rounds)
        hipLaunchKernelGGL((ffn_stream_kernel<T, WM, 1, NG, 2, 1, 1, 2>), dim3(NT / NG, T_), block, 0, s, a);
    else
        hipLaunchKernelGGL((ffn_stream_kernel<T, WM, 1, 1, 1, 1, 1, 2>), dim3(NT, T_), block, 0, s, a);
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_pairs_t(const FfnArgs &a, int stage, int wmode, hipStream_t s)
{
    switch (wmode) {
    case kWI8: return launch_pairs_w<T, kWI8>(a, stage, s);
    case kWF8Block: return launch_pairs_w<T, kWF8Block>(a, stage, s);
    case kWI8Block: return launch_pairs_w<T, kWI8Block>(a, stage, s);
    default: return launch_pairs_w<T, kW16>(a, stage, s);
    }
}

hipError_t launch_ffn_pairs(const FfnArgs &a, int stage, int act, int wmode, hipStream_t s)
{
    if (a.pair_P <= 0) return hipSuccess;
    if (a.pair_P > kPairDirectMax || a.pair_K <= 0 || a.pair_K > kPairDirectMaxK || a.pair_P % a.pair_K != 0)
        return hipErrorInvalidValue;
    return act == 0 ? launch_pairs_t<__bf16>(a, stage, wmode, s) : launch_pairs_t<_Float16>(a, stage, wmode, s);
}

hipError_t launch_ffn_stream(const FfnArgs &a, int stage, int act, int wmode, int64_t max_items, bool wide,
                             bool few_rows, hipStream_t s)
{
    const int32_t n_segments = (int32_t)max_items;
    if (n_segments <= 0) return hipSuccess;
    return act == 0 ? launch_w<__bf16>(a, stage, wmode, n_segments, wide, few_rows, s)
                    : launch_w<_Float16>(a, stage, wmode, n_segments, wide, few_rows, s);
}

}  // namespace ek
