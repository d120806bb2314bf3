// Ragged grouped SwiGLU FFN, MFMA tile kernel (work items of 17..128 rows).
//
// Same arithmetic as the weight-streaming kernel (TorchFFN's closure,
// ek-computation/src/ffn/expert_torch.rs:81-84, with its storage roundings),
// for segments long enough that the contraction, not weight traffic, is the
// cost.  One workgroup of four wavefronts owns one work item (BM = 16*MR rows
// of one expert) x BN output channels:
//   - the four waves split the channels; each wave keeps every row of the
//     tile, so a weight element is fetched and dequantised once per workgroup,
//     straight from the chunked HBM layout into MFMA "A" operands (no LDS);
//   - the activation rows (gathered through row_token for stage 1) are staged
//     global -> registers -> LDS in 64-wide k steps, double buffered, one
//     barrier per step, and read back as MFMA "B" operands by all four waves;
//     rows are padded to 72 elements so the 16-byte fragment reads of 16 lanes
//     fall in 16 distinct bank groups;
//   - fp32 accumulators: MR x NR x NMAT tiles of 16x16 per wave.
// Workgroups are numbered so that each XCD walks a contiguous range of
// (item, channel block) pairs: neighbours share the activation tile and, for
// the tiles of one expert, the weights, in that XCD's L2.
#include "ek_internal.h"
#include "ek_mfma.h"

namespace ek {

template <typename T, bool W8, int NMAT, int MR>
__device__ __forceinline__ void tile_body(const FfnArgs &a, const WorkItem item, const int nb, T *smem)
{
    using V8 = typename Act<T>::V8;
    constexpr int NR = NMAT == 2 ? 2 : 4;      // channel tiles per wave and matrix
    constexpr int BM = MR * 16;
    constexpr int BK = 64;                      // contraction elements per step
    constexpr int LDK = BK + 8;                 // padded LDS row
    constexpr int KE = W8 ? 64 : 32;            // contraction elements per weight chunk
    constexpr int CPS = BK / KE;                // weight chunks per step, channel tile and matrix
    constexpr int XP = BM * 8 / 256;            // 16-byte pieces of the x tile per thread and step
    constexpr int NWC = NR * NMAT * CPS;        // weight chunks per step per wave
    typedef T XTile[BM][LDK];
    XTile *sX = reinterpret_cast<XTile *>(smem);   // [2][BM][LDK]

    const int e = item.expert, row0 = item.row0, nrows = item.nrows;
    const ExpertSlab slab = a.slabs[e];
    const uint8_t *wmat = NMAT == 2 ? slab.upgate : slab.down;
    if (wmat == nullptr) return;                // expert not loaded: pack has flagged the call

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int NT = a.N >> 4;
    const int KT = a.Kdim / KE;                 // chunks along k
    const int nsteps = a.Kdim / BK;

    // ---- x tile: global -> LDS assignment -------------------------------------
    const T *xsrc[XP];
    int xdst[XP];
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const int p = tid + i * 256;
        const int r = p >> 3, c = p & 7;
        const int rr = min(r, nrows - 1);       // rows past the item re-read its last row
        const int64_t row = a.rows ? (int64_t)a.rows[row0 + rr] : (int64_t)(row0 + rr);
        xsrc[i] = (const T *)a.x + row * a.x_stride + c * 8;
        xdst[i] = r * LDK + c * 8;
    }

    // ---- weights: this wave's channel tiles -------------------------------------
    const uint8_t *wp[NR];
    float ws[NR][NMAT], wc[NR][NMAT];
    int ct[NR];
#pragma unroll
    for (int nr = 0; nr < NR; ++nr) {
        ct[nr] = (nb * 4 + wave) * NR + nr;
        const int ctc = min(ct[nr], NT - 1);    // channel tiles past N recompute the last one
        wp[nr] = wmat + (int64_t)ctc * KT * (NMAT * kChunkBytes) + lane * 16;
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            float sv = 1.f;
            if constexpr (W8) {
                const int ch = ctc * 16 + j;
                sv = NMAT == 2 ? (m == 0 ? slab.s_up[ch] : slab.s_gate[ch]) : slab.s_down[ch];
            }
            ws[nr][m] = sv;
            wc[nr][m] = -128.f * sv;
        }
    }

    f32x4 acc[MR][NR][NMAT];
#pragma unroll
    for (int mr = 0; mr < MR; ++mr)
#pragma unroll
        for (int nr = 0; nr < NR; ++nr)
#pragma unroll
            for (int m = 0; m < NMAT; ++m) acc[mr][nr][m] = (f32x4){0.f, 0.f, 0.f, 0.f};

    uint4 wcur[NWC], wnext[NWC], xreg[XP];

#define EK_LOAD_W(dst, step)                                                                   \
    _Pragma("unroll") for (int nr = 0; nr < NR; ++nr)                                          \
    _Pragma("unroll") for (int c = 0; c < CPS; ++c)                                            \
    _Pragma("unroll") for (int m = 0; m < NMAT; ++m)                                           \
        dst[(nr * CPS + c) * NMAT + m] =                                                       \
            ldg16(wp[nr] + (int64_t)(((step) * CPS + c) * NMAT + m) * kChunkBytes)
#define EK_LOAD_X(step)                                                                        \
    _Pragma("unroll") for (int i = 0; i < XP; ++i) xreg[i] = ldg16(xsrc[i] + (step) * BK)
#define EK_STORE_X(buf)                                                                        \
    _Pragma("unroll") for (int i = 0; i < XP; ++i) *(uint4 *)(&sX[buf][0][0] + xdst[i]) = xreg[i]

    EK_LOAD_X(0);
    EK_LOAD_W(wcur, 0);
    EK_STORE_X(0);
    __syncthreads();

    for (int step = 0; step < nsteps; ++step) {
        const int buf = step & 1;
        const bool more = step + 1 < nsteps;
        if (more) {
            EK_LOAD_X(step + 1);
            EK_LOAD_W(wnext, step + 1);
        }
        // two MFMA k-groups of 32 per step
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            V8 af[NR][NMAT];
#pragma unroll
            for (int nr = 0; nr < NR; ++nr)
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    if constexpr (W8) {
                        const uint4 q = wcur[nr * NMAT + m];
                        af[nr][m] = h == 0 ? dequant_u8x8<T>(q.x, q.y, ws[nr][m], wc[nr][m])
                                           : dequant_u8x8<T>(q.z, q.w, ws[nr][m], wc[nr][m]);
                    } else {
                        af[nr][m] = __builtin_bit_cast(V8, wcur[(nr * CPS + h) * NMAT + m]);
                    }
                }
            // lane (j, g) supplies k = g*16 + h*8 .. +8 (int8 chunk order) or h*32 + g*8 .. +8
            const int koff = W8 ? g * 16 + h * 8 : h * 32 + g * 8;
#pragma unroll
            for (int mr = 0; mr < MR; ++mr) {
                const V8 bf = *(const V8 *)&sX[buf][mr * 16 + j][koff];
#pragma unroll
                for (int nr = 0; nr < NR; ++nr)
#pragma unroll
                    for (int m = 0; m < NMAT; ++m)
                        acc[mr][nr][m] = Act<T>::mfma(af[nr][m], bf, acc[mr][nr][m]);
            }
        }
        if (more) {
            EK_STORE_X(buf ^ 1);
#pragma unroll
            for (int i = 0; i < NWC; ++i) wcur[i] = wnext[i];
        }
        __syncthreads();
    }

    // ---- epilogue: lane (g, j) holds channels ct*16 + 4g + r of row mr*16 + j ----
    typedef T T4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int mr = 0; mr < MR; ++mr) {
        const int r_in = mr * 16 + j;
        if (r_in >= nrows) continue;
        T *orow = (T *)a.out + (int64_t)(row0 + r_in) * a.out_stride;
#pragma unroll
        for (int nr = 0; nr < NR; ++nr) {
            if (ct[nr] >= NT) continue;
            T4 o;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if constexpr (NMAT == 2) o[r] = swiglu_rounded<T>(acc[mr][nr][0][r], acc[mr][nr][1][r]);
                else o[r] = (T)acc[mr][nr][0][r];
            }
            *(uint2 *)(orow + ct[nr] * 16 + 4 * g) = __builtin_bit_cast(uint2, o);
        }
    }
}

#undef EK_LOAD_W
#undef EK_LOAD_X
#undef EK_STORE_X

// One launch covers the three tile lists.  Workgroup b runs on XCD b % 8
// (round-robin dispatch), so each XCD is given a contiguous eighth of every
// list: first its 128-row items, then its 64-row, then its 32-row ones, each
// times nb_count channel blocks.  Neighbouring workgroups of an XCD then share
// the activation tile (same item) and mostly the expert's weights in its L2,
// and every XCD gets the same mix of long and short items.
template <typename T, bool W8, int NMAT>
__global__ __launch_bounds__(256, 2) void ffn_tile_kernel(FfnArgs a, int nb_count)
{
    __shared__ __attribute__((aligned(16))) T smem[2 * 128 * (64 + 8)];
    const int x = blockIdx.x & 7;
    int i = blockIdx.x >> 3;
    const int n128 = a.lists.count[kListT128], n64 = a.lists.count[kListT64], n32 = a.lists.count[kListT32];
    const int lo128 = x * n128 / 8, s128 = (x + 1) * n128 / 8 - lo128;
    const int lo64 = x * n64 / 8, s64 = (x + 1) * n64 / 8 - lo64;
    const int lo32 = x * n32 / 8, s32 = (x + 1) * n32 / 8 - lo32;
    if (i < s128 * nb_count) {
        tile_body<T, W8, NMAT, 8>(a, a.lists.items[kListT128][lo128 + i / nb_count], i % nb_count, smem);
        return;
    }
    i -= s128 * nb_count;
    if (i < s64 * nb_count) {
        tile_body<T, W8, NMAT, 4>(a, a.lists.items[kListT64][lo64 + i / nb_count], i % nb_count, smem);
        return;
    }
    i -= s64 * nb_count;
    if (i < s32 * nb_count)
        tile_body<T, W8, NMAT, 2>(a, a.lists.items[kListT32][lo32 + i / nb_count], i % nb_count, smem);
}

template <typename T, bool W8, int NMAT>
static hipError_t launch_t(const FfnArgs &a, const int64_t max_items[kNumLists], hipStream_t s)
{
    constexpr int NR = NMAT == 2 ? 2 : 4;
    const int NT = a.N / 16;
    const int nb_count = (NT + 4 * NR - 1) / (4 * NR);
    const int64_t per_xcd = (max_items[kListT128] + 7) / 8 + (max_items[kListT64] + 7) / 8 +
                            (max_items[kListT32] + 7) / 8;
    const int64_t blocks = per_xcd * nb_count * 8;
    if (blocks <= 0) return hipSuccess;
    hipLaunchKernelGGL((ffn_tile_kernel<T, W8, NMAT>), dim3((unsigned)blocks), dim3(256), 0, s, a, nb_count);
    return hipGetLastError();
}

hipError_t launch_ffn_tile(const FfnArgs &a, int stage, int act, bool w8,
                           const int64_t max_items[kNumLists], hipStream_t s)
{
    if (act == 0) {
        if (w8) return stage == 1 ? launch_t<__bf16, true, 2>(a, max_items, s)
                                  : launch_t<__bf16, true, 1>(a, max_items, s);
        return stage == 1 ? launch_t<__bf16, false, 2>(a, max_items, s)
                          : launch_t<__bf16, false, 1>(a, max_items, s);
    }
    if (w8) return stage == 1 ? launch_t<_Float16, true, 2>(a, max_items, s)
                              : launch_t<_Float16, true, 1>(a, max_items, s);
    return stage == 1 ? launch_t<_Float16, false, 2>(a, max_items, s)
                      : launch_t<_Float16, false, 1>(a, max_items, s);
}

}  // namespace ek
