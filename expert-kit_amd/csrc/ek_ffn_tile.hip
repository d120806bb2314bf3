// Ragged grouped SwiGLU FFN, MFMA tile kernel (work items of 17..128 rows).
//
// Same arithmetic as the weight-streaming kernel (TorchFFN's closure,
// ek-computation/src/ffn/expert_torch.rs:81-84, with its storage roundings),
// for segments long enough that the contraction, not weight traffic, is the
// cost.  One workgroup of eight wavefronts (two per SIMD, one workgroup per CU)
// owns one work item (BM = 16*MR rows of one expert) x BN output channels:
//   - the eight waves split the channels; each wave keeps every row of the
//     tile, so a weight element is fetched and dequantised once per workgroup;
//   - everything is brought in by LDS-DMA (global_load_lds_dwordx4: global ->
//     LDS without passing through registers) in steps of 64 contraction
//     elements, three stages deep with one-byte weights (while step s is being
//     multiplied, the loads of steps s+1 and s+2 are in flight) and two stages
//     deep with 16-bit weights, whose stage is 80 KiB (measured on MI355X
//     against 32-element steps three deep: a lone bf16 DeepSeek-V3 expert
//     runs 6 to 13 % faster, fewer barriers and waits per MFMA).  The
//     weight chunks of a wave land in a wave-private region in exactly the
//     chunked HBM layout (lane l's 16 bytes at l*16), the activation rows
//     (gathered through row_token for stage 1) in an XOR-swizzled tile whose
//     16-byte fragment reads are bank-conflict free;
//   - completion is tracked by hand: the DMA is issued from inline asm, so the
//     only vector-memory operations of a wave in the main loop are its own
//     DMAs, in program order, and `s_waitcnt vmcnt(n)` with n = the DMAs of
//     the younger stage is exact; one s_barrier per step publishes the
//     activation tile and retires the stage that is overwritten next;
//   - MFMA 32x32x16 (weights as the A operand: 32 channels x 16 k; activation
//     rows as B: 16 k x 32 rows): one wavefront alone keeps the matrix pipe
//     full with it (one issue per 32 cycles), which 16x16x32 does not; fp32
//     accumulators: (MR/2) x 2 tiles of 32x32 per wave;
// Each XCD walks a contiguous eighth of every work list, so neighbouring
// workgroups share the activation tile and mostly the expert's weights in
// that XCD's L2.
// The kernel exists in two forms, chosen by the host per launch: wide (two column blocks of 32
// channels per wave: the figures above) and narrow (one column block per wave, so half the
// channels per workgroup and twice the workgroups per item, three stages with 16-bit weights
// too) for launches whose tiles would leave most of the chip idle.  Every output element is the
// same sum in the same order in both.  In the wide form the 32- and 64-row items of a launch whose
// tiles fill the chip take a third path, run_mid below: weights from HBM straight into registers.
#include "ek_internal.h"
#include "ek_mfma.h"

namespace ek {

typedef __attribute__((address_space(3))) void *lds_ptr;

// One LDS-DMA of 16 bytes per lane: lane l's bytes land at lds_addr + l*16.
// lds_addr must be wave-uniform (it travels in M0).
__device__ __forceinline__ void dma16(const void *gaddr, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gaddr), "s"(lds_addr)
                 : "memory");
}
template <int N> __device__ __forceinline__ void wait_vmcnt()
{
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
// s_waitcnt vmcnt(n) for a wave-uniform run-time n: the count is an immediate, so this is a
// jump over the possible values.  n beyond 24 waits for 24 (stricter, hence safe).
__device__ __forceinline__ void wait_vmcnt_dyn(int n)
{
    switch (n) {
#define EK_CASE(k) case k: wait_vmcnt<k>(); break;
        EK_CASE(0) EK_CASE(1) EK_CASE(2) EK_CASE(3) EK_CASE(4) EK_CASE(5) EK_CASE(6) EK_CASE(7)
        EK_CASE(8) EK_CASE(9) EK_CASE(10) EK_CASE(11) EK_CASE(12) EK_CASE(13) EK_CASE(14) EK_CASE(15)
        EK_CASE(16) EK_CASE(17) EK_CASE(18) EK_CASE(19) EK_CASE(20) EK_CASE(21) EK_CASE(22) EK_CASE(23)
#undef EK_CASE
    default: wait_vmcnt<24>(); break;
    }
}
__device__ __forceinline__ void block_barrier()
{
    asm volatile("s_barrier" : : : "memory");
}
// Workgroup barrier that publishes LDS only: this wave's LDS reads and writes have completed, its
// global loads stay in flight (__syncthreads would wait for them as well).
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");
}

constexpr int kCusPerXcd = 32;   // MI355X: 8 XCDs x 32 CUs

// A step covers 64 contraction elements: one weight chunk per channel tile with one-byte
// weights, two with 16-bit ones (KC).  One-byte weights run three stages deep (two steps of
// loads in flight), 16-bit weights, whose stage is 80 KiB, two (one step in flight, of the
// same length in time: the step has as many MFMAs and no conversion work).
// WAVES wavefronts per workgroup, each with CB column blocks of 32 channels; BMMAX = rows of the
// tallest tile.
template <bool W8, int WAVES, int CB, int BMMAX> struct TileGeom {
    static constexpr int BK = 64;                    // contraction elements per step
    static constexpr int KC = W8 ? 1 : 2;            // weight chunks along k per channel tile and step
    static constexpr int PPR = BK / 8;               // 16-byte pieces per activation row and step
    static constexpr int XS = BMMAX * BK * 2;        // bytes of an activation stage
    static constexpr int WS = WAVES * 2 * CB * KC * kChunkBytes;
    static constexpr int STAGE = XS + WS;
    // 16-bit weights: two stages of 80 KiB with two column blocks per wave, three of 48 KiB with one
    static constexpr int STAGES = W8 || CB == 1 ? 3 : 2;
    // block scales: [tile parity][wave][scale row][block]; a wave has one scale row per column block,
    // two (up, gate) when its single column block holds both matrices
    static constexpr int SCALE_ROWS = CB == 1 ? 2 : CB;
    static constexpr int SCALE_BYTES = 2 * WAVES * SCALE_ROWS * 64 * 4;
};

// XOR key of a row: fragment reads of 16 consecutive rows and one piece index
// hit 16 distinct 16-byte bank groups (also 8 distinct ones per half).
template <int PPR> __device__ __forceinline__ int swizzle_key(int row)
{
    if constexpr (PPR == 8) return (row & 7) ^ ((row >> 3) & 1);
    else return ((row >> 1) & 3) ^ ((row >> 3) & 1);
}

// What one wavefront needs to know about one tile (work item x channel block).
template <typename T, int NR, int LX, int CB> struct TileCtx {
    const uint8_t *wp[NR];   // this lane's 16 bytes of the wave's weight chunks at step 0
    const T *xsrc[LX];       // this lane's 16-byte pieces of the activation tile at step 0
    float as[CB], ac[CB];    // dequantisation constants of the lane's channel, per column block
    int row0, nrows;         // the item's packed rows
    int chan0;               // first output channel of the wave's block
    int sslot;               // block-scaled weights: which of the two LDS scale areas holds this tile's rows
};

// All tiles of one class (MR*16-row items) that fall to this workgroup: tiles first,
// first + stride, ... of `ntiles`, tile = (item, channel block).  The LDS-DMA pipeline
// runs across tile boundaries: the first two steps of the next tile are issued during the
// last two steps of the current one, so only the epilogue separates two tiles.
constexpr int kTileScaleBlocks = 64;   // 128-wide scale blocks along the contraction: K <= 8192

template <typename T, int WM, int NMAT, int MR, int kTileWaves, int CB, int BMMAX>
__device__ __forceinline__ void run_tiles(const FfnArgs &a, const WorkItem *items, const int ntiles,
                                          const int nb_count, const int first, const int stride,
                                          uint8_t *lds, const uint32_t lds_base)
{
    using V8 = typename Act<T>::V8;
    constexpr bool W8 = WM != kW16;            // one-byte weights
    using G = TileGeom<W8, kTileWaves, CB, BMMAX>;
    constexpr int NWC = 2 * CB;                // channel tiles x matrices per wave
    constexpr int NR = NWC / NMAT;             // channel tiles per wave and matrix
    constexpr int KC = G::KC;
    constexpr int NWCH = NWC * KC;             // weight chunks per wave and step
    constexpr int NS = G::STAGES, AHEAD = NS - 1;   // stages; steps of loads in flight
    constexpr int BM = MR * 16;
    constexpr int BK = G::BK, PPR = G::PPR;
    constexpr int XINSTR = BM * PPR / 64;      // DMA instructions per activation stage
    constexpr int LX = (XINSTR + kTileWaves - 1) / kTileWaves;   // ... per wave
    constexpr int LOADS = NWCH + LX;           // DMAs per wave and stage
    constexpr int RB = MR / 2;                 // 32-row blocks
    constexpr int NGRP = BK / 16;              // MFMA k-groups per step
    constexpr int kRowBlockBytes = 32 * PPR * 16;
    static_assert(RB >= 1, "items have at least 32 rows");
    static_assert(BM <= BMMAX, "the activation stage holds the tile");
    static_assert(NMAT == 1 || CB % 2 == 0 || CB == 1, "up and gate blocks come in pairs, or share one block");
    // CB == 1 with two matrices: the wave's one column block is {16 up channels, 16 gate channels}
    // of the same 16 hidden channels (lanes 0-15 / 16-31 of the A operand), and a lane's accumulator
    // holds up in registers 0-7 and gate of the same channels in registers 8-15.
    constexpr bool kSplitBlock = NMAT == 2 && CB == 1;
    typedef TileCtx<T, NR, LX, CB> Ctx;

    if (first >= ntiles) return;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, l32 = lane & 31, kg = lane >> 5, hh = l32 >> 4;
    const int NT = a.N >> 4;
    const int nsteps = a.Kdim / BK;             // one-byte weights: >= 2 (hidden, inter >= 128)

    // ---- tile-independent lane constants ---------------------------------------
    // activation tile: DMA instruction q brings pieces q*64 .. q*64+63 (row-major, PPR per
    // row, piece index XOR-swizzled by the row's key)
    int xrow[LX], xcol[LX];
    uint32_t xdst[LX];
#pragma unroll
    for (int i = 0; i < LX; ++i) {
        const int q = (wave + i * kTileWaves) % XINSTR;    // surplus waves repeat an instruction
        const int sidx = q * 64 + lane;
        xrow[i] = sidx / PPR;
        xcol[i] = ((sidx % PPR) ^ swizzle_key<PPR>(xrow[i])) * 8;
        xdst[i] = q * 1024;
    }
    const uint32_t w_off = G::XS + wave * (NWCH * kChunkBytes);  // wave-private weight region
    // MFMA 32x32x16 operands.  The wave's 2*CB weight chunks (16 channels each) form CB
    // column blocks of 32 channels: {up, gate} pairs of the same 32 channels (stage 1: block cb is
    // matrix cb % 2 of channel pair cb / 2) or CB * 32 consecutive channels (stage 2).  Lane l feeds channel l%32 and k-half kg = l/32 of the
    // A operand, and row l%32 of a 32-row block of the B operand.  A 16-byte LDS read of
    // weight slot (2*tt + kg) gives the lane the A operands of two MFMAs (int8) or one
    // (16-bit, whose two chunks per channel tile lie side by side: k-group grp is read grp);
    // the matching B operand is the 16-byte piece with the same k.
    int aoff[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        const int nr = kSplitBlock ? 0 : (NMAT == 2 ? cb >> 1 : cb) * 2 + hh;
        const int m = kSplitBlock ? hh : (NMAT == 2 ? (cb & 1) : 0);
        aoff[cb] = (nr * NMAT + m) * KC * kChunkBytes + kg * 256 + j * 16;
    }
    int boff[NGRP];
#pragma unroll
    for (int grp = 0; grp < NGRP; ++grp) {
        const int c = W8 ? ((grp >> 1) * 2 + kg) * 2 + (grp & 1) : grp * 2 + kg;
        boff[grp] = (l32 * PPR + (c ^ swizzle_key<PPR>(j))) * 16;
    }

    // Fills `c` for the first tile at or after index t (stepping by stride) whose expert is
    // loaded; returns its index or -1.
    // block scales: the wave's 32-channel column blocks lie in one 128-row block
    // each, so a step's scale is one number per column block; the tile's rows of the scale
    // matrices sit in a wave-private LDS area (two areas: the next tile's rows are fetched while
    // this one's are in use)
    constexpr int SCB = G::SCALE_ROWS;
    float *const sc_area = (float *)(lds + NS * G::STAGE) + wave * (SCB * kTileScaleBlocks);
    constexpr int kScaleSlotFloats = kTileWaves * SCB * kTileScaleBlocks;
    auto fetch = [&](int t, Ctx &c, int sslot) -> int {
        for (; t < ntiles; t += stride) {
            const WorkItem item = items[t / nb_count];
            const int nb = t % nb_count;
            const ExpertSlab slab = a.slabs[item.expert];
            const uint8_t *wmat = NMAT == 2 ? slab.upgate : slab.down;
            if (wmat == nullptr) continue;       // not loaded: pack has flagged the call
            c.row0 = item.row0;
            c.nrows = item.nrows;
            const int cblock = nb * kTileWaves + wave;
            c.chan0 = cblock * NR * 16;
#pragma unroll
            for (int nr = 0; nr < NR; ++nr) {
                const int ctc = min(cblock * NR + nr, NT - 1);   // tiles past N recompute the last one
                c.wp[nr] = wmat + (int64_t)ctc * (nsteps * KC) * (NMAT * kChunkBytes) + lane * 16;
            }
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                float sv = 1.f;
                if constexpr (WM == kWI8) {
                    const int nr = kSplitBlock ? 0 : (NMAT == 2 ? cb >> 1 : cb) * 2 + hh;
                    const int ch = min(cblock * NR + nr, NT - 1) * 16 + j;
                    const bool gate = kSplitBlock ? hh == 1 : (cb & 1) == 1;
                    sv = NMAT == 2 ? (gate ? slab.s_gate[ch] : slab.s_up[ch]) : slab.s_down[ch];
                }
                c.as[cb] = sv;
                c.ac[cb] = -128.f * sv;
            }
            if constexpr (block_scaled(WM)) {
                const int KB = (a.Kdim + 127) >> 7;
#pragma unroll
                for (int sr = 0; sr < (kSplitBlock ? 2 : CB); ++sr) {
                    // scale row sr belongs to column block sr, or to matrix sr of the one split block
                    const int ct = min(cblock * NR + (kSplitBlock ? 0 : (NMAT == 2 ? sr >> 1 : sr) * 2), NT - 1);
                    const float *smat = NMAT == 2 ? ((sr & 1) == 0 ? slab.s_up : slab.s_gate) : slab.s_down;
                    if (lane < KB)
                        sc_area[sslot * kScaleSlotFloats + sr * kTileScaleBlocks + lane] = smat[(int64_t)((ct * 16) >> 7) * KB + lane];
                }
            }
            c.sslot = sslot;
            if constexpr (block_scaled(WM)) {
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
#pragma unroll
            for (int i = 0; i < LX; ++i) {
                const int rr = min(xrow[i], item.nrows - 1);     // rows past the item re-read its last row
                const int64_t row = a.rows ? (int64_t)a.rows[item.row0 + rr] : (int64_t)(item.row0 + rr);
                c.xsrc[i] = (const T *)a.x + row * a.x_stride + xcol[i];
            }
            return t;
        }
        return -1;
    };

#define EK_ISSUE(ctx, step, ring)                                                               \
    {                                                                                           \
        const uint32_t st_ = lds_base + (ring) * G::STAGE;                                      \
        _Pragma("unroll") for (int nr = 0; nr < NR; ++nr)                                       \
        _Pragma("unroll") for (int m = 0; m < NMAT; ++m)                                        \
        _Pragma("unroll") for (int kc = 0; kc < KC; ++kc)                                       \
            dma16((ctx).wp[nr] + (int64_t)(((step) * KC + kc) * NMAT + m) * kChunkBytes,        \
                  st_ + w_off + ((nr * NMAT + m) * KC + kc) * kChunkBytes);                     \
        _Pragma("unroll") for (int i = 0; i < LX; ++i)                                          \
            dma16((ctx).xsrc[i] + (step) * BK, st_ + xdst[i]);                                  \
    }

    Ctx cur, nxt;
    int tc = fetch(first, cur, 0);
    if (tc < 0) return;
    int ring = 0;                                // stage of the current step
    block_barrier();                             // every wave has left the previous class's stages
    EK_ISSUE(cur, 0, 0);
    if constexpr (AHEAD == 2) EK_ISSUE(cur, 1, 1);

    // The next tile's addresses are needed AHEAD steps before this one ends.  Fetching them
    // makes the wave wait on ordinary loads, i.e. on every vector-memory operation issued
    // before them: it is done a step earlier still, right after the barrier and before
    // the step's DMAs are issued, when only DMAs that are a step old are in flight.
    const int fstep = nsteps > AHEAD + 1 ? nsteps - AHEAD - 1 : 0;
    int pend_st = 0;   // global stores of the previous tile's epilogue, issued after the DMAs of
                       // this tile's first two steps (stores count in vmcnt like loads)
    while (true) {
        int tn = -1;

        f32x16 acc[RB][CB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[rb][cb][r] = 0.f;

        u32x4 af[2][CB];
        V8 bf[2][RB];
        for (int step = 0; step < nsteps; ++step) {
            // the DMAs of this step are older than those of the next one (of this tile or of
            // the next tile) and than the previous epilogue's stores: wait until only those remain
            if constexpr (AHEAD == 2) {
                if (step + 1 < nsteps || tn >= 0) {
                    if (step < 2 && pend_st) wait_vmcnt_dyn(LOADS + pend_st);
                    else wait_vmcnt<LOADS>();
                } else {
                    wait_vmcnt<0>();
                }
            } else {
                // one step in flight: nothing younger than this step's DMAs but, at a tile's first
                // step, the previous epilogue's stores
                if (step == 0 && pend_st) wait_vmcnt_dyn(pend_st);
                else wait_vmcnt<0>();
            }
            block_barrier();   // this step's tile is visible to all waves; the stage of the
                               // previous step is free again
            if (step == fstep) tn = fetch(tc + stride, nxt, cur.sslot ^ 1);
            const int ring2 = ring + AHEAD >= NS ? ring + AHEAD - NS : ring + AHEAD;   // (ring + AHEAD) % NS
            if (step + AHEAD < nsteps) {
                EK_ISSUE(cur, step + AHEAD, ring2);
            } else if (tn >= 0) {
                EK_ISSUE(nxt, step + AHEAD - nsteps, ring2);
            }

            const uint8_t *stage = lds + ring * G::STAGE;
            const uint8_t *wreg = stage + w_off;
            u32x4 aq[W8 ? 2 : 1][CB];   // one-byte weights: the step's A operands as stored; 16-bit: the first k-group's
#pragma unroll
            for (int tt = 0; tt < (W8 ? 2 : 1); ++tt)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) aq[tt][cb] = *(const u32x4 *)(wreg + aoff[cb] + tt * 512);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) bf[0][rb] = *(const V8 *)(stage + boff[0] + rb * kRowBlockBytes);
            float sblk[CB] = {};        // block-scaled weights: this step's scale per column block
            if constexpr (block_scaled(WM)) {
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
                    sblk[cb] = sc_area[cur.sslot * kScaleSlotFloats + (kSplitBlock ? hh : cb) * kTileScaleBlocks + (step >> 1)];
            }
            auto dq = [&](uint32_t w, int cb) -> u32x2 {
                if constexpr (WM == kWF8Block) return dequant_f8x4<T>(w, sblk[cb]);
                else if constexpr (WM == kWI8Block) return dequant_u8x4<T>(w, sblk[cb], -128.f * sblk[cb]);
                else return dequant_u8x4<T>(w, cur.as[cb], cur.ac[cb]);
            };

            // A operands of k-group grp: int8 -> half (grp & 1) of read grp >> 1, dequantised;
            // 16-bit -> read grp as it is.  Software pipeline, pinned with scheduling fences:
            // per row block 2 MFMAs, the B fragment read of the next k-group, and a share of
            // the next k-group's dequantisation.  The pipeline is rotated by one k-group across
            // steps: the MFMAs of a step's last k-group (operands already in af[1] / bf[1]) run
            // at the start of the next step, where they cover the latency of the reads above and
            // the conversion of that step's first k-group, which nothing else could overlap.
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                if (step > 0) {
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb)
                        acc[rb][cb] = Act<T>::mfma32(__builtin_bit_cast(V8, af[1][cb]), bf[1][rb], acc[rb][cb]);
                }
                if constexpr (W8) {
                    // the k-group's 2*CB dwords are spread over the row blocks
#pragma unroll
                    for (int dw = 0; dw < 2 * CB; ++dw) {
                        if (dw * RB / (2 * CB) != rb) continue;
                        const int cb = dw >> 1, part = dw & 1;
                        const u32x2 v = dq(aq[0][cb][part], cb);
                        af[0][cb][part * 2] = v[0];
                        af[0][cb][part * 2 + 1] = v[1];
                    }
                } else {
                    if (rb == RB - 1) {
#pragma unroll
                        for (int cb = 0; cb < CB; ++cb) af[0][cb] = aq[0][cb];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int grp = 0; grp + 1 < NGRP; ++grp) {
                const int cg = grp & 1, ng = cg ^ 1;
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    bf[ng][rb] = *(const V8 *)(stage + boff[grp + 1] + rb * kRowBlockBytes);
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb)
                        acc[rb][cb] = Act<T>::mfma32(__builtin_bit_cast(V8, af[cg][cb]), bf[cg][rb], acc[rb][cb]);
                    if constexpr (W8) {
                        // next group's A operands: 2 dwords per column block, spread over the row blocks
#pragma unroll
                        for (int dw = 0; dw < 2 * CB; ++dw) {
                            if (dw * RB / (2 * CB) != rb) continue;
                            const int cb = dw >> 1, part = dw & 1;
                            const int g1 = grp + 1;
                            const u32x2 v = dq(aq[g1 >> 1][cb][(g1 & 1) * 2 + part], cb);
                            af[ng][cb][part * 2] = v[0];
                            af[ng][cb][part * 2 + 1] = v[1];
                        }
                    } else {
                        if (rb == 0) {
#pragma unroll
                            for (int cb = 0; cb < CB; ++cb) af[ng][cb] = *(const u32x4 *)(wreg + aoff[cb] + (grp + 1) * 512);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            static_assert(((NGRP - 1) & 1) == 1, "the last k-group's operands sit in af[1] / bf[1]");
            ring = ring == NS - 1 ? 0 : ring + 1;
        }
        // the last step's last k-group
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
                acc[rb][cb] = Act<T>::mfma32(__builtin_bit_cast(V8, af[1][cb]), bf[1][rb], acc[rb][cb]);

        // ---- epilogue.  A lane holds, for row rb*32 + l%32, channels q*8 + kg*4 + (0..3),
        //      q = 0..3, of each column block: written as they are, a store instruction would
        //      touch 32 rows with 16 bytes each.  The rounded values go through LDS instead
        //      (the stage of the last step, once every wave has left it), wave-private, one
        //      32-row block at a time, and leave as whole rows: 16 bytes per lane, a row of the
        //      wave's OUTC channels per 2*OUTC/16 lanes.
        typedef T T4 __attribute__((ext_vector_type(4)));
        constexpr int OUTC = NMAT == 2 ? CB * 16 : CB * 32;   // output channels per wave
        constexpr int RS = OUTC * 2 + 16;                  // scratch row stride: 16 bytes of padding
        constexpr int PPO = OUTC * 2 / 16, RPI = 64 / PPO; // pieces per row, rows per store instruction
        static_assert(kTileWaves * 32 * RS <= G::STAGE, "epilogue scratch fits one stage");
        block_barrier();
        pend_st = 0;
        if (cur.chan0 < a.N) {
            uint8_t *scr = lds + (ring == 0 ? NS - 1 : ring - 1) * G::STAGE + wave * (32 * RS);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                if (rb * 32 >= cur.nrows) break;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if constexpr (kSplitBlock) {
                        if (q < 2) {
                            T4 o;
#pragma unroll
                            for (int r = 0; r < 4; ++r)
                                o[r] = swiglu_rounded<T>(acc[rb][0][q * 4 + r], acc[rb][0][(q + 2) * 4 + r]);
                            *(uint2 *)(scr + l32 * RS + (q * 8 + kg * 4) * 2) = __builtin_bit_cast(uint2, o);
                        }
                    } else if constexpr (NMAT == 2) {
#pragma unroll
                        for (int c2 = 0; c2 < CB / 2; ++c2) {
                            T4 o;
#pragma unroll
                            for (int r = 0; r < 4; ++r)
                                o[r] = swiglu_rounded<T>(acc[rb][2 * c2][q * 4 + r], acc[rb][2 * c2 + 1][q * 4 + r]);
                            *(uint2 *)(scr + l32 * RS + (c2 * 32 + q * 8 + kg * 4) * 2) = __builtin_bit_cast(uint2, o);
                        }
                    } else {
#pragma unroll
                        for (int cb = 0; cb < CB; ++cb) {
                            T4 o;
#pragma unroll
                            for (int r = 0; r < 4; ++r) o[r] = (T)acc[rb][cb][q * 4 + r];
                            *(uint2 *)(scr + l32 * RS + (cb * 32 + q * 8 + kg * 4) * 2) = __builtin_bit_cast(uint2, o);
                        }
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int i = 0; i < 32 / RPI; ++i) {
                    if (rb * 32 + i * RPI >= cur.nrows) break;    // wave-uniform: the count below is exact
                    const int r_in = rb * 32 + i * RPI + lane / PPO;
                    const u32x4 v = *(const u32x4 *)(scr + (i * RPI + lane / PPO) * RS + (lane % PPO) * 16);
                    if (r_in < cur.nrows)
                        *(u32x4 *)((T *)a.out + (int64_t)(cur.row0 + r_in) * a.out_stride + cur.chan0 + (lane % PPO) * 8) = v;
                    pend_st += 1;
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        }
        if (tn < 0) break;
        cur = nxt;
        tc = tn;
    }
#undef EK_ISSUE
}

// ---- short tiles with weights streamed into registers ------------------------------------------
// 32- and 64-row items whose expert has one or two tiles (a few dozen rows per expert: layer
// calls between the decode and the prefill regime, the mid-sized experts of a skewed prefill) read
// weights that are cold in every cache, and with 32 or 64 rows the accumulators take 32 to 64
// registers.  This form gives the rest to the loads: a lane's 16 bytes of a 1 KiB weight chunk are
// exactly its A-operand bytes (two runs of 512 contiguous bytes per load instruction), so the
// weights come straight from HBM into registers, kMidDepth steps ahead, as the weight-streaming
// kernel fetches them, and never touch LDS.  Only the activation tile (4 or 8 KiB per step) goes
// through LDS: one 16-byte piece per thread and step, fetched one to two windows of kMidDepth
// steps ahead into a register and stored (XOR-swizzled as in run_tiles) into the other of two
// window buffers during the window before its own; one workgroup barrier per window publishes it,
// so the waves drift apart by up to a window instead of meeting at every step.  All loads are
// ordinary loads: the compiler counts them.
// Loads run across tile boundaries like run_tiles' DMAs.  Arithmetic, operand layouts, channel
// split over the waves and the epilogue are run_tiles' (wide form): same bits.
// 16-bit weights bring twice the bytes per step: two steps ahead then hold what four steps of
// one-byte weights hold (64 registers per lane, 128 KiB per CU in flight).
// Needs a contraction of a multiple of 64 * mid_depth elements, at least 2 * mid_depth steps long;
// the caller falls back to run_tiles otherwise.
constexpr int kMidDepth = 4;                    // one-byte weights
constexpr int mid_depth(int wm) { return wm == kW16 ? 2 : kMidDepth; }
constexpr int kMidXStep = 8192;                 // bytes reserved per step of the activation tile (64 rows x 64 k x 2)
constexpr int kMidXBuf = kMidDepth * kMidXStep; // one window (of kMidDepth steps at most)
constexpr int kMidScratch = 2 * kMidXBuf;       // epilogue scratch behind the two window buffers
constexpr int kMidEnd = kMidScratch + 8 * 32 * 144;      // end of what this form stores into with waves of other tiles in flight
// The block scales ([tile parity][wave][column block][block], wave-private) do not live in that
// range: a wave fetches its first tile's scale rows before the barrier that separates this form from
// the class that ran before it, while slower waves may still be reading that class's stages and
// epilogue scratch.  They share run_tiles' own scale area behind its stages (same layout, and a wave
// touches only its own part of it in either form).

template <typename T> struct MidCtx {
    const uint8_t *wl[2];    // this lane's bytes of the column block's weight chunks at step 0, slot tt = 0
    const T *xsrc;           // this thread's 16-byte piece of the activation tile at step 0
    float as[2], ac[2];
    int row0, nrows, chan0;
    int sslot;               // block-scaled weights: which of the two LDS scale areas holds this tile's rows
};

template <typename T, int WM, int NMAT, int MR>
__device__ __forceinline__ void run_mid(const FfnArgs &a, const WorkItem *items, const int ntiles,
                                        const int nb_count, const int first, const int stride, uint8_t *lds,
                                        float *scales)
{
    using V8 = typename Act<T>::V8;
    constexpr bool W8 = WM != kW16;
    constexpr int WAVES = 8, CB = 2, NR = 4 / NMAT, D = mid_depth(WM), KC = W8 ? 1 : 2;
    constexpr int NQ = W8 ? 2 : 4;             // 16-byte loads per lane, column block and step
    constexpr int BM = MR * 16, RB = MR / 2, BK = 64, PPR = 8, NGRP = 4;
    constexpr int kRowBlockBytes = 32 * PPR * 16;
    static_assert(MR == 2 || MR == 4, "32- and 64-row items");
    typedef MidCtx<T> Ctx;
    if (first >= ntiles) return;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, l32 = lane & 31, kg = lane >> 5, hh = l32 >> 4;
    const int NT = a.N >> 4;
    const int nsteps = a.Kdim / BK;
    // this thread's piece of the activation tile
    const int xrow = tid / PPR, xpiece = tid % PPR;
    const bool xactive = xrow < BM;
    const int xdst = (xrow * PPR + (xpiece ^ swizzle_key<PPR>(xrow))) * 16;
    int boff[NGRP];
#pragma unroll
    for (int grp = 0; grp < NGRP; ++grp) {
        const int c = W8 ? ((grp >> 1) * 2 + kg) * 2 + (grp & 1) : grp * 2 + kg;
        boff[grp] = (l32 * PPR + (c ^ swizzle_key<PPR>(j))) * 16;
    }
    // block scales: as in run_tiles, the tile's rows of the scale matrices in a wave-private LDS area
    float *const sc_area = scales + wave * (CB * kTileScaleBlocks);
    constexpr int kScaleSlotFloats = WAVES * CB * kTileScaleBlocks;
    auto fetch = [&](int t, Ctx &c, int sslot) -> int {
        for (; t < ntiles; t += stride) {
            const WorkItem item = items[t / nb_count];
            const int nb = t % nb_count;
            const ExpertSlab slab = a.slabs[item.expert];
            const uint8_t *wmat = NMAT == 2 ? slab.upgate : slab.down;
            if (wmat == nullptr) continue;       // not loaded: pack has flagged the call
            c.row0 = item.row0;
            c.nrows = item.nrows;
            c.sslot = sslot;
            const int cblock = nb * WAVES + wave;
            c.chan0 = cblock * NR * 16;
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const int nr = (NMAT == 2 ? 0 : cb) * 2 + hh, m = NMAT == 2 ? cb : 0;
                const int ctc = min(cblock * NR + nr, NT - 1);   // tiles past N recompute the last one
                c.wl[cb] = wmat + ((int64_t)ctc * nsteps * KC * NMAT + m) * kChunkBytes + (kg * 16 + j) * 16;
                float sv = 1.f;
                if constexpr (WM == kWI8) {
                    const int ch = ctc * 16 + j;
                    sv = NMAT == 2 ? (cb == 0 ? slab.s_up[ch] : slab.s_gate[ch]) : slab.s_down[ch];
                }
                c.as[cb] = sv;
                c.ac[cb] = -128.f * sv;
                if constexpr (block_scaled(WM)) {
                    const int KB = (a.Kdim + 127) >> 7;
                    const int ct = min(cblock * NR + (NMAT == 2 ? 0 : cb * 2), NT - 1);
                    const float *smat = NMAT == 2 ? (cb == 0 ? slab.s_up : slab.s_gate) : slab.s_down;
                    if (lane < KB)
                        sc_area[sslot * kScaleSlotFloats + cb * kTileScaleBlocks + lane] = smat[(int64_t)((ct * 16) >> 7) * KB + lane];
                }
            }
            if constexpr (block_scaled(WM)) {
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
            const int rr = min(min(xrow, BM - 1), item.nrows - 1);   // rows past the item (and threads past the tile) re-read its last row
            const int64_t row = a.rows ? (int64_t)a.rows[item.row0 + rr] : (int64_t)(item.row0 + rr);
            c.xsrc = (const T *)a.x + row * a.x_stride + xpiece * 8;
            return t;
        }
        return -1;
    };
    u32x4 wq[D][NQ][CB];     // ring of weight bytes: slot s % D holds step s
    // load q of a step: one-byte weights, the two halves of the step's chunk; 16-bit weights, the
    // two halves of its two chunks (k-group q)
    auto w_off = [&](int step, int q) -> int64_t {
        return W8 ? (int64_t)step * (NMAT * kChunkBytes) + q * 512
                  : (int64_t)(step * 2 + (q >> 1)) * (NMAT * kChunkBytes) + (q & 1) * 512;
    };
    u32x4 xq[D];             // activation pieces of the window after next: slot u holds its step u
    auto load_w = [&](const Ctx &c, int step, int slot) {
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
                wq[slot][q][cb] = __builtin_bit_cast(u32x4, ldg16_once(c.wl[cb] + w_off(step, q)));
    };
    auto load_x = [&](const Ctx &c, int step, int slot) {
        xq[slot] = __builtin_bit_cast(u32x4, ldg16(c.xsrc + step * BK));
    };
    // The loads of a step are unconditional and land in the ring slot they refill (no copies, no
    // merges of register values across branches: the compiler then keeps the ring in place and waits
    // for exactly the loads a step needs).  Past the last tile's end they re-read its first steps.

    Ctx cur, nxt;
    int tc = fetch(first, cur, 0);
    if (tc < 0) return;
    nxt = cur;
#pragma unroll
    for (int v = 0; v < D; ++v) { load_w(cur, v, v); load_x(cur, v, v); }
    block_barrier();                             // every wave has left the previous class's LDS
    int par = 0;                                 // buffer of the current window
#pragma unroll
    for (int v = 0; v < D; ++v) {
        if (xactive) *(u32x4 *)(lds + v * kMidXStep + xdst) = xq[v];
        load_x(cur, D + v, v);                   // (nsteps >= 2 D)
    }
    lds_barrier();
    const int fstep = nsteps - 2 * D;            // the next tile's addresses are needed from here on
    while (true) {
        int tn = -1;
        f32x16 acc[RB][CB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[rb][cb][r] = 0.f;
        for (int step0 = 0; step0 < nsteps; step0 += D) {
#pragma unroll
            for (int u = 0; u < D; ++u) {
                const int step = step0 + u;
                if (step == fstep) {
                    tn = fetch(tc + stride, nxt, cur.sslot ^ 1);
                    if (tn < 0) nxt = cur;
                }
                // the piece of step + D goes to the other window buffer; its slot takes step + 2 D
                if (xactive) *(u32x4 *)(lds + (par ^ 1) * kMidXBuf + u * kMidXStep + xdst) = xq[u];
                {
                    const bool in_cur = step + 2 * D < nsteps;
                    const T *xp = in_cur ? cur.xsrc : nxt.xsrc;
                    const int xs = in_cur ? step + 2 * D : step + 2 * D - nsteps;
                    xq[u] = __builtin_bit_cast(u32x4, ldg16(xp + xs * BK));
                }
                u32x4 (&aq)[NQ][CB] = wq[u];
                const uint8_t *stage = lds + par * kMidXBuf + u * kMidXStep;
                u32x4 af[2][CB];
                V8 bf[2][RB];
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) bf[0][rb] = *(const V8 *)(stage + boff[0] + rb * kRowBlockBytes);
                float sblk[CB] = {};        // block-scaled weights: this step's scale per column block
                if constexpr (block_scaled(WM)) {
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb)
                        sblk[cb] = sc_area[cur.sslot * kScaleSlotFloats + cb * kTileScaleBlocks + (step >> 1)];
                }
                auto dq = [&](uint32_t w, int cb) -> u32x2 {
                    if constexpr (WM == kWF8Block) return dequant_f8x4<T>(w, sblk[cb]);
                    else if constexpr (WM == kWI8Block) return dequant_u8x4<T>(w, sblk[cb], -128.f * sblk[cb]);
                    else return dequant_u8x4<T>(w, cur.as[cb], cur.ac[cb]);
                };
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    if constexpr (W8) {
                        const u32x2 lo = dq(aq[0][cb][0], cb);
                        const u32x2 hi = dq(aq[0][cb][1], cb);
                        af[0][cb] = u32x4{lo[0], lo[1], hi[0], hi[1]};
                    } else {
                        af[0][cb] = aq[0][cb];
                    }
                }
#pragma unroll
                for (int grp = 0; grp < NGRP; ++grp) {
                    const int cg = grp & 1, ng = cg ^ 1;
                    if (grp + 1 < NGRP) {
#pragma unroll
                        for (int rb = 0; rb < RB; ++rb) bf[ng][rb] = *(const V8 *)(stage + boff[grp + 1] + rb * kRowBlockBytes);
                    }
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                        for (int cb = 0; cb < CB; ++cb)
                            acc[rb][cb] = Act<T>::mfma32(__builtin_bit_cast(V8, af[cg][cb]), bf[cg][rb], acc[rb][cb]);
                    if (grp + 1 < NGRP) {
                        const int g1 = grp + 1;
#pragma unroll
                        for (int cb = 0; cb < CB; ++cb) {
                            if constexpr (W8) {
                                const u32x2 lo = dq(aq[g1 >> 1][cb][(g1 & 1) * 2], cb);
                                const u32x2 hi = dq(aq[g1 >> 1][cb][(g1 & 1) * 2 + 1], cb);
                                af[ng][cb] = u32x4{lo[0], lo[1], hi[0], hi[1]};
                            } else {
                                af[ng][cb] = aq[g1][cb];
                            }
                        }
                    }
                }
                // this step's weight bytes have been converted: their slot takes step + D
                {
                    const bool in_cur = step + D < nsteps;
                    const int ws = in_cur ? step + D : step + D - nsteps;
#pragma unroll
                    for (int q = 0; q < NQ; ++q)
#pragma unroll
                        for (int cb = 0; cb < CB; ++cb) {
                            const uint8_t *wp_ = in_cur ? cur.wl[cb] : nxt.wl[cb];
                            wq[u][q][cb] = __builtin_bit_cast(u32x4, ldg16_once(wp_ + w_off(ws, q)));
                        }
                }
            }
            par ^= 1;
            lds_barrier();         // the next window's buffer is complete; this window's may be overwritten
        }
        // ---- epilogue: as run_tiles, through a wave-private scratch behind the two buffers
        typedef T T4 __attribute__((ext_vector_type(4)));
        constexpr int OUTC = NMAT == 2 ? 32 : 64;
        constexpr int RS = OUTC * 2 + 16;
        constexpr int PPO = OUTC * 2 / 16, RPI = 64 / PPO;
        if (cur.chan0 < a.N) {
            uint8_t *scr = lds + kMidScratch + wave * (32 * RS);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                if (rb * 32 >= cur.nrows) break;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if constexpr (NMAT == 2) {
                        T4 o;
#pragma unroll
                        for (int r = 0; r < 4; ++r) o[r] = swiglu_rounded<T>(acc[rb][0][q * 4 + r], acc[rb][1][q * 4 + r]);
                        *(uint2 *)(scr + l32 * RS + (q * 8 + kg * 4) * 2) = __builtin_bit_cast(uint2, o);
                    } else {
#pragma unroll
                        for (int cb = 0; cb < CB; ++cb) {
                            T4 o;
#pragma unroll
                            for (int r = 0; r < 4; ++r) o[r] = (T)acc[rb][cb][q * 4 + r];
                            *(uint2 *)(scr + l32 * RS + (cb * 32 + q * 8 + kg * 4) * 2) = __builtin_bit_cast(uint2, o);
                        }
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int i = 0; i < 32 / RPI; ++i) {
                    const int r_in = rb * 32 + i * RPI + lane / PPO;
                    const u32x4 v = *(const u32x4 *)(scr + (i * RPI + lane / PPO) * RS + (lane % PPO) * 16);
                    if (r_in < cur.nrows)
                        *(u32x4 *)((T *)a.out + (int64_t)(cur.row0 + r_in) * a.out_stride + cur.chan0 + (lane % PPO) * 8) = v;
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        }
        if (tn < 0) break;
        cur = nxt;
        tc = tn;
    }
    lds_barrier();
}

// Persistent launch: one workgroup per CU (the LDS stages fill it), numbered so that
// workgroup b runs on XCD b % 8 (round-robin dispatch).  Each XCD is given a contiguous
// eighth of every work list, and its workgroups walk that eighth's tiles side by side:
// neighbouring CUs share the activation tile (same item) and mostly the expert's weights
// in the XCD's L2.  Every workgroup's tile sequence is fixed by its index: no queues, no
// spinning, and it ends when its indices run out.
template <typename T, int WM, int NMAT, int WAVES, int CB>
__global__ __launch_bounds__(WAVES * 64, 1) void ffn_tile_kernel(FfnArgs a, int nb_count)
{
    using G = TileGeom<WM != kW16, WAVES, CB, 128>;
    __shared__ __attribute__((aligned(1024)))
    uint8_t lds[G::STAGES * G::STAGE + (block_scaled(WM) ? G::SCALE_BYTES : 0)];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr)lds;
    const int x = blockIdx.x & 7, slot = blockIdx.x >> 3, nslots = gridDim.x >> 3;
    const int n128 = a.lists.count[kListT128], n64 = a.lists.count[kListT64], n32 = a.lists.count[kListT32];
    const int lo128 = x * n128 / 8, s128 = (x + 1) * n128 / 8 - lo128;
    const int lo64 = x * n64 / 8, s64 = (x + 1) * n64 / 8 - lo64;
    const int lo32 = x * n32 / 8, s32 = (x + 1) * n32 / 8 - lo32;
    run_tiles<T, WM, NMAT, 8, WAVES, CB, 128>(a, a.lists.items[kListT128] + lo128, s128 * nb_count, nb_count, slot, nslots, lds, lds_base);
    // the shorter classes start where the long one left the CUs least loaded
    const int r64 = (slot + nslots - (s128 * nb_count) % nslots) % nslots;
    if constexpr (CB == 2 && WAVES == 8) {
        // the register-streamed form for the short items of a launch whose tiles fill the chip
        // (measured: DeepSeek-V3 int8 layer at 512 / 1024 tokens -5 / -8 %, the ragged Qwen3 fp16
        // chain -2.5 %); with a few tiles beside a long streaming chain (Qwen3 fp16 decode with
        // skewed routing: +5 %) run_tiles' form is the faster one
        const int nsteps = a.Kdim / 64;
        if (nsteps % mid_depth(WM) == 0 && nsteps >= 2 * mid_depth(WM) &&
            (int64_t)(n128 + n64 + n32) * nb_count >= (int64_t)gridDim.x) {
            const int r32m = (r64 + nslots - (s64 * nb_count) % nslots) % nslots;
            static_assert(kMidEnd <= G::STAGES * G::STAGE, "the register-streamed form's buffers end before the scale area");
            static_assert(TileGeom<true, 8, 2, 128>::SCALE_ROWS == 2, "both forms lay the scale area out alike");
            float *const scales = (float *)(lds + G::STAGES * G::STAGE);
            run_mid<T, WM, NMAT, 4>(a, a.lists.items[kListT64] + lo64, s64 * nb_count, nb_count, r64, nslots, lds, scales);
            run_mid<T, WM, NMAT, 2>(a, a.lists.items[kListT32] + lo32, s32 * nb_count, nb_count, r32m, nslots, lds, scales);
            return;
        }
    }
    run_tiles<T, WM, NMAT, 4, WAVES, CB, 128>(a, a.lists.items[kListT64] + lo64, s64 * nb_count, nb_count, r64, nslots, lds, lds_base);
    const int r32 = (r64 + nslots - (s64 * nb_count) % nslots) % nslots;
    run_tiles<T, WM, NMAT, 2, WAVES, CB, 128>(a, a.lists.items[kListT32] + lo32, s32 * nb_count, nb_count, r32, nslots, lds, lds_base);
}

template <typename T, int WM, int NMAT, int WAVES, int CB>
static hipError_t launch_t(const FfnArgs &a, const int64_t max_items[kNumLists], hipStream_t s)
{
    constexpr int NR = 2 * CB / NMAT;            // channel tiles per wave and matrix
    const int NT = a.N / 16;
    const int nb_count = (NT + WAVES * NR - 1) / (WAVES * NR);
    const int64_t per_xcd = (max_items[kListT128] + 7) / 8 + (max_items[kListT64] + 7) / 8 +
                            (max_items[kListT32] + 7) / 8;
    int64_t slots = per_xcd * nb_count;          // tiles an XCD can get at most
    if (slots <= 0) return hipSuccess;
    if (slots > kCusPerXcd) slots = kCusPerXcd;
    hipLaunchKernelGGL((ffn_tile_kernel<T, WM, NMAT, WAVES, CB>), dim3((unsigned)(slots * 8)), dim3(WAVES * 64), 0, s, a,
                       nb_count);
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_w(const FfnArgs &a, int stage, int wmode, const int64_t max_items[kNumLists], bool narrow,
                           hipStream_t s)
{
    switch (wmode) {
    case kWI8:
        if (narrow)
            return stage == 1 ? launch_t<T, kWI8, 2, 8, 1>(a, max_items, s) : launch_t<T, kWI8, 1, 8, 1>(a, max_items, s);
        return stage == 1 ? launch_t<T, kWI8, 2, 8, 2>(a, max_items, s) : launch_t<T, kWI8, 1, 8, 2>(a, max_items, s);
    case kWF8Block:
        if (narrow)
            return stage == 1 ? launch_t<T, kWF8Block, 2, 8, 1>(a, max_items, s) : launch_t<T, kWF8Block, 1, 8, 1>(a, max_items, s);
        return stage == 1 ? launch_t<T, kWF8Block, 2, 8, 2>(a, max_items, s) : launch_t<T, kWF8Block, 1, 8, 2>(a, max_items, s);
    case kWI8Block:
        if (narrow)
            return stage == 1 ? launch_t<T, kWI8Block, 2, 8, 1>(a, max_items, s) : launch_t<T, kWI8Block, 1, 8, 1>(a, max_items, s);
        return stage == 1 ? launch_t<T, kWI8Block, 2, 8, 2>(a, max_items, s) : launch_t<T, kWI8Block, 1, 8, 2>(a, max_items, s);
    default:
        if (narrow)
            return stage == 1 ? launch_t<T, kW16, 2, 8, 1>(a, max_items, s) : launch_t<T, kW16, 1, 8, 1>(a, max_items, s);
        return stage == 1 ? launch_t<T, kW16, 2, 8, 2>(a, max_items, s) : launch_t<T, kW16, 1, 8, 2>(a, max_items, s);
    }
}

hipError_t launch_ffn_tile(const FfnArgs &a, int stage, int act, int wmode,
                           const int64_t max_items[kNumLists], bool narrow, hipStream_t s)
{
    // forms that run three stages deep issue a tile's first two steps up front: the contraction
    // must have two (one-byte weights: hidden, inter >= 128 always; 16-bit: the narrow form)
    if ((narrow || wmode != kW16) && a.Kdim < 128) return hipErrorInvalidValue;
    return act == 0 ? launch_w<__bf16>(a, stage, wmode, max_items, narrow, s)
                    : launch_w<_Float16>(a, stage, wmode, max_items, narrow, s);
}

}  // namespace ek
