// Internal declarations shared by the HIP kernels and the C-ABI host code.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ek {

// ---- HBM weight layout ------------------------------------------------------
// A weight matrix [N, K] (row-major, out_features x in_features) is stored as
// 1 KiB chunks.  One chunk is what one wavefront fetches with a single 16-byte
// load per lane and feeds to MFMA without any shuffle:
//   chunk (nt, kt) covers rows nt*16 .. nt*16+15 and KE consecutive k
//   (KE = 64 for int8, 32 for 16-bit types); lane l = g*16 + i holds the
//   16 bytes W[nt*16 + i][kt*KE + g*KE/4 .. + KE/4).
// A "matrix group" interleaves NMAT matrices of equal shape chunk by chunk
// (up and gate are one group, so one wave streams one contiguous range):
//   byte offset of chunk (nt, kt, m) = ((nt*KT + kt)*NMAT + m) * 1024.
// int8 values are stored offset-binary (q + 128, i.e. q ^ 0x80) so that
// v_cvt_f32_ubyte* converts them; the kernels fold the -128 into the
// dequantisation fma.
constexpr int kChunkBytes = 1024;

// How a layer keeps its weights in HBM.
enum WeightMode {
    kW16 = 0,        // the activation type (bf16 / fp16): 32 contraction elements per 1 KiB chunk
    kWI8 = 1,        // int8, offset-binary, one fp32 scale per output channel: 64 per chunk
    kWF8Block = 2,   // fp8 e4m3fn, one fp32 scale per 128 x 128 block: 64 per chunk
    kWI8Block = 3    // int8, offset-binary, one fp32 scale per 128 x 128 block: 64 per chunk
};
constexpr bool block_scaled(int wm) { return wm == kWF8Block || wm == kWI8Block; }

struct ExpertSlab {           // device addresses of one expert's tensors
    const uint8_t *upgate;    // matrix group {up, gate}: N = I, K = H
    const uint8_t *down;      // matrix group {down}:     N = H, K = I
    const float *s_up;        // fp32 scales: [I] per channel (kWI8), [ceil(I/128), ceil(H/128)] per block
    const float *s_gate;      //   (kWF8Block, kWI8Block), nullptr for 16-bit weights; same shape as s_up
    const float *s_down;      // [H] per channel, [ceil(H/128), ceil(I/128)] per block
};

// ---- work lists ---------------------------------------------------------------
// The pack step cuts every expert segment into work items for the FFN kernels:
// as many full 128-row tiles as fit, then the remainder r by size:
//   r <= 16 -> one weight-streaming item, r <= 32 / <= 64 / <= 128 -> one MFMA
//   tile of 32 / 64 / 128 rows.
// Items of one class are stored expert-ascending, rows ascending.  List sizes
// depend on the routing, list capacities only on P, so grids are fixed on the
// host and kernels drop items beyond the device-side count.
//
// Wide cut (per-expert entry points only, decided on the host): when a call's tile items
// would occupy a small part of the chip (see wide_cut_pays), every segment is cut into
// weight-streaming items of up to kWideRows rows instead and the tile lists stay empty.
struct WorkItem {
    int32_t expert;
    int32_t row0;    // first packed position
    int32_t nrows;
    int32_t pad;
};
enum { kListStream = 0, kListT32 = 1, kListT64 = 2, kListT128 = 3, kNumLists = 4 };
struct WorkLists {
    WorkItem *items[kNumLists];
    int32_t *count;              // [kNumLists]
};
constexpr int kWideRows = 64;
// tile_items: work items the ordinary cut would give the tile kernel; one of them spreads
// over ceil(inter / 128) workgroups in stage 1 (the tile kernel's narrow form, which such calls
// get), and below half a chip of them the call takes as long as one tile's two contractions
// however few rows it has: ~30 us + (hidden + inter) x 13.6 ns, with one-byte and 16-bit weights
// alike.  The streaming kernel spreads every item over inter / 16 workgroups, each of which reads
// its item's rows, and its time grows with the rows: ~ rows x (53 ns + hidden x inter x 14.8 fs).
// Fitted on MI355X to one DeepSeek-V3 expert (hidden 7168, inter 2048; tiled 152-158 us from 64 to
// 1024 rows with int8 weights, 150 us with bf16; streamed 143 / 188 / 199 us at 512 / 640 / 768
// rows) and to the Qwen3 shape (2048, 768: tiled 66 us fp16, 69 us int8; streamed 37 / 46 / 62 us
// at 512 / 640 / 768 rows).
inline double tile_call_us(int64_t hidden, int64_t inter) { return 30.0 + (double)(hidden + inter) * 0.0136; }
inline bool wide_cut_pays(int64_t tile_items, int64_t rows, int64_t hidden, int64_t inter)
{
    if (tile_items <= 0 || tile_items * ((inter + 255) / 256) >= 128) return false;
    const double streamed_us = (double)rows * (0.053 + 1.48e-8 * (double)hidden * (double)inter);
    return streamed_us < 0.92 * tile_call_us(hidden, inter);
}
inline int64_t list_capacity(int list, int64_t P, int64_t E)
{
    const int64_t min_rows[kNumLists] = {1, 17, 33, 65};
    const int64_t by_rows = P / min_rows[list];
    if (list == kListT128) return by_rows;
    return by_rows < E ? by_rows : E;
}

// ---- router (logits -> ids, gate weights) -------------------------------------
struct RouterArgs {
    const void *logits;       // [T, E]
    int32_t logits_dt;        // 0 bf16, 1 f16, 2 f32
    const float *bias;        // [E] or nullptr (kind 4: added to the scores for the choice only)
    int64_t T;
    int32_t E, K;
    int32_t kind;             // ek_router_kind
    int32_t renorm;
    int32_t n_group, topk_group;
    int32_t mask_neg_inf;     // kind 4: experts outside the kept groups compete with -inf instead of 0
    float routed_scaling;
    int32_t *ids;             // [T, K]
    void *w;                  // [T, K]
    int32_t w_dt;             // 0 bf16, 1 f16, 2 f32
};
// needs E <= 1024, K <= 64, n_group <= 64 (checked by the caller)
hipError_t launch_router(const RouterArgs &a, hipStream_t s);

// ---- routing (pack) ---------------------------------------------------------
struct PackArgs {
    const int32_t *ids;       // [P]
    int64_t P;
    int32_t E;
    int32_t K;
    int32_t nblocks;          // ceil(P / kPackChunk)
    const ExpertSlab *slabs;  // [E]; upgate == nullptr means "not loaded"
    int32_t *block_hist;      // [nblocks][E]
    int32_t *counts;          // [E]
    int32_t *offsets;         // [E+1]
    int32_t *perm;            // [P]
    int32_t *inv_perm;        // [P]
    int32_t *row_token;       // [P]  perm[j] / K
    int32_t *err;             // bit 0: id out of range, bit 1: expert not loaded
    uint64_t *activation;     // [E] running sum of counts over calls, or nullptr
    int32_t *tile_items_host; // pinned host word that receives the number of tile items cut, or nullptr
    WorkLists lists;
};
constexpr int kPackChunk = 4096;   // pairs per workgroup
constexpr int kPackThreads = 256;
constexpr int kMaxExperts = 1024;

// writes *err itself (one kernel of every pack stores the call's word: nothing to clear first,
// no memset node: graph-capture safe)
void launch_pack(const PackArgs &a, hipStream_t s);
// work lists for one segment [0, n) of expert e (per-expert forward)
void launch_single_lists(const WorkLists &lists, int32_t expert, int32_t n, bool wide, hipStream_t s);
// lists that hold the one segment (expert, rows row0 .. row0+n-1) and nothing else; mode 0: the usual
// cut, 1: 16-row streaming items, 2: streaming items of up to kWideRows rows.  row_token, if given,
// receives row0 + t -> t.
void launch_segment_lists(const WorkLists &lists, int32_t expert, int32_t row0, int32_t n, int32_t *row_token, int mode,
                          hipStream_t s);
// appends the segment (expert, rows row0 .. row0+n-1) to the lists pack has built and maps
// its rows to tokens 0 .. n-1.  as_stream: 0 the usual cut; 1 all rows as 16-row streaming items;
// 2 all rows as streaming items of up to kWideRows rows, which replace the streaming list (the
// caller passes a list of their own)
void launch_append_segment(const WorkLists &lists, int32_t expert, int32_t row0, int32_t n, int32_t *row_token,
                           int as_stream, hipStream_t s);
void launch_gather(const void *x, const int32_t *row_token, int64_t P, int64_t row_bytes, void *xp,
                   hipStream_t s);

// ---- grouped FFN -------------------------------------------------------------
struct FfnArgs {
    const void *x;            // activations, row stride x_stride elements
    int64_t x_stride;
    const int32_t *rows;      // packed position -> row of x, or nullptr (identity)
    const ExpertSlab *slabs;  // [E]
    void *out;                // stage 1: h [P, N]; stage 2: yp [P, N]
    int64_t out_stride;
    int32_t N;                // output channels of this stage
    int32_t Kdim;             // contraction length of this stage
    WorkLists lists;          // device work lists and their lengths
    // pair-direct launches (launch_ffn_pairs): pair p = t * pair_K + k is its own one-row item,
    // x row t (stage 1) or p (stage 2), out row p; no lists
    const int32_t *pair_ids = nullptr;   // [pair_P] expert of pair p
    int32_t pair_K = 0, pair_P = 0, n_experts = 0;
    const void *pair_w = nullptr;        // [pair_P] gate weights (stage 2)
    int32_t pair_w_f32 = 0;              // gate weights are fp32 instead of the activation type
    int32_t pair_shared = 0;             // 1: every token also runs expert n_experts (the shared expert) as item
                                         // pair_P + t (x row t, out row pair_P + t); its rounded output is added
                                         // to the rounded weighted sum, as the combine kernel adds it
    void *pair_y = nullptr;              // [T, N] stage 2: the weighted sum over a token's pairs
    int32_t *pair_err = nullptr;         // stage 1 writes the call's error word (PackArgs::err)
    uint64_t *pair_activation = nullptr; // [n_experts] or nullptr (PackArgs::activation)
    int32_t *pair_tile_items_host = nullptr;   // receives 0 (PackArgs::tile_items_host), or nullptr
};
// Most pairs a pair-direct call may hold (one wave writes the call's bookkeeping) and its
// largest top-k (one wave per pair of a token in stage 2's workgroups).
constexpr int kPairDirectMax = 64, kPairDirectMaxK = 8;
// A decode call of a few pairs without pack and combine kernels: stage 1 runs every pair as a
// one-row item straight from the ids (and stores what the pack kernel would have stored of the
// call's bookkeeping: error word, activation counters, zero tile items); stage 2 computes a
// token's pairs in one workgroup, one wave each, and adds them in k order with the gate weights:
// the arithmetic of the streaming kernel followed by launch_combine, bit for bit.  Pairs whose
// id is out of range or whose expert is not loaded add nothing.  T = pair_P / pair_K.
hipError_t launch_ffn_pairs(const FfnArgs &a, int stage, int act, int wmode, hipStream_t s);
// stage = 1: up/gate + SwiGLU epilogue;  stage = 2: down projection
// act: 0 bf16, 1 f16;  wmode: WeightMode
// weight-streaming kernel over lists.items[kListStream]; max_items = grid bound;
// wide: items hold up to kWideRows rows (else up to 16); few_rows: about four rows or fewer per
// item on average (a hint for the launch shape; the results do not depend on it)
hipError_t launch_ffn_stream(const FfnArgs &a, int stage, int act, int wmode, int64_t max_items, bool wide,
                             bool few_rows, hipStream_t s);
// MFMA tile kernel over the three tile lists (128-row items first, then 64,
// then 32); max_items[l] bounds list l.  A workgroup covers tile_channels(stage, narrow) output
// channels of one item; the narrow form (half the channels per workgroup, so twice the workgroups
// per item; same bits) is for launches that would leave most of the chip without a tile.
hipError_t launch_ffn_tile(const FfnArgs &a, int stage, int act, int wmode,
                           const int64_t max_items[kNumLists], bool narrow, hipStream_t s);
// hidden channels (stage 1) / output channels (stage 2) per tile workgroup
constexpr int tile_channels(int stage, bool narrow) { return (stage == 1 ? 256 : 512) / (narrow ? 2 : 1); }

// ---- combine ----------------------------------------------------------------
struct CombineArgs {
    const void *yp;           // [P, H] packed expert outputs
    const int32_t *inv_perm;  // [T*K]
    const void *w;            // [T, K]
    void *y;                  // [T, H]
    int64_t T;
    int32_t K;
    int64_t H;
    int32_t act;              // 0 bf16, 1 f16
    int32_t w_f32;            // gate weights are fp32 (DeepSeek shim) instead of act dtype
    const void *shared;       // [T, H] shared-expert output added to the rounded sum, or nullptr
};
void launch_combine(const CombineArgs &a, hipStream_t s);

// ---- batched row copies -----------------------------------------------------
// One launch moves the rows of many requests between the callers' buffers and a staging buffer
// (instead of one asynchronous copy per request, ~4 us of host time each).
struct RowCopy {
    const uint8_t *src;
    uint8_t *dst;
    int64_t src_pitch, dst_pitch;   // bytes from one row to the next
    int32_t rows;
    int32_t row_bytes;              // a multiple of 16; src and dst are 16-byte aligned
};
// segs: n entries the device can read (device memory or pinned host memory), unchanged until the
// kernel has run
void launch_rows_copy(const RowCopy *segs, int n, hipStream_t s);

// one wave idling for iters x ~1000 cycles (see pick_side_stream in ek_capi.hip)
void launch_idle(int iters, hipStream_t s);

// ---- weight ingestion -------------------------------------------------------
// src [N, K] row-major of src_dtype (ek_dtype numbering) -> chunked layout at
// dst, matrix m of an nmat-group.  dst_dtype: 0 bf16, 1 f16, 3 int8.  block_scale (16-bit
// destinations only, may be nullptr): [ceil(N/128), ceil(K/128)] factors of scale_dtype.
void launch_tile_weights(const void *src, int src_dtype, int64_t N, int64_t K, uint8_t *dst,
                         int dst_dtype, int m, int nmat, const void *block_scale, int scale_dtype,
                         hipStream_t s);
void launch_scales_to_f32(const void *src, int src_dtype, int64_t n, float *dst, hipStream_t s);

}  // namespace ek
