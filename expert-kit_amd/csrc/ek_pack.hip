// Routing / pack kernels: (token, slot) -> per-expert contiguous segments.
//
// Reproduces, as a stable counting sort, the grouping that
// NaiveExecutor::break_down_to_egress builds with per-expert push lists
// (ek-computation/src/controller/executor.rs:283-304): within an expert's
// segment the pairs keep ascending flat index t*K + k.
//
// Three launches, all integer work, all HBM/LDS bound:
//   pack_hist : one LDS histogram per 4096-pair chunk
//   pack_scan : per-expert exclusive scan over chunks, then a wavefront
//               prefix scan over experts -> counts, offsets, and the FFN
//               kernels' work lists
//   pack_rank : stable rank of every pair inside its chunk by wave-level
//               match (ballots over the id bits) -> perm, inv_perm, row_token
// (calls of at most 4096 pairs run all of it in one workgroup, pack_fused)
// plus a coalesced row gather (assemble_seq_tensors, executor.rs:112-133).
#include "ek_internal.h"

namespace ek {

__global__ __launch_bounds__(kPackThreads) void pack_hist_kernel(PackArgs a)
{
    __shared__ int32_t hist[kMaxExperts];
    for (int i = threadIdx.x; i < a.E; i += kPackThreads) hist[i] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kPackChunk;
    const int64_t end = min(base + (int64_t)kPackChunk, a.P);
    // (ids out of range are left out; the scan kernel sees that the counts do not add up to P)
    for (int64_t p = base + threadIdx.x; p < end; p += kPackThreads) {
        const int32_t id = a.ids[p];
        if ((uint32_t)id < (uint32_t)a.E) atomicAdd(&hist[id], 1);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < a.E; i += kPackThreads)
        a.block_hist[(int64_t)blockIdx.x * a.E + i] = hist[i];
}

// Exclusive prefix sum of one int per thread over a 1024-thread workgroup:
// shuffles inside each wavefront, then the 16 wave totals through LDS.
// Returns the exclusive prefix; *total receives the workgroup sum.
__device__ __forceinline__ int32_t block_exclusive_scan(int32_t v, int32_t *wave_tot, int32_t *total)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int32_t incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int32_t up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
    }
    __syncthreads();   // wave_tot may still be read from a previous scan
    if (lane == 63) wave_tot[wave] = incl;
    __syncthreads();
    int32_t base = 0, sum = 0;
    for (int w = 0; w < 16; ++w) {
        const int32_t t = wave_tot[w];
        if (w < wave) base += t;
        sum += t;
    }
    *total = sum;
    return base + incl - v;
}

// The same for five ints per thread at once (one pair of barriers instead of five): the offsets
// and the four work lists' positions of the one-workgroup pack.  wave_tot: [16][5].
__device__ __forceinline__ void block_exclusive_scan5(const int32_t (&v)[5], int32_t (*wave_tot)[5],
                                                      int32_t (&excl)[5], int32_t (&total)[5])
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int32_t incl[5];
#pragma unroll
    for (int i = 0; i < 5; ++i) incl[i] = v[i];
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
#pragma unroll
        for (int i = 0; i < 5; ++i) {
            const int32_t up = __shfl_up(incl[i], d, 64);
            if (lane >= d) incl[i] += up;
        }
    }
    __syncthreads();   // wave_tot may still be read from a previous scan
    if (lane == 63) {
#pragma unroll
        for (int i = 0; i < 5; ++i) wave_tot[wave][i] = incl[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 5; ++i) {
        int32_t base = 0, sum = 0;
        for (int w = 0; w < 16; ++w) {
            const int32_t t = wave_tot[w][i];
            if (w < wave) base += t;
            sum += t;
        }
        total[i] = sum;
        excl[i] = base + incl[i] - v[i];
    }
}

// How one segment of n rows is cut into work items (see WorkLists).
struct SegmentCut {
    int32_t n128, n64, n32, ns;
};
__device__ __forceinline__ SegmentCut cut_segment(int32_t n)
{
    SegmentCut c;
    const int32_t r = n & 127;
    c.n128 = (n >> 7) + (r > 64);
    c.n64 = r > 32 && r <= 64;
    c.n32 = r > 16 && r <= 32;
    c.ns = r > 0 && r <= 16;
    return c;
}
__device__ __forceinline__ void emit_items(const WorkLists &l, int32_t e, int32_t seg0, int32_t n,
                                           int32_t p128, int32_t p64, int32_t p32, int32_t ps)
{
    const int32_t full = n >> 7, r = n & 127;
    for (int32_t t = 0; t < full; ++t) l.items[kListT128][p128 + t] = WorkItem{e, seg0 + t * 128, 128, 0};
    const WorkItem rem{e, seg0 + full * 128, r, 0};
    if (r > 64) l.items[kListT128][p128 + full] = rem;
    else if (r > 32) l.items[kListT64][p64] = rem;
    else if (r > 16) l.items[kListT32][p32] = rem;
    else if (r > 0) l.items[kListStream][ps] = rem;
}

// One workgroup of 1024 threads; thread e owns expert e.
__global__ __launch_bounds__(1024) void pack_scan_kernel(PackArgs a)
{
    __shared__ int32_t wave_tot[16];
    const int e = threadIdx.x;
    int32_t total = 0;
    if (e < a.E) {
        // exclusive prefix over chunks, 16 chunks' counts in flight at a time (one dependent load
        // per chunk made this kernel's time: 10 us at 9 chunks)
        for (int b0 = 0; b0 < a.nblocks; b0 += 16) {
            int32_t v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u)
                v[u] = b0 + u < a.nblocks ? a.block_hist[(int64_t)(b0 + u) * a.E + e] : 0;
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                if (b0 + u < a.nblocks) a.block_hist[(int64_t)(b0 + u) * a.E + e] = total;
                total += v[u];
            }
        }
        a.counts[e] = total;
        if (a.activation) a.activation[e] += (uint64_t)total;
    }
    const bool unloaded = e < a.E && total > 0 && a.slabs != nullptr && a.slabs[e].upgate == nullptr;
    const int any_unloaded = __syncthreads_or(unloaded);
    int32_t sum;
    const int32_t off = block_exclusive_scan(total, wave_tot, &sum);
    if (e < a.E) a.offsets[e] = off;
    if (e == 0) {
        a.offsets[a.E] = sum;
        // the error word is written, not accumulated: every pair with an id in range was counted once
        a.err[0] = ((int64_t)sum != a.P ? 1 : 0) | (any_unloaded ? 2 : 0);
    }
    if (a.lists.count == nullptr) return;
    const SegmentCut c = cut_segment(total);
    int32_t s128, s64, s32, ss;
    const int32_t p128 = block_exclusive_scan(c.n128, wave_tot, &s128);
    const int32_t p64 = block_exclusive_scan(c.n64, wave_tot, &s64);
    const int32_t p32 = block_exclusive_scan(c.n32, wave_tot, &s32);
    const int32_t ps = block_exclusive_scan(c.ns, wave_tot, &ss);
    if (e < a.E && total > 0) emit_items(a.lists, e, off, total, p128, p64, p32, ps);
    if (e == 0) {
        a.lists.count[kListT128] = s128;
        a.lists.count[kListT64] = s64;
        a.lists.count[kListT32] = s32;
        a.lists.count[kListStream] = ss;
        if (a.tile_items_host) *a.tile_items_host = s128 + s64 + s32;
    }
}

// Work lists that hold one segment and nothing else: rows row0 .. row0+n-1 of expert e.
// mode 0: the usual cut; 1: 16-row streaming items; 2: streaming items of up to kWideRows rows.
// row_token, if given, maps the segment's rows to tokens 0 .. n-1.
__global__ __launch_bounds__(256) void segment_lists_kernel(WorkLists l, int32_t e, int32_t row0, int32_t n,
                                                            int32_t *row_token, int32_t mode)
{
    if (row_token)
        for (int32_t t = threadIdx.x; t < n; t += 256) row_token[row0 + t] = t;
    if (mode) {
        const int32_t per = mode == 2 ? kWideRows : 16, items = (n + per - 1) / per;
        for (int32_t t = threadIdx.x; t < items; t += 256)
            l.items[kListStream][t] = WorkItem{e, row0 + t * per, min(per, n - t * per), 0};
        if (threadIdx.x == 0) {
            l.count[kListT128] = l.count[kListT64] = l.count[kListT32] = 0;
            l.count[kListStream] = items;
        }
        return;
    }
    const SegmentCut c = cut_segment(n);
    const int32_t full = n >> 7;
    for (int32_t t = threadIdx.x; t < full; t += 256) l.items[kListT128][t] = WorkItem{e, row0 + t * 128, 128, 0};
    if (threadIdx.x == 0) {
        if (n & 127) emit_items(l, e, row0 + full * 128, n & 127, full, 0, 0, 0);    // the remainder, into its class
        l.count[kListT128] = c.n128;
        l.count[kListT64] = c.n64;
        l.count[kListT32] = c.n32;
        l.count[kListStream] = c.ns;
    }
}

__global__ __launch_bounds__(256) void append_segment_kernel(WorkLists l, int32_t e, int32_t row0, int32_t n,
                                                             int32_t *row_token, int32_t as_stream)
{
    const int32_t p128 = l.count[kListT128], p64 = l.count[kListT64], p32 = l.count[kListT32],
                  ps = l.count[kListStream];
    __syncthreads();   // every thread has read the old lengths before thread 0 replaces them
    if (as_stream) {
        // a decode-sized segment: as one tile per 128 rows it would run on a handful of CUs for
        // the length of the whole contraction; as streaming items it spreads over the chip.
        // as_stream = 1: 16-row items appended to the list; 2: items of up to kWideRows rows
        // that become the whole list (a list of their own, for a launch of their own)
        const int32_t per = as_stream == 2 ? kWideRows : 16, at = as_stream == 2 ? 0 : ps;
        const int32_t items = (n + per - 1) / per;
        for (int32_t t = threadIdx.x; t < items; t += 256)
            l.items[kListStream][at + t] = WorkItem{e, row0 + t * per, min(per, n - t * per), 0};
        for (int32_t t = threadIdx.x; t < n; t += 256) row_token[row0 + t] = t;
        if (threadIdx.x == 0) l.count[kListStream] = at + items;
        return;
    }
    const SegmentCut c = cut_segment(n);
    const int32_t full = n >> 7, r = n & 127;
    for (int32_t t = threadIdx.x; t < full; t += 256) l.items[kListT128][p128 + t] = WorkItem{e, row0 + t * 128, 128, 0};
    for (int32_t t = threadIdx.x; t < n; t += 256) row_token[row0 + t] = t;
    if (threadIdx.x == 0) {
        const WorkItem rem{e, row0 + full * 128, r, 0};
        if (r > 64) l.items[kListT128][p128 + full] = rem;
        else if (r > 32) l.items[kListT64][p64] = rem;
        else if (r > 16) l.items[kListT32][p32] = rem;
        else if (r > 0) l.items[kListStream][ps] = rem;
        l.count[kListT128] = p128 + c.n128;
        l.count[kListT64] = p64 + c.n64;
        l.count[kListT32] = p32 + c.n32;
        l.count[kListStream] = ps + c.ns;
    }
}

void launch_append_segment(const WorkLists &lists, int32_t expert, int32_t row0, int32_t n, int32_t *row_token,
                           int as_stream, hipStream_t s)
{
    hipLaunchKernelGGL(append_segment_kernel, dim3(1), dim3(256), 0, s, lists, expert, row0, n, row_token,
                       as_stream);
}

void launch_single_lists(const WorkLists &lists, int32_t expert, int32_t n, bool wide, hipStream_t s)
{
    hipLaunchKernelGGL(segment_lists_kernel, dim3(1), dim3(256), 0, s, lists, expert, 0, n, (int32_t *)nullptr, wide ? 2 : 0);
}

void launch_segment_lists(const WorkLists &lists, int32_t expert, int32_t row0, int32_t n, int32_t *row_token, int mode,
                          hipStream_t s)
{
    hipLaunchKernelGGL(segment_lists_kernel, dim3(1), dim3(256), 0, s, lists, expert, row0, n, row_token, mode);
}

__global__ __launch_bounds__(kPackThreads) void pack_rank_kernel(PackArgs a, int nbits)
{
    constexpr int kWaves = kPackThreads / 64;
    constexpr int kSub = kPackChunk / kWaves;   // pairs per wave, consecutive
    __shared__ int32_t wbase[kWaves][kMaxExperts];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < kWaves * kMaxExperts; i += kPackThreads) (&wbase[0][0])[i] = 0;
    __syncthreads();
    const int64_t start = (int64_t)blockIdx.x * kPackChunk + (int64_t)wave * kSub;
    for (int it = 0; it < kSub / 64; ++it) {
        const int64_t p = start + it * 64 + lane;
        if (p < a.P) {
            const int32_t id = a.ids[p];
            if ((uint32_t)id < (uint32_t)a.E) atomicAdd(&wbase[wave][id], 1);
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < a.E; e += kPackThreads) {
        int32_t run = a.offsets[e] + a.block_hist[(int64_t)blockIdx.x * a.E + e];
        for (int w = 0; w < kWaves; ++w) {
            const int32_t t = wbase[w][e];
            wbase[w][e] = run;
            run += t;
        }
    }
    __syncthreads();
    // Each wave walks its own consecutive pairs 64 at a time; lanes holding
    // the same expert id find each other with one ballot per id bit, so the
    // rank inside the group is the number of lower lanes in the group.
    for (int it = 0; it < kSub / 64; ++it) {
        const int64_t p = start + it * 64 + lane;
        int32_t id = 0;
        bool valid = false;
        if (p < a.P) {
            id = a.ids[p];
            valid = (uint32_t)id < (uint32_t)a.E;
            if (!valid) a.inv_perm[p] = -1;
        }
        uint64_t m = __ballot(valid);
        for (int b = 0; b < nbits; ++b) {
            const bool bit = (id >> b) & 1;
            const uint64_t bb = __ballot(bit);
            m &= bit ? bb : ~bb;
        }
        if (valid) {
            const int32_t rank = __popcll(m & ((1ull << lane) - 1ull));
            const int32_t pos = wbase[wave][id] + rank;
            const bool leader = (m >> lane) == 1ull;   // highest lane of the group
            if (leader) wbase[wave][id] = pos + 1;
            a.perm[pos] = (int32_t)p;
            a.inv_perm[p] = pos;
            a.row_token[pos] = (int32_t)(p / a.K);
        }
    }
}

// Whole pack step in one workgroup, for calls of at most kPackFusedMax pairs
// (decode batches): histogram, scans, work lists and stable ranks without
// leaving LDS, and no separate clear of the error word.  16 wavefronts; wave w
// owns the consecutive pairs [w*sub, (w+1)*sub) and keeps them in registers.
constexpr int kPackFusedMax = 4096;
__global__ __launch_bounds__(1024) void pack_fused_kernel(PackArgs a, int nbits)
{
    extern __shared__ int32_t lds[];          // wbase[16][E], then wave_tot5[16][5], err
    int32_t (*wave_tot5)[5] = (int32_t (*)[5])(lds + 16 * a.E);
    int32_t *lerr = lds + 16 * a.E + 80;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int kIter = kPackFusedMax / 1024;   // 64-pair groups per wave
    for (int i = threadIdx.x; i < 16 * a.E; i += 1024) lds[i] = 0;
    if (threadIdx.x == 0) *lerr = 0;
    const int64_t start = (int64_t)wave * (kIter * 64);
    int32_t id[kIter];
    bool bad = false;
#pragma unroll
    for (int it = 0; it < kIter; ++it) {
        const int64_t p = start + it * 64 + lane;
        id[it] = p < a.P ? a.ids[p] : -1;
        if (p < a.P && (uint32_t)id[it] >= (uint32_t)a.E) { bad = true; id[it] = -1; }
    }
    __syncthreads();
    if (bad) atomicOr(lerr, 1);
#pragma unroll
    for (int it = 0; it < kIter; ++it)
        if (id[it] >= 0) atomicAdd(&lds[wave * a.E + id[it]], 1);
    __syncthreads();
    const int e = threadIdx.x;
    int32_t total = 0;
    if (e < a.E) {
        for (int w = 0; w < 16; ++w) total += lds[w * a.E + e];
        a.counts[e] = total;
        if (a.activation) a.activation[e] += (uint64_t)total;
        if (total > 0 && a.slabs != nullptr && a.slabs[e].upgate == nullptr) atomicOr(lerr, 2);
    }
    // offsets and the four lists' positions in one scan
    const SegmentCut c = cut_segment(total);
    const int32_t v5[5] = {total, c.n128, c.n64, c.n32, c.ns};
    int32_t ex[5], tot5[5];
    block_exclusive_scan5(v5, wave_tot5, ex, tot5);
    const int32_t off = ex[0];
    if (e < a.E) {
        a.offsets[e] = off;
        int32_t run = off;
        for (int w = 0; w < 16; ++w) {
            const int32_t t = lds[w * a.E + e];
            lds[w * a.E + e] = run;
            run += t;
        }
    }
    if (e == 0) a.offsets[a.E] = tot5[0];
    if (a.lists.count != nullptr) {
        if (e < a.E && total > 0) emit_items(a.lists, e, off, total, ex[1], ex[2], ex[3], ex[4]);
        if (e == 0) {
            a.lists.count[kListT128] = tot5[1];
            a.lists.count[kListT64] = tot5[2];
            a.lists.count[kListT32] = tot5[3];
            a.lists.count[kListStream] = tot5[4];
            if (a.tile_items_host) *a.tile_items_host = tot5[1] + tot5[2] + tot5[3];
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) a.err[0] = *lerr;
#pragma unroll
    for (int it = 0; it < kIter; ++it) {
        const int64_t p = start + it * 64 + lane;
        const bool valid = id[it] >= 0;
        if (p < a.P && !valid) a.inv_perm[p] = -1;
        uint64_t m = __ballot(valid);
        for (int b = 0; b < nbits; ++b) {
            const bool bit = (id[it] >> b) & 1;
            const uint64_t bb = __ballot(bit);
            m &= bit ? bb : ~bb;
        }
        if (valid) {
            const int32_t rank = __popcll(m & ((1ull << lane) - 1ull));
            const int32_t pos = lds[wave * a.E + id[it]] + rank;
            const bool leader = (m >> lane) == 1ull;
            if (leader) lds[wave * a.E + id[it]] = pos + 1;
            a.perm[pos] = (int32_t)p;
            a.inv_perm[p] = pos;
            a.row_token[pos] = (int32_t)(p / a.K);
        }
    }
}

void launch_pack(const PackArgs &a, hipStream_t s)
{
    if (a.P <= 0) {
        // offsets and counts must still be defined (all zero)
        PackArgs z = a;
        z.nblocks = 0;
        z.P = 0;
        hipLaunchKernelGGL(pack_scan_kernel, dim3(1), dim3(1024), 0, s, z);
        return;
    }
    int nbits = 0;
    while ((1 << nbits) < a.E) ++nbits;
    // the one-workgroup form keeps 16 histograms in dynamic LDS: up to 64 KiB of it (E <= 1018).
    // (One workgroup for longer calls was measured and is slower, 85 against 43 us at 65536 pairs:
    // a single CU's memory pipeline then takes every scattered store of perm and row_token.)
    const size_t lds_bytes = sizeof(int32_t) * (16 * (size_t)a.E + 96);
    if (a.P <= kPackFusedMax && lds_bytes <= 65536) {
        hipLaunchKernelGGL(pack_fused_kernel, dim3(1), dim3(1024), lds_bytes, s, a, nbits);
        return;
    }
    hipLaunchKernelGGL(pack_hist_kernel, dim3(a.nblocks), dim3(kPackThreads), 0, s, a);
    hipLaunchKernelGGL(pack_scan_kernel, dim3(1), dim3(1024), 0, s, a);
    hipLaunchKernelGGL(pack_rank_kernel, dim3(a.nblocks), dim3(kPackThreads), 0, s, a, nbits);
}

// Xp[j, :] = x[row_token[j], :], 16 bytes per lane, one workgroup per row slice.
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint4 *x, const int32_t *row_token,
                                                         int64_t P, int64_t row_vec, uint4 *xp)
{
    const int64_t j = blockIdx.y;
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (j >= P || c >= row_vec) return;
    xp[j * row_vec + c] = x[(int64_t)row_token[j] * row_vec + c];
}

void launch_gather(const void *x, const int32_t *row_token, int64_t P, int64_t row_bytes, void *xp,
                   hipStream_t s)
{
    if (P <= 0) return;
    const int64_t row_vec = row_bytes / 16;
    // grid.y is limited to 65535: walk P in slabs
    for (int64_t j0 = 0; j0 < P; j0 += 65535) {
        const int64_t nj = (P - j0) < 65535 ? (P - j0) : 65535;
        hipLaunchKernelGGL(gather_rows_kernel, dim3((row_vec + 255) / 256, nj), dim3(256), 0, s,
                           (const uint4 *)x, row_token + j0, nj, row_vec,
                           (uint4 *)xp + j0 * row_vec);
    }
}

}  // namespace ek
