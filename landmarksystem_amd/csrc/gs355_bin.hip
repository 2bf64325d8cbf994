// Tile-bucketed sort for gfx950: the fast equivalent of "duplicate keys ->
// radix sort -> tile ranges" of the rasterizer behind
// GaussianRasterizer.forward (benchmarks/nerf/origin_gs/gs_model.py:211-220).
//
// The 64-bit key is (tile_id << 32 | depth bits).  Its high word is known when
// a pair is generated, so the most significant digit is resolved by counting:
// pairs are counted per tile, an exclusive scan of the counts gives every tile
// its slot range (these ARE the per-tile ranges), and pairs are scattered into
// their tile's bucket (in one level, or through coarse bins of 16 tiles when
// the frame holds many pairs).  What remains is an independent sort of each
// bucket by its low word, done by one workgroup per tile entirely in LDS (up
// to 10240 pairs in the 160 KB of a CU; larger buckets run radix passes
// through global memory).  Bucket order after the scatter is arbitrary, so
// pairs are ordered by (depth bits, Gaussian index): exactly the order a
// stable sort of the emission-ordered keys produces.
//
// No workgroup waits on another; persistent loops run over fixed lists, or
// take entries from a counter until it passes the list's length.
#include <atomic>

#include "gs355_internal.h"

namespace gs355 {

namespace {

// splats touching more tiles than this are queued and expanded by a wavefront each (8 and 16 measured slower, 64 and
// 128 the same)
constexpr int kInlineTiles = 32;
constexpr int kBinItems = 4;      // Gaussians per thread and round of the binning walk

// ---------------------------------------------------------------------------
// Counting.  Workgroup c owns Gaussians [c * per_group, (c+1) * per_group) and a private array of counters in LDS.
//   up to kBinMaxTiles tiles:  one counter per tile; matrix[c][t] = pairs of this slice that fall in tile t.  No
//                              global atomic is issued anywhere on this path.
//   more tiles (kWide):        one counter per coarse bin of kCoarseTiles consecutive tiles, matrix[c][b]; the
//                              tiles' own totals are counted later, from the pairs of each bin (fine_count_kernel).
// A thread walks the tile rectangle of its own Gaussian; rectangles of more than kInlineTiles tiles are queued and
// walked by the wavefronts, one rectangle each at a time.
template <bool kWide>
__global__ __launch_bounds__(kBinThreads) void tile_count_kernel(FrameArgs f, int32_t P, int per_group,
                                                                 const uint64_t* __restrict__ rects,
                                                                 uint32_t* __restrict__ matrix,
                                                                 uint32_t* __restrict__ group_visible)
{
    extern __shared__ uint32_t s_count[];  // [tiles], or [coarse bins] when kWide
    __shared__ uint32_t s_queue[kBinItems * kBinThreads];
    __shared__ uint32_t s_nqueue, s_visible;

    if (f.p_device) {  // the slices follow the device-side count: as many Gaussians per workgroup as on the host side
        P = effective_count(f, P);
        per_group = (P + (int)gridDim.x - 1) / (int)gridDim.x;
        per_group = max(kBinThreads, (per_group + kBinThreads - 1) / kBinThreads * kBinThreads);
    }
    const int T = f.grid_x * f.grid_y;
    const int counters = kWide ? (T + kCoarseTiles - 1) >> kCoarseShift : T;
    const int tid = threadIdx.x, c = blockIdx.x;
    for (int t = tid; t < counters; t += kBinThreads) s_count[t] = 0u;
    if (tid == 0) s_visible = 0;
    const int g_begin = min(P, c * per_group);
    const int g_end = min(P, g_begin + per_group);
    uint32_t visible = 0;
    auto add = [&](int t) { atomicAdd(&s_count[kWide ? t >> kCoarseShift : t], 1u); };

    // a thread's Gaussians of a round: their rectangles are requested together, and those of the next round before
    // this round's are walked (a slice is a dozen rounds or more, each otherwise a memory latency plus its walk)
    uint64_t ahead[kBinItems];
#pragma unroll
    for (int u = 0; u < kBinItems; ++u) ahead[u] = g_begin < g_end ? rects[min(g_begin + u * kBinThreads + tid, g_end - 1)] : 0ull;
    for (int base = g_begin; base < g_end; base += kBinItems * kBinThreads) {
        if (tid == 0) s_nqueue = 0;
        __syncthreads();
        uint64_t rr[kBinItems];
#pragma unroll
        for (int u = 0; u < kBinItems; ++u) rr[u] = ahead[u];
        if (base + kBinItems * kBinThreads < g_end) {  // uniform
#pragma unroll
            for (int u = 0; u < kBinItems; ++u)
                ahead[u] = rects[min(base + (kBinItems + u) * kBinThreads + tid, g_end - 1)];
        }
#pragma unroll
        for (int u = 0; u < kBinItems; ++u) {
            const int i = base + u * kBinThreads + tid;
            if (i < g_end) {
                const uint64_t r = rr[u];
                const int x0 = (int)(r & 0xFFFF), y0 = (int)((r >> 16) & 0xFFFF), x1 = (int)((r >> 32) & 0xFFFF),
                          y1 = (int)(r >> 48);
                const int area = (x1 - x0) * (y1 - y0);
                if (area > 0) {
                    ++visible;
                    if (area > kInlineTiles) {
                        s_queue[atomicAdd(&s_nqueue, 1u)] = (uint32_t)i;
                    } else if (kWide) {  // a rectangle row: one request per coarse bin it crosses
                        for (int ty = y0; ty < y1; ++ty) {
                            int ta = ty * f.grid_x + x0;
                            const int tb = ty * f.grid_x + x1;
                            while (ta < tb) {
                                const int stop = min(tb, ((ta >> kCoarseShift) + 1) << kCoarseShift);
                                atomicAdd(&s_count[ta >> kCoarseShift], (uint32_t)(stop - ta));
                                ta = stop;
                            }
                        }
                    } else {
                        for (int ty = y0; ty < y1; ++ty)
                            for (int tx = x0; tx < x1; ++tx) add(ty * f.grid_x + tx);
                    }
                }
            }
        }
        __syncthreads();
        // large rectangles: one per wavefront at a time, 64 tiles per step (the sixteen wavefronts work on sixteen
        // rectangles side by side; the whole workgroup on one rectangle left most of its threads idle)
        const uint32_t nq = s_nqueue;
        for (uint32_t k = (uint32_t)tid >> 6; k < nq; k += kBinThreads / 64) {
            const uint64_t r = rects[s_queue[k]];
            const int x0 = (int)(r & 0xFFFF), y0 = (int)((r >> 16) & 0xFFFF), x1 = (int)((r >> 32) & 0xFFFF),
                      y1 = (int)(r >> 48);
            const int w = x1 - x0, area = w * (y1 - y0);
            for (int e = tid & 63; e < area; e += 64) add((y0 + e / w) * f.grid_x + x0 + e % w);
        }
        __syncthreads();
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) visible += __shfl_down(visible, d, 64);
    if ((tid & 63) == 0 && visible) atomicAdd(&s_visible, visible);
    __syncthreads();
    uint32_t* __restrict__ row = matrix + (size_t)c * counters;
    for (int t = tid; t < counters; t += kBinThreads) row[t] = s_count[t];
    if (tid == 0) group_visible[c] = s_visible;
}

// ---------------------------------------------------------------------------
// Scatter.  Writing every pair straight into its tile's bucket spreads a
// workgroup's stores over thousands of buckets: each 8-byte store then costs a
// whole 32-byte sector of memory traffic.  Frames of many pairs therefore take
// two levels: the pairs go first into coarse bins of kCoarseTiles consecutive
// tiles (a workgroup keeps a few hundred write streams going, which the L2
// merges into full lines), then workgroups read each bin back (contiguous)
// and spread it over the bin's 16 buckets in line-sized runs.  The coarse bin of
// tiles [16 b, 16 b + 16) is the concatenation of their buckets, so the same
// slot arithmetic serves both levels: a slice's pairs of bin b start at
// tile_base[16 b] plus the sum of the slice prefixes of the bin's tiles.  A
// coarse pair carries the tile's position within its bin in the low four bits
// of the index word.  The two launches of the second level cost some 40 us
// whatever the frame holds, so frames below kTwoLevelMinKeys pairs scatter in
// one level; the key count is only known on the device, so both variants are
// launched and each returns at once when the other one applies.
constexpr uint32_t kTwoLevelMinKeys = 6u << 20;

// The walk of the counting kernel with one cursor per column: a coarse bin (kShift = kCoarseShift) or a tile
// (kShift = 0, straight into the buckets).  The tiles of one rectangle row are consecutive, so a row takes one slot
// request per coarse bin it crosses instead of one per tile.  Runs only when min_keys <= pairs of the frame <
// max_keys.  (Two variants were measured slower: staging each round in LDS ordered by bin, so that consecutive
// lanes store consecutive pairs, walks the rectangles twice; walking a thread's rectangles side by side to keep
// several slot requests in flight costs more in bookkeeping than the latency it hides.)
template <int kShift, bool kWide>
__global__ __launch_bounds__(kBinThreads) void scatter_kernel(FrameArgs f, int32_t P, int per_group,
                                                              const uint64_t* __restrict__ rects,
                                                              const uint32_t* __restrict__ depth_bits,
                                                              const gs355_header* __restrict__ header,
                                                              uint32_t min_keys, uint32_t max_keys,
                                                              const uint32_t* __restrict__ matrix,
                                                              const uint32_t* __restrict__ bases,
                                                              uint64_t* __restrict__ dst)
{
    static_assert(!kWide || kShift > 0, "beyond kBinMaxTiles tiles only coarse bins fit in LDS");
    extern __shared__ uint32_t s_bin[];  // [columns] next free slot of this slice in each column
    __shared__ uint32_t s_queue[kBinItems * kBinThreads];
    __shared__ uint32_t s_nqueue;

    if (header->overflow || header->num_keys < min_keys || header->num_keys >= max_keys) return;
    if (f.p_device) {
        P = effective_count(f, P);
        per_group = (P + (int)gridDim.x - 1) / (int)gridDim.x;
        per_group = max(kBinThreads, (per_group + kBinThreads - 1) / kBinThreads * kBinThreads);
    }
    constexpr int kSpan = 1 << kShift;
    const int T = f.grid_x * f.grid_y, bins = (T + kSpan - 1) >> kShift;
    const int tid = threadIdx.x, c = blockIdx.x, wave = tid >> 6, lane = tid & 63;
    // a column's first slot for this slice: the column's base (kWide: bases[b]; else the base of its first tile)
    // plus what the earlier slices put into it (the matrix holds that per bin when kWide, else per tile)
    const uint32_t* __restrict__ row = matrix + (size_t)c * (kWide ? bins : T);
    for (int b = tid; b < bins; b += kBinThreads)
        s_bin[b] = kWide ? bases[b] + row[b] : kShift ? bases[b << kShift] : bases[b] + row[b];
    if (!kWide && kShift) {
        __syncthreads();
        for (int t = tid; t < T; t += kBinThreads) {
            const uint32_t before = row[t];
            if (before) atomicAdd(&s_bin[t >> kShift], before);
        }
    }
    const int g_begin = min(P, c * per_group);
    const int g_end = min(P, g_begin + per_group);
    // the tiles [ta, tb) of one rectangle row, cut where they cross into the next column
    auto emit_row = [&](int ta, int tb, uint64_t payload) {
        while (ta < tb) {
            const int stop = min(tb, ((ta >> kShift) + 1) << kShift);
            uint32_t slot = atomicAdd(&s_bin[ta >> kShift], (uint32_t)(stop - ta));
            // the segment's slots are consecutive: two pairs per 16-byte store where the slot is even (every store
            // is a 64-byte request on the way to the L2, however few bytes it carries)
            if ((slot & 1u) && ta < stop) dst[slot++] = payload | (uint64_t)(ta++ & (kSpan - 1));
            for (; ta + 1 < stop; ta += 2, slot += 2) {
                ulonglong2 two;
                two.x = payload | (uint64_t)(ta & (kSpan - 1));
                two.y = payload | (uint64_t)((ta + 1) & (kSpan - 1));
                *reinterpret_cast<ulonglong2*>(dst + slot) = two;
            }
            if (ta < stop) dst[slot] = payload | (uint64_t)(ta++ & (kSpan - 1));
        }
    };

    for (int first = g_begin; first < g_end; first += kBinItems * kBinThreads) {
        if (tid == 0) s_nqueue = 0;
        __syncthreads();
        uint64_t rr[kBinItems];
        uint32_t dd[kBinItems];
#pragma unroll
        for (int u = 0; u < kBinItems; ++u) {
            const int i = min(first + u * kBinThreads + tid, g_end - 1);
            rr[u] = rects[i];
            dd[u] = depth_bits[i];
        }
#pragma unroll
        for (int u = 0; u < kBinItems; ++u) {
            const int i = first + u * kBinThreads + tid;
            if (i < g_end) {
                const uint64_t r = rr[u];
                const int x0 = (int)(r & 0xFFFF), y0 = (int)((r >> 16) & 0xFFFF), x1 = (int)((r >> 32) & 0xFFFF),
                          y1 = (int)(r >> 48);
                const int area = (x1 - x0) * (y1 - y0);
                if (area > kInlineTiles) {
                    s_queue[atomicAdd(&s_nqueue, 1u)] = (uint32_t)i;
                } else if (area > 0) {
                    const uint64_t payload = ((uint64_t)dd[u] << 32) | ((uint64_t)(uint32_t)i << kShift);
                    for (int ty = y0; ty < y1; ++ty) emit_row(ty * f.grid_x + x0, ty * f.grid_x + x1, payload);
                }
            }
        }
        __syncthreads();
        // large rectangles: one per wavefront at a time, 64 tiles per step
        const uint32_t nq = s_nqueue;
        for (uint32_t k = wave; k < nq; k += kBinThreads / 64) {
            const uint32_t gi = s_queue[k];
            const uint64_t r = rects[gi];
            const int x0 = (int)(r & 0xFFFF), y0 = (int)((r >> 16) & 0xFFFF), x1 = (int)((r >> 32) & 0xFFFF),
                      y1 = (int)(r >> 48);
            const int w = x1 - x0, area = w * (y1 - y0);
            const uint64_t payload = ((uint64_t)depth_bits[gi] << 32) | ((uint64_t)gi << kShift);
            for (int e = lane; e < area; e += 64) {
                const int t = (y0 + e / w) * f.grid_x + x0 + e % w;
                const uint32_t slot = atomicAdd(&s_bin[t >> kShift], 1u);
                dst[slot] = payload | (uint64_t)(t & (kSpan - 1));
            }
        }
        __syncthreads();
    }
}

// Second level: the pairs of a coarse bin (contiguous) go to the buckets of the bin's tiles, a chunk of kFineChunk pairs
// at a time.  Chunks never cross a bin; chunk_base[b] = chunks of the bins before b, chunk_base[bins] = all of them
// (tile_publish_kernel).  The kFineGrid workgroups take equal, contiguous runs of chunks, so every workgroup has work
// however the pairs are spread over the bins, and a bin of many pairs is shared by many workgroups.  A chunk is split
// by tile inside LDS first (wave-level ranking by the four tile bits, a scan over the per-wave counts), the
// workgroup reserves a run of slots per bucket with one global atomic each, and consecutive lanes then store
// consecutive pairs of one bucket: full-line writes instead of one memory transaction per pair.  Order inside a
// bucket is arbitrary, as the sort expects.
constexpr int kFineThreads = 256;
constexpr int kFineWaves = kFineThreads / 64;
constexpr int kFineItems = 8;                             // pairs per thread and chunk
constexpr int kFineChunk = kFineThreads * kFineItems;  // 2048 pairs = 16 KB of LDS
constexpr int kFineGrid = 8192;                          // a chunk per workgroup at 6M Gaussians / 1080p, a few each at 4K

// A workgroup's run of chunks.  next() gives the following chunk's bin, first pair and pair count.
struct ChunkRun {
    const uint32_t* chunk_base;
    uint32_t c, c_end;  // next chunk, end of the run
    int b, bins;        // bin of chunk c (once begun)

    __device__ ChunkRun(const uint32_t* __restrict__ base, int n_bins) : chunk_base(base), b(0), bins(n_bins)
    {
        const uint32_t total = base[n_bins], per = (total + gridDim.x - 1) / gridDim.x;
        c = min(total, blockIdx.x * per);
        c_end = min(total, c + per);
        if (c < c_end) {  // the bin that holds chunk c: the last one whose base is <= c
            int lo = 0, hi = n_bins;  // base[lo] <= c < base[hi]
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (base[mid] <= c) lo = mid;
                else hi = mid;
            }
            b = lo;
        }
    }
    // `first_pair(bin)`: where the bin's pairs start in the coarse buffer
    template <typename First>
    __device__ bool next(First first_pair, uint32_t num_keys, int& bin, uint32_t& j0, uint32_t& n, uint32_t& bin_begin,
                         uint32_t& bin_end)
    {
        if (c >= c_end) return false;
        while (chunk_base[b + 1] <= c) ++b;  // (bins without pairs have no chunks)
        bin = b;
        bin_begin = first_pair(b);
        bin_end = b + 1 < bins ? first_pair(b + 1) : num_keys;
        j0 = bin_begin + (c - chunk_base[b]) * (uint32_t)kFineChunk;
        n = min((uint32_t)kFineChunk, bin_end - j0);
        ++c;
        return true;
    }
};

__global__ __launch_bounds__(kFineThreads) void fine_scatter_kernel(const gs355_header* __restrict__ header,
                                                                    uint32_t min_keys,
                                                                    const uint32_t* __restrict__ tile_base,
                                                                    uint32_t* __restrict__ cursor, int T,
                                                                    const uint32_t* __restrict__ chunk_base,
                                                                    const uint64_t* __restrict__ coarse,
                                                                    uint64_t* __restrict__ buckets)
{
    __shared__ uint64_t s_stage[kFineChunk];
    __shared__ uint32_t s_count[kFineWaves][kCoarseTiles];  // pairs per (wavefront, tile) of the chunk, then their offsets
    __shared__ uint32_t s_start[kCoarseTiles + 1];          // first staged position of each tile's pairs
    __shared__ uint32_t s_slot[kCoarseTiles];               // first reserved slot of each bucket for this chunk
    if (header->overflow || header->num_keys < min_keys) return;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const uint64_t lanes_below = (1ull << lane) - 1ull;
    const uint32_t num_keys = header->num_keys;
    ChunkRun run(chunk_base, (T + kCoarseTiles - 1) >> kCoarseShift);
    int bin;
    uint32_t j0, n, begin, end;
    while (run.next([&](int b) { return tile_base[b << kCoarseShift]; }, num_keys, bin, j0, n, begin, end)) {
        const int t0 = bin << kCoarseShift;
        for (int k = tid; k < kFineWaves * kCoarseTiles; k += kFineThreads) (&s_count[0][0])[k] = 0;
        __syncthreads();
        // a wavefront owns kFineItems x 64 consecutive pairs of the chunk
        uint64_t v[kFineItems];
        uint32_t rank[kFineItems];
#pragma unroll
        for (int u = 0; u < kFineItems; ++u) {
            const uint32_t p = (uint32_t)(wave * kFineItems + u) * 64u + lane;
            v[u] = p < n ? coarse[j0 + p] : 0ull;
        }
#pragma unroll
        for (int u = 0; u < kFineItems; ++u) {
            const uint32_t p = (uint32_t)(wave * kFineItems + u) * 64u + lane;
            const bool valid = p < n;
            const uint32_t d = (uint32_t)v[u] & (kCoarseTiles - 1);
            uint64_t peers = __ballot(valid);
#pragma unroll
            for (int bit = 0; bit < kCoarseShift; ++bit) {
                const bool one = (d >> bit) & 1u;
                const uint64_t m = __ballot(one);
                peers &= one ? m : ~m;
            }
            uint32_t before = 0;
            if (valid) {
                const int leader = __ffsll((unsigned long long)peers) - 1;
                if (lane == leader) before = atomicAdd(&s_count[wave][d], (uint32_t)__popcll(peers));
                before = __shfl(before, leader, 64);
            }
            rank[u] = before + (uint32_t)__popcll(peers & lanes_below);
        }
        __syncthreads();
        if (tid < kCoarseTiles) {  // per tile: its total in the chunk, and the slots it gets in its bucket
            uint32_t total = 0;
#pragma unroll
            for (int w = 0; w < kFineWaves; ++w) {
                const uint32_t c = s_count[w][tid];
                s_count[w][tid] = total;  // pairs of this tile in earlier wavefronts
                total += c;
            }
            s_start[tid + 1] = total;
            s_slot[tid] = total && t0 + tid < T ? atomicAdd(&cursor[t0 + tid], total) : 0u;
        }
        __syncthreads();
        if (tid < 64) {  // exclusive scan of the tiles' totals (at most 64 tiles per bin)
            const uint32_t c = tid < kCoarseTiles ? s_start[tid + 1] : 0u;
            uint32_t inc = c;
#pragma unroll
            for (int d = 1; d < kCoarseTiles; d <<= 1) {
                const uint32_t up = __shfl_up(inc, d, 64);
                if (lane >= d) inc += up;
            }
            if (tid < kCoarseTiles) s_start[tid] = inc - c;  // (the reads above are this wavefront's own, already done)
            if (tid == kCoarseTiles - 1) s_start[kCoarseTiles] = inc;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kFineItems; ++u) {
            const uint32_t p = (uint32_t)(wave * kFineItems + u) * 64u + lane;
            if (p < n) {
                const uint32_t d = (uint32_t)v[u] & (kCoarseTiles - 1);
                s_stage[s_start[d] + s_count[wave][d] + rank[u]] = v[u];
            }
        }
        __syncthreads();
        for (uint32_t p = tid; p < n; p += kFineThreads) {
            const uint64_t pair = s_stage[p];
            const uint32_t low = (uint32_t)pair, d = low & (kCoarseTiles - 1);
            const uint32_t slot = s_slot[d] + (p - s_start[d]);
            // (a slot outside the bin cannot happen with pairs the coarse level wrote; the test keeps corrupted input
            // from reaching other memory)
            if (slot >= begin && slot < end) buckets[slot] = (pair & 0xFFFFFFFF00000000ull) | (uint64_t)(low >> kCoarseShift);
        }
        __syncthreads();
    }
}

// Pairs per tile, counted from the coarse bins (images of more tiles than a slice can count in LDS): the chunks of
// the fine scatter, a wavefront-level count by the four tile bits, one global atomic per tile and chunk.
// `bin_base` [bins]: first pair of each bin; `totals` [T] and `block_sums` [T / 64] (pairs per 64 tiles) cleared
// beforehand.
__global__ __launch_bounds__(kFineThreads) void fine_count_kernel(const gs355_header* __restrict__ header,
                                                                  const uint32_t* __restrict__ bin_base, int bins,
                                                                  int T, const uint32_t* __restrict__ chunk_base,
                                                                  const uint64_t* __restrict__ coarse,
                                                                  uint32_t* __restrict__ totals,
                                                                  uint64_t* __restrict__ block_sums,
                                                                  uint32_t* __restrict__ list_counts)
{
    __shared__ uint32_t s_count[kCoarseTiles];
    if (blockIdx.x == 0 && threadIdx.x < 4) list_counts[threadIdx.x] = 0u;  // filled by tile_publish_kernel
    if (header->overflow) return;
    const int tid = threadIdx.x, lane = tid & 63;
    const uint32_t num_keys = header->num_keys;
    ChunkRun run(chunk_base, bins);
    int bin;
    uint32_t j0, n, begin, end;
    while (run.next([&](int b) { return bin_base[b]; }, num_keys, bin, j0, n, begin, end)) {
        const int t0 = bin << kCoarseShift;
        if (tid < kCoarseTiles) s_count[tid] = 0;
        __syncthreads();
        uint64_t v[kFineItems];
#pragma unroll
        for (int u = 0; u < kFineItems; ++u) {
            const uint32_t p = (uint32_t)(u * kFineThreads + tid);
            v[u] = p < n ? coarse[j0 + p] : 0ull;
        }
#pragma unroll
        for (int u = 0; u < kFineItems; ++u) {
            const bool valid = (uint32_t)(u * kFineThreads + tid) < n;
            const uint32_t d = (uint32_t)v[u] & (kCoarseTiles - 1);
            uint64_t peers = __ballot(valid);
#pragma unroll
            for (int bit = 0; bit < kCoarseShift; ++bit) {
                const bool one = (d >> bit) & 1u;
                const uint64_t m = __ballot(one);
                peers &= one ? m : ~m;
            }
            if (valid && lane == __ffsll((unsigned long long)peers) - 1) atomicAdd(&s_count[d], (uint32_t)__popcll(peers));
        }
        __syncthreads();
        if (tid < kCoarseTiles && t0 + tid < T && s_count[tid]) {
            atomicAdd(&totals[t0 + tid], s_count[tid]);
            atomicAdd(reinterpret_cast<unsigned long long*>(&block_sums[(t0 + tid) >> 6]), (unsigned long long)s_count[tid]);
        }
        __syncthreads();
    }
}

// Exclusive prefix of every tile's counts over the slices (in place), the
// tile's total and the total of the workgroup's tiles.  A workgroup covers 64 tiles; its four wavefronts take a
// quarter of the slices each (loads of a thread are issued in batches, so many
// are in flight), exchange their quarter sums through LDS and write the
// prefixes shifted by the quarters before them.
__global__ __launch_bounds__(256) void slice_prefix_kernel(uint32_t* __restrict__ matrix, int groups, int tiles,
                                                           uint32_t* __restrict__ totals,
                                                           uint64_t* __restrict__ block_sums,
                                                           uint32_t* __restrict__ bin_sums,
                                                           uint32_t* __restrict__ block_classes,
                                                           uint32_t* __restrict__ list_counts)
{
    __shared__ uint32_t s_part[4][64];
    if (blockIdx.x == 0 && threadIdx.x < 4) list_counts[threadIdx.x] = 0u;  // filled by tile_publish_kernel
    const int lane = threadIdx.x & 63, part = threadIdx.x >> 6;
    const int t = blockIdx.x * 64 + lane;
    const int per = (groups + 3) / 4;
    const int c0 = min(part * per, groups), c1 = min(c0 + per, groups);
    const bool live = t < tiles;
    // pass 1: sum of this thread's quarter
    uint32_t sum = 0;
    for (int c = c0; c < c1 && live; c += 16) {
        uint32_t v[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) v[k] = matrix[(size_t)min(c + k, c1 - 1) * tiles + t];
#pragma unroll
        for (int k = 0; k < 16; ++k) sum += c + k < c1 ? v[k] : 0u;
    }
    s_part[part][lane] = sum;
    __syncthreads();
    uint32_t run = 0, total = 0;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t v = s_part[p][lane];
        if (p < part) run += v;
        total += v;
    }
    // pass 2: the quarter's values again (now cached), replaced by the running sum before them
    for (int c = c0; c < c1 && live; c += 16) {
        uint32_t v[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) v[k] = matrix[(size_t)min(c + k, c1 - 1) * tiles + t];
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            if (c + k < c1) {
                matrix[(size_t)(c + k) * tiles + t] = run;
                run += v[k];
            }
        }
    }
    if (part == 0) {
        if (live) totals[t] = total;
        uint64_t sum64 = live ? total : 0u;  // the 64 tiles of this workgroup are one block of the layout's scan
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) sum64 += __shfl_down(sum64, d, 64);
        if (lane == 0) block_sums[blockIdx.x] = sum64;
        if (block_classes) {  // columns are tiles: how many of the 64 fall in each larger sorter size class, a byte each
            const uint32_t v = live ? total : 0u;
            const uint32_t n1 = (uint32_t)__popcll(__ballot(v > (uint32_t)kTileSortCap[0] && v <= (uint32_t)kTileSortCap[1]));
            const uint32_t n2 = (uint32_t)__popcll(__ballot(v > (uint32_t)kTileSortCap[1] && v <= (uint32_t)kTileSortCap[2]));
            const uint32_t n3 = (uint32_t)__popcll(__ballot(v > (uint32_t)kTileSortCap[2] && v <= (uint32_t)kTileSortCap[3]));
            if (lane == 0) block_classes[blockIdx.x] = n1 | (n2 << 8) | (n3 << 16);
        }
        if (bin_sums) {  // columns are tiles: the pairs of each coarse bin (kCoarseTiles consecutive tiles)
            uint32_t bin = live ? total : 0u;
#pragma unroll
            for (int d = 1; d < kCoarseTiles; d <<= 1) bin += __shfl_xor(bin, d, 64);
            if ((lane & (kCoarseTiles - 1)) == 0 && live) bin_sums[t >> kCoarseShift] = bin;
        }
    }
}

// Layout of the buckets from the tiles' totals: one wavefront per block of 64 tiles, four per workgroup.  Every
// workgroup adds up the block totals itself (a few hundred words, at most 9000): those before its own blocks give its
// first slot, all of them the frame's key count, which decides overflow before anything is published — so no
// workgroup waits for another and no separate scan pass is launched.  Workgroup 0 also writes the frame header and
// the work list of the scatter's second level: chunk_base[b] = chunks of kFineChunk pairs in the coarse bins before
// b, chunk_base[bins] = all (`bin_pairs`, the pairs per bin, may be the same array).  With kTiles the wavefronts
// publish tile bases, the scatter's cursors, the ranges and the lists of buckets too large for the small sorter
// (`lists[0..3]` cleared by an earlier kernel); without, the columns are coarse bins and only their bases are
// written.  `totals` and `tile_base` may be the same array.  `header_known`: second layout of a frame (by tile,
// after the one by coarse bin): the header stands, and nothing is done on overflow.
template <bool kTiles>
__global__ __launch_bounds__(256) void tile_publish_kernel(const uint32_t* totals, uint32_t tiles,
                                                           const uint64_t* __restrict__ block_sums, uint32_t n_blocks,
                                                           const uint32_t* __restrict__ group_visible, int groups,
                                                           uint32_t n_cap, gs355_header* __restrict__ header,
                                                           gs355_header* __restrict__ header_copy, bool header_known,
                                                           uint32_t* tile_base,
                                                           uint32_t* __restrict__ ranges, uint32_t* __restrict__ lists,
                                                           const uint32_t* bin_pairs, int bins, uint32_t* chunk_base,
                                                           const uint32_t* __restrict__ block_classes)
{
    __shared__ uint64_t s_before[4], s_total[4];
    __shared__ uint32_t s_vis[4], s_chunks[4], s_class[3];
    if (header_known && header->overflow) return;
    if (threadIdx.x < 3) s_class[threadIdx.x] = 0u;
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint32_t first_block = blockIdx.x * 4u, block = first_block + (uint32_t)wave;
    {
        uint64_t before = 0, total = 0;
        for (uint32_t b = threadIdx.x; b < n_blocks; b += 256u) {
            const uint64_t v = block_sums[b];
            total += v;
            before += b < first_block ? v : 0ull;
        }
        uint32_t vis = 0;
        if (blockIdx.x == 0 && !header_known) {
            for (int c = threadIdx.x; c < groups; c += 256) vis += group_visible[c];
            // buckets per larger sorter size class, for the header (counted per block by the slice prefix)
            if (block_classes) {
                uint32_t n1 = 0, n2 = 0, n3 = 0;
                for (uint32_t b = threadIdx.x; b < n_blocks; b += 256u) {
                    const uint32_t w = block_classes[b];
                    n1 += w & 0xFFu;
                    n2 += (w >> 8) & 0xFFu;
                    n3 += (w >> 16) & 0xFFu;
                }
                if (n1) atomicAdd(&s_class[0], n1);
                if (n2) atomicAdd(&s_class[1], n2);
                if (n3) atomicAdd(&s_class[2], n3);
            }
        }
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) {
            before += __shfl_down(before, d, 64);
            total += __shfl_down(total, d, 64);
            vis += __shfl_down(vis, d, 64);
        }
        if (lane == 0) {
            s_before[wave] = before;
            s_total[wave] = total;
            s_vis[wave] = vis;
        }
    }
    __syncthreads();
    const uint64_t total = (s_total[0] + s_total[1]) + (s_total[2] + s_total[3]);
    const bool overflow = total > (uint64_t)n_cap;
    if (blockIdx.x == 0 && threadIdx.x == 0 && !header_known) {
        header->num_keys_total = total;
        header->num_keys = overflow ? n_cap : (uint32_t)total;
        header->overflow = overflow ? 1u : 0u;
        header->num_visible = (s_vis[0] + s_vis[1]) + (s_vis[2] + s_vis[3]);
        const bool counted = block_classes != nullptr;
        for (int c = 0; c < 3; ++c) header->sort_class_count[c] = counted ? s_class[c] : 0xFFFFFFFFu;
        if (header_copy) {  // (may be host memory: plain stores, complete when the kernel is)
            header_copy->num_keys_total = total;
            header_copy->num_keys = overflow ? n_cap : (uint32_t)total;
            header_copy->overflow = overflow ? 1u : 0u;
            header_copy->num_visible = (s_vis[0] + s_vis[1]) + (s_vis[2] + s_vis[3]);
            for (int c = 0; c < 3; ++c) header_copy->sort_class_count[c] = counted ? s_class[c] : 0xFFFFFFFFu;
        }
    }
    if (overflow) return;  // later stages do nothing either

    if (blockIdx.x == 0 && bins > 0) {
        const int per_thread = (bins + 255) / 256;
        const int q0 = min((int)threadIdx.x * per_thread, bins), q1 = min(q0 + per_thread, bins);
        uint32_t chunks = 0;
        for (int q = q0; q < q1; ++q) chunks += (bin_pairs[q] + (uint32_t)kFineChunk - 1u) / (uint32_t)kFineChunk;
        uint32_t cinc = chunks;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(cinc, d, 64);
            if (lane >= d) cinc += up;
        }
        if (lane == 63) s_chunks[wave] = cinc;
        __syncthreads();
        uint32_t run = cinc - chunks;
        for (int w = 0; w < wave; ++w) run += s_chunks[w];
        for (int q = q0; q < q1; ++q) {  // (each element is read before it is overwritten, by its own thread)
            const uint32_t n = (bin_pairs[q] + (uint32_t)kFineChunk - 1u) / (uint32_t)kFineChunk;
            chunk_base[q] = run;
            run += n;
        }
        if (threadIdx.x == 255) chunk_base[bins] = run;
    }

    uint64_t base = (s_before[0] + s_before[1]) + (s_before[2] + s_before[3]);  // first slot of the workgroup's blocks
    for (int w = 0; w < wave; ++w) base += first_block + (uint32_t)w < n_blocks ? block_sums[first_block + w] : 0ull;
    const uint32_t t = block * 64u + (uint32_t)lane;
    const bool live = t < tiles;
    const uint32_t v = live ? totals[t] : 0u;
    uint32_t inc = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = __shfl_up(inc, d, 64);
        if (lane >= d) inc += up;
    }
    if (block * 64u >= tiles) return;  // (uniform per wavefront)
    const uint32_t first = (uint32_t)base + inc - v;
    if (live) tile_base[t] = first;
    if (!kTiles) return;
    if (live) {
        ranges[2 * t] = v ? first : 0u;
        ranges[2 * t + 1] = v ? first + v : 0u;
        tile_base[tiles + t] = first;  // the bucket's next free slot during the scatter
    }
    // buckets beyond the smallest sorter's capacity go on the list of their size class (order within a list is free):
    // one request per wavefront and class
    int cls = -1;
    if (v > (uint32_t)kTileSortCap[3]) cls = -1;  // beyond the LDS sorters: sorted by its own workgroup of the class-0 kernel
    else if (v > (uint32_t)kTileSortCap[2]) cls = 2;
    else if (v > (uint32_t)kTileSortCap[1]) cls = 1;
    else if (v > (uint32_t)kTileSortCap[0]) cls = 0;
    const uint64_t lanes_below = (1ull << lane) - 1ull;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint64_t m = __ballot(cls == c);
        if (m == 0ull) continue;
        uint32_t at = 0;
        if (lane == __ffsll((unsigned long long)m) - 1) at = atomicAdd(&lists[c], (uint32_t)__popcll(m));
        at = __shfl(at, __ffsll((unsigned long long)m) - 1, 64);
        if (cls == c) lists[kListHeader + (size_t)c * tiles + at + (uint32_t)__popcll(m & lanes_below)] = t;
    }
}

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kRounds = 4;                      // 64-key rounds per wave per chunk
constexpr int kChunk = kWaves * kRounds * 64;  // 1024 pairs ranked per iteration

// ---------------------------------------------------------------------------
// Storage of a bucket during sorting: two words per pair.
struct LdsPairs {
    uint32_t* d;  // depth bits
    uint32_t* i;  // Gaussian index
    __device__ __forceinline__ void load(uint32_t j, uint32_t& kd, uint32_t& ki) const
    {
        kd = d[j];
        ki = i[j];
    }
    __device__ __forceinline__ void store(uint32_t j, uint32_t kd, uint32_t ki) const
    {
        d[j] = kd;
        i[j] = ki;
    }
};

struct GlobalPairs {
    uint64_t* p;  // depth bits << 32 | Gaussian index
    __device__ __forceinline__ void load(uint32_t j, uint32_t& kd, uint32_t& ki) const
    {
        const uint64_t v = p[j];
        kd = (uint32_t)(v >> 32);
        ki = (uint32_t)v;
    }
    __device__ __forceinline__ void store(uint32_t j, uint32_t kd, uint32_t ki) const
    {
        p[j] = ((uint64_t)kd << 32) | (uint64_t)ki;
    }
};

struct SortScratch {
    uint32_t* hist;           // [256] digit totals, then running digit bases
    uint32_t (*cnt)[256];     // [kWaves][256] per-wave digit counts of the current chunk
    uint32_t* flags;          // [8] small flags / partial sums
};

// One stable 8-bit LSD pass over n pairs, digit taken from the depth word
// (by_depth) or the index word.  Returns false (and moves nothing) when every
// pair has the same digit.
template <typename Src, typename Dst>
__device__ bool radix_pass(const Src src, const Dst dst, uint32_t n, int shift, bool by_depth, const SortScratch sc)
{
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    sc.hist[tid] = 0;
    if (tid < 8) sc.flags[tid] = 0;
    __syncthreads();
    for (uint32_t j = tid; j < n; j += kThreads) {
        uint32_t kd, ki;
        src.load(j, kd, ki);
        atomicAdd(&sc.hist[((by_depth ? kd : ki) >> shift) & 255u], 1u);
    }
    __syncthreads();
    {
        // exclusive scan of the 256 digit totals; detect the single-digit case
        const uint32_t h = sc.hist[tid];
        uint32_t inc = h;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(inc, d, 64);
            if (lane >= d) inc += up;
        }
        if (lane == 63) sc.flags[wave] = inc;
        if (h == n) sc.flags[4] = 1;
        __syncthreads();
        uint32_t off = 0;
        for (int w = 0; w < wave; ++w) off += sc.flags[w];
        sc.hist[tid] = off + inc - h;
        const bool single = sc.flags[4] != 0;
        __syncthreads();
        if (single) return false;
    }
    const uint64_t lanes_below = (1ull << lane) - 1ull;
    for (uint32_t c0 = 0; c0 < n; c0 += kChunk) {
#pragma unroll
        for (int w = 0; w < kWaves; ++w) sc.cnt[w][tid] = 0;
        __syncthreads();
        uint32_t kd[kRounds], ki[kRounds], rank[kRounds];
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const uint32_t j = c0 + (uint32_t)(wave * kRounds + r) * 64u + lane;
            const bool valid = j < n;
            kd[r] = 0;
            ki[r] = 0;
            if (valid) src.load(j, kd[r], ki[r]);
            const uint32_t dgt = ((by_depth ? kd[r] : ki[r]) >> shift) & 255u;
            uint64_t peers = __ballot(valid);
#pragma unroll
            for (int bit = 0; bit < 8; ++bit) {
                const bool one = (dgt >> bit) & 1u;
                const uint64_t m = __ballot(one);
                peers &= one ? m : ~m;
            }
            uint32_t pre = 0;
            const uint32_t below = (uint32_t)__popcll(peers & lanes_below);
            if (valid) {
                const int leader = __ffsll((unsigned long long)peers) - 1;
                if (lane == leader) pre = atomicAdd(&sc.cnt[wave][dgt], (uint32_t)__popcll(peers));
                pre = __shfl(pre, leader, 64);
            }
            rank[r] = pre + below;
        }
        __syncthreads();
        {
            uint32_t run = sc.hist[tid];
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                const uint32_t c = sc.cnt[w][tid];
                sc.cnt[w][tid] = run;
                run += c;
            }
            sc.hist[tid] = run;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kRounds; ++r) {
            const uint32_t j = c0 + (uint32_t)(wave * kRounds + r) * 64u + lane;
            if (j < n) {
                const uint32_t dgt = ((by_depth ? kd[r] : ki[r]) >> shift) & 255u;
                dst.store(sc.cnt[wave][dgt] + rank[r], kd[r], ki[r]);
            }
        }
        __syncthreads();
    }
    return true;
}

// Sort n pairs held in buffer A (B is scratch of the same size) by
// (depth bits, index).  Returns true if the result is in B.
template <typename Buf>
__device__ bool sort_pairs(const Buf A, const Buf B, uint32_t n, const SortScratch sc)
{
    bool in_b = false;
    // depth passes; pairs of one tile rarely share depth bits, so the index
    // word is only brought in when a tie is actually present
    for (int pass = 0; pass < 4; ++pass) {
        const bool moved = in_b ? radix_pass(B, A, n, pass * 8, true, sc) : radix_pass(A, B, n, pass * 8, true, sc);
        if (moved) in_b = !in_b;
    }
    {
        const Buf cur = in_b ? B : A;
        if (threadIdx.x == 0) sc.flags[5] = 0;
        __syncthreads();
        bool tie = false;
        for (uint32_t j = threadIdx.x; j + 1 < n; j += kThreads) {
            uint32_t d0, i0, d1, i1;
            cur.load(j, d0, i0);
            cur.load(j + 1, d1, i1);
            tie |= (d0 == d1) && (i0 > i1);
        }
        if (tie) sc.flags[5] = 1;
        __syncthreads();
        const bool any = sc.flags[5] != 0;
        __syncthreads();
        if (!any) return in_b;
    }
    // equal depth bits out of index order: full (index, then depth) stable sort
    for (int pass = 0; pass < 8; ++pass) {
        const bool by_depth = pass >= 4;
        const int shift = (pass & 3) * 8;
        const bool moved = in_b ? radix_pass(B, A, n, shift, by_depth, sc) : radix_pass(A, B, n, shift, by_depth, sc);
        if (moved) in_b = !in_b;
    }
    return in_b;
}

template <typename Buf>
__device__ __forceinline__ void write_sorted(const Buf cur, uint32_t n, uint32_t tile, uint64_t* out_keys,
                                             uint32_t* out_vals)
{
    for (uint32_t j = threadIdx.x; j < n; j += kThreads) {
        uint32_t kd, ki;
        cur.load(j, kd, ki);
        out_keys[j] = ((uint64_t)tile << 32) | (uint64_t)kd;
        out_vals[j] = ki;
    }
}

// ---------------------------------------------------------------------------
// In-LDS bucket sorter: kT threads, up to kT * kR pairs, every pass ranks the
// whole bucket at once (each wavefront owns kR * 64 consecutive positions).
// LDS holds the bucket once (depth bits, index: 8 B per pair) plus two 16-bit
// permutations that ping-pong between passes (4 B per pair).
template <int kT, int kR>
struct LdsSorter {
    static constexpr int kW = kT / 64;
    static constexpr int kCap = kT * kR;
    // fine bins per thread of the counting pass (measured at 1080p / 6M Gaussians, the two larger classes together:
    // 1 / 2 / 3 / 4 bins = 0.169 / 0.155 / 0.147 / 0.145 ms)
    static constexpr int kBinsPer = kT >= 512 ? 4 : 2;
    static constexpr int kB = kBinsPer * kT;                      // fine bins
    // counters: [kW][256] words for the radix passes, or the fine bins and 512 coarse words of the counting pass
    static constexpr int kCounterWords = kB + 512 > kW * 256 ? kB + 512 : kW * 256;
    static constexpr size_t kBytes = (size_t)kCap * 12 + (size_t)kCounterWords * 4 + 192;

    uint32_t* depth;     // [kCap]
    uint32_t* index;     // [kCap]
    uint16_t* perm0;     // two permutations of [kCap] each, back to back
    uint32_t (*cnt)[256];  // [kW][256]
    uint32_t* flags;     // [48]

    __device__ explicit LdsSorter(uint32_t* lds)
    {
        depth = lds;
        index = lds + kCap;
        perm0 = reinterpret_cast<uint16_t*>(lds + 2 * kCap);
        cnt = reinterpret_cast<uint32_t(*)[256]>(lds + 3 * kCap);
        flags = lds + 3 * kCap + kCounterWords;
    }

    __device__ __forceinline__ uint16_t* perm(int which) const { return perm0 + which * kCap; }

    // One stable pass.  `src` < 0: the input order is the identity.  Returns the
    // buffer holding the output order (unchanged when all digits are equal).
    __device__ int pass(uint32_t n, int shift, bool by_depth, int src) const
    {
        const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
        for (int k = tid; k < kW * 256; k += kT) (&cnt[0][0])[k] = 0;
        if (tid == 0) flags[8] = 0;
        __syncthreads();
        const int dst = src == 0 ? 1 : 0;
        const uint64_t lanes_below = (1ull << lane) - 1ull;
        uint32_t ent[kR];  // entry | digit << 16
        uint32_t rank[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            ent[r] = 0;
            rank[r] = 0;
            if ((uint32_t)(wave * kR + r) * 64u >= n) continue;  // whole round past the end (uniform per wavefront)
            const uint32_t j = (uint32_t)(wave * kR + r) * 64u + lane;
            const bool valid = j < n;
            const uint32_t e = valid ? (src < 0 ? j : (uint32_t)perm(src)[j]) : 0u;
            const uint32_t key = valid ? (by_depth ? depth[e] : index[e]) : 0u;
            const uint32_t dgt = (key >> shift) & 255u;
            uint64_t peers = __ballot(valid);
#pragma unroll
            for (int bit = 0; bit < 8; ++bit) {
                const bool one = (dgt >> bit) & 1u;
                const uint64_t m = __ballot(one);
                peers &= one ? m : ~m;
            }
            uint32_t pre = 0;
            const uint32_t below = (uint32_t)__popcll(peers & lanes_below);
            if (valid) {
                const int leader = __ffsll((unsigned long long)peers) - 1;
                if (lane == leader) pre = atomicAdd(&cnt[wave][dgt], (uint32_t)__popcll(peers));
                pre = __shfl(pre, leader, 64);
            }
            rank[r] = pre + below;
            ent[r] = e | (dgt << 16);
        }
        __syncthreads();
        // digit totals, exclusive scan over the 256 digits (wavefronts 0..3), per-wave bases
        uint32_t total = 0, inc = 0;
        if (tid < 256) {
#pragma unroll
            for (int w = 0; w < kW; ++w) total += cnt[w][tid];
            if (total == n) flags[8] = 1;  // every pair has this digit: nothing to move
            inc = total;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t up = __shfl_up(inc, d, 64);
                if (lane >= d) inc += up;
            }
            if (lane == 63) flags[wave] = inc;
        }
        __syncthreads();
        if (tid < 256) {
            uint32_t base = inc - total;
            for (int w = 0; w < wave; ++w) base += flags[w];
#pragma unroll
            for (int w = 0; w < kW; ++w) {
                const uint32_t c = cnt[w][tid];
                cnt[w][tid] = base;
                base += c;
            }
        }
        __syncthreads();
        const bool single = flags[8] != 0;
        if (!single) {
#pragma unroll
            for (int r = 0; r < kR; ++r) {
                const uint32_t j = (uint32_t)(wave * kR + r) * 64u + lane;
                if (j < n) perm(dst)[cnt[wave][ent[r] >> 16] + rank[r]] = (uint16_t)ent[r];
            }
        }
        __syncthreads();
        return single ? src : dst;
    }

    // Sort the n loaded pairs by (depth bits, index); returns the buffer with
    // the final order.
    __device__ int sort(uint32_t n, uint32_t varying) const
    {
        int cur = -1;
        // bytes of the depth word that are identical in every pair need no pass
        // (inside one tile the exponent byte of the depths usually is)
        for (int p = 0; p < 4; ++p)
            if ((varying >> (p * 8)) & 255u) cur = pass(n, p * 8, true, cur);
        if (cur < 0) {  // no pass moved anything (all depth bits equal, or n == 1): start from the identity
            for (uint32_t j = threadIdx.x; j < n; j += kT) perm(0)[j] = (uint16_t)j;
            cur = 0;
            __syncthreads();
        }
        // Bucket order before the sort is arbitrary, so pairs with equal depth
        // bits may be out of index order.  Such runs are rare and short: a few
        // rounds of odd-even transposition inside runs settle them; only if a
        // round still swaps after that is the full (index, depth) sort run.
        uint16_t* const P = perm(cur);
        bool unsettled = true;
        for (int round = 0; round < 4 && unsettled; ++round) {
            if (threadIdx.x == 0) flags[10] = 0;
            __syncthreads();
            bool swapped = false;
            for (int phase = 0; phase < 2; ++phase) {
                for (uint32_t j = 2u * threadIdx.x + phase; j + 1 < n; j += 2u * kT) {
                    const uint32_t e0 = P[j], e1 = P[j + 1];
                    if (depth[e0] == depth[e1] && index[e0] > index[e1]) {
                        P[j] = (uint16_t)e1;
                        P[j + 1] = (uint16_t)e0;
                        swapped = true;
                    }
                }
                __syncthreads();
            }
            if (swapped) flags[10] = 1;
            __syncthreads();
            unsettled = flags[10] != 0;
            __syncthreads();
        }
        if (!unsettled) return cur;
        for (int p = 0; p < 8; ++p) cur = pass(n, (p & 3) * 8, p >= 4, cur);
        return cur;
    }

    // Fast path: one counting pass over a monotone map of the depth onto kT bins leaves a handful of pairs per
    // bin; every pair then ranks itself among the members of its bin by (depth bits, index).  Bins are ordered and
    // each bin is fully ordered, so the result is the exact total order whatever order the LDS atomics ran in.
    // Depths along the rays of a tile cluster (most splats sit near the ground), so the map is adaptive: a
    // 256-bin histogram over [dmin, dmax] gives a piecewise-linear estimate of each pair's final position, and
    // the bin is that position scaled to kT.  Returns the buffer holding the order, or -2 when some bin is still
    // too full for this to pay: the caller then runs the radix passes.
    static constexpr uint32_t kMaxBin = 256;

    __device__ int bucket_sort(uint32_t n, uint32_t dmin, uint32_t dmax) const
    {
        const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
        uint32_t* const count = &cnt[0][0];  // [kB] pairs per bin, then the bin's first slot
        uint32_t* const coarse = count + kB;  // [256] pairs per coarse bin, then their exclusive prefix
        const uint32_t range = dmax - dmin;
        if (range == 0) return -2;
        // coarse(d) = floor((d - dmin) * 256 / (range + 1)) as the high word of a 32x32 multiply, whose low word is
        // the position inside the coarse bin as a 0.32 fraction; a range below 256 gives every depth its own bin
        const bool direct = range < 256u;
        const uint32_t mult = direct ? 0u : (uint32_t)((256ull << 32) / ((uint64_t)range + 1ull));
        // position -> bin: floor(pos * kB / n) for n > kB, else the position itself (one pair per bin)
        const bool spread = n > (uint32_t)kB;
        const uint32_t to_bin = spread ? (uint32_t)(((uint64_t)kB << 32) / (uint64_t)n) : 0u;
        // (the counters were cleared by the caller, before the barrier that made dmin and dmax known)
        uint32_t cbin[kR], frac[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t j = (uint32_t)r * kT + tid;
            cbin[r] = 0;
            frac[r] = 0;
            if (j < n) {
                const uint32_t rel = depth[j] - dmin;
                const uint64_t wide = (uint64_t)rel * mult;
                cbin[r] = direct ? rel : (uint32_t)(wide >> 32);
                frac[r] = direct ? 0u : (uint32_t)wide;
                atomicAdd(&coarse[cbin[r]], 1u);
            }
        }
        __syncthreads();
        if (tid < 256) {  // exclusive scan of the coarse counts (wavefronts 0..3)
            const uint32_t own = coarse[tid];
            uint32_t inc = own;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t up = __shfl_up(inc, d, 64);
                if (lane >= d) inc += up;
            }
            if (lane == 63) flags[16 + wave] = inc;
            // (a thread replaces the one count that only it has read) exclusive within the wavefront: the
            // wavefronts' totals are added by whoever reads it, which saves a barrier
            coarse[tid] = inc - own;
            coarse[256 + tid] = own;
        }
        __syncthreads();
        const uint32_t before1 = flags[16], before2 = before1 + flags[17], before3 = before2 + flags[18];
        uint32_t bin[kR], slot[kR];
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t j = (uint32_t)r * kT + tid;
            bin[r] = 0;
            slot[r] = 0;
            if (j < n) {
                const uint32_t cb = cbin[r];
                const uint32_t before = cb >= 192u ? before3 : cb >= 128u ? before2 : cb >= 64u ? before1 : 0u;
                const uint32_t pos = coarse[cb] + before + __umulhi(frac[r], coarse[256 + cb]);  // in [0, n)
                bin[r] = min(spread ? __umulhi(pos, to_bin) : pos, (uint32_t)kB - 1u);
                slot[r] = atomicAdd(&count[bin[r]], 1u);
            }
        }
        __syncthreads();
        // exclusive scan of the kB bin counts (a thread owns kBinsPer consecutive bins); remember whether any bin
        // is over-full
        uint32_t mine[kBinsPer], c = 0;
        bool overfull = false;
#pragma unroll
        for (int i = 0; i < kBinsPer; ++i) {
            mine[i] = count[kBinsPer * tid + i];
            c += mine[i];
            overfull = overfull || mine[i] > kMaxBin;
        }
        uint32_t inc = c;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(inc, d, 64);
            if (lane >= d) inc += up;
        }
        if (lane == 63) flags[16 + wave] = inc;
        if (overfull) flags[8] = 1;
        __syncthreads();
        if (flags[8] != 0) {
            __syncthreads();
            return -2;
        }
        uint32_t first = inc - c;
        for (int w = 0; w < wave; ++w) first += flags[16 + w];
#pragma unroll
        for (int i = 0; i < kBinsPer; ++i) {
            count[kBinsPer * tid + i] = first;
            first += mine[i];
        }
        __syncthreads();
        uint16_t* const P = perm(0);
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t j = (uint32_t)r * kT + tid;
            if (j < n) P[count[bin[r]] + slot[r]] = (uint16_t)j;
        }
        __syncthreads();
        // every pair ranks itself among the members of its bin (independent reads, evenly spread over the
        // threads whatever the bin sizes are) and takes the slot of that rank
        uint16_t* const Q = perm(1);
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t j = (uint32_t)r * kT + tid;
            if (j < n) {
                const uint32_t b = bin[r];
                const uint32_t lo_slot = count[b];
                const uint32_t hi_slot = b + 1 < (uint32_t)kB ? count[b + 1] : n;
                const uint32_t md = depth[j], mi = index[j];
                uint32_t rank = 0;
                for (uint32_t q = lo_slot; q < hi_slot; ++q) {
                    const uint32_t e = P[q];
                    const uint32_t ed = depth[e], ei = index[e];
                    rank += (ed < md || (ed == md && ei < mi)) ? 1u : 0u;
                }
                Q[lo_slot + rank] = (uint16_t)j;
            }
        }
        __syncthreads();
        return 1;
    }

    // A bucket on its way from memory: where it lies and this thread's pairs of it (requested, not yet used).
    struct Fetched {
        uint32_t tile, lo, n;
        uint64_t v[kR];
    };

    __device__ __forceinline__ void fetch_range(Fetched& f, uint32_t tile, const uint32_t* __restrict__ ranges) const
    {
        f.tile = tile;
        f.lo = ranges[2 * tile];
        f.n = ranges[2 * tile + 1] - f.lo;
    }

    // the whole bucket is requested before the first pair is used: one memory latency, not one per round
    __device__ __forceinline__ void fetch_pairs(Fetched& f, const uint64_t* __restrict__ buckets) const
    {
        const bool mine = f.n != 0 && f.n <= (uint32_t)kCap;
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t j = (uint32_t)r * kT + threadIdx.x;
            f.v[r] = mine && j < f.n ? __builtin_nontemporal_load(&buckets[f.lo + j]) : 0ull;  // (read once)
        }
    }

    // Sorts the fetched bucket and writes it out; ends with a barrier.
    __device__ void sort_fetched(const Fetched& f, uint64_t* __restrict__ out_keys, uint32_t* __restrict__ out_vals) const
    {
        const uint32_t lo = f.lo, n = f.n, tile = f.tile;
        if (n == 0 || n > (uint32_t)kCap) return;  // uniform over the workgroup
        if (threadIdx.x == 0) {
            flags[11] = 0;
            flags[12] = 0xFFFFFFFFu;
            flags[13] = 0;
            flags[14] = 0xFFFFFFFFu;
        }
        __syncthreads();
        // depth bits that differ somewhere in the bucket = (OR of all) ^ (AND of all)
        uint32_t any = 0, all = 0xFFFFFFFFu, dmin = 0xFFFFFFFFu, dmax = 0;
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const uint32_t j = (uint32_t)r * kT + threadIdx.x;
            if (j < n) {
                const uint32_t dj = (uint32_t)(f.v[r] >> 32);
                depth[j] = dj;
                index[j] = (uint32_t)f.v[r];
                any |= dj;
                all &= dj;
                dmin = min(dmin, dj);
                dmax = max(dmax, dj);
            }
        }
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) {
            any |= __shfl_xor(any, d, 64);
            all &= __shfl_xor(all, d, 64);
            dmin = min(dmin, (uint32_t)__shfl_xor(dmin, d, 64));
            dmax = max(dmax, (uint32_t)__shfl_xor(dmax, d, 64));
        }
        if ((threadIdx.x & 63) == 0) {
            atomicOr(&flags[11], any);
            atomicAnd(&flags[14], all);
            atomicMin(&flags[12], dmin);
            atomicMax(&flags[13], dmax);
        }
        {  // the counting sort's counters, cleared here so that it needs no barrier of its own for it
            uint32_t* const count = &cnt[0][0];
#pragma unroll
            for (int i = 0; i < kBinsPer; ++i) count[i * kT + threadIdx.x] = 0;
            if (threadIdx.x < 256) count[kB + threadIdx.x] = 0;
            if (threadIdx.x == 0) flags[8] = 0;
        }
        __syncthreads();
        int cur = bucket_sort(n, flags[12], flags[13]);
        if (cur == -2) cur = sort(n, flags[11] ^ flags[14]);
        for (uint32_t j = threadIdx.x; j < n; j += kT) {
            const uint32_t e = cur < 0 ? j : (uint32_t)perm(cur)[j];
            // (no later stage reads the sorted keys: a streaming store, which leaves the cache to the records the
            // blend is about to gather)
            __builtin_nontemporal_store(((uint64_t)tile << 32) | (uint64_t)depth[e], &out_keys[lo + j]);
            out_vals[lo + j] = index[e];
        }
        __syncthreads();
    }

    __device__ void run(uint32_t tile, const uint32_t* __restrict__ ranges, const uint64_t* __restrict__ buckets,
                        uint64_t* __restrict__ out_keys, uint32_t* __restrict__ out_vals) const
    {
        Fetched f;
        fetch_range(f, tile, ranges);
        fetch_pairs(f, buckets);
        sort_fetched(f, out_keys, out_vals);
    }
};

// Smallest size class: one workgroup per tile; tiles with larger buckets leave at once, except those beyond the
// capacity of the largest LDS sorter, which are sorted here by radix passes through global memory, ping-ponging
// between the bucket and the tile's slice of the output keys (their scratch lies over the LDS sorter's area).
// `skip_classes` (bit c: the sorter of larger class c is not launched for this frame, the caller expecting no bucket
// of that size): such a bucket, should there be one after all, takes the global-memory route too, so every bucket is
// sorted whatever the caller expected.
template <int kT, int kR>
__global__ __launch_bounds__(kT) void tile_sort_each_kernel(const gs355_header* __restrict__ header,
                                                            const uint32_t* __restrict__ ranges,
                                                            uint64_t* __restrict__ buckets,
                                                            uint64_t* __restrict__ out_keys,
                                                            uint32_t* __restrict__ out_vals, uint32_t skip_classes)
{
    extern __shared__ uint32_t s_dyn[];
    if (header->overflow) return;
    static_assert(kT == kThreads, "the global-memory passes are written for kThreads threads");
    static_assert((256 + kWaves * 256 + 8) * sizeof(uint32_t) <= LdsSorter<kT, kR>::kBytes, "scratch of the global passes");
    const uint32_t tile = blockIdx.x;
    const uint32_t lo = ranges[2 * tile], n = ranges[2 * tile + 1] - lo;
    bool through_global = n > (uint32_t)kTileSortCap[3];
    if (skip_classes != 0u && n > (uint32_t)kTileSortCap[0] && !through_global) {
        const int cls = n <= (uint32_t)kTileSortCap[1] ? 0 : n <= (uint32_t)kTileSortCap[2] ? 1 : 2;
        through_global = (skip_classes >> cls) & 1u;
    }
    if (through_global) {  // (uniform over the workgroup)
        const SortScratch sc = {s_dyn, reinterpret_cast<uint32_t(*)[256]>(s_dyn + 256), s_dyn + 256 + kWaves * 256};
        const GlobalPairs A = {buckets + lo}, B = {out_keys + lo};
        const bool in_b = sort_pairs(A, B, n, sc);
        // when the result sits in the output slice itself, each element is rewritten in place by the thread that read it
        write_sorted(in_b ? B : A, n, tile, out_keys + lo, out_vals + lo);
        return;
    }
    const LdsSorter<kT, kR> sorter(s_dyn);
    sorter.run(tile, ranges, buckets, out_keys, out_vals);
}

// Larger size classes: one workgroup per entry of the class list made by tile_publish_kernel.  The number of
// entries is only known on the device, so a launch has a workgroup per tile and those past the list's end leave at
// once: the hardware's own dispatch hands out the buckets.  (Persistent workgroups that fetched their work from a
// counter spent 8-14 us per bucket on dependent requests -- counter, list entry, range, pairs -- whatever the
// bucket held, requesting the next bucket inside the current sort did not hide them, and even a plain strided loop
// around the sort costs a sixth of the kernel's time in registers kept alive across it.)  kStrided: a launch
// smaller than the list, for the class whose workgroups fill a CU each.
template <int kT, int kR, bool kStrided>
__device__ __forceinline__ void tile_sort_list_body(const gs355_header* __restrict__ header,
                                                    const uint32_t* __restrict__ ranges,
                                                    const uint32_t* __restrict__ list,
                                                    const uint32_t* __restrict__ list_count,
                                                    const uint64_t* __restrict__ buckets,
                                                    uint64_t* __restrict__ out_keys, uint32_t* __restrict__ out_vals,
                                                    uint32_t* lds)
{
    if (header->overflow) return;
    const LdsSorter<kT, kR> sorter(lds);
    const uint32_t count = *list_count;
    if (kStrided) {
        for (uint32_t k = blockIdx.x; k < count; k += gridDim.x) sorter.run(list[k], ranges, buckets, out_keys, out_vals);
    } else if (blockIdx.x < count) {
        sorter.run(list[blockIdx.x], ranges, buckets, out_keys, out_vals);
    }
}

// 1024 threads x 5 rounds, held to 64 VGPRs so that two workgroups share a CU
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8))) void tile_sort_list_1024x5_kernel(
    const gs355_header* __restrict__ header, const uint32_t* __restrict__ ranges, const uint32_t* __restrict__ list,
    const uint32_t* __restrict__ list_count, const uint64_t* __restrict__ buckets, uint64_t* __restrict__ out_keys,
    uint32_t* __restrict__ out_vals)
{
    extern __shared__ uint32_t s_dyn[];
    tile_sort_list_body<1024, 5, false>(header, ranges, list, list_count, buckets, out_keys, out_vals, s_dyn);
}

template <int kT, int kR, bool kStrided>
__global__ __launch_bounds__(kT) void tile_sort_list_kernel(const gs355_header* __restrict__ header,
                                                            const uint32_t* __restrict__ ranges,
                                                            const uint32_t* __restrict__ list,
                                                            const uint32_t* __restrict__ list_count,
                                                            const uint64_t* __restrict__ buckets,
                                                            uint64_t* __restrict__ out_keys,
                                                            uint32_t* __restrict__ out_vals)
{
    extern __shared__ uint32_t s_dyn[];
    tile_sort_list_body<kT, kR, kStrided>(header, ranges, list, list_count, buckets, out_keys, out_vals, s_dyn);
}

}  // namespace

int bin_groups(int32_t P, int* per_group)
{
    // slices are multiples of the workgroup size so that every pass over a slice is full
    int per = (P + kBinMaxGroups - 1) / kBinMaxGroups;
    per = (per + kBinThreads - 1) / kBinThreads * kBinThreads;
    if (per < kBinThreads) per = kBinThreads;
    *per_group = per;
    const int groups = (P + per - 1) / per;
    return groups < 1 ? 1 : groups;
}

// Dynamic LDS beyond 64 KB has to be allowed per kernel.  The limits are raised once per process and device to
// the largest size any launch can ask for, so that concurrent frames of different image sizes (other streams,
// other threads) never lower the limit under each other.
template <typename K>
static hipError_t raise_lds_limit(K kernel, size_t bytes)
{
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)bytes);
}

static int allow_large_lds()
{
    constexpr int kMaxDevices = 64;
    static std::atomic<int> done[kMaxDevices];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return set_error(GS355_EHIP, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return set_error(GS355_EINVAL, "device index %d is outside [0, %d)", dev, kMaxDevices);
    if (done[dev].load(std::memory_order_acquire)) return GS355_OK;
    const size_t bin_bytes = (size_t)kBinMaxTiles * sizeof(uint32_t);
    if ((e = raise_lds_limit(tile_count_kernel<false>, bin_bytes)) != hipSuccess ||
        (e = raise_lds_limit(tile_count_kernel<true>, bin_bytes)) != hipSuccess ||
        (e = raise_lds_limit(scatter_kernel<0, false>, bin_bytes)) != hipSuccess ||
        (e = raise_lds_limit(scatter_kernel<kCoarseShift, true>, bin_bytes)) != hipSuccess ||
        (e = raise_lds_limit(tile_sort_list_1024x5_kernel, LdsSorter<1024, 5>::kBytes)) != hipSuccess ||
        (e = raise_lds_limit(tile_sort_list_kernel<1024, 10, true>, LdsSorter<1024, 10>::kBytes)) != hipSuccess)
        return set_error(GS355_EHIP, "LDS limit of the binning / tile sort kernels: %s", hipGetErrorString(e));
    done[dev].store(1, std::memory_order_release);  // racing threads set the same values
    return GS355_OK;
}

static inline int coarse_bins(int tiles) { return (tiles + kCoarseTiles - 1) >> kCoarseShift; }
// the tile_base array: u32[2][tiles], u64[blocks of 64 tiles], u32[coarse bins + 1] chunk bases
static inline uint32_t* chunk_bases(uint32_t* tile_base, int tiles)
{
    return tile_base + 2 * (size_t)tiles + 2 * (size_t)((tiles + 63) / 64);
}

int launch_tile_count(const FrameArgs& f, int32_t P, const uint64_t* rects, uint32_t* matrix, uint32_t* group_visible,
                      hipStream_t s)
{
    int per_group;
    const int groups = bin_groups(P, &per_group);
    const int T = f.grid_x * f.grid_y;
    int rc = allow_large_lds();
    if (rc) return rc;
    if (T <= kBinMaxTiles)
        hipLaunchKernelGGL(tile_count_kernel<false>, dim3(groups), dim3(kBinThreads), (size_t)T * sizeof(uint32_t), s, f,
                           P, per_group, rects, matrix, group_visible);
    else
        hipLaunchKernelGGL(tile_count_kernel<true>, dim3(groups), dim3(kBinThreads),
                           (size_t)coarse_bins(T) * sizeof(uint32_t), s, f, P, per_group, rects, matrix, group_visible);
    GS355_CHECK_LAUNCH("bin: count");
    return GS355_OK;
}

// Bases of `columns` buckets from their totals (block sums already in `blocks`), and the per-tile outputs with kTiles.
// `bases` may be `totals`, unless `bin_pairs` is `totals` too (workgroup 0 reads every bin's pairs while the others
// already write bases).
template <bool kTiles>
static int launch_layout(const uint32_t* totals, uint32_t* bases, int columns, const uint64_t* blocks,
                         const uint32_t* group_visible, int groups, uint32_t n_cap, gs355_header* header,
                         gs355_header* header_copy, bool header_known, uint32_t* ranges, uint32_t* lists, const uint32_t* bin_pairs, int bins,
                         uint32_t* chunk_base, const uint32_t* block_classes, hipStream_t s)
{
    const int n_blocks = (columns + 63) / 64;
    hipLaunchKernelGGL(tile_publish_kernel<kTiles>, dim3((n_blocks + 3) / 4), dim3(256), 0, s, totals, (uint32_t)columns,
                       blocks, (uint32_t)n_blocks, group_visible, groups, n_cap, header, header_copy, header_known, bases, ranges, lists,
                       bin_pairs, bins, chunk_base, block_classes);
    GS355_CHECK_LAUNCH("bin: layout");
    return GS355_OK;
}

// Up to kBinMaxTiles tiles: everything the later stages need (tile bases, cursors, ranges, size-class lists,
// header).  Beyond: the header and the coarse bins' bases (in tile_cursor[0, bins)); the per-tile layout follows
// in launch_tile_scatter once the pairs of each bin can be counted by tile.
int launch_tile_layout(int32_t P, uint32_t* matrix, const uint32_t* group_visible, int tiles, uint32_t n_cap,
                       gs355_header* header, gs355_header* header_copy, uint32_t* tile_base, uint32_t* ranges, uint32_t* lists, hipStream_t s)
{
    int per_group;
    const int groups = bin_groups(P, &per_group);
    uint64_t* blocks = reinterpret_cast<uint64_t*>(tile_base + 2 * (size_t)tiles);
    const int bins = coarse_bins(tiles);
    uint32_t* chunk_base = chunk_bases(tile_base, tiles);
    uint32_t* block_classes = chunk_base + bins + 1;  // [ceil(tiles / 64)]
    if (tiles <= kBinMaxTiles) {
        // (the pairs of each coarse bin go to chunk_base, which the block scan turns into chunk bases in place)
        hipLaunchKernelGGL(slice_prefix_kernel, dim3((tiles + 63) / 64), dim3(256), 0, s, matrix, groups, tiles,
                           tile_base, blocks, chunk_base, block_classes, lists);
        GS355_CHECK_LAUNCH("bin: slice prefix");
        return launch_layout<true>(tile_base, tile_base, tiles, blocks, group_visible, groups, n_cap, header, header_copy, false, ranges,
                                   lists, chunk_base, bins, chunk_base, block_classes, s);
    }
    // (both in the cursor half of tile_base, which the tile-level layout of launch_tile_scatter overwrites later)
    uint32_t* bin_base = tile_base + tiles;
    uint32_t* bin_pairs = bin_base + bins;
    hipLaunchKernelGGL(slice_prefix_kernel, dim3((bins + 63) / 64), dim3(256), 0, s, matrix, groups, bins, bin_pairs,
                       blocks, (uint32_t*)nullptr, (uint32_t*)nullptr, lists);
    GS355_CHECK_LAUNCH("bin: slice prefix");
    return launch_layout<false>(bin_pairs, bin_base, bins, blocks, group_visible, groups, n_cap, header, header_copy, false, ranges,
                                lists, bin_pairs, bins, chunk_base, nullptr, s);
}

int launch_tile_scatter(const FrameArgs& f, int32_t P, const uint64_t* rects, const uint32_t* depth_bits,
                        gs355_header* header, const uint32_t* matrix, const uint32_t* group_visible, uint32_t n_cap,
                        uint32_t* tile_base, uint32_t* ranges, uint32_t* lists, uint64_t* buckets, uint64_t* coarse,
                        int levels, hipStream_t s)
{
    int per_group;
    const int groups = bin_groups(P, &per_group);
    const int T = f.grid_x * f.grid_y, bins = coarse_bins(T);
    uint32_t* tile_cursor = tile_base + T;
    const size_t coarse_lds = (size_t)bins * sizeof(uint32_t);
    int rc = allow_large_lds();
    if (rc) return rc;
    uint32_t min_keys = 0;  // pairs from which the two levels run
    bool fine = true;
    if (T <= kBinMaxTiles) {
        if (levels != 2) {
            min_keys = levels == 1 ? UINT32_MAX : kTwoLevelMinKeys;
            hipLaunchKernelGGL((scatter_kernel<0, false>), dim3(groups), dim3(kBinThreads), (size_t)T * sizeof(uint32_t), s,
                               f, P, per_group, rects, depth_bits, header, 0u, min_keys, matrix, tile_base, buckets);
            GS355_CHECK_LAUNCH("bin: scatter");
        }
        fine = levels != 1;
        if (fine) {
            hipLaunchKernelGGL((scatter_kernel<kCoarseShift, false>), dim3(groups), dim3(kBinThreads), coarse_lds, s, f, P,
                               per_group, rects, depth_bits, header, min_keys, UINT32_MAX, matrix, tile_base, coarse);
            GS355_CHECK_LAUNCH("bin: coarse scatter");
        }
    } else {
        const uint32_t* bin_base = tile_cursor;  // (replaced by the tiles' cursors once the coarse level is done)
        hipLaunchKernelGGL((scatter_kernel<kCoarseShift, true>), dim3(groups), dim3(kBinThreads), coarse_lds, s, f, P,
                           per_group, rects, depth_bits, header, 0u, UINT32_MAX, matrix, bin_base, coarse);
        GS355_CHECK_LAUNCH("bin: coarse scatter");
        uint64_t* blocks = reinterpret_cast<uint64_t*>(tile_base + 2 * (size_t)T);
        if ((rc = launch_fill_u32(tile_base, (size_t)T, 0u, s))) return rc;
        if ((rc = launch_fill_u32(reinterpret_cast<uint32_t*>(blocks), 2 * (size_t)((T + 63) / 64), 0u, s))) return rc;
        hipLaunchKernelGGL(fine_count_kernel, dim3(kFineGrid), dim3(kFineThreads), 0, s, header, bin_base, bins, T,
                           chunk_bases(tile_base, T), coarse, tile_base, blocks, lists);
        GS355_CHECK_LAUNCH("bin: fine count");
        if ((rc = launch_layout<true>(tile_base, tile_base, T, blocks, group_visible, groups, n_cap, header, nullptr, true, ranges,
                                      lists, (const uint32_t*)nullptr, 0, (uint32_t*)nullptr, nullptr, s)))
            return rc;
    }
    if (fine) {
        hipLaunchKernelGGL(fine_scatter_kernel, dim3(kFineGrid), dim3(kFineThreads), 0, s, header, min_keys, tile_base,
                           tile_cursor, T, chunk_bases(tile_base, T), coarse, buckets);
        GS355_CHECK_LAUNCH("bin: fine scatter");
    }
    return GS355_OK;
}

int launch_tile_sort(const gs355_header* header, int tiles, const uint32_t* ranges, uint32_t* lists, uint64_t* buckets,
                     uint64_t* out_keys, uint32_t* out_vals, uint32_t skip_classes, hipStream_t s)
{
    using S0 = LdsSorter<256, 4>;    // <= 1024 pairs, one workgroup per tile
    using S1 = LdsSorter<512, 4>;    // <= 2048
    using S2 = LdsSorter<1024, 5>;   // <= 5120
    using S3 = LdsSorter<1024, 10>;  // <= 10240
    static_assert(S0::kCap == kTileSortCap[0] && S1::kCap == kTileSortCap[1] && S2::kCap == kTileSortCap[2] &&
                      S3::kCap == kTileSortCap[3], "size classes out of step with the layout kernel");
    int rc;
    if ((rc = allow_large_lds())) return rc;
    const uint32_t* list0 = lists + kListHeader;
    hipLaunchKernelGGL((tile_sort_each_kernel<256, 4>), dim3(tiles), dim3(256), S0::kBytes, s, header, ranges, buckets,
                       out_keys, out_vals, skip_classes);
    GS355_CHECK_LAUNCH("tile sort: class 0");
    // A launch per larger class, a workgroup per tile: those past the end of the class's list leave at once, which
    // costs nothing measurable (sizing the launch by the list's expected length changed no kernel's time).  The
    // largest class is the exception: a workgroup of it fills a CU, so its launch is the chip's size and strides.
    // (skip_classes: bit c set = the caller expects list c to be empty; the kernel above has sorted what is on it)
    if (!(skip_classes & 1u)) {
        hipLaunchKernelGGL((tile_sort_list_kernel<512, 4, false>), dim3(tiles), dim3(512), S1::kBytes, s, header, ranges,
                           list0, lists + 0, buckets, out_keys, out_vals);
        GS355_CHECK_LAUNCH("tile sort: class 1");
    }
    if (!(skip_classes & 2u)) {
        hipLaunchKernelGGL(tile_sort_list_1024x5_kernel, dim3(tiles), dim3(1024), S2::kBytes, s, header, ranges,
                           list0 + (size_t)tiles, lists + 1, buckets, out_keys, out_vals);
        GS355_CHECK_LAUNCH("tile sort: class 2");
    }
    if (!(skip_classes & 4u)) {
        hipLaunchKernelGGL((tile_sort_list_kernel<1024, 10, true>), dim3(tiles < 256 ? tiles : 256), dim3(1024), S3::kBytes,
                           s, header, ranges, list0 + 2 * (size_t)tiles, lists + 2, buckets, out_keys, out_vals);
        GS355_CHECK_LAUNCH("tile sort: class 3");
    }
    return GS355_OK;
}

}  // namespace gs355
