// Stable LSD radix sort of (64-bit key, 32-bit value) pairs for gfx950: the
// sort stage of the rasterizer behind GaussianRasterizer.forward
// (benchmarks/nerf/origin_gs/gs_model.py:211-220).  Keys are
// (tile_id << 32 | depth bits); only the low 32 + ceil(log2(tiles)) bits can
// differ, so ceil(bits / 8) passes of 8-bit digits are run.
//
// Per pass: per-workgroup digit histograms -> exclusive scan (digit-major,
// workgroup-minor) -> stable scatter.  A workgroup owns 4096 consecutive keys;
// each of its 4 waves owns 1024 of them and walks them 64 at a time, so loads
// are coalesced and the rank of a key inside its digit follows index order:
// wave-level match (ballots over the digit bits) ranks the 64 keys of a round,
// an LDS counter per (wave, digit) carries the rank across rounds.
// The key count is read from the workspace header on the device; workgroups
// past it contribute empty histograms and exit.
#include "gs355_internal.h"

namespace gs355 {

namespace {

constexpr int kWaves = kSortThreads / 64;
constexpr int kWaveKeys = 64 * kSortItems;

__global__ __launch_bounds__(kSortThreads) void radix_hist_kernel(const gs355_header* __restrict__ header,
                                                                  const uint64_t* __restrict__ keys, int shift,
                                                                  uint32_t* __restrict__ hist)
{
    __shared__ uint32_t s_hist[kRadix];
    const uint32_t n = header->overflow ? 0u : header->num_keys;
    const uint32_t nb = gridDim.x, b = blockIdx.x;
    s_hist[threadIdx.x] = 0;
    __syncthreads();
    const size_t base = (size_t)b * kSortTile;
    if (base < n) {
#pragma unroll
        for (int k = 0; k < kSortItems; ++k) {
            const size_t j = base + (size_t)k * kSortThreads + threadIdx.x;
            if (j < n) atomicAdd(&s_hist[(uint32_t)(keys[j] >> shift) & (kRadix - 1)], 1u);
        }
    }
    __syncthreads();
    hist[(size_t)threadIdx.x * nb + b] = s_hist[threadIdx.x];
}

__global__ __launch_bounds__(kSortThreads) void radix_scatter_kernel(const gs355_header* __restrict__ header,
                                                                     const uint64_t* __restrict__ keys_in,
                                                                     const uint32_t* __restrict__ vals_in,
                                                                     uint64_t* __restrict__ keys_out,
                                                                     uint32_t* __restrict__ vals_out, int shift,
                                                                     const uint32_t* __restrict__ hist_scanned)
{
    __shared__ uint32_t s_cnt[kWaves][kRadix];
    const uint32_t n = header->overflow ? 0u : header->num_keys;
    const uint32_t nb = gridDim.x, b = blockIdx.x;
    const size_t base = (size_t)b * kSortTile;
    if (base >= n) return;  // whole workgroup leaves together: no barrier was reached yet

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) s_cnt[w][threadIdx.x] = 0;
    __syncthreads();

    uint64_t key[kSortItems];
    uint32_t val[kSortItems];
    uint32_t rank[kSortItems];
    const size_t wbase = base + (size_t)wave * kWaveKeys;
    const uint64_t lanes_below = (1ull << lane) - 1ull;
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const size_t j = wbase + (size_t)r * 64 + lane;
        const bool valid = j < n;
        key[r] = valid ? keys_in[j] : ~0ull;
        val[r] = valid ? vals_in[j] : 0u;
    }
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const size_t j = wbase + (size_t)r * 64 + lane;
        const bool valid = j < n;
        const uint32_t d = (uint32_t)(key[r] >> shift) & (kRadix - 1);
        uint64_t peers = __ballot(valid);
#pragma unroll
        for (int bit = 0; bit < kRadixBits; ++bit) {
            const bool one = (d >> bit) & 1u;
            const uint64_t m = __ballot(one);
            peers &= one ? m : ~m;
        }
        // `peers` = valid lanes of this round holding the same digit (garbage on invalid lanes)
        uint32_t pre = 0;
        const uint32_t below = (uint32_t)__popcll(peers & lanes_below);
        if (valid) {
            const int leader = __ffsll((unsigned long long)peers) - 1;
            if (lane == leader) pre = atomicAdd(&s_cnt[wave][d], (uint32_t)__popcll(peers));
            pre = __shfl(pre, leader, 64);
        }
        rank[r] = pre + below;
    }
    __syncthreads();
    {
        // thread t = digit t: turn per-wave counts into global bases
        const uint32_t d = threadIdx.x;
        uint32_t run = hist_scanned[(size_t)d * nb + b];
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const uint32_t c = s_cnt[w][d];
            s_cnt[w][d] = run;
            run += c;
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const size_t j = wbase + (size_t)r * 64 + lane;
        if (j < n) {
            const uint32_t d = (uint32_t)(key[r] >> shift) & (kRadix - 1);
            const uint32_t pos = s_cnt[wave][d] + rank[r];
            keys_out[pos] = key[r];
            vals_out[pos] = val[r];
        }
    }
}

}  // namespace

int launch_sort(const gs355_header* header, uint32_t n_cap, int passes, uint64_t* keys0, uint64_t* keys1,
                uint32_t* vals0, uint32_t* vals1, uint32_t* hist, uint32_t* scan_tmp, hipStream_t s)
{
    if (n_cap == 0) return GS355_OK;
    const uint32_t nb = (n_cap + kSortTile - 1) / kSortTile;
    uint64_t* kin = keys0;
    uint64_t* kout = keys1;
    uint32_t* vin = vals0;
    uint32_t* vout = vals1;
    for (int p = 0; p < passes; ++p) {
        const int shift = p * kRadixBits;
        hipLaunchKernelGGL(radix_hist_kernel, dim3(nb), dim3(kSortThreads), 0, s, header, kin, shift, hist);
        GS355_CHECK_LAUNCH("sort: histogram");
        const int rc = launch_exclusive_scan(hist, hist, (size_t)kRadix * nb, scan_tmp, s);
        if (rc) return rc;
        hipLaunchKernelGGL(radix_scatter_kernel, dim3(nb), dim3(kSortThreads), 0, s, header, kin, vin, kout, vout,
                           shift, hist);
        GS355_CHECK_LAUNCH("sort: scatter");
        uint64_t* tk = kin; kin = kout; kout = tk;
        uint32_t* tv = vin; vin = vout; vout = tv;
    }
    return GS355_OK;
}

}  // namespace gs355
