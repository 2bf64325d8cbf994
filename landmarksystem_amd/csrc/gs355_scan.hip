// Prefix sums for gfx950: the inclusive scan of tiles_touched that gives every
// Gaussian its slot range in the key list (the scan stage of the rasterizer
// behind GaussianRasterizer.forward, benchmarks/nerf/origin_gs/gs_model.py:
// 211-220), and the exclusive scan of the radix sort's digit histograms.
//
// Reduce-then-scan in three launches (tile sums, one workgroup over the tile
// sums, rescan with the tile prefix).  No workgroup ever waits on another, so
// the grid always drains.
#include "gs355_internal.h"

namespace gs355 {

namespace {

__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v)
{
    const int lane = __lane_id();
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = __shfl_up(v, d, 64);
        if (lane >= d) v += up;
    }
    return v;
}

__device__ __forceinline__ uint64_t wave_inclusive_scan64(uint64_t v)
{
    const int lane = __lane_id();
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint64_t up = __shfl_up(v, d, 64);
        if (lane >= d) v += up;
    }
    return v;
}

// Inclusive scan over the 256 threads of a workgroup; returns this thread's
// inclusive value and the workgroup total.
__device__ __forceinline__ uint32_t block_inclusive_scan(uint32_t v, uint32_t* s_wave /*[4]*/, uint32_t& total)
{
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint32_t inc = wave_inclusive_scan(v);
    if (lane == 63) s_wave[wave] = inc;
    __syncthreads();
    uint32_t base = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w)
        if (w < wave) base += s_wave[w];
    total = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
    __syncthreads();
    return inc + base;
}

// ---- tile sums -----------------------------------------------------------
// `n_device` (optional): device-side element count; elements at and beyond it count as zero.
template <bool kCountVisible>
__global__ __launch_bounds__(kScanThreads) void tile_sum_kernel(const uint32_t* __restrict__ in,
                                                                const int32_t* __restrict__ radii, size_t n,
                                                                const uint32_t* __restrict__ n_device,
                                                                uint64_t* __restrict__ sums,
                                                                uint32_t* __restrict__ visible)
{
    __shared__ uint64_t s_sum[4];
    __shared__ uint32_t s_vis[4];
    if (n_device && (size_t)*n_device < n) n = *n_device;
    const size_t base = (size_t)blockIdx.x * kScanTile;
    uint64_t acc = 0;
    uint32_t vis = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        const size_t j = base + (size_t)k * kScanThreads + threadIdx.x;
        if (j < n) {
            acc += in[j];
            if (kCountVisible) vis += radii[j] > 0 ? 1u : 0u;
        }
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
        acc += __shfl_down(acc, d, 64);
        vis += __shfl_down(vis, d, 64);
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        s_sum[wave] = acc;
        s_vis[wave] = vis;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        sums[blockIdx.x] = s_sum[0] + s_sum[1] + s_sum[2] + s_sum[3];
        if (kCountVisible) visible[blockIdx.x] = s_vis[0] + s_vis[1] + s_vis[2] + s_vis[3];
    }
}

// ---- one workgroup: exclusive scan of the tile sums (in place), totals -----
__global__ __launch_bounds__(256) void scan_sums_kernel(uint64_t* __restrict__ sums, const uint32_t* __restrict__ visible,
                                                        uint32_t nb, gs355_header* __restrict__ header, uint32_t n_cap,
                                                        gs355_header* __restrict__ header_copy)
{
    __shared__ uint64_t s_wave[4];
    __shared__ uint64_t s_carry;
    if (threadIdx.x == 0) s_carry = 0;
    __syncthreads();
    uint32_t vis = 0;
    for (uint32_t base = 0; base < nb; base += 256) {
        const uint32_t j = base + threadIdx.x;
        const uint64_t v = j < nb ? sums[j] : 0;
        if (header && j < nb) vis += visible[j];
        const uint64_t inc = wave_inclusive_scan64(v);
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        if (lane == 63) s_wave[wave] = inc;
        __syncthreads();
        uint64_t off = s_carry;
        for (int w = 0; w < wave; ++w) off += s_wave[w];
        if (j < nb) sums[j] = off + inc - v;
        __syncthreads();
        if (threadIdx.x == 255) s_carry = off + inc;
        __syncthreads();
    }
    if (header) {
        __shared__ uint32_t s_vis[4];
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) vis += __shfl_down(vis, d, 64);
        if ((threadIdx.x & 63) == 0) s_vis[threadIdx.x >> 6] = vis;
        __syncthreads();
        if (threadIdx.x == 0) {
            const uint64_t total = s_carry;
            header->num_keys_total = total;
            header->num_keys = total > n_cap ? n_cap : (uint32_t)total;
            header->overflow = total > n_cap ? 1u : 0u;
            header->num_visible = s_vis[0] + s_vis[1] + s_vis[2] + s_vis[3];
            header->sort_class_count[0] = header->sort_class_count[1] = header->sort_class_count[2] = 0xFFFFFFFFu;
            if (header_copy) {  // (may be host memory: plain stores, complete when the kernel is)
                header_copy->num_keys_total = total;
                header_copy->num_keys = total > n_cap ? n_cap : (uint32_t)total;
                header_copy->overflow = total > n_cap ? 1u : 0u;
                header_copy->num_visible = s_vis[0] + s_vis[1] + s_vis[2] + s_vis[3];
                header_copy->sort_class_count[0] = header_copy->sort_class_count[1] = header_copy->sort_class_count[2] =
                    0xFFFFFFFFu;
            }
        }
    }
}

// ---- rescan each tile with its prefix --------------------------------------
template <bool kInclusive>
__global__ __launch_bounds__(kScanThreads) void tile_scan_kernel(const uint32_t* in, size_t n,
                                                                 const uint32_t* __restrict__ n_device,
                                                                 const uint64_t* __restrict__ sums,
                                                                 uint32_t* out /* may alias in */)
{
    __shared__ uint32_t s_wave[4];
    if (n_device && (size_t)*n_device < n) n = *n_device;
    const size_t base = (size_t)blockIdx.x * kScanTile;
    // blocked arrangement: thread t owns items [t*kScanItems, (t+1)*kScanItems)
    uint32_t v[kScanItems];
    uint32_t local = 0;
    const size_t first = base + (size_t)threadIdx.x * kScanItems;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        v[k] = first + k < n ? in[first + k] : 0u;
        local += v[k];
    }
    uint32_t total;
    const uint32_t inc = block_inclusive_scan(local, s_wave, total);
    uint32_t run = (uint32_t)sums[blockIdx.x] + (inc - local);
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        if (kInclusive) {
            run += v[k];
            if (first + k < n) out[first + k] = run;
        } else {
            if (first + k < n) out[first + k] = run;
            run += v[k];
        }
    }
}

}  // namespace

size_t scan_tmp_words(size_t n)
{
    const size_t nb = (n + kScanTile - 1) / kScanTile;
    return nb * 3 + 8;  // u64 sum + u32 visible per tile
}

int launch_scan_offsets(const uint32_t* tiles_touched, const int32_t* radii, int32_t P, const uint32_t* p_device,
                        uint32_t* offsets, uint32_t* scan_tmp, gs355_header* header, gs355_header* header_copy,
                        uint32_t n_cap, hipStream_t s)
{
    const uint32_t nb = (uint32_t)(((size_t)P + kScanTile - 1) / kScanTile);
    uint64_t* sums = reinterpret_cast<uint64_t*>(scan_tmp);
    uint32_t* visible = scan_tmp + 2 * (size_t)(nb ? nb : 1);
    if (nb) {
        hipLaunchKernelGGL(tile_sum_kernel<true>, dim3(nb), dim3(kScanThreads), 0, s, tiles_touched, radii, (size_t)P,
                           p_device, sums, visible);
        GS355_CHECK_LAUNCH("scan: tile sums");
    }
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(256), 0, s, sums, visible, nb, header, n_cap, header_copy);
    GS355_CHECK_LAUNCH("scan: sums");
    if (nb) {
        hipLaunchKernelGGL(tile_scan_kernel<true>, dim3(nb), dim3(kScanThreads), 0, s, tiles_touched, (size_t)P,
                           p_device, sums, offsets);
        GS355_CHECK_LAUNCH("scan: tiles");
    }
    return GS355_OK;
}

int launch_exclusive_scan(const uint32_t* in, uint32_t* out, size_t n, uint32_t* tmp, hipStream_t s)
{
    if (n == 0) return GS355_OK;
    const uint32_t nb = (uint32_t)((n + kScanTile - 1) / kScanTile);
    uint64_t* sums = reinterpret_cast<uint64_t*>(tmp);
    hipLaunchKernelGGL(tile_sum_kernel<false>, dim3(nb), dim3(kScanThreads), 0, s, in, (const int32_t*)nullptr, n,
                       (const uint32_t*)nullptr, sums, (uint32_t*)nullptr);
    GS355_CHECK_LAUNCH("scan: tile sums");
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(256), 0, s, sums, (const uint32_t*)nullptr, nb,
                       (gs355_header*)nullptr, 0u, (gs355_header*)nullptr);
    GS355_CHECK_LAUNCH("scan: sums");
    hipLaunchKernelGGL(tile_scan_kernel<false>, dim3(nb), dim3(kScanThreads), 0, s, in, n, (const uint32_t*)nullptr, sums,
                       out);
    GS355_CHECK_LAUNCH("scan: tiles");
    return GS355_OK;
}

}  // namespace gs355
