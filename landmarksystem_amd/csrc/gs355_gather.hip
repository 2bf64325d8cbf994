// Row compaction for the eval-mode gather of the reference's vanilla model
// (benchmarks/nerf/origin_gs/gs_model.py:199-208): after the visibility
// prefilter the model keeps, of means3D, shs, opacity, scales and rotations (or
// colours / covariances), the rows of the visible Gaussians, in order -- five
// boolean-index operations there, one pass over all arrays here.
//
// Three launches, nothing waits for the host: every workgroup counts the
// selected rows of its run of kGatherRows rows; an exclusive scan turns the
// counts into output bases; every workgroup then lists its selected rows in
// LDS (ballot ranks, in order) and copies them array by array with
// consecutive lanes writing consecutive 16-byte (or 4-byte) units of the
// output, so the stores are whole lines and the loads are whole rows.
#include <type_traits>

#include "gs355_internal.h"

namespace gs355 {

namespace {

constexpr int kGatherThreads = 256;
constexpr int kGatherRows = 1024;  // rows per workgroup (four rounds of one row per thread)

struct GatherArrays {  // by-value kernel argument
    const char* src[GS355_GATHER_MAX_ARRAYS];
    char* dst[GS355_GATHER_MAX_ARRAYS];
    uint32_t row_bytes[GS355_GATHER_MAX_ARRAYS];
    int32_t n;
};

__global__ __launch_bounds__(kGatherThreads) void gather_count_kernel(const uint8_t* __restrict__ mask, int32_t P,
                                                                     uint32_t* __restrict__ counts)
{
    __shared__ uint32_t s_wave[kGatherThreads / 64];
    const size_t base = (size_t)blockIdx.x * kGatherRows;
    uint32_t mine = 0;
#pragma unroll
    for (int r = 0; r < kGatherRows / kGatherThreads; ++r) {
        const size_t row = base + (size_t)r * kGatherThreads + threadIdx.x;
        mine += (row < (size_t)P && mask[row] != 0) ? 1u : 0u;
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) mine += __shfl_xor(mine, d);
    if ((threadIdx.x & 63) == 0) s_wave[threadIdx.x >> 6] = mine;
    __syncthreads();
    if (threadIdx.x == 0) counts[blockIdx.x] = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
}

// copies `rows` selected rows (source row numbers in s_rows, relative to the workgroup's first row) of one array;
// kUnit = bytes per lane and step (16 when the row size allows it, else 4)
template <int kUnit>
__device__ __forceinline__ void copy_rows(const char* __restrict__ src, char* __restrict__ dst, uint32_t row_bytes,
                                          uint32_t rows, const uint16_t* s_rows)
{
    using Word = typename std::conditional<kUnit == 16, uint4, uint32_t>::type;
    const uint32_t per_row = row_bytes / kUnit;
    const uint32_t magic = (uint32_t)((0x100000000ull + per_row - 1) / per_row);  // u / per_row for u < 2^16 * per_row
    const uint32_t total = rows * per_row;
    constexpr int kInFlight = 4;
    for (uint32_t u0 = threadIdx.x; u0 < total; u0 += kGatherThreads * kInFlight) {
        Word w[kInFlight];
#pragma unroll
        for (int k = 0; k < kInFlight; ++k) {
            const uint32_t u = u0 + (uint32_t)k * kGatherThreads;
            if (u < total) {
                const uint32_t r = per_row == 1 ? u : __umulhi(u, magic);
                const uint32_t within = u - r * per_row;
                w[k] = *reinterpret_cast<const Word*>(src + (size_t)s_rows[r] * row_bytes + (size_t)within * kUnit);
            }
        }
#pragma unroll
        for (int k = 0; k < kInFlight; ++k) {
            const uint32_t u = u0 + (uint32_t)k * kGatherThreads;
            if (u < total) *reinterpret_cast<Word*>(dst + (size_t)u * kUnit) = w[k];
        }
    }
}

__global__ __launch_bounds__(kGatherThreads) void gather_rows_kernel(const uint8_t* __restrict__ mask, int32_t P,
                                                                    const uint32_t* __restrict__ bases,
                                                                    const uint32_t* __restrict__ counts,
                                                                    GatherArrays a, uint32_t* __restrict__ count_out)
{
    __shared__ uint16_t s_rows[kGatherRows];
    __shared__ uint32_t s_wave[kGatherRows / 64];
    const size_t first = (size_t)blockIdx.x * kGatherRows;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t out_base = bases[blockIdx.x];
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0 && count_out) *count_out = out_base + counts[blockIdx.x];
    // ranks in row order: round r covers rows [first + 256 r, first + 256 (r + 1)), a wavefront 64 consecutive rows
    bool sel[kGatherRows / kGatherThreads];
    uint32_t below[kGatherRows / kGatherThreads];
#pragma unroll
    for (int r = 0; r < kGatherRows / kGatherThreads; ++r) {
        const size_t row = first + (size_t)r * kGatherThreads + threadIdx.x;
        sel[r] = row < (size_t)P && mask[row] != 0;
        const uint64_t m = __ballot(sel[r]);
        below[r] = (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
        if (lane == 0) s_wave[r * (kGatherThreads / 64) + wave] = (uint32_t)__popcll(m);
    }
    __syncthreads();
    uint32_t selected = 0;
#pragma unroll
    for (int r = 0; r < kGatherRows / kGatherThreads; ++r) {
        uint32_t before = 0;
        for (int w = 0; w < r * (kGatherThreads / 64) + wave; ++w) before += s_wave[w];
        if (sel[r]) s_rows[before + below[r]] = (uint16_t)(r * kGatherThreads + threadIdx.x);
    }
    for (int w = 0; w < kGatherRows / 64; ++w) selected += s_wave[w];
    __syncthreads();
    if (selected == 0) return;
    for (int k = 0; k < a.n; ++k) {
        const uint32_t rb = a.row_bytes[k];
        const char* src = a.src[k] + first * rb;
        char* dst = a.dst[k] + (size_t)out_base * rb;
        if (((rb | (uint32_t)(uintptr_t)a.src[k] | (uint32_t)(uintptr_t)a.dst[k]) & 15u) == 0)
            copy_rows<16>(src, dst, rb, selected, s_rows);
        else
            copy_rows<4>(src, dst, rb, selected, s_rows);
    }
}

}  // namespace

size_t gather_scratch_words(int32_t P)
{
    const size_t nb = ((size_t)P + kGatherRows - 1) / kGatherRows;
    return 2 * (nb ? nb : 1) + scan_tmp_words(nb ? nb : 1);
}

int launch_gather_rows(int32_t P, const uint8_t* mask, int32_t n_arrays, const gs355_gather_array* arrays,
                       uint32_t* count_out, uint32_t* scratch, hipStream_t s)
{
    const uint32_t nb = (uint32_t)(((size_t)P + kGatherRows - 1) / kGatherRows);
    if (nb == 0) {
        if (count_out) return launch_fill_u32(count_out, 1, 0u, s);
        return GS355_OK;
    }
    uint32_t* counts = scratch;
    uint32_t* bases = scratch + nb;
    uint32_t* tmp = scratch + 2 * (size_t)nb;
    GatherArrays a = {};
    a.n = n_arrays;
    for (int k = 0; k < n_arrays; ++k) {
        a.src[k] = static_cast<const char*>(arrays[k].src);
        a.dst[k] = static_cast<char*>(arrays[k].dst);
        a.row_bytes[k] = arrays[k].row_bytes;
    }
    hipLaunchKernelGGL(gather_count_kernel, dim3(nb), dim3(kGatherThreads), 0, s, mask, P, counts);
    GS355_CHECK_LAUNCH("gather: count");
    const int rc = launch_exclusive_scan(counts, bases, nb, tmp, s);
    if (rc) return rc;
    hipLaunchKernelGGL(gather_rows_kernel, dim3(nb), dim3(kGatherThreads), 0, s, mask, P, bases, counts, a, count_out);
    GS355_CHECK_LAUNCH("gather: rows");
    return GS355_OK;
}

}  // namespace gs355
