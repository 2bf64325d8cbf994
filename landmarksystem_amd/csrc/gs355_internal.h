// Internal declarations shared by the gs355 translation units (host side).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gs355.h"

namespace gs355 {

constexpr int kTile = GS355_TILE;
constexpr int kRecordFloats = 12;  // px, py, conic xyz, opacity, r, g, b, depth, pad, pad

// radix sort geometry: 256 threads x kSortItems keys per workgroup, 8-bit digits
constexpr int kSortThreads = 256;
constexpr int kSortItems = 16;
constexpr int kSortTile = kSortThreads * kSortItems;
constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;

// tile-bucketed sort: buckets up to kTileSortCap[3] pairs are sorted in LDS; larger ones go through global memory
constexpr int kTileSortCap[4] = {1024, 2048, 5120, 10240};  // in-LDS sorter size classes (pairs per bucket)

// scan geometry: 256 threads x 16 items per workgroup
constexpr int kScanThreads = 256;
constexpr int kScanItems = 16;
constexpr int kScanTile = kScanThreads * kScanItems;

struct FrameArgs {  // by-value kernel argument
    int32_t W, H, grid_x, grid_y;
    float tanfovx, tanfovy, focal_x, focal_y, scale_modifier;
    int32_t sh_degree, sh_coeffs;
    const float* viewmatrix;
    const float* projmatrix;
    const float* campos;
    const float* bg;
    const uint32_t* p_device;  // optional device-side number of Gaussians (gs355_gaussians.P_device)
};

// Number of Gaussians a kernel processes: the host's P, or the device-side count when there is one.
__device__ __forceinline__ int effective_count(const FrameArgs& f, int P)
{
    if (!f.p_device) return P;
    const uint32_t n = *f.p_device;
    return n < (uint32_t)P ? (int)n : P;
}

// Extras of the radii-only preprocess when it serves the anchor prefilter (by-value kernel argument).
struct FilterArgs {
    int32_t scale_stride = 3;   // floats between the scale rows
    int32_t use_lod = 0;
    gs355_anchor_lod lod = {};
    float log2_fork = 1.0f;     // (float)log2((double)fork), as the reference's host-side math.log2(fork)
    uint8_t* lod_mask = nullptr;  // optional
    uint8_t* visible = nullptr;   // optional: radius > 0
};

int set_error(int code, const char* fmt, ...);

// Tile rectangle of a splat.  Only subtractions, additions and divisions by 16:
// nothing a compiler could contract, so every translation unit gets the same
// rectangle from the same (px, py, radius).
struct Rect {
    int x0, y0, x1, y1;
};

// min(grid, max(0, (int)v)) with truncation toward zero, defined for any v.
__device__ __forceinline__ int tile_clamp(float v, int grid)
{
    if (!(v > 0.0f)) return 0;
    if (v >= (float)grid) return grid;
    return (int)v;
}

__device__ __forceinline__ Rect tile_rect(float px, float py, int radius, int grid_x, int grid_y)
{
    const float r = (float)radius;
    Rect q;
    q.x0 = tile_clamp((px - r) / 16.0f, grid_x);
    q.y0 = tile_clamp((py - r) / 16.0f, grid_y);
    q.x1 = tile_clamp((px + r + 15.0f) / 16.0f, grid_x);
    q.y1 = tile_clamp((py + r + 15.0f) / 16.0f, grid_y);
    return q;
}

// Exponent of one (pixel, Gaussian) pair,  hx dx^2 + ny dx dy + hz dy^2  with hx = -conic_x / 2, ny = -conic_y,
// hz = -conic_z / 2 and (dx, dy) = centre - pixel, as two nested multiply-adds: five instructions.  The forward
// blend and the backward blend both call this, so the two passes see the same value and decide alike.
__device__ __forceinline__ float pair_exponent(float dx, float dy, float hx, float ny, float hz)
{
#pragma clang fp contract(off)
    const float u = hx * dx;
    const float v = __builtin_fmaf(ny, dy, u);
    const float w = hz * dy;
    const float z = w * dy;
    return __builtin_fmaf(dx, v, z);
}

// The hardware exp2 is monotone, so exp2(t) < 1/255 exactly when t < kAlphaCut, the smallest float whose exp2 reaches
// 1/255 (found by running v_exp_f32 over every float between -8.2 and -7.8).  The blend (forward and backward) decides
// on t = power * log2(e) + log2(opacity) and leaves the exp2 (a quarter-rate instruction) to the pairs that pass; the
// forward blend's verification variant decides on the exponential itself, and the tests hold the two to identical
// images on scenes full of opacities around 1/255.
constexpr float kAlphaCut = -7.99435329f;  // bits 0xc0ffd1be

// stage launchers (each returns a gs355_status)
int launch_preprocess(const FrameArgs& f, const gs355_gaussians& g, bool radii_only, float* records,
                      uint32_t* tiles_touched, uint64_t* rects, uint32_t* depth_bits, int32_t* radii, hipStream_t s);
int launch_scan_offsets(const uint32_t* tiles_touched, const int32_t* radii, int32_t P, const uint32_t* p_device,
                        uint32_t* offsets, uint32_t* scan_tmp, gs355_header* header, gs355_header* header_copy, uint32_t n_cap, hipStream_t s);
int launch_anchor_filter(const FrameArgs& f, const gs355_gaussians& g, const FilterArgs& x, int32_t* radii, hipStream_t s);
int launch_duplicate(const FrameArgs& f, int32_t P, const float* records, const int32_t* radii,
                     const uint32_t* offsets, const gs355_header* header, uint64_t* keys, uint32_t* values,
                     hipStream_t s);
int launch_sort(const gs355_header* header, uint32_t n_cap, int passes, uint64_t* keys0, uint64_t* keys1,
                uint32_t* vals0, uint32_t* vals1, uint32_t* hist, uint32_t* scan_tmp, hipStream_t s);
int launch_ranges(const gs355_header* header, uint32_t n_cap, const uint64_t* keys, uint32_t* ranges, int tiles,
                  hipStream_t s);
int launch_blend(const FrameArgs& f, const gs355_header* header, const uint32_t* ranges, const uint32_t* values, const float* records,
                 float* image, float* depth, float* alpha, bool cull, hipStream_t s);

int launch_render_backward(const FrameArgs& f, const gs355_gaussians& g, const gs355_header* header,
                           const uint32_t* ranges, const uint32_t* values, const float* records,
                           const uint32_t* tiles_touched, const uint64_t* rects, const gs355_backward_inputs& in,
                           uint32_t* first_key, uint32_t* scan_tmp, float* key_grads, const gs355_gradients& out,
                           hipStream_t s);

// Number of lanes below this one that `mask` (uniform over the wavefront) holds: the hardware's masked bit count.
__device__ __forceinline__ uint32_t lanes_below_in(uint64_t mask)
{
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// Orders one wavefront's LDS writes before its later LDS reads (and the reverse).  The hardware executes a
// wavefront's LDS instructions in order; the fences (wavefront scope: no instructions) and the scheduling
// barrier keep the compiler from moving the accesses across this point.
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

int launch_fill_u32(uint32_t* p, size_t n, uint32_t v, hipStream_t s);

// tile-bucketed path
constexpr int kBinThreads = 1024;       // threads per binning workgroup
constexpr int kBinMaxGroups = 256;      // binning workgroups (each owns a contiguous slice of the Gaussians)
constexpr int kBinMaxTiles = 36000;     // counters of one workgroup that fit in LDS (4 B each)
constexpr int kCoarseShift = 4;         // the scatter's first level: bins of 16 consecutive tiles
constexpr int kCoarseTiles = 1 << kCoarseShift;
// up to kBinMaxTiles tiles a slice counts per tile; beyond, per coarse bin (tile totals counted from the bins)
constexpr int kBinMaxTilesWide = kBinMaxTiles * kCoarseTiles;
constexpr int kCoarseMaxGaussians = 1 << (32 - kCoarseShift);  // a coarse pair's index shares its word with the tile bits
int bin_groups(int32_t P, int* per_group);
// words of the slice matrix: [slices][tiles], or [slices][coarse bins] beyond kBinMaxTiles tiles
inline size_t bin_matrix_words(size_t tiles)
{
    const size_t columns = tiles <= (size_t)kBinMaxTiles ? tiles : (tiles + kCoarseTiles - 1) >> kCoarseShift;
    return (size_t)kBinMaxGroups * columns;
}
// tile_base: u32[2][tiles] (bases, then the scatter's cursors), then u64[ceil(tiles / 64)] (bases of blocks of 64 tiles),
// then u32[coarse bins + 1] (chunks of the second scatter level before each bin).  Beyond kBinMaxTiles tiles launch_tile_layout
// publishes the header and the coarse bins' bases only; ranges, lists and tile bases follow in launch_tile_scatter.
int launch_tile_count(const FrameArgs& f, int32_t P, const uint64_t* rects, uint32_t* matrix, uint32_t* group_visible,
                      hipStream_t s);
int launch_tile_layout(int32_t P, uint32_t* matrix, const uint32_t* group_visible, int tiles, uint32_t n_cap,
                       gs355_header* header, gs355_header* header_copy, uint32_t* tile_base, uint32_t* ranges, uint32_t* lists, hipStream_t s);
// `coarse`: a second buffer of the buckets' size (first level of the two-level scatter).  `levels`: 1 or 2 = that
// scatter whatever the frame holds, 0 = chosen on the device by the key count (both variants are launched); images
// beyond kBinMaxTiles tiles always take two levels
int launch_tile_scatter(const FrameArgs& f, int32_t P, const uint64_t* rects, const uint32_t* depth_bits,
                        gs355_header* header, const uint32_t* matrix, const uint32_t* group_visible, uint32_t n_cap,
                        uint32_t* tile_base, uint32_t* ranges, uint32_t* lists, uint64_t* buckets, uint64_t* coarse,
                        int levels, hipStream_t s);
// lists: u32[kListHeader + 4 * tiles]: the four class counts, four spare words, the four lists
constexpr int kListHeader = 8;
int launch_tile_sort(const gs355_header* header, int tiles, const uint32_t* ranges, uint32_t* lists,
                     uint64_t* buckets, uint64_t* out_keys, uint32_t* out_vals, uint32_t skip_classes, hipStream_t s);

// row compaction by a byte mask (gs355_gather_rows); scratch: gather_scratch_words(P) words
size_t gather_scratch_words(int32_t P);
int launch_gather_rows(int32_t P, const uint8_t* mask, int32_t n_arrays, const gs355_gather_array* arrays,
                       uint32_t* count_out, uint32_t* scratch, hipStream_t s);

// generic exclusive scan of u32 (n <= 2^32-1); tmp needs scan_tmp_words(n) words
size_t scan_tmp_words(size_t n);
int launch_exclusive_scan(const uint32_t* in, uint32_t* out, size_t n, uint32_t* tmp, hipStream_t s);

#define GS355_CHECK_LAUNCH(what)                                                        \
    do {                                                                                \
        hipError_t e__ = hipGetLastError();                                             \
        if (e__ != hipSuccess) return set_error(GS355_EHIP, "%s: %s", what, hipGetErrorString(e__)); \
    } while (0)

}  // namespace gs355
