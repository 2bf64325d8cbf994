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
};

int set_error(int code, const char* fmt, ...);

// stage launchers (each returns a gs355_status)
int launch_preprocess(const FrameArgs& f, const gs355_gaussians& g, bool radii_only, float* records,
                      uint32_t* tiles_touched, int32_t* radii, hipStream_t s);
int launch_scan_offsets(const uint32_t* tiles_touched, const int32_t* radii, int32_t P, uint32_t* offsets,
                        uint32_t* scan_tmp, gs355_header* header, uint32_t n_cap, hipStream_t s);
int launch_duplicate(const FrameArgs& f, int32_t P, const float* records, const int32_t* radii,
                     const uint32_t* offsets, const gs355_header* header, uint64_t* keys, uint32_t* values,
                     hipStream_t s);
int launch_sort(const gs355_header* header, uint32_t n_cap, int passes, uint64_t* keys0, uint64_t* keys1,
                uint32_t* vals0, uint32_t* vals1, uint32_t* hist, uint32_t* scan_tmp, hipStream_t s);
int launch_ranges(const gs355_header* header, uint32_t n_cap, const uint64_t* keys, uint32_t* ranges, int tiles,
                  hipStream_t s);
int launch_blend(const FrameArgs& f, const gs355_header* header, const uint32_t* ranges, const uint32_t* values, const float* records,
                 float* image, float* depth, float* alpha, bool cull, hipStream_t s);

// generic exclusive scan of u32 (n <= 2^32-1); tmp needs scan_tmp_words(n) words
size_t scan_tmp_words(size_t n);
int launch_exclusive_scan(const uint32_t* in, uint32_t* out, size_t n, uint32_t* tmp, hipStream_t s);

#define GS355_CHECK_LAUNCH(what)                                                        \
    do {                                                                                \
        hipError_t e__ = hipGetLastError();                                             \
        if (e__ != hipSuccess) return set_error(GS355_EHIP, "%s: %s", what, hipGetErrorString(e__)); \
    } while (0)

}  // namespace gs355
