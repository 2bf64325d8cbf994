// Host side of the gs355 C ABI: argument validation, workspace layout and the
// stage sequence of GaussianRasterizer.forward / .visible_filter (reference
// call sites: benchmarks/nerf/origin_gs/gs_model.py:211-220, 327-329).
// Validation runs before any HIP call so that error paths are testable on a
// machine without a GPU.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "gs355_internal.h"

namespace gs355 {

static thread_local char g_error[512] = "";

int set_error(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return code;
}

namespace {

constexpr size_t kAlign = 256;
constexpr uint32_t kKnownStages = GS355_STAGE_ALL | GS355_STAGE_BLEND_PLAIN | GS355_STAGE_TILE_COUNT | GS355_STAGE_TILESORT | GS355_STAGE_TILE_SCATTER |
                                  GS355_STAGE_TILE_SCATTER_TWO_LEVEL | GS355_STAGE_TILE_SCATTER_ONE_LEVEL |
                                  GS355_STAGE_TILESORT_SKIP_1 | GS355_STAGE_TILESORT_SKIP_2 | GS355_STAGE_TILESORT_SKIP_3;
constexpr uint32_t kScatterModifiers = GS355_STAGE_TILE_SCATTER_TWO_LEVEL | GS355_STAGE_TILE_SCATTER_ONE_LEVEL;
constexpr uint32_t kStageModifiers =
    kScatterModifiers | GS355_STAGE_TILESORT_SKIP_1 | GS355_STAGE_TILESORT_SKIP_2 | GS355_STAGE_TILESORT_SKIP_3;
constexpr int64_t kMaxKeys = (1ll << 32) - 1 - kSortTile;  // key slots are indexed with u32

size_t align_up(size_t v) { return (v + kAlign - 1) / kAlign * kAlign; }

int ceil_log2(uint32_t v)
{
    int b = 0;
    while ((1ull << b) < v) ++b;
    return b;
}

int check_dims(int32_t P, int64_t n_cap, int32_t W, int32_t H)
{
    if (P < 0) return set_error(GS355_EINVAL, "P must be >= 0 (got %d)", P);
    if (W <= 0 || H <= 0) return set_error(GS355_EINVAL, "image size must be positive (got %dx%d)", W, H);
    if (n_cap < 0) return set_error(GS355_EINVAL, "n_cap must be >= 0 (got %lld)", (long long)n_cap);
    if (n_cap > kMaxKeys)
        return set_error(GS355_EOVERFLOW, "n_cap %lld exceeds the 32-bit key index range (%lld)", (long long)n_cap,
                         (long long)kMaxKeys);
    const int64_t gx = (W + kTile - 1) / kTile, gy = (H + kTile - 1) / kTile;
    if (gx > 65535 || gy > 65535)
        return set_error(GS355_EOVERFLOW, "image %dx%d has more than 65535 tiles along an axis", W, H);
    if (gx * gy > (1ll << 24))
        return set_error(GS355_EOVERFLOW, "image %dx%d has more than 2^24 tiles", W, H);
    return GS355_OK;
}

int make_layout(int32_t P, int64_t n_cap, int32_t W, int32_t H, gs355_layout* L)
{
    const int rc = check_dims(P, n_cap, W, H);
    if (rc) return rc;
    const size_t tiles = (size_t)((W + kTile - 1) / kTile) * (size_t)((H + kTile - 1) / kTile);
    const size_t p = (size_t)P, n = (size_t)n_cap;
    const size_t sort_blocks = (n + kSortTile - 1) / kSortTile;
    const size_t hist_words = (size_t)kRadix * sort_blocks;
    size_t tmp_words = scan_tmp_words(p);
    if (scan_tmp_words(hist_words) > tmp_words) tmp_words = scan_tmp_words(hist_words);

    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t at = off;
        off = align_up(off + (bytes ? bytes : 1));
        return at;
    };
    std::memset(L, 0, sizeof *L);
    L->header = take(sizeof(gs355_header));
    L->records = take(p * kRecordFloats * sizeof(float));
    L->tiles_touched = take(p * sizeof(uint32_t));
    L->rects = take(p * sizeof(uint64_t));
    L->depth_bits = take(p * sizeof(uint32_t));
    L->offsets = take(p * sizeof(uint32_t));
    L->scan_tmp = take(tmp_words * sizeof(uint32_t));
    L->keys[0] = take(n * sizeof(uint64_t));
    L->keys[1] = take(n * sizeof(uint64_t));
    L->values[0] = take(n * sizeof(uint32_t));
    L->values[1] = take(n * sizeof(uint32_t));
    L->sort_hist = take(hist_words * sizeof(uint32_t));
    L->ranges = take(tiles * 2 * sizeof(uint32_t));
    L->bin_matrix = take((tiles <= (size_t)kBinMaxTilesWide ? bin_matrix_words(tiles) : 0) * sizeof(uint32_t));
    L->tile_base = take((2 * tiles + 3 * ((tiles + 63) / 64) + (tiles + kCoarseTiles - 1) / kCoarseTiles + 1) * sizeof(uint32_t));
    L->bin_visible = take((size_t)kBinMaxGroups * sizeof(uint32_t));
    L->tile_lists = take((kListHeader + 4 * tiles) * sizeof(uint32_t));
    L->total_bytes = off;
    L->sort_bits = 32 + ceil_log2((uint32_t)tiles);
    L->sort_passes = (L->sort_bits + kRadixBits - 1) / kRadixBits;
    L->unsorted_buffer = 0;
    L->sorted_buffer = L->sort_passes & 1;
    return GS355_OK;
}

int check_frame(const gs355_frame* f, bool need_colour)
{
    if (!f) return set_error(GS355_EINVAL, "frame is NULL");
    if (f->image_width <= 0 || f->image_height <= 0)
        return set_error(GS355_EINVAL, "image size must be positive (got %dx%d)", f->image_width, f->image_height);
    if (!f->viewmatrix || !f->projmatrix)
        return set_error(GS355_EINVAL, "viewmatrix / projmatrix must be device pointers to 16 floats");
    if (!(f->tanfovx > 0.0f) || !(f->tanfovy > 0.0f))
        return set_error(GS355_EINVAL, "tanfovx / tanfovy must be positive");
    if (need_colour) {
        if (!f->bg) return set_error(GS355_EINVAL, "bg must be a device pointer to 3 floats");
    }
    return GS355_OK;
}

int check_geometry_inputs(const gs355_gaussians* g)
{
    if (!g) return set_error(GS355_EINVAL, "gaussians is NULL");
    if (g->P < 0) return set_error(GS355_EINVAL, "P must be >= 0 (got %d)", g->P);
    if (g->P == 0) return GS355_OK;
    if (!g->means3D) return set_error(GS355_EINVAL, "means3D is NULL");
    const bool has_sr = g->scales != nullptr && g->rotations != nullptr;
    const bool any_sr = g->scales != nullptr || g->rotations != nullptr;
    const bool has_cov = g->cov3D_precomp != nullptr;
    if ((has_sr && has_cov) || (!has_sr && !has_cov) || (any_sr && !has_sr))
        return set_error(GS355_EINVAL, "Please provide exactly one of either scale/rotation pair or precomputed 3D covariance!");
    return GS355_OK;
}

int check_colour_inputs(const gs355_frame* f, const gs355_gaussians* g)
{
    if (g->P == 0) return GS355_OK;
    if ((g->shs != nullptr) == (g->colors_precomp != nullptr))
        return set_error(GS355_EINVAL, "Please provide excatly one of either SHs or precomputed colors!");
    if (!g->opacities) return set_error(GS355_EINVAL, "opacities is NULL");
    if (g->shs) {
        if (f->sh_degree < 0 || f->sh_degree > 3)
            return set_error(GS355_EINVAL, "sh_degree must be in [0,3] (got %d)", f->sh_degree);
        const int need = (f->sh_degree + 1) * (f->sh_degree + 1);
        if (f->sh_coeffs < need)
            return set_error(GS355_EINVAL, "shs holds %d coefficients per Gaussian, sh_degree %d needs %d", f->sh_coeffs,
                             f->sh_degree, need);
        if (!f->campos) return set_error(GS355_EINVAL, "campos must be a device pointer to 3 floats");
    }
    return GS355_OK;
}

FrameArgs make_args(const gs355_frame* f)
{
    FrameArgs a;
    a.W = f->image_width;
    a.H = f->image_height;
    a.grid_x = (a.W + kTile - 1) / kTile;
    a.grid_y = (a.H + kTile - 1) / kTile;
    a.tanfovx = f->tanfovx;
    a.tanfovy = f->tanfovy;
    a.focal_x = (float)a.W / (2.0f * f->tanfovx);
    a.focal_y = (float)a.H / (2.0f * f->tanfovy);
    a.scale_modifier = f->scale_modifier;
    a.sh_degree = f->sh_degree;
    a.sh_coeffs = f->sh_coeffs;
    a.viewmatrix = f->viewmatrix;
    a.projmatrix = f->projmatrix;
    a.campos = f->campos;
    a.bg = f->bg;
    a.p_device = nullptr;
    return a;
}

}  // namespace
}  // namespace gs355

using namespace gs355;

extern "C" {

int gs355_version(void) { return GS355_VERSION; }

const char* gs355_last_error(void) { return g_error; }

int gs355_workspace_layout(int32_t P, int64_t n_cap, int32_t width, int32_t height, gs355_layout* out)
{
    if (!out) return set_error(GS355_EINVAL, "layout output is NULL");
    return make_layout(P, n_cap, width, height, out);
}

int gs355_run(const gs355_frame* frame, const gs355_gaussians* g, void* workspace, size_t workspace_bytes,
              int64_t n_cap, const gs355_outputs* out, uint32_t stage_mask, void* stream)
{
    int rc;
    if ((stage_mask & ~kKnownStages) != 0 || (stage_mask & ~kStageModifiers) == 0 ||
        (stage_mask & kScatterModifiers) == kScatterModifiers)
        return set_error(GS355_EINVAL, "stage_mask 0x%x selects no known stage", stage_mask);
    if ((rc = check_frame(frame, true))) return rc;
    if ((rc = check_geometry_inputs(g))) return rc;
    if ((rc = check_colour_inputs(frame, g))) return rc;
    if (!out) return set_error(GS355_EINVAL, "outputs is NULL");
    if ((stage_mask & GS355_STAGE_PREPROCESS) && g->P > 0 && !out->radii)
        return set_error(GS355_EINVAL, "outputs.radii is NULL");
    if ((stage_mask & (GS355_STAGE_BLEND | GS355_STAGE_BLEND_PLAIN)) && !out->image) return set_error(GS355_EINVAL, "outputs.image is NULL");
    gs355_layout L;
    if ((rc = make_layout(g->P, n_cap, frame->image_width, frame->image_height, &L))) return rc;
    if (stage_mask & (GS355_STAGE_TILE_COUNT | GS355_STAGE_TILE_SCATTER | GS355_STAGE_TILESORT)) {
        if ((int64_t)((frame->image_width + kTile - 1) / kTile) * ((frame->image_height + kTile - 1) / kTile) > kBinMaxTilesWide)
            return set_error(GS355_EINVAL, "the tile-bucketed stages support at most %d tiles; use the classic stages",
                             kBinMaxTilesWide);
        if (g->P > kCoarseMaxGaussians)
            return set_error(GS355_EINVAL, "the tile-bucketed stages support at most %d Gaussians; use the classic stages",
                             kCoarseMaxGaussians);
    }
    if (!workspace) return set_error(GS355_EINVAL, "workspace is NULL");
    if ((reinterpret_cast<uintptr_t>(workspace) & (kAlign - 1)) != 0)
        return set_error(GS355_EINVAL, "workspace must be 256-byte aligned");
    if (workspace_bytes < L.total_bytes)
        return set_error(GS355_ENOSPC, "workspace has %zu bytes, %zu needed (P=%d, n_cap=%lld, %dx%d)", workspace_bytes,
                         L.total_bytes, g->P, (long long)n_cap, frame->image_width, frame->image_height);

    char* ws = static_cast<char*>(workspace);
    auto* header = reinterpret_cast<gs355_header*>(ws + L.header);
    auto* records = reinterpret_cast<float*>(ws + L.records);
    auto* touched = reinterpret_cast<uint32_t*>(ws + L.tiles_touched);
    auto* rects = reinterpret_cast<uint64_t*>(ws + L.rects);
    auto* depth_bits = reinterpret_cast<uint32_t*>(ws + L.depth_bits);
    auto* offsets = reinterpret_cast<uint32_t*>(ws + L.offsets);
    auto* scan_tmp = reinterpret_cast<uint32_t*>(ws + L.scan_tmp);
    uint64_t* keys[2] = {reinterpret_cast<uint64_t*>(ws + L.keys[0]), reinterpret_cast<uint64_t*>(ws + L.keys[1])};
    uint32_t* vals[2] = {reinterpret_cast<uint32_t*>(ws + L.values[0]), reinterpret_cast<uint32_t*>(ws + L.values[1])};
    auto* hist = reinterpret_cast<uint32_t*>(ws + L.sort_hist);
    auto* ranges = reinterpret_cast<uint32_t*>(ws + L.ranges);
    auto* bin_matrix = reinterpret_cast<uint32_t*>(ws + L.bin_matrix);
    auto* tile_base = reinterpret_cast<uint32_t*>(ws + L.tile_base);
    auto* bin_visible = reinterpret_cast<uint32_t*>(ws + L.bin_visible);
    auto* tile_lists = reinterpret_cast<uint32_t*>(ws + L.tile_lists);
    hipStream_t s = static_cast<hipStream_t>(stream);
    FrameArgs fa = make_args(frame);
    fa.p_device = g->P_device;
    const uint32_t cap = (uint32_t)n_cap;

    if (stage_mask & GS355_STAGE_PREPROCESS)
        if ((rc = launch_preprocess(fa, *g, false, records, touched, rects, depth_bits, out->radii, s))) return rc;
    if (stage_mask & GS355_STAGE_SCAN)
        if ((rc = launch_scan_offsets(touched, out->radii, g->P, g->P_device, offsets, scan_tmp, header,
                                      static_cast<gs355_header*>(out->header_copy), cap, s)))
            return rc;
    if (stage_mask & GS355_STAGE_DUPLICATE)
        if ((rc = launch_duplicate(fa, g->P, records, out->radii, offsets, header, keys[0], vals[0], s))) return rc;
    if (stage_mask & GS355_STAGE_SORT)
        if ((rc = launch_sort(header, cap, L.sort_passes, keys[0], keys[1], vals[0], vals[1], hist, scan_tmp, s)))
            return rc;
    if (stage_mask & GS355_STAGE_RANGES)
        if ((rc = launch_ranges(header, cap, keys[L.sorted_buffer], ranges, fa.grid_x * fa.grid_y, s))) return rc;
    // tile-bucketed path: buckets live in the buffer the sorted keys do not use
    const int tiles = fa.grid_x * fa.grid_y;
    uint64_t* buckets = keys[1 - L.sorted_buffer];
    if (stage_mask & GS355_STAGE_TILE_COUNT) {
        if ((rc = launch_tile_count(fa, g->P, rects, bin_matrix, bin_visible, s))) return rc;
        if ((rc = launch_tile_layout(g->P, bin_matrix, bin_visible, tiles, cap, header,
                                     static_cast<gs355_header*>(out->header_copy), tile_base, ranges, tile_lists,
                                     s)))
            return rc;
    }
    if (stage_mask & GS355_STAGE_TILE_SCATTER)
        // (the buffer the sorted keys will go to is free until the sort: it holds the coarse level of the scatter)
        if ((rc = launch_tile_scatter(fa, g->P, rects, depth_bits, header, bin_matrix, bin_visible, cap, tile_base, ranges,
                                      tile_lists, buckets, keys[L.sorted_buffer],
                                      (stage_mask & GS355_STAGE_TILE_SCATTER_TWO_LEVEL)   ? 2
                                      : (stage_mask & GS355_STAGE_TILE_SCATTER_ONE_LEVEL) ? 1
                                                                                          : 0,
                                      s)))
            return rc;
    if (stage_mask & GS355_STAGE_TILESORT)
        if ((rc = launch_tile_sort(header, tiles, ranges, tile_lists, buckets, keys[L.sorted_buffer],
                                   vals[L.sorted_buffer],
                                   ((stage_mask & GS355_STAGE_TILESORT_SKIP_1) ? 1u : 0u) |
                                       ((stage_mask & GS355_STAGE_TILESORT_SKIP_2) ? 2u : 0u) |
                                       ((stage_mask & GS355_STAGE_TILESORT_SKIP_3) ? 4u : 0u),
                                   s)))
            return rc;
    if (stage_mask & (GS355_STAGE_BLEND | GS355_STAGE_BLEND_PLAIN))
        if ((rc = launch_blend(fa, header, ranges, vals[L.sorted_buffer], records, out->image, out->depth, out->alpha,
                               (stage_mask & GS355_STAGE_BLEND) != 0, s)))
            return rc;
    return GS355_OK;
}

int gs355_render(const gs355_frame* frame, const gs355_gaussians* g, void* workspace, size_t workspace_bytes,
                 int64_t n_cap, const gs355_outputs* out, void* stream)
{
    return gs355_run(frame, g, workspace, workspace_bytes, n_cap, out, GS355_PIPELINE_FAST, stream);
}

int gs355_visible_filter(const gs355_frame* frame, const gs355_gaussians* g, int32_t* radii, void* stream)
{
    int rc;
    if ((rc = check_frame(frame, false))) return rc;
    if ((rc = check_geometry_inputs(g))) return rc;
    if (g->P > 0 && !radii) return set_error(GS355_EINVAL, "radii is NULL");
    if (g->P_device) return set_error(GS355_EINVAL, "visible_filter does not take a device-side Gaussian count");
    const FrameArgs fa = make_args(frame);
    return launch_preprocess(fa, *g, true, nullptr, nullptr, nullptr, nullptr, radii, static_cast<hipStream_t>(stream));
}

namespace {
struct BackwardScratch {
    size_t first_key, scan_tmp, key_grads, total;
};
BackwardScratch backward_scratch(int32_t P, int64_t n_cap)
{
    BackwardScratch b;
    size_t off = 0;
    b.first_key = off;
    off = align_up(off + (size_t)P * sizeof(uint32_t) + 4);
    b.scan_tmp = off;
    off = align_up(off + scan_tmp_words((size_t)P) * sizeof(uint32_t));
    b.key_grads = off;
    off = align_up(off + (size_t)n_cap * GS355_KEY_GRAD_FLOATS * sizeof(float) + 4);
    b.total = off;
    return b;
}
}  // namespace

int gs355_backward_scratch_bytes(int32_t P, int64_t n_cap, size_t* bytes)
{
    if (!bytes) return set_error(GS355_EINVAL, "bytes is NULL");
    if (P < 0) return set_error(GS355_EINVAL, "P must be >= 0 (got %d)", P);
    if (n_cap < 0 || n_cap > kMaxKeys) return set_error(GS355_EINVAL, "n_cap out of range (got %lld)", (long long)n_cap);
    *bytes = backward_scratch(P, n_cap).total;
    return GS355_OK;
}

int gs355_render_backward(const gs355_frame* frame, const gs355_gaussians* g, const void* workspace,
                          size_t workspace_bytes, int64_t n_cap, const gs355_backward_inputs* in, void* scratch,
                          size_t scratch_bytes, const gs355_gradients* grads, void* stream)
{
    int rc;
    if ((rc = check_frame(frame, true))) return rc;
    if ((rc = check_geometry_inputs(g))) return rc;
    if ((rc = check_colour_inputs(frame, g))) return rc;
    if (g->P_device) return set_error(GS355_EINVAL, "the backward pass does not take a device-side Gaussian count");
    if (!in) return set_error(GS355_EINVAL, "backward inputs is NULL");
    if (!grads) return set_error(GS355_EINVAL, "gradients is NULL");
    if (!in->image || !in->dL_dimage) return set_error(GS355_EINVAL, "image / dL_dimage is NULL");
    if (in->dL_ddepth && !in->depth) return set_error(GS355_EINVAL, "dL_ddepth is given but the forward depth is NULL");
    if (in->dL_dalpha && !in->alpha) return set_error(GS355_EINVAL, "dL_dalpha is given but the forward alpha is NULL");
    if (g->P > 0 && !in->radii) return set_error(GS355_EINVAL, "radii is NULL");
    if ((grads->shs && !g->shs) || (grads->colors_precomp && !g->colors_precomp) || (grads->scales && !g->scales) ||
        (grads->rotations && !g->rotations) || (grads->cov3D_precomp && !g->cov3D_precomp))
        return set_error(GS355_EINVAL, "a gradient is requested for an input that was not given");
    gs355_layout L;
    if ((rc = make_layout(g->P, n_cap, frame->image_width, frame->image_height, &L))) return rc;
    if (!workspace) return set_error(GS355_EINVAL, "workspace is NULL");
    if ((reinterpret_cast<uintptr_t>(workspace) & (kAlign - 1)) != 0)
        return set_error(GS355_EINVAL, "workspace must be 256-byte aligned");
    if (workspace_bytes < L.total_bytes)
        return set_error(GS355_ENOSPC, "workspace has %zu bytes, %zu needed (P=%d, n_cap=%lld, %dx%d)", workspace_bytes,
                         L.total_bytes, g->P, (long long)n_cap, frame->image_width, frame->image_height);
    const BackwardScratch B = backward_scratch(g->P, n_cap);
    if (g->P > 0 && !scratch) return set_error(GS355_EINVAL, "scratch is NULL");
    if ((reinterpret_cast<uintptr_t>(scratch) & (kAlign - 1)) != 0)
        return set_error(GS355_EINVAL, "scratch must be 256-byte aligned");
    if (scratch_bytes < B.total)
        return set_error(GS355_ENOSPC, "scratch has %zu bytes, %zu needed (P=%d, n_cap=%lld)", scratch_bytes, B.total,
                         g->P, (long long)n_cap);
    const char* ws = static_cast<const char*>(workspace);
    char* sc = static_cast<char*>(scratch);
    return launch_render_backward(make_args(frame), *g, reinterpret_cast<const gs355_header*>(ws + L.header),
                                  reinterpret_cast<const uint32_t*>(ws + L.ranges),
                                  reinterpret_cast<const uint32_t*>(ws + L.values[L.sorted_buffer]),
                                  reinterpret_cast<const float*>(ws + L.records),
                                  reinterpret_cast<const uint32_t*>(ws + L.tiles_touched),
                                  reinterpret_cast<const uint64_t*>(ws + L.rects), *in,
                                  reinterpret_cast<uint32_t*>(sc + B.first_key),
                                  reinterpret_cast<uint32_t*>(sc + B.scan_tmp),
                                  reinterpret_cast<float*>(sc + B.key_grads), *grads, static_cast<hipStream_t>(stream));
}

int gs355_anchor_filter(const gs355_frame* frame, const gs355_gaussians* anchors, int32_t scale_stride,
                        const gs355_anchor_lod* lod, uint8_t* lod_mask, uint8_t* visible, int32_t* radii, void* stream)
{
    int rc;
    if ((rc = check_frame(frame, false))) return rc;
    if ((rc = check_geometry_inputs(anchors))) return rc;
    if (scale_stride < 3) return set_error(GS355_EINVAL, "scale_stride must be >= 3 (got %d)", scale_stride);
    if (anchors->P_device) return set_error(GS355_EINVAL, "the anchor filter does not take a device-side count");
    if (anchors->P > 0 && !visible) return set_error(GS355_EINVAL, "visible is NULL");
    FilterArgs x;
    x.scale_stride = scale_stride;
    x.visible = visible;
    if (lod) {
        if (anchors->P > 0 && (!lod->level || !lod->extra_level))
            return set_error(GS355_EINVAL, "lod: level / extra_level is NULL");
        if (lod->rounding < 0 || lod->rounding > 2)
            return set_error(GS355_EINVAL, "lod: rounding must be 0 (floor), 1 (round) or 2 (ceil), got %d", lod->rounding);
        if (!frame->campos) return set_error(GS355_EINVAL, "lod: frame.campos must be a device pointer to 3 floats");
        if (!(lod->fork > 1.0f) || !(lod->standard_dist > 0.0f) || lod->max_level < 0)
            return set_error(GS355_EINVAL, "lod: fork must be > 1, standard_dist > 0, max_level >= 0");
        x.use_lod = 1;
        x.lod = *lod;
        x.log2_fork = (float)std::log2((double)lod->fork);
        x.lod_mask = lod_mask;
    }
    const FrameArgs fa = make_args(frame);
    return launch_anchor_filter(fa, *anchors, x, radii, static_cast<hipStream_t>(stream));
}

int gs355_gather_scratch_bytes(int32_t P, size_t* bytes)
{
    if (P < 0) return set_error(GS355_EINVAL, "P must be >= 0 (got %d)", P);
    if (!bytes) return set_error(GS355_EINVAL, "bytes is NULL");
    *bytes = gather_scratch_words(P) * sizeof(uint32_t);
    return GS355_OK;
}

int gs355_gather_rows(int32_t P, const uint8_t* mask, int32_t n_arrays, const gs355_gather_array* arrays,
                      uint32_t* count, void* scratch, size_t scratch_bytes, void* stream)
{
    if (P < 0) return set_error(GS355_EINVAL, "P must be >= 0 (got %d)", P);
    if (n_arrays < 0 || n_arrays > GS355_GATHER_MAX_ARRAYS)
        return set_error(GS355_EINVAL, "n_arrays must be in [0, %d] (got %d)", GS355_GATHER_MAX_ARRAYS, n_arrays);
    if (n_arrays > 0 && !arrays) return set_error(GS355_EINVAL, "arrays is NULL");
    for (int k = 0; k < n_arrays; ++k) {
        const gs355_gather_array& a = arrays[k];
        if (a.row_bytes == 0 || (a.row_bytes & 3u) || a.row_bytes > GS355_GATHER_MAX_ROW_BYTES)
            return set_error(GS355_EINVAL, "arrays[%d]: row_bytes must be a multiple of 4 in [4, %d] (got %u)", k,
                             GS355_GATHER_MAX_ROW_BYTES, a.row_bytes);
        if (P > 0 && (!a.src || !a.dst)) return set_error(GS355_EINVAL, "arrays[%d]: src / dst is NULL", k);
        if (((uintptr_t)a.src | (uintptr_t)a.dst) & 3u)
            return set_error(GS355_EINVAL, "arrays[%d]: src / dst must be 4-byte aligned", k);
    }
    if (P > 0 && !mask) return set_error(GS355_EINVAL, "mask is NULL");
    if (P > 0 && !scratch) return set_error(GS355_EINVAL, "scratch is NULL");
    if (((uintptr_t)scratch & 7u) || ((uintptr_t)count & 3u))
        return set_error(GS355_EINVAL, "scratch must be 8-byte aligned, count 4-byte aligned");
    const size_t need = gather_scratch_words(P) * sizeof(uint32_t);
    if (P > 0 && scratch_bytes < need)
        return set_error(GS355_ENOSPC, "gather scratch too small: %zu bytes given, %zu needed", scratch_bytes, need);
    return launch_gather_rows(P, mask, n_arrays, arrays, count, static_cast<uint32_t*>(scratch),
                              static_cast<hipStream_t>(stream));
}

}  // extern "C"
