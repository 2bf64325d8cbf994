/*
 * gs355 -- C ABI of the MI355X (gfx950) rasterizer for 3D Gaussian splatting:
 * the forward pass, its backward pass, and the anchor decode in front of it.
 *
 * This library replaces the native extension behind the reference's Python
 * package `opt_gaussian_rasterization` (third-party CUDA submodule, empty in
 * the reference tree: .gitmodules:1-4).  The reference binds it through a
 * torch C++ extension; the entry points below are what that binding calls for
 * this path, restated as plain C:
 *
 *   GaussianRasterizer.forward(...)         -> gs355_render / gs355_run
 *       call sites: benchmarks/nerf/origin_gs/gs_model.py:211-220,
 *                   benchmarks/nerf/scaffold_gs/gs_model.py:218-227,
 *                   benchmarks/nerf/octree_gs/gs_model.py:306-315
 *   GaussianRasterizer.visible_filter(...)  -> gs355_visible_filter
 *       call sites: origin_gs/gs_model.py:327-329, scaffold_gs/gs_model.py:
 *                   432-434, octree_gs/gs_model.py:491-493
 *   ScaffoldGS / OctreeGS.prefilter_voxel   -> gs355_anchor_filter (one pass for the models' own sequence)
 *       call sites: scaffold_gs/gs_model.py:385-436, octree_gs/gs_model.py:445-497
 *   GaussianModel.forward's gather of the visible rows -> gs355_gather_rows
 *       call site:  origin_gs/gs_model.py:199-208 (five boolean-index operations)
 *   autograd backward of forward(...)       -> gs355_render_backward
 *       call site:  benchmarks/nerf/origin_gs/gs_trainer.py:117-124 (loss.backward())
 *   GaussianRasterizationSettings(...)      -> gs355_frame
 *       built at:   origin_gs/gs_model.py:148-161 (and the two siblings)
 *
 * Rules of the boundary
 *   - extern "C", plain pointers and sizes; no torch, pybind or C++ types.
 *   - Every device buffer (inputs, outputs, workspace) is owned by the caller;
 *     the library allocates no device memory and keeps no pointer after return.
 *   - Work is enqueued on the stream passed in (a hipStream_t cast to void*;
 *     NULL = the default stream).  No call synchronises the device.
 *   - Return 0 on success, a negative gs355_status otherwise;
 *     gs355_last_error() gives the message of the calling thread's last error.
 *     Argument validation happens before any HIP call, so every GS355_EINVAL /
 *     GS355_ENOSPC is reachable on a machine without a GPU.
 *   - All tensors are contiguous fp32 (int32 for radii) in device memory.
 */
#ifndef GS355_H
#define GS355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GS355_VERSION 3
#define GS355_API __attribute__((visibility("default")))
#define GS355_TILE 16 /* tile edge in pixels */

typedef enum gs355_status {
    GS355_OK = 0,
    GS355_EINVAL = -1,    /* bad argument (null pointer, bad size, exclusive inputs violated) */
    GS355_ENOSPC = -2,    /* workspace smaller than gs355_workspace_layout() requires */
    GS355_EOVERFLOW = -3, /* P, the image or the key capacity exceed the 32-bit ranges the kernels index with */
    GS355_EHIP = -4       /* a HIP runtime call failed */
} gs355_status;

/* Per-frame record: the fields of GaussianRasterizationSettings.  The four
 * tensors stay where the reference keeps them (device memory, after
 * `camera.cuda()`), so no host read-back is needed per frame.  `prefiltered`
 * and `debug` of the reference's record have no effect on results and are not
 * part of the ABI. */
typedef struct gs355_frame {
    int32_t image_width, image_height;
    float tanfovx, tanfovy;
    float scale_modifier;
    int32_t sh_degree;       /* active SH degree, 0..3 */
    int32_t sh_coeffs;       /* coefficient rows M of `shs` ([P,M,3]); >= (sh_degree+1)^2 */
    const float *viewmatrix; /* device f32[16]: torch [4,4] row-major, p_view = [p,1] @ viewmatrix */
    const float *projmatrix; /* device f32[16]: p_hom = [p,1] @ projmatrix */
    const float *campos;     /* device f32[3] */
    const float *bg;         /* device f32[3] */
} gs355_frame;

/* Inputs of forward(): exactly one of shs / colors_precomp, exactly one of
 * (scales, rotations) / cov3D_precomp. */
typedef struct gs355_gaussians {
    int32_t P;
    const float *means3D;        /* [P,3] */
    const float *shs;            /* [P,M,3] or NULL */
    const float *colors_precomp; /* [P,3] or NULL */
    const float *opacities;      /* [P] ([P,1] contiguous) */
    const float *scales;         /* [P,3] or NULL */
    const float *rotations;      /* [P,4] (r,x,y,z) or NULL */
    const float *cov3D_precomp;  /* [P,6] (xx,xy,xz,yy,yz,zz) or NULL */
    /* Optional (NULL = unused): device u32 holding the number of Gaussians when only the device knows it (the
     * output of gs355_decode).  The kernels then process min(P, *P_device) Gaussians, read when they run; P is the
     * capacity the arrays are sized for and launches are sized by.  radii[i] is not written for i >= *P_device.
     * Forward rendering only (gs355_run / gs355_render). */
    const uint32_t *P_device;
} gs355_gaussians;

/* Outputs of forward().  image and radii are required for a full render;
 * depth and alpha may be NULL. */
typedef struct gs355_outputs {
    float *image;   /* [3,H,W] */
    float *depth;   /* [H,W]  sum of depth * alpha * T, or NULL */
    float *alpha;   /* [H,W]  1 - T_final, or NULL */
    int32_t *radii; /* [P] */
    /* Optional (NULL = unused): where the stage that writes the workspace header (scan or tile count) stores a
     * second copy of its 64 bytes.  Pinned host memory is fine (the GPU addresses it like its own): the caller
     * then learns the key count and the overflow flag by waiting for that stage, without enqueuing a copy. */
    void *header_copy;
} gs355_outputs;

/* Words of the workspace header (u32 unless noted), written by the scan stage (classic pipeline) or the
 * tile-count stage (fast pipeline). */
typedef struct gs355_header {
    uint64_t num_keys_total; /* exact number of (tile, Gaussian) keys the frame needs */
    uint32_t num_keys;       /* min(num_keys_total, key capacity): what later stages process */
    uint32_t overflow;       /* 1 if num_keys_total > key capacity (the frame must be redone with more) */
    uint32_t num_visible;    /* Gaussians with radius > 0 */
    /* Tile-count stage, images of at most 36000 tiles: buckets in each of the three larger sorter size classes
     * (1025..2048, 2049..5120, 5121..10240 pairs); 0xFFFFFFFF = not counted (scan stage, larger images).  What a
     * caller needs to choose GS355_STAGE_TILESORT_SKIP_* for the next frame. */
    uint32_t sort_class_count[3];
    uint32_t reserved[8];
} gs355_header;

/* Byte offsets of every array inside the caller's workspace (each 256-byte
 * aligned).  Tests read intermediates through these. */
typedef struct gs355_layout {
    size_t header;        /* gs355_header */
    size_t records;       /* f32[P][12]: px, py, conic_x, conic_y, conic_z, opacity, r, g, b, depth, reach_x, reach_y */
    size_t tiles_touched; /* u32[P] */
    size_t rects;         /* u16[P][4] tile rectangle (x0, y0, x1, y1), all zero when culled */
    size_t depth_bits;    /* u32[P]    view depth as raw bits (written for survivors only) */
    size_t offsets;       /* u32[P]   inclusive prefix sum of tiles_touched */
    size_t scan_tmp;      /* u32[...] block sums of the scans */
    size_t keys[2];       /* u64[n_cap] x 2 (ping-pong) */
    size_t values[2];     /* u32[n_cap] x 2 */
    size_t sort_hist;     /* u32[...] per-block digit histograms of the radix sort */
    size_t ranges;        /* u32[tiles][2] */
    size_t bin_matrix;    /* u32[slices][tiles] pairs per (slice of Gaussians, tile), then their prefix over slices;
                           * beyond 36000 tiles u32[slices][ceil(tiles/16)], per bin of 16 consecutive tiles */
    size_t tile_base;     /* u32[2][tiles]   first slot of each tile's bucket; its next free slot during the scatter;
                           * then u64[ceil(tiles/64)], the first slot of each block of 64 tiles, and
                           * u32[ceil(tiles/16)+1], the work list of the scatter's second level, and
                           * u32[ceil(tiles/64)], buckets per larger sorter size class in each block of 64 tiles */
    size_t bin_visible;   /* u32[slices]     visible Gaussians per slice */
    size_t tile_lists;    /* u32[8+4*tiles]  counts, work counters and lists of the buckets of each larger sorter size class */
    size_t total_bytes;
    int32_t unsorted_buffer; /* which keys/values buffer the duplicate stage writes (0) */
    int32_t sorted_buffer;   /* which buffer holds the sorted pairs after the sort stage */
    int32_t sort_passes;     /* radix passes the sort stage runs for this image size */
    int32_t sort_bits;       /* significant key bits: 32 + ceil(log2(tiles)) */
} gs355_layout;

/* Stages of gs355_run, in pipeline order. */
enum {
    GS355_STAGE_PREPROCESS = 1, /* per-Gaussian cull / EWA / conic / radius / colour -> records, tiles_touched, radii */
    GS355_STAGE_SCAN = 2,       /* inclusive scan of tiles_touched -> offsets, header */
    GS355_STAGE_DUPLICATE = 4,  /* (tile << 32 | depth bits, index) for each tile of each survivor */
    GS355_STAGE_SORT = 8,       /* stable LSD radix sort of the pairs by key */
    GS355_STAGE_RANGES = 16,    /* per-tile [first, last) in the sorted keys */
    GS355_STAGE_BLEND = 32,     /* front-to-back alpha blending per 16x16 tile */
    GS355_STAGE_ALL = 63, /* the six stages above: the classic pipeline */
    /* Verification variant of the blend stage: every staged Gaussian is evaluated on every pixel of the tile
     * (no per-block culling).  Produces the same image as GS355_STAGE_BLEND; not part of GS355_STAGE_ALL. */
    GS355_STAGE_BLEND_PLAIN = 64,
    /* Tile-bucketed equivalent of SCAN + DUPLICATE + SORT + RANGES: same sorted keys, values, ranges and
     * header, far less memory traffic.
     *   TILE_COUNT    pairs per (slice of Gaussians, tile) in LDS-private counters; prefix over slices; tile
     *                 bases = ranges; header (key count, overflow, visible count).  Beyond 36000 tiles the
     *                 slices count per bin of 16 consecutive tiles, and ranges follow with TILE_SCATTER.
     *   TILE_SCATTER  (depth bits << 32 | index) pairs into their tile's bucket: straight for frames of fewer
     *                 than 6 * 2^20 pairs, through bins of 16 consecutive tiles beyond (decided on the device;
     *                 always beyond 36000 tiles).  The decision costs the launch of the variant that then does
     *                 nothing; a caller that knows the size of its frames (say from the previous frame's header)
     *                 names the variant with one of the modifiers below.  Either variant is correct for any frame.
     *   TILESORT      every bucket sorted by (depth bits, index) in LDS
     * Needs tiles <= 576000 (every 8K image and beyond) and P <= 2^28; otherwise use the classic stages. */
    GS355_STAGE_TILE_COUNT = 128,
    GS355_STAGE_TILESORT = 256,
    GS355_STAGE_TILE_SCATTER = 512,
    GS355_STAGE_TILE_SCATTER_TWO_LEVEL = 1024, /* modifier of TILE_SCATTER: through the bins whatever the key count */
    GS355_STAGE_TILE_SCATTER_ONE_LEVEL = 2048, /* modifier of TILE_SCATTER: straight into the buckets (ignored beyond 36000 tiles) */
    /* Modifiers of TILESORT: do not launch the sorter of the 2nd / 3rd / 4th size class (1025..2048, 2049..5120,
     * 5121..10240 pairs per bucket).  A launch over an empty class costs 4-6 us, and most frames leave one or more
     * classes empty (header.sort_class_count of the previous frame is a good predictor).  A hint, not a promise:
     * buckets of a skipped class are still sorted, one workgroup each through global memory -- same result, slower. */
    GS355_STAGE_TILESORT_SKIP_1 = 4096,
    GS355_STAGE_TILESORT_SKIP_2 = 8192,
    GS355_STAGE_TILESORT_SKIP_3 = 16384,
    GS355_PIPELINE_FAST = 1 | 128 | 512 | 256 | 32
};

GS355_API int gs355_version(void);
GS355_API const char *gs355_last_error(void);

/* Workspace the caller must provide for P Gaussians, a key capacity of n_cap
 * (tile, Gaussian) pairs and a width x height image. */
GS355_API int gs355_workspace_layout(int32_t P, int64_t n_cap, int32_t width, int32_t height, gs355_layout *out);

/* Run the stages selected in stage_mask (they must be run in pipeline order
 * over the same workspace; a later call may continue where an earlier one
 * stopped).  Stages after the scan read the key count from the workspace
 * header on the device, so no host synchronisation is needed between stages;
 * if header.overflow is set the results of those stages are to be discarded
 * and the frame redone with a larger n_cap. */
GS355_API int gs355_run(const gs355_frame *frame, const gs355_gaussians *g, void *workspace, size_t workspace_bytes,
              int64_t n_cap, const gs355_outputs *out, uint32_t stage_mask, void *stream);

/* The whole frame (GS355_PIPELINE_FAST): the body of GaussianRasterizer.forward. */
GS355_API int gs355_render(const gs355_frame *frame, const gs355_gaussians *g, void *workspace, size_t workspace_bytes,
                 int64_t n_cap, const gs355_outputs *out, void *stream);

/* GaussianRasterizer.visible_filter: radii only (cull, covariance, radius,
 * non-empty tile rectangle); needs no workspace.  shs/colors/opacities of
 * `g` are ignored and may be NULL. */
GS355_API int gs355_visible_filter(const gs355_frame *frame, const gs355_gaussians *g, int32_t *radii, void *stream);

/* Level-of-detail selection of Octree-GS anchors in eval mode (OctreeGSEncoding.set_anchor_mask,
 * landmark/nerf_components/model_components/fields/encodings/octreegs_encoding.py:238-264): an anchor is
 * kept when  level <= clamp(R(log2(standard_dist / dist) / log2(fork) + extra_level), 0, max_level),
 * dist = |anchor + (voxel_size / 2) / fork^level - campos| * resolution_scale, R = floor / round-half-even / ceil. */
typedef struct gs355_anchor_lod {
    const float *level;       /* f32[A] */
    const float *extra_level; /* f32[A] */
    float voxel_size, standard_dist, fork, resolution_scale;
    int32_t rounding;  /* 0 floor, 1 round, 2 ceil (the reference's dist2level) */
    int32_t max_level; /* max(level) - min(level) */
} gs355_anchor_lod;

/* The anchor-level visibility prefilter of the Scaffold-GS / Octree-GS models as one pass
 * (scaffold_gs/gs_model.py:385-436; octree_gs/gs_model.py:216-218,445-497): optional level-of-detail mask,
 * then GaussianRasterizer.visible_filter on the anchors that passed it, thresholded (> 0).  Produces what the
 * models' own sequence of calls produces, without gathering the selected anchors and scattering the result
 * back.  `anchors`: P = number of anchors, means3D, rotations and scales, of which the first three columns of
 * rows `scale_stride` floats apart are used (3 for f32[A,3], 6 for the models' f32[A,6]); cov3D_precomp instead
 * of scales / rotations is accepted as in gs355_visible_filter.  `lod` NULL: every anchor passes (Scaffold-GS).
 * Outputs: visible u8[A] (required); lod_mask u8[A] and radii i32[A] (0 for anchors outside the mask) optional. */
GS355_API int gs355_anchor_filter(const gs355_frame *frame, const gs355_gaussians *anchors, int32_t scale_stride,
                                  const gs355_anchor_lod *lod, uint8_t *lod_mask, uint8_t *visible, int32_t *radii,
                                  void *stream);

/* The eval-mode gather of the reference's vanilla model (benchmarks/nerf/origin_gs/gs_model.py:199-208: means3D,
 * shs, opacity, scales, rotations -- or override colours / covariances -- indexed by the prefilter's visible mask,
 * five boolean-index operations there) as one pass: the rows of up to GS355_GATHER_MAX_ARRAYS row-major arrays
 * whose mask byte is non-zero are copied, in order, to the front of the destination arrays (each sized for all P
 * rows, or for the number of selected rows if the caller knows it), and the number of selected rows is stored in
 * *count (device word, optional).  row_bytes: a multiple of 4, at most GS355_GATHER_MAX_ROW_BYTES; sources and
 * destinations 4-byte aligned (16-byte aligned arrays of 16-byte-multiple rows are copied 16 bytes at a time).
 * scratch: gs355_gather_scratch_bytes(P), caller-owned device memory. */
#define GS355_GATHER_MAX_ARRAYS 8
#define GS355_GATHER_MAX_ROW_BYTES 4096
typedef struct gs355_gather_array {
    const void *src; /* [P][row_bytes] */
    void *dst;       /* [>= selected rows][row_bytes] */
    uint32_t row_bytes;
} gs355_gather_array;
GS355_API int gs355_gather_scratch_bytes(int32_t P, size_t *bytes);
GS355_API int gs355_gather_rows(int32_t P, const uint8_t *mask, int32_t n_arrays, const gs355_gather_array *arrays,
                      uint32_t *count, void *scratch, size_t scratch_bytes, void *stream);

/* ---------------------------------------------------------------------------
 * Backward pass of GaussianRasterizer.forward: what autograd calls when the reference trains through the
 * rasterizer (loss.backward(), benchmarks/nerf/origin_gs/gs_trainer.py:117-124; `means2D.grad` feeds
 * densification, landmark/nerf_components/model_components/fields/encodings/gaussian_encoding.py:729-743 with
 * origin_gs/gs_model.py:129-139,225-236).  It runs over the workspace the forward pass of the same frame left
 * behind (records, sorted values, ranges: nothing else may have used that workspace in between) and the
 * forward outputs. */
#define GS355_KEY_GRAD_FLOATS 12 /* scratch floats per (tile, Gaussian) key */

typedef struct gs355_backward_inputs {
    const float *image;     /* [3,H,W] forward output */
    const float *depth;     /* [H,W]   forward output; required when dL_ddepth is given */
    const float *alpha;     /* [H,W]   forward output; required when dL_dalpha is given */
    const int32_t *radii;   /* [P]     forward output */
    const float *dL_dimage; /* [3,H,W] */
    const float *dL_ddepth; /* [H,W] or NULL */
    const float *dL_dalpha; /* [H,W] or NULL */
} gs355_backward_inputs;

/* Gradients with respect to the inputs of forward(); any pointer may be NULL (that gradient is not written).
 * Every element is written (zeros for culled Gaussians), so the buffers need no initialisation.  means2D is
 * the screen-space gradient in normalised device units (pixel-space gradient times W/2 and H/2, third
 * component 0), the convention the reference's densification thresholds are tuned for.  The gradient passes
 * through min(0.99, opacity * G) unchanged. */
typedef struct gs355_gradients {
    float *means3D;        /* [P,3] */
    float *means2D;        /* [P,3] */
    float *shs;            /* [P,M,3] */
    float *colors_precomp; /* [P,3] */
    float *opacities;      /* [P] */
    float *scales;         /* [P,3] */
    float *rotations;      /* [P,4] */
    float *cov3D_precomp;  /* [P,6] */
} gs355_gradients;

/* Bytes of scratch gs355_render_backward needs for P Gaussians and a key capacity of n_cap: one 48-byte
 * gradient record per key, and the index of each Gaussian's first record. */
GS355_API int gs355_backward_scratch_bytes(int32_t P, int64_t n_cap, size_t *bytes);

/* frame, g, workspace, workspace_bytes, n_cap: exactly what the forward call (gs355_render, or gs355_run through
 * the blend stage) was given.  Every sum is taken in a fixed order (no floating-point atomics in global memory
 * except within a tile's batch in LDS), so only the last bits may vary from run to run. */
GS355_API int gs355_render_backward(const gs355_frame *frame, const gs355_gaussians *g, const void *workspace,
                                    size_t workspace_bytes, int64_t n_cap, const gs355_backward_inputs *in,
                                    void *scratch, size_t scratch_bytes, const gs355_gradients *grads, void *stream);

/* ---------------------------------------------------------------------------
 * Anchor decode for Scaffold-GS / Octree-GS: replaces AnchorDecoder.forward
 * (landmark/nerf_components/model_components/fields/anchor_decoder.py:108-242) and the kernels of its
 * fused twin (fused_anchor_decoder.py:69-244: fusedKernels.*, FusedMatmul.simple2layer -- an empty
 * third-party submodule in the reference tree).  Supported: feat_dim 32, 1..10 offsets, the feature bank
 * (:163-177), the level input (:179-186) and the training-mode by-products (:239-242); not the appearance
 * embedding (:204-211).  Heads are indexed 0 = opacity (tanh), 1 = covariance (7 per offset), 2 = colour
 * (sigmoid). */
typedef struct gs355_decoder {
    int32_t feat_dim;    /* 32 */
    int32_t n_offsets;   /* 1..10 */
    int32_t in_dim[3];   /* 36 = [feat | view | dist], 35 = [feat | view] (the head's add_*_dist is False); with
                            add_level every head takes [feat | view | level] (36), as the reference feeds it
                            (anchor_decoder.py:181-182 drops the distance from both inputs) */
    const float *w0[3];  /* device f32[32, in_dim]   nn.Linear weight layout [out, in] */
    const float *b0[3];  /* device f32[32] */
    const float *w1[3];  /* device f32[k, 32], k = n_offsets, 7 n_offsets, 3 n_offsets */
    const float *b1[3];  /* device f32[k] */
    int32_t add_level;   /* 1: the fourth extra input of the heads is anchors.level instead of the distance */
    int32_t bank_in_dim; /* 0 = no feature bank; 3 = bank MLP on the view direction; 4 = on [view | level] */
    const float *bank_w0; /* device f32[32, bank_in_dim]  mlp_feature_bank.0.weight */
    const float *bank_b0; /* device f32[32] */
    const float *bank_w1; /* device f32[3, 32]            mlp_feature_bank.2.weight (softmax over the 3 outputs) */
    const float *bank_b1; /* device f32[3] */
    int32_t fp32_features; /* 0: anchor features are fp16-representable (what fp16 checkpoints hold) and enter the
                              matrix cores as one fp16 operand; 1: general fp32 features, carried as hi + lo fp16
                              pairs (two more matrix instructions per head). */
    int32_t fp32_weights;  /* 0: every weight (w0, w1 of the three heads) is fp16-representable and enters the matrix
                              cores as one fp16 operand; 1: general fp32 weights (what an fp32-trained state_dict.th
                              holds), carried as hi + lo fp16 pairs like the features.  Declaring fp32 weights as
                              fp16 rounds them to 11 significant bits (pre-activations then move by ~1e-3 relative). */
} gs355_decoder;

typedef struct gs355_anchors {
    int32_t A;
    const float *anchor;         /* [A,3] */
    const float *feat;           /* [A,32], 16-byte aligned */
    const float *offset;         /* [A,n_offsets,3] */
    const float *scaling;        /* [A,6] (exp-activated; 0..2 scale offsets, 3..5 scale Gaussians) */
    const uint8_t *visible_mask; /* [A] 0/1 (a torch.bool tensor) */
    const float *campos;         /* device f32[3] */
    const float *level;          /* [A] (the reference's [A,1]); required with add_level or bank_in_dim 4, else NULL */
} gs355_anchors;

typedef struct gs355_decoded {
    float *xyz;     /* [G,3] */
    float *color;   /* [G,3] */
    float *opacity; /* [G,1] */
    float *scaling; /* [G,3] */
    float *rot;     /* [G,4] */
    /* gs355_decode only, each optional (NULL = not written): */
    uint32_t *count;       /* device u32: G, the number of Gaussians the call emits (also when G > capacity) */
    uint32_t *num_visible; /* device u32: visible anchors */
    float *neural_opacity; /* [A_vis * n_offsets] tanh of every offset of the visible anchors (room for A * n) */
    uint8_t *mask;         /* [A_vis * n_offsets] opacity > 0 (room for A * n) */
} gs355_decoded;

GS355_API int gs355_decode_scratch_bytes(int32_t A, size_t *bytes);

/* Pass 1: counts[a] = offsets of anchor a with opacity > 0 (0 for invisible anchors); offsets = exclusive
 * prefix sum of counts.  G = offsets[A-1] + counts[A-1] is the number of Gaussians pass 2 emits. */
GS355_API int gs355_decode_count(const gs355_decoder *dec, const gs355_anchors *an, uint32_t *counts, uint32_t *offsets,
                       void *scratch, size_t scratch_bytes, void *stream);

/* gs355_decode_count for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same inputs, outputs and
 * results as gs355_decode_count; the scan's scratch is a fixed array inside the library (one copy per GPU,
 * 49 440 bytes, held until the process ends) instead of a caller buffer, and no allocating routine is called.
 * At most 2^24 anchors: more returns GS355_ENOSPC.  The device that owns `stream` and the buffers must be the
 * current device.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (different streams
 * or threads) race; calls on one stream are ordered.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress), so make that call outside any graph capture. */
GS355_API int gs355_decode_count_static(const gs355_decoder *dec, const gs355_anchors *an, uint32_t *counts,
                                        uint32_t *offsets, void *stream);

/* Pass 2: decode all heads and write the kept Gaussians in boolean-mask order (row-major over visible anchor,
 * offset) into outputs with room for `capacity` Gaussians.  The optional fields of `out` are ignored. */
GS355_API int gs355_decode_emit(const gs355_decoder *dec, const gs355_anchors *an, const uint32_t *offsets, int64_t capacity,
                      const gs355_decoded *out, void *stream);

/* The whole decode with nothing read back: count phase (feature bank, opacity head, kept offsets per run of
 * anchors, a one-workgroup scan over the runs) and emit phase.  The outputs have room for `capacity` Gaussians
 * (n_offsets per anchor always suffices); G stays on the device in out->count, where gs355_gaussians.P_device of
 * the rasterizer can read it.  Gaussians beyond `capacity` are not written.  `phases`: both for one call; or the
 * count phase alone (only out->count / out->num_visible are written), then -- after the caller has read G and
 * sized its outputs -- the emit phase with the same decoder, anchors and workspace, untouched in between.  With a
 * feature bank the mixed features of the visible anchors go through the workspace.  gs355_decode_count / _emit
 * above do not support the feature bank. */
enum { GS355_DECODE_COUNT = 1, GS355_DECODE_EMIT = 2, GS355_DECODE_ALL = 3 };
GS355_API int gs355_decode_workspace_bytes(int32_t A, int32_t n_offsets, int32_t with_feature_bank, size_t *bytes);
GS355_API int gs355_decode(const gs355_decoder *dec, const gs355_anchors *an, int64_t capacity, const gs355_decoded *out,
                           void *workspace, size_t workspace_bytes, uint32_t phases, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GS355_H */
