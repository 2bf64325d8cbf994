/*
 * CPU oracle for the 3D-Gaussian-splatting forward rasterizer.
 *
 * THIS IS TEST INFRASTRUCTURE.  It is a scalar, plain-C restatement of the
 * algorithm behind the reference's `GaussianRasterizer.forward` /
 * `.visible_filter` (called at benchmarks/nerf/origin_gs/gs_model.py:211-220,
 * 327-329; scaffold_gs/gs_model.py:218-227, 432-434; octree_gs/gs_model.py:
 * 306-315, 491-493).  Only tests, the smoke check and the CPU-baseline leg of
 * the benchmark may link or call it; the shipped library never does.
 *
 * The rasterizer itself is a third-party CUDA package
 * (InternLandMark/OptGaussianRasterization, branch main, no pinned commit,
 * .gitmodules:1-4) whose directory is empty in the reference tree, so the
 * arithmetic below restates the published tile rasterizer of Kerbl et al. 2023
 * ("3D Gaussian Splatting for Real-Time Radiance Field Rendering") in the
 * form of the diff-gaussian-rasterization lineage that the reference's call
 * sites identify, and follows the in-tree Python statements where they exist:
 *   - SH -> RGB            landmark/nerf_components/utils/sh_utils.py:24-109
 *                          and benchmarks/nerf/origin_gs/gs_model.py:184-193
 *   - scale/quat -> cov3D  landmark/nerf_components/model_components/fields/
 *                          encodings/gaussian_encoding.py:22-38 and
 *                          landmark/nerf_components/utils/general_utils.py:53-102
 *   - matrix conventions   landmark/nerf_components/utils/graphics_utils.py:43-77
 *                          landmark/nerf_components/data/cameras.py:34-108
 *
 * Pinning status (no golden vectors exist in the reference for this path, so
 * each function is pinned by closed forms / invariants / brute force in
 * tests/test_oracle_*.py):
 *   orc_preprocess      closed forms (on-axis isotropic Gaussian, identity
 *                       quaternion, hand-computed NDC), SH textbook values,
 *                       integer brute force of the tile rectangle
 *   orc_scan            numpy.cumsum
 *   orc_duplicate_keys  integer identities on key fields
 *   orc_sort_pairs      numpy.argsort(kind="stable")
 *   orc_tile_ranges     numpy.searchsorted, partition invariant
 *   orc_blend           single-/two-Gaussian closed forms, weight-sum
 *                       invariant, independent brute-force per-pixel renderer
 * The rasterizer as a whole remains "parity unpinned" against the absent
 * third-party CUDA source: nothing in the reference holds its outputs.
 *
 * All arithmetic that feeds the integer pipeline (depth bits, radius, tile
 * rectangle) is IEEE fp32 evaluated in the written order; build with
 * -ffp-contract=off so no multiply-add is fused.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_TILE 16

typedef struct {
    int32_t image_width, image_height;
    float tanfovx, tanfovy;
    float scale_modifier;
    int32_t sh_degree;   /* active degree 0..3 */
    int32_t sh_coeffs;   /* coefficient rows per Gaussian in `shs` (M) */
    float viewmatrix[16]; /* torch [4,4] row-major; p_view = [p,1] @ viewmatrix */
    float projmatrix[16]; /* torch [4,4] row-major; p_hom  = [p,1] @ projmatrix */
    float campos[3];
    float bg[3];
} orc_frame;

typedef struct {
    int32_t P;
    const float *means3D;        /* [P,3] */
    const float *shs;            /* [P,M,3] or NULL */
    const float *colors_precomp; /* [P,3] or NULL */
    const float *opacities;      /* [P] */
    const float *scales;         /* [P,3] or NULL */
    const float *rotations;      /* [P,4] (r,x,y,z) or NULL */
    const float *cov3D_precomp;  /* [P,6] (xx,xy,xz,yy,yz,zz) or NULL */
} orc_gaussians;

int orc_set_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
    return omp_get_max_threads();
#else
    (void)n;
    return 1;
#endif
}

/* SH basis constants: landmark/nerf_components/utils/sh_utils.py:24-36 */
static const float SH_C0 = 0.28209479177387814f;
static const float SH_C1 = 0.4886025119029199f;
static const float SH_C2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                               -1.0925484305920792f, 0.5462742152960396f};
static const float SH_C3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                               0.3731763325901154f, -0.4570457994644658f, 1.445305721320277f,
                               -0.5900435899266435f};

/* cov3D from scale and quaternion: Sigma = R diag((mod*s)^2) R^T, packed
 * (xx,xy,xz,yy,yz,zz).  general_utils.py:64-102 (build_rotation,
 * build_scaling_rotation), gaussian_encoding.py:22-38 (L L^T, strip_symmetric).
 * The quaternion is used as given (not renormalised). */
void orc_cov3d(const float s_in[3], float mod, const float q[4], float out[6])
{
    float s[3] = {mod * s_in[0], mod * s_in[1], mod * s_in[2]};
    float r = q[0], x = q[1], y = q[2], z = q[3];
    float R[3][3];
    R[0][0] = 1.f - 2.f * (y * y + z * z);
    R[0][1] = 2.f * (x * y - r * z);
    R[0][2] = 2.f * (x * z + r * y);
    R[1][0] = 2.f * (x * y + r * z);
    R[1][1] = 1.f - 2.f * (x * x + z * z);
    R[1][2] = 2.f * (y * z - r * x);
    R[2][0] = 2.f * (x * z - r * y);
    R[2][1] = 2.f * (y * z + r * x);
    R[2][2] = 1.f - 2.f * (x * x + y * y);
    float L[3][3];
    for (int i = 0; i < 3; ++i)
        for (int k = 0; k < 3; ++k) L[i][k] = R[i][k] * s[k];
    int n = 0;
    for (int i = 0; i < 3; ++i)
        for (int j = i; j < 3; ++j)
            out[n++] = (L[i][0] * L[j][0] + L[i][1] * L[j][1]) + L[i][2] * L[j][2];
}

/* SH degree 0..3 to RGB: sh_utils.py:67-94 with sh laid out [M,3]
 * (coefficient-major, RGB innermost), then +0.5 and clamp at 0
 * (origin_gs/gs_model.py:192-193). */
void orc_sh_to_rgb(int deg, const float *sh, const float dir_in[3], float rgb[3])
{
    float dx = dir_in[0], dy = dir_in[1], dz = dir_in[2];
    float len = sqrtf((dx * dx + dy * dy) + dz * dz);
    float x = dx / len, y = dy / len, z = dz / len;
    for (int c = 0; c < 3; ++c) {
#define SH(k) sh[(k)*3 + c]
        float res = SH_C0 * SH(0);
        if (deg > 0) {
            res = res - SH_C1 * y * SH(1) + SH_C1 * z * SH(2) - SH_C1 * x * SH(3);
            if (deg > 1) {
                float xx = x * x, yy = y * y, zz = z * z;
                float xy = x * y, yz = y * z, xz = x * z;
                res = res + SH_C2[0] * xy * SH(4) + SH_C2[1] * yz * SH(5) +
                      SH_C2[2] * (2.0f * zz - xx - yy) * SH(6) + SH_C2[3] * xz * SH(7) +
                      SH_C2[4] * (xx - yy) * SH(8);
                if (deg > 2) {
                    res = res + SH_C3[0] * y * (3.0f * xx - yy) * SH(9) + SH_C3[1] * xy * z * SH(10) +
                          SH_C3[2] * y * (4.0f * zz - xx - yy) * SH(11) +
                          SH_C3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy) * SH(12) +
                          SH_C3[4] * x * (4.0f * zz - xx - yy) * SH(13) + SH_C3[5] * z * (xx - yy) * SH(14) +
                          SH_C3[6] * x * (xx - 3.0f * yy) * SH(15);
                }
            }
        }
#undef SH
        res += 0.5f;
        rgb[c] = res < 0.f ? 0.f : res;
    }
}

/* Tile coordinate min(grid, max(0, (int)v)) with truncation toward zero,
 * written so that values outside the int range (and NaN -> 0) are defined. */
static inline int tile_clamp(float v, int grid)
{
    if (!(v > 0.0f)) return 0;
    if (v >= (float)grid) return grid;
    return (int)v;
}

/* Tile rectangle of a splat of integer radius r centred at (px,py). */
void orc_tile_rect(float px, float py, int r, int grid_x, int grid_y, int32_t rect[4])
{
    float fr = (float)r;
    rect[0] = tile_clamp((px - fr) / 16.0f, grid_x);
    rect[1] = tile_clamp((py - fr) / 16.0f, grid_y);
    rect[2] = tile_clamp((px + fr + 15.0f) / 16.0f, grid_x);
    rect[3] = tile_clamp((py + fr + 15.0f) / 16.0f, grid_y);
}

/* One Gaussian of the per-Gaussian preprocess.  Returns the radius (0 =
 * culled).  Outputs are written only for survivors, except radius/touched. */
static int preprocess_one(const orc_frame *f, const orc_gaussians *g, int i, int radii_only,
                          float *depth, float *xy, float *conic_opacity, float *rgb,
                          int32_t *rect_out, uint32_t *touched)
{
    const float *V = f->viewmatrix, *Pm = f->projmatrix;
    float x = g->means3D[3 * i], y = g->means3D[3 * i + 1], z = g->means3D[3 * i + 2];
    float pvx = ((V[0] * x + V[4] * y) + V[8] * z) + V[12];
    float pvy = ((V[1] * x + V[5] * y) + V[9] * z) + V[13];
    float pvz = ((V[2] * x + V[6] * y) + V[10] * z) + V[14];
    if (pvz <= 0.2f) return 0;

    float phx = ((Pm[0] * x + Pm[4] * y) + Pm[8] * z) + Pm[12];
    float phy = ((Pm[1] * x + Pm[5] * y) + Pm[9] * z) + Pm[13];
    float phw = ((Pm[3] * x + Pm[7] * y) + Pm[11] * z) + Pm[15];
    float pw = 1.0f / (phw + 0.0000001f);
    float ppx = phx * pw, ppy = phy * pw;

    float S[6];
    if (g->cov3D_precomp) {
        memcpy(S, g->cov3D_precomp + 6 * (size_t)i, sizeof S);
    } else {
        orc_cov3d(g->scales + 3 * (size_t)i, f->scale_modifier, g->rotations + 4 * (size_t)i, S);
    }
    float Sg[3][3] = {{S[0], S[1], S[2]}, {S[1], S[3], S[4]}, {S[2], S[4], S[5]}};

    float W_img = (float)f->image_width, H_img = (float)f->image_height;
    float fx = W_img / (2.0f * f->tanfovx);
    float fy = H_img / (2.0f * f->tanfovy);
    float limx = 1.3f * f->tanfovx, limy = 1.3f * f->tanfovy;
    float tz = pvz;
    float txtz = pvx / tz, tytz = pvy / tz;
    float tx = fminf(limx, fmaxf(-limx, txtz)) * tz;
    float ty = fminf(limy, fmaxf(-limy, tytz)) * tz;
    float J00 = fx / tz, J02 = -(fx * tx) / (tz * tz);
    float J11 = fy / tz, J12 = -(fy * ty) / (tz * tz);
    /* world->view rotation rows: Wv[i][k] = V[k][i] */
    float A[2][3];
    for (int k = 0; k < 3; ++k) {
        A[0][k] = J00 * V[4 * k + 0] + J02 * V[4 * k + 2];
        A[1][k] = J11 * V[4 * k + 1] + J12 * V[4 * k + 2];
    }
    float B[2][3];
    for (int i2 = 0; i2 < 2; ++i2)
        for (int k = 0; k < 3; ++k)
            B[i2][k] = (A[i2][0] * Sg[0][k] + A[i2][1] * Sg[1][k]) + A[i2][2] * Sg[2][k];
    float c00 = (B[0][0] * A[0][0] + B[0][1] * A[0][1]) + B[0][2] * A[0][2];
    float c01 = (B[0][0] * A[1][0] + B[0][1] * A[1][1]) + B[0][2] * A[1][2];
    float c11 = (B[1][0] * A[1][0] + B[1][1] * A[1][1]) + B[1][2] * A[1][2];
    float a = c00 + 0.3f, b = c01, c = c11 + 0.3f;
    float det = a * c - b * b;
    if (det == 0.0f) return 0;
    float det_inv = 1.0f / det;
    float mid = 0.5f * (a + c);
    float q = sqrtf(fmaxf(0.1f, mid * mid - det));
    float l1 = mid + q, l2 = mid - q;
    float rf = ceilf(3.0f * sqrtf(fmaxf(l1, l2)));
    if (!(rf < 1073741824.0f)) return 0; /* non-finite or absurd footprint: treated as culled */
    int radius = (int)rf;
    float px = ((ppx + 1.0f) * W_img - 1.0f) * 0.5f;
    float py = ((ppy + 1.0f) * H_img - 1.0f) * 0.5f;
    int grid_x = (f->image_width + ORC_TILE - 1) / ORC_TILE;
    int grid_y = (f->image_height + ORC_TILE - 1) / ORC_TILE;
    int32_t rect[4];
    orc_tile_rect(px, py, radius, grid_x, grid_y, rect);
    int area = (rect[2] - rect[0]) * (rect[3] - rect[1]);
    if (area == 0) return 0;
    if (radii_only) return radius;

    depth[i] = pvz;
    xy[2 * i] = px;
    xy[2 * i + 1] = py;
    conic_opacity[4 * i + 0] = c * det_inv;
    conic_opacity[4 * i + 1] = -b * det_inv;
    conic_opacity[4 * i + 2] = a * det_inv;
    conic_opacity[4 * i + 3] = g->opacities[i];
    if (g->colors_precomp) {
        memcpy(rgb + 3 * (size_t)i, g->colors_precomp + 3 * (size_t)i, 3 * sizeof(float));
    } else {
        float dir[3] = {x - f->campos[0], y - f->campos[1], z - f->campos[2]};
        orc_sh_to_rgb(f->sh_degree, g->shs + (size_t)i * f->sh_coeffs * 3, dir, rgb + 3 * (size_t)i);
    }
    memcpy(rect_out + 4 * (size_t)i, rect, sizeof rect);
    *touched = (uint32_t)area;
    return radius;
}

/* Per-Gaussian preprocess over all P.  Arrays are zero-filled for culled
 * Gaussians.  rect is (min_x, min_y, max_x, max_y) in tiles. */
void orc_preprocess(const orc_frame *f, const orc_gaussians *g, float *depth, int32_t *radii, float *xy,
                    float *conic_opacity, float *rgb, int32_t *rect, uint32_t *tiles_touched)
{
    int P = g->P;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < P; ++i) {
        depth[i] = 0.f;
        xy[2 * i] = xy[2 * i + 1] = 0.f;
        for (int k = 0; k < 4; ++k) conic_opacity[4 * (size_t)i + k] = 0.f;
        for (int k = 0; k < 3; ++k) rgb[3 * (size_t)i + k] = 0.f;
        for (int k = 0; k < 4; ++k) rect[4 * (size_t)i + k] = 0;
        uint32_t t = 0;
        radii[i] = preprocess_one(f, g, i, 0, depth, xy, conic_opacity, rgb, rect, &t);
        tiles_touched[i] = t;
    }
}

/* visible_filter: radii only (cull, covariance, radius, non-empty rect). */
void orc_visible_filter(const orc_frame *f, const orc_gaussians *g, int32_t *radii)
{
    int P = g->P;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < P; ++i) radii[i] = preprocess_one(f, g, i, 1, 0, 0, 0, 0, 0, 0);
}

/* Inclusive prefix sum; returns the total as u64 (offsets wrap at 2^32). */
uint64_t orc_scan(const uint32_t *touched, int P, uint32_t *offsets)
{
    uint64_t acc = 0;
    for (int i = 0; i < P; ++i) {
        acc += touched[i];
        offsets[i] = (uint32_t)acc;
    }
    return acc;
}

/* Emit (tile<<32 | depth bits, gaussian index) for every tile of every
 * survivor's rectangle, y outer / x inner, at offsets[i-1]. */
void orc_duplicate_keys(int P, const int32_t *radii, const int32_t *rect, const float *depth,
                        const uint32_t *offsets, int grid_x, uint64_t *keys, uint32_t *values)
{
#pragma omp parallel for schedule(static)
    for (int i = 0; i < P; ++i) {
        if (radii[i] <= 0) continue;
        uint64_t off = i == 0 ? 0 : offsets[i - 1];
        uint32_t dbits;
        memcpy(&dbits, depth + i, 4);
        for (int ty = rect[4 * i + 1]; ty < rect[4 * i + 3]; ++ty)
            for (int tx = rect[4 * i + 0]; tx < rect[4 * i + 2]; ++tx) {
                uint64_t key = (uint64_t)(uint32_t)(ty * grid_x + tx);
                key <<= 32;
                key |= dbits;
                keys[off] = key;
                values[off] = (uint32_t)i;
                ++off;
            }
    }
}

/* Stable ascending sort of (key,value) by key: bottom-up merge sort. */
void orc_sort_pairs(uint64_t n, uint64_t *keys, uint32_t *values)
{
    if (n < 2) return;
    uint64_t *kb = (uint64_t *)malloc(n * sizeof *kb);
    uint32_t *vb = (uint32_t *)malloc(n * sizeof *vb);
    uint64_t *ks = keys, *kd = kb;
    uint32_t *vs = values, *vd = vb;
    for (uint64_t w = 1; w < n; w *= 2) {
#pragma omp parallel for schedule(dynamic, 16)
        for (uint64_t lo = 0; lo < n; lo += 2 * w) {
            uint64_t mid = lo + w < n ? lo + w : n, hi = lo + 2 * w < n ? lo + 2 * w : n;
            uint64_t a = lo, b = mid, o = lo;
            while (a < mid && b < hi) {
                if (ks[b] < ks[a]) { kd[o] = ks[b]; vd[o++] = vs[b++]; }
                else               { kd[o] = ks[a]; vd[o++] = vs[a++]; }
            }
            while (a < mid) { kd[o] = ks[a]; vd[o++] = vs[a++]; }
            while (b < hi)  { kd[o] = ks[b]; vd[o++] = vs[b++]; }
        }
        uint64_t *tk = ks; ks = kd; kd = tk;
        uint32_t *tv = vs; vs = vd; vd = tv;
    }
    if (ks != keys) {
        memcpy(keys, ks, n * sizeof *keys);
        memcpy(values, vs, n * sizeof *values);
    }
    free(kb);
    free(vb);
}

/* ranges[t] = [first, one-past-last) index of tile t in the sorted keys;
 * tiles without keys get (0,0). */
void orc_tile_ranges(uint64_t n, const uint64_t *keys, int tiles, uint32_t *ranges)
{
    memset(ranges, 0, (size_t)tiles * 2 * sizeof *ranges);
    for (uint64_t j = 0; j < n; ++j) {
        uint32_t t = (uint32_t)(keys[j] >> 32);
        if (j == 0) ranges[2 * t] = 0;
        else {
            uint32_t tp = (uint32_t)(keys[j - 1] >> 32);
            if (tp != t) { ranges[2 * tp + 1] = (uint32_t)j; ranges[2 * t] = (uint32_t)j; }
        }
        if (j == n - 1) ranges[2 * t + 1] = (uint32_t)n;
    }
}

/* Front-to-back alpha blending.  out_rgb [3,H,W], out_depth [H,W], out_alpha
 * [H,W].  `fragile` (optional, [H,W]) counts, per pixel (saturating at 255), the
 * discrete decisions (power>0, alpha<1/255, T(1-alpha)<1e-4) that were taken
 * within rounding distance of their threshold, so that a second implementation
 * with a different exp() or multiply-add fusion may legitimately decide
 * otherwise.  0 = every decision of the pixel is safe; each counted decision can
 * move the pixel by at most one contribution of weight 1/255 (or the 1e-4
 * remainder of a finished pixel).
 * stats (optional): [0]=evaluated (pixel,Gaussian) pairs, [1]=accepted pairs,
 * [2]=sum over tiles of 256 * (range entries consumed before every pixel of
 * the tile was finished). */
void orc_blend(const orc_frame *f, const uint32_t *ranges, const uint32_t *values, const float *xy,
               const float *conic_opacity, const float *rgb, const float *depth, float *out_rgb,
               float *out_depth, float *out_alpha, uint8_t *fragile, uint64_t *stats)
{
    int W = f->image_width, H = f->image_height;
    int grid_x = (W + ORC_TILE - 1) / ORC_TILE, grid_y = (H + ORC_TILE - 1) / ORC_TILE;
    uint64_t evaluated = 0, accepted = 0, tilework = 0;
#pragma omp parallel for schedule(dynamic, 4) reduction(+ : evaluated, accepted, tilework)
    for (int t = 0; t < grid_x * grid_y; ++t) {
        int tx0 = (t % grid_x) * ORC_TILE, ty0 = (t / grid_x) * ORC_TILE;
        uint32_t lo = ranges[2 * t], hi = ranges[2 * t + 1];
        uint32_t deepest = 0;
        for (int py = ty0; py < ty0 + ORC_TILE; ++py)
            for (int px = tx0; px < tx0 + ORC_TILE; ++px) {
                /* pixels outside the image still iterate (they keep the tile
                 * busy in the tiled kernel) but write nothing */
                int inside = px < W && py < H;
                float T = 1.f, C0 = 0.f, C1 = 0.f, C2 = 0.f, D = 0.f;
                int frag = 0;
                uint32_t j = lo;
                if (inside) {
                    for (; j < hi; ++j) {
                        uint32_t gi = values[j];
                        float dx = xy[2 * gi] - (float)px, dy = xy[2 * gi + 1] - (float)py;
                        const float *co = conic_opacity + 4 * (size_t)gi;
                        float t1 = co[0] * dx * dx, t2 = co[2] * dy * dy, t3 = co[1] * dx * dy;
                        float power = -0.5f * (t1 + t2) - t3;
                        ++evaluated;
                        if (fabsf(power) <= 1e-5f * (fabsf(t1) + fabsf(t2) + fabsf(t3))) ++frag;
                        if (power > 0.f) continue;
                        float alpha = fminf(0.99f, co[3] * expf(power));
                        /* rounding distance of alpha: the exponential's own 1e-4, plus what the exponent can
                         * move by when its three terms are summed in another order or with fused multiply-adds
                         * (4 units in the last place of the sum of their magnitudes) */
                        float slack = 1e-4f + 4.0f * 1.1920929e-7f * (fabsf(t1) + fabsf(t2) + fabsf(t3));
                        if (fabsf(alpha - 1.0f / 255.0f) < slack * (1.0f / 255.0f)) ++frag;
                        if (alpha < 1.0f / 255.0f) continue;
                        float test_T = T * (1.f - alpha);
                        if (fabsf(test_T - 0.0001f) < 1e-4f * 0.0001f) ++frag;
                        if (test_T < 0.0001f) break;
                        ++accepted;
                        C0 += rgb[3 * (size_t)gi] * alpha * T;
                        C1 += rgb[3 * (size_t)gi + 1] * alpha * T;
                        C2 += rgb[3 * (size_t)gi + 2] * alpha * T;
                        D += depth[gi] * alpha * T;
                        T = test_T;
                    }
                    size_t o = (size_t)py * W + px;
                    out_rgb[o] = C0 + T * f->bg[0];
                    out_rgb[(size_t)H * W + o] = C1 + T * f->bg[1];
                    out_rgb[2 * (size_t)H * W + o] = C2 + T * f->bg[2];
                    if (out_depth) out_depth[o] = D;
                    if (out_alpha) out_alpha[o] = 1.f - T;
                    if (fragile) fragile[o] = (uint8_t)(frag > 255 ? 255 : frag);
                    uint32_t used = (j < hi ? j + 1 : hi) - lo;
                    if (used > deepest) deepest = used;
                }
            }
        tilework += 256ull * deepest;
    }
    if (stats) { stats[0] = evaluated; stats[1] = accepted; stats[2] = tilework; }
}
