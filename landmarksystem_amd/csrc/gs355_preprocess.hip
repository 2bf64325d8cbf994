// Per-Gaussian preprocess and key duplication for gfx950.
//
// Replaces the per-Gaussian stage of the rasterizer behind the reference's
// GaussianRasterizer.forward / .visible_filter (call sites:
// benchmarks/nerf/origin_gs/gs_model.py:211-220, 327-329).  The in-tree Python
// statements of two sub-steps are followed for layout and constants:
//   SH -> RGB            landmark/nerf_components/utils/sh_utils.py:24-94
//   scale/quat -> cov3D  landmark/nerf_components/utils/general_utils.py:64-102
//
// This translation unit is compiled with -ffp-contract=off: depth bits,
// radius and the tile rectangle feed the integer pipeline (keys, sort order,
// ranges), so every expression here is evaluated as unfused IEEE fp32 in the
// written order, with correctly rounded division and square root.
#include "gs355_internal.h"

namespace gs355 {

namespace {

constexpr float kShC0 = 0.28209479177387814f;
constexpr float kShC1 = 0.4886025119029199f;
constexpr float kShC2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                            -1.0925484305920792f, 0.5462742152960396f};
constexpr float kShC3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                            0.3731763325901154f, -0.4570457994644658f, 1.445305721320277f,
                            -0.5900435899266435f};

// 3D covariance, packed upper triangle, from scale and (r,x,y,z) quaternion.
__device__ __forceinline__ void covariance3d(const float* __restrict__ scale, float mod,
                                             const float* __restrict__ quat, float cov[6])
{
    const float sx = mod * scale[0], sy = mod * scale[1], sz = mod * scale[2];
    const float r = quat[0], x = quat[1], y = quat[2], z = quat[3];
    // rows of the rotation, each column scaled by its axis length
    const float l00 = (1.f - 2.f * (y * y + z * z)) * sx, l01 = (2.f * (x * y - r * z)) * sy,
                l02 = (2.f * (x * z + r * y)) * sz;
    const float l10 = (2.f * (x * y + r * z)) * sx, l11 = (1.f - 2.f * (x * x + z * z)) * sy,
                l12 = (2.f * (y * z - r * x)) * sz;
    const float l20 = (2.f * (x * z - r * y)) * sx, l21 = (2.f * (y * z + r * x)) * sy,
                l22 = (1.f - 2.f * (x * x + y * y)) * sz;
    cov[0] = (l00 * l00 + l01 * l01) + l02 * l02;
    cov[1] = (l00 * l10 + l01 * l11) + l02 * l12;
    cov[2] = (l00 * l20 + l01 * l21) + l02 * l22;
    cov[3] = (l10 * l10 + l11 * l11) + l12 * l12;
    cov[4] = (l10 * l20 + l11 * l21) + l12 * l22;
    cov[5] = (l20 * l20 + l21 * l21) + l22 * l22;
}

// Real SH basis of degree 0..3 at the unit direction (dx, dy, dz), with the
// sign of each term folded in, so that colour = sum_k basis[k] * sh[k].
// Each value is the product the closed-form expression multiplies the
// coefficient by, associated the same way ((C * a) * b).
__device__ __forceinline__ void sh_basis(int degree, float dx, float dy, float dz, float b[16])
{
    const float len = sqrtf((dx * dx + dy * dy) + dz * dz);
    dx = dx / len;
    dy = dy / len;
    dz = dz / len;
    b[0] = kShC0;
    if (degree > 0) {
        b[1] = -(kShC1 * dy);
        b[2] = kShC1 * dz;
        b[3] = -(kShC1 * dx);
        if (degree > 1) {
            const float xx = dx * dx, yy = dy * dy, zz = dz * dz;
            const float xy = dx * dy, yz = dy * dz, xz = dx * dz;
            b[4] = kShC2[0] * xy;
            b[5] = kShC2[1] * yz;
            b[6] = kShC2[2] * (2.0f * zz - xx - yy);
            b[7] = kShC2[3] * xz;
            b[8] = kShC2[4] * (xx - yy);
            if (degree > 2) {
                b[9] = kShC3[0] * dy * (3.0f * xx - yy);
                b[10] = kShC3[1] * xy * dz;
                b[11] = kShC3[2] * dy * (4.0f * zz - xx - yy);
                b[12] = kShC3[3] * dz * (2.0f * zz - 3.0f * xx - 3.0f * yy);
                b[13] = kShC3[4] * dx * (4.0f * zz - xx - yy);
                b[14] = kShC3[5] * dz * (xx - yy);
                b[15] = kShC3[6] * dx * (xx - 3.0f * yy);
            }
        }
    }
}

// res[c] += sum over coefficients k in [kFirst, kFirst + kCount) below
// `terms` of basis[k] * sh[3 * (k - kFirst) + c], added one by one in
// ascending k: `sh` points at coefficient kFirst of a [M,3] block
// (coefficient-major, RGB innermost) in global memory or in LDS.
template <int kFirst, int kCount>
__device__ __forceinline__ void sh_accumulate(int terms, const float* sh, const float b[16], float res[3])
{
#pragma unroll
    for (int k = 0; k < kCount; ++k) {
        if (kFirst + k < terms) {
#pragma unroll
            for (int c = 0; c < 3; ++c) res[c] = res[c] + b[kFirst + k] * sh[3 * k + c];
        }
    }
}

__device__ __forceinline__ void sh_finish(float res[3])
{
#pragma unroll
    for (int c = 0; c < 3; ++c) {
        const float v = res[c] + 0.5f;
        res[c] = v < 0.0f ? 0.0f : v;
    }
}

// SH blocks (16 coefficients, 192 B) are staged through LDS; the stride keeps the 16-B reads of the 64 lanes on
// distinct banks (stride = 4 mod 8 floats).
constexpr int kShStride = 52;  // floats per Gaussian in the staging area

// One wavefront fetches the SH blocks of up to 64 Gaussians with coalesced 16-B loads (twelve lanes per block)
// and each lane then evaluates the colour of its own entry from LDS.  `owner[e]` is the position of entry e's
// Gaussian within the workgroup's 256 (entries are the workgroup's surviving Gaussians, packed in order), so the
// loads touch survivors' blocks only, however few of the 256 survived.  A row of the staging area holds an
// entry's 48 coefficients and, in its 4 floats of padding, the Gaussian's position on the way in and its colour
// on the way out.
template <int kLoads>  // 16-B loads per lane: 64 * kLoads >= 12 * count
__device__ __forceinline__ void sh_colour_of_entries(float4* __restrict__ mine, const float* __restrict__ shs,
                                                     size_t group_first, const uint8_t* __restrict__ owner,
                                                     int first_entry, int count, int lane, int degree,
                                                     const float* campos)
{
    // all loads are issued before the first LDS write, so they are in flight together; slots past the last
    // entry re-read that entry (same value, same address)
    float4 v[kLoads];
    int dst[kLoads];
#pragma unroll
    for (int it = 0; it < kLoads; ++it) {
        const int q4 = it * 64 + lane;
        const int e = min(q4 / 12, count - 1), m = q4 % 12;
        const float4* __restrict__ block =
            reinterpret_cast<const float4*>(shs + (group_first + owner[first_entry + e]) * 48);
        {  // (read once per frame: a streaming load, which leaves the cache to the records the blend gathers)
            typedef float f4v __attribute__((ext_vector_type(4)));
            const f4v t = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(block) + m);
            v[it] = make_float4(t.x, t.y, t.z, t.w);
        }
        dst[it] = e * (kShStride / 4) + m;
    }
#pragma unroll
    for (int it = 0; it < kLoads; ++it) mine[dst[it]] = v[it];
    wave_lds_sync();
    if (lane < count) {
        float* __restrict__ row = reinterpret_cast<float*>(mine) + lane * kShStride;
        float b[16], rgb[3] = {0.f, 0.f, 0.f};
        sh_basis(degree, row[48] - campos[0], row[49] - campos[1], row[50] - campos[2], b);
        sh_accumulate<0, 16>((degree + 1) * (degree + 1), row, b, rgb);
        sh_finish(rgb);
#pragma unroll
        for (int c = 0; c < 3; ++c) row[48 + c] = rgb[c];
    }
}

// Octree-GS level-of-detail test of one anchor, in the reference's order of fp32 operations
// (octreegs_encoding.py:251-264).
__device__ __forceinline__ bool lod_keeps(const gs355_anchor_lod& l, float log2_fork, int i, float x, float y, float z,
                                          const float* campos)
{
    const float level = l.level[i];
    const float shift = (0.5f * l.voxel_size) / powf(l.fork, level);
    const float dx = (x + shift) - campos[0], dy = (y + shift) - campos[1], dz = (z + shift) - campos[2];
    const float dist = sqrtf((dx * dx + dy * dy) + dz * dz) * l.resolution_scale;
    const float pred = log2f(l.standard_dist / dist) / log2_fork + l.extra_level[i];
    float r = l.rounding == 0 ? floorf(pred) : l.rounding == 1 ? rintf(pred) : ceilf(pred);
    r = fminf(fmaxf(r, 0.0f), (float)l.max_level);  // NaN -> 0
    return level <= r;
}

template <bool kRadiiOnly>
__global__ __launch_bounds__(256) void preprocess_kernel(FrameArgs f, gs355_gaussians g, FilterArgs fx,
                                                         float* __restrict__ records,
                                                         uint32_t* __restrict__ tiles_touched,
                                                         uint64_t* __restrict__ rects,
                                                         uint32_t* __restrict__ depth_bits,
                                                         int32_t* __restrict__ radii)
{
    // staging area for the 16-coefficient SH blocks of each wavefront's 64 Gaussians
    __shared__ float4 s_sh[kRadiiOnly ? 1 : 4 * 64 * kShStride / 4];
    // the workgroup's surviving Gaussians, packed in order: position within the workgroup; survivors per wavefront
    __shared__ uint8_t s_owner[kRadiiOnly ? 1 : 256];
    __shared__ int s_alive[4];

    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const bool valid = i < effective_count(f, g.P);
    const float* __restrict__ V = f.viewmatrix;
    const float* __restrict__ M = f.projmatrix;

    // ---- geometry: cull, covariance, EWA projection, conic, radius, tile rectangle ----
    int radius = 0;
    uint32_t touched = 0;
    uint64_t rect_packed = 0;  // x0 | y0 << 16 | x1 << 32 | y1 << 48, zero when culled
    float x = 0.f, y = 0.f, z = 0.f, vz = 0.f, px = 0.f, py = 0.f, ca = 0.f, cc = 0.f, qx = 0.f, qy = 0.f, qz = 0.f;
    // Every per-Gaussian geometry input is requested up front, before the cull
    // decides whether it is needed: one memory latency instead of a chain of
    // dependent ones (culled Gaussians cost 28 to 32 B of extra reads).
    float cov[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, scale[3] = {0.f, 0.f, 0.f}, quat[4] = {0.f, 0.f, 0.f, 0.f};
    float opacity = 0.f;
    bool gated = false;  // anchor outside the level-of-detail mask (anchor prefilter only)
// (the per-Gaussian inputs are read once per frame: streaming loads)
#define GEO_LOAD(p) __builtin_nontemporal_load(&(p))
    if (valid) {
        x = GEO_LOAD(g.means3D[3 * (size_t)i]);
        y = GEO_LOAD(g.means3D[3 * (size_t)i + 1]);
        z = GEO_LOAD(g.means3D[3 * (size_t)i + 2]);
        if (kRadiiOnly && fx.use_lod) {
            gated = !lod_keeps(fx.lod, fx.log2_fork, i, x, y, z, f.campos);
            if (fx.lod_mask) fx.lod_mask[i] = gated ? 0 : 1;
        }
        if (g.cov3D_precomp) {
#pragma unroll
            for (int k = 0; k < 6; ++k) cov[k] = g.cov3D_precomp[6 * (size_t)i + k];
        } else {
#pragma unroll
            for (int k = 0; k < 3; ++k) scale[k] = GEO_LOAD(g.scales[(kRadiiOnly ? fx.scale_stride : 3) * (size_t)i + k]);
#pragma unroll
            for (int k = 0; k < 4; ++k) quat[k] = GEO_LOAD(g.rotations[4 * (size_t)i + k]);
        }
        if (!kRadiiOnly) opacity = GEO_LOAD(g.opacities[i]);
    }
    if (valid && !gated) do {
        const float vx = ((V[0] * x + V[4] * y) + V[8] * z) + V[12];
        const float vy = ((V[1] * x + V[5] * y) + V[9] * z) + V[13];
        vz = ((V[2] * x + V[6] * y) + V[10] * z) + V[14];
        if (vz <= 0.2f) break;  // behind or too close to the camera plane

        const float hx = ((M[0] * x + M[4] * y) + M[8] * z) + M[12];
        const float hy = ((M[1] * x + M[5] * y) + M[9] * z) + M[13];
        const float hw = ((M[3] * x + M[7] * y) + M[11] * z) + M[15];
        const float inv_w = 1.0f / (hw + 0.0000001f);
        const float ndc_x = hx * inv_w, ndc_y = hy * inv_w;

        if (!g.cov3D_precomp) covariance3d(scale, f.scale_modifier, quat, cov);

        // EWA splatting: Jacobian of the perspective projection at the
        // (frustum-clamped) view-space mean, times the world->view rotation.
        const float lim_x = 1.3f * f.tanfovx, lim_y = 1.3f * f.tanfovy;
        const float tz = vz;
        const float tx = fminf(lim_x, fmaxf(-lim_x, vx / tz)) * tz;
        const float ty = fminf(lim_y, fmaxf(-lim_y, vy / tz)) * tz;
        const float j00 = f.focal_x / tz, j02 = -(f.focal_x * tx) / (tz * tz);
        const float j11 = f.focal_y / tz, j12 = -(f.focal_y * ty) / (tz * tz);
        // a[r][k] = sum_i J[r][i] * Rwv[i][k], Rwv[i][k] = V[4k+i]
        const float a00 = j00 * V[0] + j02 * V[2], a01 = j00 * V[4] + j02 * V[6], a02 = j00 * V[8] + j02 * V[10];
        const float a10 = j11 * V[1] + j12 * V[2], a11 = j11 * V[5] + j12 * V[6], a12 = j11 * V[9] + j12 * V[10];
        // b = a * Sigma
        const float b00 = (a00 * cov[0] + a01 * cov[1]) + a02 * cov[2];
        const float b01 = (a00 * cov[1] + a01 * cov[3]) + a02 * cov[4];
        const float b02 = (a00 * cov[2] + a01 * cov[4]) + a02 * cov[5];
        const float b10 = (a10 * cov[0] + a11 * cov[1]) + a12 * cov[2];
        const float b11 = (a10 * cov[1] + a11 * cov[3]) + a12 * cov[4];
        const float b12 = (a10 * cov[2] + a11 * cov[4]) + a12 * cov[5];
        // 2D covariance b * a^T with the 0.3 px low-pass on the diagonal
        ca = ((b00 * a00 + b01 * a01) + b02 * a02) + 0.3f;
        const float cb = (b00 * a10 + b01 * a11) + b02 * a12;
        cc = ((b10 * a10 + b11 * a11) + b12 * a12) + 0.3f;

        const float det = ca * cc - cb * cb;
        if (det == 0.0f) break;
        const float det_inv = 1.0f / det;
        const float mid = 0.5f * (ca + cc);
        const float disc = sqrtf(fmaxf(0.1f, mid * mid - det));
        const float lambda1 = mid + disc, lambda2 = mid - disc;
        const float rf = ceilf(3.0f * sqrtf(fmaxf(lambda1, lambda2)));
        if (!(rf < 1073741824.0f)) break;  // non-finite or absurd footprint
        const int rad = (int)rf;

        px = ((ndc_x + 1.0f) * (float)f.W - 1.0f) * 0.5f;
        py = ((ndc_y + 1.0f) * (float)f.H - 1.0f) * 0.5f;
        const Rect q = tile_rect(px, py, rad, f.grid_x, f.grid_y);
        const int area = (q.x1 - q.x0) * (q.y1 - q.y0);
        if (area == 0) break;

        radius = rad;
        touched = (uint32_t)area;
        rect_packed = (uint64_t)q.x0 | ((uint64_t)q.y0 << 16) | ((uint64_t)q.x1 << 32) | ((uint64_t)q.y1 << 48);
        qx = cc * det_inv;
        qy = -cb * det_inv;
        qz = ca * det_inv;
    } while (false);

    if (valid && radii) __builtin_nontemporal_store(radius, &radii[i]);  // (no later stage reads radii)
    if (kRadiiOnly) {
        if (valid && fx.visible) fx.visible[i] = radius > 0 ? 1 : 0;
        return;
    }
    if (valid) {
        __builtin_nontemporal_store(touched, &tiles_touched[i]);  // (read by the classic scan and the backward pass only)
        rects[i] = rect_packed;
    }
    const bool alive = radius > 0;

    // ---- colour ----
    float rgb[3] = {0.f, 0.f, 0.f};
    if (g.colors_precomp) {
        if (alive) {
            rgb[0] = g.colors_precomp[3 * (size_t)i];
            rgb[1] = g.colors_precomp[3 * (size_t)i + 1];
            rgb[2] = g.colors_precomp[3 * (size_t)i + 2];
        }
    } else {
        // Full 192-B blocks: the survivors of the workgroup are packed (in order) and each wavefront fetches the
        // SH blocks of 64 of them with coalesced loads through LDS, so the memory system sees dense wavefronts
        // however many Gaussians were culled.  Other block sizes: every survivor fetches its own block.  Same
        // values and the same order of additions either way.
        const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        const bool packed = f.sh_coeffs == 16 && (reinterpret_cast<uintptr_t>(g.shs) & 15u) == 0;  // uniform
        if (packed) {
            const uint64_t m = __ballot(alive);
            if (lane == 0) s_alive[wave] = __popcll(m);
            __syncthreads();
            int before = 0, total = 0;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                before += w < wave ? s_alive[w] : 0;
                total += s_alive[w];
            }
            // packed entry e lives in row e of the staging area
            float* __restrict__ my_row = reinterpret_cast<float*>(s_sh) +
                                         (before + __popcll(m & ((1ull << lane) - 1ull))) * kShStride;
            if (alive) {
                s_owner[before + __popcll(m & ((1ull << lane) - 1ull))] = (uint8_t)threadIdx.x;
                my_row[48] = x;
                my_row[49] = y;
                my_row[50] = z;
            }
            __syncthreads();
            // each wavefront takes a quarter of the packed survivors (entry e sits in row e of the staging area)
            const int share = (total + 3) / 4, first_entry = wave * share;
            if (first_entry < total) {
                float4* __restrict__ rows = s_sh + first_entry * (kShStride / 4);
                const size_t group_first = (size_t)blockIdx.x * blockDim.x;
                const int count = min(share, total - first_entry);
                if (count <= 16)  // uniform: fewer survivors, fewer load rounds
                    sh_colour_of_entries<3>(rows, g.shs, group_first, s_owner, first_entry, count, lane, f.sh_degree, f.campos);
                else if (count <= 32)
                    sh_colour_of_entries<6>(rows, g.shs, group_first, s_owner, first_entry, count, lane, f.sh_degree, f.campos);
                else
                    sh_colour_of_entries<12>(rows, g.shs, group_first, s_owner, first_entry, count, lane, f.sh_degree, f.campos);
            }
            __syncthreads();
            if (alive) {
#pragma unroll
                for (int c = 0; c < 3; ++c) rgb[c] = my_row[48 + c];
            }
        } else if (alive) {
            float b[16];
            sh_basis(f.sh_degree, x - f.campos[0], y - f.campos[1], z - f.campos[2], b);
            sh_accumulate<0, 16>((f.sh_degree + 1) * (f.sh_degree + 1), g.shs + (size_t)i * f.sh_coeffs * 3, b, rgb);
            sh_finish(rgb);
        }
    }
    if (!alive) return;

    // Reach of the splat for the blend stage's per-block culling: half-extents
    // (ex, ey) of the axis-aligned box around the region where alpha can reach
    // 1/255, i.e. where 0.5 d^T Q d <= ln(255 * opacity).  The box is enlarged
    // by more than the rounding error of the blend's fp32 evaluation of the
    // exponent (bounded below by `noise`), so a pixel block outside the box is
    // certain to take the blend's `alpha < 1/255` branch on all of its pixels.
    // +inf = never cull (large or ill-conditioned splats), -inf = never visible.
    float ex, ey;
    {
        const float reach = (float)radius + 24.0f;  // |d| over every pixel of every touched tile
        const float noise = 2.4e-7f * (fabsf(qx) + fabsf(qy) + fabsf(qz)) * reach * reach;
        if (opacity != opacity || !(noise < 0.02f)) {
            ex = ey = INFINITY;
        } else if (!(opacity * 255.0f * 1.0001f >= 1.0f)) {
            ex = ey = -INFINITY;
        } else {
            const float tau = fmaxf(__logf(opacity * 255.0f), 0.0f) * 1.001f + 0.05f;
            ex = sqrtf(2.0f * tau * ca) * 1.001f + 0.01f;
            ey = sqrtf(2.0f * tau * cc) * 1.001f + 0.01f;
        }
    }

    float4* __restrict__ rec = reinterpret_cast<float4*>(records + (size_t)i * kRecordFloats);
    rec[0] = make_float4(px, py, qx, qy);
    rec[1] = make_float4(qz, opacity, rgb[0], rgb[1]);
    rec[2] = make_float4(rgb[2], vz, ex, ey);
    depth_bits[i] = __float_as_uint(vz);
}

// One workgroup expands the keys of 256 consecutive Gaussians.  Output slots
// are walked by consecutive lanes (coalesced stores); each slot finds its
// source Gaussian by binary search over the group's offsets held in LDS.
__global__ __launch_bounds__(256) void duplicate_kernel(FrameArgs f, int32_t P, const float* __restrict__ records,
                                                        const int32_t* __restrict__ radii,
                                                        const uint32_t* __restrict__ offsets,
                                                        const gs355_header* __restrict__ header,
                                                        uint64_t* __restrict__ keys, uint32_t* __restrict__ values)
{
    __shared__ uint32_t s_end[256];    // inclusive offset of each Gaussian of the group
    __shared__ uint32_t s_depth[256];  // depth bits
    __shared__ int s_x0[256], s_y0[256], s_w[256];

    if (header->overflow) return;  // capacity too small: the caller redoes the frame
    P = effective_count(f, P);
    const int t = threadIdx.x;
    const int g0 = blockIdx.x * 256;
    if (g0 >= P) return;  // uniform
    const int i = g0 + t;
    const uint32_t begin = g0 == 0 ? 0u : offsets[g0 - 1];
    uint32_t end_i = begin;
    if (i < P) {
        end_i = offsets[i];
        const int rad = radii[i];
        if (rad > 0) {
            const float* rec = records + (size_t)i * kRecordFloats;
            const Rect q = tile_rect(rec[0], rec[1], rad, f.grid_x, f.grid_y);
            s_x0[t] = q.x0;
            s_y0[t] = q.y0;
            s_w[t] = q.x1 - q.x0;
            s_depth[t] = __float_as_uint(rec[9]);
        }
    }
    s_end[t] = end_i;  // threads past P repeat `begin`, harmless: never selected
    __syncthreads();
    const int last = min(255, P - 1 - g0);
    const uint32_t end = s_end[last];

    for (uint32_t j = begin + t; j < end; j += 256) {
        // smallest k with s_end[k] > j
        int lo = 0, hi = last;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (s_end[mid] > j) hi = mid;
            else lo = mid + 1;
        }
        const uint32_t first = lo == 0 ? begin : s_end[lo - 1];
        const uint32_t local = j - first;
        const int w = s_w[lo];
        const int ty = s_y0[lo] + (int)(local / (uint32_t)w);
        const int tx = s_x0[lo] + (int)(local % (uint32_t)w);
        keys[j] = ((uint64_t)(uint32_t)(ty * f.grid_x + tx) << 32) | (uint64_t)s_depth[lo];
        values[j] = (uint32_t)(g0 + lo);
    }
}

}  // namespace

int launch_preprocess(const FrameArgs& f, const gs355_gaussians& g, bool radii_only, float* records,
                      uint32_t* tiles_touched, uint64_t* rects, uint32_t* depth_bits, int32_t* radii, hipStream_t s)
{
    if (g.P == 0) return GS355_OK;
    const dim3 block(256), grid((g.P + 255) / 256);
    const FilterArgs none;
    if (radii_only)
        hipLaunchKernelGGL(preprocess_kernel<true>, grid, block, 0, s, f, g, none, records, tiles_touched, rects,
                           depth_bits, radii);
    else
        hipLaunchKernelGGL(preprocess_kernel<false>, grid, block, 0, s, f, g, none, records, tiles_touched, rects,
                           depth_bits, radii);
    GS355_CHECK_LAUNCH("preprocess");
    return GS355_OK;
}

int launch_anchor_filter(const FrameArgs& f, const gs355_gaussians& g, const FilterArgs& x, int32_t* radii, hipStream_t s)
{
    if (g.P == 0) return GS355_OK;
    hipLaunchKernelGGL(preprocess_kernel<true>, dim3((g.P + 255) / 256), dim3(256), 0, s, f, g, x, (float*)nullptr,
                       (uint32_t*)nullptr, (uint64_t*)nullptr, (uint32_t*)nullptr, radii);
    GS355_CHECK_LAUNCH("anchor filter");
    return GS355_OK;
}

int launch_duplicate(const FrameArgs& f, int32_t P, const float* records, const int32_t* radii,
                     const uint32_t* offsets, const gs355_header* header, uint64_t* keys, uint32_t* values,
                     hipStream_t s)
{
    if (P == 0) return GS355_OK;
    hipLaunchKernelGGL(duplicate_kernel, dim3((P + 255) / 256), dim3(256), 0, s, f, P, records, radii, offsets,
                       header, keys, values);
    GS355_CHECK_LAUNCH("duplicate");
    return GS355_OK;
}

}  // namespace gs355
