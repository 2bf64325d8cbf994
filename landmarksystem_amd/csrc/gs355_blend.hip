// Per-tile range identification and front-to-back alpha blending for gfx950:
// the last two stages of the rasterizer behind GaussianRasterizer.forward
// (benchmarks/nerf/origin_gs/gs_model.py:211-220; output consumed as a
// [3,H,W] image at tests/test_inference_framework/test_inference.py:195-197).
//
// Blending: one 256-thread workgroup per 16x16 pixel tile, each of its four
// wavefronts owning an 8x8 pixel quadrant, each group of 16 lanes a 4x4 block
// of it.  The tile's depth-sorted Gaussians are staged through LDS in batches
// of 256 records (48 B each); every 4x4 block gets its own list of the staged
// Gaussians that can reach it, and the four lane groups of a wavefront walk
// their lists side by side, so one pass of the pixel arithmetic serves four
// different Gaussians.  A wavefront stops as soon as a ballot shows all of
// its 64 pixels finished, and the workgroup stops fetching batches once all
// four wavefronts have.
#include "gs355_internal.h"

namespace gs355 {

namespace {

__global__ void fill_u32_kernel(uint32_t* __restrict__ p, size_t n, uint32_t v)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

__global__ __launch_bounds__(256) void ranges_kernel(const gs355_header* __restrict__ header,
                                                     const uint64_t* __restrict__ keys, uint32_t* __restrict__ ranges,
                                                     uint32_t tiles)
{
    if (header->overflow) return;
    const uint32_t n = header->num_keys;
    const size_t j = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    const uint32_t t = (uint32_t)(keys[j] >> 32);
    if (t >= tiles) return;  // cannot happen for keys made by the duplicate stage
    if (j == 0) {
        ranges[2 * t] = 0;
    } else {
        const uint32_t tp = (uint32_t)(keys[j - 1] >> 32);
        if (tp != t) {
            if (tp < tiles) ranges[2 * tp + 1] = (uint32_t)j;
            ranges[2 * t] = (uint32_t)j;
        }
    }
    if (j == n - 1) ranges[2 * t + 1] = n;
}

// One (pixel, Gaussian) pair: exponent, alpha, the three discrete tests and the
// accumulation.  The exponent is evaluated with unfused multiplies and adds in
// a fixed order (contraction is switched off for it), so the sign test and the
// alpha threshold see the same value as a scalar evaluation of the formula.
//
// A pixel's transmittance T stays >= 1e-4 while it is live, so the sign of T
// carries the "finished" state: T > 0 live, T <= 0 finished with |T| the final
// transmittance (pixels outside the image start at -1).  A finished pixel can
// neither accumulate (its test_T is <= 0) nor finish again.
struct PixelState {
    float T, c0, c1, c2, depth;
};

__device__ __forceinline__ float splat_exponent(float dx, float dy, float qx, float qy, float qz)
{
#pragma clang fp contract(off)
    const float t1 = (qx * dx) * dx;
    const float t2 = (qz * dy) * dy;
    const float t3 = (qy * dx) * dy;
    return -0.5f * (t1 + t2) - t3;
}

__device__ __forceinline__ void blend_one(PixelState& p, float pxf, float pyf, const float4 a, const float4 b,
                                          const float4 c)
{
    const float dx = a.x - pxf, dy = a.y - pyf;
    const float power = splat_exponent(dx, dy, a.z, a.w, b.x);
    const float alpha = fminf(0.99f, b.y * __expf(power));
    if (power > 0.0f || alpha < 1.0f / 255.0f) return;
    const float test_T = p.T * (1.0f - alpha);
    if (test_T >= 0.0001f) {
        const float w = alpha * p.T;
        p.c0 += b.z * w;
        p.c1 += b.w * w;
        p.c2 += c.x * w;
        p.depth += c.y * w;
        p.T = test_T;
    } else if (p.T > 0.0f) {
        p.T = -p.T;  // this Gaussian is not applied; the pixel is finished
    }
}

// kCull: each wavefront first tests the staged Gaussians (one per lane) against
// the four 4x4 blocks of its quadrant, using the bounding box of the
// alpha >= 1/255 region from the record, and appends the survivors, in depth
// order, to the list of each block they can reach.  A (block, Gaussian) pair
// that is left out is one whose 16 pixels would all have taken the
// `alpha < 1/255` branch, and every pixel still sees its Gaussians front to
// back with the same arithmetic, so both variants produce identical images.
template <bool kCull>
__global__ __launch_bounds__(256) void blend_kernel(FrameArgs f, const gs355_header* __restrict__ header,
                                                    const uint32_t* __restrict__ ranges,
                                                    const uint32_t* __restrict__ values,
                                                    const float* __restrict__ records, float* __restrict__ image,
                                                    float* __restrict__ out_depth, float* __restrict__ out_alpha)
{
    __shared__ float4 s_a[256];  // px, py, conic_x, conic_y
    __shared__ float4 s_b[256];  // conic_z, opacity, r, g
    __shared__ float4 s_c[256];  // b, depth, reach_x, reach_y
    __shared__ uint32_t s_wave_done[4];
    // per wavefront and 4x4 block: staged-record numbers of the Gaussians that can reach the block
    __shared__ uint8_t s_list[kCull ? 4 : 1][4][256 + 4];

    if (header->overflow) return;
    const int tile = blockIdx.x;
    const int tile_x = tile % f.grid_x, tile_y = tile / f.grid_x;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int group = lane >> 4, sub = lane & 15;  // 4x4 block within the quadrant, pixel within the block
    const int qx0 = tile_x * kTile + (wave & 1) * 8, qy0 = tile_y * kTile + (wave >> 1) * 8;
    const int px = qx0 + (group & 1) * 4 + (sub & 3), py = qy0 + (group >> 1) * 4 + (sub >> 2);
    const bool inside = px < f.W && py < f.H;
    const float pxf = (float)px, pyf = (float)py;
    // pixel-centre bounds of the quadrant's two block columns and two block rows
    const float x_lo0 = (float)qx0, x_hi0 = (float)(qx0 + 3), x_lo1 = (float)(qx0 + 4), x_hi1 = (float)(qx0 + 7);
    const float y_lo0 = (float)qy0, y_hi0 = (float)(qy0 + 3), y_lo1 = (float)(qy0 + 4), y_hi1 = (float)(qy0 + 7);
    const uint64_t lanes_below = (1ull << lane) - 1ull;

    const uint32_t lo = ranges[2 * tile], hi = ranges[2 * tile + 1];
    PixelState p = {inside ? 1.0f : -1.0f, 0.0f, 0.0f, 0.0f, 0.0f};

    for (uint32_t base = lo; base < hi; base += 256) {
        const bool wave_done = __ballot(p.T > 0.0f) == 0ull;
        if (lane == 0) s_wave_done[wave] = wave_done ? 1u : 0u;
        const uint32_t j = base + tid;
        if (j < hi) {
            const uint32_t g = values[j];
            const float4* __restrict__ rec = reinterpret_cast<const float4*>(records + (size_t)g * kRecordFloats);
            s_a[tid] = rec[0];
            s_b[tid] = rec[1];
            s_c[tid] = rec[2];
        }
        __syncthreads();
        if ((s_wave_done[0] & s_wave_done[1] & s_wave_done[2] & s_wave_done[3]) != 0u) break;
        const int count = (int)min(256u, hi - base);
        if (!wave_done) {
            if (kCull) {
                // ---- lists: which staged Gaussians reach which 4x4 block (lane = Gaussian) ----
                uint32_t len[4] = {0u, 0u, 0u, 0u};  // uniform over the wavefront
                for (int chunk = 0; chunk < count; chunk += 64) {
                    const int k = chunk + lane;
                    bool in_x0 = false, in_x1 = false, in_y0 = false, in_y1 = false;
                    if (k < count) {
                        const float4 a = s_a[k];
                        const float4 c = s_c[k];
                        const float bx_lo = a.x - c.z, bx_hi = a.x + c.z, by_lo = a.y - c.w, by_hi = a.y + c.w;
                        in_x0 = bx_hi >= x_lo0 && bx_lo <= x_hi0;
                        in_x1 = bx_hi >= x_lo1 && bx_lo <= x_hi1;
                        in_y0 = by_hi >= y_lo0 && by_lo <= y_hi0;
                        in_y1 = by_hi >= y_lo1 && by_lo <= y_hi1;
                    }
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        const bool hit = ((b & 1) ? in_x1 : in_x0) && ((b >> 1) ? in_y1 : in_y0);
                        const uint64_t m = __ballot(hit);
                        if (hit) s_list[wave][b][len[b] + (uint32_t)__popcll(m & lanes_below)] = (uint8_t)k;
                        len[b] += (uint32_t)__popcll(m);
                    }
                }
                // a wavefront's LDS operations execute in order: its list writes precede the reads below
                wave_lds_sync();
                // ---- the four lane groups walk their lists side by side ----
                const uint32_t my_len = group == 0 ? len[0] : group == 1 ? len[1] : group == 2 ? len[2] : len[3];
                const uint32_t longest = max(max(len[0], len[1]), max(len[2], len[3]));
                const uint8_t* __restrict__ mine = s_list[wave][group];
                uint32_t k_next = mine[0];  // read ahead by one entry (entries past the end are never used)
                for (uint32_t i = 0; i < longest; ++i) {
                    const uint32_t kk = k_next;
                    k_next = mine[i + 1];
                    if (i < my_len) blend_one(p, pxf, pyf, s_a[kk], s_b[kk], s_c[kk]);
                    if (__ballot(p.T > 0.0f) == 0ull) break;
                }
            } else {
                for (int k = 0; k < count; ++k) {
                    if (__ballot(p.T > 0.0f) == 0ull) break;
                    blend_one(p, pxf, pyf, s_a[k], s_b[k], s_c[k]);
                }
            }
        }
        __syncthreads();
    }

    if (inside) {
        const size_t plane = (size_t)f.W * f.H;
        const size_t o = (size_t)py * f.W + px;
        const float T = fabsf(p.T);
        image[o] = p.c0 + T * f.bg[0];
        image[plane + o] = p.c1 + T * f.bg[1];
        image[2 * plane + o] = p.c2 + T * f.bg[2];
        if (out_depth) out_depth[o] = p.depth;
        if (out_alpha) out_alpha[o] = 1.0f - T;
    }
}

}  // namespace

int launch_fill_u32(uint32_t* p, size_t n, uint32_t v, hipStream_t s)
{
    if (n == 0) return GS355_OK;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, n, v);
    GS355_CHECK_LAUNCH("fill");
    return GS355_OK;
}

int launch_ranges(const gs355_header* header, uint32_t n_cap, const uint64_t* keys, uint32_t* ranges, int tiles,
                  hipStream_t s)
{
    const int rc = launch_fill_u32(ranges, (size_t)tiles * 2, 0u, s);
    if (rc) return rc;
    if (n_cap == 0) return GS355_OK;
    hipLaunchKernelGGL(ranges_kernel, dim3((n_cap + 255) / 256), dim3(256), 0, s, header, keys, ranges,
                       (uint32_t)tiles);
    GS355_CHECK_LAUNCH("ranges");
    return GS355_OK;
}

int launch_blend(const FrameArgs& f, const gs355_header* header, const uint32_t* ranges, const uint32_t* values,
                 const float* records, float* image, float* depth, float* alpha, bool cull, hipStream_t s)
{
    const int tiles = f.grid_x * f.grid_y;
    if (cull)
        hipLaunchKernelGGL(blend_kernel<true>, dim3(tiles), dim3(256), 0, s, f, header, ranges, values, records, image,
                           depth, alpha);
    else
        hipLaunchKernelGGL(blend_kernel<false>, dim3(tiles), dim3(256), 0, s, f, header, ranges, values, records, image,
                           depth, alpha);
    GS355_CHECK_LAUNCH("blend");
    return GS355_OK;
}

}  // namespace gs355
