// Per-tile range identification and front-to-back alpha blending for gfx950:
// the last two stages of the rasterizer behind GaussianRasterizer.forward
// (benchmarks/nerf/origin_gs/gs_model.py:211-220; output consumed as a
// [3,H,W] image at tests/test_inference_framework/test_inference.py:195-197).
//
// Blending: one 256-thread workgroup per 16x16 pixel tile, each of its four
// wavefronts owning an 8x8 pixel quadrant.  The tile's depth-sorted Gaussians
// are staged through LDS in batches of 256 records (48 B each); a wavefront
// stops reading as soon as a ballot shows all of its 64 pixels finished, and
// the workgroup stops fetching batches once all four wavefronts have.
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

__global__ __launch_bounds__(256) void blend_kernel(FrameArgs f, const gs355_header* __restrict__ header,
                                                    const uint32_t* __restrict__ ranges,
                                                    const uint32_t* __restrict__ values,
                                                    const float* __restrict__ records, float* __restrict__ image,
                                                    float* __restrict__ out_depth, float* __restrict__ out_alpha)
{
    __shared__ float4 s_a[256];  // px, py, conic_x, conic_y
    __shared__ float4 s_b[256];  // conic_z, opacity, r, g
    __shared__ float2 s_c[256];  // b, depth
    __shared__ uint32_t s_wave_done[4];

    if (header->overflow) return;
    const int tile = blockIdx.x;
    const int tile_x = tile % f.grid_x, tile_y = tile / f.grid_x;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int px = tile_x * kTile + (wave & 1) * 8 + (lane & 7);
    const int py = tile_y * kTile + (wave >> 1) * 8 + (lane >> 3);
    const bool inside = px < f.W && py < f.H;
    const float pxf = (float)px, pyf = (float)py;

    const uint32_t lo = ranges[2 * tile], hi = ranges[2 * tile + 1];
    float T = 1.0f, c0 = 0.0f, c1 = 0.0f, c2 = 0.0f, dsum = 0.0f;
    bool done = !inside;

    for (uint32_t base = lo; base < hi; base += 256) {
        const bool wave_done = __ballot(!done) == 0ull;
        if (lane == 0) s_wave_done[wave] = wave_done ? 1u : 0u;
        const uint32_t j = base + tid;
        if (j < hi) {
            const uint32_t g = values[j];
            const float4* __restrict__ rec = reinterpret_cast<const float4*>(records + (size_t)g * kRecordFloats);
            const float4 r0 = rec[0], r1 = rec[1];
            const float2 r2 = *reinterpret_cast<const float2*>(rec + 2);
            s_a[tid] = r0;
            s_b[tid] = r1;
            s_c[tid] = r2;
        }
        __syncthreads();
        if ((s_wave_done[0] & s_wave_done[1] & s_wave_done[2] & s_wave_done[3]) != 0u) break;
        const int count = (int)min(256u, hi - base);
        if (!wave_done) {
            for (int k = 0; k < count; ++k) {
                if (__ballot(!done) == 0ull) break;
                if (done) continue;
                const float4 a = s_a[k];
                const float4 b = s_b[k];
                const float dx = a.x - pxf, dy = a.y - pyf;
                const float power = -0.5f * (a.z * dx * dx + b.x * dy * dy) - a.w * dx * dy;
                if (power > 0.0f) continue;
                const float alpha = fminf(0.99f, b.y * __expf(power));
                if (alpha < 1.0f / 255.0f) continue;
                const float test_T = T * (1.0f - alpha);
                if (test_T < 0.0001f) {
                    done = true;
                    continue;
                }
                const float2 c = s_c[k];
                const float w = alpha * T;
                c0 += b.z * w;
                c1 += b.w * w;
                c2 += c.x * w;
                dsum += c.y * w;
                T = test_T;
            }
        }
        __syncthreads();
    }

    if (inside) {
        const size_t plane = (size_t)f.W * f.H;
        const size_t o = (size_t)py * f.W + px;
        image[o] = c0 + T * f.bg[0];
        image[plane + o] = c1 + T * f.bg[1];
        image[2 * plane + o] = c2 + T * f.bg[2];
        if (out_depth) out_depth[o] = dsum;
        if (out_alpha) out_alpha[o] = 1.0f - T;
    }
}

}  // namespace

int launch_ranges(const gs355_header* header, uint32_t n_cap, const uint64_t* keys, uint32_t* ranges, int tiles,
                  hipStream_t s)
{
    const size_t words = (size_t)tiles * 2;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s, ranges, words, 0u);
    GS355_CHECK_LAUNCH("ranges: clear");
    if (n_cap == 0) return GS355_OK;
    hipLaunchKernelGGL(ranges_kernel, dim3((n_cap + 255) / 256), dim3(256), 0, s, header, keys, ranges,
                       (uint32_t)tiles);
    GS355_CHECK_LAUNCH("ranges");
    return GS355_OK;
}

int launch_blend(const FrameArgs& f, const gs355_header* header, const uint32_t* ranges, const uint32_t* values,
                 const float* records, float* image, float* depth, float* alpha, hipStream_t s)
{
    const int tiles = f.grid_x * f.grid_y;
    hipLaunchKernelGGL(blend_kernel, dim3(tiles), dim3(256), 0, s, f, header, ranges, values, records, image, depth,
                       alpha);
    GS355_CHECK_LAUNCH("blend");
    return GS355_OK;
}

}  // namespace gs355
