// Per-tile range identification and front-to-back alpha blending for gfx950:
// the last two stages of the rasterizer behind GaussianRasterizer.forward
// (benchmarks/nerf/origin_gs/gs_model.py:211-220; output consumed as a
// [3,H,W] image at tests/test_inference_framework/test_inference.py:195-197).
//
// Blending: one 256-thread workgroup per 16x16 pixel tile, each of its four
// wavefronts owning an 8x8 pixel quadrant, each group of 16 lanes a 4x4 block
// of it.  The tile's depth-sorted Gaussians are staged through LDS in batches
// of 256 records (48 B each, rescaled while staging so that the per-pixel
// arithmetic needs no constant multiplies); every 4x4 block gets its own list
// of the staged Gaussians that can reach it, and the four lane groups of a
// wavefront walk their lists side by side, four entries per round, so one
// pass of the pixel arithmetic serves four different Gaussians.  A wavefront
// stops as soon as a ballot shows all of its 64 pixels finished, and the
// workgroup stops fetching batches once all four wavefronts have.
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
// accumulation.  The staged record carries hx = -conic_x / 2, ny = -conic_y and
// hz = -conic_z / 2, so the exponent
//     power = hx dx^2 + ny dx dy + hz dy^2
// is two nested multiply-adds (pair_exponent: five instructions), and the
// opacity enters through its base-2 logarithm:
//     alpha = min(0.99, exp2(power * log2(e) + log2(opacity))),
// one more multiply-add and the hardware exp2.  Fused multiply-adds round
// once where the scalar formula rounds twice, so `power` agrees with a scalar
// evaluation to the rounding of its terms, not bit for bit: a pair whose alpha
// lies within that distance of 1/255 may be decided either way (the checker
// counts those pairs per pixel).
//
// A pixel's transmittance T stays >= 1e-4 while it is live, so the sign of T
// carries the "finished" state: T > 0 live, T <= 0 finished with |T| the final
// transmittance (pixels outside the image start at -1).  A finished pixel can
// neither accumulate (its test_T is <= 0) nor finish again.
struct PixelState {
    float T, c0, c1, c2, depth;
};

// a = px, py, hx, ny;  b = hz, log2(opacity), r, g;  rec_c + entry = b, depth (read only by pixels that accept)
template <bool kCutOnExponent>
__device__ __forceinline__ void blend_one(PixelState& p, float pxf, float pyf, const float4 a, const float4 b,
                                          const char* rec_c, uint32_t entry)
{
    const float dx = a.x - pxf, dy = a.y - pyf;
    const float power = pair_exponent(dx, dy, a.z, a.w, b.x);
    const float t = __builtin_fmaf(power, 1.4426950408889634f, b.y);
    float alpha;
    if (kCutOnExponent) {
        if (power > 0.0f || t < kAlphaCut) return;
        alpha = fminf(0.99f, __builtin_amdgcn_exp2f(t));
    } else {
        alpha = fminf(0.99f, __builtin_amdgcn_exp2f(t));
        if (power > 0.0f || alpha < 1.0f / 255.0f) return;
    }
    // w = alpha T is the pair's weight and T - alpha T, rounded once, the transmittance behind it
    const float w = alpha * p.T;
    const float test_T = __builtin_fmaf(-alpha, p.T, p.T);
    const bool apply = test_T >= 0.0001f;
    if (apply) {
        const float2 cd = *reinterpret_cast<const float2*>(rec_c + entry);
        p.c0 = __builtin_fmaf(b.z, w, p.c0);
        p.c1 = __builtin_fmaf(b.w, w, p.c1);
        p.c2 = __builtin_fmaf(cd.x, w, p.c2);
        p.depth = __builtin_fmaf(cd.y, w, p.depth);
    }
    p.T = apply ? test_T : -fabsf(p.T);  // not applied: the pixel is finished (and stays so)
}

using ListEntry = uint16_t;
constexpr int kBatch = 256;            // records staged per round
constexpr uint32_t kNullEntry = kBatch * 16;  // list entry of the null record (opacity 0: rejected by every pixel)
constexpr int kListWords = kBatch + 8;  // entries per list: a batch, padded to a multiple of four, one round read ahead

// kCull: each wavefront first tests the staged Gaussians (one per lane) against
// the four 4x4 blocks of its quadrant, using the bounding box of the
// alpha >= 1/255 region from the record, and appends the survivors, in depth
// order, to the list of each block they can reach.  A (block, Gaussian) pair
// that is left out is one whose 16 pixels would all have taken the
// `alpha < 1/255` branch, and every pixel still sees its Gaussians front to
// back with the same arithmetic, so both variants produce identical images.
// List entries are the byte offsets of the staged records (16 x record number)
// in 16 bits (32-bit entries would serve as LDS addresses as they are, but the
// larger lists cost two workgroups per CU and 20 % of the kernel's speed); the
// lists are padded with the null record to a common length that is a multiple
// of four, so the walk needs no per-entry length test, reads four entries at
// a time and checks for finished wavefronts once per four entries.
template <bool kCull>
__global__ __launch_bounds__(256) void blend_kernel(FrameArgs f, const gs355_header* __restrict__ header,
                                                    const uint32_t* __restrict__ ranges,
                                                    const uint32_t* __restrict__ values,
                                                    const float* __restrict__ records, float* __restrict__ image,
                                                    float* __restrict__ out_depth, float* __restrict__ out_alpha)
{
    __shared__ float4 s_a[kBatch + 1];  // px, py, -conic_x / 2, -conic_y          (+ the null record)
    __shared__ float4 s_b[kBatch + 1];  // -conic_z / 2, log2(opacity), r, g
    __shared__ float4 s_c[kBatch + 1];  // b, depth, reach_x, reach_y
    __shared__ uint32_t s_wave_done[4];
    // per wavefront and 4x4 block: byte offsets of the staged records of the Gaussians that can reach the block
    __shared__ __align__(8) ListEntry s_list[kCull ? 4 : 1][4][kListWords];

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

    const uint32_t lo = ranges[2 * tile], hi = ranges[2 * tile + 1];
    PixelState p = {inside ? 1.0f : -1.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (tid == 0) {  // the null record: zero conic and log2(opacity) = -inf give alpha = 0
        s_a[kBatch] = make_float4(0.f, 0.f, 0.f, 0.f);
        s_b[kBatch] = make_float4(0.f, -__builtin_inff(), 0.f, 0.f);
        s_c[kBatch] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    const char* const rec_a = reinterpret_cast<const char*>(s_a);
    const char* const rec_b = reinterpret_cast<const char*>(s_b);
    const char* const rec_c = reinterpret_cast<const char*>(s_c);
    auto blend_entry = [&](uint32_t entry) {
        blend_one<kCull>(p, pxf, pyf, *reinterpret_cast<const float4*>(rec_a + entry),
                         *reinterpret_cast<const float4*>(rec_b + entry), rec_c, entry);
    };

    for (uint32_t base = lo; base < hi; base += kBatch) {
        const uint64_t live = __ballot(p.T > 0.0f);  // lanes whose pixel is still accumulating
        const bool wave_done = live == 0ull;
        if (lane == 0) s_wave_done[wave] = wave_done ? 1u : 0u;
        const uint32_t j = base + tid;
        if (j < hi) {
            const uint32_t g = values[j];
            const float4* __restrict__ rec = reinterpret_cast<const float4*>(records + (size_t)g * kRecordFloats);
            const float4 r0 = rec[0], r1 = rec[1], r2 = rec[2];
            // a negative opacity gives a negative alpha, which every pixel rejects: log2(0) = -inf does the same
            const float log2o = __builtin_amdgcn_logf(r1.y < 0.0f ? 0.0f : r1.y);
            s_a[tid] = make_float4(r0.x, r0.y, -0.5f * r0.z, -r0.w);
            s_b[tid] = make_float4(-0.5f * r1.x, log2o, r1.z, r1.w);
            s_c[tid] = r2;
        }
        __syncthreads();
        if ((s_wave_done[0] & s_wave_done[1] & s_wave_done[2] & s_wave_done[3]) != 0u) break;
        const int count = (int)min((uint32_t)kBatch, hi - base);
        if (!wave_done) {
            if (kCull) {
                // ---- lists: which staged Gaussians reach which 4x4 block (lane = Gaussian) ----
                uint32_t len[4] = {0u, 0u, 0u, 0u};  // uniform over the wavefront
                // Every comparison goes straight into a lane mask (a ballot of one compare is the compare's own
                // result register), the masks are combined in scalar registers, and a lane's rank among a mask's
                // lanes is the hardware's masked bit count: a per-lane flag carried into a ballot costs two vector
                // instructions more per ballot, and ranks through `mask & lanes_below` two more per rank.
                for (int chunk = 0; chunk < count; chunk += 64) {
                    const int k = chunk + lane;  // < kBatch: slots past `count` hold older records, masked by `valid`
                    const uint64_t valid = __ballot(k < count);
                    const float4 a = s_a[k];
                    const float4 c = s_c[k];
                    const float bx_lo = a.x - c.z, bx_hi = a.x + c.z, by_lo = a.y - c.w, by_hi = a.y + c.w;
                    const uint64_t in_x0 = __ballot(bx_hi >= x_lo0) & __ballot(bx_lo <= x_hi0) & valid;
                    const uint64_t in_x1 = __ballot(bx_hi >= x_lo1) & __ballot(bx_lo <= x_hi1) & valid;
                    const uint64_t in_y0 = __ballot(by_hi >= y_lo0) & __ballot(by_lo <= y_hi0);
                    const uint64_t in_y1 = __ballot(by_hi >= y_lo1) & __ballot(by_lo <= y_hi1);
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        // a block whose 16 pixels have all finished gets no entries (its lane group idles through
                        // the null record while the other blocks of the wavefront are served)
                        if (((live >> (16 * b)) & 0xFFFFull) == 0ull) continue;
                        const uint64_t m = ((b & 1) ? in_x1 : in_x0) & ((b >> 1) ? in_y1 : in_y0);
                        if (__builtin_amdgcn_inverse_ballot_w64(m))
                            s_list[wave][b][len[b] + lanes_below_in(m)] = (ListEntry)(k * 16);
                        len[b] += (uint32_t)__popcll(m);
                    }
                }
                const uint32_t longest = (uint32_t)__builtin_amdgcn_readfirstlane(
                    (int)max(max(len[0], len[1]), max(len[2], len[3])));
                const uint32_t quads = (longest + 3u) / 4u;
                // pad every list with the null record up to the common length
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    for (uint32_t at = len[b] + (uint32_t)lane; at < quads * 4u; at += 64u)
                        s_list[wave][b][at] = (ListEntry)kNullEntry;
                // a wavefront's LDS operations execute in order: its list writes precede the reads below
                wave_lds_sync();
                // ---- the four lane groups walk their lists side by side, four entries per round ----
                const uint2* __restrict__ mine = reinterpret_cast<const uint2*>(s_list[wave][group]);
                uint2 next = mine[0];  // read ahead by one round (rounds past the end are never used)
                for (uint32_t i = 0; i < quads; ++i) {
                    const uint2 e = next;
                    next = mine[i + 1];
                    blend_entry(e.x & 0xFFFFu);
                    blend_entry(e.x >> 16);
                    blend_entry(e.y & 0xFFFFu);
                    blend_entry(e.y >> 16);
                    if (__ballot(p.T > 0.0f) == 0ull) break;
                }
            } else {
                for (int k = 0; k < count; ++k) {
                    if (__ballot(p.T > 0.0f) == 0ull) break;
                    blend_entry((uint32_t)k * 16u);
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
