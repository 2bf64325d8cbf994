// Backward pass of the rasterizer for gfx950: the gradients the reference's training loop pulls through
// GaussianRasterizer.forward (loss.backward() at benchmarks/nerf/origin_gs/gs_trainer.py:117-124; the
// screen-space gradient of `means2D` feeds densification, landmark/nerf_components/model_components/fields/
// encodings/gaussian_encoding.py:729-743).
//
// Two kernels over the forward pass's workspace (records, sorted values, ranges):
//   blend_backward   per 16x16 tile, the forward blend's walk repeated FRONT TO BACK with the same per-block
//                    lists and the same per-pair decisions.  With f_i = colour_i . dL/dpixel, w_i = alpha_i T_i,
//                    prefix P_i = sum_{j<=i} w_j f_j and R = out_pixel . dL/dpixel - T_final dL/dalpha_out (all
//                    known from the forward outputs), dL/dalpha_i = T_i f_i - (R - P_i) / (1 - alpha_i): no
//                    division by a transmittance and no second, reversed walk.  Per-pair contributions are summed
//                    over the 16 pixels of a block by lane exchanges inside the 16-lane row, added to the staged
//                    Gaussian's accumulators in LDS (one LDS atomic per step: LDS float atomics are slow), and
//                    written once per batch of 128 as one 48-byte record per (tile, Gaussian) key.  No global
//                    atomics (they cost more than the rest of the kernel): the records of a Gaussian are
//                    consecutive, in the order its tile rectangle is walked, and the next kernel sums them in
//                    that order, so gradients are identical from run to run.
//   preprocess_backward  per Gaussian: conic -> 2-D covariance -> Jacobian / 3-D covariance -> scale, rotation,
//                    mean; pixel position -> mean; colour -> SH coefficients and view direction -> mean.
// min(0.99, opacity * G) passes the gradient unchanged, and the `means2D` gradient is in normalised device units
// (pixel gradient times W/2, H/2), as the published backward pass of this rasterizer family does.
#include "gs355_internal.h"

namespace gs355 {

namespace {

constexpr int kGradFloats = 10;  // accumulators per staged Gaussian in LDS
constexpr int kKeyFloats = GS355_KEY_GRAD_FLOATS;  // per-key record: dpx, dpy, dconic xyz, dopacity, drgb, ddepth, 2 unused

// Record slot of the key (tile, Gaussian): the Gaussian's keys in the order its tile rectangle is walked
// (row by row), after those of all Gaussians before it.
__device__ __forceinline__ uint32_t key_slot(uint32_t first, uint64_t rect, int tile_x, int tile_y)
{
    const int x0 = (int)(rect & 0xffffu), y0 = (int)((rect >> 16) & 0xffffu), x1 = (int)((rect >> 32) & 0xffffu);
    return first + (uint32_t)((tile_y - y0) * (x1 - x0) + (tile_x - x0));
}

template <int kCtrl>
__device__ __forceinline__ float dpp(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xf, 0xf, false));
}

// Two values reduced over a lane pair in one exchange: the lane with `upper` clear keeps a, the other keeps b,
// each adds its partner's copy of the value it keeps.
template <int kCtrl>
__device__ __forceinline__ float keep_one_of_two(float a, float b, bool upper)
{
    const float send = upper ? a : b, keep = upper ? b : a;
    return keep + dpp<kCtrl>(send);
}

struct PixelGrad {
    float g0, g1, g2, g3;  // dL/d(r, g, b, depth) of this pixel
    float R;               // out . g - T_final * dL/dalpha_out
};

// One 16-lane row evaluates staged Gaussian `a, b, c` on its 16 pixels.  Returns false if no lane of the wavefront
// blended its pair; otherwise lane s < 10 of each row returns in `sum` the row's total of accumulator s:
// the moments of dL/dpower over the pixel offsets (dpow dx, dpow dy, dpow dx^2, dpow dx dy, dpow dy^2),
// dL/dopacity, dL/d(r, g, b, depth).  T carries the forward blend's state (sign = finished).
// b.y is log2(opacity): opacity * exp(power) is evaluated exactly as the forward blend evaluates it (one multiply-add
// into the hardware exp2, decided on the exponent before the exp2), so both passes take the same decisions.  The
// opacity's accumulator receives sum(dL/dpower) = opacity * dL/dopacity; the caller divides once per Gaussian.
__device__ __forceinline__ bool backward_one(float& T, float& prefix, const PixelGrad& pg, float pxf, float pyf,
                                             const float4 a, const float4 b, const float4 c, bool enabled, int sub,
                                             float& sum)
{
    const float dx = a.x - pxf, dy = a.y - pyf;
    const float power = pair_exponent(dx, dy, a.z, a.w, b.x);  // a.z, a.w, b.x = -conic_x / 2, -conic_y, -conic_z / 2
    const float t = __builtin_fmaf(power, 1.4426950408889634f, b.y);
    const bool accept = enabled && !(power > 0.0f || t < kAlphaCut);  // the forward blend's decision, on the exponent
    if (__ballot(accept) == 0ull) return false;
    const float raw = __builtin_amdgcn_exp2f(t);  // opacity * exp(power)
    const float alpha = fminf(0.99f, raw);
    const float test_T = __builtin_fmaf(-alpha, T, T);  // T - alpha T, as the forward blend forms it
    const bool hit = accept && test_T >= 0.0001f;
    if (accept && !hit && T > 0.0f) T = -T;
    if (__ballot(hit) == 0ull) return false;
    float w = 0.0f, dpow = 0.0f;
    if (hit) {
        w = alpha * T;
        const float fg = b.z * pg.g0 + b.w * pg.g1 + c.x * pg.g2 + c.y * pg.g3;
        prefix += w * fg;
        const float dalpha = T * fg - (pg.R - prefix) * __builtin_amdgcn_rcpf(1.0f - alpha);
        dpow = raw * dalpha;  // the gradient passes through min(0.99, .) unchanged
        T = test_T;
    }
    const float dop = dpow;  // (times 1 / opacity, once per Gaussian, when the batch's sums are turned into records)
    const float mx = dpow * dx, my = dpow * dy;
    // ten sums over the row's 16 lanes, transposed as they are reduced: after the exchanges inside lane pairs and
    // quads a lane holds one of four (then two) values, the quads' partial sums are rotated together, and lane s
    // ends with the total of value s
    const bool b0 = (sub & 1) != 0, b1 = (sub & 2) != 0;
    const float u0 = keep_one_of_two<0xB1>(mx, my, b0);            // quad_perm [1,0,3,2]
    const float u1 = keep_one_of_two<0xB1>(mx * dx, mx * dy, b0);
    const float u2 = keep_one_of_two<0xB1>(my * dy, dop, b0);
    const float u3 = keep_one_of_two<0xB1>(w * pg.g0, w * pg.g1, b0);
    const float u4 = keep_one_of_two<0xB1>(w * pg.g2, w * pg.g3, b0);
    float t0 = keep_one_of_two<0x4E>(u0, u1, b1);                  // quad_perm [2,3,0,1]: value 2 b1 + b0
    float t1 = keep_one_of_two<0x4E>(u2, u3, b1);                  // value 4 + 2 b1 + b0
    float t2 = u4 + dpp<0x4E>(u4);                                 // value 8 + b0
    t0 += dpp<0x124>(t0);                                          // row_ror:4
    t1 += dpp<0x124>(t1);
    t2 += dpp<0x124>(t2);
    t0 += dpp<0x128>(t0);                                          // row_ror:8
    t1 += dpp<0x128>(t1);
    t2 += dpp<0x128>(t2);
    sum = sub < 4 ? t0 : sub < 8 ? t1 : t2;
    return true;
}

__global__ __launch_bounds__(256) void blend_backward_kernel(
    FrameArgs f, const gs355_header* __restrict__ header, const uint32_t* __restrict__ ranges,
    const uint32_t* __restrict__ values, const float* __restrict__ records, const float* __restrict__ image,
    const float* __restrict__ out_depth, const float* __restrict__ out_alpha, const float* __restrict__ g_image,
    const float* __restrict__ g_depth, const float* __restrict__ g_alpha, const uint64_t* __restrict__ rects,
    const uint32_t* __restrict__ first_key, float* __restrict__ key_grads)
{
    // staged Gaussians per round: 128 (13 KB of LDS per workgroup) leaves the register file as the limit on resident
    // wavefronts; 256 measured 2 % slower
    constexpr int kBatch = 128;
    __shared__ float4 s_a[kBatch];  // px, py, -conic_x / 2, -conic_y   (rescaled as the forward blend stages them)
    __shared__ float4 s_b[kBatch];  // -conic_z / 2, log2(opacity), r, g
    __shared__ float4 s_c[kBatch];  // b, depth, reach_x, reach_y
    __shared__ float s_grad[kBatch * kGradFloats];
    __shared__ uint32_t s_wave_done[4];
    __shared__ uint8_t s_list[4][4][kBatch + 4];

    if (header->overflow) return;
    const int tile = blockIdx.x;
    const int tile_x = tile % f.grid_x, tile_y = tile / f.grid_x;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int group = lane >> 4, sub = lane & 15;
    const int qx0 = tile_x * kTile + (wave & 1) * 8, qy0 = tile_y * kTile + (wave >> 1) * 8;
    const int px = qx0 + (group & 1) * 4 + (sub & 3), py = qy0 + (group >> 1) * 4 + (sub >> 2);
    const bool inside = px < f.W && py < f.H;
    const float pxf = (float)px, pyf = (float)py;
    const float x_lo0 = (float)qx0, x_hi0 = (float)(qx0 + 3), x_lo1 = (float)(qx0 + 4), x_hi1 = (float)(qx0 + 7);
    const float y_lo0 = (float)qy0, y_hi0 = (float)(qy0 + 3), y_lo1 = (float)(qy0 + 4), y_hi1 = (float)(qy0 + 7);

    PixelGrad pg = {0.f, 0.f, 0.f, 0.f, 0.f};
    if (inside) {
        const size_t plane = (size_t)f.W * f.H;
        const size_t o = (size_t)py * f.W + px;
        pg.g0 = g_image[o];
        pg.g1 = g_image[plane + o];
        pg.g2 = g_image[2 * plane + o];
        pg.R = image[o] * pg.g0 + image[plane + o] * pg.g1 + image[2 * plane + o] * pg.g2;
        if (g_depth) {
            pg.g3 = g_depth[o];
            pg.R += out_depth[o] * pg.g3;
        }
        if (g_alpha) pg.R -= (1.0f - out_alpha[o]) * g_alpha[o];
    }

    const uint32_t lo = ranges[2 * tile], hi = ranges[2 * tile + 1];
    float T = inside ? 1.0f : -1.0f, prefix = 0.0f;

    uint32_t base = lo;
    for (; base < hi; base += kBatch) {
        const bool wave_done = __ballot(T > 0.0f) == 0ull;
        if (lane == 0) s_wave_done[wave] = wave_done ? 1u : 0u;
        const uint32_t j = base + tid;
        const bool staging = tid < kBatch && j < hi;  // this thread stages (and later writes the record of) a Gaussian
        uint32_t slot = 0;
        if (staging) {
            const uint32_t g = values[j];
            const float4* __restrict__ rec = reinterpret_cast<const float4*>(records + (size_t)g * kRecordFloats);
            const float4 r0 = rec[0], r1 = rec[1];
            const float opacity = r1.y < 0.0f ? 0.0f : r1.y;  // as the forward blend: a negative opacity never blends
            s_a[tid] = make_float4(r0.x, r0.y, -0.5f * r0.z, -r0.w);
            s_b[tid] = make_float4(-0.5f * r1.x, __builtin_amdgcn_logf(opacity), r1.z, r1.w);
            s_c[tid] = rec[2];
            slot = key_slot(first_key[g], rects[g], tile_x, tile_y);
        }
        if (tid < kBatch) {
            float2* __restrict__ row = reinterpret_cast<float2*>(s_grad + tid * kGradFloats);
#pragma unroll
            for (int k = 0; k < kGradFloats / 2; ++k) row[k] = make_float2(0.f, 0.f);
        }
        __syncthreads();
        if ((s_wave_done[0] & s_wave_done[1] & s_wave_done[2] & s_wave_done[3]) != 0u) break;
        const int count = (int)min((uint32_t)kBatch, hi - base);
        if (!wave_done) {
            // ---- lists: which staged Gaussians reach which 4x4 block (lane = Gaussian), as the forward blend ----
            uint32_t len[4] = {0u, 0u, 0u, 0u};
            for (int chunk = 0; chunk < count; chunk += 64) {
                // lane masks straight from the comparisons, combined in scalar registers (as the forward blend)
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
                    const uint64_t m = ((b & 1) ? in_x1 : in_x0) & ((b >> 1) ? in_y1 : in_y0);
                    if (__builtin_amdgcn_inverse_ballot_w64(m)) s_list[wave][b][len[b] + lanes_below_in(m)] = (uint8_t)k;
                    len[b] += (uint32_t)__popcll(m);
                }
            }
            wave_lds_sync();
            const uint32_t my_len = group == 0 ? len[0] : group == 1 ? len[1] : group == 2 ? len[2] : len[3];
            const uint32_t longest = max(max(len[0], len[1]), max(len[2], len[3]));
            const uint8_t* __restrict__ mine = s_list[wave][group];
            uint32_t k_next = mine[0];
            for (uint32_t i = 0; i < longest; ++i) {
                const uint32_t kk = k_next;
                k_next = mine[i + 1];
                float sum;
                if (backward_one(T, prefix, pg, pxf, pyf, s_a[kk], s_b[kk], s_c[kk], i < my_len, sub, sum)) {
                    // lane s of each row adds accumulator s of the row's Gaussian
                    if (sub < 10 && i < my_len && sum != 0.0f) atomicAdd(&s_grad[kk * kGradFloats + sub], sum);
                }
                if (__ballot(T > 0.0f) == 0ull) break;
            }
        }
        __syncthreads();
        // ---- this batch's records: the moments turned into gradients of position and conic ----
        if (staging) {
            const float* __restrict__ m = s_grad + tid * kGradFloats;
            const float4 a = s_a[tid];
            const float hz = s_b[tid].x;
            const float inv_opacity = __builtin_amdgcn_exp2f(-s_b[tid].y);  // s_b.y = log2(opacity)
            float4* __restrict__ dst = reinterpret_cast<float4*>(key_grads + (size_t)slot * kKeyFloats);
            // d power / d centre = -(conic_x dx + conic_y dy, conic_z dy + conic_y dx), with conic_x = -2 a.z etc.
            dst[0] = make_float4(2.0f * a.z * m[0] + a.w * m[1], 2.0f * hz * m[1] + a.w * m[0], -0.5f * m[2], -m[3]);
            // m[5] = sum of opacity * dL/dopacity over the tile's pixels (zero, not 0 * inf, for a Gaussian that never blended)
            dst[1] = make_float4(-0.5f * m[4], m[5] != 0.0f ? m[5] * inv_opacity : 0.0f, m[6], m[7]);
            dst[2] = make_float4(m[8], m[9], 0.f, 0.f);
        }
    }
    // keys the tile never reached (every pixel finished before them) contribute nothing: every record is written
    for (uint32_t j = base + tid; j < hi; j += 256) {
        const uint32_t g = values[j];
        float4* __restrict__ dst =
            reinterpret_cast<float4*>(key_grads + (size_t)key_slot(first_key[g], rects[g], tile_x, tile_y) * kKeyFloats);
        dst[0] = dst[1] = dst[2] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

constexpr float kShC0 = 0.28209479177387814f;
constexpr float kShC1 = 0.4886025119029199f;
constexpr float kShC2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f, -1.0925484305920792f,
                            0.5462742152960396f};
constexpr float kShC3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f, 0.3731763325901154f,
                            -0.4570457994644658f, 1.445305721320277f, -0.5900435899266435f};

// Real SH basis (sh_utils.py:67-94) and its gradient with respect to the unit direction.
__device__ __forceinline__ void sh_basis_grad(int deg, float x, float y, float z, float b[16], float bx[16],
                                              float by[16], float bz[16])
{
#pragma unroll
    for (int k = 0; k < 16; ++k) b[k] = bx[k] = by[k] = bz[k] = 0.0f;
    b[0] = kShC0;
    if (deg < 1) return;
    b[1] = -kShC1 * y; by[1] = -kShC1;
    b[2] = kShC1 * z;  bz[2] = kShC1;
    b[3] = -kShC1 * x; bx[3] = -kShC1;
    if (deg < 2) return;
    const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
    b[4] = kShC2[0] * xy; bx[4] = kShC2[0] * y; by[4] = kShC2[0] * x;
    b[5] = kShC2[1] * yz; by[5] = kShC2[1] * z; bz[5] = kShC2[1] * y;
    b[6] = kShC2[2] * (2.0f * zz - xx - yy); bx[6] = kShC2[2] * -2.0f * x; by[6] = kShC2[2] * -2.0f * y;
    bz[6] = kShC2[2] * 4.0f * z;
    b[7] = kShC2[3] * xz; bx[7] = kShC2[3] * z; bz[7] = kShC2[3] * x;
    b[8] = kShC2[4] * (xx - yy); bx[8] = kShC2[4] * 2.0f * x; by[8] = kShC2[4] * -2.0f * y;
    if (deg < 3) return;
    b[9] = kShC3[0] * y * (3.0f * xx - yy); bx[9] = kShC3[0] * 6.0f * xy; by[9] = kShC3[0] * (3.0f * xx - 3.0f * yy);
    b[10] = kShC3[1] * xy * z; bx[10] = kShC3[1] * yz; by[10] = kShC3[1] * xz; bz[10] = kShC3[1] * xy;
    b[11] = kShC3[2] * y * (4.0f * zz - xx - yy); bx[11] = kShC3[2] * -2.0f * xy;
    by[11] = kShC3[2] * (4.0f * zz - xx - 3.0f * yy); bz[11] = kShC3[2] * 8.0f * yz;
    b[12] = kShC3[3] * z * (2.0f * zz - 3.0f * xx - 3.0f * yy); bx[12] = kShC3[3] * -6.0f * xz;
    by[12] = kShC3[3] * -6.0f * yz; bz[12] = kShC3[3] * (6.0f * zz - 3.0f * xx - 3.0f * yy);
    b[13] = kShC3[4] * x * (4.0f * zz - xx - yy); bx[13] = kShC3[4] * (4.0f * zz - 3.0f * xx - yy);
    by[13] = kShC3[4] * -2.0f * xy; bz[13] = kShC3[4] * 8.0f * xz;
    b[14] = kShC3[5] * z * (xx - yy); bx[14] = kShC3[5] * 2.0f * xz; by[14] = kShC3[5] * -2.0f * yz;
    bz[14] = kShC3[5] * (xx - yy);
    b[15] = kShC3[6] * x * (xx - 3.0f * yy); bx[15] = kShC3[6] * (3.0f * xx - 3.0f * yy); by[15] = kShC3[6] * -6.0f * xy;
}

constexpr int kShStride = 52;  // floats per Gaussian in the SH staging area (16-B reads of 64 lanes on distinct banks)

// kMode 0: SH blocks (if any) are read and written by their own lanes.  1 and 2: 16-coefficient blocks, 16-byte
// aligned, staged through LDS; 2 also fetches the coefficients (needed for degree > 0 only).
template <int kMode>
__global__ __launch_bounds__(256) void preprocess_backward_kernel(FrameArgs f, gs355_gaussians g,
                                                                  const int32_t* __restrict__ radii,
                                                                  const float* __restrict__ records,
                                                                  const uint32_t* __restrict__ tiles_touched,
                                                                  const uint32_t* __restrict__ first_key,
                                                                  const float* __restrict__ key_grads,
                                                                  gs355_gradients out)
{
    // Full 16-coefficient SH blocks travel through LDS: each wavefront moves the 12 KB of its 64 Gaussians'
    // coefficients (in) and coefficient gradients (out) with coalesced 16-B accesses; a lane works on its own row.
    __shared__ float4 s_sh[kMode == 0 ? 1 : 4 * 64 * kShStride / 4];

    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const bool valid = i < g.P;
    const size_t si = (size_t)(valid ? i : g.P - 1);
    const int M = f.sh_coeffs;
    const bool alive = valid && radii[si] > 0;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const size_t wave_first = (size_t)blockIdx.x * blockDim.x + (size_t)wave * 64;
    const int count = (int)min((size_t)64, (size_t)g.P > wave_first ? (size_t)g.P - wave_first : (size_t)0);
    constexpr bool staged = kMode != 0, fetch_sh = kMode == 2;
    float4* __restrict__ mine = s_sh + (staged ? wave * 64 * (kShStride / 4) : 0);
    float* __restrict__ my_row = reinterpret_cast<float*>(mine) + (staged ? lane * kShStride : 0);

    float dmean[3] = {0.f, 0.f, 0.f}, d2[3] = {0.f, 0.f, 0.f}, dscale[3] = {0.f, 0.f, 0.f};
    float drot[4] = {0.f, 0.f, 0.f, 0.f}, dcov[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, dcol[3] = {0.f, 0.f, 0.f};
    float dop = 0.f;
    float b[16], gcol[3] = {0.f, 0.f, 0.f};
    float nx = 0.f, ny = 0.f, nz = 0.f, inv_len = 0.f;
    float bx[16], by[16], bz[16];
    int K = 0;
    if (alive) {
        const float* __restrict__ V = f.viewmatrix;
        const float* __restrict__ Pm = f.projmatrix;
        // the Gaussian's keys are consecutive records; summed in order, so the result does not vary between runs.
        // Four records are requested at a time (indices past the last one re-read it and are not added).
        float4 A0 = make_float4(0.f, 0.f, 0.f, 0.f), A1 = A0, A2 = A0;
        {
            const float4* __restrict__ rec = reinterpret_cast<const float4*>(key_grads + (size_t)first_key[si] * kKeyFloats);
            const uint32_t n = tiles_touched[si];
            for (uint32_t k0 = 0; k0 < n; k0 += 4) {
                float4 r[4][3];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const size_t k = min(k0 + (uint32_t)u, n - 1);
#pragma unroll
                    for (int q = 0; q < 3; ++q) r[u][q] = rec[3 * k + q];
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (k0 + (uint32_t)u < n) {
                        A0.x += r[u][0].x; A0.y += r[u][0].y; A0.z += r[u][0].z; A0.w += r[u][0].w;
                        A1.x += r[u][1].x; A1.y += r[u][1].y; A1.z += r[u][1].z; A1.w += r[u][1].w;
                        A2.x += r[u][2].x; A2.y += r[u][2].y;
                    }
                }
            }
        }
        const float g_px = A0.x, g_py = A0.y, gA = A0.z, gB = A0.w, gC = A1.x;
        dop = A1.y;
        dcol[0] = A1.z; dcol[1] = A1.w; dcol[2] = A2.x;
        const float g_depth = A2.y;
        const float x = g.means3D[3 * si], y = g.means3D[3 * si + 1], z = g.means3D[3 * si + 2];

        // ---- pixel position ----
        const float phx = Pm[0] * x + Pm[4] * y + Pm[8] * z + Pm[12];
        const float phy = Pm[1] * x + Pm[5] * y + Pm[9] * z + Pm[13];
        const float phw = Pm[3] * x + Pm[7] * y + Pm[11] * z + Pm[15];
        const float pw = 1.0f / (phw + 0.0000001f);
        d2[0] = g_px * 0.5f * (float)f.W;
        d2[1] = g_py * 0.5f * (float)f.H;
        const float d_phx = d2[0] * pw, d_phy = d2[1] * pw;
        const float d_phw = -(pw * pw) * (phx * d2[0] + phy * d2[1]);
#pragma unroll
        for (int k = 0; k < 3; ++k) dmean[k] = Pm[4 * k] * d_phx + Pm[4 * k + 1] * d_phy + Pm[4 * k + 3] * d_phw;

        // ---- 3-D covariance, Jacobian of the projection, 2-D covariance, conic: in double precision ----
        // An elongated splat (axes 50:1) hides its thin axes in the low bits of the fp32 covariance, and its 2-D
        // determinant is a difference of nearly equal products; the gradients of scale and rotation are small
        // differences of terms built from them.  fp64 vector arithmetic runs at the fp32 rate on this chip and
        // the kernel waits for memory, so the chain costs nothing in double and loses nothing.
        typedef double real;
        real S[6], s[3] = {0., 0., 0.}, q[4] = {0., 0., 0., 0.}, R[3][3] = {};
        if (g.cov3D_precomp) {
#pragma unroll
            for (int k = 0; k < 6; ++k) S[k] = g.cov3D_precomp[6 * si + k];
        } else {
#pragma unroll
            for (int k = 0; k < 3; ++k) s[k] = (real)f.scale_modifier * (real)g.scales[3 * si + k];
#pragma unroll
            for (int k = 0; k < 4; ++k) q[k] = g.rotations[4 * si + k];
            const real r = q[0], qx = q[1], qy = q[2], qz = q[3];
            R[0][0] = 1. - 2. * (qy * qy + qz * qz); R[0][1] = 2. * (qx * qy - r * qz); R[0][2] = 2. * (qx * qz + r * qy);
            R[1][0] = 2. * (qx * qy + r * qz); R[1][1] = 1. - 2. * (qx * qx + qz * qz); R[1][2] = 2. * (qy * qz - r * qx);
            R[2][0] = 2. * (qx * qz - r * qy); R[2][1] = 2. * (qy * qz + r * qx); R[2][2] = 1. - 2. * (qx * qx + qy * qy);
            int n = 0;
#pragma unroll
            for (int a = 0; a < 3; ++a)
#pragma unroll
                for (int c = a; c < 3; ++c)
                    S[n++] = R[a][0] * s[0] * R[c][0] * s[0] + R[a][1] * s[1] * R[c][1] * s[1] + R[a][2] * s[2] * R[c][2] * s[2];
        }
        const real Sm[3][3] = {{S[0], S[1], S[2]}, {S[1], S[3], S[4]}, {S[2], S[4], S[5]}};

        real Vd[12];  // the three columns of the view matrix the chain uses, rows 0..2
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            Vd[3 * k] = V[4 * k];
            Vd[3 * k + 1] = V[4 * k + 1];
            Vd[3 * k + 2] = V[4 * k + 2];
        }
        const real xd = x, yd = y, zd = z;
        const real pvx = Vd[0] * xd + Vd[3] * yd + Vd[6] * zd + (real)V[12];
        const real pvy = Vd[1] * xd + Vd[4] * yd + Vd[7] * zd + (real)V[13];
        const real tz = Vd[2] * xd + Vd[5] * yd + Vd[8] * zd + (real)V[14];
        const real fx = (real)f.W / (2. * (real)f.tanfovx), fy = (real)f.H / (2. * (real)f.tanfovy);
        const real limx = 1.3 * (real)f.tanfovx, limy = 1.3 * (real)f.tanfovy;
        const real itz = 1. / tz, itz2 = itz * itz;
        const real rx = pvx * itz, ry = pvy * itz;
        const real cx = rx > limx ? limx : rx < -limx ? -limx : 0.;  // non-zero: clamped to +-lim
        const real cy = ry > limy ? limy : ry < -limy ? -limy : 0.;
        const real tx = cx != 0. ? cx * tz : pvx, ty = cy != 0. ? cy * tz : pvy;
        const real J00 = fx * itz, J02 = -(fx * tx) * itz2;
        const real J11 = fy * itz, J12 = -(fy * ty) * itz2;
        real a0[3], a1[3], Sa0[3], Sa1[3];
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            a0[k] = J00 * Vd[3 * k] + J02 * Vd[3 * k + 2];
            a1[k] = J11 * Vd[3 * k + 1] + J12 * Vd[3 * k + 2];
        }
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            Sa0[k] = Sm[k][0] * a0[0] + Sm[k][1] * a0[1] + Sm[k][2] * a0[2];
            Sa1[k] = Sm[k][0] * a1[0] + Sm[k][1] * a1[1] + Sm[k][2] * a1[2];
        }
        const real ca = a0[0] * Sa0[0] + a0[1] * Sa0[1] + a0[2] * Sa0[2] + 0.3;
        const real cb = a0[0] * Sa1[0] + a0[1] * Sa1[1] + a0[2] * Sa1[2];
        const real cc = a1[0] * Sa1[0] + a1[1] * Sa1[1] + a1[2] * Sa1[2] + 0.3;
        const real D = 1. / (ca * cc - cb * cb), D2 = D * D;
        // conic = (cc, -cb, ca) / det; with det - ca cc = -cb^2 the derivatives need no difference of near-equal terms
        const real gAd = gA, gBd = gB, gCd = gC;
        const real d_ca = D2 * (-cc * cc * gAd + cb * cc * gBd - cb * cb * gCd);
        const real d_cb = D2 * (2. * cb * cc * gAd - (ca * cc + cb * cb) * gBd + 2. * ca * cb * gCd);
        const real d_cc = D2 * (-cb * cb * gAd + ca * cb * gBd - ca * ca * gCd);
        // symmetric gradient of the 3-D covariance, packed with the off-diagonal entries counted once each
        real dS[3][3];
#pragma unroll
        for (int k = 0; k < 3; ++k)
#pragma unroll
            for (int l = 0; l < 3; ++l)
                dS[k][l] = d_ca * a0[k] * a0[l] + d_cb * 0.5 * (a0[k] * a1[l] + a1[k] * a0[l]) + d_cc * a1[k] * a1[l];
        real d_J00 = 0., d_J02 = 0., d_J11 = 0., d_J12 = 0.;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const real d_a0 = 2. * d_ca * Sa0[k] + d_cb * Sa1[k];
            const real d_a1 = 2. * d_cc * Sa1[k] + d_cb * Sa0[k];
            d_J00 += d_a0 * Vd[3 * k];
            d_J02 += d_a0 * Vd[3 * k + 2];
            d_J11 += d_a1 * Vd[3 * k + 1];
            d_J12 += d_a1 * Vd[3 * k + 2];
        }
        const real itz3 = itz2 * itz;
        const real d_tx = d_J02 * (-fx * itz2), d_ty = d_J12 * (-fy * itz2);
        const real d_tz = d_J00 * (-fx * itz2) + d_J11 * (-fy * itz2) + d_J02 * (2. * fx * tx * itz3) +
                          d_J12 * (2. * fy * ty * itz3);
        const real d_pvx = cx != 0. ? 0. : d_tx, d_pvy = cy != 0. ? 0. : d_ty;
        const real d_pvz = d_tz + cx * d_tx + cy * d_ty + (real)g_depth;
#pragma unroll
        for (int k = 0; k < 3; ++k)
            dmean[k] += (float)(Vd[3 * k] * d_pvx + Vd[3 * k + 1] * d_pvy + Vd[3 * k + 2] * d_pvz);

        if (g.cov3D_precomp) {
            dcov[0] = (float)dS[0][0]; dcov[1] = (float)(2. * dS[0][1]); dcov[2] = (float)(2. * dS[0][2]);
            dcov[3] = (float)dS[1][1]; dcov[4] = (float)(2. * dS[1][2]); dcov[5] = (float)dS[2][2];
        } else {
            // Sigma = L L^T with L = R diag(s): dL = 2 dS L
            real dR[3][3];
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                real ds = 0.;
#pragma unroll
                for (int a = 0; a < 3; ++a) {
                    const real dL = 2. * (dS[a][0] * R[0][k] + dS[a][1] * R[1][k] + dS[a][2] * R[2][k]) * s[k];
                    ds += dL * R[a][k];
                    dR[a][k] = dL * s[k];
                }
                dscale[k] = (float)(ds * (real)f.scale_modifier);
            }
            const real r = q[0], qx = q[1], qy = q[2], qz = q[3];
            drot[0] = (float)(2. * (-qz * dR[0][1] + qy * dR[0][2] + qz * dR[1][0] - qx * dR[1][2] - qy * dR[2][0] + qx * dR[2][1]));
            drot[1] = (float)(2. * (qy * dR[0][1] + qz * dR[0][2] + qy * dR[1][0] - 2. * qx * dR[1][1] - r * dR[1][2] +
                                    qz * dR[2][0] + r * dR[2][1] - 2. * qx * dR[2][2]));
            drot[2] = (float)(2. * (-2. * qy * dR[0][0] + qx * dR[0][1] + r * dR[0][2] + qx * dR[1][0] + qz * dR[1][2] -
                                    r * dR[2][0] + qz * dR[2][1] - 2. * qy * dR[2][2]));
            drot[3] = (float)(2. * (-2. * qz * dR[0][0] - r * dR[0][1] + qx * dR[0][2] + r * dR[1][0] - 2. * qz * dR[1][1] +
                                    qy * dR[1][2] + qx * dR[2][0] + qy * dR[2][1]));
        }

        // ---- colour: view direction, SH basis and its gradient ----
        if (g.shs) {
            const float dirx = x - f.campos[0], diry = y - f.campos[1], dirz = z - f.campos[2];
            inv_len = 1.0f / sqrtf(dirx * dirx + diry * diry + dirz * dirz);
            nx = dirx * inv_len;
            ny = diry * inv_len;
            nz = dirz * inv_len;
            sh_basis_grad(f.sh_degree, nx, ny, nz, b, bx, by, bz);
            K = (f.sh_degree + 1) * (f.sh_degree + 1);
            // the forward pass clamped the colour at zero: a zero in the record means no gradient
            const float* __restrict__ rec = records + si * kRecordFloats;
            gcol[0] = rec[6] > 0.0f ? dcol[0] : 0.0f;
            gcol[1] = rec[7] > 0.0f ? dcol[1] : 0.0f;
            gcol[2] = rec[8] > 0.0f ? dcol[2] : 0.0f;
        }
    }

    // ---- SH coefficients: their part of the mean's gradient (through the view direction), and their own ----
    if (g.shs) {
        if (fetch_sh) {
            // coefficients of the wavefront's Gaussians: all loads in flight together, then into the rows (slots
            // past the last Gaussian re-read it)
            float4 sh_in[12];
#pragma unroll
            for (int it = 0; it < 12; ++it) {
                const int q4 = it * 64 + lane;
                const size_t e = min(wave_first + (size_t)(q4 / 12), (size_t)g.P - 1);
                sh_in[it] = reinterpret_cast<const float4*>(g.shs + e * 48)[q4 % 12];
            }
#pragma unroll
            for (int it = 0; it < 12; ++it) {
                const int q4 = it * 64 + lane;
                mine[(q4 / 12) * (kShStride / 4) + q4 % 12] = sh_in[it];
            }
            wave_lds_sync();
        }
        if (alive && f.sh_degree > 0) {
            const float* __restrict__ sh = staged ? my_row : g.shs + si * M * 3;
            float dn[3] = {0.f, 0.f, 0.f};
#pragma unroll
            for (int k = 1; k < 16; ++k) {
                if (k < K) {
                    const float t = gcol[0] * sh[3 * k] + gcol[1] * sh[3 * k + 1] + gcol[2] * sh[3 * k + 2];
                    dn[0] += t * bx[k];
                    dn[1] += t * by[k];
                    dn[2] += t * bz[k];
                }
            }
            const float dot = nx * dn[0] + ny * dn[1] + nz * dn[2];
            dmean[0] += (dn[0] - nx * dot) * inv_len;
            dmean[1] += (dn[1] - ny * dot) * inv_len;
            dmean[2] += (dn[2] - nz * dot) * inv_len;
        }
        if (out.shs) {
            if (staged) {
                wave_lds_sync();  // rows were read above
#pragma unroll
                for (int k = 0; k < 16; ++k) {
                    const float bk = (alive && k < K) ? b[k] : 0.0f;
                    my_row[3 * k] = bk * gcol[0];
                    my_row[3 * k + 1] = bk * gcol[1];
                    my_row[3 * k + 2] = bk * gcol[2];
                }
                wave_lds_sync();
#pragma unroll
                for (int it = 0; it < 12; ++it) {
                    const int q4 = it * 64 + lane;
                    const int e = q4 / 12, m = q4 % 12;
                    if (e < count) reinterpret_cast<float4*>(out.shs + (wave_first + e) * 48)[m] = mine[e * (kShStride / 4) + m];
                }
            } else if (valid) {
                float* __restrict__ o = out.shs + si * M * 3;
#pragma unroll
                for (int k = 0; k < 16; ++k) {
                    if (k < M) {
                        const float bk = (alive && k < K) ? b[k] : 0.0f;
                        o[3 * k] = bk * gcol[0];
                        o[3 * k + 1] = bk * gcol[1];
                        o[3 * k + 2] = bk * gcol[2];
                    }
                }
                for (int k = 48; k < 3 * M; ++k) o[k] = 0.0f;  // coefficient rows beyond degree 3
            }
        }
    }
    if (!valid) return;

    if (out.means3D)
#pragma unroll
        for (int k = 0; k < 3; ++k) out.means3D[3 * si + k] = dmean[k];
    if (out.means2D)
#pragma unroll
        for (int k = 0; k < 3; ++k) out.means2D[3 * si + k] = d2[k];
    if (out.opacities) out.opacities[i] = dop;
    if (out.colors_precomp)
#pragma unroll
        for (int k = 0; k < 3; ++k) out.colors_precomp[3 * si + k] = dcol[k];
    if (out.scales)
#pragma unroll
        for (int k = 0; k < 3; ++k) out.scales[3 * si + k] = dscale[k];
    if (out.rotations)
#pragma unroll
        for (int k = 0; k < 4; ++k) out.rotations[4 * si + k] = drot[k];
    if (out.cov3D_precomp)
#pragma unroll
        for (int k = 0; k < 6; ++k) out.cov3D_precomp[6 * si + k] = dcov[k];
}

}  // namespace

int launch_render_backward(const FrameArgs& f, const gs355_gaussians& g, const gs355_header* header,
                           const uint32_t* ranges, const uint32_t* values, const float* records,
                           const uint32_t* tiles_touched, const uint64_t* rects, const gs355_backward_inputs& in,
                           uint32_t* first_key, uint32_t* scan_tmp, float* key_grads, const gs355_gradients& out,
                           hipStream_t s)
{
    if (g.P == 0) return GS355_OK;
    int rc = launch_exclusive_scan(tiles_touched, first_key, (size_t)g.P, scan_tmp, s);
    if (rc) return rc;
    const int tiles = f.grid_x * f.grid_y;
    hipLaunchKernelGGL(blend_backward_kernel, dim3(tiles), dim3(256), 0, s, f, header, ranges, values, records,
                       in.image, in.depth, in.alpha, in.dL_dimage, in.dL_ddepth, in.dL_dalpha, rects, first_key,
                       key_grads);
    GS355_CHECK_LAUNCH("blend backward");
    const bool staged = g.shs != nullptr && f.sh_coeffs == 16 && (reinterpret_cast<uintptr_t>(g.shs) & 15u) == 0 &&
                        (out.shs == nullptr || (reinterpret_cast<uintptr_t>(out.shs) & 15u) == 0);
    const dim3 grid((g.P + 255) / 256), block(256);
    if (!staged)
        hipLaunchKernelGGL(preprocess_backward_kernel<0>, grid, block, 0, s, f, g, in.radii, records, tiles_touched,
                           first_key, key_grads, out);
    else if (f.sh_degree == 0)
        hipLaunchKernelGGL(preprocess_backward_kernel<1>, grid, block, 0, s, f, g, in.radii, records, tiles_touched,
                           first_key, key_grads, out);
    else
        hipLaunchKernelGGL(preprocess_backward_kernel<2>, grid, block, 0, s, f, g, in.radii, records, tiles_touched,
                           first_key, key_grads, out);
    GS355_CHECK_LAUNCH("preprocess backward");
    return GS355_OK;
}

}  // namespace gs355
