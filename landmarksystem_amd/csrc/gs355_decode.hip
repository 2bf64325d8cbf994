// Scaffold-GS / Octree-GS anchor decode on the gfx950 matrix cores.
//
// Replaces AnchorDecoder.forward in eval mode (landmark/nerf_components/
// model_components/fields/anchor_decoder.py:108-242; MLP shapes :79-104; the
// reference's fused twin is fused_anchor_decoder.py:69-244, whose CUDA kernels
// are an empty submodule) for the configuration the Scaffold-GS model builds
// (scaffold_gs/gs_model.py:126-134): no feature bank, no level / appearance
// inputs, three two-layer MLPs  [feat(32) | view(3) | dist(1)] -> 32 -> ReLU ->
// {n, 7n, 3n}  with tanh / none / sigmoid, mask opacity > 0, then
// scaling = anchor_scaling[3:6] * sigmoid(cov[0:3]), rot = normalize(cov[3:7]),
// xyz = anchor + offset * anchor_scaling[0:3].
//
// Everything is computed transposed so that the two layers chain without any
// data movement: weights are the A operand (rows = output units), 32 anchors
// are the columns of one v_mfma_f32_32x32x16_f16 tile (the gfx950 form: 16
// k values per instruction, 8 per lane), and the accumulator layout of layer 1
// (lane = anchor, registers = hidden units 8b+4*half+t) feeds layer 2's B
// operand directly: which k value sits in which of a lane's 8 slots is free
// as long as both operands agree, so the weights of layer 2 are simply loaded
// in the order the accumulator registers come in.
//
// Precision: weights and anchor features are rounded to fp16 (exact for fp16
// checkpoints); the four fp32-only inputs (view direction, distance) and the
// hidden activations enter the matrix cores as hi + lo fp16 pairs, so the
// result carries fp32-level accuracy with fp32 accumulation.
//
// Work follows the visible anchors: a wavefront takes runs of 128 consecutive
// anchors, packs the visible ones (in order) into dense tiles of 32 and decodes
// those only.
//
// Output order is the reference's boolean-mask order: row-major over (visible
// anchor, offset).  Two launches: count kept offsets per anchor (opacity head
// only) -> exclusive scan -> emit (all heads; the opacity head is recomputed
// with the identical instruction sequence, so counts and emission agree).
#include <atomic>

#include "gs355_internal.h"

namespace gs355 {

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kFeat = 32;

struct DecodeArgs {
    int A, n;       // anchors, offsets per anchor
    int in_dim[3];  // 35 or 36 per head (opacity, cov, color)
    const float* anchor;
    const float* feat;
    const float* offset;
    const float* scaling;
    const uint8_t* visible;
    const float* campos;
    const float* w0[3];
    const float* b0[3];
    const float* w1[3];
    const float* b1[3];
};

__device__ __forceinline__ half8_t to_half8(const float v[8])
{
    half8_t h;
#pragma unroll
    for (int j = 0; j < 8; ++j) h[j] = (_Float16)v[j];
    return h;
}

// Eight entries of row `row` of a [rows x cols] row-major fp32 weight matrix, as one lane's share of an A
// operand: slots 0..3 hold columns ka..ka+3, slots 4..7 columns kb..kb+3 (zero outside the matrix).  Loads are
// unconditional at clamped (in-range) positions and masked afterwards, so that none of them waits for another:
// the fragments of a head are fetched with all loads in flight together.
__device__ __forceinline__ half8_t weight_fragment(const float* __restrict__ w, int rows, int cols, int row, int ka,
                                                   int kb, bool enable = true)
{
    float v[8];
    const int r = min(row, rows - 1);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = w[(size_t)r * cols + min((j < 4 ? ka : kb - 4) + j, cols - 1)];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (enable && row < rows && (j < 4 ? ka : kb - 4) + j < cols) ? v[j] : 0.0f;
    return to_half8(v);
}

// Bias for an accumulator: register v = 4b + t holds row 8b + 4*half + t.  `bias` is the head's bias vector
// staged in LDS, zero-padded to a multiple of 32 rows.
__device__ __forceinline__ floatx16 bias_rows(const float* bias, int row0, int half)
{
    floatx16 c;
#pragma unroll
    for (int v = 0; v < 16; ++v) c[v] = bias[row0 + 8 * (v >> 2) + 4 * half + (v & 3)];
    return c;
}

// Weight fragments of one head, held in registers for the whole kernel.
//   layer 1, k-steps 0 and 1: the 32 anchor features, slot j of half h <-> feature 16s + 8h + j
//   layer 1, k-step 2:        the four fp32-only inputs twice on half 0 (slots 0..3 meet their hi parts, slots
//                             4..7 their lo parts, both against W0[:, 32..35]); half 1 is zero
//   layer 2, k-step s:        slot j of half h <-> hidden unit 16s + 4h + j (j < 4) or 16s + 8 + 4h + (j - 4),
//                             the units held by accumulator registers 8s..8s+7 of that lane
template <int kTiles>
struct HeadWeights {
    half8_t w0[3];          // layer 1: [32 x in]
    half8_t w1[kTiles][2];  // layer 2: [outputs x 32] in row tiles of 32
};

template <int kTiles>
__device__ __forceinline__ void load_head(const DecodeArgs& d, int head, int outputs, int row, int half,
                                          HeadWeights<kTiles>& w)
{
    const int in = d.in_dim[head];
#pragma unroll
    for (int s = 0; s < 2; ++s) w.w0[s] = weight_fragment(d.w0[head], kFeat, in, row, 16 * s + 8 * half, 16 * s + 8 * half + 4);
    w.w0[2] = weight_fragment(d.w0[head], kFeat, in, row, 32, 32, half == 0);
#pragma unroll
    for (int r = 0; r < kTiles; ++r)
#pragma unroll
        for (int s = 0; s < 2; ++s)
            w.w1[r][s] = weight_fragment(d.w1[head], outputs, kFeat, 32 * r + row, 16 * s + 4 * half,
                                         16 * s + 8 + 4 * half);
}

// One head for one tile of 32 anchors: returns up to kTiles accumulators of the
// second layer (rows = outputs 32r + 8b + 4*half + t, column = this lane's anchor).
template <int kTiles>
__device__ __forceinline__ void run_head(const HeadWeights<kTiles>& w, const float* bias0, const float* bias1,
                                         const half8_t X[3], int half, floatx16 out[kTiles])
{
    // layer 1: hidden = W0 [32 x in] * X^T + b0
    floatx16 h = bias_rows(bias0, 0, half);
#pragma unroll
    for (int s = 0; s < 3; ++s) h = __builtin_amdgcn_mfma_f32_32x32x16_f16(w.w0[s], X[s], h, 0, 0, 0);
    // ReLU, then hi/lo split: registers 8s..8s+7 are the B operand of k-step s
    half8_t hh[2], hl[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        float r[8], lo[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            r[j] = fmaxf(h[8 * s + j], 0.0f);
            const _Float16 top = (_Float16)r[j];
            lo[j] = r[j] - (float)top;
        }
        hh[s] = to_half8(r);
        hl[s] = to_half8(lo);
    }
    // layer 2: out = W1 [outputs x 32] * hidden + b1
#pragma unroll
    for (int r = 0; r < kTiles; ++r) {
        floatx16 c = bias_rows(bias1, 32 * r, half);
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(w.w1[r][s], hh[s], c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(w.w1[r][s], hl[s], c, 0, 0, 0);
        }
        out[r] = c;
    }
}

// Store the rows of an accumulator that exist (< outputs) into the tile's LDS block.
__device__ __forceinline__ void store_rows(float* __restrict__ dst_anchor, int base, int outputs, int row0, int half,
                                           const floatx16& c)
{
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int r = row0 + 8 * (v >> 2) + 4 * half + (v & 3);
        if (r < outputs) dst_anchor[base + r] = c[v];
    }
}

// Per-lane inputs of one tile of 32 anchors.
template <bool kCountOnly>
struct TileInputs {
    float4 f[4] = {};          // features 16s + 8*half .. +7 in f[2s], f[2s+1], s = 0..1
    float pos[3] = {0.f, 0.f, 0.f};
    float sc3[3] = {0.f, 0.f, 0.f};
    uint32_t first_slot = 0;
    float ofv[kCountOnly ? 1 : 5][3] = {};
};

// A wavefront takes runs of kRun consecutive anchors, packs the visible ones (in order) into dense tiles of 32
// and runs the MLPs on those only: the work follows the number of visible anchors, not of anchors.
constexpr int kRun = 128;

template <bool kCountOnly>
__global__ __launch_bounds__(256) void decode_kernel(DecodeArgs d, uint32_t* __restrict__ counts,
                                                     const uint32_t* __restrict__ offsets, uint32_t capacity,
                                                     float* __restrict__ xyz, float* __restrict__ color,
                                                     float* __restrict__ opacity, float* __restrict__ scaling_out,
                                                     float* __restrict__ rot)
{
    // per wavefront: [32 anchors][stride] floats; stride odd -> conflict-free column access.  Emit pass: the
    // 11n head outputs of an anchor, then its scaling (6), position (3) and first output slot (1).
    constexpr int kStrideMax = kCountOnly ? 11 : 123;
    constexpr int kListFloats = kCountOnly ? 0 : 160;  // 320 16-bit item numbers after the anchors' rows
    constexpr int kRunFloats = kRun / 4;                // kRun 8-bit positions of the run's visible anchors
    __shared__ float s_out[4][32 * kStrideMax + kListFloats + kRunFloats];

    // biases of the three heads, zero-padded: b0 at [head*32], b1 of opacity / cov / colour at 96 / 128 / 224
    __shared__ float s_bias[256];

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, half = lane >> 5, col = lane & 31;
    const int n = d.n;
    {
        const int t = threadIdx.x;
        float v = 0.0f;
        if (t < 96) v = d.b0[t >> 5][t & 31];
        else if (t < 128) v = (t - 96) < n ? d.b1[0][t - 96] : 0.0f;
        else if (t < 224) v = (t - 128) < 7 * n ? d.b1[1][t - 128] : 0.0f;
        else v = (t - 224) < 3 * n ? d.b1[2][t - 224] : 0.0f;
        s_bias[t] = v;
    }
    __syncthreads();
    HeadWeights<1> w_op;
    load_head<1>(d, 0, n, col, half, w_op);
    HeadWeights<3> w_cov;
    HeadWeights<1> w_col;
    if (!kCountOnly) {
        load_head<3>(d, 1, 7 * n, col, half, w_cov);
        load_head<1>(d, 2, 3 * n, col, half, w_col);
    }
    const int stride = kCountOnly ? 11 : 11 * n + 13;
    const int items = 32 * n;  // (anchor, offset) pairs of a tile: item = anchor_in_tile * n + offset
    const int inv_n = (65536 + n - 1) / n;  // item / n == (item * inv_n) >> 16 for item < 32 n, n <= 10
    const uint64_t lanes_below = (1ull << lane) - 1ull;
    const int runs = (d.A + kRun - 1) / kRun;
    float* __restrict__ mine = s_out[wave];
    uint8_t* __restrict__ run_list = reinterpret_cast<uint8_t*>(mine + 32 * kStrideMax + kListFloats);
    const float cx = d.campos[0], cy = d.campos[1], cz = d.campos[2];

    for (int run = blockIdx.x * 4 + wave; run < runs; run += gridDim.x * 4) {
      // positions (within the run) of its visible anchors, in order: lane covers anchors lane and 64 + lane
      const int base = run * kRun;
      const int a0 = base + lane, a1 = base + 64 + lane;
      const bool v0 = a0 < d.A && d.visible[a0] != 0, v1 = a1 < d.A && d.visible[a1] != 0;
      const uint64_t m0 = __ballot(v0), m1 = __ballot(v1);
      const int n0 = __popcll(m0), nvis = n0 + __popcll(m1);
      if (kCountOnly) {  // anchors that are not decoded keep nothing
          if (!v0 && a0 < d.A) counts[a0] = 0;
          if (!v1 && a1 < d.A) counts[a1] = 0;
      }
      if (nvis == 0) continue;  // uniform
      if (v0) run_list[__popcll(m0 & lanes_below)] = (uint8_t)lane;
      if (v1) run_list[n0 + __popcll(m1 & lanes_below)] = (uint8_t)(64 + lane);
      wave_lds_sync();
      for (int first = 0; first < nvis; first += 32) {  // dense tiles of the run
        const bool vis = first + col < nvis;  // lanes l and l+32 share entry first + l
        const int a = vis ? base + (int)run_list[first + col] : 0;
        const uint64_t any = __ballot(vis);  // bits l and l + 32 belong to entry l of the tile
        // Everything the tile needs from global memory is requested here, before the first use.
        TileInputs<kCountOnly> in;
        if (vis) {
            const float4* __restrict__ f4 = reinterpret_cast<const float4*>(d.feat + (size_t)a * kFeat);
#pragma unroll
            for (int s = 0; s < 2; ++s) {  // features 16s + 8*half .. +7
                in.f[2 * s] = f4[4 * s + 2 * half];
                in.f[2 * s + 1] = f4[4 * s + 2 * half + 1];
            }
#pragma unroll
            for (int k = 0; k < 3; ++k) in.pos[k] = d.anchor[3 * (size_t)a + k];
        }
        if constexpr (!kCountOnly) {
            // half 0: scaling[0..2] (offset scale), half 1: scaling[3..5] (Gaussian scale)
            if (vis) {
#pragma unroll
                for (int k = 0; k < 3; ++k) in.sc3[k] = d.scaling[6 * (size_t)a + 3 * half + k];
            }
            if (vis) in.first_slot = offsets[a];  // entry 0's value is the tile's first output slot
            // the learned offsets of the items this lane's position covers (item = entry * n + offset)
#pragma unroll
            for (int r = 0; r < 5; ++r) {
                const int it = r * 64 + lane;
                const int al = (it * inv_n) >> 16;
                const bool want = it < items && ((any >> al) & 1ull);
                const int ai = want ? base + (int)run_list[first + al] : 0;
                const float* __restrict__ of = d.offset + ((size_t)ai * n + (want ? it - al * n : 0)) * 3;
#pragma unroll
                for (int k = 0; k < 3; ++k) in.ofv[r][k] = want ? of[k] : 0.0f;
            }
        }
        // B operand: X^T, column = anchor; slots as described at HeadWeights
        half8_t X[3];
        const float ax = in.pos[0], ay = in.pos[1], az = in.pos[2];
        {
            float x8[8];
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                x8[0] = in.f[2 * s].x, x8[1] = in.f[2 * s].y, x8[2] = in.f[2 * s].z, x8[3] = in.f[2 * s].w;
                x8[4] = in.f[2 * s + 1].x, x8[5] = in.f[2 * s + 1].y, x8[6] = in.f[2 * s + 1].z, x8[7] = in.f[2 * s + 1].w;
                X[s] = to_half8(x8);  // all zero for an invisible anchor
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) x8[j] = 0.0f;
            if (vis && half == 0) {
                float vx = ax - cx, vy = ay - cy, vz = az - cz;
                const float dist = sqrtf(vx * vx + vy * vy + vz * vz);
                vx /= dist;
                vy /= dist;
                vz /= dist;
                const float in4[4] = {vx, vy, vz, dist};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const _Float16 top = (_Float16)in4[t];
                    x8[t] = (float)top;
                    x8[4 + t] = in4[t] - (float)top;
                }
            }
            X[2] = to_half8(x8);
        }

        // ---- opacity head ----
        floatx16 op[1];
        run_head<1>(w_op, s_bias, s_bias + 96, X, half, op);
        // the mask opacity > 0 is the sign of the pre-activation (tanh is odd, monotone and tanh(x) = x for the
        // smallest floats), so tanh itself is only evaluated for the offsets that are kept
        store_rows(mine + col * stride, 0, n, 0, half, op[0]);
        if (kCountOnly) {
            wave_lds_sync();
            if (half == 0 && vis) {
                uint32_t kept = 0;
                for (int m = 0; m < n; ++m) kept += mine[col * stride + m] > 0.0f ? 1u : 0u;
                counts[a] = kept;
            }
            wave_lds_sync();
            continue;
        }

        // ---- covariance and colour heads ----
        floatx16 cv[3];
        run_head<3>(w_cov, s_bias + 32, s_bias + 128, X, half, cv);
#pragma unroll
        for (int r = 0; r < 3; ++r) store_rows(mine + col * stride, n, 7 * n, 32 * r, half, cv[r]);
        floatx16 cl[1];
        run_head<1>(w_col, s_bias + 64, s_bias + 224, X, half, cl);
        store_rows(mine + col * stride, 8 * n, 3 * n, 0, half, cl[0]);
        {
            float* __restrict__ extra = mine + col * stride + 11 * n;
#pragma unroll
            for (int k = 0; k < 3; ++k) extra[3 * half + k] = in.sc3[k];
            if (half == 0) {
                extra[6] = ax;
                extra[7] = ay;
                extra[8] = az;
                reinterpret_cast<uint32_t*>(extra)[9] = in.first_slot;
            }
        }
        wave_lds_sync();

        // ---- compact the kept (anchor, offset) items of the tile: about one in five survives the mask, and the
        // activations below are the expensive part, so they run on dense wavefronts of survivors only ----
        uint16_t* __restrict__ list = reinterpret_cast<uint16_t*>(mine + 32 * stride);  // [32 n] item numbers
        uint32_t total = 0;
#pragma unroll
        for (int r = 0; r < 5; ++r) {
            if (r * 64 >= items) break;  // uniform
            const int it = r * 64 + lane;
            bool kept = false;
            if (it < items) {
                const int al = (it * inv_n) >> 16, m = it - al * n;
                kept = ((any >> al) & 1ull) && mine[al * stride + m] > 0.0f;
            }
            const uint64_t b = __ballot(kept);
            if (kept) list[total + (uint32_t)__popcll(b & lanes_below)] = (uint16_t)it;
            total += (uint32_t)__popcll(b);
        }
        wave_lds_sync();

        // Items are numbered anchor-major and the slots come from an exclusive scan of the per-anchor counts, so
        // the survivors of a tile occupy consecutive output slots from the slot of its first anchor: lanes write
        // consecutive addresses.  No global reads in here: the learned offsets sit in registers of the lane that
        // requested them (item = round * 64 + lane) and are fetched across lanes.
        const uint32_t tile_slot = reinterpret_cast<const uint32_t*>(mine)[11 * n + 9];
        for (uint32_t s0 = 0; s0 < total; s0 += 64) {  // uniform
            const uint32_t s = s0 + lane;
            const bool live = s < total;
            const int it = live ? (int)list[s] : 0;
            float off3[3] = {0.f, 0.f, 0.f};
#pragma unroll
            for (int r = 0; r < 5; ++r) {
#pragma unroll
                for (int k = 0; k < 3; ++k) {
                    const float got = __shfl(in.ofv[r][k], it & 63, 64);
                    if ((it >> 6) == r) off3[k] = got;
                }
            }
            const uint32_t pos = tile_slot + s;
            if (!live || pos >= capacity) continue;  // the second cannot happen when capacity comes from the count pass
            const int al = (it * inv_n) >> 16, m = it - al * n;
            const float* __restrict__ o = mine + al * stride;
            const float* __restrict__ extra = o + 11 * n;
            const float* __restrict__ c7 = o + n + 7 * m;
            const float* __restrict__ c3 = o + 8 * n + 3 * m;
            opacity[pos] = tanhf(o[m]);
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                color[3 * (size_t)pos + k] = 1.0f / (1.0f + expf(-c3[k]));
                scaling_out[3 * (size_t)pos + k] = extra[3 + k] * (1.0f / (1.0f + expf(-c7[k])));
                xyz[3 * (size_t)pos + k] = extra[6 + k] + off3[k] * extra[k];
            }
            const float q0 = c7[3], q1 = c7[4], q2 = c7[5], q3 = c7[6];
            const float norm = fmaxf(sqrtf(q0 * q0 + q1 * q1 + q2 * q2 + q3 * q3), 1e-12f);
            rot[4 * (size_t)pos + 0] = q0 / norm;
            rot[4 * (size_t)pos + 1] = q1 / norm;
            rot[4 * (size_t)pos + 2] = q2 / norm;
            rot[4 * (size_t)pos + 3] = q3 / norm;
        }
        wave_lds_sync();
      }
    }
}

}  // namespace

struct DecodeLaunch {
    DecodeArgs args;
};

static int fill_args(const gs355_decoder* dec, const gs355_anchors* an, DecodeArgs* out)
{
    if (!dec || !an) return set_error(GS355_EINVAL, "decoder / anchors is NULL");
    if (dec->feat_dim != kFeat)
        return set_error(GS355_EINVAL, "anchor decode supports feat_dim 32 only (got %d)", dec->feat_dim);
    if (dec->n_offsets < 1 || dec->n_offsets > 10)
        return set_error(GS355_EINVAL, "anchor decode supports 1..10 offsets per anchor (got %d)", dec->n_offsets);
    if (an->A < 0) return set_error(GS355_EINVAL, "A must be >= 0 (got %d)", an->A);
    for (int j = 0; j < 3; ++j) {
        if (dec->in_dim[j] != kFeat + 3 && dec->in_dim[j] != kFeat + 4)
            return set_error(GS355_EINVAL, "head %d: input width must be 35 or 36 (got %d)", j, dec->in_dim[j]);
        if (!dec->w0[j] || !dec->b0[j] || !dec->w1[j] || !dec->b1[j])
            return set_error(GS355_EINVAL, "head %d: weight or bias pointer is NULL", j);
    }
    if (an->A > 0 && (!an->anchor || !an->feat || !an->offset || !an->scaling || !an->visible_mask || !an->campos))
        return set_error(GS355_EINVAL, "anchor inputs must all be non-NULL");
    if (an->A > 0 && (reinterpret_cast<uintptr_t>(an->feat) & 15u) != 0)
        return set_error(GS355_EINVAL, "anchor features must be 16-byte aligned");
    DecodeArgs a;
    a.A = an->A;
    a.n = dec->n_offsets;
    a.anchor = an->anchor;
    a.feat = an->feat;
    a.offset = an->offset;
    a.scaling = an->scaling;
    a.visible = an->visible_mask;
    a.campos = an->campos;
    for (int j = 0; j < 3; ++j) {
        a.in_dim[j] = dec->in_dim[j];
        a.w0[j] = dec->w0[j];
        a.b0[j] = dec->b0[j];
        a.w1[j] = dec->w1[j];
        a.b1[j] = dec->b1[j];
    }
    *out = a;
    return GS355_OK;
}

// Persistent workgroups (4 wavefronts, each walking runs of kRun anchors): at most `cap` of them, about what
// the chip holds at once, so the weight fragments are fetched once per resident workgroup.
static dim3 decode_grid(int A, int cap)
{
    const int runs = (A + kRun - 1) / kRun;
    int blocks = (runs + 3) / 4;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return dim3(blocks);
}

}  // namespace gs355

using namespace gs355;

// ---- gs355_decode_count for callers that cannot allocate -----------------------------------------------------
// The scan's block sums live in a file-scope device array instead of a caller-provided scratch buffer.  Every
// GPU holds its own copy of the array at its own address; host code never uses the array's name as an address
// (it is a host-side stand-in) but the pointer hipGetSymbolAddress returns for the current device, resolved
// once per device and kept.
constexpr int32_t kStaticCountMaxAnchors = 1 << 24;
constexpr size_t kStaticScratchWords = ((size_t)kStaticCountMaxAnchors / kScanTile) * 3 + 8 + 64;
static __device__ __align__(256) uint32_t scratch[kStaticScratchWords];

constexpr int kMaxDevices = 64;
static std::atomic<uint32_t*> g_scratch_ptr[kMaxDevices];

static int static_scratch(uint32_t** out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return set_error(GS355_EHIP, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return set_error(GS355_EINVAL, "device index %d is outside [0, %d)", dev, kMaxDevices);
    uint32_t* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        void* q = nullptr;
        e = hipGetSymbolAddress(&q, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !q)
            return set_error(GS355_EHIP, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        p = static_cast<uint32_t*>(q);
        g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing threads resolve the same address
    }
    *out = p;
    return GS355_OK;
}

extern "C" {

int gs355_decode_scratch_bytes(int32_t A, size_t* bytes)
{
    if (!bytes) return set_error(GS355_EINVAL, "bytes is NULL");
    if (A < 0) return set_error(GS355_EINVAL, "A must be >= 0 (got %d)", A);
    *bytes = scan_tmp_words((size_t)A) * sizeof(uint32_t) + 256;
    return GS355_OK;
}

int gs355_decode_count(const gs355_decoder* dec, const gs355_anchors* an, uint32_t* counts, uint32_t* offsets,
                       void* scratch_buf, size_t scratch_bytes, void* stream)
{
    DecodeArgs a;
    int rc = fill_args(dec, an, &a);
    if (rc) return rc;
    if (a.A == 0) return GS355_OK;
    if (!counts || !offsets || !scratch_buf) return set_error(GS355_EINVAL, "counts / offsets / scratch is NULL");
    size_t need = 0;
    gs355_decode_scratch_bytes(a.A, &need);
    if (scratch_bytes < need)
        return set_error(GS355_ENOSPC, "decode scratch has %zu bytes, %zu needed", scratch_bytes, need);
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(decode_kernel<true>, decode_grid(a.A, 1024), dim3(256), 0, s, a, counts, (const uint32_t*)nullptr, 0u,
                       (float*)nullptr, (float*)nullptr, (float*)nullptr, (float*)nullptr, (float*)nullptr);
    GS355_CHECK_LAUNCH("decode: count");
    return launch_exclusive_scan(counts, offsets, (size_t)a.A, static_cast<uint32_t*>(scratch_buf), s);
}

int gs355_decode_count_static(const gs355_decoder* dec, const gs355_anchors* an, uint32_t* counts, uint32_t* offsets,
                              void* stream)
{
    DecodeArgs a;
    int rc = fill_args(dec, an, &a);
    if (rc) return rc;
    if (a.A > kStaticCountMaxAnchors)
        return set_error(GS355_ENOSPC, "gs355_decode_count_static handles at most %d anchors (got %d); use gs355_decode_count",
                         kStaticCountMaxAnchors, a.A);
    if (a.A == 0) return GS355_OK;
    if (!counts || !offsets) return set_error(GS355_EINVAL, "counts / offsets is NULL");
    static_assert(kStaticScratchWords * sizeof(uint32_t) >=
                      (((size_t)kStaticCountMaxAnchors + kScanTile - 1) / kScanTile * 3 + 8) * sizeof(uint32_t) + 256,
                  "static scratch covers the scan of the largest accepted anchor count");
    uint32_t* tmp = nullptr;
    if ((rc = static_scratch(&tmp))) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(decode_kernel<true>, decode_grid(a.A, 1024), dim3(256), 0, s, a, counts, (const uint32_t*)nullptr, 0u,
                       (float*)nullptr, (float*)nullptr, (float*)nullptr, (float*)nullptr, (float*)nullptr);
    GS355_CHECK_LAUNCH("decode: count");
    // the scan writes every block sum before it reads it: nothing in the array has to start at zero
    return launch_exclusive_scan(counts, offsets, (size_t)a.A, tmp, s);
}

int gs355_decode_emit(const gs355_decoder* dec, const gs355_anchors* an, const uint32_t* offsets, int64_t capacity,
                      const gs355_decoded* out, void* stream)
{
    DecodeArgs a;
    int rc = fill_args(dec, an, &a);
    if (rc) return rc;
    if (a.A == 0 || capacity == 0) return GS355_OK;
    if (capacity < 0 || capacity > 0xFFFFFFFFll)
        return set_error(GS355_EINVAL, "capacity must be in [0, 2^32) (got %lld)", (long long)capacity);
    if (!offsets) return set_error(GS355_EINVAL, "offsets is NULL");
    if (!out || !out->xyz || !out->color || !out->opacity || !out->scaling || !out->rot)
        return set_error(GS355_EINVAL, "decoded outputs must all be non-NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(decode_kernel<false>, decode_grid(a.A, 512), dim3(256), 0, s, a, (uint32_t*)nullptr, offsets,
                       (uint32_t)capacity, out->xyz, out->color, out->opacity, out->scaling, out->rot);
    GS355_CHECK_LAUNCH("decode: emit");
    return GS355_OK;
}

}  // extern "C"
