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
// Precision: fp32 accumulation throughout.  Weights and anchor features that
// fp16 holds exactly (fp16 checkpoints) enter the matrix cores as one fp16
// operand; general fp32 weights and features, the four fp32-only inputs (view
// direction, distance) and the hidden activations enter as hi + lo fp16
// pairs (22 significant bits; the lo x lo products, 2^-22 of a term, are
// left out), so the result carries fp32-level accuracy either way.  The low
// parts of the weights live in LDS, their high parts in registers.
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
    const float* level;  // per-anchor level: the fourth fp32-only input instead of the distance (add_level), or NULL
    int split_feat;      // features enter as hi + lo fp16 pairs (fp32 features that fp16 cannot represent)
    int weights_lo;      // weights enter as hi + lo fp16 pairs (fp32 weights that fp16 cannot represent)
    const float* w0[3];
    const float* b0[3];
    const float* w1[3];
    const float* b1[3];
    // one-call decode (gs355_decode): the count pass leaves per-run totals behind, a one-workgroup scan turns
    // them into run bases, and the emit pass (which recomputes the opacity head: matrix instructions are cheap
    // here, registers and memory requests are not) places its Gaussians from those instead of per-anchor offsets
    uint2* run_totals;       // [runs] (kept offsets, visible anchors) per run of kRun anchors, or NULL
    const uint2* run_base;   // [runs] exclusive prefix of run_totals, or NULL
    float* neural_opacity;   // [A_vis * n] tanh of every pre-activation, in visible-anchor order, or NULL
    uint8_t* kept_mask;      // [A_vis * n] pre-activation > 0, or NULL
};

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

// Eight floats as hi + lo fp16 pairs (hi = the value rounded to fp16, lo = what that rounding left over, rounded
// to fp16), converted two at a time (one packed conversion per pair and direction).
__device__ __forceinline__ void split_half8(const float v[8], half8_t& hi, half8_t& lo)
{
    half2_t h[4], l[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float2_t x = {v[2 * j], v[2 * j + 1]};
        h[j] = __builtin_convertvector(x, half2_t);
        l[j] = __builtin_convertvector(x - __builtin_convertvector(h[j], float2_t), half2_t);
    }
    hi = (half8_t){h[0][0], h[0][1], h[1][0], h[1][1], h[2][0], h[2][1], h[3][0], h[3][1]};
    lo = (half8_t){l[0][0], l[0][1], l[1][0], l[1][1], l[2][0], l[2][1], l[3][0], l[3][1]};
}

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
// `lo`: what the fp16 rounding of each entry left over, itself rounded to fp16.
__device__ __forceinline__ half8_t weight_fragment(const float* __restrict__ w, int rows, int cols, int row, int ka,
                                                   int kb, bool enable = true, bool lo = false)
{
    float v[8];
    const int r = min(row, rows - 1);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = w[(size_t)r * cols + min((j < 4 ? ka : kb - 4) + j, cols - 1)];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (enable && row < rows && (j < 4 ? ka : kb - 4) + j < cols) ? v[j] : 0.0f;
    if (lo) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] -= (float)(_Float16)v[j];
    }
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
                                          HeadWeights<kTiles>& w, bool lo = false)
{
    const int in = d.in_dim[head];
#pragma unroll
    for (int s = 0; s < 2; ++s)
        w.w0[s] = weight_fragment(d.w0[head], kFeat, in, row, 16 * s + 8 * half, 16 * s + 8 * half + 4, true, lo);
    w.w0[2] = weight_fragment(d.w0[head], kFeat, in, row, 32, 32, half == 0, lo);
#pragma unroll
    for (int r = 0; r < kTiles; ++r)
#pragma unroll
        for (int s = 0; s < 2; ++s)
            w.w1[r][s] = weight_fragment(d.w1[head], outputs, kFeat, 32 * r + row, 16 * s + 4 * half,
                                         16 * s + 8 + 4 * half, true, lo);
}

// The low parts of a head's weight fragments, kept in LDS: [fragment][lane], fragments in the order w0[0..2],
// w1[0][0], w1[0][1], w1[1][0], ...  Every wavefront holds the same fragments in its lanes, so the workgroup shares
// one copy; `store_head_lo` is called by one wavefront per head.
template <int kTiles>
__device__ __forceinline__ void store_head_lo(const DecodeArgs& d, int head, int outputs, int row, int half, int lane,
                                              half8_t (*dst)[64], bool lo = true)
{
    HeadWeights<kTiles> w;
    load_head<kTiles>(d, head, outputs, row, half, w, lo);
#pragma unroll
    for (int s = 0; s < 3; ++s) dst[s][lane] = w.w0[s];
#pragma unroll
    for (int r = 0; r < kTiles; ++r)
#pragma unroll
        for (int s = 0; s < 2; ++s) dst[3 + 2 * r + s][lane] = w.w1[r][s];
}

// Store an accumulator's rows into the anchor's LDS row, head outputs at `base`.  Rows that do not exist
// (>= outputs; their accumulators hold zeros: masked weights, zero bias) are stored too, all of them at row
// `outputs` -- the first word after the head, which the stores that follow in program order overwrite (the next
// head's first output, or the anchor's scaling) -- so that no store is predicated: 16 conditional stores cost five
// instructions and a branch each.  A row tile that lies inside the head entirely takes constant offsets.
__device__ __forceinline__ void store_rows(float* __restrict__ dst_anchor, int base, int outputs, int row0, int half,
                                           const floatx16& c)
{
    float* __restrict__ dst = dst_anchor + base;
    const int lane_row = row0 + 4 * half;
    if (row0 + 32 <= outputs) {  // uniform
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[lane_row + 8 * (v >> 2) + (v & 3)] = c[v];
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) dst[min(lane_row + 8 * (v >> 2) + (v & 3), outputs)] = c[v];
    }
}

// One head for one tile of 32 anchors: the kTiles accumulators of the second layer (rows = outputs
// 32r + 8b + 4*half + t, column = this lane's anchor) go to the anchor's LDS row as soon as each is complete
// (one accumulator live at a time).
// `wlo`: the head's low weight fragments in LDS (kWLo), read right before their matrix instruction.
// kWInLds: the weight fragments themselves are read from `whi` (same order as `wlo`) instead of `w`: the
// covariance head's nine fragments would otherwise hold 36 registers for the whole kernel.
template <int kTiles, bool kSplit, bool kWLo, bool kWInLds = false>
__device__ __forceinline__ void run_head(const HeadWeights<kTiles>& w, const half8_t (*whi)[64],
                                         const half8_t (*wlo)[64], int lane,
                                         const float* bias0, const float* bias1, const half8_t X[kSplit ? 5 : 3],
                                         int half, float* __restrict__ dst_anchor, int base, int outputs)
{
    // layer 1: hidden = W0 [32 x in] * X^T + b0  (X[3], X[4]: the low parts of features that fp16 cannot hold)
    floatx16 h = bias_rows(bias0, 0, half);
    half8_t w0[3];
#pragma unroll
    for (int s = 0; s < 3; ++s) w0[s] = kWInLds ? whi[s][lane] : w.w0[s];
#pragma unroll
    for (int s = 0; s < 3; ++s) h = __builtin_amdgcn_mfma_f32_32x32x16_f16(w0[s], X[s], h, 0, 0, 0);
    if constexpr (kSplit) {
#pragma unroll
        for (int s = 0; s < 2; ++s) h = __builtin_amdgcn_mfma_f32_32x32x16_f16(w0[s], X[3 + s], h, 0, 0, 0);
    }
    if constexpr (kWLo) {  // low parts of the weights against the high parts of the inputs
#pragma unroll
        for (int s = 0; s < 3; ++s) h = __builtin_amdgcn_mfma_f32_32x32x16_f16(wlo[s][lane], X[s], h, 0, 0, 0);
    }
    // ReLU, then hi/lo split: registers 8s..8s+7 are the B operand of k-step s
    half8_t hh[2], hl[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        float r[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) r[j] = __builtin_amdgcn_fmed3f(h[8 * s + j], 0.0f, __builtin_inff());  // ReLU in one instruction
        split_half8(r, hh[s], hl[s]);
    }
    // layer 2: out = W1 [outputs x 32] * hidden + b1
#pragma unroll
    for (int r = 0; r < kTiles; ++r) {
        floatx16 c = bias_rows(bias1, 32 * r, half);
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const half8_t w1 = kWInLds ? whi[3 + 2 * r + s][lane] : w.w1[r][s];
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(w1, hh[s], c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(w1, hl[s], c, 0, 0, 0);
            if constexpr (kWLo) c = __builtin_amdgcn_mfma_f32_32x32x16_f16(wlo[3 + 2 * r + s][lane], hh[s], c, 0, 0, 0);
        }
        store_rows(dst_anchor, base, outputs, 32 * r, half, c);
    }
}

// 1 / (1 + exp(-x)) from the hardware exp2 and reciprocal (each within 1 ulp; the product x log2(e) adds
// |x| 2^-24 to the exponent): relative error below 1e-6 for any x, against the 3e-5 the decode is held to.
__device__ __forceinline__ float fast_sigmoid(float x)
{
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}

// Per-lane inputs of one tile of 32 anchors.
template <bool kCountOnly>
struct TileInputs {
    float4 f[4] = {};          // features 16s + 8*half .. +7 in f[2s], f[2s+1], s = 0..1
    float pos[3] = {0.f, 0.f, 0.f};
    float sc3[3] = {0.f, 0.f, 0.f};
    float extra = 0.f;  // the anchor's level when it replaces the distance
    uint32_t first_slot = 0;
    float ofv[kCountOnly ? 1 : 5][3] = {};
};

// A wavefront takes runs of kRun consecutive anchors, packs the visible ones (in order) into dense tiles of 32
// and runs the MLPs on those only: the work follows the number of visible anchors, not of anchors.
constexpr int kRun = 128;

// kSplit: the features enter as hi + lo fp16 pairs (general fp32 features; two more matrix instructions per head).
// kWLo: so do the weights (general fp32 weights; their low fragments take 19 KB of LDS in the emit pass, which
// then runs three wavefronts per workgroup so that two workgroups still share a CU, held to 256 registers).
constexpr int decode_waves(bool count_only, bool weights_lo) { return (weights_lo && !count_only) ? 3 : 4; }

template <bool kCountOnly, bool kSplit, bool kWLo>
__global__ __launch_bounds__((64 * decode_waves(kCountOnly, kWLo)), (!kCountOnly ? 2 : 4)) void decode_kernel(DecodeArgs d, uint32_t* __restrict__ counts,
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
    constexpr int kWaves = decode_waves(kCountOnly, kWLo);
    __shared__ float s_out[kWaves][32 * kStrideMax + kListFloats + kRunFloats];

    // biases of the three heads, zero-padded: b0 at [head*32], b1 of opacity / cov / colour at 96 / 128 / 224
    __shared__ float s_bias[256];
    // low parts of the weight fragments: opacity head 0..4, covariance 5..13, colour 14..18
    __shared__ half8_t s_wlo[kWLo ? (kCountOnly ? 5 : 19) : 1][kWLo ? 64 : 1];
    // the covariance head's weight fragments (0..8) and, where LDS has room for them beside the low parts, the
    // colour head's (9..13), for the emit pass: read from here right before their matrix instruction instead of
    // holding 36 + 20 registers for the whole kernel
    constexpr bool kColourInLds = !kCountOnly && !kWLo;
    __shared__ half8_t s_whi[kCountOnly ? 1 : (kColourInLds ? 14 : 9)][kCountOnly ? 1 : 64];
    const half8_t (*const whi)[64] = reinterpret_cast<const half8_t (*)[64]>(s_whi);
    const half8_t (*const wlo)[64] = reinterpret_cast<const half8_t (*)[64]>(s_wlo);

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, half = lane >> 5, col = lane & 31;
    const int n = d.n;
    for (int t = threadIdx.x; t < 256; t += 64 * kWaves) {
        float v = 0.0f;
        if (t < 96) v = d.b0[t >> 5][t & 31];
        else if (t < 128) v = (t - 96) < n ? d.b1[0][t - 96] : 0.0f;
        else if (t < 224) v = (t - 128) < 7 * n ? d.b1[1][t - 128] : 0.0f;
        else v = (t - 224) < 3 * n ? d.b1[2][t - 224] : 0.0f;
        s_bias[t] = v;
    }
    if constexpr (kWLo) {
        if (wave == 0) store_head_lo<1>(d, 0, n, col, half, lane, s_wlo);
        if constexpr (!kCountOnly) {
            if (wave == 1) store_head_lo<3>(d, 1, 7 * n, col, half, lane, s_wlo + 5);
            if (wave == 2) store_head_lo<1>(d, 2, 3 * n, col, half, lane, s_wlo + 14);
        }
    }
    if constexpr (!kCountOnly) {
        if (wave == kWaves - 1) store_head_lo<3>(d, 1, 7 * n, col, half, lane, s_whi, false);
        if constexpr (kColourInLds) {
            if (wave == kWaves - 2) store_head_lo<1>(d, 2, 3 * n, col, half, lane, s_whi + 9, false);
        }
    }
    __syncthreads();
    HeadWeights<1> w_op;
    load_head<1>(d, 0, n, col, half, w_op);
    const HeadWeights<3> w_cov = {};  // unused: read from s_whi
    HeadWeights<1> w_col = {};
    if (!kCountOnly && !kColourInLds) load_head<1>(d, 2, 3 * n, col, half, w_col);
    const int stride = kCountOnly ? 11 : 11 * n + 13;
    const int items = 32 * n;  // (anchor, offset) pairs of a tile: item = anchor_in_tile * n + offset
    const int inv_n = (65536 + n - 1) / n;  // item / n == (item * inv_n) >> 16 for item < 32 n, n <= 10
    const uint64_t lanes_below = (1ull << lane) - 1ull;
    const int runs = (d.A + kRun - 1) / kRun;
    float* __restrict__ mine = s_out[wave];
    uint8_t* __restrict__ run_list = reinterpret_cast<uint8_t*>(mine + 32 * kStrideMax + kListFloats);
    const float cx = d.campos[0], cy = d.campos[1], cz = d.campos[2];

    for (int run = blockIdx.x * kWaves + wave; run < runs; run += gridDim.x * kWaves) {
      // positions (within the run) of its visible anchors, in order: lane covers anchors lane and 64 + lane
      const int base = run * kRun;
      const int a0 = base + lane, a1 = base + 64 + lane;
      const bool v0 = a0 < d.A && d.visible[a0] != 0, v1 = a1 < d.A && d.visible[a1] != 0;
      const uint64_t m0 = __ballot(v0), m1 = __ballot(v1);
      const int n0 = __popcll(m0), nvis = n0 + __popcll(m1);
      if (kCountOnly && counts) {  // anchors that are not decoded keep nothing
          if (!v0 && a0 < d.A) counts[a0] = 0;
          if (!v1 && a1 < d.A) counts[a1] = 0;
      }
      if (nvis == 0) {  // uniform
          if (kCountOnly && d.run_totals && lane == 0) d.run_totals[run] = make_uint2(0u, 0u);
          continue;
      }
      uint32_t run_kept = 0;  // count pass: this lane's share of the run's kept offsets
      // emit pass of the one-call decode: the run's first output slot, advanced tile by tile (uniform), and the
      // rank of its first visible anchor among all visible anchors
      uint32_t run_slot = 0, run_rank = 0;
      if (!kCountOnly && d.run_base) {
          const uint2 rb = d.run_base[run];
          run_slot = rb.x;
          run_rank = rb.y;
      }
      if (v0) run_list[__popcll(m0 & lanes_below)] = (uint8_t)lane;
      if (v1) run_list[n0 + __popcll(m1 & lanes_below)] = (uint8_t)(64 + lane);
      wave_lds_sync();
      // Everything a tile needs from global memory is requested before the first use, and without a
      // condition: a lane without an anchor (or an item without one) reads anchor 0's data, which nothing uses
      // (matrix columns are independent, and only items of visible anchors are ever emitted) -- conditional
      // loads would each become a branch, and the values' first use would wait inside the condition.
      // Features, position and level of the tile's anchors.
      auto fetch_anchor = [&](int a, TileInputs<kCountOnly>& in) {
        const float4* __restrict__ f4 = reinterpret_cast<const float4*>(d.feat + (size_t)a * kFeat);
#pragma unroll
        for (int s = 0; s < 2; ++s) {  // features 16s + 8*half .. +7
            in.f[2 * s] = f4[4 * s + 2 * half];
            in.f[2 * s + 1] = f4[4 * s + 2 * half + 1];
        }
#pragma unroll
        for (int k = 0; k < 3; ++k) in.pos[k] = d.anchor[3 * (size_t)a + k];
        if (d.level) in.extra = d.level[a];
      };
      // The count pass has registers to spare and a run's tiles are otherwise a chain of memory latencies: it
      // requests the next tile's inputs before it waits for the current tile's.
      TileInputs<kCountOnly> ahead;
      if constexpr (kCountOnly) fetch_anchor(col < nvis ? base + (int)run_list[col] : 0, ahead);
      for (int first = 0; first < nvis; first += 32) {  // dense tiles of the run
        const bool vis = first + col < nvis;  // lanes l and l+32 share entry first + l
        const int a = vis ? base + (int)run_list[first + col] : 0;
        const uint64_t any = __ballot(vis);  // bits l and l + 32 belong to entry l of the tile
        TileInputs<kCountOnly> in;
        if constexpr (kCountOnly) {
            in = ahead;
            if (first + 32 < nvis)  // uniform
                fetch_anchor(first + 32 + col < nvis ? base + (int)run_list[first + 32 + col] : 0, ahead);
        } else {
            {  // as fetch_anchor, written out: through the lambda this pass spills three times as many registers
                const float4* __restrict__ f4 = reinterpret_cast<const float4*>(d.feat + (size_t)a * kFeat);
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    in.f[2 * s] = f4[4 * s + 2 * half];
                    in.f[2 * s + 1] = f4[4 * s + 2 * half + 1];
                }
#pragma unroll
                for (int k = 0; k < 3; ++k) in.pos[k] = d.anchor[3 * (size_t)a + k];
                if (d.level) in.extra = d.level[a];
            }
            // half 0: scaling[0..2] (offset scale), half 1: scaling[3..5] (Gaussian scale)
#pragma unroll
            for (int k = 0; k < 3; ++k) in.sc3[k] = d.scaling[6 * (size_t)a + 3 * half + k];
            if (offsets) in.first_slot = offsets[a];  // entry 0's value is the tile's first output slot
            // the learned offsets of the items this lane's position covers (item = entry * n + offset)
            int item_anchor[5], item_offset[5];
#pragma unroll
            for (int r = 0; r < 5; ++r) {
                const int it = min(r * 64 + lane, items - 1);
                const int al = (it * inv_n) >> 16;
                item_offset[r] = it - al * n;
                item_anchor[r] = (int)run_list[min(first + al, nvis - 1)];
            }
#pragma unroll
            for (int r = 0; r < 5; ++r) {
                const float* __restrict__ of = d.offset + ((size_t)(base + item_anchor[r]) * n + item_offset[r]) * 3;
#pragma unroll
                for (int k = 0; k < 3; ++k) in.ofv[r][k] = of[k];
            }
        }
        // B operand: X^T, column = anchor; slots as described at HeadWeights
        half8_t X[kSplit ? 5 : 3];
        const float ax = in.pos[0], ay = in.pos[1], az = in.pos[2];
        {
            float x8[8];
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                x8[0] = in.f[2 * s].x, x8[1] = in.f[2 * s].y, x8[2] = in.f[2 * s].z, x8[3] = in.f[2 * s].w;
                x8[4] = in.f[2 * s + 1].x, x8[5] = in.f[2 * s + 1].y, x8[6] = in.f[2 * s + 1].z, x8[7] = in.f[2 * s + 1].w;
                if constexpr (kSplit) split_half8(x8, X[s], X[3 + s]);  // the second: what the fp16 rounding left over
                else X[s] = to_half8(x8);                               // all zero for an invisible anchor
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) x8[j] = 0.0f;
            if (vis && half == 0) {
                float vx = ax - cx, vy = ay - cy, vz = az - cz;
                const float dist = sqrtf(vx * vx + vy * vy + vz * vz);
                vx /= dist;
                vy /= dist;
                vz /= dist;
                const float in4[4] = {vx, vy, vz, d.level ? in.extra : dist};
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
        // the mask opacity > 0 is the sign of the pre-activation (tanh is odd, monotone and tanh(x) = x for the
        // smallest floats), so tanh itself is only evaluated for the offsets that are kept
        run_head<1, kSplit, kWLo>(w_op, nullptr, wlo, lane, s_bias, s_bias + 96, X, half, mine + col * stride, 0, n);
        if (kCountOnly) {
            wave_lds_sync();
            if (half == 0 && vis) {
                uint32_t kept = 0;
                for (int m = 0; m < n; ++m) kept += mine[col * stride + m] > 0.0f ? 1u : 0u;
                if (counts) counts[a] = kept;
                run_kept += kept;
            }
            wave_lds_sync();
            continue;
        }

        // ---- covariance and colour heads ----
        run_head<3, kSplit, kWLo, true>(w_cov, whi, wlo + (kWLo ? 5 : 0), lane, s_bias + 32, s_bias + 128, X, half,
                                        mine + col * stride, n, 7 * n);
        run_head<1, kSplit, kWLo, kColourInLds>(w_col, whi + (kColourInLds ? 9 : 0), wlo + (kWLo ? 14 : 0), lane,
                                                s_bias + 64, s_bias + 224, X, half, mine + col * stride, 8 * n, 3 * n);
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
        float pre[5];  // the items' opacity pre-activations, all requested before the first is looked at
        bool exists[5];
#pragma unroll
        for (int r = 0; r < 5; ++r) {
            const int it = min(r * 64 + lane, items - 1);
            const int al = (it * inv_n) >> 16, m = it - al * n;
            pre[r] = mine[al * stride + m];
            exists[r] = r * 64 + lane < items && ((any >> al) & 1ull);
        }
#pragma unroll
        for (int r = 0; r < 5; ++r) {
            if (r * 64 >= items) break;  // uniform
            const bool kept = exists[r] && pre[r] > 0.0f;
            const uint64_t b = __ballot(kept);
            if (kept) list[total + (uint32_t)__popcll(b & lanes_below)] = (uint16_t)(r * 64 + lane);
            total += (uint32_t)__popcll(b);
        }
        wave_lds_sync();

        // Items are numbered anchor-major and the slots come from an exclusive scan of the per-anchor counts, so
        // the survivors of a tile occupy consecutive output slots from the slot of its first anchor: lanes write
        // consecutive addresses.  No global reads in here: the learned offsets sit in registers of the lane that
        // requested them (item = round * 64 + lane) and are fetched across lanes.
        const uint32_t tile_slot = d.run_base ? run_slot : reinterpret_cast<const uint32_t*>(mine)[11 * n + 9];
        run_slot += total;
        // training-mode by-products: tanh of every pre-activation of the visible anchors and the mask, indexed by
        // (visible anchor, offset): the tile's entries are the run's visible anchors first .. first + 31
        if (d.neural_opacity || d.kept_mask) {
            const size_t row0 = ((size_t)run_rank + (size_t)first) * (size_t)n;
#pragma unroll
            for (int r = 0; r < 5; ++r) {
                const int it = r * 64 + lane;
                if (it >= items) break;
                const int al = (it * inv_n) >> 16, m = it - al * n;
                if ((any >> al) & 1ull) {
                    const float v = mine[al * stride + m];
                    if (d.neural_opacity) d.neural_opacity[row0 + (size_t)it] = tanhf(v);
                    if (d.kept_mask) d.kept_mask[row0 + (size_t)it] = v > 0.0f ? 1 : 0;
                }
            }
        }
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
                color[3 * (size_t)pos + k] = fast_sigmoid(c3[k]);
                scaling_out[3 * (size_t)pos + k] = extra[3 + k] * fast_sigmoid(c7[k]);
                xyz[3 * (size_t)pos + k] = extra[6 + k] + off3[k] * extra[k];
            }
            const float q0 = c7[3], q1 = c7[4], q2 = c7[5], q3 = c7[6];
            // q / max(|q|, 1e-12) with one reciprocal square root (1 ulp) instead of a root and four divisions
            const float inv = __builtin_amdgcn_rsqf(fmaxf(q0 * q0 + q1 * q1 + q2 * q2 + q3 * q3, 1e-24f));
            rot[4 * (size_t)pos + 0] = q0 * inv;
            rot[4 * (size_t)pos + 1] = q1 * inv;
            rot[4 * (size_t)pos + 2] = q2 * inv;
            rot[4 * (size_t)pos + 3] = q3 * inv;
        }
        wave_lds_sync();
      }
      if (kCountOnly && d.run_totals) {  // the run's totals: kept offsets (summed over the lanes), visible anchors
          uint32_t t = run_kept;
#pragma unroll
          for (int off = 32; off > 0; off >>= 1) t += (uint32_t)__shfl_xor((int)t, off, 64);
          if (lane == 0) d.run_totals[run] = make_uint2(t, (uint32_t)nvis);
      }
    }
}

// One workgroup: exclusive prefix of the per-run totals (kept offsets, visible anchors) and the grand totals.
__global__ __launch_bounds__(1024) void run_scan_kernel(const uint2* __restrict__ totals, uint2* __restrict__ base,
                                                        uint32_t runs, uint32_t* __restrict__ num_emitted,
                                                        uint32_t* __restrict__ num_visible)
{
    __shared__ uint2 s_wave[16];
    __shared__ uint2 s_carry;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) s_carry = make_uint2(0u, 0u);
    __syncthreads();
    for (uint32_t first = 0; first < runs; first += 1024) {
        const uint32_t j = first + threadIdx.x;
        const uint2 v = j < runs ? totals[j] : make_uint2(0u, 0u);
        uint32_t ix = v.x, iy = v.y;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t ux = (uint32_t)__shfl_up((int)ix, d, 64), uy = (uint32_t)__shfl_up((int)iy, d, 64);
            if (lane >= d) {
                ix += ux;
                iy += uy;
            }
        }
        if (lane == 63) s_wave[wave] = make_uint2(ix, iy);
        __syncthreads();
        uint2 before = s_carry;
        for (int w = 0; w < wave; ++w) {
            before.x += s_wave[w].x;
            before.y += s_wave[w].y;
        }
        if (j < runs) base[j] = make_uint2(before.x + ix - v.x, before.y + iy - v.y);
        __syncthreads();
        if (threadIdx.x == 1023) s_carry = make_uint2(before.x + ix, before.y + iy);
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        if (num_emitted) *num_emitted = s_carry.x;
        if (num_visible) *num_visible = s_carry.y;
    }
}

// Feature bank (anchor_decoder.py:163-177): a small MLP of the view direction (and the level) gives three softmax
// weights per anchor that mix the feature vector with its 4x and 2x strided copies:
//     feat'[j] = feat[4 (j mod 8)] w0 + feat[2 (j mod 16)] w1 + feat[j] w2 .
// One thread per visible anchor, fp32 throughout; the decode then reads the mixed features.
struct BankArgs {
    int A, in_dim;  // 3 = view direction, 4 = view direction and level
    const float* anchor;
    const float* feat;
    const uint8_t* visible;
    const float* campos;
    const float* level;
    const float* w0;  // [32, in_dim]
    const float* b0;  // [32]
    const float* w1;  // [3, 32]
    const float* b1;  // [3]
    float* mixed;     // [A, 32]
};

__global__ __launch_bounds__(256) void feature_bank_kernel(BankArgs k)
{
    __shared__ float s_w0[kFeat * 4], s_b0[kFeat], s_w1[3 * kFeat], s_b1[3];
    for (int t = threadIdx.x; t < kFeat * k.in_dim; t += 256) s_w0[t] = k.w0[t];
    for (int t = threadIdx.x; t < 3 * kFeat; t += 256) s_w1[t] = k.w1[t];
    if (threadIdx.x < kFeat) s_b0[threadIdx.x] = k.b0[threadIdx.x];
    if (threadIdx.x < 3) s_b1[threadIdx.x] = k.b1[threadIdx.x];
    __syncthreads();
    const int a = blockIdx.x * 256 + threadIdx.x;
    if (a >= k.A || k.visible[a] == 0) return;
    float in[4];
    {
        float vx = k.anchor[3 * (size_t)a] - k.campos[0], vy = k.anchor[3 * (size_t)a + 1] - k.campos[1],
              vz = k.anchor[3 * (size_t)a + 2] - k.campos[2];
        const float dist = sqrtf(vx * vx + vy * vy + vz * vz);
        in[0] = vx / dist;
        in[1] = vy / dist;
        in[2] = vz / dist;
        in[3] = k.in_dim > 3 ? k.level[a] : 0.0f;
    }
    float logit[3] = {s_b1[0], s_b1[1], s_b1[2]};
    for (int h = 0; h < kFeat; ++h) {
        float v = s_b0[h];
        for (int c = 0; c < k.in_dim; ++c) v += s_w0[h * k.in_dim + c] * in[c];
        v = fmaxf(v, 0.0f);
#pragma unroll
        for (int o = 0; o < 3; ++o) logit[o] += s_w1[o * kFeat + h] * v;
    }
    const float top = fmaxf(logit[0], fmaxf(logit[1], logit[2]));
    float w[3] = {expf(logit[0] - top), expf(logit[1] - top), expf(logit[2] - top)};
    const float sum = w[0] + w[1] + w[2];
#pragma unroll
    for (int o = 0; o < 3; ++o) w[o] /= sum;
    float f[kFeat];
    const float4* __restrict__ src = reinterpret_cast<const float4*>(k.feat + (size_t)a * kFeat);
#pragma unroll
    for (int q = 0; q < kFeat / 4; ++q) {
        const float4 v = src[q];
        f[4 * q] = v.x, f[4 * q + 1] = v.y, f[4 * q + 2] = v.z, f[4 * q + 3] = v.w;
    }
    float4* __restrict__ dst = reinterpret_cast<float4*>(k.mixed + (size_t)a * kFeat);
#pragma unroll
    for (int q = 0; q < kFeat / 4; ++q) {
        float o4[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int j = 4 * q + t;
            o4[t] = f[4 * (j % 8)] * w[0] + f[2 * (j % 16)] * w[1] + f[j] * w[2];
        }
        dst[q] = make_float4(o4[0], o4[1], o4[2], o4[3]);
    }
}

}  // namespace

struct DecodeLaunch {
    DecodeArgs args;
};

static int fill_args(const gs355_decoder* dec, const gs355_anchors* an, bool allow_bank, DecodeArgs* out)
{
    if (!dec || !an) return set_error(GS355_EINVAL, "decoder / anchors is NULL");
    if (dec->feat_dim != kFeat)
        return set_error(GS355_EINVAL, "anchor decode supports feat_dim 32 only (got %d)", dec->feat_dim);
    if (dec->n_offsets < 1 || dec->n_offsets > 10)
        return set_error(GS355_EINVAL, "anchor decode supports 1..10 offsets per anchor (got %d)", dec->n_offsets);
    if (an->A < 0) return set_error(GS355_EINVAL, "A must be >= 0 (got %d)", an->A);
    for (int j = 0; j < 3; ++j) {
        if (dec->add_level) {
            // the reference concatenates [feat | view | level] for every head once a level is given
            // (anchor_decoder.py:181-182), so a head built with a distance column as well cannot be fed
            if (dec->in_dim[j] != kFeat + 4)
                return set_error(GS355_EINVAL, "head %d: with add_level the input is [feat | view | level], 36 wide "
                                 "(got %d; a head with add_*_dist expects a width the reference never provides)",
                                 j, dec->in_dim[j]);
        } else if (dec->in_dim[j] != kFeat + 3 && dec->in_dim[j] != kFeat + 4) {
            return set_error(GS355_EINVAL, "head %d: input width must be 35 or 36 (got %d)", j, dec->in_dim[j]);
        }
        if (!dec->w0[j] || !dec->b0[j] || !dec->w1[j] || !dec->b1[j])
            return set_error(GS355_EINVAL, "head %d: weight or bias pointer is NULL", j);
    }
    if (dec->bank_in_dim != 0) {
        if (!allow_bank) return set_error(GS355_EINVAL, "the feature bank is supported by gs355_decode only");
        if (dec->bank_in_dim != 3 && dec->bank_in_dim != 4)
            return set_error(GS355_EINVAL, "bank_in_dim must be 0, 3 or 4 (got %d)", dec->bank_in_dim);
        if (!dec->bank_w0 || !dec->bank_b0 || !dec->bank_w1 || !dec->bank_b1)
            return set_error(GS355_EINVAL, "feature bank: weight or bias pointer is NULL");
    }
    if (an->A > 0 && (!an->anchor || !an->feat || !an->offset || !an->scaling || !an->visible_mask || !an->campos))
        return set_error(GS355_EINVAL, "anchor inputs must all be non-NULL");
    if (an->A > 0 && (dec->add_level || dec->bank_in_dim == 4) && !an->level)
        return set_error(GS355_EINVAL, "anchors.level is NULL but the decoder takes the level as an input");
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
    a.level = dec->add_level ? an->level : nullptr;
    a.split_feat = (dec->fp32_features || dec->bank_in_dim != 0) ? 1 : 0;  // bank-mixed features are general floats
    a.weights_lo = dec->fp32_weights ? 1 : 0;
    for (int j = 0; j < 3; ++j) {
        a.in_dim[j] = dec->in_dim[j];
        a.w0[j] = dec->w0[j];
        a.b0[j] = dec->b0[j];
        a.w1[j] = dec->w1[j];
        a.b1[j] = dec->b1[j];
    }
    a.run_totals = nullptr;
    a.run_base = nullptr;
    a.neural_opacity = nullptr;
    a.kept_mask = nullptr;
    *out = a;
    return GS355_OK;
}

// Persistent workgroups (4 wavefronts, each walking runs of kRun anchors): at most `cap` of them, about what
// the chip holds at once, so the weight fragments are fetched once per resident workgroup.
static dim3 decode_grid(int A, int cap, int waves = 4)
{
    const int runs = (A + kRun - 1) / kRun;
    int blocks = (runs + waves - 1) / waves;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return dim3(blocks);
}

// Launch the count or the emit pass in the variant the features and the weights need.  `cap`: most workgroups.
template <bool kCountOnly, bool kSplit, bool kWLo>
static void launch_variant(int cap, hipStream_t s, const DecodeArgs& a, uint32_t* counts, const uint32_t* offsets,
                           uint32_t capacity, float* xyz, float* color, float* opacity, float* scaling, float* rot)
{
    constexpr int kWaves = decode_waves(kCountOnly, kWLo);
    hipLaunchKernelGGL((decode_kernel<kCountOnly, kSplit, kWLo>), decode_grid(a.A, cap, kWaves), dim3(64 * kWaves), 0, s, a,
                       counts, offsets, capacity, xyz, color, opacity, scaling, rot);
}

static void launch_decode(bool count_only, int cap, hipStream_t s, const DecodeArgs& a, uint32_t* counts,
                          const uint32_t* offsets, uint32_t capacity, const gs355_decoded* out)
{
    float* xyz = out ? out->xyz : nullptr;
    float* color = out ? out->color : nullptr;
    float* opacity = out ? out->opacity : nullptr;
    float* scaling = out ? out->scaling : nullptr;
    float* rot = out ? out->rot : nullptr;
#define GS355_DECODE_CASE(C, S, W)                                                                             \
    if (count_only == C && (a.split_feat != 0) == S && (a.weights_lo != 0) == W)                               \
        launch_variant<C, S, W>(cap, s, a, counts, offsets, capacity, xyz, color, opacity, scaling, rot);
    GS355_DECODE_CASE(true, false, false)
    GS355_DECODE_CASE(true, false, true)
    GS355_DECODE_CASE(true, true, false)
    GS355_DECODE_CASE(true, true, true)
    GS355_DECODE_CASE(false, false, false)
    GS355_DECODE_CASE(false, false, true)
    GS355_DECODE_CASE(false, true, false)
    GS355_DECODE_CASE(false, true, true)
#undef GS355_DECODE_CASE
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
    int rc = fill_args(dec, an, false, &a);
    if (rc) return rc;
    if (a.A == 0) return GS355_OK;
    if (!counts || !offsets || !scratch_buf) return set_error(GS355_EINVAL, "counts / offsets / scratch is NULL");
    size_t need = 0;
    gs355_decode_scratch_bytes(a.A, &need);
    if (scratch_bytes < need)
        return set_error(GS355_ENOSPC, "decode scratch has %zu bytes, %zu needed", scratch_bytes, need);
    hipStream_t s = static_cast<hipStream_t>(stream);
    launch_decode(true, 1024, s, a, counts, nullptr, 0u, nullptr);
    GS355_CHECK_LAUNCH("decode: count");
    return launch_exclusive_scan(counts, offsets, (size_t)a.A, static_cast<uint32_t*>(scratch_buf), s);
}

int gs355_decode_count_static(const gs355_decoder* dec, const gs355_anchors* an, uint32_t* counts, uint32_t* offsets,
                              void* stream)
{
    DecodeArgs a;
    int rc = fill_args(dec, an, false, &a);
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
    launch_decode(true, 1024, s, a, counts, nullptr, 0u, nullptr);
    GS355_CHECK_LAUNCH("decode: count");
    // the scan writes every block sum before it reads it: nothing in the array has to start at zero
    return launch_exclusive_scan(counts, offsets, (size_t)a.A, tmp, s);
}

int gs355_decode_emit(const gs355_decoder* dec, const gs355_anchors* an, const uint32_t* offsets, int64_t capacity,
                      const gs355_decoded* out, void* stream)
{
    DecodeArgs a;
    int rc = fill_args(dec, an, false, &a);
    if (rc) return rc;
    if (a.A == 0 || capacity == 0) return GS355_OK;
    if (capacity < 0 || capacity > 0xFFFFFFFFll)
        return set_error(GS355_EINVAL, "capacity must be in [0, 2^32) (got %lld)", (long long)capacity);
    if (!offsets) return set_error(GS355_EINVAL, "offsets is NULL");
    if (!out || !out->xyz || !out->color || !out->opacity || !out->scaling || !out->rot)
        return set_error(GS355_EINVAL, "decoded outputs must all be non-NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    launch_decode(false, 512, s, a, nullptr, offsets, (uint32_t)capacity, out);
    GS355_CHECK_LAUNCH("decode: emit");
    return GS355_OK;
}

namespace {
struct FusedLayout {
    size_t run_totals, run_base, mixed, total;
};
FusedLayout fused_layout(int32_t A, int32_t n, bool bank)
{
    auto up = [](size_t v) { return (v + 255) / 256 * 256; };
    const size_t runs = ((size_t)A + kRun - 1) / kRun;
    FusedLayout L;
    size_t off = 0;
    (void)n;
    L.run_totals = off;
    off = up(off + runs * sizeof(uint2) + 8);
    L.run_base = off;
    off = up(off + runs * sizeof(uint2) + 8);
    L.mixed = off;
    if (bank) off = up(off + (size_t)A * kFeat * sizeof(float) + 4);
    L.total = off;
    return L;
}
}  // namespace

int gs355_decode_workspace_bytes(int32_t A, int32_t n_offsets, int32_t with_feature_bank, size_t* bytes)
{
    if (!bytes) return set_error(GS355_EINVAL, "bytes is NULL");
    if (A < 0) return set_error(GS355_EINVAL, "A must be >= 0 (got %d)", A);
    if (n_offsets < 1 || n_offsets > 10)
        return set_error(GS355_EINVAL, "anchor decode supports 1..10 offsets per anchor (got %d)", n_offsets);
    *bytes = fused_layout(A, n_offsets, with_feature_bank != 0).total;
    return GS355_OK;
}

int gs355_decode(const gs355_decoder* dec, const gs355_anchors* an, int64_t capacity, const gs355_decoded* out,
                 void* workspace, size_t workspace_bytes, uint32_t phases, void* stream)
{
    if (phases == 0 || (phases & ~(uint32_t)(GS355_DECODE_COUNT | GS355_DECODE_EMIT)) != 0)
        return set_error(GS355_EINVAL, "phases must be GS355_DECODE_COUNT, GS355_DECODE_EMIT or both (got 0x%x)", phases);
    const bool do_count = (phases & GS355_DECODE_COUNT) != 0, do_emit = (phases & GS355_DECODE_EMIT) != 0;
    DecodeArgs a;
    int rc = fill_args(dec, an, true, &a);
    if (rc) return rc;
    if (capacity < 0 || capacity > 0xFFFFFFFFll)
        return set_error(GS355_EINVAL, "capacity must be in [0, 2^32) (got %lld)", (long long)capacity);
    if (!out) return set_error(GS355_EINVAL, "decoded outputs is NULL");
    if (do_emit && capacity > 0 && (!out->xyz || !out->color || !out->opacity || !out->scaling || !out->rot))
        return set_error(GS355_EINVAL, "decoded outputs must all be non-NULL");
    const bool bank = dec->bank_in_dim != 0;
    const FusedLayout L = fused_layout(a.A, a.n, bank);
    if (a.A > 0) {
        if (!workspace) return set_error(GS355_EINVAL, "workspace is NULL");
        if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
            return set_error(GS355_EINVAL, "workspace must be 256-byte aligned");
        if (workspace_bytes < L.total)
            return set_error(GS355_ENOSPC, "decode workspace has %zu bytes, %zu needed", workspace_bytes, L.total);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (a.A == 0) {
        if (do_count && out->count && (rc = launch_fill_u32(out->count, 1, 0u, s))) return rc;
        if (do_count && out->num_visible && (rc = launch_fill_u32(out->num_visible, 1, 0u, s))) return rc;
        return GS355_OK;
    }
    char* ws = static_cast<char*>(workspace);
    const uint32_t runs = (uint32_t)(((size_t)a.A + kRun - 1) / kRun);
    if (bank) a.feat = reinterpret_cast<float*>(ws + L.mixed);  // written by the count phase, read by both passes
    uint2* run_base = reinterpret_cast<uint2*>(ws + L.run_base);
    if (do_count) {
        if (bank) {
            BankArgs b;
            b.A = a.A;
            b.in_dim = dec->bank_in_dim;
            b.anchor = a.anchor;
            b.feat = an->feat;
            b.visible = a.visible;
            b.campos = a.campos;
            b.level = an->level;
            b.w0 = dec->bank_w0;
            b.b0 = dec->bank_b0;
            b.w1 = dec->bank_w1;
            b.b1 = dec->bank_b1;
            b.mixed = reinterpret_cast<float*>(ws + L.mixed);
            hipLaunchKernelGGL(feature_bank_kernel, dim3((a.A + 255) / 256), dim3(256), 0, s, b);
            GS355_CHECK_LAUNCH("decode: feature bank");
        }
        a.run_totals = reinterpret_cast<uint2*>(ws + L.run_totals);
        launch_decode(true, 1024, s, a, nullptr, nullptr, 0u, nullptr);
        GS355_CHECK_LAUNCH("decode: count");
        hipLaunchKernelGGL(run_scan_kernel, dim3(1), dim3(1024), 0, s, a.run_totals, run_base, runs, out->count,
                           out->num_visible);
        GS355_CHECK_LAUNCH("decode: run scan");
    }
    if (!do_emit) return GS355_OK;
    if (capacity == 0 && !out->neural_opacity && !out->mask) return GS355_OK;
    a.run_totals = nullptr;
    a.run_base = run_base;
    a.neural_opacity = out->neural_opacity;
    a.kept_mask = out->mask;
    launch_decode(false, 512, s, a, nullptr, nullptr, (uint32_t)capacity, out);
    GS355_CHECK_LAUNCH("decode: emit");
    return GS355_OK;
}

}  // extern "C"
