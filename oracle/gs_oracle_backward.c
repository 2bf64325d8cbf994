/*
 * CPU oracle for the backward pass of the 3D-Gaussian-splatting rasterizer.
 *
 * THIS IS TEST INFRASTRUCTURE (see gs_oracle.c): only tests, the smoke check
 * and the CPU-baseline leg of the benchmark may link or call it.
 *
 * What it restates.  The reference trains through the same third-party
 * rasterizer it renders with (loss.backward() at benchmarks/nerf/origin_gs/
 * gs_trainer.py:117-124; the screen-space gradient of `means2D` feeds
 * densification, landmark/nerf_components/model_components/fields/encodings/
 * gaussian_encoding.py:729-743 and origin_gs/gs_model.py:129-139,225-236).
 * The CUDA source of that rasterizer is absent from the reference tree
 * (.gitmodules:1-4), so this file restates the published backward pass of the
 * tile rasterizer of Kerbl et al. 2023 in the form of the
 * diff-gaussian-rasterization lineage:
 *   - per pixel, the blended Gaussians are walked BACK TO FRONT, carrying the
 *     colour accumulated behind the current one;
 *   - alpha = min(0.99, opacity * G) lets the gradient through the min
 *     unchanged (the published kernel computes dL/dG = opacity * dL/dalpha
 *     whether or not the clamp is active);
 *   - the gradient of `means2D` is reported in normalised device units
 *     (pixel-space gradient times W/2 and H/2), third component zero;
 *   - everything else is the exact derivative of the forward arithmetic in
 *     gs_oracle.c (the published kernel adds 1e-7 to the squared determinant
 *     of the 2-D covariance and ignores the dependence of a clamped Jacobian
 *     on depth; both are below the tolerance the gradients are compared at and
 *     apply to off-screen Gaussians only).
 * The per-pair decisions (sign test, 1/255 threshold, 1e-4 stop) are taken in
 * fp32 exactly as orc_blend takes them; the gradient arithmetic itself runs in
 * double precision so that the oracle is the more exact side of a comparison.
 *
 * Pinning (tests/test_oracle_backward.py): reverse-mode differentiation by
 * torch.autograd of the independent PyTorch statement of the forward pass
 * (oracle/torch_oracle.py) in fp64, itself checked there against central
 * finite differences; closed forms for one Gaussian.  Against the absent CUDA
 * source the backward pass is "parity unpinned", like the forward pass.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_TILE 16
#define ORC_GRAD 10 /* per-Gaussian accumulators: d/dpx, d/dpy, d/dconic(x,y,z), d/dopacity, d/drgb(3), d/ddepth */

typedef struct {
    int32_t image_width, image_height;
    float tanfovx, tanfovy;
    float scale_modifier;
    int32_t sh_degree;
    int32_t sh_coeffs;
    float viewmatrix[16];
    float projmatrix[16];
    float campos[3];
    float bg[3];
} orc_frame;

typedef struct {
    int32_t P;
    const float *means3D;
    const float *shs;
    const float *colors_precomp;
    const float *opacities;
    const float *scales;
    const float *rotations;
    const float *cov3D_precomp;
} orc_gaussians;

typedef struct {
    uint32_t g;
    float dx, dy, G, alpha, T;
} orc_hit;

#define ORC_ADD(target, value)                 \
    do {                                       \
        double v__ = (value);                  \
        _Pragma("omp atomic") (target) += v__; \
    } while (0)

/* Backward of orc_blend.  g_rgb [3,H,W]; g_depth, g_alpha [H,W] or NULL.
 * acc: double[P][ORC_GRAD], zero-filled by the caller; pixel-space gradients
 * of (px, py), of the conic as it enters the exponent
 * power = -0.5 (cx dx^2 + cz dy^2) - cy dx dy, of opacity, colour and depth. */
void orc_blend_backward(const orc_frame *f, const uint32_t *ranges, const uint32_t *values, const float *xy,
                        const float *conic_opacity, const float *rgb, const float *depth, const float *g_rgb,
                        const float *g_depth, const float *g_alpha, double *acc)
{
    int W = f->image_width, H = f->image_height;
    int grid_x = (W + ORC_TILE - 1) / ORC_TILE, grid_y = (H + ORC_TILE - 1) / ORC_TILE;
    /* tiles in parallel; a Gaussian's accumulators are shared between the tiles it touches, hence the atomic adds
     * (doubles: the order of the additions changes the sums by ~1e-16 relative, far below any comparison) */
#pragma omp parallel
    {
    size_t cap = 1024;
    orc_hit *hits = (orc_hit *)malloc(cap * sizeof *hits);
#pragma omp for schedule(dynamic, 4)
    for (int t = 0; t < grid_x * grid_y; ++t) {
        int tx0 = (t % grid_x) * ORC_TILE, ty0 = (t / grid_x) * ORC_TILE;
        uint32_t lo = ranges[2 * t], hi = ranges[2 * t + 1];
        for (int py = ty0; py < ty0 + ORC_TILE && py < H; ++py)
            for (int px = tx0; px < tx0 + ORC_TILE && px < W; ++px) {
                /* forward, as orc_blend: the list of blended Gaussians and the final transmittance */
                size_t n = 0;
                float T = 1.f;
                for (uint32_t j = lo; j < hi; ++j) {
                    uint32_t gi = values[j];
                    float dx = xy[2 * gi] - (float)px, dy = xy[2 * gi + 1] - (float)py;
                    const float *co = conic_opacity + 4 * (size_t)gi;
                    float t1 = co[0] * dx * dx, t2 = co[2] * dy * dy, t3 = co[1] * dx * dy;
                    float power = -0.5f * (t1 + t2) - t3;
                    if (power > 0.f) continue;
                    float G = expf(power);
                    float alpha = fminf(0.99f, co[3] * G);
                    if (alpha < 1.0f / 255.0f) continue;
                    float test_T = T * (1.f - alpha);
                    if (test_T < 0.0001f) break;
                    if (n == cap) {
                        cap *= 2;
                        hits = (orc_hit *)realloc(hits, cap * sizeof *hits);
                    }
                    hits[n].g = gi; hits[n].dx = dx; hits[n].dy = dy; hits[n].G = G; hits[n].alpha = alpha; hits[n].T = T;
                    ++n;
                    T = test_T;
                }
                size_t o = (size_t)py * W + px;
                double gc[4] = {g_rgb[o], g_rgb[(size_t)H * W + o], g_rgb[2 * (size_t)H * W + o],
                                g_depth ? g_depth[o] : 0.0};
                double ga = g_alpha ? g_alpha[o] : 0.0;
                double T_final = T;
                /* what lies behind the last Gaussian: background colour, no depth; alpha_out = 1 - T_final */
                double bg_dot = f->bg[0] * gc[0] + f->bg[1] * gc[1] + f->bg[2] * gc[2] - ga;
                double behind[4] = {0, 0, 0, 0}; /* colour/depth accumulated behind the current Gaussian */
                double last_alpha = 0.0, last_col[4] = {0, 0, 0, 0};
                for (size_t k = n; k-- > 0;) {
                    const orc_hit *h = hits + k;
                    const float *co = conic_opacity + 4 * (size_t)h->g;
                    double a = h->alpha, Tk = h->T;
                    double col[4] = {rgb[3 * (size_t)h->g], rgb[3 * (size_t)h->g + 1], rgb[3 * (size_t)h->g + 2],
                                     depth[h->g]};
                    double *A = acc + (size_t)h->g * ORC_GRAD;
                    double dL_dalpha = 0.0;
                    for (int c = 0; c < 4; ++c) {
                        behind[c] = last_alpha * last_col[c] + (1.0 - last_alpha) * behind[c];
                        last_col[c] = col[c];
                        dL_dalpha += (col[c] - behind[c]) * gc[c];
                        ORC_ADD(A[6 + c], a * Tk * gc[c]);
                    }
                    dL_dalpha *= Tk;
                    last_alpha = a;
                    dL_dalpha += (-T_final / (1.0 - a)) * bg_dot;
                    double G = h->G, dx = h->dx, dy = h->dy;
                    double dL_dG = co[3] * dL_dalpha; /* through the min(0.99, .) unchanged */
                    double dL_dpower = G * dL_dG;
                    ORC_ADD(A[0], dL_dpower * (-(double)co[0] * dx - (double)co[1] * dy));
                    ORC_ADD(A[1], dL_dpower * (-(double)co[2] * dy - (double)co[1] * dx));
                    ORC_ADD(A[2], dL_dpower * (-0.5 * dx * dx));
                    ORC_ADD(A[3], dL_dpower * (-dx * dy));
                    ORC_ADD(A[4], dL_dpower * (-0.5 * dy * dy));
                    ORC_ADD(A[5], G * dL_dalpha);
                }
            }
    }
    free(hits);
    }
}

static const double SH_C0 = 0.28209479177387814;
static const double SH_C1 = 0.4886025119029199;
static const double SH_C2[5] = {1.0925484305920792, -1.0925484305920792, 0.31539156525252005, -1.0925484305920792,
                                0.5462742152960396};
static const double SH_C3[7] = {-0.5900435899266435, 2.890611442640554, -0.4570457994644658, 0.3731763325901154,
                                -0.4570457994644658, 1.445305721320277, -0.5900435899266435};

/* Real SH basis of sh_utils.py:67-94 and its gradient with respect to the unit direction. */
static void sh_basis(int deg, double x, double y, double z, double b[16], double bx[16], double by[16], double bz[16])
{
    for (int k = 0; k < 16; ++k) b[k] = bx[k] = by[k] = bz[k] = 0.0;
    b[0] = SH_C0;
    if (deg < 1) return;
    b[1] = -SH_C1 * y; by[1] = -SH_C1;
    b[2] = SH_C1 * z;  bz[2] = SH_C1;
    b[3] = -SH_C1 * x; bx[3] = -SH_C1;
    if (deg < 2) return;
    double xx = x * x, yy = y * y, zz = z * z, xy = x * y, yz = y * z, xz = x * z;
    b[4] = SH_C2[0] * xy;                  bx[4] = SH_C2[0] * y;      by[4] = SH_C2[0] * x;
    b[5] = SH_C2[1] * yz;                  by[5] = SH_C2[1] * z;      bz[5] = SH_C2[1] * y;
    b[6] = SH_C2[2] * (2.0 * zz - xx - yy); bx[6] = SH_C2[2] * -2.0 * x; by[6] = SH_C2[2] * -2.0 * y; bz[6] = SH_C2[2] * 4.0 * z;
    b[7] = SH_C2[3] * xz;                  bx[7] = SH_C2[3] * z;      bz[7] = SH_C2[3] * x;
    b[8] = SH_C2[4] * (xx - yy);           bx[8] = SH_C2[4] * 2.0 * x; by[8] = SH_C2[4] * -2.0 * y;
    if (deg < 3) return;
    b[9] = SH_C3[0] * y * (3.0 * xx - yy);
    bx[9] = SH_C3[0] * 6.0 * xy; by[9] = SH_C3[0] * (3.0 * xx - 3.0 * yy);
    b[10] = SH_C3[1] * xy * z;
    bx[10] = SH_C3[1] * yz; by[10] = SH_C3[1] * xz; bz[10] = SH_C3[1] * xy;
    b[11] = SH_C3[2] * y * (4.0 * zz - xx - yy);
    bx[11] = SH_C3[2] * -2.0 * xy; by[11] = SH_C3[2] * (4.0 * zz - xx - 3.0 * yy); bz[11] = SH_C3[2] * 8.0 * yz;
    b[12] = SH_C3[3] * z * (2.0 * zz - 3.0 * xx - 3.0 * yy);
    bx[12] = SH_C3[3] * -6.0 * xz; by[12] = SH_C3[3] * -6.0 * yz; bz[12] = SH_C3[3] * (6.0 * zz - 3.0 * xx - 3.0 * yy);
    b[13] = SH_C3[4] * x * (4.0 * zz - xx - yy);
    bx[13] = SH_C3[4] * (4.0 * zz - 3.0 * xx - yy); by[13] = SH_C3[4] * -2.0 * xy; bz[13] = SH_C3[4] * 8.0 * xz;
    b[14] = SH_C3[5] * z * (xx - yy);
    bx[14] = SH_C3[5] * 2.0 * xz; by[14] = SH_C3[5] * -2.0 * yz; bz[14] = SH_C3[5] * (xx - yy);
    b[15] = SH_C3[6] * x * (xx - 3.0 * yy);
    bx[15] = SH_C3[6] * (3.0 * xx - 3.0 * yy); by[15] = SH_C3[6] * -6.0 * xy;
}

/* Backward of orc_preprocess for the Gaussians with radii > 0 (the others get
 * zero gradients).  acc: the accumulators of orc_blend_backward.  Outputs
 * (each may be NULL when the matching input is): d_means3D [P,3], d_means2D
 * [P,3], d_shs [P,M,3], d_colors [P,3], d_opacities [P], d_scales [P,3],
 * d_rotations [P,4], d_cov3D [P,6]; all doubles. */
void orc_preprocess_backward(const orc_frame *f, const orc_gaussians *g, const int32_t *radii, const double *acc,
                             double *d_means3D, double *d_means2D, double *d_shs, double *d_colors,
                             double *d_opacities, double *d_scales, double *d_rotations, double *d_cov3D)
{
    const float *V = f->viewmatrix, *Pm = f->projmatrix;
    int M = f->sh_coeffs;
    double W_img = f->image_width, H_img = f->image_height;
    double fx = W_img / (2.0 * (double)f->tanfovx), fy = H_img / (2.0 * (double)f->tanfovy);
    double limx = 1.3 * (double)f->tanfovx, limy = 1.3 * (double)f->tanfovy;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < g->P; ++i) {
        if (radii[i] <= 0) continue;
        const double *A = acc + (size_t)i * ORC_GRAD;
        double x = g->means3D[3 * i], y = g->means3D[3 * i + 1], z = g->means3D[3 * i + 2];
        double dmean[3] = {0, 0, 0};

        /* ---- pixel position: px = ((phx / (phw + 1e-7) + 1) W - 1) / 2 ---- */
        double phx = Pm[0] * x + Pm[4] * y + Pm[8] * z + Pm[12];
        double phy = Pm[1] * x + Pm[5] * y + Pm[9] * z + Pm[13];
        double phw = Pm[3] * x + Pm[7] * y + Pm[11] * z + Pm[15];
        double pw = 1.0 / (phw + 0.0000001);
        double d_ppx = A[0] * 0.5 * W_img, d_ppy = A[1] * 0.5 * H_img;
        double d_phx = d_ppx * pw, d_phy = d_ppy * pw;
        double d_phw = -(pw * pw) * (phx * d_ppx + phy * d_ppy);
        for (int k = 0; k < 3; ++k) dmean[k] += Pm[4 * k + 0] * d_phx + Pm[4 * k + 1] * d_phy + Pm[4 * k + 3] * d_phw;
        if (d_means2D) {
            d_means2D[3 * i] = d_ppx;
            d_means2D[3 * i + 1] = d_ppy;
            d_means2D[3 * i + 2] = 0.0;
        }

        /* ---- 3-D covariance (from scale / rotation, or given) ---- */
        double S[3][3], R[3][3], s[3] = {0, 0, 0}, q[4] = {0, 0, 0, 0};
        if (g->cov3D_precomp) {
            const float *c = g->cov3D_precomp + 6 * (size_t)i;
            S[0][0] = c[0]; S[0][1] = S[1][0] = c[1]; S[0][2] = S[2][0] = c[2];
            S[1][1] = c[3]; S[1][2] = S[2][1] = c[4]; S[2][2] = c[5];
        } else {
            for (int k = 0; k < 3; ++k) s[k] = (double)f->scale_modifier * g->scales[3 * (size_t)i + k];
            for (int k = 0; k < 4; ++k) q[k] = g->rotations[4 * (size_t)i + k];
            double r = q[0], qx = q[1], qy = q[2], qz = q[3];
            R[0][0] = 1 - 2 * (qy * qy + qz * qz); R[0][1] = 2 * (qx * qy - r * qz); R[0][2] = 2 * (qx * qz + r * qy);
            R[1][0] = 2 * (qx * qy + r * qz); R[1][1] = 1 - 2 * (qx * qx + qz * qz); R[1][2] = 2 * (qy * qz - r * qx);
            R[2][0] = 2 * (qx * qz - r * qy); R[2][1] = 2 * (qy * qz + r * qx); R[2][2] = 1 - 2 * (qx * qx + qy * qy);
            for (int a = 0; a < 3; ++a)
                for (int b = 0; b < 3; ++b) {
                    S[a][b] = 0;
                    for (int k = 0; k < 3; ++k) S[a][b] += R[a][k] * s[k] * R[b][k] * s[k];
                }
        }

        /* ---- view-space position and the Jacobian of the projection ---- */
        double pvx = V[0] * x + V[4] * y + V[8] * z + V[12];
        double pvy = V[1] * x + V[5] * y + V[9] * z + V[13];
        double pvz = V[2] * x + V[6] * y + V[10] * z + V[14];
        double tz = pvz;
        double rx = pvx / tz, ry = pvy / tz;
        int clamp_x = rx > limx ? 1 : rx < -limx ? -1 : 0, clamp_y = ry > limy ? 1 : ry < -limy ? -1 : 0;
        double tx = clamp_x ? clamp_x * limx * tz : pvx, ty = clamp_y ? clamp_y * limy * tz : pvy;
        double J00 = fx / tz, J02 = -(fx * tx) / (tz * tz), J11 = fy / tz, J12 = -(fy * ty) / (tz * tz);
        double a0[3], a1[3];
        for (int k = 0; k < 3; ++k) {
            a0[k] = J00 * V[4 * k + 0] + J02 * V[4 * k + 2];
            a1[k] = J11 * V[4 * k + 1] + J12 * V[4 * k + 2];
        }
        double Sa0[3], Sa1[3];
        for (int k = 0; k < 3; ++k) {
            Sa0[k] = S[k][0] * a0[0] + S[k][1] * a0[1] + S[k][2] * a0[2];
            Sa1[k] = S[k][0] * a1[0] + S[k][1] * a1[1] + S[k][2] * a1[2];
        }
        double ca = a0[0] * Sa0[0] + a0[1] * Sa0[1] + a0[2] * Sa0[2] + 0.3;
        double cb = a0[0] * Sa1[0] + a0[1] * Sa1[1] + a0[2] * Sa1[2];
        double cc = a1[0] * Sa1[0] + a1[1] * Sa1[1] + a1[2] * Sa1[2] + 0.3;
        double det = ca * cc - cb * cb, D = 1.0 / det, D2 = D * D;
        /* conic = (cc, -cb, ca) / det */
        double gA = A[2], gB = A[3], gC = A[4];
        double d_ca = gA * (-cc * cc * D2) + gB * (cb * cc * D2) + gC * (D - ca * cc * D2);
        double d_cb = gA * (2 * cb * cc * D2) + gB * (-D - 2 * cb * cb * D2) + gC * (2 * ca * cb * D2);
        double d_cc = gA * (D - ca * cc * D2) + gB * (ca * cb * D2) + gC * (-ca * ca * D2);
        /* cov2D = [a0;a1] S [a0;a1]^T */
        double dS[3][3];
        for (int k = 0; k < 3; ++k)
            for (int l = 0; l < 3; ++l)
                dS[k][l] = d_ca * a0[k] * a0[l] + d_cb * 0.5 * (a0[k] * a1[l] + a1[k] * a0[l]) + d_cc * a1[k] * a1[l];
        double d_a0[3], d_a1[3];
        for (int k = 0; k < 3; ++k) {
            d_a0[k] = 2 * d_ca * Sa0[k] + d_cb * Sa1[k];
            d_a1[k] = 2 * d_cc * Sa1[k] + d_cb * Sa0[k];
        }
        double d_J00 = 0, d_J02 = 0, d_J11 = 0, d_J12 = 0;
        for (int k = 0; k < 3; ++k) {
            d_J00 += d_a0[k] * V[4 * k + 0];
            d_J02 += d_a0[k] * V[4 * k + 2];
            d_J11 += d_a1[k] * V[4 * k + 1];
            d_J12 += d_a1[k] * V[4 * k + 2];
        }
        double tz2 = tz * tz, tz3 = tz2 * tz;
        double d_tx = d_J02 * (-fx / tz2), d_ty = d_J12 * (-fy / tz2);
        double d_tz = d_J00 * (-fx / tz2) + d_J11 * (-fy / tz2) + d_J02 * (2 * fx * tx / tz3) + d_J12 * (2 * fy * ty / tz3);
        double d_pvx = clamp_x ? 0.0 : d_tx, d_pvy = clamp_y ? 0.0 : d_ty;
        double d_pvz = d_tz + (clamp_x ? clamp_x * limx * d_tx : 0.0) + (clamp_y ? clamp_y * limy * d_ty : 0.0);
        d_pvz += A[9]; /* depth output: the blended quantity is the view-space z */
        for (int k = 0; k < 3; ++k) dmean[k] += V[4 * k + 0] * d_pvx + V[4 * k + 1] * d_pvy + V[4 * k + 2] * d_pvz;

        if (g->cov3D_precomp) {
            if (d_cov3D) {
                double *o = d_cov3D + 6 * (size_t)i;
                o[0] = dS[0][0]; o[1] = dS[0][1] + dS[1][0]; o[2] = dS[0][2] + dS[2][0];
                o[3] = dS[1][1]; o[4] = dS[1][2] + dS[2][1]; o[5] = dS[2][2];
            }
        } else {
            /* Sigma = L L^T, L = R diag(s): dL = (dS + dS^T) L */
            double L[3][3], dL[3][3];
            for (int a = 0; a < 3; ++a)
                for (int k = 0; k < 3; ++k) L[a][k] = R[a][k] * s[k];
            for (int a = 0; a < 3; ++a)
                for (int k = 0; k < 3; ++k) {
                    dL[a][k] = 0;
                    for (int b = 0; b < 3; ++b) dL[a][k] += (dS[a][b] + dS[b][a]) * L[b][k];
                }
            double dR[3][3];
            for (int k = 0; k < 3; ++k) {
                double ds = 0;
                for (int a = 0; a < 3; ++a) {
                    ds += dL[a][k] * R[a][k];
                    dR[a][k] = dL[a][k] * s[k];
                }
                if (d_scales) d_scales[3 * (size_t)i + k] = ds * (double)f->scale_modifier;
            }
            if (d_rotations) {
                double r = q[0], qx = q[1], qy = q[2], qz = q[3];
                double *o = d_rotations + 4 * (size_t)i;
                o[0] = 2 * (-qz * dR[0][1] + qy * dR[0][2] + qz * dR[1][0] - qx * dR[1][2] - qy * dR[2][0] + qx * dR[2][1]);
                o[1] = 2 * (qy * dR[0][1] + qz * dR[0][2] + qy * dR[1][0] - 2 * qx * dR[1][1] - r * dR[1][2] + qz * dR[2][0] +
                            r * dR[2][1] - 2 * qx * dR[2][2]);
                o[2] = 2 * (-2 * qy * dR[0][0] + qx * dR[0][1] + r * dR[0][2] + qx * dR[1][0] + qz * dR[1][2] - r * dR[2][0] +
                            qz * dR[2][1] - 2 * qy * dR[2][2]);
                o[3] = 2 * (-2 * qz * dR[0][0] - r * dR[0][1] + qx * dR[0][2] + r * dR[1][0] - 2 * qz * dR[1][1] + qy * dR[1][2] +
                            qx * dR[2][0] + qy * dR[2][1]);
            }
        }

        /* ---- colour ---- */
        if (g->colors_precomp) {
            if (d_colors)
                for (int c = 0; c < 3; ++c) d_colors[3 * (size_t)i + c] = A[6 + c];
        } else {
            double dir[3] = {x - f->campos[0], y - f->campos[1], z - f->campos[2]};
            double len = sqrt(dir[0] * dir[0] + dir[1] * dir[1] + dir[2] * dir[2]);
            double n[3] = {dir[0] / len, dir[1] / len, dir[2] / len};
            double b[16], bx[16], by[16], bz[16];
            sh_basis(f->sh_degree, n[0], n[1], n[2], b, bx, by, bz);
            int K = (f->sh_degree + 1) * (f->sh_degree + 1);
            const float *sh = g->shs + (size_t)i * M * 3;
            double dn[3] = {0, 0, 0};
            for (int c = 0; c < 3; ++c) {
                double res = 0;
                for (int k = 0; k < K; ++k) res += b[k] * sh[3 * k + c];
                double gcol = (res + 0.5 < 0.0) ? 0.0 : A[6 + c]; /* clamp_min(., 0) */
                for (int k = 0; k < M; ++k)
                    if (d_shs) d_shs[((size_t)i * M + k) * 3 + c] = k < K ? b[k] * gcol : 0.0;
                for (int k = 0; k < K; ++k) {
                    dn[0] += gcol * sh[3 * k + c] * bx[k];
                    dn[1] += gcol * sh[3 * k + c] * by[k];
                    dn[2] += gcol * sh[3 * k + c] * bz[k];
                }
            }
            double dot = n[0] * dn[0] + n[1] * dn[1] + n[2] * dn[2];
            for (int k = 0; k < 3; ++k) dmean[k] += (dn[k] - n[k] * dot) / len;
        }

        if (d_opacities) d_opacities[i] = A[5];
        if (d_means3D)
            for (int k = 0; k < 3; ++k) d_means3D[3 * (size_t)i + k] = dmean[k];
    }
}
