/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement ("oracle") of deformable aggregation
 * (multi-camera, multi-scale bilinear sampling with one weight per channel group).
 * Nothing in the shipped library links, loads or calls this file.
 *
 * The loops restate the goldens of the reference's own tests:
 *   forward   tests/torch/test_deformable_aggregation.py:29-126
 *   backward  tests/torch/test_deformable_aggregation_grad.py:33-181
 * (a sample is skipped unless 0 < x < 1 and 0 < y < 1; pixel coordinates x*W-0.5, y*H-0.5;
 *  corner predicates h_low >= 0, w_low >= 0, h_high <= H-1, w_high <= W-1; the location
 *  gradient is W * (d/dx of the bilinear form) * weight * grad, summed over scales and groups).
 *
 * Parity pins (tests/test_oracle.py): the same operator expressed through the multi-scale
 * deformable attention oracle (locations broadcast over scales and groups, weights permuted
 * and masked), a hand-computed case, and finite differences.
 *
 * Layouts (row-major, contiguous):
 *   feat [bs, num_feat, C]   spatial_shape [cams, scales, 2]=(H,W)   scale_start_index [cams, scales]
 *   loc [bs, anchors, pts, cams, 2]=(x,y)   weights [bs, anchors, pts, cams, scales, groups]
 *   out [bs, anchors, C]; group g owns channels [g*C/groups, (g+1)*C/groups)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define DAGG_DEFINE(SUFFIX, REAL, FLOOR)                                                                    \
    int dagg_oracle_forward_##SUFFIX(const REAL* feat, const int32_t* ss, const int32_t* ssi, const REAL* loc, \
        const REAL* wts, REAL* out, int64_t bs, int64_t nf, int64_t C, int64_t cams, int64_t scales,         \
        int64_t A, int64_t P, int64_t G)                                                                     \
    {                                                                                                       \
        if (G <= 0 || C % G) return -1;                                                                      \
        const int64_t cg = C / G;                                                                           \
        _Pragma("omp parallel for collapse(2) schedule(static)")                                            \
        for (int64_t b = 0; b < bs; ++b) {                                                                  \
            for (int64_t a = 0; a < A; ++a) {                                                               \
                REAL* o = out + (b * A + a) * C;                                                            \
                for (int64_t c = 0; c < C; ++c) o[c] = 0;                                                   \
                for (int64_t p = 0; p < P; ++p)                                                             \
                for (int64_t cam = 0; cam < cams; ++cam) {                                                  \
                    const REAL x = loc[(((b * A + a) * P + p) * cams + cam) * 2];                           \
                    const REAL y = loc[(((b * A + a) * P + p) * cams + cam) * 2 + 1];                       \
                    if (!(x > 0 && x < 1 && y > 0 && y < 1)) continue;                                      \
                    for (int64_t sc = 0; sc < scales; ++sc) {                                               \
                        const int64_t H = ss[(cam * scales + sc) * 2], W = ss[(cam * scales + sc) * 2 + 1]; \
                        const int64_t base = ssi[cam * scales + sc];                                        \
                        const REAL h_im = y * (REAL)H - (REAL)0.5, w_im = x * (REAL)W - (REAL)0.5;          \
                        const REAL fy = FLOOR(h_im), fx = FLOOR(w_im);                                      \
                        const int64_t y0 = (int64_t)fy, x0 = (int64_t)fx;                                   \
                        const REAL lh = h_im - fy, lw = w_im - fx, hh = 1 - lh, hw = 1 - lw;                \
                        const REAL wgt[4] = {hh * hw, hh * lw, lh * hw, lh * lw};                           \
                        const REAL* wrow = wts + ((((b * A + a) * P + p) * cams + cam) * scales + sc) * G;  \
                        for (int k = 0; k < 4; ++k) {                                                       \
                            const int64_t yy = y0 + (k >> 1), xx = x0 + (k & 1);                            \
                            if (yy < 0 || yy > H - 1 || xx < 0 || xx > W - 1) continue;                     \
                            const REAL* v = feat + (b * nf + base + yy * W + xx) * C;                       \
                            for (int64_t c = 0; c < C; ++c) o[c] += wgt[k] * v[c] * wrow[c / cg];           \
                        }                                                                                   \
                    }                                                                                       \
                }                                                                                           \
            }                                                                                               \
        }                                                                                                   \
        return 0;                                                                                           \
    }                                                                                                       \
    int dagg_oracle_backward_##SUFFIX(const REAL* feat, const int32_t* ss, const int32_t* ssi, const REAL* loc, \
        const REAL* wts, const REAL* gout, REAL* gfeat, REAL* gloc, REAL* gw, int64_t bs, int64_t nf,       \
        int64_t C, int64_t cams, int64_t scales, int64_t A, int64_t P, int64_t G)                           \
    {                                                                                                       \
        if (G <= 0 || C % G) return -1;                                                                      \
        const int64_t cg = C / G;                                                                           \
        memset(gfeat, 0, sizeof(REAL) * (size_t)(bs * nf * C));                                             \
        memset(gloc, 0, sizeof(REAL) * (size_t)(bs * A * P * cams * 2));                                    \
        memset(gw, 0, sizeof(REAL) * (size_t)(bs * A * P * cams * scales * G));                             \
        /* serial over anchors: grad_feat rows are shared between anchors */                               \
        for (int64_t b = 0; b < bs; ++b)                                                                    \
        for (int64_t a = 0; a < A; ++a) {                                                                   \
            const REAL* go = gout + (b * A + a) * C;                                                        \
            for (int64_t p = 0; p < P; ++p)                                                                 \
            for (int64_t cam = 0; cam < cams; ++cam) {                                                      \
                const int64_t li = ((b * A + a) * P + p) * cams + cam;                                      \
                const REAL x = loc[li * 2], y = loc[li * 2 + 1];                                            \
                if (!(x > 0 && x < 1 && y > 0 && y < 1)) continue;                                          \
                for (int64_t sc = 0; sc < scales; ++sc) {                                                   \
                    const int64_t H = ss[(cam * scales + sc) * 2], W = ss[(cam * scales + sc) * 2 + 1];     \
                    const int64_t base = ssi[cam * scales + sc];                                            \
                    const REAL h_im = y * (REAL)H - (REAL)0.5, w_im = x * (REAL)W - (REAL)0.5;              \
                    const REAL fy = FLOOR(h_im), fx = FLOOR(w_im);                                          \
                    const int64_t y0 = (int64_t)fy, x0 = (int64_t)fx;                                       \
                    const REAL lh = h_im - fy, lw = w_im - fx, hh = 1 - lh, hw = 1 - lw;                    \
                    const REAL wgt[4] = {hh * hw, hh * lw, lh * hw, lh * lw};                               \
                    /* d(bilinear)/dh and /dw coefficients of the four corners */                          \
                    const REAL dh[4] = {-hw, -lw, hw, lw}, dw[4] = {-hh, hh, -lh, lh};                       \
                    const REAL* wrow = wts + (li * scales + sc) * G;                                        \
                    REAL* gwrow = gw + (li * scales + sc) * G;                                              \
                    for (int k = 0; k < 4; ++k) {                                                           \
                        const int64_t yy = y0 + (k >> 1), xx = x0 + (k & 1);                                \
                        if (yy < 0 || yy > H - 1 || xx < 0 || xx > W - 1) continue;                         \
                        const int64_t row = (b * nf + base + yy * W + xx) * C;                              \
                        for (int64_t c = 0; c < C; ++c) {                                                   \
                            const REAL top = go[c] * wrow[c / cg];                                          \
                            const REAL v = feat[row + c];                                                   \
                            gfeat[row + c] += wgt[k] * top;                                                 \
                            gwrow[c / cg] += go[c] * wgt[k] * v;                                            \
                            gloc[li * 2] += (REAL)W * dw[k] * v * top;                                      \
                            gloc[li * 2 + 1] += (REAL)H * dh[k] * v * top;                                  \
                        }                                                                                   \
                    }                                                                                       \
                }                                                                                           \
            }                                                                                               \
        }                                                                                                   \
        return 0;                                                                                           \
    }

DAGG_DEFINE(f64, double, floor)
DAGG_DEFINE(f32, float, floorf)
