/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement ("oracle") of multi-scale deformable
 * attention, direct bilinear form.  Nothing in the shipped library links, loads or
 * calls this file; it is the checker the HIP kernels are compared against and the
 * "port" CPU baseline that the benchmark times next to the GPU.
 *
 * The arithmetic follows the per-thread (SIMT) statement of the operator in the
 * reference:
 *   validity of a sample      kernels/multi_scale_deformable_attn/op_kernel/arch35/multi_scale_deformable_attn.cpp:16-34
 *   corner predicates/weights kernels/multi_scale_deformable_attn/op_kernel/arch35/multi_scale_deformable_attn.cpp:36-80
 *   pixel-space coordinates   kernels/multi_scale_deformable_attn/op_kernel/msda.h:351-389   (x*W-0.5, y*H-0.5)
 *   bilinear weights          kernels/multi_scale_deformable_attn/op_kernel/msda.h:487-539
 *   gradients                 kernels/multi_scale_deformable_attn/op_kernel/multi_scale_deformable_attn_grad.cpp:208-249
 *                             kernels/multi_scale_deformable_attn/op_kernel/arch35/multi_scale_deformable_attn_grad.cpp:16-145
 *   dtype / extra-level rule  mx_driving/csrc/MultiScaleDeformableAttn.cpp:93-101
 *
 * Parity pins (tests/test_oracle.py): agreement with torch's grid_sample
 * (bilinear, zeros, align_corners=False) in float64, closed forms (constant and
 * affine value fields, pixel-centre samples), hand-computed 2x3 fixtures, finite
 * differences for the three gradients, and the reference's NaN/Inf known answers
 * (tests/torch/test_multi_scale_deformable_attn.py:266-282).
 * Unpinned: behaviour when attention_weights carries more levels than
 * spatial_shapes (only the intent "extra levels ignored, zero grads" is recoverable).
 *
 * Layouts (row-major, contiguous):
 *   value [bs, nk, nh, hd]   shapes [nl,2]=(H,W)   lsi [nl]
 *   loc   [bs, nq, nh, nl_attn, np, 2]=(x,y)   attn [bs, nq, nh, nl_attn, np]
 *   out   [bs, nq, nh*hd]
 * Only the first nl of the nl_attn levels are sampled.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define MSDA_DEFINE(SUFFIX, REAL, FLOOR)                                                                  \
    int msda_oracle_forward_##SUFFIX(const REAL* value, const int32_t* shapes, const int32_t* lsi,       \
        const REAL* loc, const REAL* attn, REAL* out, int64_t bs, int64_t nk, int64_t nh, int64_t hd,    \
        int64_t nl, int64_t nl_attn, int64_t nq, int64_t np)                                             \
    {                                                                                                     \
        if (nl > nl_attn) return -1;                                                                      \
        _Pragma("omp parallel for collapse(2) schedule(static)")                                          \
        for (int64_t b = 0; b < bs; ++b) {                                                                \
            for (int64_t q = 0; q < nq; ++q) {                                                            \
                for (int64_t h = 0; h < nh; ++h) {                                                        \
                    REAL* o = out + ((b * nq + q) * nh + h) * hd;                                         \
                    for (int64_t c = 0; c < hd; ++c) o[c] = 0;                                            \
                    for (int64_t l = 0; l < nl; ++l) {                                                    \
                        const int64_t H = shapes[2 * l], W = shapes[2 * l + 1], base = lsi[l];            \
                        for (int64_t p = 0; p < np; ++p) {                                                \
                            const int64_t s = (((b * nq + q) * nh + h) * nl_attn + l) * np + p;           \
                            const REAL x = loc[2 * s], y = loc[2 * s + 1], a = attn[s];                   \
                            const REAL w_im = x * (REAL)W - (REAL)0.5, h_im = y * (REAL)H - (REAL)0.5;    \
                            if (!(h_im > -1 && w_im > -1 && h_im < (REAL)H && w_im < (REAL)W)) continue;  \
                            const REAL fx = FLOOR(w_im), fy = FLOOR(h_im);                                \
                            const int64_t x0 = (int64_t)fx, y0 = (int64_t)fy;                             \
                            const REAL lw = w_im - fx, lh = h_im - fy, hw = 1 - lw, hh = 1 - lh;          \
                            const REAL wgt[4] = {hh * hw, hh * lw, lh * hw, lh * lw};                     \
                            for (int k = 0; k < 4; ++k) {                                                 \
                                const int64_t yy = y0 + (k >> 1), xx = x0 + (k & 1);                      \
                                if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue;                     \
                                const REAL* v = value + ((b * nk + base + yy * W + xx) * nh + h) * hd;    \
                                const REAL wa = wgt[k];                                                   \
                                for (int64_t c = 0; c < hd; ++c) o[c] += a * (wa * v[c]);                 \
                            }                                                                             \
                        }                                                                                 \
                    }                                                                                     \
                }                                                                                         \
            }                                                                                             \
        }                                                                                                 \
        return 0;                                                                                         \
    }                                                                                                     \
                                                                                                          \
    int msda_oracle_backward_##SUFFIX(const REAL* value, const int32_t* shapes, const int32_t* lsi,      \
        const REAL* loc, const REAL* attn, const REAL* grad_out, REAL* grad_value, REAL* grad_loc,       \
        REAL* grad_attn, int64_t bs, int64_t nk, int64_t nh, int64_t hd, int64_t nl, int64_t nl_attn,    \
        int64_t nq, int64_t np)                                                                           \
    {                                                                                                     \
        if (nl > nl_attn) return -1;                                                                      \
        memset(grad_value, 0, sizeof(REAL) * (size_t)(bs * nk * nh * hd));                                \
        memset(grad_loc, 0, sizeof(REAL) * (size_t)(bs * nq * nh * nl_attn * np * 2));                    \
        memset(grad_attn, 0, sizeof(REAL) * (size_t)(bs * nq * nh * nl_attn * np));                       \
        /* (b,h) pairs own disjoint slices of grad_value, so they can run in parallel. */                 \
        _Pragma("omp parallel for collapse(2) schedule(dynamic)")                                         \
        for (int64_t b = 0; b < bs; ++b) {                                                                \
            for (int64_t h = 0; h < nh; ++h) {                                                            \
                for (int64_t q = 0; q < nq; ++q) {                                                        \
                    const REAL* g = grad_out + ((b * nq + q) * nh + h) * hd;                              \
                    for (int64_t l = 0; l < nl; ++l) {                                                    \
                        const int64_t H = shapes[2 * l], W = shapes[2 * l + 1], base = lsi[l];            \
                        for (int64_t p = 0; p < np; ++p) {                                                \
                            const int64_t s = (((b * nq + q) * nh + h) * nl_attn + l) * np + p;           \
                            const REAL x = loc[2 * s], y = loc[2 * s + 1], a = attn[s];                   \
                            const REAL w_im = x * (REAL)W - (REAL)0.5, h_im = y * (REAL)H - (REAL)0.5;    \
                            if (!(h_im > -1 && w_im > -1 && h_im < (REAL)H && w_im < (REAL)W)) continue;  \
                            const REAL fx = FLOOR(w_im), fy = FLOOR(h_im);                                \
                            const int64_t x0 = (int64_t)fx, y0 = (int64_t)fy;                             \
                            const REAL lw = w_im - fx, lh = h_im - fy, hw = 1 - lw, hh = 1 - lh;          \
                            const REAL wgt[4] = {hh * hw, hh * lw, lh * hw, lh * lw};                     \
                            REAL d[4] = {0, 0, 0, 0};                                                     \
                            for (int k = 0; k < 4; ++k) {                                                 \
                                const int64_t yy = y0 + (k >> 1), xx = x0 + (k & 1);                      \
                                if (yy < 0 || yy >= H || xx < 0 || xx >= W) continue;                     \
                                const int64_t row = ((b * nk + base + yy * W + xx) * nh + h) * hd;        \
                                const REAL* v = value + row;                                              \
                                REAL* gv = grad_value + row;                                              \
                                const REAL wa = wgt[k] * a;                                               \
                                REAL dot = 0;                                                             \
                                for (int64_t c = 0; c < hd; ++c) {                                        \
                                    gv[c] += wa * g[c];                                                   \
                                    dot += v[c] * g[c];                                                   \
                                }                                                                         \
                                d[k] = dot;                                                               \
                            }                                                                             \
                            grad_attn[s] = wgt[0] * d[0] + wgt[1] * d[1] + wgt[2] * d[2] + wgt[3] * d[3]; \
                            grad_loc[2 * s] = (REAL)W * a * (hh * (d[1] - d[0]) + lh * (d[3] - d[2]));    \
                            grad_loc[2 * s + 1] = (REAL)H * a * (hw * (d[2] - d[0]) + lw * (d[3] - d[1]));\
                        }                                                                                 \
                    }                                                                                     \
                }                                                                                         \
            }                                                                                             \
        }                                                                                                 \
        return 0;                                                                                         \
    }

MSDA_DEFINE(f64, double, floor)
MSDA_DEFINE(f32, float, floorf)

#ifdef _OPENMP
#include <omp.h>
int msda_oracle_threads(void) { return omp_get_max_threads(); }
void msda_oracle_set_threads(int n) { if (n > 0) omp_set_num_threads(n); }
#else
int msda_oracle_threads(void) { return 1; }
void msda_oracle_set_threads(int n) { (void)n; }
#endif
