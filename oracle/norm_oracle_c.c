/* Scalar C restatement of the eager normalization formulas.
 * TEST INFRASTRUCTURE ONLY: nothing shipped links or loads this file.
 *
 * It follows the same reference lines as oracle/norm_oracle.py
 *   RMSNorm: teletron/models/dit/dit_fusedlayers.py:360-370
 *   AdaLN  : teletron/models/dit/dit_fusedlayers.py:198,223
 * but shares no code with PyTorch: bf16 is handled as raw uint16 with an
 * explicit round-to-nearest-even, every rounding point of the eager graph is
 * spelled out, and row statistics / column sums are accumulated in double and
 * rounded once (the value any correct fp32 summation order approximates).
 * Agreement between this file and the PyTorch restatement is what pins the
 * rounding points; build with -ffp-contract=off so no multiply-add is fused.
 *
 * "T" variants: element type of x / params / outputs is bf16 (uint16) or
 * float.  For float every "round to T" is the identity.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even, NaN kept quiet */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline float rnd_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

/* ---------------------------------------------------------------- RMSNorm */

void oc_rmsnorm_fwd_bf16(const uint16_t *x, const uint16_t *w, uint16_t *out, float *rstd,
                         long rows, long cols, double eps) {
    for (long n = 0; n < rows; ++n) {
        const uint16_t *xr = x + n * cols;
        double ss = 0.0;
        for (long c = 0; c < cols; ++c) {
            float v = bf16_to_f32(xr[c]);
            ss += (double)v * (double)v;
        }
        float ms = (float)(ss / (double)cols);
        float r = 1.0f / sqrtf(ms + (float)eps);
        rstd[n] = r;
        for (long c = 0; c < cols; ++c) {
            float y = rnd_bf16(bf16_to_f32(xr[c]) * r);         /* .type_as(x) */
            out[n * cols + c] = f32_to_bf16(y * bf16_to_f32(w[c])); /* * weight */
        }
    }
}

void oc_rmsnorm_fwd_f32(const float *x, const float *w, float *out, float *rstd,
                        long rows, long cols, double eps) {
    for (long n = 0; n < rows; ++n) {
        const float *xr = x + n * cols;
        double ss = 0.0;
        for (long c = 0; c < cols; ++c) ss += (double)xr[c] * (double)xr[c];
        float ms = (float)(ss / (double)cols);
        float r = 1.0f / sqrtf(ms + (float)eps);
        rstd[n] = r;
        for (long c = 0; c < cols; ++c) out[n * cols + c] = (xr[c] * r) * w[c];
    }
}

/* dw_acc: caller-provided double[cols] scratch */
void oc_rmsnorm_bwd_bf16(const uint16_t *x, const uint16_t *w, const float *rstd, const uint16_t *g,
                         uint16_t *dx, uint16_t *dw, double *dw_acc, long rows, long cols) {
    for (long c = 0; c < cols; ++c) dw_acc[c] = 0.0;
    for (long n = 0; n < rows; ++n) {
        const uint16_t *xr = x + n * cols, *gr = g + n * cols;
        float r = rstd[n];
        double dot = 0.0;
        for (long c = 0; c < cols; ++c) {
            float gy = rnd_bf16(bf16_to_f32(gr[c]) * bf16_to_f32(w[c])); /* grad of y, bf16 */
            float xh = bf16_to_f32(xr[c]) * r;
            dot += (double)(gy * xh);
        }
        float m = (float)(dot / (double)cols);
        for (long c = 0; c < cols; ++c) {
            float gv = bf16_to_f32(gr[c]);
            float gy = rnd_bf16(gv * bf16_to_f32(w[c]));
            float xh = bf16_to_f32(xr[c]) * r;
            dx[n * cols + c] = f32_to_bf16(r * (gy - xh * m));
            dw_acc[c] += (double)rnd_bf16(gv * rnd_bf16(xh));            /* g*y in bf16, then summed */
        }
    }
    for (long c = 0; c < cols; ++c) dw[c] = f32_to_bf16((float)dw_acc[c]);
}

void oc_rmsnorm_bwd_f32(const float *x, const float *w, const float *rstd, const float *g,
                        float *dx, float *dw, double *dw_acc, long rows, long cols) {
    for (long c = 0; c < cols; ++c) dw_acc[c] = 0.0;
    for (long n = 0; n < rows; ++n) {
        const float *xr = x + n * cols, *gr = g + n * cols;
        float r = rstd[n];
        double dot = 0.0;
        for (long c = 0; c < cols; ++c) dot += (double)((gr[c] * w[c]) * (xr[c] * r));
        float m = (float)(dot / (double)cols);
        for (long c = 0; c < cols; ++c) {
            float gy = gr[c] * w[c];
            float xh = xr[c] * r;
            dx[n * cols + c] = r * (gy - xh * m);
            dw_acc[c] += (double)(gr[c] * xh);
        }
    }
    for (long c = 0; c < cols; ++c) dw[c] = (float)dw_acc[c];
}

/* ------------------------------------------------------------------ AdaLN */

static void row_moments_bf16(const uint16_t *xr, long cols, double eps, float *mean, float *rstd) {
    double s = 0.0;
    for (long c = 0; c < cols; ++c) s += (double)bf16_to_f32(xr[c]);
    double mu = s / (double)cols;
    double m2 = 0.0;
    for (long c = 0; c < cols; ++c) {
        double d = (double)bf16_to_f32(xr[c]) - mu;
        m2 += d * d;
    }
    float var = (float)(m2 / (double)cols);
    *mean = (float)mu;
    *rstd = 1.0f / sqrtf(var + (float)eps);
}

static void row_moments_f32(const float *xr, long cols, double eps, float *mean, float *rstd) {
    double s = 0.0;
    for (long c = 0; c < cols; ++c) s += (double)xr[c];
    double mu = s / (double)cols;
    double m2 = 0.0;
    for (long c = 0; c < cols; ++c) {
        double d = (double)xr[c] - mu;
        m2 += d * d;
    }
    float var = (float)(m2 / (double)cols);
    *mean = (float)mu;
    *rstd = 1.0f / sqrtf(var + (float)eps);
}

/* x [batch, seq, cols]; scale, shift [batch, cols] */
void oc_adaln_fwd_bf16(const uint16_t *x, const uint16_t *scale, const uint16_t *shift,
                       uint16_t *out, float *mean, float *rstd,
                       long batch, long seq, long cols, double eps) {
    for (long b = 0; b < batch; ++b)
        for (long s = 0; s < seq; ++s) {
            long n = b * seq + s;
            const uint16_t *xr = x + n * cols;
            float mu, r;
            row_moments_bf16(xr, cols, eps, &mu, &r);
            mean[n] = mu;
            rstd[n] = r;
            for (long c = 0; c < cols; ++c) {
                float xn = rnd_bf16((bf16_to_f32(xr[c]) - mu) * r);      /* LayerNorm output */
                float t = rnd_bf16(1.0f + bf16_to_f32(scale[b * cols + c])); /* 1 + scale */
                float p = rnd_bf16(xn * t);                              /* xn * (1+scale) */
                out[n * cols + c] = f32_to_bf16(p + bf16_to_f32(shift[b * cols + c]));
            }
        }
}

void oc_adaln_fwd_f32(const float *x, const float *scale, const float *shift,
                      float *out, float *mean, float *rstd,
                      long batch, long seq, long cols, double eps) {
    for (long b = 0; b < batch; ++b)
        for (long s = 0; s < seq; ++s) {
            long n = b * seq + s;
            const float *xr = x + n * cols;
            float mu, r;
            row_moments_f32(xr, cols, eps, &mu, &r);
            mean[n] = mu;
            rstd[n] = r;
            for (long c = 0; c < cols; ++c) {
                float xn = (xr[c] - mu) * r;
                float t = 1.0f + scale[b * cols + c];
                out[n * cols + c] = xn * t + shift[b * cols + c];
            }
        }
}

/* acc: caller-provided double[2*cols] scratch */
void oc_adaln_bwd_bf16(const uint16_t *x, const uint16_t *scale, const float *mean, const float *rstd,
                       const uint16_t *g, uint16_t *dx, uint16_t *dscale, uint16_t *dshift,
                       double *acc, long batch, long seq, long cols) {
    double *a_scale = acc, *a_shift = acc + cols;
    for (long b = 0; b < batch; ++b) {
        for (long c = 0; c < cols; ++c) a_scale[c] = a_shift[c] = 0.0;
        for (long s = 0; s < seq; ++s) {
            long n = b * seq + s;
            const uint16_t *xr = x + n * cols, *gr = g + n * cols;
            float mu = mean[n], r = rstd[n];
            double s1 = 0.0, s2 = 0.0;
            for (long c = 0; c < cols; ++c) {
                float t = rnd_bf16(1.0f + bf16_to_f32(scale[b * cols + c]));
                float gx = rnd_bf16(bf16_to_f32(gr[c]) * t);            /* grad of xn, bf16 */
                float xh = (bf16_to_f32(xr[c]) - mu) * r;
                s1 += (double)gx;
                s2 += (double)(gx * xh);
            }
            float m1 = (float)(s1 / (double)cols), m2 = (float)(s2 / (double)cols);
            for (long c = 0; c < cols; ++c) {
                float gv = bf16_to_f32(gr[c]);
                float t = rnd_bf16(1.0f + bf16_to_f32(scale[b * cols + c]));
                float gx = rnd_bf16(gv * t);
                float xh = (bf16_to_f32(xr[c]) - mu) * r;
                dx[n * cols + c] = f32_to_bf16(r * (gx - m1 - xh * m2));
                a_shift[c] += (double)gv;
                a_scale[c] += (double)rnd_bf16(gv * rnd_bf16(xh));      /* g*xn in bf16, then summed */
            }
        }
        for (long c = 0; c < cols; ++c) {
            dscale[b * cols + c] = f32_to_bf16((float)a_scale[c]);
            dshift[b * cols + c] = f32_to_bf16((float)a_shift[c]);
        }
    }
}

void oc_adaln_bwd_f32(const float *x, const float *scale, const float *mean, const float *rstd,
                      const float *g, float *dx, float *dscale, float *dshift,
                      double *acc, long batch, long seq, long cols) {
    double *a_scale = acc, *a_shift = acc + cols;
    for (long b = 0; b < batch; ++b) {
        for (long c = 0; c < cols; ++c) a_scale[c] = a_shift[c] = 0.0;
        for (long s = 0; s < seq; ++s) {
            long n = b * seq + s;
            const float *xr = x + n * cols, *gr = g + n * cols;
            float mu = mean[n], r = rstd[n];
            double s1 = 0.0, s2 = 0.0;
            for (long c = 0; c < cols; ++c) {
                float gx = gr[c] * (1.0f + scale[b * cols + c]);
                float xh = (xr[c] - mu) * r;
                s1 += (double)gx;
                s2 += (double)(gx * xh);
            }
            float m1 = (float)(s1 / (double)cols), m2 = (float)(s2 / (double)cols);
            for (long c = 0; c < cols; ++c) {
                float gx = gr[c] * (1.0f + scale[b * cols + c]);
                float xh = (xr[c] - mu) * r;
                dx[n * cols + c] = r * (gx - m1 - xh * m2);
                a_shift[c] += (double)gr[c];
                a_scale[c] += (double)(gr[c] * xh);
            }
        }
        for (long c = 0; c < cols; ++c) {
            dscale[b * cols + c] = (float)a_scale[c];
            dshift[b * cols + c] = (float)a_shift[c];
        }
    }
}

/* ---- gated residual update in front of the AdaLN (teletron/models/dit/dit_layerspec.py:152):
 * h2 = rnd(h + rnd(attn * gate[b])).  The norm of h2 is oc_adaln_fwd_bf16 on the result. */
void oc_gated_residual_fwd_bf16(const uint16_t *h, const uint16_t *attn, const uint16_t *gate,
                                uint16_t *h2, long batch, long seq, long cols) {
    for (long b = 0; b < batch; ++b)
        for (long s = 0; s < seq; ++s)
            for (long c = 0; c < cols; ++c) {
                long i = (b * seq + s) * cols + c;
                float m = rnd_bf16(bf16_to_f32(attn[i]) * bf16_to_f32(gate[b * cols + c]));
                h2[i] = f32_to_bf16(bf16_to_f32(h[i]) + m);
            }
}

/* Backward of the update, given dxn = the norm's dx (bf16, from oc_adaln_bwd_bf16) and dh2 = the
 * gradient reaching h2 from its later uses (may be NULL):
 *   dh = rnd(dxn + dh2); dattn = rnd(dh * gate[b]); dgate[b,c] = sum_s rnd(dh * attn).
 * acc: caller-provided double[cols] scratch. */
void oc_gated_residual_bwd_bf16(const uint16_t *dxn, const uint16_t *dh2, const uint16_t *attn,
                                const uint16_t *gate, uint16_t *dh, uint16_t *dattn, uint16_t *dgate,
                                double *acc, long batch, long seq, long cols) {
    for (long b = 0; b < batch; ++b) {
        for (long c = 0; c < cols; ++c) acc[c] = 0.0;
        for (long s = 0; s < seq; ++s)
            for (long c = 0; c < cols; ++c) {
                long i = (b * seq + s) * cols + c;
                float d = bf16_to_f32(dxn[i]);
                if (dh2) d = rnd_bf16(d + bf16_to_f32(dh2[i]));
                dh[i] = f32_to_bf16(d);
                dattn[i] = f32_to_bf16(d * bf16_to_f32(gate[b * cols + c]));
                acc[c] += (double)rnd_bf16(d * bf16_to_f32(attn[i]));
            }
        for (long c = 0; c < cols; ++c) dgate[b * cols + c] = f32_to_bf16((float)acc[c]);
    }
}
