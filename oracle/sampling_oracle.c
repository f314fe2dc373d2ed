/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the DCNv4 / flash-deformable-attention
 * sampling operators.  Nothing shipped (the dcnv4_amd package, its C-ABI library)
 * may link, import or call this file; only tests/, the smoke check and the
 * benchmark's CPU-baseline leg do, and only as the checker.
 *
 * Scalar double-precision restatement of the operator arithmetic the reference
 * implements in its CUDA kernels (paths relative to /root/reference):
 *   bilinear gather               DCNv4_op/src/cuda/common.h:41-98
 *   bilinear scatter + partials   DCNv4_op/src/cuda/common.h:100-212
 *   DCNv4 forward                 DCNv4_op/src/cuda/dcnv4_im2col_cuda.cuh:142-244
 *   DCNv4 backward                DCNv4_op/src/cuda/dcnv4_col2im_cuda.cuh:196-366
 *   flash attn forward            DCNv4_op/src/cuda/flash_deform_im2col_cuda.cuh:129-209
 *   flash attn backward           DCNv4_op/src/cuda/flash_deform_col2im_cuda.cuh:171-318
 *   output extents                DCNv4_op/src/cuda/dcnv4_cuda.cu:48-52
 *
 * Parity pins (tests/test_oracle_*.py): agreement in fp64 with an independent
 * torch grid_sample formulation (oracle/torch_core.py), closed forms (zero
 * offsets + unit mask == 3x3 zero-padded box sum; integer offsets == shifted
 * copy; L=K=1 attention == one bilinear tap), linearity, exact zeros for
 * out-of-range taps, and central finite differences of the forward for every
 * gradient.  One deliberate deviation from the reference kernel: an
 * out-of-range attention tap contributes 0 to the softmax Jacobian (the
 * reference reads an unwritten shared-memory slot there,
 * flash_deform_col2im_cuda.cuh:272-293).
 *
 * Coordinate precision: the reference forms every sampling coordinate in its opmath type, which
 * is fp32 for fp32/fp16/bf16 tensors (dcnv4_im2col_cuda.cuh:203-224, flash_deform_im2col_cuda.cuh:
 * 184-189).  With coord32 != 0 the oracle rounds exactly those operations to fp32, in source
 * order and without fused multiply-add, and does everything downstream (weights, sums) in
 * double; with coord32 == 0 coordinates are double too (the mathematical ideal the pins use).
 *
 * All tensors are dense row-major double arrays in the operator's own layouts.
 * Loops over the batch run under OpenMP; every image is independent, so the
 * gradient scatter needs no atomics.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
  int y0, x0;        /* top-left corner (may be -1)                       */
  double wt[4];      /* corner weights: (y0,x0) (y0,x1) (y1,x0) (y1,x1)   */
  double dwy[4];     /* d wt / d y                                        */
  double dwx[4];     /* d wt / d x                                        */
  int ok[4];         /* corner lies inside the image                      */
} tap_t;

/* common.h:48-58 (weights) and :74-90 (per-corner bounds). */
static int make_tap(double y, double x, int H, int W, tap_t *t) {
  if (!(y > -1.0 && x > -1.0 && y < (double)H && x < (double)W)) return 0;
  const int y0 = (int)floor(y), x0 = (int)floor(x);
  const double ly = y - y0, lx = x - x0, hy = 1.0 - ly, hx = 1.0 - lx;
  t->y0 = y0; t->x0 = x0;
  t->wt[0] = hy * hx; t->wt[1] = hy * lx; t->wt[2] = ly * hx; t->wt[3] = ly * lx;
  t->dwy[0] = -hx; t->dwy[1] = -lx; t->dwy[2] = hx; t->dwy[3] = lx;
  t->dwx[0] = -hy; t->dwx[1] = hy; t->dwx[2] = -ly; t->dwx[3] = ly;
  t->ok[0] = (y0 >= 0 && x0 >= 0);
  t->ok[1] = (y0 >= 0 && x0 + 1 < W);
  t->ok[2] = (y0 + 1 < H && x0 >= 0);
  t->ok[3] = (y0 + 1 < H && x0 + 1 < W);
  return 1;
}

static inline int64_t corner_pixel(const tap_t *t, int c, int W) {
  return (int64_t)(t->y0 + (c >> 1)) * W + (t->x0 + (c & 1));
}

static void softmax_inplace(double *p, int n) {
  double mx = p[0], s = 0.0;
  for (int i = 1; i < n; ++i) mx = p[i] > mx ? p[i] : mx;
  for (int i = 0; i < n; ++i) { p[i] = exp(p[i] - mx); s += p[i]; }
  for (int i = 0; i < n; ++i) p[i] /= s;
}

int oracle_out_extent(int in, int pad, int dil, int k, int stride) {
  return (in + 2 * pad - (dil * (k - 1) + 1)) / stride + 1;   /* dcnv4_cuda.cu:48-52 */
}

/* ------------------------------------------------------------------ DCNv4 */

typedef struct {
  int B, H, W, G, D, kh, kw, sh, sw, ph, pw, dh, dw, remove_center, softmax, P_pad;
  double offset_scale;
  int coord32;
} dcn_args_t;

/* Sampling position of kernel tap (i = x index, j = y index) for output pixel
 * (ho, wo): dcnv4_im2col_cuda.cuh:203-224. */
static inline void dcn_position(const dcn_args_t *a, int ho, int wo, int i, int j,
                                double off_x, double off_y, double *y, double *x) {
  const int half_w = (a->dw * (a->kw - 1)) >> 1, half_h = (a->dh * (a->kh - 1)) >> 1;
  const int p0_w = half_w - a->pw + wo * a->sw, p0_h = half_h - a->ph + ho * a->sh;
  if (a->coord32) {       /* every operation rounded to fp32; built with -ffp-contract=off */
    const float sc = (float)a->offset_scale;
    const float bx = (float)p0_w - (float)half_w * sc, by = (float)p0_h - (float)half_h * sc;
    const float tx = ((float)(i * a->dw) + (float)off_x) * sc, ty = ((float)(j * a->dh) + (float)off_y) * sc;
    *x = (double)(bx + tx);
    *y = (double)(by + ty);
    return;
  }
  *x = (p0_w - half_w * a->offset_scale) + (i * a->dw + off_x) * a->offset_scale;
  *y = (p0_h - half_h * a->offset_scale) + (j * a->dh + off_y) * a->offset_scale;
}

/* Attention tap position: loc * extent - 0.5 (flash_deform_im2col_cuda.cuh:188-189). */
static inline double fda_position(double loc, int extent, int coord32) {
  if (coord32) {
    const float prod = (float)loc * (float)extent;
    return (double)(prod - 0.5f);
  }
  return loc * extent - 0.5;
}

void oracle_dcnv4_forward(const double *value, const double *offset_mask, double *out,
                          int B, int H, int W, int G, int D, int kh, int kw, int sh, int sw,
                          int ph, int pw, int dh, int dw, double offset_scale,
                          int remove_center, int softmax, int P_pad, int coord32) {
  dcn_args_t a = {B, H, W, G, D, kh, kw, sh, sw, ph, pw, dh, dw, remove_center, softmax, P_pad,
                  offset_scale, coord32};
  const int Ho = oracle_out_extent(H, ph, dh, kh, sh), Wo = oracle_out_extent(W, pw, dw, kw, sw);
  const int Kp = kh * kw - (remove_center ? 1 : 0), C = G * D;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < B; ++b)
    for (int ho = 0; ho < Ho; ++ho) {
      double m[64];
      for (int wo = 0; wo < Wo; ++wo)
        for (int g = 0; g < G; ++g) {
          const int64_t q = ((int64_t)b * Ho + ho) * Wo + wo;
          const double *om = offset_mask + q * P_pad + (int64_t)g * 3 * Kp;
          double *o = out + q * C + (int64_t)g * D;
          for (int k = 0; k < Kp; ++k) m[k] = om[2 * Kp + k];
          if (softmax) softmax_inplace(m, Kp);
          for (int c = 0; c < D; ++c) o[c] = 0.0;
          int k = 0;
          for (int i = 0; i < kw; ++i)
            for (int j = 0; j < kh; ++j) {
              if (remove_center && i == kw / 2 && j == kh / 2) continue;
              double y, x; tap_t t;
              dcn_position(&a, ho, wo, i, j, om[2 * k], om[2 * k + 1], &y, &x);
              if (make_tap(y, x, H, W, &t))
                for (int cn = 0; cn < 4; ++cn) {
                  if (!t.ok[cn]) continue;
                  const double *v = value + ((int64_t)b * H * W + corner_pixel(&t, cn, W)) * C + g * D;
                  const double s = m[k] * t.wt[cn];
                  for (int c = 0; c < D; ++c) o[c] += s * v[c];
                }
              ++k;
            }
        }
    }
}

void oracle_dcnv4_backward(const double *value, const double *offset_mask, const double *grad_out,
                           double *grad_value, double *grad_om,
                           int B, int H, int W, int G, int D, int kh, int kw, int sh, int sw,
                           int ph, int pw, int dh, int dw, double offset_scale,
                           int remove_center, int softmax, int P_pad, int coord32) {
  dcn_args_t a = {B, H, W, G, D, kh, kw, sh, sw, ph, pw, dh, dw, remove_center, softmax, P_pad,
                  offset_scale, coord32};
  const int Ho = oracle_out_extent(H, ph, dh, kh, sh), Wo = oracle_out_extent(W, pw, dw, kw, sw);
  const int Kp = kh * kw - (remove_center ? 1 : 0), C = G * D;
  memset(grad_value, 0, sizeof(double) * (size_t)B * H * W * C);
  memset(grad_om, 0, sizeof(double) * (size_t)B * Ho * Wo * P_pad);
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    double m[64], gm[64];
    for (int ho = 0; ho < Ho; ++ho)
      for (int wo = 0; wo < Wo; ++wo)
        for (int g = 0; g < G; ++g) {
          const int64_t q = ((int64_t)b * Ho + ho) * Wo + wo;
          const double *om = offset_mask + q * P_pad + (int64_t)g * 3 * Kp;
          double *gom = grad_om + q * P_pad + (int64_t)g * 3 * Kp;
          const double *go = grad_out + q * C + (int64_t)g * D;
          for (int k = 0; k < Kp; ++k) m[k] = om[2 * Kp + k];
          if (softmax) softmax_inplace(m, Kp);
          int k = 0;
          for (int i = 0; i < kw; ++i)
            for (int j = 0; j < kh; ++j) {
              if (remove_center && i == kw / 2 && j == kh / 2) continue;
              double y, x, gx = 0.0, gy = 0.0, gz = 0.0; tap_t t;
              dcn_position(&a, ho, wo, i, j, om[2 * k], om[2 * k + 1], &y, &x);
              if (make_tap(y, x, H, W, &t))
                for (int cn = 0; cn < 4; ++cn) {
                  if (!t.ok[cn]) continue;
                  const int64_t e = ((int64_t)b * H * W + corner_pixel(&t, cn, W)) * C + g * D;
                  for (int c = 0; c < D; ++c) {
                    grad_value[e + c] += go[c] * m[k] * t.wt[cn];       /* common.h:153 */
                    gx += t.dwx[cn] * value[e + c] * go[c];             /* common.h:188-201 */
                    gy += t.dwy[cn] * value[e + c] * go[c];
                    gz += t.wt[cn] * value[e + c] * go[c];              /* common.h:203-211 */
                  }
                }
              gom[2 * k] = gx * offset_scale * m[k];
              gom[2 * k + 1] = gy * offset_scale * m[k];
              gm[k] = gz;
              ++k;
            }
          if (softmax) {          /* dcnv4_col2im_cuda.cuh:352-365: p_i (g_i - sum_j p_j g_j) */
            double dot = 0.0;
            for (int kk = 0; kk < Kp; ++kk) dot += m[kk] * gm[kk];
            for (int kk = 0; kk < Kp; ++kk) gom[2 * Kp + kk] = m[kk] * (gm[kk] - dot);
          } else {
            for (int kk = 0; kk < Kp; ++kk) gom[2 * Kp + kk] = gm[kk];
          }
        }
  }
}

/* ------------------------------------------- flash deformable attention */

void oracle_flash_deform_attn_forward(const double *value, const int64_t *shapes,
                                      const int64_t *level_start, const double *sla, double *out,
                                      int B, int N, int G, int D, int L, int K, int Q, int coord32) {
  const int LK = L * K;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < B; ++b)
    for (int q = 0; q < Q; ++q) {
      double p[64];
      for (int g = 0; g < G; ++g) {
        const int64_t row = ((int64_t)b * Q + q) * G + g;
        const double *s = sla + row * 3 * LK;           /* flash_deform_im2col_cuda.cuh:145-149 */
        double *o = out + row * D;
        for (int t = 0; t < LK; ++t) p[t] = s[2 * LK + t];
        softmax_inplace(p, LK);
        for (int c = 0; c < D; ++c) o[c] = 0.0;
        for (int l = 0; l < L; ++l) {
          const int Hl = (int)shapes[2 * l], Wl = (int)shapes[2 * l + 1];
          for (int k = 0; k < K; ++k) {
            const int t = l * K + k; tap_t tp;
            const double x = fda_position(s[2 * t], Wl, coord32), y = fda_position(s[2 * t + 1], Hl, coord32);
            if (!make_tap(y, x, Hl, Wl, &tp)) continue;
            for (int cn = 0; cn < 4; ++cn) {
              if (!tp.ok[cn]) continue;
              const double *v = value + (((int64_t)b * N + level_start[l] + corner_pixel(&tp, cn, Wl)) * G + g) * D;
              const double w = p[t] * tp.wt[cn];
              for (int c = 0; c < D; ++c) o[c] += w * v[c];
            }
          }
        }
      }
    }
}

void oracle_flash_deform_attn_backward(const double *value, const int64_t *shapes,
                                       const int64_t *level_start, const double *sla,
                                       const double *grad_out, double *grad_value, double *grad_sla,
                                       int B, int N, int G, int D, int L, int K, int Q, int coord32) {
  const int LK = L * K;
  memset(grad_value, 0, sizeof(double) * (size_t)B * N * G * D);
  memset(grad_sla, 0, sizeof(double) * (size_t)B * Q * G * 3 * LK);
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    double p[64], a[64];
    for (int q = 0; q < Q; ++q)
      for (int g = 0; g < G; ++g) {
        const int64_t row = ((int64_t)b * Q + q) * G + g;
        const double *s = sla + row * 3 * LK;
        double *gs = grad_sla + row * 3 * LK;
        const double *go = grad_out + row * D;
        for (int t = 0; t < LK; ++t) p[t] = s[2 * LK + t];
        softmax_inplace(p, LK);
        for (int l = 0; l < L; ++l) {
          const int Hl = (int)shapes[2 * l], Wl = (int)shapes[2 * l + 1];
          for (int k = 0; k < K; ++k) {
            const int t = l * K + k; tap_t tp;
            const double x = fda_position(s[2 * t], Wl, coord32), y = fda_position(s[2 * t + 1], Hl, coord32);
            double gx = 0.0, gy = 0.0, gz = 0.0;
            if (make_tap(y, x, Hl, Wl, &tp))
              for (int cn = 0; cn < 4; ++cn) {
                if (!tp.ok[cn]) continue;
                const int64_t e = (((int64_t)b * N + level_start[l] + corner_pixel(&tp, cn, Wl)) * G + g) * D;
                for (int c = 0; c < D; ++c) {
                  grad_value[e + c] += go[c] * p[t] * tp.wt[cn];
                  gx += tp.dwx[cn] * value[e + c] * go[c];
                  gy += tp.dwy[cn] * value[e + c] * go[c];
                  gz += tp.wt[cn] * value[e + c] * go[c];
                }
              }
            gs[2 * t] = gx * Wl * p[t];          /* flash_deform_col2im_cuda.cuh:273-276 */
            gs[2 * t + 1] = gy * Hl * p[t];
            a[t] = gz;
          }
        }
        double dot = 0.0;                          /* softmax Jacobian, :301-316 in closed form */
        for (int t = 0; t < LK; ++t) dot += p[t] * a[t];
        for (int t = 0; t < LK; ++t) gs[2 * LK + t] = p[t] * (a[t] - dot);
      }
  }
}
