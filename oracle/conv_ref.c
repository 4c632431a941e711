/*
 * conv_ref.c -- plain-C restatement of the hot-path arithmetic.  TEST INFRASTRUCTURE ONLY:
 * it is the brute-force side of the oracle checks (tests/test_oracle.py) and may be linked or
 * loaded only by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg.
 *
 * All tensors are double, dense channels-last:
 *   activations [N][D][H][W][C]; conv weight [Cout][kd][kh][kw][Cin]; transposed-conv weight
 *   [Cin][kd][kh][kw][Cout]  (the memory order of a channels_last_3d parameter).
 * Index order follows the reference kernels: the output row m unravels as (n, od, oh, ow) with
 * ow fastest, the fused tap index is (kd*KH + kh)*KW + kw, the input coordinate of tap t at
 * output o is o*stride + t*dilation - padding (triton_conv3d/gather_gemm.py:194-260).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

typedef struct {
  int n, cin, id, ih, iw, cout, kd, kh, kw, sd, sh, sw, pd, ph, pw, dd, dh, dw;
} ref_conv_desc;

static int out_extent(int in, int k, int s, int p, int d) { return (in + 2 * p - d * (k - 1) - 1) / s + 1; }

#define X_AT(n_, d_, h_, w_, c_) x[((((size_t)(n_) * p->id + (d_)) * p->ih + (h_)) * p->iw + (w_)) * p->cin + (c_)]
#define Y_AT(n_, d_, h_, w_, c_) y[((((size_t)(n_) * od + (d_)) * oh + (h_)) * ow + (w_)) * p->cout + (c_)]
#define W_AT(co_, a_, b_, c_, ci_) w[((((size_t)(co_) * p->kd + (a_)) * p->kh + (b_)) * p->kw + (c_)) * p->cin + (ci_)]

/* y = conv3d(x, w) + bias   (triton_conv3d/gather_gemm.py:187-341) */
void ref_conv3d_fwd(const ref_conv_desc* p, const double* x, const double* w, const double* bias, double* y) {
  const int od = out_extent(p->id, p->kd, p->sd, p->pd, p->dd), oh = out_extent(p->ih, p->kh, p->sh, p->ph, p->dh),
            ow = out_extent(p->iw, p->kw, p->sw, p->pw, p->dw);
  for (int n = 0; n < p->n; ++n)
    for (int zd = 0; zd < od; ++zd)
      for (int zh = 0; zh < oh; ++zh)
        for (int zw = 0; zw < ow; ++zw)
          for (int co = 0; co < p->cout; ++co) {
            double acc = 0.0;
            for (int a = 0; a < p->kd; ++a) {
              const int id = zd * p->sd + a * p->dd - p->pd;
              if (id < 0 || id >= p->id) continue;
              for (int b = 0; b < p->kh; ++b) {
                const int ih = zh * p->sh + b * p->dh - p->ph;
                if (ih < 0 || ih >= p->ih) continue;
                for (int c = 0; c < p->kw; ++c) {
                  const int iw = zw * p->sw + c * p->dw - p->pw;
                  if (iw < 0 || iw >= p->iw) continue;
                  for (int ci = 0; ci < p->cin; ++ci) acc += X_AT(n, id, ih, iw, ci) * W_AT(co, a, b, c, ci);
                }
              }
            }
            Y_AT(n, zd, zh, zw, co) = acc + (bias ? bias[co] : 0.0);
          }
}

/* gx[i] += gy[o] * w for every (o, tap) with o*s + tap*dil - p == i: the scatter form, so that
 * it is an independent statement of what the gather form in bwd_data.py:1-58 must equal. */
void ref_conv3d_dgrad(const ref_conv_desc* p, const double* y /* gy */, const double* w, double* gx) {
  const int od = out_extent(p->id, p->kd, p->sd, p->pd, p->dd), oh = out_extent(p->ih, p->kh, p->sh, p->ph, p->dh),
            ow = out_extent(p->iw, p->kw, p->sw, p->pw, p->dw);
  const size_t nx = (size_t)p->n * p->id * p->ih * p->iw * p->cin;
  for (size_t i = 0; i < nx; ++i) gx[i] = 0.0;
  for (int n = 0; n < p->n; ++n)
    for (int zd = 0; zd < od; ++zd)
      for (int zh = 0; zh < oh; ++zh)
        for (int zw = 0; zw < ow; ++zw)
          for (int a = 0; a < p->kd; ++a) {
            const int id = zd * p->sd + a * p->dd - p->pd;
            if (id < 0 || id >= p->id) continue;
            for (int b = 0; b < p->kh; ++b) {
              const int ih = zh * p->sh + b * p->dh - p->ph;
              if (ih < 0 || ih >= p->ih) continue;
              for (int c = 0; c < p->kw; ++c) {
                const int iw = zw * p->sw + c * p->dw - p->pw;
                if (iw < 0 || iw >= p->iw) continue;
                for (int co = 0; co < p->cout; ++co) {
                  const double g = Y_AT(n, zd, zh, zw, co);
                  for (int ci = 0; ci < p->cin; ++ci)
                    gx[((((size_t)n * p->id + id) * p->ih + ih) * p->iw + iw) * p->cin + ci] += g * W_AT(co, a, b, c, ci);
                }
              }
            }
          }
}

/* gw[co][tap][ci] = sum_v gy[v][co] * x[v (+) tap][ci]   (triton_conv3d/reduce_gemm.py:232-393) */
void ref_conv3d_wgrad(const ref_conv_desc* p, const double* x, const double* y /* gy */, double* gw) {
  const int od = out_extent(p->id, p->kd, p->sd, p->pd, p->dd), oh = out_extent(p->ih, p->kh, p->sh, p->ph, p->dh),
            ow = out_extent(p->iw, p->kw, p->sw, p->pw, p->dw);
  for (int co = 0; co < p->cout; ++co)
    for (int a = 0; a < p->kd; ++a)
      for (int b = 0; b < p->kh; ++b)
        for (int c = 0; c < p->kw; ++c)
          for (int ci = 0; ci < p->cin; ++ci) {
            double acc = 0.0;
            for (int n = 0; n < p->n; ++n)
              for (int zd = 0; zd < od; ++zd) {
                const int id = zd * p->sd + a * p->dd - p->pd;
                if (id < 0 || id >= p->id) continue;
                for (int zh = 0; zh < oh; ++zh) {
                  const int ih = zh * p->sh + b * p->dh - p->ph;
                  if (ih < 0 || ih >= p->ih) continue;
                  for (int zw = 0; zw < ow; ++zw) {
                    const int iw = zw * p->sw + c * p->dw - p->pw;
                    if (iw < 0 || iw >= p->iw) continue;
                    acc += Y_AT(n, zd, zh, zw, co) * X_AT(n, id, ih, iw, ci);
                  }
                }
              }
            gw[((((size_t)co * p->kd + a) * p->kh + b) * p->kw + c) * p->cin + ci] = acc;
          }
}

/* kernel == stride transposed convolution  (triton_conv3d/transposed.py:205-319)
 * y[n][d*kd+a][h*kh+b][w*kw+c][oc] = bias[oc] + sum_ic x[n][d][h][w][ic] * wt[ic][a][b][c][oc] */
void ref_convT3d_fwd(int n_, int cin, int id, int ih, int iw, int cout, int kd, int kh, int kw, const double* x,
                     const double* wt, const double* bias, double* y) {
  const int od = id * kd, oh = ih * kh, ow = iw * kw;
  for (int n = 0; n < n_; ++n)
    for (int d = 0; d < id; ++d)
      for (int h = 0; h < ih; ++h)
        for (int w = 0; w < iw; ++w)
          for (int a = 0; a < kd; ++a)
            for (int b = 0; b < kh; ++b)
              for (int c = 0; c < kw; ++c)
                for (int oc = 0; oc < cout; ++oc) {
                  double acc = bias ? bias[oc] : 0.0;
                  for (int ic = 0; ic < cin; ++ic)
                    acc += x[((((size_t)n * id + d) * ih + h) * iw + w) * cin + ic] *
                           wt[((((size_t)ic * kd + a) * kh + b) * kw + c) * cout + oc];
                  y[((((size_t)n * od + d * kd + a) * oh + h * kh + b) * ow + w * kw + c) * cout + oc] = acc;
                }
}

/* GroupNorm forward over (N, S, C): two-pass mean/variance per (n, group)
 * (ScaFFold/unet/triton_group_norm.py:609-810); relu spelled y <= 0 ? 0 : y. */
void ref_groupnorm_fwd(int n_, long s_, int c_, int groups, double eps, int relu, const double* x, const double* gamma,
                       const double* beta, double* y, double* mean, double* rstd) {
  const int cg = c_ / groups;
  for (int n = 0; n < n_; ++n)
    for (int g = 0; g < groups; ++g) {
      double sum = 0.0;
      for (long s = 0; s < s_; ++s)
        for (int c = g * cg; c < (g + 1) * cg; ++c) sum += x[((size_t)n * s_ + s) * c_ + c];
      const double m = (double)s_ * cg, mu = sum / m;
      double sq = 0.0;
      for (long s = 0; s < s_; ++s)
        for (int c = g * cg; c < (g + 1) * cg; ++c) {
          const double d = x[((size_t)n * s_ + s) * c_ + c] - mu;
          sq += d * d;
        }
      const double r = 1.0 / sqrt(sq / m + eps);
      mean[n * groups + g] = mu;
      rstd[n * groups + g] = r;
      for (long s = 0; s < s_; ++s)
        for (int c = g * cg; c < (g + 1) * cg; ++c) {
          const size_t i = ((size_t)n * s_ + s) * c_ + c;
          double v = (x[i] - mu) * r * (gamma ? gamma[c] : 1.0) + (beta ? beta[c] : 0.0);
          if (relu && v <= 0.0) v = 0.0;
          y[i] = v;
        }
    }
}

/* GroupNorm backward (triton_group_norm.py:813-1043):
 * dx = rstd * (g*gamma - mean_g(g*gamma) - xhat * mean_g(g*gamma*xhat)), dgamma = sum g*xhat, dbeta = sum g,
 * with g = dy gated by the sign of the recomputed pre-activation when relu. */
void ref_groupnorm_bwd(int n_, long s_, int c_, int groups, int relu, const double* dy, const double* x, const double* gamma,
                       const double* beta, const double* mean, const double* rstd, double* dx, double* dgamma, double* dbeta) {
  const int cg = c_ / groups;
  for (int c = 0; c < c_; ++c) { dgamma[c] = 0.0; dbeta[c] = 0.0; }
  for (int n = 0; n < n_; ++n)
    for (int g = 0; g < groups; ++g) {
      const double mu = mean[n * groups + g], r = rstd[n * groups + g], m = (double)s_ * cg;
      double a = 0.0, b = 0.0;
      for (long s = 0; s < s_; ++s)
        for (int c = g * cg; c < (g + 1) * cg; ++c) {
          const size_t i = ((size_t)n * s_ + s) * c_ + c;
          const double w = gamma ? gamma[c] : 1.0, xh = (x[i] - mu) * r;
          double d = dy[i];
          if (relu && xh * w + (beta ? beta[c] : 0.0) <= 0.0) d = 0.0;
          a += d * w;
          b += d * w * xh;
          dgamma[c] += d * xh;
          dbeta[c] += d;
        }
      a /= m;
      b /= m;
      for (long s = 0; s < s_; ++s)
        for (int c = g * cg; c < (g + 1) * cg; ++c) {
          const size_t i = ((size_t)n * s_ + s) * c_ + c;
          const double w = gamma ? gamma[c] : 1.0, xh = (x[i] - mu) * r;
          double d = dy[i];
          if (relu && xh * w + (beta ? beta[c] : 0.0) <= 0.0) d = 0.0;
          dx[i] = r * (d * w - a - xh * b);
        }
    }
}
