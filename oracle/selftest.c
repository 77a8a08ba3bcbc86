/* TEST INFRASTRUCTURE ONLY -- drives every oracle function once on small, awkward shapes
 * (ragged planes, stride, dilation, rotation groups, samples far outside the scope and the
 * image) with exactly-sized heap buffers, so that a build with AddressSanitizer and
 * UndefinedBehaviorSanitizer (`make -C oracle sanitize`) catches an out-of-bounds index or an
 * overflowing int in the restatement.  Checks one closed form on the way: scope == kernel with
 * zero offsets is a plain depthwise convolution. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include "dk_oracle.h"

static unsigned long long rng = 88172645463325252ull;
static double uni(void) { /* xorshift, uniform in [-1, 1) */
  rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17;
  return (double)(rng >> 11) / 9007199254740992.0 * 2.0 - 1.0;
}
static float *fill_f(long n, double scale) {
  float *p = (float *)malloc((size_t)(n > 0 ? n : 1) * sizeof(float));
  for (long i = 0; i < n; ++i) p[i] = (float)(uni() * scale);
  return p;
}
static double *fill_d(long n, double scale) {
  double *p = (double *)malloc((size_t)(n > 0 ? n : 1) * sizeof(double));
  for (long i = 0; i < n; ++i) p[i] = uni() * scale;
  return p;
}
static int out_size(int n, int k, int s, int p, int d) { return (n + 2 * p - (d * (k - 1) + 1)) / s + 1; }

#define RUN_CONV(REAL, S, FILL, rot_scale, off_scale)                                                   \
  do {                                                                                                    \
    const long nx = (long)a.batch * a.channel * a.in_h * a.in_w, ny = (long)a.batch * a.channel * a.out_h * a.out_w; \
    const long nr = (long)a.batch * a.groups * a.k_h * a.k_w * 2 * a.out_h * a.out_w;                    \
    const long no = (long)a.batch * a.k_h * a.k_w * 2 * a.out_h * a.out_w;                               \
    const long nw = (long)a.channel * a.scope_h * a.scope_w;                                             \
    REAL *x = FILL(nx, 1.0), *rot = FILL(nr, rot_scale), *off = FILL(no, off_scale), *w = FILL(nw, 0.5);  \
    REAL *go = FILL(ny, 1.0), *y = FILL(ny, 0), *gx = FILL(nx, 0), *gw = FILL(nw, 0), *gr = FILL(nr, 0), *gf = FILL(no, 0); \
    dko_sample_depthwise_forward##S(&a, x, rot, w, y);                                                   \
    dko_sample_depthwise_backward_data##S(&a, go, rot, w, gx);                                           \
    dko_sample_depthwise_backward_filter##S(&a, go, x, rot, gw);                                         \
    dko_sample_depthwise_backward_rotation##S(&a, go, x, rot, w, gr);                                    \
    dko_deformable_sample_depthwise_forward##S(&a, x, off, rot, w, y);                                   \
    dko_deformable_sample_depthwise_backward_data##S(&a, go, off, rot, w, gx);                           \
    dko_deformable_sample_depthwise_backward_filter##S(&a, go, x, off, rot, gw);                         \
    dko_deformable_sample_depthwise_backward_offset##S(&a, go, x, off, rot, w, gf);                      \
    dko_deformable_sample_depthwise_backward_rotation##S(&a, go, x, off, rot, w, gr);                    \
    for (long i = 0; i < ny; ++i) if (!isfinite((double)y[i])) { printf("non-finite output\n"); return 1; } \
    free(x); free(rot); free(off); free(w); free(go); free(y); free(gx); free(gw); free(gr); free(gf);   \
  } while (0)

static int conv_closed_form(void) {
  /* scope == kernel, zero offsets: out = depthwise 3x3 convolution, zero padded */
  dko_args a = {1, 2, 5, 4, 3, 3, 1, 1, 1, 1, 1, 1, 5, 4, 3, 3, 1};
  double *x = fill_d(2 * 20, 1.0), *w = fill_d(18, 1.0), *rot = (double *)calloc(18 * 20, sizeof(double));
  double *y = fill_d(40, 0);
  dko_sample_depthwise_forward_f64(&a, x, rot, w, y);
  double worst = 0;
  for (int c = 0; c < 2; ++c)
    for (int h = 0; h < 5; ++h)
      for (int v = 0; v < 4; ++v) {
        double s = 0;
        for (int i = 0; i < 3; ++i)
          for (int j = 0; j < 3; ++j) {
            const int ih = h - 1 + i, iw = v - 1 + j;
            if (ih >= 0 && ih < 5 && iw >= 0 && iw < 4) s += x[c * 20 + ih * 4 + iw] * w[c * 9 + i * 3 + j];
          }
        worst = fmax(worst, fabs(s - y[c * 20 + h * 4 + v]));
      }
  free(x); free(w); free(rot); free(y);
  if (worst > 1e-12) { printf("depthwise closed form off by %g\n", worst); return 1; }
  return 0;
}

int main(void) {
  const int shapes[][13] = {
      /* batch channel in_h in_w k_h k_w stride_h stride_w pad_h pad_w dil_h dil_w groups */
      {2, 6, 9, 7, 3, 3, 1, 1, 1, 1, 1, 1, 1},
      {1, 6, 10, 11, 3, 3, 2, 2, 1, 1, 1, 1, 3},
      {2, 4, 8, 9, 5, 3, 1, 2, 2, 0, 1, 1, 2},
      {1, 3, 12, 5, 3, 3, 1, 1, 2, 2, 2, 2, 1},
      {1, 2, 3, 3, 1, 1, 1, 1, 0, 0, 1, 1, 1},
  };
  const int scopes[][2] = {{4, 4}, {5, 5}, {7, 4}, {3, 3}, {2, 2}};
  for (int i = 0; i < 5; ++i) {
    const int *s = shapes[i];
    dko_args a = {s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7], s[8], s[9], s[10], s[11],
                  out_size(s[2], s[4], s[6], s[8], s[10]), out_size(s[3], s[5], s[7], s[9], s[11]),
                  scopes[i][0], scopes[i][1], s[12]};
    RUN_CONV(float, _f32, fill_f, 1.0, 2.0);
    RUN_CONV(double, _f64, fill_d, 6.0, 30.0); /* most samples outside the scope / the image */
  }
  /* N-d sampler, 1 to 4 dimensions, coordinates reaching beyond both ends */
  for (int dims = 1; dims <= 4; ++dims) {
    const int ext[4] = {5, 3, 4, 2};
    long prod = 1;
    double shape_d[4];
    float shape_f[4];
    for (int d = 0; d < dims; ++d) { prod *= ext[d]; shape_d[d] = ext[d]; shape_f[d] = (float)ext[d]; }
    const int B = 37, C = 3;
    double *data = fill_d(C * prod, 1.0), *coord = fill_d((long)B * dims, 7.0), *go = fill_d((long)B * C, 1.0);
    double *out = fill_d((long)B * C, 0), *gd = fill_d(C * prod, 0), *gc = fill_d((long)B * dims * C, 0);
    dko_nd_linear_sample_forward_f64(B, C, dims, prod, data, shape_d, coord, out);
    dko_nd_linear_sample_backward_data_f64(B, C, dims, prod, go, shape_d, coord, gd);
    dko_nd_linear_sample_backward_coord_f64(B, C, dims, prod, go, data, shape_d, coord, gc);
    free(data); free(coord); free(go); free(out); free(gd); free(gc);
    float *dataf = fill_f(C * prod, 1.0), *coordf = fill_f((long)B * dims, 7.0), *gof = fill_f((long)B * C, 1.0);
    float *outf = fill_f((long)B * C, 0), *gdf = fill_f(C * prod, 0), *gcf = fill_f((long)B * dims * C, 0);
    dko_nd_linear_sample_forward_f32(B, C, dims, prod, dataf, shape_f, coordf, outf);
    dko_nd_linear_sample_backward_data_f32(B, C, dims, prod, gof, shape_f, coordf, gdf);
    dko_nd_linear_sample_backward_coord_f32(B, C, dims, prod, gof, dataf, shape_f, coordf, gcf);
    free(dataf); free(coordf); free(gof); free(outf); free(gdf); free(gcf);
  }
  if (conv_closed_form()) return 1;
  printf("oracle selftest ok\n");
  return 0;
}
