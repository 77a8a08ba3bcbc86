/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference arithmetic.
 *
 * This file is included twice by dk_oracle.c, once with REAL=float (suffix
 * _f32) and once with REAL=double (suffix _f64).  Every function follows one
 * CUDA kernel or device helper of the reference and cites it as
 *   K.cu  = deformable_kernels/ops/deform_kernel/csrc/filter_sample_depthwise_cuda_kernel.cu
 *   ND.cu = deformable_kernels/ops/deform_kernel/csrc/nd_linear_sample_cuda_kernel.cu
 * Arithmetic is done in REAL in the same operation order as the reference's
 * scalar_t code (including the promotion of the centring term to double);
 * the reference's global atomicAdd scatters become plain serial sums in
 * thread-id order, which is the one place where order is ours to choose.
 *
 * Nothing that ships (the HIP library, the Python package) may call this.
 */

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUFFIX)

/* ---- scope-tile helpers ------------------------------------------------ */

/* K.cu:51-83 planar_bilinear: zero-outside bilinear read of an
 * height x width tile at real (h, w). */
static REAL FN(planar_bilinear)(const REAL *data, int height, int width, REAL h, REAL w) {
  if (h > -1 && w > -1 && h < height && w < width) {
    int h_low = (int)floor((double)h);
    int w_low = (int)floor((double)w);
    int h_high = h_low + 1;
    int w_high = w_low + 1;
    const REAL lh = h - h_low;
    const REAL lw = w - w_low;
    const REAL hh = 1 - lh, hw = 1 - lw;
    REAL val = 0;
    if (h_low >= 0 && w_low >= 0) val += hh * hw * data[h_low * width + w_low];
    if (h_low >= 0 && w_high <= width - 1) val += hh * lw * data[h_low * width + w_high];
    if (h_high <= height - 1 && w_low >= 0) val += lh * hw * data[h_high * width + w_low];
    if (h_high <= height - 1 && w_high <= width - 1) val += lh * lw * data[h_high * width + w_high];
    return val;
  }
  return 0;
}

/* K.cu:85-114 planar_bilinear_backward_data: scatter coef * partial_sum onto
 * the (at most) four tile cells; the reference uses atomicAdd. */
static void FN(planar_bilinear_backward_data)(REAL partial_sum, int height, int width, REAL h,
                                              REAL w, REAL *filter_gradient) {
  if (h > -1 && w > -1 && h < height && w < width) {
    int h_low = (int)floor((double)h);
    int w_low = (int)floor((double)w);
    int h_high = h_low + 1;
    int w_high = w_low + 1;
    const REAL lh = h - h_low;
    const REAL lw = w - w_low;
    const REAL hh = 1 - lh, hw = 1 - lw;
    if (h_low >= 0 && w_low >= 0) filter_gradient[h_low * width + w_low] += hh * hw * partial_sum;
    if (h_low >= 0 && w_high <= width - 1)
      filter_gradient[h_low * width + w_high] += hh * lw * partial_sum;
    if (h_high <= height - 1 && w_low >= 0)
      filter_gradient[h_high * width + w_low] += lh * hw * partial_sum;
    if (h_high <= height - 1 && w_high <= width - 1)
      filter_gradient[h_high * width + w_high] += lh * lw * partial_sum;
  }
}

/* K.cu:116-163 planar_bilinear_backward_coord: partial_sum * dB/dh (bp_dir 0)
 * or dB/dw (bp_dir 1), floor-based piecewise-linear derivative. */
static REAL FN(planar_bilinear_backward_coord)(REAL partial_sum, const REAL *filter, int height,
                                               int width, REAL h, REAL w, int bp_dir) {
  if (h > -1 && w > -1 && h < height && w < width) {
    int h_low = (int)floor((double)h);
    int w_low = (int)floor((double)w);
    int h_high = h_low + 1;
    int w_high = w_low + 1;
    const REAL lh = h - h_low;
    const REAL lw = w - w_low;
    const REAL hh = 1 - lh, hw = 1 - lw;
    if (bp_dir == 0) {
      REAL g = 0;
      if (h_low >= 0 && w_low >= 0) g -= hw * partial_sum * filter[h_low * width + w_low];
      if (h_low >= 0 && w_high <= width - 1) g -= lw * partial_sum * filter[h_low * width + w_high];
      if (h_high <= height - 1 && w_low >= 0) g += hw * partial_sum * filter[h_high * width + w_low];
      if (h_high <= height - 1 && w_high <= width - 1)
        g += lw * partial_sum * filter[h_high * width + w_high];
      return g;
    } else {
      REAL g = 0;
      if (h_low >= 0 && w_low >= 0) g -= hh * partial_sum * filter[h_low * width + w_low];
      if (h_low >= 0 && w_high <= width - 1) g += hh * partial_sum * filter[h_low * width + w_high];
      if (h_high <= height - 1 && w_low >= 0) g -= lh * partial_sum * filter[h_high * width + w_low];
      if (h_high <= height - 1 && w_high <= width - 1)
        g += lh * partial_sum * filter[h_high * width + w_high];
      return g;
    }
  }
  return 0;
}

/* ---- image-plane helpers ----------------------------------------------- */

/* K.cu:165-199 deformable_im2col_bilinear: zero-padded bilinear read of an
 * image plane; the caller has already checked -1 < h < height, -1 < w < width. */
static REAL FN(im2col_bilinear)(const REAL *bottom_data, int height, int width, REAL h, REAL w) {
  int h_low = (int)floor((double)h);
  int w_low = (int)floor((double)w);
  int h_high = h_low + 1;
  int w_high = w_low + 1;
  REAL lh = h - h_low;
  REAL lw = w - w_low;
  REAL hh = 1 - lh, hw = 1 - lw;
  REAL v1 = 0, v2 = 0, v3 = 0, v4 = 0;
  if (h_low >= 0 && w_low >= 0) v1 = bottom_data[h_low * width + w_low];
  if (h_low >= 0 && w_high <= width - 1) v2 = bottom_data[h_low * width + w_high];
  if (h_high <= height - 1 && w_low >= 0) v3 = bottom_data[h_high * width + w_low];
  if (h_high <= height - 1 && w_high <= width - 1) v4 = bottom_data[h_high * width + w_high];
  REAL w1 = hh * hw, w2 = hh * lw, w3 = lh * hw, w4 = lh * lw;
  return (w1 * v1 + w2 * v2 + w3 * v3 + w4 * v4);
}

/* K.cu:201-229 deformable_im2col_bilinear_backward: scatter onto the image
 * plane (atomicAdd in the reference). */
static void FN(im2col_bilinear_backward)(REAL partial_sum, REAL h, REAL w, int height, int width,
                                         REAL *data_gradient) {
  int h_low = (int)floor((double)h);
  int w_low = (int)floor((double)w);
  int h_high = h_low + 1;
  int w_high = w_low + 1;
  REAL lh = h - h_low;
  REAL lw = w - w_low;
  REAL hh = 1 - lh, hw = 1 - lw;
  if (h_low >= 0 && w_low >= 0) data_gradient[h_low * width + w_low] += hh * hw * partial_sum;
  if (h_low >= 0 && w_high <= width - 1) data_gradient[h_low * width + w_high] += hh * lw * partial_sum;
  if (h_high <= height - 1 && w_low >= 0) data_gradient[h_high * width + w_low] += lh * hw * partial_sum;
  if (h_high <= height - 1 && w_high <= width - 1)
    data_gradient[h_high * width + w_high] += lh * lw * partial_sum;
}

/* K.cu:231-268 get_coordinate_weight: d(image bilinear)/dh (bp_dir 0) or /dw. */
static REAL FN(coordinate_weight)(REAL ah, REAL aw, int height, int width, const REAL *im,
                                  int bp_dir) {
  int h_low = (int)floor((double)ah);
  int w_low = (int)floor((double)aw);
  int h_high = h_low + 1;
  int w_high = w_low + 1;
  REAL weight = 0;
  if (bp_dir == 0) {
    if (h_low >= 0 && w_low >= 0) weight += -1 * (w_low + 1 - aw) * im[h_low * width + w_low];
    if (h_low >= 0 && w_high <= width - 1) weight += -1 * (aw - w_low) * im[h_low * width + w_high];
    if (h_high <= height - 1 && w_low >= 0) weight += (w_low + 1 - aw) * im[h_high * width + w_low];
    if (h_high <= height - 1 && w_high <= width - 1)
      weight += (aw - w_low) * im[h_high * width + w_high];
  } else {
    if (h_low >= 0 && w_low >= 0) weight += -1 * (h_low + 1 - ah) * im[h_low * width + w_low];
    if (h_low >= 0 && w_high <= width - 1) weight += (h_low + 1 - ah) * im[h_low * width + w_high];
    if (h_high <= height - 1 && w_low >= 0) weight += -1 * (ah - h_low) * im[h_high * width + w_low];
    if (h_high <= height - 1 && w_high <= width - 1)
      weight += (ah - h_low) * im[h_high * width + w_high];
  }
  return weight;
}

/* Scope coordinate of tap f with kernel-space offset r: the reference writes
 * `f + r + (scope - filter) / 2.0` (K.cu:338-341): int + scalar_t in scalar_t,
 * then + double in double, rounded back to scalar_t on assignment. */
static inline REAL FN(scope_coord)(int f, REAL r, int scope, int filter) {
  REAL t = (REAL)f + r;
  return (REAL)((double)t + (scope - filter) / 2.0);
}

/* Offset of the h-component of tap (f_h, f_w) of sampling group g, image b,
 * at output pixel (oh, ow) in rotation[N, G*kh*kw*2, Ho, Wo] (K.cu:307-310,
 * 331-336); the w-component sits out_h*out_w further on. */
static inline long FN(rot_index)(const dko_args *a, int b, int g, int f_h, int f_w, int oh, int ow) {
  return (((long)(b * a->groups + g) * (a->k_h * a->k_w) + (f_h * a->k_w + f_w)) * 2) *
             ((long)a->out_h * a->out_w) +
         ((long)oh * a->out_w + ow);
}

/* ---- local deformable kernel (kernel-space offsets only) ---------------- */

/* K.cu:270-386 SampleDepthwiseConv2dForwardKernel (both branches compute the
 * same sum; taps in the zero padding are skipped). */
void FN(dko_sample_depthwise_forward)(const dko_args *a, const REAL *input, const REAL *rotation,
                                      const REAL *filter, REAL *output) {
  const long plane_o = (long)a->out_h * a->out_w;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < a->batch; ++b)
    for (int c = 0; c < a->channel; ++c) {
      const REAL *in = input + ((long)b * a->channel + c) * a->in_h * a->in_w;
      const REAL *flt = filter + (long)c * a->scope_h * a->scope_w;
      const int g = c % a->groups;
      for (int oh = 0; oh < a->out_h; ++oh)
        for (int ow = 0; ow < a->out_w; ++ow) {
          REAL sum = 0;
          for (int f_h = 0; f_h < a->k_h; ++f_h) {
            const int in_h = oh * a->stride_h - a->pad_h + f_h * a->dil_h;
            for (int f_w = 0; f_w < a->k_w; ++f_w) {
              const int in_w = ow * a->stride_w - a->pad_w + f_w * a->dil_w;
              if (in_h >= 0 && in_h < a->in_h && in_w >= 0 && in_w < a->in_w) {
                const long ro = FN(rot_index)(a, b, g, f_h, f_w, oh, ow);
                const REAL fh = FN(scope_coord)(f_h, rotation[ro], a->scope_h, a->k_h);
                const REAL fw = FN(scope_coord)(f_w, rotation[ro + plane_o], a->scope_w, a->k_w);
                sum += in[in_h * a->in_w + in_w] *
                       FN(planar_bilinear)(flt, a->scope_h, a->scope_w, fh, fw);
              }
            }
          }
          output[((long)b * a->channel + c) * plane_o + (long)oh * a->out_w + ow] = sum;
        }
    }
}

/* K.cu:577-669 SampleDepthwiseConv2dBackwardDataKernel: gather over the
 * outputs that read input element (in_h, in_w). */
void FN(dko_sample_depthwise_backward_data)(const dko_args *a, const REAL *out_grad,
                                            const REAL *rotation, const REAL *filter,
                                            REAL *in_grad) {
  const long plane_o = (long)a->out_h * a->out_w;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < a->batch; ++b)
    for (int c = 0; c < a->channel; ++c) {
      const REAL *og = out_grad + ((long)b * a->channel + c) * plane_o;
      const REAL *flt = filter + (long)c * a->scope_h * a->scope_w;
      const int g = c % a->groups;
      for (int in_h = 0; in_h < a->in_h; ++in_h)
        for (int in_w = 0; in_w < a->in_w; ++in_w) {
          /* K.cu:611-620: C integer division (truncation) as in the reference. */
          int oh_start = (in_h + a->pad_h - (a->k_h - 1) * a->dil_h + a->stride_h - 1) / a->stride_h;
          if (oh_start < 0) oh_start = 0;
          int oh_end = (in_h + a->pad_h) / a->stride_h;
          if (oh_end > a->out_h - 1) oh_end = a->out_h - 1;
          int ow_start = (in_w + a->pad_w - (a->k_w - 1) * a->dil_w + a->stride_w - 1) / a->stride_w;
          if (ow_start < 0) ow_start = 0;
          int ow_end = (in_w + a->pad_w) / a->stride_w;
          if (ow_end > a->out_w - 1) ow_end = a->out_w - 1;
          REAL sum = 0;
          for (int oh = oh_start; oh <= oh_end; ++oh) {
            int f_h = in_h + a->pad_h - oh * a->stride_h;
            if (f_h % a->dil_h != 0) continue;
            f_h /= a->dil_h;
            for (int ow = ow_start; ow <= ow_end; ++ow) {
              int f_w = in_w + a->pad_w - ow * a->stride_w;
              if (f_w % a->dil_w != 0) continue;
              f_w /= a->dil_w;
              const long ro = FN(rot_index)(a, b, g, f_h, f_w, oh, ow);
              const REAL fh = FN(scope_coord)(f_h, rotation[ro], a->scope_h, a->k_h);
              const REAL fw = FN(scope_coord)(f_w, rotation[ro + plane_o], a->scope_w, a->k_w);
              sum += og[(long)oh * a->out_w + ow] *
                     FN(planar_bilinear)(flt, a->scope_h, a->scope_w, fh, fw);
            }
          }
          in_grad[((long)b * a->channel + c) * a->in_h * a->in_w + (long)in_h * a->in_w + in_w] = sum;
        }
    }
}

/* K.cu:836-955 SampleDepthwiseConv2dBackwardFilterKernel: the reference
 * atomically scatters onto filter_backprop[c]; here the sum runs serially in
 * thread-id order (b, oh, ow, f_h, f_w) per channel, ADDING into filter_grad
 * (the Python caller passes zeros, F/fsd.py:80). */
void FN(dko_sample_depthwise_backward_filter)(const dko_args *a, const REAL *out_grad,
                                              const REAL *input, const REAL *rotation,
                                              REAL *filter_grad) {
  const long plane_o = (long)a->out_h * a->out_w;
#pragma omp parallel for schedule(static)
  for (int c = 0; c < a->channel; ++c) {
    REAL *fg = filter_grad + (long)c * a->scope_h * a->scope_w;
    const int g = c % a->groups;
    for (int b = 0; b < a->batch; ++b) {
      const REAL *in = input + ((long)b * a->channel + c) * a->in_h * a->in_w;
      const REAL *og = out_grad + ((long)b * a->channel + c) * plane_o;
      for (int oh = 0; oh < a->out_h; ++oh)
        for (int ow = 0; ow < a->out_w; ++ow) {
          const REAL out_bp = og[(long)oh * a->out_w + ow];
          for (int f_h = 0; f_h < a->k_h; ++f_h) {
            const int in_row = oh * a->stride_h - a->pad_h + f_h * a->dil_h;
            for (int f_w = 0; f_w < a->k_w; ++f_w) {
              const int in_col = ow * a->stride_w - a->pad_w + f_w * a->dil_w;
              if (in_row >= 0 && in_row < a->in_h && in_col >= 0 && in_col < a->in_w) {
                const long ro = FN(rot_index)(a, b, g, f_h, f_w, oh, ow);
                REAL partial_sum = in[in_row * a->in_w + in_col] * out_bp;
                const REAL fh = FN(scope_coord)(f_h, rotation[ro], a->scope_h, a->k_h);
                const REAL fw = FN(scope_coord)(f_w, rotation[ro + plane_o], a->scope_w, a->k_w);
                FN(planar_bilinear_backward_data)(partial_sum, a->scope_h, a->scope_w, fh, fw, fg);
              }
            }
          }
        }
    }
  }
}

/* K.cu:1285-1370 SampleDepthwiseConv2dBackwardRotationKernel: one value per
 * (b, g, f_h, f_w, dir, oh, ow), serial sum over the channels of group g. */
void FN(dko_sample_depthwise_backward_rotation)(const dko_args *a, const REAL *out_grad,
                                                const REAL *input, const REAL *rotation,
                                                const REAL *filter, REAL *rotation_grad) {
  const long plane_o = (long)a->out_h * a->out_w;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < a->batch; ++b)
    for (int g = 0; g < a->groups; ++g)
      for (int f_h = 0; f_h < a->k_h; ++f_h)
        for (int f_w = 0; f_w < a->k_w; ++f_w)
          for (int dir = 0; dir < 2; ++dir)
            for (int oh = 0; oh < a->out_h; ++oh)
              for (int ow = 0; ow < a->out_w; ++ow) {
                const int in_row = oh * a->stride_h - a->pad_h + f_h * a->dil_h;
                const int in_col = ow * a->stride_w - a->pad_w + f_w * a->dil_w;
                const long ro = FN(rot_index)(a, b, g, f_h, f_w, oh, ow);
                const REAL fh = FN(scope_coord)(f_h, rotation[ro], a->scope_h, a->k_h);
                const REAL fw = FN(scope_coord)(f_w, rotation[ro + plane_o], a->scope_w, a->k_w);
                REAL coord_gradient = 0;
                if (in_row >= 0 && in_row < a->in_h && in_col >= 0 && in_col < a->in_w) {
                  for (int c = g; c < a->channel; c += a->groups) {
                    const REAL out_bp =
                        out_grad[((long)b * a->channel + c) * plane_o + (long)oh * a->out_w + ow];
                    REAL partial_sum = input[((long)b * a->channel + c) * a->in_h * a->in_w +
                                             (long)in_row * a->in_w + in_col] *
                                       out_bp;
                    coord_gradient += FN(planar_bilinear_backward_coord)(
                        partial_sum, filter + (long)c * a->scope_h * a->scope_w, a->scope_h,
                        a->scope_w, fh, fw, dir);
                  }
                }
                rotation_grad[ro + dir * plane_o] = coord_gradient;
              }
}

/* ---- deformable kernel + image-space offsets ----------------------------- */

/* Offset of the h-component of tap (f_h, f_w) in offset[N, kh*kw*2, Ho, Wo]
 * (K.cu:470-472, 490-491): shared by all channels, no groups. */
static inline long FN(off_index)(const dko_args *a, int b, int f_h, int f_w, int oh, int ow) {
  return (((long)b * (a->k_h * a->k_w) + (f_h * a->k_w + f_w)) * 2) * ((long)a->out_h * a->out_w) +
         ((long)oh * a->out_w + ow);
}

/* K.cu:433-528 DeformableSampleDepthwiseConv2dForwardKernel. */
void FN(dko_deformable_sample_depthwise_forward)(const dko_args *a, const REAL *input,
                                                 const REAL *offset, const REAL *rotation,
                                                 const REAL *filter, REAL *output) {
  const long plane_o = (long)a->out_h * a->out_w;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < a->batch; ++b)
    for (int c = 0; c < a->channel; ++c) {
      const REAL *in = input + ((long)b * a->channel + c) * a->in_h * a->in_w;
      const REAL *flt = filter + (long)c * a->scope_h * a->scope_w;
      const int g = c % a->groups;
      for (int oh = 0; oh < a->out_h; ++oh)
        for (int ow = 0; ow < a->out_w; ++ow) {
          REAL sum = 0;
          for (int f_h = 0; f_h < a->k_h; ++f_h) {
            const int in_h = oh * a->stride_h - a->pad_h + f_h * a->dil_h;
            for (int f_w = 0; f_w < a->k_w; ++f_w) {
              const int in_w = ow * a->stride_w - a->pad_w + f_w * a->dil_w;
              const long oo = FN(off_index)(a, b, f_h, f_w, oh, ow);
              const REAL input_h = in_h + offset[oo];
              const REAL input_w = in_w + offset[oo + plane_o];
              if (input_h > -1 && input_w > -1 && input_h < a->in_h && input_w < a->in_w) {
                const long ro = FN(rot_index)(a, b, g, f_h, f_w, oh, ow);
                const REAL cur_input = FN(im2col_bilinear)(in, a->in_h, a->in_w, input_h, input_w);
                const REAL fh = FN(scope_coord)(f_h, rotation[ro], a->scope_h, a->k_h);
                const REAL fw = FN(scope_coord)(f_w, rotation[ro + plane_o], a->scope_w, a->k_w);
                sum += cur_input * FN(planar_bilinear)(flt, a->scope_h, a->scope_w, fh, fw);
              }
            }
          }
          output[((long)b * a->channel + c) * plane_o + (long)oh * a->out_w + ow] = sum;
        }
    }
}

/* K.cu:704-795 DeformableSampleDepthwiseConv2dBackwardDataKernel: scatter in
 * the reference's thread-id order (b, f_h, f_w, c, oh, ow), ADDING into
 * in_grad (the Python caller passes zeros, F/fsd.py:153).  Parallel over
 * (b, c): every (b, c) plane is written by one thread only. */
void FN(dko_deformable_sample_depthwise_backward_data)(const dko_args *a, const REAL *out_grad,
                                                       const REAL *offset, const REAL *rotation,
                                                       const REAL *filter, REAL *in_grad) {
  const long plane_o = (long)a->out_h * a->out_w;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < a->batch; ++b)
    for (int c = 0; c < a->channel; ++c) {
      const int g = c % a->groups;
      REAL *ig = in_grad + ((long)b * a->channel + c) * a->in_h * a->in_w;
      const REAL *flt = filter + (long)c * a->scope_h * a->scope_w;
      for (int f_h = 0; f_h < a->k_h; ++f_h)
        for (int f_w = 0; f_w < a->k_w; ++f_w)
          for (int oh = 0; oh < a->out_h; ++oh)
            for (int ow = 0; ow < a->out_w; ++ow) {
              const int in_row = oh * a->stride_h - a->pad_h + f_h * a->dil_h;
              const int in_col = ow * a->stride_w - a->pad_w + f_w * a->dil_w;
              const long oo = FN(off_index)(a, b, f_h, f_w, oh, ow);
              const REAL input_h = in_row + offset[oo];
              const REAL input_w = in_col + offset[oo + plane_o];
              if (input_h > -1 && input_w > -1 && input_h < a->in_h && input_w < a->in_w) {
                const long ro = FN(rot_index)(a, b, g, f_h, f_w, oh, ow);
                const REAL out_bp =
                    out_grad[((long)b * a->channel + c) * plane_o + (long)oh * a->out_w + ow];
                const REAL fh = FN(scope_coord)(f_h, rotation[ro], a->scope_h, a->k_h);
                const REAL fw = FN(scope_coord)(f_w, rotation[ro + plane_o], a->scope_w, a->k_w);
                REAL cur_weight = FN(planar_bilinear)(flt, a->scope_h, a->scope_w, fh, fw);
                const REAL partial_sum = cur_weight * out_bp;
                FN(im2col_bilinear_backward)(partial_sum, input_h, input_w, a->in_h, a->in_w, ig);
              }
            }
    }
}

/* K.cu:1002-1097 DeformableSampleDepthwiseConv2dBackwardFilterKernel (ADDS
 * into filter_grad, serial per channel in thread-id order). */
void FN(dko_deformable_sample_depthwise_backward_filter)(const dko_args *a, const REAL *out_grad,
                                                         const REAL *input, const REAL *offset,
                                                         const REAL *rotation,
                                                         REAL *filter_grad) {
  const long plane_o = (long)a->out_h * a->out_w;
#pragma omp parallel for schedule(static)
  for (int c = 0; c < a->channel; ++c) {
    REAL *fg = filter_grad + (long)c * a->scope_h * a->scope_w;
    const int g = c % a->groups;
    for (int b = 0; b < a->batch; ++b) {
      const REAL *in = input + ((long)b * a->channel + c) * a->in_h * a->in_w;
      const REAL *og = out_grad + ((long)b * a->channel + c) * plane_o;
      for (int oh = 0; oh < a->out_h; ++oh)
        for (int ow = 0; ow < a->out_w; ++ow) {
          const REAL out_bp = og[(long)oh * a->out_w + ow];
          for (int f_h = 0; f_h < a->k_h; ++f_h) {
            const int in_row = oh * a->stride_h - a->pad_h + f_h * a->dil_h;
            for (int f_w = 0; f_w < a->k_w; ++f_w) {
              const int in_col = ow * a->stride_w - a->pad_w + f_w * a->dil_w;
              const long oo = FN(off_index)(a, b, f_h, f_w, oh, ow);
              const REAL input_h = in_row + offset[oo];
              const REAL input_w = in_col + offset[oo + plane_o];
              if (input_h > -1 && input_w > -1 && input_h < a->in_h && input_w < a->in_w) {
                const long ro = FN(rot_index)(a, b, g, f_h, f_w, oh, ow);
                const REAL partial_sum =
                    FN(im2col_bilinear)(in, a->in_h, a->in_w, input_h, input_w) * out_bp;
                const REAL fh = FN(scope_coord)(f_h, rotation[ro], a->scope_h, a->k_h);
                const REAL fw = FN(scope_coord)(f_w, rotation[ro + plane_o], a->scope_w, a->k_w);
                FN(planar_bilinear_backward_data)(partial_sum, a->scope_h, a->scope_w, fh, fw, fg);
              }
            }
          }
        }
    }
  }
}

/* K.cu:1147-1243 DeformableSampleDepthwiseConv2dBackwardOffsetKernel: serial
 * sum over ALL channels (each with its own group's rotation). */
void FN(dko_deformable_sample_depthwise_backward_offset)(const dko_args *a, const REAL *out_grad,
                                                         const REAL *input, const REAL *offset,
                                                         const REAL *rotation, const REAL *filter,
                                                         REAL *offset_grad) {
  const long plane_o = (long)a->out_h * a->out_w;
#pragma omp parallel for schedule(static)
  for (int b = 0; b < a->batch; ++b)
    for (int f_h = 0; f_h < a->k_h; ++f_h)
      for (int f_w = 0; f_w < a->k_w; ++f_w)
        for (int dir = 0; dir < 2; ++dir)
          for (int oh = 0; oh < a->out_h; ++oh)
            for (int ow = 0; ow < a->out_w; ++ow) {
              const int in_row = oh * a->stride_h - a->pad_h + f_h * a->dil_h;
              const int in_col = ow * a->stride_w - a->pad_w + f_w * a->dil_w;
              const long oo = FN(off_index)(a, b, f_h, f_w, oh, ow);
              const REAL input_h = in_row + offset[oo];
              const REAL input_w = in_col + offset[oo + plane_o];
              REAL coord_gradient = 0;
              if (input_h > -1 && input_w > -1 && input_h < a->in_h && input_w < a->in_w) {
                for (int c = 0; c < a->channel; ++c) {
                  const int g = c % a->groups;
                  const long ro = FN(rot_index)(a, b, g, f_h, f_w, oh, ow);
                  REAL fh = FN(scope_coord)(f_h, rotation[ro], a->scope_h, a->k_h);
                  REAL fw = FN(scope_coord)(f_w, rotation[ro + plane_o], a->scope_w, a->k_w);
                  const REAL out_bp =
                      out_grad[((long)b * a->channel + c) * plane_o + (long)oh * a->out_w + ow];
                  REAL cur_weight = FN(planar_bilinear)(
                      filter + (long)c * a->scope_h * a->scope_w, a->scope_h, a->scope_w, fh, fw);
                  REAL partial_sum = cur_weight * out_bp;
                  coord_gradient +=
                      FN(coordinate_weight)(input_h, input_w, a->in_h, a->in_w,
                                            input + ((long)b * a->channel + c) * a->in_h * a->in_w,
                                            dir) *
                      partial_sum;
                }
              }
              offset_grad[oo + dir * plane_o] = coord_gradient;
            }
}

/* K.cu:1410-1507 DeformableSampleDepthwiseConv2dBackwardRotationKernel. */
void FN(dko_deformable_sample_depthwise_backward_rotation)(const dko_args *a, const REAL *out_grad,
                                                           const REAL *input, const REAL *offset,
                                                           const REAL *rotation,
                                                           const REAL *filter,
                                                           REAL *rotation_grad) {
  const long plane_o = (long)a->out_h * a->out_w;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < a->batch; ++b)
    for (int g = 0; g < a->groups; ++g)
      for (int f_h = 0; f_h < a->k_h; ++f_h)
        for (int f_w = 0; f_w < a->k_w; ++f_w)
          for (int dir = 0; dir < 2; ++dir)
            for (int oh = 0; oh < a->out_h; ++oh)
              for (int ow = 0; ow < a->out_w; ++ow) {
                const int in_row = oh * a->stride_h - a->pad_h + f_h * a->dil_h;
                const int in_col = ow * a->stride_w - a->pad_w + f_w * a->dil_w;
                const long oo = FN(off_index)(a, b, f_h, f_w, oh, ow);
                const long ro = FN(rot_index)(a, b, g, f_h, f_w, oh, ow);
                const REAL input_h = in_row + offset[oo];
                const REAL input_w = in_col + offset[oo + plane_o];
                REAL coord_gradient = 0;
                if (input_h > -1 && input_w > -1 && input_h < a->in_h && input_w < a->in_w) {
                  REAL fh = FN(scope_coord)(f_h, rotation[ro], a->scope_h, a->k_h);
                  REAL fw = FN(scope_coord)(f_w, rotation[ro + plane_o], a->scope_w, a->k_w);
                  for (int c = g; c < a->channel; c += a->groups) {
                    const REAL out_bp =
                        out_grad[((long)b * a->channel + c) * plane_o + (long)oh * a->out_w + ow];
                    REAL partial_sum =
                        FN(im2col_bilinear)(input + ((long)b * a->channel + c) * a->in_h * a->in_w,
                                            a->in_h, a->in_w, input_h, input_w) *
                        out_bp;
                    coord_gradient += FN(planar_bilinear_backward_coord)(
                        partial_sum, filter + (long)c * a->scope_h * a->scope_w, a->scope_h,
                        a->scope_w, fh, fw, dir);
                  }
                }
                rotation_grad[ro + dir * plane_o] = coord_gradient;
              }
}

/* ---- N-d linear sample ---------------------------------------------------- */

/* ND.cu:45-88 nd_linear; `shape` holds the spatial sizes as REAL and is cast
 * to int per use exactly as the reference does (ND.cu:49). */
static REAL FN(nd_linear)(const REAL *data, const REAL *shape, const REAL *coord, int dims) {
  for (int d = 0; d < dims; d++) {
    REAL x = coord[d];
    int s = (int)shape[d];
    if (x <= -1 || x >= s) return 0;
  }
  const unsigned corners = 1u << dims;
  REAL val = 0;
  for (unsigned i = 0; i < corners; i++) {
    long data_offset = 0;
    REAL data_weight = 1;
    int out_of_scope = 0;
    for (int d = 0; d < dims; d++) {
      REAL x = coord[d];
      int s = (int)shape[d];
      data_offset *= s;
      unsigned offset = (i >> d) & 1u;
      int x_low = (int)floor((double)x);
      REAL w = x - x_low;
      if (offset == 0 && x_low >= 0) {
        data_offset += x_low;
        data_weight *= 1 - w;
      } else if (offset == 1 && x_low + 1 <= s - 1) {
        data_offset += x_low + 1;
        data_weight *= w;
      } else {
        out_of_scope = 1;
        break;
      }
    }
    if (!out_of_scope) val += data_weight * data[data_offset];
  }
  return val;
}

/* ND.cu:90-131 nd_linear_backward_data (atomicAdd in the reference). */
static void FN(nd_linear_backward_data)(REAL top_gradient, const REAL *shape, const REAL *coord,
                                        int dims, REAL *data_gradient) {
  for (int d = 0; d < dims; d++) {
    REAL x = coord[d];
    int s = (int)shape[d];
    if (x <= -1 || x >= s) return;
  }
  const unsigned corners = 1u << dims;
  for (unsigned i = 0; i < corners; i++) {
    long data_offset = 0;
    REAL data_weight = 1;
    int out_of_scope = 0;
    for (int d = 0; d < dims; d++) {
      REAL x = coord[d];
      int s = (int)shape[d];
      data_offset *= s;
      unsigned offset = (i >> d) & 1u;
      int x_low = (int)floor((double)x);
      REAL w = x - x_low;
      if (offset == 0 && x_low >= 0) {
        data_offset += x_low;
        data_weight *= 1 - w;
      } else if (offset == 1 && x_low + 1 <= s - 1) {
        data_offset += x_low + 1;
        data_weight *= w;
      } else {
        out_of_scope = 1;
        break;
      }
    }
    if (!out_of_scope) data_gradient[data_offset] += data_weight * top_gradient;
  }
}

/* ND.cu:133-177 nd_linear_backward_coord: the weight of dimension gdim is
 * replaced by -1 (low corner) / +1 (high corner). */
static REAL FN(nd_linear_backward_coord)(REAL top_gradient, const REAL *data, const REAL *shape,
                                         const REAL *coord, int dims, int gdim) {
  for (int d = 0; d < dims; d++) {
    REAL x = coord[d];
    int s = (int)shape[d];
    if (x <= -1 || x >= s) return 0;
  }
  REAL grad = 0;
  const unsigned corners = 1u << dims;
  for (unsigned i = 0; i < corners; i++) {
    long data_offset = 0;
    REAL data_weight = 1;
    int out_of_scope = 0;
    for (int d = 0; d < dims; d++) {
      REAL x = coord[d];
      int s = (int)shape[d];
      data_offset *= s;
      unsigned offset = (i >> d) & 1u;
      int x_low = (int)floor((double)x);
      REAL w = x - x_low;
      if (offset == 0 && x_low >= 0) {
        data_offset += x_low;
        data_weight *= (d == gdim) ? (REAL)(-1) : 1 - w;
      } else if (offset == 1 && x_low + 1 <= s - 1) {
        data_offset += x_low + 1;
        data_weight *= (d == gdim) ? (REAL)(1) : w;
      } else {
        out_of_scope = 1;
        break;
      }
    }
    if (!out_of_scope) grad += top_gradient * data[data_offset] * data_weight;
  }
  return grad;
}

/* ND.cu:183-201 NdLinearSampleForwardKernel: output[b, c], c fastest;
 * prod_shape = data.stride(0) (ND.cpp:19). */
void FN(dko_nd_linear_sample_forward)(int batch, int channel, int dims, long prod_shape,
                                      const REAL *data, const REAL *shape, const REAL *coord,
                                      REAL *output) {
#pragma omp parallel for schedule(static)
  for (long b = 0; b < batch; ++b)
    for (int c = 0; c < channel; ++c)
      output[b * channel + c] = FN(nd_linear)(data + c * prod_shape, shape, coord + b * dims, dims);
}

/* ND.cu:225-243 NdLinearSampleBackwardDataKernel; in_grad is zero-filled
 * first as the host wrapper does (ND.cpp:40), then summed serially over b. */
void FN(dko_nd_linear_sample_backward_data)(int batch, int channel, int dims, long prod_shape,
                                            const REAL *out_grad, const REAL *shape,
                                            const REAL *coord, REAL *in_grad) {
  memset(in_grad, 0, sizeof(REAL) * (size_t)channel * (size_t)prod_shape);
#pragma omp parallel for schedule(static)
  for (int c = 0; c < channel; ++c)
    for (long b = 0; b < batch; ++b)
      FN(nd_linear_backward_data)(out_grad[b * channel + c], shape, coord + b * dims, dims,
                                  in_grad + c * prod_shape);
}

/* ND.cu:267-287 NdLinearSampleBackwardCoordKernel: per-channel partials
 * coord_grad_c[b, d, c]; the Python caller sums them over c
 * (functions/nd_linear_sample.py:48-55). */
void FN(dko_nd_linear_sample_backward_coord)(int batch, int channel, int dims, long prod_shape,
                                             const REAL *out_grad, const REAL *data,
                                             const REAL *shape, const REAL *coord,
                                             REAL *coord_grad_c) {
#pragma omp parallel for schedule(static)
  for (long b = 0; b < batch; ++b)
    for (int d = 0; d < dims; ++d)
      for (int c = 0; c < channel; ++c)
        coord_grad_c[(b * dims + d) * channel + c] = FN(nd_linear_backward_coord)(
            out_grad[b * channel + c], data + c * prod_shape, shape, coord + b * dims, dims, d);
}

#undef FN
#undef CAT
#undef CAT_
