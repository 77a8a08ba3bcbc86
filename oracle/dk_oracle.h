/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the deformable-kernel operators.
 *
 * A plain-C restatement of the arithmetic of the reference's CUDA kernels
 * (deformable_kernels/ops/deform_kernel/csrc/filter_sample_depthwise_cuda_kernel.cu
 * and nd_linear_sample_cuda_kernel.cu), in fp32 (_f32) and fp64 (_f64).
 * Only the tests, the smoke check and the benchmark's cpu_baseline leg may
 * link or load it; the shipped HIP library and Python package never do.
 *
 * What pins it (tests/test_oracle_*.py): torch grid_sample composites in
 * float64 with autograd for every forward and gradient, closed forms
 * (scope == kernel with zero offsets is a depthwise convolution; integer
 * offsets permute taps; offsets beyond the scope give exact zeros; zero image
 * offsets reduce the deformable variant to the local one), central finite
 * differences, brute-force corner loops and numpy.interp for the N-d sampler.
 * The reference ships no tests or golden vectors of its own.
 */
#ifndef DK_ORACLE_H
#define DK_ORACLE_H

#ifdef __cplusplus
extern "C" {
#endif

/* Field-for-field the reference's SampleDepthwiseArgs
 * (csrc/filter_sample_depthwise_cuda.h:1-28). */
typedef struct {
  int batch, channel, in_h, in_w;
  int k_h, k_w, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  int out_h, out_w;
  int scope_h, scope_w, groups;
} dko_args;

#define DKO_DECL(REAL, S)                                                                          \
  void dko_sample_depthwise_forward##S(const dko_args *, const REAL *input, const REAL *rotation,  \
                                       const REAL *filter, REAL *output);                          \
  void dko_sample_depthwise_backward_data##S(const dko_args *, const REAL *out_grad,               \
                                             const REAL *rotation, const REAL *filter,             \
                                             REAL *in_grad);                                       \
  void dko_sample_depthwise_backward_filter##S(const dko_args *, const REAL *out_grad,             \
                                               const REAL *input, const REAL *rotation,            \
                                               REAL *filter_grad);                                 \
  void dko_sample_depthwise_backward_rotation##S(const dko_args *, const REAL *out_grad,           \
                                                 const REAL *input, const REAL *rotation,          \
                                                 const REAL *filter, REAL *rotation_grad);         \
  void dko_deformable_sample_depthwise_forward##S(const dko_args *, const REAL *input,             \
                                                  const REAL *offset, const REAL *rotation,        \
                                                  const REAL *filter, REAL *output);               \
  void dko_deformable_sample_depthwise_backward_data##S(                                           \
      const dko_args *, const REAL *out_grad, const REAL *offset, const REAL *rotation,            \
      const REAL *filter, REAL *in_grad);                                                          \
  void dko_deformable_sample_depthwise_backward_filter##S(                                         \
      const dko_args *, const REAL *out_grad, const REAL *input, const REAL *offset,               \
      const REAL *rotation, REAL *filter_grad);                                                    \
  void dko_deformable_sample_depthwise_backward_offset##S(                                         \
      const dko_args *, const REAL *out_grad, const REAL *input, const REAL *offset,               \
      const REAL *rotation, const REAL *filter, REAL *offset_grad);                                \
  void dko_deformable_sample_depthwise_backward_rotation##S(                                       \
      const dko_args *, const REAL *out_grad, const REAL *input, const REAL *offset,               \
      const REAL *rotation, const REAL *filter, REAL *rotation_grad);                              \
  void dko_nd_linear_sample_forward##S(int batch, int channel, int dims, long prod_shape,          \
                                       const REAL *data, const REAL *shape, const REAL *coord,     \
                                       REAL *output);                                              \
  void dko_nd_linear_sample_backward_data##S(int batch, int channel, int dims, long prod_shape,    \
                                             const REAL *out_grad, const REAL *shape,              \
                                             const REAL *coord, REAL *in_grad);                    \
  void dko_nd_linear_sample_backward_coord##S(int batch, int channel, int dims, long prod_shape,   \
                                              const REAL *out_grad, const REAL *data,              \
                                              const REAL *shape, const REAL *coord,                \
                                              REAL *coord_grad_c);

DKO_DECL(float, _f32)
DKO_DECL(double, _f64)

/* Number of OpenMP threads the oracle will use (1 when built without OpenMP). */
int dko_max_threads(void);
void dko_set_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
