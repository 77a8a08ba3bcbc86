/*
 * dk_hip.h -- C ABI of libdk_hip.so: the deformable-kernel operators as
 * hand-written gfx950 (MI355X) HIP kernels.
 *
 * One entry point per function of the reference's two pybind11 extension
 * modules (the Python -> native boundary of the operator path):
 *
 *   filter_sample_depthwise_cuda   csrc/filter_sample_depthwise_cuda.cpp:540-569
 *   nd_linear_sample_cuda          csrc/nd_linear_sample_cuda.cpp:67-74
 *
 * Conventions shared by every entry point
 *   - plain C: raw device pointers, sizes and a descriptor struct; no torch
 *     or HIP types appear in a signature (`stream` is a hipStream_t passed
 *     as void*, NULL = the default stream);
 *   - all tensors are dense, contiguous, row-major (NCHW) and of the one
 *     dtype named in the descriptor; the caller owns all memory, including
 *     the optional workspace, whose size the matching *_workspace() query
 *     returns; the library itself never allocates;
 *   - every output buffer is OVERWRITTEN (no pre-zeroing is needed; the
 *     reference's filter/data gradients accumulate atomically into buffers
 *     its Python caller zero-fills -- functions/filter_sample_depthwise.py:64-80);
 *   - calls are asynchronous on `stream`, thread-safe and hold no global
 *     mutable state (apart from the test hook dk_test_switches());
 *   - the return value is DK_OK (0) or a negative dk_status; nothing is
 *     launched when an argument is rejected.  (The reference validates
 *     nothing and always returns 1 -- filter_sample_depthwise_cuda.cpp:61.)
 *   - fp16 / bf16 tensors are computed in fp32 registers and accumulators.
 */
#ifndef DK_HIP_H
#define DK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  DK_OK = 0,
  DK_ERR_NULL_POINTER = -1,   /* a required pointer (descriptor, tensor) is NULL        */
  DK_ERR_BAD_SHAPE = -2,      /* non-positive size, output would be empty or negative,  */
                              /* channel not divisible by rotation groups               */
  DK_ERR_BAD_DTYPE = -3,      /* dtype tag not one of dk_dtype                          */
  DK_ERR_TOO_LARGE = -4,      /* a tensor has >= 2^31 elements (32-bit plane indexing)  */
  DK_ERR_WORKSPACE = -5,      /* workspace NULL or smaller than the *_workspace() query */
  DK_ERR_LAUNCH = -6,         /* the HIP runtime refused the launch                     */
  DK_ERR_UNSUPPORTED = -7,    /* e.g. more than DK_ND_MAX_DIMS sampling dimensions      */
  DK_ERR_SCRATCH_LIMIT = -8   /* *_static entry point: the problem needs more scratch   */
                              /* memory than DK_STATIC_SCRATCH_BYTES                    */
} dk_status;

typedef enum { DK_F32 = 0, DK_F16 = 1, DK_BF16 = 2, DK_F64 = 3 } dk_dtype;

typedef enum dk_rotation_clip {
  DK_CLIP_NONE = 0,
  DK_CLIP_ROTATION = 1, /* offset r -> min(max(r, clip_min), clip_max)  (a (min, max) rotation_clip) */
  DK_CLIP_COORD = 2     /* scope coordinate f + r + (scope - k) / 2 -> the same range, both axes
                           (rotation_clip == 'scope': clip_min = 0, clip_max = scope_h - 1) */
} dk_rotation_clip;

typedef enum dk_layout { DK_LAYOUT_NCHW = 0, DK_LAYOUT_NHWC = 1 } dk_layout;

/* Geometry of one depthwise deformable-kernel layer: the fields the
 * reference packs into SampleDepthwiseArgs (csrc/filter_sample_depthwise_cuda.h:1-28)
 * from the tensor sizes and the eleven ints of each pybind call; out_h/out_w
 * are derived inside the library by the rule of filter_sample_depthwise_cuda.cpp:42-43:
 *   out = (in + 2*pad - (dil*(k-1)+1)) / stride + 1
 *
 * Tensor layouts
 *   input     [batch, channel, in_h, in_w]
 *   filter    [channel, 1, scope_h, scope_w]     the per-channel scope tile
 *   rotation  [batch, groups*k_h*k_w*2, out_h, out_w]  kernel-space offsets, channel index
 *             g*(k_h*k_w*2) + (f_h*k_w + f_w)*2 + dir, dir 0 = h, 1 = w; channel c uses g = c % groups
 *   offset    [batch, k_h*k_w*2, out_h, out_w]   image-space offsets, same (tap, dir) order
 *   output    [batch, channel, out_h, out_w]
 */
typedef struct dk_conv_desc {
  int32_t batch, channel, in_h, in_w;
  int32_t k_h, k_w;
  int32_t stride_h, stride_w;
  int32_t pad_h, pad_w;
  int32_t dil_h, dil_w;
  int32_t scope_h, scope_w;
  int32_t groups;           /* rotation groups ("sampling_group") */
  int32_t dtype;            /* dk_dtype of every tensor of the call */
  /* Clamp of the kernel-space offsets applied inside the operator, so that a caller need not
   * clamp (read, write, re-read) the rotation tensor first.  The reference's operators have no
   * such argument: its module clamps the tensor beforehand (modules/deform_kernel.py:185-212,
   * _clip_rotation).  DK_CLIP_NONE (0) reproduces the reference operator exactly.  The
   * gradient with respect to a clamped offset is zero, as torch.clamp's is. */
  int32_t rotation_clip;    /* dk_rotation_clip */
  float clip_min, clip_max; /* the range; ignored for DK_CLIP_NONE */
  /* Memory layout of the 4-d tensors of the call (input, rotation, output and their gradients;
   * the filter is always [channel][scope_h][scope_w]).  DK_LAYOUT_NCHW (0) is the reference's.
   * DK_LAYOUT_NHWC: the same logical tensors stored channels-last ([batch][h][w][channel];
   * rotation [batch][out_h][out_w][groups*k_h*k_w*2]), for networks whose other layers run
   * channels-last.  Taken by the local operator's entry points (dk_sample_depthwise_*); the
   * deformable and per-image entry points return DK_ERR_UNSUPPORTED for it.  The reference has
   * no such argument. */
  int32_t layout;           /* dk_layout */
} dk_conv_desc;

/* Output extent for the descriptor, or a negative dk_status. */
int dk_conv_out_size(const dk_conv_desc *desc, int32_t *out_h, int32_t *out_w);

/* 1 if the local operator's entry points (dk_sample_depthwise_*) serve the descriptor's `layout`, 0 if
 * they would return DK_ERR_UNSUPPORTED (a channels-last geometry whose tables do not fit LDS: e.g. 64
 * rotation groups with 3 x 3 taps and a 4 x 4 scope), a negative dk_status for an invalid descriptor.
 * DK_LAYOUT_NCHW is always served.  A caller with channels-last tensors asks first and converts to NCHW
 * when the answer is 0.  No counterpart in the reference, whose kernels take planar tensors only. */
int dk_sample_depthwise_layout_supported(const dk_conv_desc *desc);

/* ---- local deformable kernel: kernel-space offsets only ------------------- */

/* sample_depthwise_forward_cuda (filter_sample_depthwise_cuda.cpp:8-62). */
int dk_sample_depthwise_forward(const dk_conv_desc *desc, const void *input, const void *rotation,
                                const void *filter, void *output, void *stream);

/* sample_depthwise_backward_data_cuda (filter_sample_depthwise_cuda.cpp:64-119).
 * `input` is not needed for this gradient and is not an argument. */
int dk_sample_depthwise_backward_data(const dk_conv_desc *desc, const void *out_grad,
                                      const void *rotation, const void *filter, void *in_grad,
                                      void *stream);

/* sample_depthwise_backward_filter_cuda (filter_sample_depthwise_cuda.cpp:121-176).
 * Needs a workspace for per-workgroup partial sums (reduced without global atomics). */
size_t dk_sample_depthwise_backward_filter_workspace(const dk_conv_desc *desc);
int dk_sample_depthwise_backward_filter(const dk_conv_desc *desc, const void *out_grad,
                                        const void *input, const void *rotation,
                                        void *filter_grad, void *workspace,
                                        size_t workspace_bytes, void *stream);

/* The same filter gradient for callers that cannot allocate device memory or hand over a
 * workspace: tight serving loops, harnesses that forbid hipMalloc, code that is later captured
 * into a HIP graph.  No counterpart in the reference.  The per-workgroup partial sums go to a buffer of
 * DK_STATIC_SCRATCH_BYTES that is part of the library's device image (every GPU the library runs
 * on holds it until the process ends); the call allocates nothing and runs the same kernels as
 * dk_sample_depthwise_backward_filter, so the result is bit-identical to that function's.
 * Returns DK_ERR_SCRATCH_LIMIT, launching nothing, when
 * dk_sample_depthwise_backward_filter_workspace(desc) exceeds DK_STATIC_SCRATCH_BYTES.
 * All calls on one GPU share the one buffer: calls that may overlap on a GPU (different streams,
 * different host threads) race on it and must be ordered by the caller.
 * The first call for a (device, descriptor shape) pair looks the buffer's address up and sets a
 * kernel attribute -- host-side runtime calls that a stream in capture mode may refuse (the call
 * then returns DK_ERR_LAUNCH).  A caller that captures the call into a HIP graph therefore makes
 * one ordinary (warm-up) call with the same descriptor on that device first; every later call is
 * kernel launches only. */
#define DK_STATIC_SCRATCH_BYTES (8u << 20)
int dk_sample_depthwise_backward_filter_static(const dk_conv_desc *desc, const void *out_grad,
                                               const void *input, const void *rotation,
                                               void *filter_grad, void *stream);

/* sample_depthwise_backward_rotation_cuda (filter_sample_depthwise_cuda.cpp:178-235).
 * Small planes split the channel sum over several workgroups whose partial sums go through the
 * workspace and are added in a fixed order; the query returns 0 when no split is used. */
size_t dk_sample_depthwise_backward_rotation_workspace(const dk_conv_desc *desc);
int dk_sample_depthwise_backward_rotation(const dk_conv_desc *desc, const void *out_grad,
                                          const void *input, const void *rotation,
                                          const void *filter, void *rotation_grad, void *workspace,
                                          size_t workspace_bytes, void *stream);

/* The three gradients of one backward pass in one call; any of in_grad / rotation_grad /
 * filter_grad may be NULL to skip it.  Stands in for the three consecutive pybind calls of
 * SampleDepthwiseFunction.backward (functions/filter_sample_depthwise.py:63-85): one call that
 * issues the launches of the three entry points above on `stream`.  Workspace as for
 * *_backward_filter (only needed when filter_grad is requested). */
size_t dk_sample_depthwise_backward_workspace(const dk_conv_desc *desc);
int dk_sample_depthwise_backward(const dk_conv_desc *desc, const void *out_grad, const void *input,
                                 const void *rotation, const void *filter, void *in_grad,
                                 void *rotation_grad, void *filter_grad, void *workspace,
                                 size_t workspace_bytes, void *stream);

/* ---- deformable kernel with image-space offsets ---------------------------- */

/* In the forward and in the data / filter / offset gradients below, `rotation` may be NULL: the
 * kernel-space offsets are then all zero and no rotation tensor is read.  This is the call of
 * DeformKernelConv2d / DeformConv2d (modules/deform_kernel.py:276-279 passes rotation = None,
 * modules/deform_conv.py:31-42 sets scope = kernel), for which the reference allocates, fills
 * and reads a zero tensor of batch x groups*k*k*2 x out_h x out_w elements
 * (ops/deform_kernel/modules/filter_sample_depthwise.py:163-168); with scope = kernel the taps
 * then sit on the scope's own cells and the result is the depthwise deformable convolution.
 * Same values as with a tensor of zeros. */

/* deformable_sample_depthwise_forward_cuda (filter_sample_depthwise_cuda.cpp:237-294). */
int dk_deformable_sample_depthwise_forward(const dk_conv_desc *desc, const void *input,
                                           const void *offset, const void *rotation,
                                           const void *filter, void *output, void *stream);

/* deformable_sample_depthwise_backward_data_cuda (filter_sample_depthwise_cuda.cpp:296-354). */
size_t dk_deformable_sample_depthwise_backward_data_workspace(const dk_conv_desc *desc);
int dk_deformable_sample_depthwise_backward_data(const dk_conv_desc *desc, const void *out_grad,
                                                 const void *offset, const void *rotation,
                                                 const void *filter, void *in_grad,
                                                 void *workspace, size_t workspace_bytes,
                                                 void *stream);

/* deformable_sample_depthwise_backward_filter_cuda (filter_sample_depthwise_cuda.cpp:356-414). */
size_t dk_deformable_sample_depthwise_backward_filter_workspace(const dk_conv_desc *desc);
int dk_deformable_sample_depthwise_backward_filter(const dk_conv_desc *desc, const void *out_grad,
                                                   const void *input, const void *offset,
                                                   const void *rotation, void *filter_grad,
                                                   void *workspace, size_t workspace_bytes,
                                                   void *stream);

/* deformable_sample_depthwise_backward_offset_cuda (filter_sample_depthwise_cuda.cpp:416-476).
 * The workspace holds per-channel-chunk partial sums that are added in a fixed order. */
size_t dk_deformable_sample_depthwise_backward_offset_workspace(const dk_conv_desc *desc);
int dk_deformable_sample_depthwise_backward_offset(const dk_conv_desc *desc, const void *out_grad,
                                                   const void *input, const void *offset,
                                                   const void *rotation, const void *filter,
                                                   void *offset_grad, void *workspace,
                                                   size_t workspace_bytes, void *stream);

/* deformable_sample_depthwise_backward_rotation_cuda (filter_sample_depthwise_cuda.cpp:478-538).
 * Workspace as for the offset gradient. */
size_t dk_deformable_sample_depthwise_backward_rotation_workspace(const dk_conv_desc *desc);
int dk_deformable_sample_depthwise_backward_rotation(const dk_conv_desc *desc,
                                                     const void *out_grad, const void *input,
                                                     const void *offset, const void *rotation,
                                                     const void *filter, void *rotation_grad,
                                                     void *workspace, size_t workspace_bytes,
                                                     void *stream);

/* Both coordinate gradients of the deformable operator in one call -- what the reference's backward
 * (functions/filter_sample_depthwise.py:163-197) asks for with its two calls
 * deformable_sample_depthwise_backward_offset_cuda and ..._backward_rotation_cuda.  Where one pass over the
 * input can produce both (planes of up to 64 x 64 pixels) they come from one kernel; otherwise the two
 * entry points above run one after the other on the stream.  `rotation` must not be NULL here. */
size_t dk_deformable_sample_depthwise_backward_offset_rotation_workspace(const dk_conv_desc *desc);
int dk_deformable_sample_depthwise_backward_offset_rotation(const dk_conv_desc *desc, const void *out_grad,
                                                            const void *input, const void *offset,
                                                            const void *rotation, const void *filter,
                                                            void *offset_grad, void *rotation_grad,
                                                            void *workspace, size_t workspace_bytes,
                                                            void *stream);

/* ---- N-d linear sample -------------------------------------------------------
 * data [channel, shape[0..dims-1]], coord [batch, dims] in absolute index units,
 * output [batch, channel].  The reference passes `shape` as a device tensor of the
 * data's floating dtype (functions/nd_linear_sample.py:22); here it is host
 * integers in the descriptor, which removes a host-to-device copy per call. */
#define DK_ND_MAX_DIMS 8
typedef struct dk_nd_desc {
  int64_t batch;                    /* number of sample points              */
  int32_t channel;
  int32_t dims;                     /* 1..DK_ND_MAX_DIMS                    */
  int32_t shape[DK_ND_MAX_DIMS];
  int32_t dtype;
} dk_nd_desc;

/* nd_linear_sample_forward_cuda (nd_linear_sample_cuda.cpp:10-26).  For large problems the
 * library samples from a channel-last copy of `data` that it writes into the workspace (so
 * the channels of one corner are one contiguous read); the query returns 0 when the direct
 * path is used. */
size_t dk_nd_linear_sample_forward_workspace(const dk_nd_desc *desc);
int dk_nd_linear_sample_forward(const dk_nd_desc *desc, const void *data, const void *coord,
                                const void *order, void *output, void *workspace,
                                size_t workspace_bytes, void *stream);

/* With many points per cell of the volume the three functions sort the points by cell first.
 * A caller that issues more than one of them on the same coordinates (a forward and its
 * backward) can have the order computed once: dk_nd_linear_sample_order_bytes() is the size of
 * the order array (0 when the configuration does not sort: pass order = NULL then),
 * dk_nd_linear_sample_order() fills it, and the three functions take it as `order`; with
 * order = NULL they sort for themselves.  No counterpart in the reference. */
size_t dk_nd_linear_sample_order_bytes(const dk_nd_desc *desc);
size_t dk_nd_linear_sample_order_workspace(const dk_nd_desc *desc);
int dk_nd_linear_sample_order(const dk_nd_desc *desc, const void *coord, void *order,
                              void *workspace, size_t workspace_bytes, void *stream);

/* nd_linear_sample_backward_data_cuda (nd_linear_sample_cuda.cpp:29-45); in_grad is
 * fully written (the reference zero-fills it in C++ and scatters atomically).  The workspace
 * holds an fp32 accumulation image of the data's element count when one is needed (fp16 / bf16
 * gradients, and the channel-last path for large problems). */
size_t dk_nd_linear_sample_backward_data_workspace(const dk_nd_desc *desc);
int dk_nd_linear_sample_backward_data(const dk_nd_desc *desc, const void *out_grad,
                                      const void *coord, const void *order, void *in_grad,
                                      void *workspace, size_t workspace_bytes, void *stream);

/* nd_linear_sample_backward_coord_cuda (nd_linear_sample_cuda.cpp:47-64) fused with the
 * `.sum(2)` its Python caller applies (functions/nd_linear_sample.py:48-55):
 * coord_grad is [batch, dims], already summed over channels. */
size_t dk_nd_linear_sample_backward_coord_workspace(const dk_nd_desc *desc);
int dk_nd_linear_sample_backward_coord(const dk_nd_desc *desc, const void *out_grad,
                                       const void *data, const void *coord, const void *order,
                                       void *coord_grad, void *workspace, size_t workspace_bytes,
                                       void *stream);

/* ---- offset branch ---------------------------------------------------------- */

/* The 3x3 convolution that predicts the kernel-space offsets of a LocalDeformKernel2d layer
 * (modules/deform_kernel.py:165-168: nn.Conv2d(in_planes, rotation_groups*k*k*2, k, stride,
 * padding, dilation, bias=True), applied at :214).  The reference calls the framework's
 * convolution there; this entry point is a faster kernel for that one shape family: padding 1,
 * dilation 1, float32 / float16 / bfloat16 tensors, in_channels a multiple of 16, out_channels <= 16
 * or 18 or 20, width 7, 14, 28, 56 or 112.  Arithmetic: fp32 sums throughout, results rounded once;
 * float16 / bfloat16 elements are multiplied as they are (exact products) on the 16-bit matrix
 * instructions; float32 elements go to the same instructions as bfloat16 (hi, lo) pairs, hi = bf16(v),
 * lo = bf16(v - hi), all four products added: about 3.5e-6 of the result's scale against the float64
 * convolution (the framework's float32 kernels: 5e-7), an infinite element gives NaN.  The test switch
 * DK_NO_OFFSET_PAIRS restores the fp32 matrix-instruction forward (stride 1, 1e-6) and leaves the other
 * float32 passes to the caller.  dk_offset_conv_supported() tells
 * whether a shape is covered, dk_offset_conv_worthwhile() whether it is also expected to beat the
 * library convolution (every covered plane with at least 64 (image, 448-pixel tile) items); the
 * caller keeps its library convolution otherwise.
 *   input [batch, in_channels, h, w], weight [out_channels, in_channels, 3, 3],
 *   bias [out_channels], output [batch, out_channels, h, w]; workspace: packed weights. */
typedef struct dk_offset_conv_desc {
  int32_t batch, in_channels, out_channels, h, w; /* h, w: the input plane (= the output plane at stride 1) */
  int32_t dtype;  /* DK_F32, DK_F16 or DK_BF16 */
  int32_t stride; /* 0 or 1: stride 1.  2: the down-sampling layers' convolution (output ((h - 1) / 2 + 1) x (w / 2));
                     only the forward and the input gradient on input planes 14, 28, 56 or 112 wide have kernels:
                     dk_offset_conv_supported() / _worthwhile() then speak for those two */
} dk_offset_conv_desc;
int dk_offset_conv_supported(const dk_offset_conv_desc *desc);
int dk_offset_conv_worthwhile(const dk_offset_conv_desc *desc);
size_t dk_offset_conv_forward_workspace(const dk_offset_conv_desc *desc);
int dk_offset_conv_forward(const dk_offset_conv_desc *desc, const void *input, const void *weight,
                           const void *bias, void *output, void *workspace, size_t workspace_bytes,
                           void *stream);

/* Gradient of that convolution's weight, weight_grad [out_channels, in_channels, 3, 3] (fully written),
 * stride 1 and 2, up to 20 output channels: on the 16-bit matrix instructions with the pixels as the inner
 * dimension (16-bit elements as they are, float32 ones as bfloat16 pairs: about 4e-6 of the result's scale);
 * per-workgroup partial sums in the workspace are added in a fixed order.  With the test switch
 * DK_NO_OFFSET_WGRAD16 (or DK_NO_OFFSET_PAIRS for float32) the fp32 matrix-instruction kernel serves stride 1
 * with 15, 16, 18 or 20 outputs.  A workspace query of 0 / DK_ERR_UNSUPPORTED: not covered, the caller keeps
 * its library's routine. */
size_t dk_offset_conv_backward_weight_workspace(const dk_offset_conv_desc *desc);
int dk_offset_conv_backward_weight(const dk_offset_conv_desc *desc, const void *out_grad, const void *input,
                                   void *weight_grad, void *workspace, size_t workspace_bytes,
                                   void *stream);

/* Gradient of that convolution's bias: bias_grad[o] = sum over images and pixels of
 * out_grad[n][o][.], any shape; fp32 sums, the images are added in a fixed order. */
size_t dk_offset_conv_backward_bias_workspace(const dk_offset_conv_desc *desc);
int dk_offset_conv_backward_bias(const dk_offset_conv_desc *desc, const void *out_grad, void *bias_grad,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* Gradient of that convolution's input (what autograd derives for the rotation_conv call at
 * modules/deform_kernel.py:214), input_grad [batch, in_channels, h, w] (fully written; float32 at stride 2:
 * 8-byte aligned), on planes 7, 14, 28, 56 or 112 wide (stride 2: input planes 14 .. 112 wide): the same
 * shift-GEMM kernel as the forward of such planes, arithmetic as described above.  Other shapes return
 * DK_ERR_UNSUPPORTED (the workspace query 0): the caller keeps its library's routine there.
 * dk_offset_conv_backward_input_worthwhile(): 1 where the kernel is also expected to be the faster choice
 * (float32 at stride 1: from 64 input channels on planes 14 wide and wider -- with fewer channels the second,
 * nearly empty chunk of the 18 output-gradient channels' pairs costs more than the library's kernel takes). */
int dk_offset_conv_backward_input_worthwhile(const dk_offset_conv_desc *desc);
size_t dk_offset_conv_backward_input_workspace(const dk_offset_conv_desc *desc);
int dk_offset_conv_backward_input(const dk_offset_conv_desc *desc, const void *out_grad, const void *weight,
                                  void *input_grad, void *workspace, size_t workspace_bytes, void *stream);

/* ---- depthwise convolution with one kernel per image and channel ------------- */

/* The convolution GlobalDeformKernel2d applies with the kernels it has sampled for every image:
 * nn.functional.conv2d(x.view(1, n * c, h, w), weight, stride, padding, dilation, groups = n * c)
 * for a depthwise layer (modules/deform_kernel.py:103-111, weight [n * c, 1, k, k] from
 * dynamic_weight, :68-101), and the two gradients the framework derives for that call.  The
 * reference uses the framework's grouped convolution there; a convolution with n * c groups of
 * one channel each is a streaming operation, and these entry points run it as one.
 *   input [batch, channel, in_h, in_w], weight [batch, channel, k_h, k_w] (= [n * c, 1, k_h, k_w]),
 *   output [batch, channel, out_h, out_w]; weight_strides: NULL for a contiguous weight (and
 *   weight_grad), or the four non-negative element strides of its (batch, channel, k_h, k_w) axes --
 *   the sampler leaves the kernels as [n * k_h * k_w, c] (nd_linear_sample's output, :92-96), which is
 *   strides {k_h * k_w * c, 1, k_w * c, c}, and the module's transpose + reshape (:97-101) is then
 *   not needed; desc: scope_h, scope_w, groups, rotation_clip are not
 *   used (scope >= 1 and groups = 1 keep the descriptor valid); any dk_dtype.
 * dk_image_depthwise_supported() tells whether the geometry is covered (a band of one output
 * row's taps must fit a wave's share of LDS, at most 128 taps); the calls return
 * DK_ERR_UNSUPPORTED otherwise and the caller keeps its library convolution.  No workspace;
 * every result is fully written; each kernel gradient is one wave's sum in a fixed order. */
int dk_image_depthwise_supported(const dk_conv_desc *desc);
int dk_image_depthwise_forward(const dk_conv_desc *desc, const void *input, const void *weight,
                               const int64_t *weight_strides, void *output, void *stream);
int dk_image_depthwise_backward_data(const dk_conv_desc *desc, const void *out_grad, const void *weight,
                                     const int64_t *weight_strides, void *in_grad, void *stream);
int dk_image_depthwise_backward_weight(const dk_conv_desc *desc, const void *out_grad, const void *input,
                                       void *weight_grad, const int64_t *weight_strides, void *stream);

/* ---- misc ------------------------------------------------------------------- */

const char *dk_status_string(int status);

/* Test hook, not for production use: a bit mask that makes the dispatch skip a specialised kernel
 * family and run the next more general one for the same shape, so that tests can reach every
 * kernel.  Bit i belongs to the i-th of DK_NO_ROWS, DK_NO_MFMA, DK_NO_MFMA_S2, DK_NO_S2_QUADS,
 * DK_NO_DEFORM_FAST, DK_NO_DEFORM_CH, DK_NO_DEFORM_CH_BIG, DK_NO_DEFORM_MFMA, DK_NO_ND_BINS,
 * DK_NO_ND_MFMA, DK_NO_GATHER_MFMA, DK_NO_FILTER_SPLIT, DK_NO_IMAGE_FLAT, DK_NO_ND_SMALL, DK_NO_NHWC_MFMA,
 * DK_FORCE_GATHER_MFMA, DK_NO_PIXEL_LANES, DK_FORCE_PIXEL_LANES, DK_NO_OFFSET_PAIRS, DK_NO_OFFSET_WGRAD16, DK_NO_DEFORM_WINDOW, DK_FORCE_WIN2, DK_NO_NHWC_STAGED,
 * DK_FORCE_NHWC_GATHER_MFMA, DK_NO_IMAGE_PACKED.  The mask starts at 0; only a process
 * started with DK_ENABLE_TEST_SWITCHES=1 in its environment also reads the environment variables of
 * those names, once, at the first call that consults the mask (a stray variable in a production
 * environment changes nothing).  This call replaces the mask and returns the previous one.
 * Workspace queries consult it too: query and call must see the same mask.  The one piece of
 * process-wide state in the library. */
unsigned dk_test_switches(unsigned mask);

/* Library version, (major << 16) | minor.  The minor number goes up whenever a descriptor struct
 * changes (0.3: dk_conv_desc has `layout`, the *_desc_size() queries exist). */
int dk_version(void);

/* sizeof() of the descriptor structs as the library was compiled.  A binding that declares the
 * structs on its own (ctypes, cgo, JNI) compares these with its own declaration once, at load time:
 * a descriptor that is shorter than the library's is read past its end.  No counterpart in the
 * reference, whose pybind functions take the eleven ints one by one
 * (csrc/filter_sample_depthwise_cuda.cpp:540-569). */
size_t dk_conv_desc_size(void);
size_t dk_nd_desc_size(void);
size_t dk_offset_conv_desc_size(void);

#ifdef __cplusplus
}
#endif
#endif /* DK_HIP_H */
