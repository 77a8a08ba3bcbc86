// Internal interface between the C-ABI layer (dk_api.hip) and the kernel
// translation units.  Every `fast_*` function returns false, launching
// nothing, when the geometry is outside what the tuned kernels cover; the
// caller then uses the `generic_*` kernels, which take any geometry and dtype.
#pragma once

#include "dk_common.h"

#include <cstdlib>

namespace dk {

// Test switches: each bit makes the dispatch skip a specialised kernel family and take the next
// more general one, so that every kernel can be reached for the same shape.  The mask is read from
// the environment once, at the first call that looks at it (a variable DK_NO_ROWS, DK_NO_MFMA, ...
// set to anything sets its bit), and can be replaced at run time with dk_test_switches(); the
// dispatch only loads one word per call.
enum TestSwitch : unsigned {
  kNoRows = 1u << 0,        // DK_NO_ROWS         the "same-width" and stride-2 row kernels (and with them the matrix-core grad filter)
  kNoMfma = 1u << 1,        // DK_NO_MFMA         the matrix-core grad filter (the dense register form runs instead)
  kNoMfmaS2 = 1u << 2,      // DK_NO_MFMA_S2      its stride-2 form
  kNoS2Quads = 1u << 3,     // DK_NO_S2_QUADS     the stride-2 grad input over 2 x 2 input quads
  kNoDeformFast = 1u << 4,  // DK_NO_DEFORM_FAST  the tuned deformable kernels (the generic ones run instead)
  kNoDeformCh = 1u << 5,    // DK_NO_DEFORM_CH    their channel-interleaved forms
  kNoDeformChBig = 1u << 6, // DK_NO_DEFORM_CH_BIG  only the 1024-thread channel-interleaved form
  kNoDeformMfma = 1u << 7,  // DK_NO_DEFORM_MFMA  the matrix-core deformable grad filter
  kNoNdBins = 1u << 8,      // DK_NO_ND_BINS      the N-d kernels that sort the points by cell
  kNoNdMfma = 1u << 9,      // DK_NO_ND_MFMA      the matrix-core N-d kernels
  kNoGatherMfma = 1u << 10, // DK_NO_GATHER_MFMA  the matrix-core forward / grad input (the row kernels run instead)
  kNoFilterSplit = 1u << 11, // DK_NO_FILTER_SPLIT the bfloat16-pair form of the float32 matrix-core grad filter (fp32 matrix instructions instead)
  kNoNdSmall = 1u << 13,    // DK_NO_ND_SMALL     the few-points-on-a-tiny-volume path of the N-d sampler
  kNoNhwcMfma = 1u << 14,   // DK_NO_NHWC_MFMA    the matrix-core grad filter / grad rotation of the channels-last operator
  kForceGatherMfma = 1u << 15,  // DK_FORCE_GATHER_MFMA  the matrix-core forward / grad input wherever it applies, not only where it is the faster kernel
  kNoImageFlat = 1u << 12,  // DK_NO_IMAGE_FLAT   the flat-copy kernels of the per-image depthwise convolution (the band kernels run instead)
  kNoPixelLanes = 1u << 16,     // DK_NO_PIXEL_LANES     the forward / grad input with the pixels on the matrix instruction's lanes
  kForcePixelLanes = 1u << 17,  // DK_FORCE_PIXEL_LANES  ... wherever it applies, not only where it is the faster kernel
  kNoOffsetWgrad16 = 1u << 19,  // DK_NO_OFFSET_WGRAD16  the offset branch's weight gradient on 16-bit matrix instructions (the fp32 matrix-instruction kernel at stride 1, nothing at stride 2)
  kNoDeformWindow = 1u << 20,   // DK_NO_DEFORM_WINDOW   the row-window form of the matrix-core deformable grad filter (the dense register kernel runs instead)
  kForceWin2 = 1u << 21,        // DK_FORCE_WIN2         the rows-and-columns window form of that grad filter also where the row-window form applies
  kNoNhwcStaged = 1u << 22,     // DK_NO_NHWC_STAGED     the channels-last kernels that stage planar tiles in LDS / contract 32 channels per matrix instruction (the kernels named under DK_NO_NHWC_MFMA run instead)
  kForceNhwcGatherMfma = 1u << 23,  // DK_FORCE_NHWC_GATHER_MFMA  the channels-last matrix-core forward / grad input wherever it applies, not only where it is the faster kernel
  kNoImagePacked = 1u << 24,    // DK_NO_IMAGE_PACKED    the packed flat-copy kernels of the per-image depthwise convolution on 16-bit tensors (the flat-copy kernels that unpack to fp32 run instead)
  kNoOffsetPairs = 1u << 18,    // DK_NO_OFFSET_PAIRS    the offset branch's convolution on float32 tensors as bfloat16 pairs (the fp32 matrix-instruction forward runs instead, the other passes are not offered)
};
unsigned test_switches();  // dk_api.hip
inline bool path_disabled(unsigned sw) { return (test_switches() & sw) != 0; }

// hipFuncAttributeMaxDynamicSharedMemorySize belongs to (kernel, device) and does not change once
// set: the first launch of a kernel on a device sets it, later launches only look it up.
bool allow_max_dynamic_lds(const void* kernel);  // dk_api.hip
// The same with a given bound, for kernels whose static LDS arrays leave less room (the bound is only
// ever raised).
bool allow_dynamic_lds(const void* kernel, int bytes);

// Upper bound handed to hipFuncAttributeMaxDynamicSharedMemorySize for the kernels that need more
// than 64 KB of LDS: the attribute is per kernel, not per launch, so a launch must not lower what a
// concurrent one (another host thread, another shape) relies on.  A gfx950 CU has 160 KB of LDS;
// the kernels' small static arrays come out of the same budget, so the bound stays 8 KB below.
constexpr int kMaxDynamicLds = 152 * 1024;

template <typename CT, typename T>
void launch_reduce_partials(const CT* partial, int parts, long count, T* out, hipStream_t stream);

// ---- forward / grad input on the matrix cores (dk_local_mfma.hip): same-width geometries, scope <= 16 cells
template <typename T>
bool mfma_local_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                       hipStream_t stream);

// ---- forward / grad input with the pixels on the lanes of the matrix instruction (dk_local_lanes.hip): same-width
//      geometries, scope <= 16 cells; no LDS staging of the source tensor
template <typename T>
bool lanes_local_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                        hipStream_t stream);

// ---- tuned local path (dk_local_fast.hip): 3x3 taps, scope 3x3 / 4x4 / 5x5, fp32/fp16/bf16
template <typename T>
bool fast_local_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter,
                       T* dst, hipStream_t stream);
size_t fast_local_grad_rotation_workspace(const Geo& g);
template <typename T>
bool fast_local_grad_rotation(const Geo& g, const T* gout, const T* x, const T* rot,
                              const T* filter, T* grot, void* ws, hipStream_t stream);
size_t fast_local_grad_filter_workspace(const Geo& g);
template <typename T>
bool fast_local_grad_filter(const Geo& g, const T* gout, const T* x, const T* rot, T* gfilter,
                            void* ws, hipStream_t stream);

// ---- tuned deformable path (dk_deform_fast.hip): 3x3 taps, scope 3x3 / 4x4 / 5x5, fp32/fp16/bf16,
//      input planes at most 64 columns wide that fit LDS
template <typename T>
bool fast_deform_forward(const Geo& g, const T* x, const T* off, const T* rot, const T* filter, T* out,
                         hipStream_t stream);
size_t fast_deform_grad_input_workspace(const Geo& g);
template <typename T>
bool fast_deform_grad_input(const Geo& g, const T* gout, const T* off, const T* rot, const T* filter, T* gin,
                            void* ws, hipStream_t stream);
// rotation = false: gradient w.r.t. the image-space offsets
size_t fast_deform_grad_coord_workspace(const Geo& g, bool rotation);
template <typename T>
bool fast_deform_grad_coord(const Geo& g, bool rotation, const T* gout, const T* x, const T* off, const T* rot,
                            const T* filter, T* result, void* ws, hipStream_t stream);
// both coordinate gradients from one pass over the input; 0 / false where only the separate kernels apply
size_t fast_deform_grad_coords_workspace(const Geo& g);
template <typename T>
bool fast_deform_grad_coords(const Geo& g, const T* gout, const T* x, const T* off, const T* rot, const T* filter,
                             T* goff, T* grot, void* ws, hipStream_t stream);
size_t fast_deform_grad_filter_workspace(const Geo& g);
template <typename T>
bool fast_deform_grad_filter(const Geo& g, const T* gout, const T* x, const T* off, const T* rot, T* gfilter,
                             void* ws, hipStream_t stream);

// ---- generic path (dk_generic.hip): any geometry, all four dtypes, local and deformable
template <typename T>
void generic_forward(const Geo& g, bool deform, const T* x, const T* off, const T* rot,
                     const T* filter, T* out, hipStream_t stream);
template <typename T>
void generic_local_grad_input(const Geo& g, const T* gout, const T* rot, const T* filter, T* gin,
                              hipStream_t stream);
size_t generic_deform_grad_input_workspace(const Geo& g, int dtype);
template <typename T>
void generic_deform_grad_input(const Geo& g, const T* gout, const T* off, const T* rot,
                               const T* filter, T* gin, void* ws, hipStream_t stream);
template <typename T>
void generic_grad_rotation(const Geo& g, bool deform, const T* gout, const T* x, const T* off,
                           const T* rot, const T* filter, T* grot, hipStream_t stream);
template <typename T>
void generic_grad_offset(const Geo& g, const T* gout, const T* x, const T* off, const T* rot,
                         const T* filter, T* goff, hipStream_t stream);
size_t generic_grad_filter_workspace(const Geo& g, int dtype);
template <typename T>
void generic_grad_filter(const Geo& g, bool deform, const T* gout, const T* x, const T* off,
                         const T* rot, T* gfilter, void* ws, hipStream_t stream);

// dk_offset_conv.hip: the 3x3 offset-branch convolution (stride 1, padding 1; fp32 / fp16 / bf16 tensors, fp32 arithmetic)
bool offset_conv_supported(int cin, int cout, int h, int w);
bool offset_conv_worthwhile(int batch, int cin, int cout, int h, int w);
size_t offset_conv_workspace(int batch, int cin, int cout, int h, int w);
size_t offset_conv_bias_grad_workspace(int batch, int cout);
template <typename T>
void offset_conv_bias_grad(int batch, int cout, int plane, const T* gout, T* gbias, void* ws, hipStream_t stream);
size_t offset_conv_wgrad_workspace(int batch, int cin, int cout, int h, int w);
template <typename T>
bool offset_conv_wgrad(int batch, int cin, int cout, int h, int w, const T* x, const T* gout, T* gweight, void* ws,
                       hipStream_t stream);
template <typename T>
bool offset_conv_forward(int batch, int cin, int cout, int h, int w, const T* x, const T* weight, const T* bias, T* out,
                         void* ws, hipStream_t stream);

// dk_offset_conv16.hip: forward and input gradient of the same convolution on 16-bit matrix instructions
// (fp16 / bf16 tensors, planes 7 / 14 / 28 / 56 / 112 wide, at most 32 output channels)
bool offset_conv16_supported(int cin, int cout, int h, int w);
size_t offset_conv16_workspace(int batch, int cin, int cout, int h, int w, bool pairs = false);  // pairs: float32 tensors
template <typename T>
bool offset_conv16_forward(int batch, int cin, int cout, int h, int w, const T* x, const T* weight, const T* bias,
                           T* out, void* ws, hipStream_t stream);
template <typename T>
bool offset_conv16_backward_input(int batch, int cin, int cout, int h, int w, const T* gout, const T* weight, T* gin,
                                  void* ws, hipStream_t stream);

// ... and its forward with stride 2 (input planes 14 / 28 / 56 / 112 wide; h, w: the input plane)
bool offset_conv16_s2_supported(int cin, int cout, int h, int w);
size_t offset_conv16_s2_workspace(int batch, int cin, int cout, int h, int w, bool pairs = false);
template <typename T>
bool offset_conv16_s2_forward(int batch, int cin, int cout, int h, int w, const T* x, const T* weight, const T* bias,
                              T* out, void* ws, hipStream_t stream);
size_t offset_conv16_s2_backward_input_workspace(int cin, int cout, bool pairs = false);
template <typename T>
bool offset_conv16_s2_backward_input(int batch, int cin, int cout, int h, int w, const T* gout, const T* weight,
                                     T* gin, void* ws, hipStream_t stream);

// dk_offset_wgrad16.hip: the weight gradient of that convolution on 16-bit matrix instructions, stride 1 (planes
// 7 .. 112 wide) and 2 (input planes 14 .. 112 wide), up to 20 outputs, input channels a multiple of 16; float32
// tensors as bfloat16 pairs.  h, w: the input plane.  Workspace 0: not covered.
bool offset_wgrad16_supported(int cin, int cout, int h, int w, int stride);
size_t offset_wgrad16_workspace(int batch, int cin, int cout, int h, int w, int stride, bool pairs);
template <typename T>
bool offset_wgrad16(int batch, int cin, int cout, int h, int w, int stride, const T* x, const T* gout, T* gweight,
                    void* ws, hipStream_t stream);

// dk_local_fast.hip: the matrix-core grad filter on channels-last tensors (false / workspace 0: not covered)
size_t fast_local_grad_filter_cl_workspace(const Geo& g);
template <typename T>
bool fast_local_grad_filter_cl(const Geo& g, const T* gout, const T* x, const T* rot, T* gfilter, void* ws,
                               hipStream_t stream);

// dk_local_nhwc.hip: the local operator on channels-last tensors, all dtypes, any geometry whose tables fit LDS
bool nhwc_supported(const Geo& g, int dtype);
template <typename T>
void nhwc_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                 hipStream_t stream);
size_t nhwc_grad_rotation_workspace(const Geo& g, int dtype);
template <typename T>
void nhwc_grad_rotation(const Geo& g, const T* gout, const T* x, const T* rot, const T* filter, T* grot, void* ws,
                        hipStream_t stream);
size_t nhwc_grad_filter_workspace(const Geo& g, int dtype);
template <typename T>
void nhwc_grad_filter(const Geo& g, const T* gout, const T* x, const T* rot, T* gfilter, void* ws,
                      hipStream_t stream);

// dk_image_conv.hip: depthwise convolution with one kernel per (image, channel) plane, all dtypes
bool image_conv_supported(const Geo& g, int dtype);
// wstrides: element strides of the kernel tensor's (image, channel, tap row, tap column) axes, or null
// for a contiguous [N, C, k_h, k_w] tensor
template <typename T>
bool image_conv_forward(const Geo& g, const long* wstrides, const T* x, const T* weight, T* out, hipStream_t stream);
template <typename T>
bool image_conv_grad_input(const Geo& g, const long* wstrides, const T* gout, const T* weight, T* gin,
                           hipStream_t stream);
template <typename T>
bool image_conv_grad_weight(const Geo& g, const long* wstrides, const T* gout, const T* x, T* gweight,
                            hipStream_t stream);

}  // namespace dk
