// Internal interface between the C-ABI layer (dk_api.hip) and the kernel
// translation units.  Every `fast_*` function returns false, launching
// nothing, when the geometry is outside what the tuned kernels cover; the
// caller then uses the `generic_*` kernels, which take any geometry and dtype.
#pragma once

#include "dk_common.h"

#include <cstdlib>

namespace dk {

// Test switches.  Setting one of these environment variables (to anything) makes the dispatch
// skip a specialised kernel family and take the next more general one, so that every kernel can
// be reached for the same shape:
//   DK_NO_ROWS         the "same-width" row kernels (and with them the matrix-core grad filter)
//   DK_NO_MFMA         the matrix-core grad filter (the dense register form runs instead)
//   DK_NO_DEFORM_FAST  the tuned deformable kernels (the generic ones run instead)
// Read at every call, so a test can toggle them inside one process.
inline bool path_disabled(const char* name) { return std::getenv(name) != nullptr; }

// Upper bound handed to hipFuncAttributeMaxDynamicSharedMemorySize for the kernels that need more
// than 64 KB of LDS: the attribute is per kernel, not per launch, so a launch must not lower what a
// concurrent one (another host thread, another shape) relies on.  A gfx950 CU has 160 KB of LDS;
// the kernels' small static arrays come out of the same budget, so the bound stays 8 KB below.
constexpr int kMaxDynamicLds = 152 * 1024;

template <typename CT, typename T>
void launch_reduce_partials(const CT* partial, int parts, long count, T* out, hipStream_t stream);

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

// dk_offset_conv.hip: the 3x3 offset-branch convolution (stride 1, padding 1, fp32)
bool offset_conv_supported(int cin, int cout, int h, int w);
bool offset_conv_worthwhile(int batch, int cin, int cout, int h, int w);
size_t offset_conv_workspace(int batch, int cin, int cout, int h, int w);
size_t offset_conv_bias_grad_workspace(int batch, int cout);
void offset_conv_bias_grad(int batch, int cout, int plane, const float* gout, float* gbias, void* ws,
                           hipStream_t stream);
size_t offset_conv_wgrad_workspace(int batch, int cin, int cout, int h, int w);
bool offset_conv_wgrad(int batch, int cin, int cout, int h, int w, const float* x, const float* gout, float* gweight,
                       void* ws, hipStream_t stream);
bool offset_conv_forward(int batch, int cin, int cout, int h, int w, const float* x, const float* weight,
                         const float* bias, float* out, void* ws, hipStream_t stream);

}  // namespace dk
