// Internal interface of the N-d linear sample kernels (dk_nd.hip).
#pragma once

#include "dk_common.h"

namespace dk {

// bytes of workspace for the channel-last copy of `data` (0 when the direct path is used)
size_t nd_data_cl_workspace(const dk_nd_desc& d);
template <typename T>
void nd_forward(const dk_nd_desc& d, const T* data, const T* coord, T* out, void* ws,
                hipStream_t stream);
size_t nd_grad_data_workspace(const dk_nd_desc& d);
template <typename T>
void nd_grad_data(const dk_nd_desc& d, const T* gout, const T* coord, T* gdata, void* ws,
                  hipStream_t stream);
template <typename T>
void nd_grad_coord(const dk_nd_desc& d, const T* gout, const T* data, const T* coord, T* gcoord,
                   void* ws, hipStream_t stream);

}  // namespace dk
