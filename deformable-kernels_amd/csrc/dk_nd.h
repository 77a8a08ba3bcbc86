// Internal interface of the N-d linear sample kernels (dk_nd.hip).
#pragma once

#include "dk_common.h"

namespace dk {

// bytes of workspace for the channel-last copy of `data` (0 when the direct path is used)
size_t nd_data_cl_workspace(const dk_nd_desc& d);
template <typename T>
void nd_forward(const dk_nd_desc& d, const T* data, const T* coord, T* out, void* ws, const int* order,
                hipStream_t stream);
size_t nd_grad_data_workspace(const dk_nd_desc& d);
template <typename T>
void nd_grad_data(const dk_nd_desc& d, const T* gout, const T* coord, T* gdata, void* ws, const int* order,
                  hipStream_t stream);
template <typename T>
void nd_grad_coord(const dk_nd_desc& d, const T* gout, const T* data, const T* coord, T* gcoord,
                   void* ws, const int* order, hipStream_t stream);
// the points' order by cell (0 bytes when the call's kernels do not sort), to be computed once and
// handed to the three calls above
size_t nd_order_bytes(const dk_nd_desc& d);
size_t nd_sort_workspace(const dk_nd_desc& d);
template <typename T>
void nd_order(const dk_nd_desc& d, const T* coord, int* order, void* ws, hipStream_t stream);

}  // namespace dk
