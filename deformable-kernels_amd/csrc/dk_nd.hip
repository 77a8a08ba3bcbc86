// N-d linear sample: out[b, c] = multilinear(data[c], coord[b]), zero outside.
//
// ND.cu = deformable_kernels/ops/deform_kernel/csrc/nd_linear_sample_cuda_kernel.cu
//   nd_linear ND.cu:45-88, nd_linear_backward_data ND.cu:90-131,
//   nd_linear_backward_coord ND.cu:133-177; kernels ND.cu:183-287.
//
// The per-point work (which 2^n corners exist and with what weight) does not
// depend on the channel, so each lane derives it once from its point and then
// only multiplies and adds per corner.  The coordinate gradient is reduced over
// channels inside the kernel (one wave per point, lanes over channels, shuffle
// reduction) instead of materialising the reference's [B, n, C] intermediate.
#include "dk_nd.h"

namespace dk {

namespace {

constexpr int kBlock = 256;

struct NdGeo {
  long batch;
  int channel, dims;
  long prod_shape;
  int shape[DK_ND_MAX_DIMS];
};

// Per-point corner bookkeeping: low index and fractional weight per dimension,
// and whether the whole sample is void (any x <= -1 or x >= s, ND.cu:47-53).
template <typename CT>
struct NdPoint {
  int low[DK_ND_MAX_DIMS];
  CT frac[DK_ND_MAX_DIMS];
  bool inside;
};

template <typename T, typename CT>
__device__ __forceinline__ NdPoint<CT> load_point(const NdGeo& g, const T* coord_b) {
  NdPoint<CT> p;
  p.inside = true;
#pragma unroll
  for (int d = 0; d < DK_ND_MAX_DIMS; ++d) {
    if (d < g.dims) {
      const CT x = ld(coord_b + d);
      const CT xf = floor(x);
      if (!(x > CT(-1) && x < CT(g.shape[d]))) p.inside = false;
      p.low[d] = (x > CT(-1) && x < CT(g.shape[d])) ? (int)xf : 0;
      p.frac[d] = x - xf;
    } else {
      p.low[d] = 0;
      p.frac[d] = CT(0);
    }
  }
  return p;
}

// Offset and weight of corner `i` (bit d selects low/high in dimension d,
// ND.cu:67); `skip_dim` >= 0 replaces that dimension's weight by -1 / +1
// (ND.cu:161,165).  Returns false where the reference breaks out of the corner.
template <typename CT>
__device__ __forceinline__ bool corner(const NdGeo& g, const NdPoint<CT>& p, unsigned i,
                                       int skip_dim, long& offset, CT& weight) {
  offset = 0;
  weight = CT(1);
#pragma unroll
  for (int d = 0; d < DK_ND_MAX_DIMS; ++d) {
    if (d < g.dims) {
      const int s = g.shape[d];
      offset *= s;
      const unsigned hi = (i >> d) & 1u;
      if (hi == 0 && p.low[d] >= 0) {
        offset += p.low[d];
        weight *= (d == skip_dim) ? CT(-1) : CT(1) - p.frac[d];
      } else if (hi == 1 && p.low[d] + 1 <= s - 1) {
        offset += p.low[d] + 1;
        weight *= (d == skip_dim) ? CT(1) : p.frac[d];
      } else {
        return false;
      }
    }
  }
  return true;
}

// forward, ND.cu:183-201: one thread per (b, c), c fastest.
template <typename T>
__global__ __launch_bounds__(kBlock) void nd_forward_kernel(NdGeo g, const T* __restrict__ data,
                                                            const T* __restrict__ coord,
                                                            T* __restrict__ out, long total) {
  using CT = compute_t<T>;
  for (long id = (long)blockIdx.x * kBlock + threadIdx.x; id < total; id += (long)gridDim.x * kBlock) {
    const int c = (int)(id % g.channel);
    const long b = id / g.channel;
    const NdPoint<CT> p = load_point<T, CT>(g, coord + b * g.dims);
    CT val = 0;
    if (p.inside) {
      const T* dc = data + (size_t)c * g.prod_shape;
      for (unsigned i = 0; i < (1u << g.dims); ++i) {
        long o;
        CT w;
        if (corner<CT>(g, p, i, -1, o, w)) val += w * ld(dc + o);
      }
    }
    st(out + id, val);
  }
}

// grad data, ND.cu:225-243: scatter with hardware float atomics into a zeroed buffer.
template <typename T, typename CT>
__global__ __launch_bounds__(kBlock) void nd_grad_data_kernel(NdGeo g, const T* __restrict__ gout,
                                                              const T* __restrict__ coord,
                                                              CT* __restrict__ gdata, long total) {
  for (long id = (long)blockIdx.x * kBlock + threadIdx.x; id < total; id += (long)gridDim.x * kBlock) {
    const int c = (int)(id % g.channel);
    const long b = id / g.channel;
    const NdPoint<CT> p = load_point<T, CT>(g, coord + b * g.dims);
    if (!p.inside) continue;
    const CT go = ld(gout + id);
    CT* dc = gdata + (size_t)c * g.prod_shape;
    for (unsigned i = 0; i < (1u << g.dims); ++i) {
      long o;
      CT w;
      if (corner<CT>(g, p, i, -1, o, w)) atomicAdd(dc + o, w * go);
    }
  }
}

// grad coord, ND.cu:267-287 + the caller's sum over channels: one wave per point.
template <typename T>
__global__ __launch_bounds__(kBlock) void nd_grad_coord_kernel(NdGeo g, const T* __restrict__ gout,
                                                               const T* __restrict__ data,
                                                               const T* __restrict__ coord,
                                                               T* __restrict__ gcoord) {
  using CT = compute_t<T>;
  const int lane = threadIdx.x & 63;
  const long waves = (long)gridDim.x * (kBlock / 64);
  for (long b = (long)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6); b < g.batch; b += waves) {
    const NdPoint<CT> p = load_point<T, CT>(g, coord + b * g.dims);
    CT acc[DK_ND_MAX_DIMS];
#pragma unroll
    for (int d = 0; d < DK_ND_MAX_DIMS; ++d) acc[d] = CT(0);
    if (p.inside) {
      for (int c = lane; c < g.channel; c += 64) {
        const CT go = ld(gout + b * g.channel + c);
        const T* dc = data + (size_t)c * g.prod_shape;
        for (unsigned i = 0; i < (1u << g.dims); ++i) {
          // the corner exists for every gdim or for none: its range tests do not depend on gdim
          long o;
          CT w;
          if (!corner<CT>(g, p, i, -1, o, w)) continue;
          const CT dv = go * ld(dc + o);
#pragma unroll
          for (int d = 0; d < DK_ND_MAX_DIMS; ++d) {
            if (d < g.dims) {
              long o2;
              CT w2;
              corner<CT>(g, p, i, d, o2, w2);
              acc[d] += dv * w2;
            }
          }
        }
      }
    }
#pragma unroll
    for (int d = 0; d < DK_ND_MAX_DIMS; ++d) {
      if (d < g.dims) {
        CT v = acc[d];
        for (int sft = 32; sft > 0; sft >>= 1) v += __shfl_xor(v, sft, 64);
        if (lane == 0) st(gcoord + b * g.dims + d, v);
      }
    }
  }
}

template <typename CT>
__global__ void nd_fill_zero_kernel(CT* p, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    p[i] = CT(0);
}
template <typename CT, typename T>
__global__ void nd_convert_kernel(const CT* __restrict__ a, T* __restrict__ out, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    st(out + i, a[i]);
}

inline int grid_for(long total) {
  long b = (total + kBlock - 1) / kBlock;
  if (b > 1048576) b = 1048576;
  if (b < 1) b = 1;
  return (int)b;
}

NdGeo make_geo(const dk_nd_desc& d) {
  NdGeo g;
  g.batch = d.batch;
  g.channel = d.channel;
  g.dims = d.dims;
  g.prod_shape = 1;
  for (int i = 0; i < DK_ND_MAX_DIMS; ++i) {
    g.shape[i] = i < d.dims ? d.shape[i] : 1;
    if (i < d.dims) g.prod_shape *= d.shape[i];
  }
  return g;
}

}  // namespace

template <typename T>
void nd_forward(const dk_nd_desc& d, const T* data, const T* coord, T* out, hipStream_t stream) {
  const NdGeo g = make_geo(d);
  const long total = g.batch * g.channel;
  nd_forward_kernel<T><<<grid_for(total), kBlock, 0, stream>>>(g, data, coord, out, total);
}

size_t nd_grad_data_workspace(const dk_nd_desc& d) {
  if (d.dtype != DK_F16 && d.dtype != DK_BF16) return 0;
  size_t n = (size_t)d.channel;
  for (int i = 0; i < d.dims; ++i) n *= (size_t)d.shape[i];
  return n * sizeof(float);
}

template <typename T>
void nd_grad_data(const dk_nd_desc& d, const T* gout, const T* coord, T* gdata, void* ws,
                  hipStream_t stream) {
  using CT = compute_t<T>;
  const NdGeo g = make_geo(d);
  const long n_data = (long)g.channel * g.prod_shape;
  const long total = g.batch * g.channel;
  constexpr bool direct = sizeof(T) == sizeof(CT);
  CT* acc = direct ? reinterpret_cast<CT*>(gdata) : static_cast<CT*>(ws);
  nd_fill_zero_kernel<CT><<<grid_for(n_data), kBlock, 0, stream>>>(acc, n_data);
  if (total > 0)
    nd_grad_data_kernel<T, CT><<<grid_for(total), kBlock, 0, stream>>>(g, gout, coord, acc, total);
  if (!direct) nd_convert_kernel<CT, T><<<grid_for(n_data), kBlock, 0, stream>>>(acc, gdata, n_data);
}

template <typename T>
void nd_grad_coord(const dk_nd_desc& d, const T* gout, const T* data, const T* coord, T* gcoord,
                   hipStream_t stream) {
  const NdGeo g = make_geo(d);
  long blocks = (g.batch + 3) / 4;
  if (blocks > 65536) blocks = 65536;
  nd_grad_coord_kernel<T><<<(int)blocks, kBlock, 0, stream>>>(g, gout, data, coord, gcoord);
}

#define DK_INSTANTIATE(T)                                                                      \
  template void nd_forward<T>(const dk_nd_desc&, const T*, const T*, T*, hipStream_t);          \
  template void nd_grad_data<T>(const dk_nd_desc&, const T*, const T*, T*, void*, hipStream_t); \
  template void nd_grad_coord<T>(const dk_nd_desc&, const T*, const T*, const T*, T*, hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(double)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
#undef DK_INSTANTIATE

}  // namespace dk
