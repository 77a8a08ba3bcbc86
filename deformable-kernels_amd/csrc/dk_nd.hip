// N-d linear sample: out[b, c] = multilinear(data[c], coord[b]), zero outside.
//
// ND.cu = deformable_kernels/ops/deform_kernel/csrc/nd_linear_sample_cuda_kernel.cu
//   nd_linear ND.cu:45-88, nd_linear_backward_data ND.cu:90-131,
//   nd_linear_backward_coord ND.cu:133-177; kernels ND.cu:183-287.
//
// Two paths.
//  * Channel-last path (1..3 sampling dimensions, enough work to pay for a transpose):
//    `data` [C, P] is first copied to [P, C] in the caller's workspace, so the C values of
//    one corner are contiguous.  A wave takes 64 points: with lane <-> point it derives each
//    point's 2^n corner offsets and weights once, then walks its points with lane <-> channel,
//    broadcasting the point's corners by readlane; every corner read and every output row
//    is one contiguous run.  The reference maps adjacent threads to adjacent channels whose
//    data lie a whole volume apart (ND.cu:197-199).
//  * Direct path (any dimension count, small problems): one lane per (point, channel).
// The coordinate gradient is reduced over channels inside the kernel instead of
// materialising the reference's [B, n, C] intermediate (ND.cu:281-286 and the caller's sum).

#include "dk_kernels.h"
#include "dk_nd.h"

namespace dk {

namespace {

constexpr int kBlock = 256;
constexpr int kClMaxDims = 3;
constexpr int kClCorners = 1 << kClMaxDims;

struct NdGeo {
  long batch;
  int channel, dims;
  long prod_shape;
  int shape[DK_ND_MAX_DIMS];
};

// ---------------------------------------------------------------------------
// per-point corner bookkeeping shared by both paths
// ---------------------------------------------------------------------------
template <typename CT>
struct NdPoint {
  int low[DK_ND_MAX_DIMS];
  CT frac[DK_ND_MAX_DIMS];
  bool inside;  // false: some x <= -1 or x >= s, the whole sample is zero (ND.cu:47-53)
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
      const bool in = x > CT(-1) && x < CT(g.shape[d]);
      if (!in) p.inside = false;
      p.low[d] = in ? (int)xf : 0;
      p.frac[d] = x - xf;
    } else {
      p.low[d] = 0;
      p.frac[d] = CT(0);
    }
  }
  return p;
}

// Offset and weight of corner `i` (bit d selects low/high in dimension d, ND.cu:67);
// `skip_dim` >= 0 replaces that dimension's weight by -1 / +1 (ND.cu:161,165).
// Returns false where the reference breaks out of the corner.
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

// ---------------------------------------------------------------------------
// direct path
// ---------------------------------------------------------------------------
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

// scatter with hardware float atomics into a zeroed buffer laid out [C][P] (cl = false) or
// [P][C] (cl = true)
template <typename T, typename CT, bool CL>
__global__ __launch_bounds__(kBlock) void nd_grad_data_kernel(NdGeo g, const T* __restrict__ gout,
                                                              const T* __restrict__ coord,
                                                              CT* __restrict__ gdata, long total) {
  for (long id = (long)blockIdx.x * kBlock + threadIdx.x; id < total; id += (long)gridDim.x * kBlock) {
    const int c = (int)(id % g.channel);
    const long b = id / g.channel;
    const NdPoint<CT> p = load_point<T, CT>(g, coord + b * g.dims);
    if (!p.inside) continue;
    const CT go = ld(gout + id);
    for (unsigned i = 0; i < (1u << g.dims); ++i) {
      long o;
      CT w;
      if (corner<CT>(g, p, i, -1, o, w))
        atomicAdd(CL ? gdata + (size_t)o * g.channel + c : gdata + (size_t)c * g.prod_shape + o, w * go);
    }
  }
}

// one wave per point, lanes over channels, shuffle reduction
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
          // a corner exists for every differentiated dimension or for none
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

// ---------------------------------------------------------------------------
// channel-last path
// ---------------------------------------------------------------------------

// in [rows][cols] -> out [cols][rows], converting A -> B; 32 x 32 tiles through LDS
template <typename A, typename B>
__global__ __launch_bounds__(256) void nd_transpose_kernel(const A* __restrict__ in, B* __restrict__ out,
                                                           long rows, long cols) {
  __shared__ float tile[32][33];
  const long r0 = (long)blockIdx.y * 32, c0 = (long)blockIdx.x * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
  for (int k = 0; k < 32; k += 8) {
    const long r = r0 + ty + k, c = c0 + tx;
    tile[ty + k][tx] = (r < rows && c < cols) ? static_cast<float>(ld(in + r * cols + c)) : 0.f;
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 32; k += 8) {
    const long c = c0 + ty + k, r = r0 + tx;
    if (r < rows && c < cols) st(out + c * rows + r, tile[tx][ty + k]);
  }
}

// Corner offsets (in units of C elements of the channel-last copy) and weights of one
// point, padded to kClCorners; absent corners get weight 0 at offset 0.
struct ClCorners {
  int off[kClCorners];
  float w[kClCorners];
  unsigned present;  // bit i: corner i lies inside the volume (its weight may still be 0)
};

template <typename T>
__device__ __forceinline__ ClCorners cl_corners(const NdGeo& g, const T* coord, long b, bool valid) {
  ClCorners cc;
  cc.present = 0u;
  NdPoint<float> p;
  p.inside = false;
  if (valid) p = load_point<T, float>(g, coord + b * g.dims);
#pragma unroll
  for (int i = 0; i < kClCorners; ++i) {
    long o = 0;
    float w = 0.f;
    const bool ok = valid && p.inside && i < (1 << g.dims) && corner<float>(g, p, (unsigned)i, -1, o, w);
    cc.off[i] = ok ? (int)o : 0;
    cc.w[i] = ok ? w : 0.f;
    cc.present |= ok ? (1u << i) : 0u;
  }
  return cc;
}

// forward: a wave owns `ppw` (a power of two <= 64) consecutive points and walks them four at a
// time so that the corner reads of four points are in flight together
template <typename T>
__global__ __launch_bounds__(kBlock) void nd_forward_cl_kernel(NdGeo g, const T* __restrict__ data_cl,
                                                               const T* __restrict__ coord,
                                                               T* __restrict__ out, int ppw) {
  const int lane = threadIdx.x & 63;
  const long wave0 = ((long)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6)) * ppw;
  if (wave0 >= g.batch) return;
  const int npts = (int)min((long)ppw, g.batch - wave0);
  const ClCorners mine = cl_corners<T>(g, coord, wave0 + lane, lane < npts);
  const int ncorner = 1 << g.dims;
  constexpr int PU = 4;
  for (int q0 = 0; q0 < npts; q0 += PU) {
    int off[PU][kClCorners];
    float w[PU][kClCorners];
#pragma unroll
    for (int u = 0; u < PU; ++u) {
      const int q = min(q0 + u, npts - 1);
#pragma unroll
      for (int i = 0; i < kClCorners; ++i) {
        off[u][i] = __builtin_amdgcn_readlane(mine.off[i], q);
        w[u][i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine.w[i]), q));
      }
    }
    for (int c = lane; c < g.channel; c += 64) {
      float v[PU][kClCorners];
#pragma unroll
      for (int u = 0; u < PU; ++u)
#pragma unroll
        for (int i = 0; i < kClCorners; ++i)
          v[u][i] = i < ncorner ? ld(data_cl + (size_t)off[u][i] * g.channel + c) : 0.f;
#pragma unroll
      for (int u = 0; u < PU; ++u) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < kClCorners; ++i) acc += w[u][i] * v[u][i];
        if (q0 + u < npts) st(out + (wave0 + q0 + u) * g.channel + c, acc);
      }
    }
  }
}

// grad coord: same walk; per point the lanes' partial gradients are reduced by shuffles
template <typename T>
__global__ __launch_bounds__(kBlock) void nd_grad_coord_cl_kernel(NdGeo g, const T* __restrict__ gout,
                                                                  const T* __restrict__ data_cl,
                                                                  const T* __restrict__ coord,
                                                                  T* __restrict__ gcoord, int ppw) {
  const int lane = threadIdx.x & 63;
  const long wave0 = ((long)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6)) * ppw;
  if (wave0 >= g.batch) return;
  const int npts = (int)min((long)ppw, g.batch - wave0);
  const bool valid = lane < npts;
  const ClCorners mine = cl_corners<T>(g, coord, wave0 + lane, valid);
  const int ncorner = 1 << g.dims;
  // s[i] of point q lands in lane q: sum over channels of gout * data at corner i
  float s[kClCorners];
#pragma unroll
  for (int i = 0; i < kClCorners; ++i) s[i] = 0.f;
  for (int q = 0; q < npts; ++q) {
    int off[kClCorners];
#pragma unroll
    for (int i = 0; i < kClCorners; ++i) off[i] = __builtin_amdgcn_readlane(mine.off[i], q);
    float part[kClCorners];
#pragma unroll
    for (int i = 0; i < kClCorners; ++i) part[i] = 0.f;
    const T* grow = gout + (wave0 + q) * g.channel;
    for (int c = lane; c < g.channel; c += 64) {
      const float go = ld(grow + c);
#pragma unroll
      for (int i = 0; i < kClCorners; ++i)
        if (i < ncorner) part[i] += go * ld(data_cl + (size_t)off[i] * g.channel + c);
    }
#pragma unroll
    for (int i = 0; i < kClCorners; ++i) {
      if (i < ncorner) {
        const float v = wave_sum(part[i]);
        if (lane == q) s[i] = v;
      }
    }
  }
  if (!valid) return;
  // lane <-> point again: apply the derivative weights (ND.cu:161,165) to the corner sums
  const NdPoint<float> p = load_point<T, float>(g, coord + (wave0 + lane) * g.dims);
#pragma unroll
  for (int d = 0; d < kClMaxDims; ++d) {
    if (d < g.dims) {
      float gd = 0.f;
      if (p.inside) {
#pragma unroll
        for (int i = 0; i < kClCorners; ++i) {
          long o;
          float w;
          if (i < ncorner && corner<float>(g, p, (unsigned)i, d, o, w)) gd += s[i] * w;
        }
      }
      st(gcoord + (wave0 + lane) * g.dims + d, gd);
    }
  }
}

// grad data: scatter into the zeroed channel-last fp32 image; one 64-channel run per atomic
template <typename T>
__global__ __launch_bounds__(kBlock) void nd_grad_data_cl_kernel(NdGeo g, const T* __restrict__ gout,
                                                                 const T* __restrict__ coord,
                                                                 float* __restrict__ gdata_cl, int ppw) {
  const int lane = threadIdx.x & 63;
  const long wave0 = ((long)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6)) * ppw;
  if (wave0 >= g.batch) return;
  const int npts = (int)min((long)ppw, g.batch - wave0);
  const ClCorners mine = cl_corners<T>(g, coord, wave0 + lane, lane < npts);
  const int ncorner = 1 << g.dims;
  for (int q = 0; q < npts; ++q) {
    int off[kClCorners];
    float w[kClCorners];
#pragma unroll
    for (int i = 0; i < kClCorners; ++i) {
      off[i] = __builtin_amdgcn_readlane(mine.off[i], q);
      w[i] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine.w[i]), q));
    }
    const T* grow = gout + (wave0 + q) * g.channel;
    for (int c = lane; c < g.channel; c += 64) {
      const float go = ld(grow + c);
#pragma unroll
      for (int i = 0; i < kClCorners; ++i)
        if (i < ncorner && w[i] != 0.f) atomicAdd(gdata_cl + (size_t)off[i] * g.channel + c, w[i] * go);
    }
  }
}

// ---------------------------------------------------------------------------
// few points on a tiny volume (GlobalDeformKernel2d: 9 points per image on a 5 x 5 scope, hundreds of
// channels).  The forward takes the direct kernel above (one launch, the volume stays in cache);
// grad data and grad coord are one launch each here instead of fill + atomics + transpose /
// transpose + kernel.  These calls are bound by the latency of their few dependent loads, so both
// kernels know the number of dimensions at compile time (no branches between the loads) and issue
// every load of a stage before the first use.
//
// grad data: a small dense product on the matrix cores (below; scattering into sums instead --
// LDS or global float atomics on 25 x 256 sums that each receive 184 additions -- took 75-100 us).
// grad coord: one wave per point, lanes over channels; the volume is read where it lies.
// ---------------------------------------------------------------------------
constexpr int kSmallMaxCells = 64;

// The point's low corner and fractions for NDIM dimensions (load_point above, without its loop over
// DK_ND_MAX_DIMS); b is clamped by the caller.
template <typename T, int NDIM>
__device__ __forceinline__ NdPoint<float> small_point(const NdGeo& g, const T* coord_b) {
  float x[NDIM];
#pragma unroll
  for (int d = 0; d < NDIM; ++d) x[d] = ld(coord_b + d);
  NdPoint<float> p;
  p.inside = true;
#pragma unroll
  for (int d = 0; d < DK_ND_MAX_DIMS; ++d) {
    p.low[d] = 0;
    p.frac[d] = 0.f;
  }
#pragma unroll
  for (int d = 0; d < NDIM; ++d) {
    const float xf = floorf(x[d]);
    const bool in = x[d] > -1.f && x[d] < (float)g.shape[d];
    if (!in) p.inside = false;
    p.low[d] = in ? (int)xf : 0;
    p.frac[d] = x[d] - xf;
  }
  return p;
}

// grad data as a small dense product on the matrix cores: gdata[c][cell] = sum_b gout[b][c] * W[b][cell],
// W[b][.] being the point's 2^n corner weights spread over a row of zeros.  A workgroup of 16 waves owns
// 16 channels.  Per chunk of points it writes W into LDS (row = point, 16 cells per column tile), then
// each wave multiplies its share of the chunk's points, four at a time, with
// v_mfma_f32_16x16x4_f32 (M = channels, N = cells, K = points; fp32 products and sums).  The waves'
// 16 x 16 tiles are added in wave order at the end: no atomics, a fixed order of additions.
typedef float nd_f4 __attribute__((ext_vector_type(4)));
constexpr int kSmallTileMax = 4;                 // column tiles of 16 cells: volumes of up to 64 cells
constexpr int kSmallWBytes = 144 * 1024;         // LDS for W

template <typename T, int NDIM, int NT>
__global__ __launch_bounds__(1024) void nd_small_grad_data_kernel(NdGeo g, const T* __restrict__ gout,
                                                                   const T* __restrict__ coord,
                                                                   T* __restrict__ gdata, int chunk_points) {
  constexpr int NC = 1 << NDIM;
  constexpr int ROW = NT * 16;  // floats of a row of W
  extern __shared__ __align__(16) unsigned char small_lds[];
  float* W = reinterpret_cast<float*>(small_lds);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = min(blockIdx.x * 16 + (lane & 15), g.channel - 1);  // lanes past the last channel repeat it; not stored
  nd_f4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = nd_f4{0.f, 0.f, 0.f, 0.f};

  for (long chunk0 = 0; chunk0 < g.batch; chunk0 += chunk_points) {
    const int npts = (int)min((long)chunk_points, g.batch - chunk0);
    const int rows = (npts + 63) & ~63;  // whole 4-point steps for every wave; the extra rows stay zero
    // this thread's points of the chunk (loads first), then W = 0, then the corners' weights
    NdPoint<float> p[2];
    bool has[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const int q = threadIdx.x + 1024 * r;
      has[r] = q < npts;
      p[r] = small_point<T, NDIM>(g, coord + min(chunk0 + q, g.batch - 1) * NDIM);
    }
    __syncthreads();  // the previous chunk's products have read W
    for (int i = threadIdx.x; i < rows * ROW / 4; i += 1024) reinterpret_cast<nd_f4*>(W)[i] = nd_f4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      if (has[r] && p[r].inside) {
#pragma unroll
        for (int i = 0; i < NC; ++i) {
          long o;
          float w;
          if (corner<float>(g, p[r], (unsigned)i, -1, o, w)) W[(threadIdx.x + 1024 * r) * ROW + (int)o] = w;
        }
      }
    }
    __syncthreads();
    // wave w: rows [w * share, (w + 1) * share), share a multiple of 4
    const int share = rows / 16;
    const int r0 = wave * share;
    for (int s0 = 0; s0 < share; s0 += 32) {  // eight 4-point steps at a time, their out_grad loads first
      T raw[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int row = r0 + s0 + 4 * k + (lane >> 4);
        raw[k] = gout[min(chunk0 + row, g.batch - 1) * g.channel + c];
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (s0 + 4 * k < share) {  // uniform over the wave
          const int row = r0 + s0 + 4 * k + (lane >> 4);
          // rows past the chunk's points re-read the last point's out_grad: they are zeroed by a select, not by
          // their zero row of W (0 * Inf would put a NaN into every cell of the channel)
          const float a = row < npts ? ld(&raw[k]) : 0.f;
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, W[row * ROW + t * 16 + (lane & 15)], acc[t], 0, 0, 0);
        }
      }
    }
  }
  __syncthreads();
  // the waves' tiles through LDS (W's space), added in wave order
  float* red = W;  // [16 waves][NT][16 channels][16 cells]
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[((wave * NT + t) * 16 + 4 * (lane >> 4) + i) * 16 + (lane & 15)] = acc[t][i];
  __syncthreads();
  const int cells = (int)g.prod_shape;
  for (int i = threadIdx.x; i < NT * 256; i += 1024) {
    const int t = i >> 8, m = (i >> 4) & 15, n = i & 15;
    float v = 0.f;
    for (int w = 0; w < 16; ++w) v += red[((w * NT + t) * 16 + m) * 16 + n];
    const int co = blockIdx.x * 16 + m, cell = t * 16 + n;
    if (co < g.channel && cell < cells) st(gdata + (size_t)co * g.prod_shape + cell, v);
  }
}

template <typename T, int NDIM>
__global__ __launch_bounds__(kBlock) void nd_small_grad_coord_kernel(NdGeo g, const T* __restrict__ gout,
                                                                     const T* __restrict__ data,
                                                                     const T* __restrict__ coord,
                                                                     T* __restrict__ gcoord) {
  constexpr int NC = 1 << NDIM;
  const int lane = threadIdx.x & 63;
  const long b = (long)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (b >= g.batch) return;
  const NdPoint<float> p = small_point<T, NDIM>(g, coord + b * NDIM);
  int off[NC];
  float dw[NDIM][NC];  // derivative weights (ND.cu:161,165); 0 for a corner outside the volume
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    long o = 0;
    float w = 0.f;
    const bool ok = p.inside && corner<float>(g, p, (unsigned)i, -1, o, w);
    off[i] = ok ? (int)o : 0;
#pragma unroll
    for (int d = 0; d < NDIM; ++d) {
      long o2;
      float w2 = 0.f;
      const bool ok2 = ok && corner<float>(g, p, (unsigned)i, d, o2, w2);
      dw[d][i] = ok2 ? w2 : 0.f;
    }
  }
  float part[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) part[i] = 0.f;
  const T* grow = gout + b * g.channel;
  for (int c0 = 0; c0 < g.channel; c0 += 256) {
    // four 64-channel tiles at a time, loads first (channels past the end repeat the last one with a zero out_grad)
    T graw[4], draw[4][NC];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int c = min(c0 + 64 * t + lane, g.channel - 1);
      graw[t] = grow[c];
#pragma unroll
      for (int i = 0; i < NC; ++i) draw[t][i] = data[(size_t)c * g.prod_shape + off[i]];
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float go = c0 + 64 * t + lane < g.channel ? ld(&graw[t]) : 0.f;
#pragma unroll
      for (int i = 0; i < NC; ++i) part[i] += go * ld(&draw[t][i]);
    }
  }
  float gd[NDIM];
#pragma unroll
  for (int d = 0; d < NDIM; ++d) gd[d] = 0.f;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const float v = wave_sum(part[i]);
#pragma unroll
    for (int d = 0; d < NDIM; ++d) gd[d] += v * dw[d][i];
  }
  if (lane == 0) {
#pragma unroll
    for (int d = 0; d < NDIM; ++d) st(gcoord + b * NDIM + d, gd[d]);
  }
}

// ---------------------------------------------------------------------------
// binned channel-last path: many points per cell of the volume
//
// With more points than cells, points that fall into the same cell read (forward, grad coord)
// or update (grad data) the same 2^n corner rows.  The points are therefore sorted by cell
// first -- a radix sort of (key, point index) pairs (radix_*_kernel below), the key being the cell's low corner,
// (low[d] + 1) over extents shape[d] + 1, plus one last bin for the points outside the volume;
// a radix sort rather than a counting sort with atomics because the points of a real workload
// may all sit in a handful of cells -- and a wave walks 64
// consecutive points of the sorted order, lanes over channels: the corner rows stay in
// registers while the cell does not change (forward, grad coord), and the input gradient of a
// cell's corners is summed in registers and leaves as one atomic per corner and channel when the
// cell changes (grad data).  Results go to / come from each point's original row.
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ int point_bin(const NdGeo& g, const T* coord_b, int nbins) {
  const NdPoint<float> p = load_point<T, float>(g, coord_b);
  if (!p.inside) return nbins - 1;
  int key = 0;
#pragma unroll
  for (int d = 0; d < kClMaxDims; ++d)
    if (d < g.dims) key = key * (g.shape[d] + 1) + p.low[d] + 1;
  return key;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void nd_bin_keys_kernel(NdGeo g, const T* __restrict__ coord, int nbins,
                                                             unsigned* __restrict__ keys) {
  const long b = (long)blockIdx.x * kBlock + threadIdx.x;
  if (b < g.batch) keys[b] = (unsigned)point_bin<T>(g, coord + b * g.dims, nbins);
}

// What a wave of the binned kernels knows about its 64 sorted points: lane q holds point q.
template <typename T>
struct BinnedWave {
  int npts, id, key;
  ClCorners cc;
  // the wave's `sub`-th chunk of 64 points when a wave walks `per_wave` consecutive chunks
  __device__ __forceinline__ bool init(const NdGeo& g, const T* coord, const int* order, int nbins,
                                       int per_wave = 1, int sub = 0) {
    const int lane = threadIdx.x & 63;
    const long wave0 = (((long)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6)) * per_wave + sub) * 64;
    if (wave0 >= g.batch) return false;
    npts = (int)min(64L, g.batch - wave0);
    const bool valid = lane < npts;
    id = valid ? order[wave0 + lane] : 0;
    cc = cl_corners<T>(g, coord, id, valid);
    key = valid ? point_bin<T>(g, coord + (long)id * g.dims, nbins) : -1;
    return true;
  }
  __device__ __forceinline__ int key_of(int q) const { return __builtin_amdgcn_readlane(key, q); }
  __device__ __forceinline__ long id_of(int q) const { return __builtin_amdgcn_readlane(id, q); }
  __device__ __forceinline__ int off_of(int i, int q) const { return __builtin_amdgcn_readlane(cc.off[i], q); }
  __device__ __forceinline__ float w_of(int i, int q) const {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cc.w[i]), q));
  }
};

// Makes the corner rows just loaded count as used here, so that the wait for them sits in the
// (rare) cell-change branch.  Otherwise the compiler waits for every outstanding memory operation
// at the first use after the branch, for every point, and that includes the point's own store.
__device__ __forceinline__ void settle(float (&v)[kClCorners]) {
  asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
}

template <typename T>
__global__ __launch_bounds__(kBlock) void nd_forward_binned_kernel(NdGeo g, const T* __restrict__ data_cl,
                                                                   const T* __restrict__ coord,
                                                                   const int* __restrict__ order, int nbins,
                                                                   T* __restrict__ out) {
  BinnedWave<T> wv;
  if (!wv.init(g, coord, order, nbins)) return;
  const int lane = threadIdx.x & 63, ncorner = 1 << g.dims;
  for (int c0 = 0; c0 < g.channel; c0 += 64) {
    const int c = c0 + lane;
    const bool cin = c < g.channel;
    float v[kClCorners];
#pragma unroll
    for (int i = 0; i < kClCorners; ++i) v[i] = 0.f;
    int cur = -2;
    for (int q = 0; q < wv.npts; ++q) {
      const int key = wv.key_of(q);
      if (key != cur) {  // wave-uniform: a new cell, fetch its corner rows
        cur = key;
#pragma unroll
        for (int i = 0; i < kClCorners; ++i)
          v[i] = (cin && i < ncorner) ? ld(data_cl + (size_t)wv.off_of(i, q) * g.channel + c) : 0.f;
        settle(v);
      }
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < kClCorners; ++i) acc += wv.w_of(i, q) * v[i];
      if (cin) st(out + wv.id_of(q) * g.channel + c, acc);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void nd_grad_data_binned_kernel(NdGeo g, const T* __restrict__ gout,
                                                                     const T* __restrict__ coord,
                                                                     const int* __restrict__ order, int nbins,
                                                                     float* __restrict__ gdata_cl, int per_wave) {
  const int lane = threadIdx.x & 63, ncorner = 1 << g.dims;
  constexpr int PU = 8;  // output-gradient rows in flight
  for (int c0 = 0; c0 < g.channel; c0 += 64) {
    const int c = c0 + lane;
    const bool cin = c < g.channel;
    float acc[kClCorners];
    int at[kClCorners];
#pragma unroll
    for (int i = 0; i < kClCorners; ++i) acc[i] = 0.f, at[i] = 0;
    int cur = -2;
#define DK_FLUSH()                                                                             \
  _Pragma("unroll") for (int i = 0; i < kClCorners; ++i) if (cin && i < ncorner && acc[i] != 0.f) \
      atomicAdd(gdata_cl + (size_t)at[i] * g.channel + c, acc[i])
    // the sums of a cell stay in registers across the wave's chunks: when thousands of points
    // share a cell, fewer waves send fewer atomics to the same rows
    for (int sub = 0; sub < per_wave; ++sub) {
      BinnedWave<T> wv;
      if (!wv.init(g, coord, order, nbins, per_wave, sub)) break;
      for (int q0 = 0; q0 < wv.npts; q0 += PU) {
        float go[PU];
#pragma unroll
        for (int u = 0; u < PU; ++u)
          go[u] = (cin && q0 + u < wv.npts) ? ld(gout + wv.id_of(min(q0 + u, wv.npts - 1)) * g.channel + c) : 0.f;
#pragma unroll
        for (int u = 0; u < PU; ++u) {
          const int q = q0 + u;
          if (q < wv.npts) {
            const int key = wv.key_of(q);
            if (key != cur) {  // wave-uniform: the sums of the finished cell leave
              cur = key;
              int nat[kClCorners];
              float nacc[kClCorners];
#pragma unroll
              for (int i = 0; i < kClCorners; ++i) nacc[i] = 0.f, nat[i] = wv.off_of(i, q);
              // The next cell in key order is mostly the neighbour along the last dimension, whose
              // low-side rows are this cell's high-side rows: those sums stay in registers (rows are
              // matched by their offsets, so any other successor just flushes everything).  Atomics
              // on the volume are what bounds this kernel; this halves them.
#define DK_CARRY(HB)                                                                            \
  _Pragma("unroll") for (int i = 0; i < kClCorners; ++i) {                                      \
    if ((i & (HB)) && i < 2 * (HB)) {                                                           \
      if (at[i] == nat[i - (HB)]) {                                                             \
        nacc[i - (HB)] = acc[i];                                                                \
        acc[i] = 0.f;                                                                           \
      }                                                                                         \
    }                                                                                           \
  }
              if (g.dims == 3) {
                DK_CARRY(4)
              } else if (g.dims == 2) {
                DK_CARRY(2)
              } else {
                DK_CARRY(1)
              }
#undef DK_CARRY
              DK_FLUSH();
#pragma unroll
              for (int i = 0; i < kClCorners; ++i) acc[i] = nacc[i], at[i] = nat[i];
            }
#pragma unroll
            for (int i = 0; i < kClCorners; ++i) acc[i] += wv.w_of(i, q) * go[u];
          }
        }
      }
    }
    DK_FLUSH();
#undef DK_FLUSH
  }
}

// grad coord on the sorted points.  Per cell the eight corner rows are turned into the
// coefficients of the multilinear polynomial,
//   value = c0 + c1 f0 + c2 f1 + c3 f2 + c4 f0 f1 + c5 f0 f2 + c6 f1 f2 + c7 f0 f1 f2
// (f = fractional position; absent corners and absent dimensions enter as zeros, which is what
// skipping them amounts to), so that a point's three partial derivatives cost nine fused
// multiply-adds per channel instead of eight corner products, and three wave reductions
// instead of eight.
template <typename T>
__global__ __launch_bounds__(kBlock) void nd_grad_coord_binned_kernel(NdGeo g, const T* __restrict__ gout,
                                                                      const T* __restrict__ data_cl,
                                                                      const T* __restrict__ coord,
                                                                      const int* __restrict__ order, int nbins,
                                                                      T* __restrict__ gcoord) {
  BinnedWave<T> wv;
  if (!wv.init(g, coord, order, nbins)) return;
  const int lane = threadIdx.x & 63;
  const bool valid = lane < wv.npts;
  // lane <-> point: fractional position and its pairwise products
  NdPoint<float> p;
  p.inside = false;
#pragma unroll
  for (int d = 0; d < DK_ND_MAX_DIMS; ++d) p.frac[d] = 0.f, p.low[d] = 0;
  if (valid) p = load_point<T, float>(g, coord + (long)wv.id * g.dims);
  const float f0 = p.frac[0], f1 = p.frac[1], f2 = p.frac[2];
  const float f01 = f0 * f1, f02 = f0 * f2, f12 = f1 * f2;
  auto uni = [](float v, int q) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), q));
  };
  constexpr int PU = 4;
  float gd0 = 0.f, gd1 = 0.f, gd2 = 0.f;  // of point q, in lane q
  for (int c0 = 0; c0 < g.channel; c0 += 64) {
    const int c = c0 + lane;
    const bool cin = c < g.channel;
    float k1 = 0.f, k2 = 0.f, k3 = 0.f, k4 = 0.f, k5 = 0.f, k6 = 0.f, k7 = 0.f;
    int cur = -2;
    for (int q0 = 0; q0 < wv.npts; q0 += PU) {
      float go[PU];
#pragma unroll
      for (int u = 0; u < PU; ++u)
        go[u] = (cin && q0 + u < wv.npts) ? ld(gout + wv.id_of(min(q0 + u, wv.npts - 1)) * g.channel + c) : 0.f;
#pragma unroll
      for (int u = 0; u < PU; ++u) {
        const int q = q0 + u;
        if (q < wv.npts) {
          const int key = wv.key_of(q);
          if (key != cur) {
            cur = key;
            float v[kClCorners];
            const unsigned present = (unsigned)__builtin_amdgcn_readlane((int)wv.cc.present, q);
#pragma unroll
            for (int i = 0; i < kClCorners; ++i)
              v[i] = (cin && (present >> i & 1u)) ? ld(data_cl + (size_t)wv.off_of(i, q) * g.channel + c) : 0.f;
            settle(v);
            // corner index: bit d = high side of dimension d
            k1 = v[1] - v[0];
            k2 = v[2] - v[0];
            k3 = v[4] - v[0];
            k4 = (v[3] - v[2]) - k1;
            k5 = (v[5] - v[4]) - k1;
            k6 = (v[6] - v[4]) - k2;
            k7 = ((v[7] - v[6]) - (v[5] - v[4])) - k4;
          }
          const float u0 = uni(f0, q), u1 = uni(f1, q), u2 = uni(f2, q);
          const float u01 = uni(f01, q), u02 = uni(f02, q), u12 = uni(f12, q);
          const float d0 = fmaf(k7, u12, fmaf(k5, u2, fmaf(k4, u1, k1)));
          const float d1 = fmaf(k7, u02, fmaf(k6, u2, fmaf(k4, u0, k2)));
          const float d2 = fmaf(k7, u01, fmaf(k6, u1, fmaf(k5, u0, k3)));
          const float t0 = wave_sum(go[u] * d0);
          if (lane == q) gd0 += t0;
          if (g.dims > 1) {
            const float t1 = wave_sum(go[u] * d1);
            if (lane == q) gd1 += t1;
          }
          if (g.dims > 2) {
            const float t2 = wave_sum(go[u] * d2);
            if (lane == q) gd2 += t2;
          }
        }
      }
    }
  }
  if (!valid) return;
  const float gd[3] = {gd0, gd1, gd2};
#pragma unroll
  for (int d = 0; d < kClMaxDims; ++d)
    if (d < g.dims) st(gcoord + (long)wv.id * g.dims + d, p.inside ? gd[d] : 0.f);
}

// Orders LDS writes of a wave before the reads of its other lanes (a wave owns its LDS slice).
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

typedef float nd4 __attribute__((ext_vector_type(4)));

// grad coord on the sorted points with the sums over the channels on the matrix cores (fp32,
// channel count a multiple of 64).  With the polynomial coefficients k1 .. k7 of a cell (see
// nd_grad_coord_binned_kernel) a point's derivatives are
//   d0 = S1 + f1 S4 + f2 S5 + f1 f2 S7,  d1 = S2 + f0 S4 + f2 S6 + f0 f2 S7,
//   d2 = S3 + f0 S5 + f1 S6 + f0 f1 S7,       S_m = sum_c gout[c] * k_m[c],
// and the S_m of 16 points of one cell are a 16 x 64 by 64 x 16 product: v_mfma_f32_16x16x4_f32 with
// lane l supplying gout[point l % 16][channel 16 (l / 16) + step] and k_{l % 16}[the same channel]
// over 16 steps (step 4 j + i takes channel 16 j + 4 (l / 16) + i of the block, the same for both operands, so that
// the four lanes of a point read 64 contiguous bytes of its row with each of their four 16-byte loads; the
// coefficients go through the wave's LDS slice).  The three wave reductions per point and channel
// block of the VALU kernel (75 VALU instructions per point) become one MFMA per point.
template <typename T>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(4, 4))) void nd_grad_coord_mfma_kernel(NdGeo g, const float* __restrict__ gout,
                                                                    const float* __restrict__ data_cl,
                                                                    const float* __restrict__ coord,
                                                                    const int* __restrict__ order, int nbins,
                                                                    float* __restrict__ gcoord) {
  __shared__ __align__(16) float s_coef[kBlock / 64][8][64];  // [wave][m][channel of the block]
  __shared__ __align__(16) float s_sum[kBlock / 64][16][16];  // [wave][point of the batch][m]
  BinnedWave<float> wv;
  if (!wv.init(g, coord, order, nbins)) return;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  float(*coef)[64] = s_coef[wave];
  float(*sums)[16] = s_sum[wave];
  const bool valid = lane < wv.npts;
  NdPoint<float> p;
  p.inside = false;
#pragma unroll
  for (int d = 0; d < DK_ND_MAX_DIMS; ++d) p.frac[d] = 0.f, p.low[d] = 0;
  if (valid) p = load_point<float, float>(g, coord + (long)wv.id * g.dims);
  const float f0 = p.frac[0], f1 = p.frac[1], f2 = p.frac[2];
  const float f01 = f0 * f1, f02 = f0 * f2, f12 = f1 * f2;
  const int pr = lane & 15, kg = lane >> 4;  // MFMA row (point of the batch / coefficient index), K group
  float gd0 = 0.f, gd1 = 0.f, gd2 = 0.f;     // of point q, in lane q

  int qs = 0;
  while (qs < wv.npts) {
    // the run of points in the cell of point qs: the keys are sorted
    const int key = wv.key_of(qs);
    const int qe = qs + (int)__popcll(__ballot(wv.key == key));
    const unsigned present = (unsigned)__builtin_amdgcn_readlane((int)wv.cc.present, qs);
    nd4 acc[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[b] = nd4{0.f, 0.f, 0.f, 0.f};
    for (int c0 = 0; c0 < g.channel; c0 += 64) {
      // this lane's 16 channels of its point in batch b: issued two batches ahead of their MFMAs,
      // the first two before the cell's corner rows, so that the two latencies overlap (two buffers in turn:
      // with four the kernel takes 168 registers and a SIMD holds three waves of it; this is four)
      float av[2][16];
#define DK_ND_LOAD_A(b)                                                                          \
  if (qs + 16 * (b) < qe) {                                                                      \
    const int q_ = qs + 16 * (b) + pr;                                                           \
    const bool on_ = q_ < qe;                                                                    \
    const long id_ = __shfl(wv.id, on_ ? q_ : qs);                                               \
    const float4* rowp_ = reinterpret_cast<const float4*>(gout + id_ * g.channel + c0 + 4 * kg); \
    _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                              \
      const float4 t_ = rowp_[4 * j];  /* the four lanes of a point: 64 contiguous bytes */      \
      av[(b) & 1][4 * j] = on_ ? t_.x : 0.f;                                                     \
      av[(b) & 1][4 * j + 1] = on_ ? t_.y : 0.f;                                                 \
      av[(b) & 1][4 * j + 2] = on_ ? t_.z : 0.f;                                                 \
      av[(b) & 1][4 * j + 3] = on_ ? t_.w : 0.f;                                                 \
    }                                                                                            \
  }
#define DK_ND_MFMA(b)                                                                            \
  if (qs + 16 * (b) < qe) {                                                                      \
    _Pragma("unroll") for (int s_ = 0; s_ < 16; ++s_)                                            \
      acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[(b) & 1][s_], bv[s_], acc[b], 0, 0, 0);   \
  }
      DK_ND_LOAD_A(0)
      DK_ND_LOAD_A(1)
      {
        float v[kClCorners];
#pragma unroll
        for (int i = 0; i < kClCorners; ++i)
          v[i] = (present >> i & 1u) ? data_cl[(size_t)wv.off_of(i, qs) * g.channel + c0 + lane] : 0.f;
        // corner index: bit d = high side of dimension d
        const float k1 = v[1] - v[0], k2 = v[2] - v[0], k3 = v[4] - v[0];
        const float k4 = (v[3] - v[2]) - k1, k5 = (v[5] - v[4]) - k1, k6 = (v[6] - v[4]) - k2;
        const float k7 = ((v[7] - v[6]) - (v[5] - v[4])) - k4;
        wave_lds_sync();  // the previous block's coefficient reads are done
        coef[1][lane] = k1;
        coef[2][lane] = k2;
        coef[3][lane] = k3;
        coef[4][lane] = k4;
        coef[5][lane] = k5;
        coef[6][lane] = k6;
        coef[7][lane] = k7;
        wave_lds_sync();
      }
      float bv[16];
      {
        const bool row = pr >= 1 && pr < 8;  // rows 0 and 8 .. 15 of the coefficient matrix are zero
        const float4* src = reinterpret_cast<const float4*>(&coef[row ? pr : 1][4 * kg]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 t = src[4 * j];
          bv[4 * j] = row ? t.x : 0.f;
          bv[4 * j + 1] = row ? t.y : 0.f;
          bv[4 * j + 2] = row ? t.z : 0.f;
          bv[4 * j + 3] = row ? t.w : 0.f;
        }
      }
      DK_ND_MFMA(0)
      DK_ND_LOAD_A(2)
      DK_ND_MFMA(1)
      DK_ND_LOAD_A(3)
      DK_ND_MFMA(2)
      DK_ND_MFMA(3)
#undef DK_ND_LOAD_A
#undef DK_ND_MFMA
    }
    // D[point 4 (l / 16) + r][m = l % 16] in register r of lane l: through LDS to the points' lanes
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      if (qs + 16 * b < qe) {
        wave_lds_sync();
#pragma unroll
        for (int r = 0; r < 4; ++r) sums[4 * kg + r][pr] = acc[b][r];
        wave_lds_sync();
        const int mine = lane - (qs + 16 * b);
        if (mine >= 0 && mine < 16 && lane < qe) {
          const float4 lo4 = *reinterpret_cast<const float4*>(&sums[mine][0]);
          const float4 hi4 = *reinterpret_cast<const float4*>(&sums[mine][4]);
          const float S1 = lo4.y, S2 = lo4.z, S3 = lo4.w, S4 = hi4.x, S5 = hi4.y, S6 = hi4.z, S7 = hi4.w;
          gd0 += fmaf(f12, S7, fmaf(f2, S5, fmaf(f1, S4, S1)));
          gd1 += fmaf(f02, S7, fmaf(f2, S6, fmaf(f0, S4, S2)));
          gd2 += fmaf(f01, S7, fmaf(f1, S6, fmaf(f0, S5, S3)));
        }
      }
    }
    qs = qe;
  }
  if (!valid) return;
  const float gd[3] = {gd0, gd1, gd2};
#pragma unroll
  for (int d = 0; d < kClMaxDims; ++d)
    if (d < g.dims) gcoord[(long)wv.id * g.dims + d] = p.inside ? gd[d] : 0.f;
}

// grad data on the sorted points on the matrix cores (fp32, channel count a multiple of 64): the
// sums of a cell's corner rows over the points of a run are a product
//   D[corner][channel] = sum_p w_corner(p) * gout[p][channel],
// done 16 points at a time by v_mfma_f32_16x16x4_f32: lane l supplies w_{l % 16}(point 4 step + l / 16)
// (from the wave's LDS copy of its points' corner weights; rows 8 .. 15 are zero) and the four
// channels 4 (l % 16) .. + 3 of that point's gout row (one 16-byte load; the 16 lanes of a point read
// its 256-byte row), one MFMA per channel of the quad.  The VALU kernel spends its time on the
// per-point broadcasts (v_readlane of eight weights, key and row index per point).
template <typename T>
__global__ __launch_bounds__(kBlock) void nd_grad_data_mfma_kernel(NdGeo g, const float* __restrict__ gout,
                                                                   const float* __restrict__ coord,
                                                                   const int* __restrict__ order, int nbins,
                                                                   float* __restrict__ gdata_cl, int per_wave) {
  __shared__ __align__(16) float s_w[kBlock / 64][64][kClCorners];  // [wave][point][corner]
  __shared__ __align__(16) float s_d[kBlock / 64][kClCorners][64];  // [wave][corner][channel]
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int pr = lane & 15, kg = lane >> 4, ncorner = 1 << g.dims;
  float(*wl)[kClCorners] = s_w[wave];
  float(*dl)[64] = s_d[wave];
  for (int c0 = 0; c0 < g.channel; c0 += 64) {
    nd4 acc[4];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) acc[cb] = nd4{0.f, 0.f, 0.f, 0.f};
    int at[kClCorners];
#pragma unroll
    for (int i = 0; i < kClCorners; ++i) at[i] = 0;
    int cur = -2;
    // D[corner 4 (l / 16) + r][channel 4 (l % 16) + cb] sits in acc[cb][r] of lane l: through LDS to
    // one lane per channel, which sends the corner rows' sums
#define DK_FLUSH()                                                                                   \
  if (cur != -2) {                                                                                   \
    wave_lds_sync();                                                                                 \
    if (kg < 2) {                                                                                    \
      _Pragma("unroll") for (int r = 0; r < 4; ++r)                                                  \
        *reinterpret_cast<float4*>(&dl[4 * kg + r][4 * pr]) = make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]); \
    }                                                                                                \
    wave_lds_sync();                                                                                 \
    _Pragma("unroll") for (int i = 0; i < kClCorners; ++i) {                                         \
      if (i < ncorner) {                                                                             \
        const float v_ = dl[i][lane];                                                                \
        if (v_ != 0.f) atomicAdd(gdata_cl + (size_t)at[i] * g.channel + c0 + lane, v_);              \
      }                                                                                              \
    }                                                                                                \
  }
    // the sums of a cell stay in registers across the wave's chunks: when thousands of points
    // share a cell, fewer waves send fewer atomics to the same rows
    for (int sub = 0; sub < per_wave; ++sub) {
      BinnedWave<float> wv;
      if (!wv.init(g, coord, order, nbins, per_wave, sub)) break;
      wave_lds_sync();  // the previous chunk's weight reads are done
      *reinterpret_cast<float4*>(&wl[lane][0]) = make_float4(wv.cc.w[0], wv.cc.w[1], wv.cc.w[2], wv.cc.w[3]);
      *reinterpret_cast<float4*>(&wl[lane][4]) = make_float4(wv.cc.w[4], wv.cc.w[5], wv.cc.w[6], wv.cc.w[7]);
      wave_lds_sync();
      int qs = 0;
      while (qs < wv.npts) {
        const int key = wv.key_of(qs);
        const int qe = qs + (int)__popcll(__ballot(wv.key == key));  // the keys are sorted
        if (key != cur) {
          DK_FLUSH();
          cur = key;
#pragma unroll
          for (int i = 0; i < kClCorners; ++i) at[i] = wv.off_of(i, qs);
#pragma unroll
          for (int cb = 0; cb < 4; ++cb) acc[cb] = nd4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          if (qs + 16 * b < qe) {  // wave-uniform
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              const int q = qs + 16 * b + 4 * s + kg;
              const bool on = q < qe;
              const int qc = on ? q : qs;
              const long id = __shfl(wv.id, qc);
              const float4 t = *reinterpret_cast<const float4*>(gout + id * g.channel + c0 + 4 * pr);
              const float a = (on && pr < kClCorners) ? wl[qc][pr & (kClCorners - 1)] : 0.f;
              acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, t.x, acc[0], 0, 0, 0);
              acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, t.y, acc[1], 0, 0, 0);
              acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, t.z, acc[2], 0, 0, 0);
              acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, t.w, acc[3], 0, 0, 0);
            }
          }
        }
        qs = qe;
      }
    }
    DK_FLUSH();
#undef DK_FLUSH
  }
}

// forward on the sorted points on the matrix cores (fp32, channel count a multiple of 64): for the
// points of a cell run,
//   out[p][channel] = sum_corner w_corner(p) * row_corner[channel],
// 16 points at a time: lane l supplies w_{4 step + l / 16}(point l % 16) (from the wave's LDS copy of
// its points' corner weights) and the channels 4 (l % 16) .. + 3 of corner row 4 step + l / 16 (one
// 16-byte load per run), two steps of v_mfma_f32_16x16x4_f32 per channel of the quad; the results
// leave as 16-byte stores, the 16 lanes of a point writing its 256-byte row.
template <typename T>
__global__ __launch_bounds__(kBlock) void nd_forward_mfma_kernel(NdGeo g, const float* __restrict__ data_cl,
                                                                 const float* __restrict__ coord,
                                                                 const int* __restrict__ order, int nbins,
                                                                 float* __restrict__ out) {
  __shared__ __align__(16) float s_w[kBlock / 64][64][kClCorners];  // [wave][point][corner]
  BinnedWave<float> wv;
  if (!wv.init(g, coord, order, nbins)) return;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int pr = lane & 15, kg = lane >> 4;
  float(*wl)[kClCorners] = s_w[wave];
  *reinterpret_cast<float4*>(&wl[lane][0]) = make_float4(wv.cc.w[0], wv.cc.w[1], wv.cc.w[2], wv.cc.w[3]);
  *reinterpret_cast<float4*>(&wl[lane][4]) = make_float4(wv.cc.w[4], wv.cc.w[5], wv.cc.w[6], wv.cc.w[7]);
  wave_lds_sync();
  for (int c0 = 0; c0 < g.channel; c0 += 64) {
    int qs = 0;
    while (qs < wv.npts) {
      const int key = wv.key_of(qs);
      const int qe = qs + (int)__popcll(__ballot(wv.key == key));  // the keys are sorted
      const unsigned present = (unsigned)__builtin_amdgcn_readlane((int)wv.cc.present, qs);
      float4 bq[2];
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int o0 = wv.off_of(4 * s, qs), o1 = wv.off_of(4 * s + 1, qs), o2 = wv.off_of(4 * s + 2, qs),
                  o3 = wv.off_of(4 * s + 3, qs);
        const int o = kg == 0 ? o0 : kg == 1 ? o1 : kg == 2 ? o2 : o3;
        const bool on = present >> (4 * s + kg) & 1u;
        const float4 t = *reinterpret_cast<const float4*>(data_cl + (size_t)(on ? o : 0) * g.channel + c0 + 4 * pr);
        bq[s] = on ? t : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        if (qs + 16 * b < qe) {  // wave-uniform
          const int q = qs + 16 * b + pr;
          const bool onp = q < qe;
          const int qc = onp ? q : qs;
          nd4 acc[4];
#pragma unroll
          for (int cb = 0; cb < 4; ++cb) acc[cb] = nd4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            const float a = onp ? wl[qc][4 * s + kg] : 0.f;
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bq[s].x, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bq[s].y, acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bq[s].z, acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bq[s].w, acc[3], 0, 0, 0);
          }
          // D[point 4 (l / 16) + r][channel 4 (l % 16) + cb] in acc[cb][r] of lane l
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int qo = qs + 16 * b + 4 * kg + r;
            const long id = __shfl(wv.id, qo < qe ? qo : qs);
            if (qo < qe)
              // non-temporal: the 256-byte rows are not read again, and written with the default policy they push
              // the volume out of L2 (config 5: forward 159 -> 150 us)
              __builtin_nontemporal_store(nd4{acc[0][r], acc[1][r], acc[2][r], acc[3][r]},
                                          reinterpret_cast<nd4*>(out + id * g.channel + c0 + 4 * pr));
          }
        }
      }
      qs = qe;
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

// ---------------------------------------------------------------------------
// Sort of the (cell key, point) pairs: a least-significant-digit radix sort in two passes of at
// most 9 bits (the keys have at most 18), each pass three kernels that launch nothing but
// themselves (so the sorted path can be captured into a graph):
//   radix_count_kernel    a workgroup counts the digits of its tile of 4096 keys (LDS atomics) into
//                         table[digit][workgroup];
//   radix_scan_*_kernel   exclusive prefix sum of the table in (digit, workgroup) order (per tile of
//                         4096 entries, then over the tile sums): where each workgroup's keys of each
//                         digit start in the output;
//   radix_scatter_kernel  stable scatter.  A wave owns 1024 consecutive keys of the tile, 16 rounds
//                         of 64; the four waves' starts per digit follow from their counts; within
//                         a round a lane's rank among the lanes with its digit comes from nine
//                         ballots, and the first of them advances the wave's LDS counter.
// ---------------------------------------------------------------------------
constexpr int kSortTile = 4096, kSortWaveKeys = kSortTile / (kBlock / 64), kSortRounds = kSortWaveKeys / 64;
constexpr int kSortMaxDigits = 512;

__global__ __launch_bounds__(kBlock) void radix_count_kernel(const unsigned* __restrict__ keys, long n, int shift,
                                                             int digits, int nblocks, unsigned* __restrict__ table) {
  __shared__ unsigned h[kSortMaxDigits];
  for (int d = threadIdx.x; d < digits; d += kBlock) h[d] = 0u;
  __syncthreads();
  const long base = (long)blockIdx.x * kSortTile;
#pragma unroll 4
  for (int r = 0; r < kSortTile / kBlock; ++r) {
    const long i = base + r * kBlock + threadIdx.x;
    if (i < n) atomicAdd(&h[(keys[i] >> shift) & (unsigned)(digits - 1)], 1u);
  }
  __syncthreads();
  for (int d = threadIdx.x; d < digits; d += kBlock) table[(size_t)d * nblocks + blockIdx.x] = h[d];
}

// Exclusive prefix sum of 1024 values, one per thread of the workgroup; `total` receives their sum.
__device__ __forceinline__ unsigned block_exclusive_scan(unsigned v, unsigned* wave_sum /* [16] LDS */, unsigned& total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned incl = v;
#pragma unroll
  for (int step = 1; step < 64; step <<= 1) {
    const unsigned up = (unsigned)__shfl_up((int)incl, step);
    if (lane >= step) incl += up;
  }
  __syncthreads();  // the previous use of wave_sum is over
  if (lane == 63) wave_sum[wave] = incl;
  __syncthreads();
  unsigned before = 0u, all = 0u;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    const unsigned t = wave_sum[w];
    before += w < wave ? t : 0u;
    all += t;
  }
  total = all;
  return before + incl - v;
}

// in place, per tile of 4096 entries (a thread owns four consecutive ones); sums[tile] = the tile's sum
constexpr int kScanTile = 4096;
__global__ __launch_bounds__(1024) void radix_scan_tiles_kernel(unsigned* __restrict__ table, int total,
                                                               unsigned* __restrict__ sums) {
  __shared__ unsigned wave_sum[16];
  const int i0 = blockIdx.x * kScanTile + 4 * (int)threadIdx.x;
  unsigned v[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) v[k] = i0 + k < total ? table[i0 + k] : 0u;
  unsigned all;
  unsigned run = block_exclusive_scan(v[0] + v[1] + v[2] + v[3], wave_sum, all);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (i0 + k < total) table[i0 + k] = run;
    run += v[k];
  }
  if (threadIdx.x == 0) sums[blockIdx.x] = all;
}
// exclusive prefix sum of the tile sums, in place: one workgroup walks them 1024 at a time
__global__ __launch_bounds__(1024) void radix_scan_sums_kernel(unsigned* __restrict__ sums, int count) {
  __shared__ unsigned wave_sum[16];
  unsigned carry = 0u;
  for (int base = 0; base < count; base += 1024) {
    const int i = base + (int)threadIdx.x;
    const unsigned v = i < count ? sums[i] : 0u;
    unsigned all;
    const unsigned excl = block_exclusive_scan(v, wave_sum, all);
    if (i < count) sums[i] = carry + excl;
    carry += all;
  }
}

// idx_in == nullptr: the points are still in their own order (index = position);
// keys_out == nullptr: the keys are not needed after this pass
__global__ __launch_bounds__(kBlock) void radix_scatter_kernel(const unsigned* __restrict__ keys,
                                                               const int* __restrict__ idx_in, long n, int shift,
                                                               int digits, int nblocks,
                                                               const unsigned* __restrict__ table,
                                                               const unsigned* __restrict__ tile_start,
                                                               unsigned* __restrict__ keys_out,
                                                               int* __restrict__ idx_out) {
  constexpr int kWaves = kBlock / 64;
  __shared__ unsigned h[kWaves][kSortMaxDigits];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int e = threadIdx.x; e < kWaves * kSortMaxDigits; e += kBlock) (&h[0][0])[e] = 0u;
  __syncthreads();
  const long base = (long)blockIdx.x * kSortTile + (long)wave * kSortWaveKeys;
  const unsigned mask = (unsigned)(digits - 1);
  unsigned key[kSortRounds];
  int idx[kSortRounds];
#pragma unroll
  for (int r = 0; r < kSortRounds; ++r) {
    const long i = base + r * 64 + lane;
    key[r] = i < n ? keys[i] : 0u;
    idx[r] = i < n ? (idx_in ? idx_in[i] : (int)i) : 0;
  }
#pragma unroll
  for (int r = 0; r < kSortRounds; ++r)
    if (base + r * 64 + lane < n) atomicAdd(&h[wave][(key[r] >> shift) & mask], 1u);
  __syncthreads();
  // counts -> where each wave's keys of each digit start
  for (int d = threadIdx.x; d < digits; d += kBlock) {
    const size_t j = (size_t)d * nblocks + blockIdx.x;
    unsigned run = table[j] + tile_start[j / kScanTile];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const unsigned c = h[w][d];
      h[w][d] = run;
      run += c;
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kSortRounds; ++r) {
    const bool valid = base + r * 64 + lane < n;
    const unsigned d = (key[r] >> shift) & mask;
    // the lanes of this round with the same digit
    unsigned long long same = __ballot(valid);
    for (int b = 0; (1 << b) < digits; ++b) {
      const bool bit = (d >> b) & 1u;
      const unsigned long long set = __ballot(bit);
      same &= bit ? set : ~set;
    }
    if (valid) {
      const unsigned rank = (unsigned)__popcll(same & ((1ull << lane) - 1ull));
      const unsigned pos = h[wave][d] + rank;
      if (rank == 0u) h[wave][d] += (unsigned)__popcll(same);  // after every lane of the wave has read
      if (keys_out) keys_out[pos] = key[r];
      idx_out[pos] = idx[r];
    }
    wave_lds_sync();  // the next round reads the counters this round advanced
  }
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

size_t elem_size(int dtype) { return dtype == DK_F64 ? 8 : dtype == DK_F32 ? 4 : 2; }

// points per wave of the channel-last kernels: as many as keep at least ~8192 waves in the grid
int points_per_wave(const NdGeo& g) {
  int ppw = 64;
  while (ppw > 1 && g.batch / ppw < 8192) ppw >>= 1;
  return ppw;
}

template <typename A, typename B>
void transpose(const A* in, B* out, long rows, long cols, hipStream_t stream) {
  const dim3 grid((unsigned)((cols + 31) / 32), (unsigned)((rows + 31) / 32));
  nd_transpose_kernel<A, B><<<grid, 256, 0, stream>>>(in, out, rows, cols);
}

}  // namespace

// The channel-last path pays for a transpose of `data`; it is taken for 1..3 dimensions in
// fp32 / fp16 / bf16 when there are enough (point, channel) pairs to amortise it.
// Few points on a tiny volume: the direct kernels and the one-launch grad data (nd_small_grad_data_kernel).
bool nd_small(const dk_nd_desc& d) {
  if (d.dtype == DK_F64 || d.dims > kClMaxDims || path_disabled(kNoNdSmall)) return false;
  long prod = 1;
  for (int i = 0; i < d.dims; ++i) prod *= d.shape[i];
  return prod <= kSmallMaxCells && d.batch > 0 && d.batch * d.channel <= (1L << 20);
}

bool nd_use_channel_last(const dk_nd_desc& d) {
  if (d.dtype == DK_F64 || d.dims > kClMaxDims || nd_small(d)) return false;
  long prod = 1;
  for (int i = 0; i < d.dims; ++i) prod *= d.shape[i];
  if (prod > 2147483647L / 4) return false;  // corner offsets are kept as 32-bit element counts
  return d.batch * d.channel >= 65536 && d.channel >= 16;
}

// Bins of the counting sort (cells of low corners plus the bin of outside points), or 0 when
// the binned kernels do not apply: they pay off with several points per cell.
int nd_bins(const dk_nd_desc& d) {
  if (!nd_use_channel_last(d) || path_disabled(kNoNdBins)) return 0;
  long bins = 1;
  for (int i = 0; i < d.dims; ++i) bins *= (long)d.shape[i] + 1;
  bins += 1;
  if (bins > 262144 || d.batch < 2 * bins || d.batch < 65536 || d.batch >= (1L << 30)) return 0;
  return (int)bins;
}

size_t round256(size_t n) { return (n + 255) / 256 * 256; }

namespace {

int key_bits(int bins) {
  int bits = 1;
  while ((1L << bits) < bins) ++bits;
  return bits;
}

}  // namespace

// bytes for the sort: keys, half-sorted keys, the sorted order of the points, the half-sorted order,
// and the (digit, workgroup) table of the radix passes with its tile sums
size_t nd_sort_workspace(const dk_nd_desc& d) {
  const int bins = nd_bins(d);
  if (!bins) return 0;
  const size_t n4 = round256((size_t)d.batch * sizeof(int));
  const size_t table = (size_t)kSortMaxDigits * ((d.batch + kSortTile - 1) / kSortTile);  // entries
  return 4 * n4 + round256((table + table / kScanTile + 1) * sizeof(unsigned));
}

size_t nd_data_cl_workspace(const dk_nd_desc& d) {
  if (!nd_use_channel_last(d)) return 0;
  size_t n = (size_t)d.channel;
  for (int i = 0; i < d.dims; ++i) n *= (size_t)d.shape[i];
  return round256(n * elem_size(d.dtype)) + nd_sort_workspace(d);
}

namespace {

// Sorts the points by cell into `order` (at `sort_ws`, laid out as nd_sort_workspace says).
template <typename T>
const int* sort_points(const NdGeo& g, const T* coord, int bins, void* sort_ws, hipStream_t stream) {
  const size_t n4 = round256((size_t)g.batch * sizeof(int));
  char* base = static_cast<char*>(sort_ws);
  unsigned* keys = reinterpret_cast<unsigned*>(base);
  unsigned* keys_sorted = reinterpret_cast<unsigned*>(base + n4);
  int* order = reinterpret_cast<int*>(base + 2 * n4);
  nd_bin_keys_kernel<T><<<(unsigned)((g.batch + kBlock - 1) / kBlock), kBlock, 0, stream>>>(g, coord, bins, keys);
  {
    // two radix passes of half the key bits each (one pass for keys of up to 9 bits)
    const int bits = key_bits(bins);
    const int lo_bits = bits <= 9 ? bits : (bits + 1) / 2, hi_bits = bits - lo_bits;
    const int nblocks = (int)((g.batch + kSortTile - 1) / kSortTile);
    int* half_order = reinterpret_cast<int*>(base + 3 * n4);
    unsigned* table = reinterpret_cast<unsigned*>(base + 4 * n4);
    unsigned* sums = table + (size_t)kSortMaxDigits * nblocks;
    auto pass = [&](const unsigned* k_in, const int* i_in, int shift, int nbits, unsigned* k_out, int* i_out) {
      const int digits = 1 << nbits, total = digits * nblocks, tiles = (total + kScanTile - 1) / kScanTile;
      radix_count_kernel<<<nblocks, kBlock, 0, stream>>>(k_in, g.batch, shift, digits, nblocks, table);
      radix_scan_tiles_kernel<<<tiles, 1024, 0, stream>>>(table, total, sums);
      radix_scan_sums_kernel<<<1, 1024, 0, stream>>>(sums, tiles);
      radix_scatter_kernel<<<nblocks, kBlock, 0, stream>>>(k_in, i_in, g.batch, shift, digits, nblocks, table, sums, k_out, i_out);
    };
    if (hi_bits == 0) {
      pass(keys, nullptr, 0, lo_bits, nullptr, order);
    } else {
      pass(keys, nullptr, 0, lo_bits, keys_sorted, half_order);
      pass(keys_sorted, half_order, lo_bits, hi_bits, nullptr, order);
    }
  }
  return order;
}

size_t data_bytes(const dk_nd_desc& d) {
  size_t n = (size_t)d.channel;
  for (int i = 0; i < d.dims; ++i) n *= (size_t)d.shape[i];
  return n;
}

}  // namespace

template <typename T>
void nd_forward(const dk_nd_desc& d, const T* data, const T* coord, T* out, void* ws, const int* order,
                hipStream_t stream) {
  const NdGeo g = make_geo(d);
  if constexpr (!std::is_same<T, double>::value) {
    if (nd_use_channel_last(d)) {
      T* data_cl = static_cast<T*>(ws);
      transpose<T, T>(data, data_cl, g.channel, g.prod_shape, stream);
      if (const int bins = nd_bins(d)) {
        if (!order) order = sort_points<T>(g, coord, bins, static_cast<char*>(ws) + round256(data_bytes(d) * sizeof(T)), stream);
        if constexpr (std::is_same<T, float>::value) {
          // rows of out are written as 16-byte vectors at multiples of 4 channels
          if (g.channel % 64 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 && !path_disabled(kNoNdMfma)) {
            nd_forward_mfma_kernel<T><<<(unsigned)((g.batch + 255) / 256), kBlock, 0, stream>>>(g, data_cl, coord, order, bins, out);
            return;
          }
        }
        nd_forward_binned_kernel<T><<<(unsigned)((g.batch + 255) / 256), kBlock, 0, stream>>>(g, data_cl, coord, order, bins, out);
        return;
      }
      const int ppw = points_per_wave(g);
      const long waves = (g.batch + ppw - 1) / ppw;
      nd_forward_cl_kernel<T><<<(unsigned)((waves + 3) / 4), kBlock, 0, stream>>>(g, data_cl, coord, out, ppw);
      return;
    }
  }
  const long total = g.batch * g.channel;
  nd_forward_kernel<T><<<grid_for(total), kBlock, 0, stream>>>(g, data, coord, out, total);
}

size_t nd_grad_data_workspace(const dk_nd_desc& d) {
  if (nd_small(d)) return 0;
  size_t n = (size_t)d.channel;
  for (int i = 0; i < d.dims; ++i) n *= (size_t)d.shape[i];
  if (nd_use_channel_last(d)) return round256(n * sizeof(float)) + nd_sort_workspace(d);  // fp32 channel-last accumulation image
  if (d.dtype == DK_F16 || d.dtype == DK_BF16) return n * sizeof(float);
  return 0;
}

template <typename T>
void nd_grad_data(const dk_nd_desc& d, const T* gout, const T* coord, T* gdata, void* ws, const int* order,
                  hipStream_t stream) {
  using CT = compute_t<T>;
  const NdGeo g = make_geo(d);
  const long n_data = (long)g.channel * g.prod_shape;
  const long total = g.batch * g.channel;
  if constexpr (!std::is_same<T, double>::value) {
    if (nd_small(d)) {
      const int nt = ((int)g.prod_shape + 15) / 16;
      // points per chunk: rows of W that fit its LDS, a multiple of 64, at most two points per thread
      int chunk = kSmallWBytes / (nt * 16 * (int)sizeof(float)) / 64 * 64;
      if (chunk > 2048) chunk = 2048;
      const size_t lds = std::max<size_t>((size_t)std::min<long>(chunk, (g.batch + 63) / 64 * 64) * nt * 16 * sizeof(float),
                                          (size_t)16 * nt * 256 * sizeof(float));
      const unsigned grid = (unsigned)((g.channel + 15) / 16);
#define DK_ND_SMALL_GD(ND, NT)                                                                                                    \
  if (lds <= 64 * 1024 || allow_dynamic_lds(reinterpret_cast<const void*>(&nd_small_grad_data_kernel<T, ND, NT>), kSmallWBytes)) \
  nd_small_grad_data_kernel<T, ND, NT><<<grid, 1024, lds, stream>>>(g, gout, coord, gdata, chunk)
#define DK_ND_SMALL_GD_NT(ND)          \
  if (nt == 1) { DK_ND_SMALL_GD(ND, 1); } \
  else if (nt == 2) { DK_ND_SMALL_GD(ND, 2); } \
  else if (nt == 3) { DK_ND_SMALL_GD(ND, 3); } \
  else { DK_ND_SMALL_GD(ND, 4); }
      if (g.dims == 1) { DK_ND_SMALL_GD_NT(1) }
      else if (g.dims == 2) { DK_ND_SMALL_GD_NT(2) }
      else { DK_ND_SMALL_GD_NT(3) }
#undef DK_ND_SMALL_GD_NT
#undef DK_ND_SMALL_GD
      return;
    }
    if (nd_use_channel_last(d)) {
      float* acc = static_cast<float*>(ws);
      nd_fill_zero_kernel<float><<<grid_for(n_data), kBlock, 0, stream>>>(acc, n_data);
      if (const int bins = nd_bins(d)) {
        if (!order) order = sort_points<T>(g, coord, bins, static_cast<char*>(ws) + round256((size_t)n_data * sizeof(float)), stream);
        // chunks of 64 points per wave: as many as keep about 16 waves per CU in the grid
        int per_wave = 1;
        while (per_wave < 8 && g.batch / (64L * per_wave * 2) >= 4096) per_wave *= 2;
        const long waves = (g.batch + 64L * per_wave - 1) / (64L * per_wave);
        bool on_matrix_cores = false;
        if constexpr (std::is_same<T, float>::value)
          // rows of gout are read as 16-byte vectors at multiples of 4 channels
          on_matrix_cores = g.channel % 64 == 0 && reinterpret_cast<uintptr_t>(gout) % 16 == 0 && !path_disabled(kNoNdMfma);
        if (on_matrix_cores) {
          if constexpr (std::is_same<T, float>::value)
            nd_grad_data_mfma_kernel<T><<<(unsigned)((waves + 3) / 4), kBlock, 0, stream>>>(g, gout, coord, order, bins, acc, per_wave);
        } else {
          nd_grad_data_binned_kernel<T><<<(unsigned)((waves + 3) / 4), kBlock, 0, stream>>>(g, gout, coord, order, bins, acc, per_wave);
        }
      } else {
        const int ppw = points_per_wave(g);
        const long waves = (g.batch + ppw - 1) / ppw;
        nd_grad_data_cl_kernel<T><<<(unsigned)((waves + 3) / 4), kBlock, 0, stream>>>(g, gout, coord, acc, ppw);
      }
      transpose<float, T>(acc, gdata, g.prod_shape, g.channel, stream);
      return;
    }
  }
  constexpr bool direct = sizeof(T) == sizeof(CT);
  CT* acc = direct ? reinterpret_cast<CT*>(gdata) : static_cast<CT*>(ws);
  nd_fill_zero_kernel<CT><<<grid_for(n_data), kBlock, 0, stream>>>(acc, n_data);
  if (total > 0)
    nd_grad_data_kernel<T, CT, false><<<grid_for(total), kBlock, 0, stream>>>(g, gout, coord, acc, total);
  if (!direct) nd_convert_kernel<CT, T><<<grid_for(n_data), kBlock, 0, stream>>>(acc, gdata, n_data);
}

template <typename T>
void nd_grad_coord(const dk_nd_desc& d, const T* gout, const T* data, const T* coord, T* gcoord,
                   void* ws, const int* order, hipStream_t stream) {
  const NdGeo g = make_geo(d);
  if constexpr (!std::is_same<T, double>::value) {
    if (nd_small(d)) {
      const unsigned grid = (unsigned)((g.batch + kBlock / 64 - 1) / (kBlock / 64));
      if (g.dims == 1) nd_small_grad_coord_kernel<T, 1><<<grid, kBlock, 0, stream>>>(g, gout, data, coord, gcoord);
      else if (g.dims == 2) nd_small_grad_coord_kernel<T, 2><<<grid, kBlock, 0, stream>>>(g, gout, data, coord, gcoord);
      else nd_small_grad_coord_kernel<T, 3><<<grid, kBlock, 0, stream>>>(g, gout, data, coord, gcoord);
      return;
    }
    if (nd_use_channel_last(d)) {
      T* data_cl = static_cast<T*>(ws);
      transpose<T, T>(data, data_cl, g.channel, g.prod_shape, stream);
      if (const int bins = nd_bins(d)) {
        if (!order) order = sort_points<T>(g, coord, bins, static_cast<char*>(ws) + round256(data_bytes(d) * sizeof(T)), stream);
        if constexpr (std::is_same<T, float>::value) {
          // rows of gout are read as 16-byte vectors at multiples of 16 channels
          if (g.channel % 64 == 0 && reinterpret_cast<uintptr_t>(gout) % 16 == 0 && !path_disabled(kNoNdMfma)) {
            nd_grad_coord_mfma_kernel<T><<<(unsigned)((g.batch + 255) / 256), kBlock, 0, stream>>>(g, gout, data_cl, coord, order, bins, gcoord);
            return;
          }
        }
        nd_grad_coord_binned_kernel<T><<<(unsigned)((g.batch + 255) / 256), kBlock, 0, stream>>>(g, gout, data_cl, coord, order, bins, gcoord);
        return;
      }
      const int ppw = points_per_wave(g);
      const long waves = (g.batch + ppw - 1) / ppw;
      nd_grad_coord_cl_kernel<T><<<(unsigned)((waves + 3) / 4), kBlock, 0, stream>>>(g, gout, data_cl, coord, gcoord, ppw);
      return;
    }
  }
  long blocks = (g.batch + 3) / 4;
  if (blocks > 65536) blocks = 65536;
  nd_grad_coord_kernel<T><<<(int)blocks, kBlock, 0, stream>>>(g, gout, data, coord, gcoord);
}

// The sorted order of the points alone, for a caller that issues several of the three calls on
// the same coordinates: `order` receives batch ints; ws as nd_sort_workspace() sizes it.
size_t nd_order_bytes(const dk_nd_desc& d) { return nd_bins(d) ? (size_t)d.batch * sizeof(int) : 0; }

template <typename T>
void nd_order(const dk_nd_desc& d, const T* coord, int* order, void* ws, hipStream_t stream) {
  const NdGeo g = make_geo(d);
  if constexpr (!std::is_same<T, double>::value) {
    if (const int bins = nd_bins(d)) {
      const int* sorted = sort_points<T>(g, coord, bins, ws, stream);
      (void)hipMemcpyAsync(order, sorted, (size_t)d.batch * sizeof(int), hipMemcpyDeviceToDevice, stream);
    }
  }
}

#define DK_INSTANTIATE(T)                                                                             \
  template void nd_forward<T>(const dk_nd_desc&, const T*, const T*, T*, void*, const int*, hipStream_t);   \
  template void nd_grad_data<T>(const dk_nd_desc&, const T*, const T*, T*, void*, const int*, hipStream_t); \
  template void nd_grad_coord<T>(const dk_nd_desc&, const T*, const T*, const T*, T*, void*, const int*,    \
                                 hipStream_t);                                                         \
  template void nd_order<T>(const dk_nd_desc&, const T*, int*, void*, hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(double)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
#undef DK_INSTANTIATE

}  // namespace dk
