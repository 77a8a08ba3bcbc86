// Depthwise convolution with one kernel per (image, channel) plane: the convolution that
// GlobalDeformKernel2d applies after it has sampled a k x k kernel for every image and channel.
// The reference runs it as nn.functional.conv2d on x.view(1, N * C, H, W) with groups = N * C
// (deformable_kernels/modules/deform_kernel.py:103-111) and lets autograd derive the gradients;
// here: forward, gradient w.r.t. the input (the transposed convolution) and gradient w.r.t. the
// per-plane kernels, for depthwise layers (one input channel per kernel).
//
//   out[p, ho, wo]  = sum_{i, j} w[p, i, j] * x[p, ho * s - pad + i * dil, wo * s - pad + j * dil]
//   gin[p, h, w]    = sum_{i, j} w[p, i, j] * gout[p, (h + pad - i * dil) / s, (w + pad - j * dil) / s]   (where divisible)
//   gw[p, i, j]     = sum_{ho, wo} gout[p, ho, wo] * x[p, ho * s - pad + i * dil, wo * s - pad + j * dil]
//
// with p = n * C + c and zero outside the plane.  All three stream their tensors once (9 multiply-
// adds per element and direction): one wave owns one plane, stages a band of source rows (with the
// zero border) in LDS as compute-type values through coalesced loads, and works on horizontal
// strips of four destination pixels, so a strip's taps are read from LDS once per row.  Waves do
// not share data; no workgroup barrier is used.
#include "dk_kernels.h"

namespace dk {
namespace {

constexpr int kWave = 64;
constexpr int kWaves = 4;             // waves (planes in flight) per workgroup
constexpr int kTileBytes = 9 * 1024;  // LDS for one wave's staged band
constexpr int kStrip = 4;
constexpr int kMaxTaps = 128;         // run-time tap counts keep the plane's kernel in LDS

// Element strides of the kernel tensor's four axes (image, channel, tap row, tap column): the kernels
// may sit as [N, C, k_h, k_w] or as the N-d sampler leaves them, [N, k_h, k_w, C].
struct WLayout {
  long n, c, i, j;
};

struct ImgConv {
  int planes, channel;
  WLayout wl;
  int src_h, src_w, dst_h, dst_w;
  int k_h, k_w, stride_h, stride_w, dil_h, dil_w;
  int org_h, org_w;  // source row / column that tap (0, 0) of destination pixel (0, 0) reads
  int flip;          // the plane's taps are applied in reverse order (transposed convolution, stride 1)
  int band_rows;     // destination rows per staged band
  int pitch;         // columns of the staged band (covers every tap of every destination column, plus slack)
  int tile_elems;    // elements of one wave's LDS region
  int vec_ok;        // destination (and, for the kernel gradient, out_grad) rows allow aligned 4-element accesses
};

__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Rows rb .. rb + rows - 1, columns org_w .. org_w + pitch - 1 of the source plane into `tile`
// (row-major, `pitch` columns), zero outside the plane.  Lanes walk the band in flat order, so
// a wave's loads cover runs of consecutive addresses.
template <typename T, typename CT>
__device__ __forceinline__ void stage_band(CT* tile, const T* __restrict__ plane, const ImgConv& a, int rb, int rows,
                                           int lane) {
  const int total = rows * a.pitch;
  int tr = lane / a.pitch, tc = lane - tr * a.pitch;
  const int dr = kWave / a.pitch, dc = kWave - dr * a.pitch;
#pragma unroll 4
  for (int idx = lane; idx < total; idx += kWave) {
    const int r = rb + tr, c = a.org_w + tc;
    CT v = CT(0);
    if ((unsigned)r < (unsigned)a.src_h && (unsigned)c < (unsigned)a.src_w) v = ld(plane + (size_t)r * a.src_w + c);
    tile[idx] = v;
    tr += dr;
    tc += dc;
    if (tc >= a.pitch) {
      tc -= a.pitch;
      ++tr;
    }
  }
}

template <typename T, typename CT>
__device__ __forceinline__ void store_strip(T* row, int oc, int width, const CT (&v)[kStrip], bool vec) {
  if (vec) {  // width is a multiple of 4 and the row start is aligned: the strip is whole
    struct alignas(sizeof(T) * kStrip) Pack { T e[kStrip]; } pk;
#pragma unroll
    for (int i = 0; i < kStrip; ++i) st(pk.e + i, v[i]);
    *reinterpret_cast<Pack*>(row + oc) = pk;
  } else {
#pragma unroll
    for (int i = 0; i < kStrip; ++i)
      if (oc + i < width) st(row + oc + i, v[i]);
  }
}

template <typename T, typename CT>
__device__ __forceinline__ void load_strip(const T* row, int oc, int width, CT (&v)[kStrip], bool vec) {
  if (vec) {
    struct alignas(sizeof(T) * kStrip) Pack { T e[kStrip]; };
    const Pack pk = *reinterpret_cast<const Pack*>(row + oc);
#pragma unroll
    for (int i = 0; i < kStrip; ++i) v[i] = ld(pk.e + i);
  } else {
#pragma unroll
    for (int i = 0; i < kStrip; ++i) v[i] = oc + i < width ? ld(row + oc + i) : CT(0);
  }
}

// The plane's taps as compute-type values: K > 0 in registers (uniform loads), K == 0 in LDS.
template <typename T, typename CT, int K>
struct Taps {
  CT w[K * K];
  __device__ __forceinline__ void load(const T* __restrict__ wp, const ImgConv& a, CT*, int) {
#pragma unroll
    for (int t = 0; t < K * K; ++t) {
      const int s = a.flip ? K * K - 1 - t : t;
      w[t] = ld(wp + (s / K) * a.wl.i + (s % K) * a.wl.j);
    }
  }
  __device__ __forceinline__ CT at(int t, const CT*) const { return w[t]; }
};
template <typename T, typename CT>
struct Taps<T, CT, 0> {
  __device__ __forceinline__ void load(const T* __restrict__ wp, const ImgConv& a, CT* lds_w, int lane) {
    const int n = a.k_h * a.k_w;
    for (int t = lane; t < n; t += kWave) {
      const int s = a.flip ? n - 1 - t : t;
      lds_w[t] = ld(wp + (s / a.k_w) * a.wl.i + (s % a.k_w) * a.wl.j);
    }
  }
  __device__ __forceinline__ CT at(int t, const CT* lds_w) const { return lds_w[t]; }
};

// Forward, and the input gradient at stride 1 (the same sum with the taps reversed and the
// origin moved: source = out_grad, org = pad - (k - 1) * dil).
// K: taps per side known at compile time (0: run-time k_h x k_w); UNIT: stride 1 and dilation 1.
template <typename T, int K, bool UNIT>
__global__ __launch_bounds__(kWave* kWaves) void image_conv_kernel(ImgConv a, const T* __restrict__ src,
                                                                   const T* __restrict__ weight, T* __restrict__ dst) {
  using CT = compute_t<T>;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int plane = blockIdx.x * kWaves + wave;
  if (plane >= a.planes) return;  // whole waves leave; nothing below synchronises across waves
  CT* tile = reinterpret_cast<CT*>(lds_raw) + (size_t)wave * (a.tile_elems + (K == 0 ? kMaxTaps : 0));
  CT* lds_w = tile + a.tile_elems;
  const int kh = K ? K : a.k_h, kw = K ? K : a.k_w;
  const int sh = UNIT ? 1 : a.stride_h, sw = UNIT ? 1 : a.stride_w, dh = UNIT ? 1 : a.dil_h, dw = UNIT ? 1 : a.dil_w;

  Taps<T, CT, K> taps;
  taps.load(weight + (plane / a.channel) * a.wl.n + (plane % a.channel) * a.wl.c, a, lds_w, lane);
  const T* sp = src + (size_t)plane * a.src_h * a.src_w;
  T* dp = dst + (size_t)plane * a.dst_h * a.dst_w;
  const int strips = (a.dst_w + kStrip - 1) / kStrip;
  const int dro = kWave / strips, dso = kWave - dro * strips;

  for (int o0 = 0; o0 < a.dst_h; o0 += a.band_rows) {
    const int rows = min(a.band_rows, a.dst_h - o0);
    const int src_rows = (rows - 1) * sh + (kh - 1) * dh + 1;
    wave_sync();  // the previous band's reads are done before the tile is overwritten
    stage_band<T, CT>(tile, sp, a, o0 * sh + a.org_h, src_rows, lane);
    wave_sync();
    const int items = rows * strips;
    int orow = lane / strips, os = lane - orow * strips;
    for (int item = lane; item < items; item += kWave) {
      const int oc = os * kStrip;
      const CT* t0 = tile + orow * sh * a.pitch + oc * sw;
      CT acc[kStrip];
#pragma unroll
      for (int i = 0; i < kStrip; ++i) acc[i] = CT(0);
      if constexpr (K > 0 && UNIT) {
#pragma unroll
        for (int i = 0; i < K; ++i) {
          CT xr[kStrip + K - 1];
#pragma unroll
          for (int c = 0; c < kStrip + K - 1; ++c) xr[c] = t0[i * a.pitch + c];
#pragma unroll
          for (int j = 0; j < K; ++j)
#pragma unroll
            for (int p = 0; p < kStrip; ++p) acc[p] += taps.at(i * K + j, lds_w) * xr[p + j];
        }
      } else {
        for (int i = 0; i < kh; ++i)
          for (int j = 0; j < kw; ++j) {
            const CT wv = taps.at(i * kw + j, lds_w);
            const CT* t = t0 + i * dh * a.pitch + j * dw;
#pragma unroll
            for (int p = 0; p < kStrip; ++p) acc[p] += wv * t[p * sw];
          }
      }
      store_strip<T, CT>(dp + (size_t)(o0 + orow) * a.dst_w, oc, a.dst_w, acc, a.vec_ok != 0);
      orow += dro;
      os += dso;
      if (os >= strips) {
        os -= strips;
        ++orow;
      }
    }
  }
}

// Input gradient for strides above 1: one lane per input pixel, taps whose position is not on the
// stride's grid skipped; out_grad is read through the caches (it is 1 / (s_h * s_w) of the input's size).
template <typename T>
__global__ __launch_bounds__(256) void image_conv_grad_input_strided_kernel(ImgConv a, int pad_h, int pad_w,
                                                                            const T* __restrict__ gout,
                                                                            const T* __restrict__ weight,
                                                                            T* __restrict__ gin) {
  using CT = compute_t<T>;
  // here src_* is the input plane (the result) and dst_* the output plane (out_grad)
  const long total = (long)a.planes * a.src_h * a.src_w;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
    const int w = (int)(idx % a.src_w);
    const long rest = idx / a.src_w;
    const int h = (int)(rest % a.src_h);
    const long plane = rest / a.src_h;
    const T* gp = gout + plane * a.dst_h * a.dst_w;
    const T* wp = weight + (plane / a.channel) * a.wl.n + (plane % a.channel) * a.wl.c;
    CT acc = CT(0);
    for (int i = 0; i < a.k_h; ++i) {
      const int hh = h + pad_h - i * a.dil_h;
      if (hh < 0 || hh % a.stride_h != 0) continue;
      const int ho = hh / a.stride_h;
      if (ho >= a.dst_h) continue;
      for (int j = 0; j < a.k_w; ++j) {
        const int ww = w + pad_w - j * a.dil_w;
        if (ww < 0 || ww % a.stride_w != 0) continue;
        const int wo = ww / a.stride_w;
        if (wo >= a.dst_w) continue;
        acc += ld(wp + i * a.wl.i + j * a.wl.j) * ld(gp + (size_t)ho * a.dst_w + wo);
      }
    }
    st(gin + idx, acc);
  }
}

// Sum of v over the wave for compute types: float through DPP adds, double through shuffles.
__device__ __forceinline__ float plane_sum(float v) { return wave_sum(v); }
__device__ __forceinline__ double plane_sum(double v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
}

// Gradient w.r.t. the plane's kernel: the wave walks its plane band by band with one running sum
// per tap and lane, then adds the 64 lanes up.
template <typename T, int K, bool UNIT>
__global__ __launch_bounds__(kWave* kWaves) void image_conv_grad_weight_kernel(ImgConv a, const T* __restrict__ gout,
                                                                               const T* __restrict__ x,
                                                                               T* __restrict__ gweight) {
  using CT = compute_t<T>;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int plane = blockIdx.x * kWaves + wave;
  if (plane >= a.planes) return;
  CT* tile = reinterpret_cast<CT*>(lds_raw) + (size_t)wave * (a.tile_elems + (K == 0 ? kMaxTaps : 0));
  CT* lds_w = tile + a.tile_elems;  // K == 0: the running sums of this wave's lanes are folded here tap by tap
  const int kh = K ? K : a.k_h, kw = K ? K : a.k_w;
  const int sh = UNIT ? 1 : a.stride_h, sw = UNIT ? 1 : a.stride_w, dh = UNIT ? 1 : a.dil_h, dw = UNIT ? 1 : a.dil_w;
  const T* xp = x + (size_t)plane * a.src_h * a.src_w;
  const T* gp = gout + (size_t)plane * a.dst_h * a.dst_w;
  T* wp = gweight + (plane / a.channel) * a.wl.n + (plane % a.channel) * a.wl.c;
  const int strips = (a.dst_w + kStrip - 1) / kStrip;
  const int dro = kWave / strips, dso = kWave - dro * strips;

  if constexpr (K > 0) {
    CT sum[K * K];
#pragma unroll
    for (int t = 0; t < K * K; ++t) sum[t] = CT(0);
    for (int o0 = 0; o0 < a.dst_h; o0 += a.band_rows) {
      const int rows = min(a.band_rows, a.dst_h - o0);
      const int src_rows = (rows - 1) * sh + (K - 1) * dh + 1;
      wave_sync();
      stage_band<T, CT>(tile, xp, a, o0 * sh + a.org_h, src_rows, lane);
      wave_sync();
      const int items = rows * strips;
      int orow = lane / strips, os = lane - orow * strips;
      for (int item = lane; item < items; item += kWave) {
        const int oc = os * kStrip;
        CT gv[kStrip];
        load_strip<T, CT>(gp + (size_t)(o0 + orow) * a.dst_w, oc, a.dst_w, gv, a.vec_ok != 0);
        const CT* t0 = tile + orow * sh * a.pitch + oc * sw;
        if constexpr (UNIT) {
#pragma unroll
          for (int i = 0; i < K; ++i) {
            CT xr[kStrip + K - 1];
#pragma unroll
            for (int c = 0; c < kStrip + K - 1; ++c) xr[c] = t0[i * a.pitch + c];
#pragma unroll
            for (int j = 0; j < K; ++j)
#pragma unroll
              for (int p = 0; p < kStrip; ++p) sum[i * K + j] += gv[p] * xr[p + j];
          }
        } else {
#pragma unroll
          for (int i = 0; i < K; ++i)
#pragma unroll
            for (int j = 0; j < K; ++j) {
              const CT* t = t0 + i * dh * a.pitch + j * dw;
#pragma unroll
              for (int p = 0; p < kStrip; ++p) sum[i * K + j] += gv[p] * t[p * sw];
            }
        }
        orow += dro;
        os += dso;
        if (os >= strips) {
          os -= strips;
          ++orow;
        }
      }
    }
#pragma unroll
    for (int t = 0; t < K * K; ++t) {
      const CT total = plane_sum(sum[t]);
      if (lane == t % kWave) st(wp + (t / K) * a.wl.i + (t % K) * a.wl.j, total);
    }
  } else {
    // run-time tap count: one tap at a time over the whole plane (the tile is re-staged per band
    // and tap; this form serves unusual kernel sizes only)
    const int ntaps = kh * kw;
    for (int t = 0; t < ntaps; ++t) {
      const int i = t / kw, j = t - i * kw;
      CT sum = CT(0);
      for (int o0 = 0; o0 < a.dst_h; o0 += a.band_rows) {
        const int rows = min(a.band_rows, a.dst_h - o0);
        const int src_rows = (rows - 1) * sh + (kh - 1) * dh + 1;
        wave_sync();
        stage_band<T, CT>(tile, xp, a, o0 * sh + a.org_h, src_rows, lane);
        wave_sync();
        const int items = rows * strips;
        int orow = lane / strips, os = lane - orow * strips;
        for (int item = lane; item < items; item += kWave) {
          const int oc = os * kStrip;
          CT gv[kStrip];
          load_strip<T, CT>(gp + (size_t)(o0 + orow) * a.dst_w, oc, a.dst_w, gv, a.vec_ok != 0);
          const CT* tp = tile + (orow * sh + i * dh) * a.pitch + oc * sw + j * dw;
#pragma unroll
          for (int p = 0; p < kStrip; ++p) sum += gv[p] * tp[p * sw];
          orow += dro;
          os += dso;
          if (os >= strips) {
            os -= strips;
            ++orow;
          }
        }
      }
      const CT total = plane_sum(sum);
      if (lane == 0) st(wp + i * a.wl.i + j * a.wl.j, total);
    }
    (void)lds_w;
  }
}

// ---- host side --------------------------------------------------------------------------

// Band height and LDS layout for a pass whose destination plane is dst_h x dst_w; false when not
// even one destination row's taps fit a wave's LDS region.
bool plan(ImgConv& a, size_t elem_bytes) {
  a.pitch = (a.dst_w - 1) * a.stride_w + (a.k_w - 1) * a.dil_w + 1 + (kStrip - 1) * a.stride_w;
  const long budget = kTileBytes / (long)elem_bytes;
  const long one_row = (long)((a.k_h - 1) * a.dil_h + 1) * a.pitch;
  if (one_row > budget || (long)a.k_h * a.k_w > kMaxTaps) return false;
  // rows * stride_h more source rows per further destination row
  long rows = 1 + (budget - one_row) / ((long)a.stride_h * a.pitch);
  if (rows > a.dst_h) rows = a.dst_h;
  a.band_rows = (int)rows;
  a.tile_elems = (int)(((a.band_rows - 1) * (long)a.stride_h + (a.k_h - 1) * a.dil_h + 1) * a.pitch);
  a.tile_elems = (a.tile_elems + 3) & ~3;
  return true;
}

bool aligned_rows(const void* p, int width, size_t elem_bytes) {
  return width % kStrip == 0 && reinterpret_cast<uintptr_t>(p) % (elem_bytes * kStrip) == 0;
}

// ---------------------------------------------------------------------------
// 3 x 3 taps, stride 1, dilation 1, padding 1 (output plane = input plane), 16- and 32-bit types:
// the shape of GlobalDeformKernel2d's layers, and of the input gradient of that shape.
//
// A band of rows and its two halo rows are one contiguous range of the tensor, so the band is
// staged as a flat copy: 16-byte loads from the aligned address below the range (zeros
// beyond the tensor's ends), converted and written to LDS in the same flat order; the halo row above the plane's first row and below its last is then zeroed,
// and the taps left of column 0 / right of column W - 1 -- which are the neighbouring rows' end
// elements in the flat order -- are masked when they are read.  Each wave walks its planes
// (plane = wave index, + number of waves, ...) with the next band's loads and taps in flight
// while it computes the current one.
// ---------------------------------------------------------------------------
typedef unsigned u4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));
constexpr int kFront = 8;  // elements before a wave's staged range: the tap left of the first element reads there

template <typename T> constexpr int kPer = 16 / (int)sizeof(T);  // elements of a 16-byte load

__device__ __forceinline__ void unpack(u4 v, float (&f)[4], const float*) {
  // (through scalars: __builtin_bit_cast applied to v.y itself reads the vector's first element)
  const unsigned u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(u[i]);
}
__device__ __forceinline__ void unpack(u4 v, float (&f)[8], const __half*) {
  const unsigned u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = static_cast<float>(__builtin_bit_cast(_Float16, (unsigned short)(u[i] & 0xffffu)));
    f[2 * i + 1] = static_cast<float>(__builtin_bit_cast(_Float16, (unsigned short)(u[i] >> 16)));
  }
}
__device__ __forceinline__ void unpack(u4 v, float (&f)[8], const bf16_t*) {
  const unsigned u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(u[i] << 16);
    f[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
  }
}

struct FlatConv {
  int planes, channel;
  WLayout wl;
  int h, w, hw;
  int band_rows, bands;  // rows per band, bands per plane
  int flip;
  int tile_elems;        // floats of one staged range in LDS (kFront included)
  int vec_ok;            // the width is a multiple of 4 and the destination rows are aligned: whole-strip stores
};

// One (plane, band) of a wave's walk; everything here is uniform over the wave.
struct FlatUnit {
  int plane, band;
  int r0, r1;    // rows of the band
  int first;     // element index (whole tensor, may be negative) of the aligned start of the halo'd range
  int shift;     // position of the halo row's first element after `first`
  int chunks;    // 16-byte chunks that cover the range
};

template <typename T>
__device__ __forceinline__ FlatUnit flat_unit(const FlatConv& a, int plane, int band, bool halo) {
  FlatUnit u;
  u.plane = plane, u.band = band;
  u.r0 = band * a.band_rows;
  u.r1 = min(a.h, u.r0 + a.band_rows);
  const int rows = u.r1 - u.r0 + (halo ? 2 : 0);
  const int e0 = plane * a.hw + (u.r0 - (halo ? 1 : 0)) * a.w;  // the tensor has fewer than 2^31 bytes
  u.first = (e0 >= 0 ? e0 / kPer<T> : -((-e0 + kPer<T> - 1) / kPer<T>)) * kPer<T>;
  u.shift = e0 - u.first;
  u.chunks = (u.shift + rows * a.w + kPer<T> - 1) / kPer<T>;
  return u;
}

template <typename T, int NCH>
struct FlatLoads {
  u4 v[NCH];
  // `total`: elements of the tensor, a multiple of a chunk.  A range reaches beyond the tensor's
  // ends only with the halo row above the first plane and below the last one, which is zeroed after the
  // copy: those chunks load the tensor's first / last chunk instead (no branch, no access outside).
  __device__ __forceinline__ void issue(const T* __restrict__ src, long total, const FlatUnit& u, int lane) {
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      // Every lane loads every time (a lane past the range repeats the range's last chunk, which
      // commit() then leaves out): with a fixed number of loads per unit the waits on them can be
      // counted, and the next unit's loads stay in flight behind this unit's arithmetic.
      const int chunk = min(lane + kWave * j, u.chunks - 1);
      long e = (long)u.first + chunk * kPer<T>;
      e = e < 0 ? 0 : e;
      e = e > total - kPer<T> ? total - kPer<T> : e;
      v[j] = *reinterpret_cast<const u4*>(src + e);
    }
  }
  __device__ __forceinline__ void commit(float* tile, const FlatUnit& u, int lane) const {
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int chunk = lane + kWave * j;
      if (chunk < u.chunks) {
        float f[kPer<T>];
        unpack(v[j], f, (const T*)nullptr);
        f4* dst = reinterpret_cast<f4*>(tile + kFront + chunk * kPer<T>);
#pragma unroll
        for (int q = 0; q < kPer<T> / 4; ++q) dst[q] = f4{f[4 * q], f[4 * q + 1], f[4 * q + 2], f[4 * q + 3]};
      }
    }
  }
};

// Orders the wave's LDS writes before its LDS reads (and the other way round) without waiting for
// the global loads in flight: a wave's LDS operations execute in program order, so only the compiler
// has to be kept from moving them across this point.
__device__ __forceinline__ void lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
}

__device__ __forceinline__ void zero_row(float* row, int w, int lane) {
  for (int c = lane; c < w; c += kWave) row[c] = 0.f;
}

// Columns oc - 1 .. oc + 4 of three consecutive staged rows, zero where the column is outside the plane.
// (PR + 2 rows for a patch of PR output rows)
template <bool W4, int PR>
__device__ __forceinline__ void load_rows(const float* top, int w, int oc, float (&x)[PR + 2][kStrip + 2]) {
#pragma unroll
  for (int i = 0; i < PR + 2; ++i)
#pragma unroll
    for (int c = 0; c < kStrip + 2; ++c) x[i][c] = top[i * w + c];
  if constexpr (W4) {  // only the strip's outer columns can be outside
    const bool left = oc == 0, right = oc + kStrip == w;
#pragma unroll
    for (int i = 0; i < PR + 2; ++i) {
      x[i][0] = left ? 0.f : x[i][0];
      x[i][kStrip + 1] = right ? 0.f : x[i][kStrip + 1];
    }
  } else {
#pragma unroll
    for (int c = 0; c < kStrip + 2; ++c) {
      const bool outside = (unsigned)(oc - 1 + c) >= (unsigned)w;
#pragma unroll
      for (int i = 0; i < PR + 2; ++i) x[i][c] = outside ? 0.f : x[i][c];
    }
  }
}

__device__ __forceinline__ long tap_offset(const WLayout& wl, int t) { return (t / 3) * wl.i + (t % 3) * wl.j; }

// PR: output rows of a lane's patch (1, or 4 when the band's rows are a multiple of 4: the six staged
// rows a patch reads serve four output rows instead of three rows serving one)
template <typename T, int NCH, bool W4, int PR>
__global__ __launch_bounds__(kWave* kWaves) void image_conv3_flat_kernel(FlatConv a, const T* __restrict__ src,
                                                                         const T* __restrict__ weight,
                                                                         T* __restrict__ dst) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int first_plane = blockIdx.x * kWaves + wave, step = gridDim.x * kWaves;
  if (first_plane >= a.planes) return;  // whole waves leave; nothing below synchronises across waves
  float* tile = reinterpret_cast<float*>(lds_raw) + (size_t)wave * a.tile_elems;
  const long total = (long)a.planes * a.hw;
  const int strips = (a.w + kStrip - 1) / kStrip;
  const int dro = kWave / strips, dso = kWave - dro * strips;

  // lane t < 9 holds tap t of the plane (reversed for the transposed sum); the other lanes load tap 8 again
  // rather than branch around the load
  const long my_tap = tap_offset(a.wl, a.flip ? 8 - min(lane, 8) : min(lane, 8));
  // (kept as stored and converted when it is used: a conversion here would wait for the load)
  auto taps_of = [&](int plane) { return weight[(plane / a.channel) * a.wl.n + (plane % a.channel) * a.wl.c + my_tap]; };

  FlatUnit cur = flat_unit<T>(a, first_plane, 0, true);
  FlatLoads<T, NCH> loads;
  loads.issue(src, total, cur, lane);
  T taps_next = taps_of(first_plane);
  for (;;) {
    loads.commit(tile, cur, lane);
    float taps_cur = ld(&taps_next);
    asm volatile("" : "+v"(taps_cur));  // converted here, before the next loads are issued, not next to its use
    if (cur.r0 == 0) zero_row(tile + kFront + cur.shift, a.w, lane);
    if (cur.r1 == a.h) zero_row(tile + kFront + cur.shift + (cur.r1 - cur.r0 + 1) * a.w, a.w, lane);
    // the next band's loads fly while this one is computed
    const bool more_bands = cur.band + 1 < a.bands;
    const int next_plane = more_bands ? cur.plane : cur.plane + step;
    const bool more = next_plane < a.planes;
    const FlatUnit nxt = flat_unit<T>(a, more ? next_plane : cur.plane, more_bands ? cur.band + 1 : 0, true);
    if (more) {
      loads.issue(src, total, nxt, lane);
      if (!more_bands) taps_next = taps_of(next_plane);
    }
    lds_sync();
    float w9[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) w9[t] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, taps_cur), t));
    T* dp = dst + (size_t)cur.plane * a.hw;
    const float* band = tile + kFront + cur.shift - 1;  // column -1 of the halo row above the band's first row
    const int items = (cur.r1 - cur.r0) / PR * strips;
    int orow = lane / strips, os = lane - orow * strips;  // orow counts patches
    for (int item = lane; item < items; item += kWave) {
      const int oc = os * kStrip;
      float x[PR + 2][kStrip + 2];
      load_rows<W4, PR>(band + orow * PR * a.w + oc, a.w, oc, x);
#pragma unroll
      for (int pr = 0; pr < PR; ++pr) {
        float acc[kStrip] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
          for (int j = 0; j < 3; ++j)
#pragma unroll
            for (int p = 0; p < kStrip; ++p) acc[p] = fmaf(w9[i * 3 + j], x[pr + i][p + j], acc[p]);
        store_strip<T, float>(dp + (size_t)(cur.r0 + orow * PR + pr) * a.w, oc, a.w, acc, W4);
      }
      orow += dro;
      os += dso;
      if (os >= strips) {
        os -= strips;
        ++orow;
      }
    }
    if (!more) break;
    lds_sync();  // every lane has read its rows before the next band overwrites them
    cur = nxt;
  }
}

// Kernel gradient of that shape: input band (with halo) and out_grad band staged the same way, nine
// running sums per lane over the plane's bands, added up over the wave when the plane is done.
template <typename T, int NCH, bool W4, int PR>
__global__ __launch_bounds__(kWave* kWaves) void image_conv3_flat_grad_weight_kernel(FlatConv a,
                                                                                     const T* __restrict__ gout,
                                                                                     const T* __restrict__ x,
                                                                                     T* __restrict__ gweight) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int first_plane = blockIdx.x * kWaves + wave, step = gridDim.x * kWaves;
  if (first_plane >= a.planes) return;
  float* xtile = reinterpret_cast<float*>(lds_raw) + (size_t)wave * 2 * a.tile_elems;
  float* gtile = xtile + a.tile_elems;
  const long total = (long)a.planes * a.hw;
  const int strips = (a.w + kStrip - 1) / kStrip;
  const int dro = kWave / strips, dso = kWave - dro * strips;

  FlatUnit cur = flat_unit<T>(a, first_plane, 0, true), gcur = flat_unit<T>(a, first_plane, 0, false);
  FlatLoads<T, NCH> xl, gl;
  xl.issue(x, total, cur, lane);
  gl.issue(gout, total, gcur, lane);
  float sum[9];
#pragma unroll
  for (int t = 0; t < 9; ++t) sum[t] = 0.f;
  for (;;) {
    xl.commit(xtile, cur, lane);
    gl.commit(gtile, gcur, lane);
    if (cur.r0 == 0) zero_row(xtile + kFront + cur.shift, a.w, lane);
    if (cur.r1 == a.h) zero_row(xtile + kFront + cur.shift + (cur.r1 - cur.r0 + 1) * a.w, a.w, lane);
    const bool more_bands = cur.band + 1 < a.bands;
    const int next_plane = more_bands ? cur.plane : cur.plane + step;
    const bool more = next_plane < a.planes;
    const FlatUnit nxt = flat_unit<T>(a, more ? next_plane : cur.plane, more_bands ? cur.band + 1 : 0, true);
    const FlatUnit gnxt = flat_unit<T>(a, more ? next_plane : cur.plane, more_bands ? cur.band + 1 : 0, false);
    if (more) {
      xl.issue(x, total, nxt, lane);
      gl.issue(gout, total, gnxt, lane);
    }
    lds_sync();
    const float* band = xtile + kFront + cur.shift - 1;
    const float* gband = gtile + kFront + gcur.shift;
    const int items = (cur.r1 - cur.r0) / PR * strips;
    int orow = lane / strips, os = lane - orow * strips;  // orow counts patches
    for (int item = lane; item < items; item += kWave) {
      const int oc = os * kStrip;
      float xv[PR + 2][kStrip + 2];
      load_rows<W4, PR>(band + orow * PR * a.w + oc, a.w, oc, xv);
      float gv[PR][kStrip];
#pragma unroll
      for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int p = 0; p < kStrip; ++p) {
          gv[pr][p] = gband[(orow * PR + pr) * a.w + oc + p];
          if constexpr (!W4) gv[pr][p] = oc + p < a.w ? gv[pr][p] : 0.f;
        }
#pragma unroll
      for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
          for (int j = 0; j < 3; ++j)
#pragma unroll
            for (int p = 0; p < kStrip; ++p) sum[i * 3 + j] = fmaf(gv[pr][p], xv[pr + i][p + j], sum[i * 3 + j]);
      orow += dro;
      os += dso;
      if (os >= strips) {
        os -= strips;
        ++orow;
      }
    }
    if (!more_bands) {  // the plane is done
      float mine = 0.f;
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        const float total = wave_sum(sum[t]);
        mine = lane == t ? total : mine;
        sum[t] = 0.f;
      }
      if (lane < 9)
        st(gweight + (cur.plane / a.channel) * a.wl.n + (cur.plane % a.channel) * a.wl.c + tap_offset(a.wl, lane), mine);
    }
    if (!more) break;
    lds_sync();
    cur = nxt;
    gcur = gnxt;
  }
}

// ---------------------------------------------------------------------------
// The flat kernels for 16-bit tensors whose rows are a multiple of 4 elements: the staged range stays packed (two
// elements per LDS word, written as loaded: no conversion when it is staged, half the LDS traffic) and the sums
// run on v_dot2_f32_{f16,bf16} (two products per instruction, fp32 accumulation).  With rows and planes of an even
// number of elements the pair (x[c], x[c + 1]) of an even column c is one word.  An output of an even column takes
// (w1, w2) . (x[c], x[c + 1]) + (0, w0) . (x[c - 2], x[c - 1]), one of an odd column (w0, w1) . (x[c - 1], x[c]) +
// (w2, 0) . (x[c + 1], x[c + 2]): six instructions per output instead of nine multiply-adds.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float dot2(unsigned a, unsigned b, float c, const __half*) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, a), __builtin_bit_cast(h2, b), c, false);
}
__device__ __forceinline__ float dot2(unsigned a, unsigned b, float c, const bf16_t*) {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, a), __builtin_bit_cast(b2, b), c, false);
}
// (lo, hi) as two elements of the tensor's type in one word; the values are exact in that type
__device__ __forceinline__ unsigned pack2(float lo, float hi, const __half*) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(unsigned, h2{static_cast<_Float16>(lo), static_cast<_Float16>(hi)});
}
__device__ __forceinline__ unsigned pack2(float lo, float hi, const bf16_t*) { return pack_bf16(lo, hi); }

template <typename T, int NCH>
struct FlatLoads16 : FlatLoads<T, NCH> {
  // the chunks go to the tile as they are
  __device__ __forceinline__ void commit16(unsigned* tile, const FlatUnit& u, int lane) const {
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int chunk = lane + kWave * j;
      if (chunk < u.chunks) *reinterpret_cast<u4*>(tile + (kFront + chunk * kPer<T>) / 2) = this->v[j];
    }
  }
};

__device__ __forceinline__ void zero_row16(unsigned* row, int w, int lane) {
  for (int c = lane; c < w / 2; c += kWave) row[c] = 0u;
}

// The words of columns oc - 2 .. oc + 5 of PR + 2 consecutive staged rows (oc a multiple of 4); the element left
// of column 0 and the one right of the last column read as zero (only the outer words can hold them).
template <int PR>
__device__ __forceinline__ void load_rows16(const unsigned* top, int w, int oc, unsigned (&x)[PR + 2][4]) {
  const bool left = oc == 0, right = oc + kStrip == w;
#pragma unroll
  for (int i = 0; i < PR + 2; ++i) {
#pragma unroll
    for (int c = 0; c < 4; ++c) x[i][c] = top[(i * w) / 2 + c];
    x[i][0] = left ? 0u : x[i][0];
    x[i][3] = right ? 0u : x[i][3];
  }
}

template <typename T, int NCH, int PR>
__global__ __launch_bounds__(kWave* kWaves) void image_conv3_flat16_kernel(FlatConv a, const T* __restrict__ src,
                                                                           const T* __restrict__ weight,
                                                                           T* __restrict__ dst) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int first_plane = blockIdx.x * kWaves + wave, step = gridDim.x * kWaves;
  if (first_plane >= a.planes) return;
  unsigned* tile = reinterpret_cast<unsigned*>(lds_raw) + (size_t)wave * (a.tile_elems / 2);
  const long total = (long)a.planes * a.hw;
  const int strips = a.w / kStrip;
  const int dro = kWave / strips, dso = kWave - dro * strips;
  const long my_tap = tap_offset(a.wl, a.flip ? 8 - min(lane, 8) : min(lane, 8));
  auto taps_of = [&](int plane) { return weight[(plane / a.channel) * a.wl.n + (plane % a.channel) * a.wl.c + my_tap]; };

  FlatUnit cur = flat_unit<T>(a, first_plane, 0, true);
  FlatLoads16<T, NCH> loads;
  loads.issue(src, total, cur, lane);
  T taps_next = taps_of(first_plane);
  for (;;) {
    loads.commit16(tile, cur, lane);
    float taps_cur = ld(&taps_next);
    asm volatile("" : "+v"(taps_cur));
    // the halo rows above the first and below the last row of the plane (the range starts at an even element)
    if (cur.r0 == 0) zero_row16(tile + (kFront + cur.shift) / 2, a.w, lane);
    if (cur.r1 == a.h) zero_row16(tile + (kFront + cur.shift + (cur.r1 - cur.r0 + 1) * a.w) / 2, a.w, lane);
    const bool more_bands = cur.band + 1 < a.bands;
    const int next_plane = more_bands ? cur.plane : cur.plane + step;
    const bool more = next_plane < a.planes;
    const FlatUnit nxt = flat_unit<T>(a, more ? next_plane : cur.plane, more_bands ? cur.band + 1 : 0, true);
    if (more) {
      loads.issue(src, total, nxt, lane);
      if (!more_bands) taps_next = taps_of(next_plane);
    }
    lds_sync();
    float w9[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) w9[t] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, taps_cur), t));
    unsigned wa[3], wb[3], wc[3], wd[3];  // (w1, w2), (0, w0), (w0, w1), (w2, 0) of each tap row
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      wa[i] = pack2(w9[3 * i + 1], w9[3 * i + 2], src);
      wb[i] = pack2(0.f, w9[3 * i], src);
      wc[i] = pack2(w9[3 * i], w9[3 * i + 1], src);
      wd[i] = pack2(w9[3 * i + 2], 0.f, src);
    }
    T* dp = dst + (size_t)cur.plane * a.hw;
    const unsigned* band = tile + (kFront + cur.shift - 2) / 2;  // column -2 of the halo row above the band's first row
    const int items = (cur.r1 - cur.r0) / PR * strips;
    int orow = lane / strips, os = lane - orow * strips;
    for (int item = lane; item < items; item += kWave) {
      const int oc = os * kStrip;
      unsigned x[PR + 2][4];
      load_rows16<PR>(band + (orow * PR * a.w + oc) / 2, a.w, oc, x);
#pragma unroll
      for (int pr = 0; pr < PR; ++pr) {
        float acc[kStrip] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 3; ++i) {
          const unsigned* r = x[pr + i];
          acc[0] = dot2(r[1], wa[i], dot2(r[0], wb[i], acc[0], src), src);
          acc[1] = dot2(r[1], wc[i], dot2(r[2], wd[i], acc[1], src), src);
          acc[2] = dot2(r[2], wa[i], dot2(r[1], wb[i], acc[2], src), src);
          acc[3] = dot2(r[2], wc[i], dot2(r[3], wd[i], acc[3], src), src);
        }
        store_strip<T, float>(dp + (size_t)(cur.r0 + orow * PR + pr) * a.w, oc, a.w, acc, true);
      }
      orow += dro;
      os += dso;
      if (os >= strips) {
        os -= strips;
        ++orow;
      }
    }
    if (!more) break;
    lds_sync();
    cur = nxt;
  }
}

// Kernel gradient of that shape: per staged row the three alignments of its pairs -- (x[c - 1], x[c]), (x[c], x[c + 1]),
// (x[c + 1], x[c + 2]) for the even columns of the strip -- are formed once (v_alignbit_b32) and serve the three
// tap rows that read the row; a pair of out_grad elements against a pair of inputs is one instruction.
template <typename T, int NCH, int PR>
__global__ __launch_bounds__(kWave* kWaves) void image_conv3_flat16_grad_weight_kernel(FlatConv a,
                                                                                       const T* __restrict__ gout,
                                                                                       const T* __restrict__ x,
                                                                                       T* __restrict__ gweight) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int first_plane = blockIdx.x * kWaves + wave, step = gridDim.x * kWaves;
  if (first_plane >= a.planes) return;
  unsigned* xtile = reinterpret_cast<unsigned*>(lds_raw) + (size_t)wave * a.tile_elems;  // two tiles of tile_elems / 2 words
  unsigned* gtile = xtile + a.tile_elems / 2;
  const long total = (long)a.planes * a.hw;
  const int strips = a.w / kStrip;
  const int dro = kWave / strips, dso = kWave - dro * strips;

  FlatUnit cur = flat_unit<T>(a, first_plane, 0, true), gcur = flat_unit<T>(a, first_plane, 0, false);
  FlatLoads16<T, NCH> xl, gl;
  xl.issue(x, total, cur, lane);
  gl.issue(gout, total, gcur, lane);
  float sum[9];
#pragma unroll
  for (int t = 0; t < 9; ++t) sum[t] = 0.f;
  for (;;) {
    xl.commit16(xtile, cur, lane);
    gl.commit16(gtile, gcur, lane);
    if (cur.r0 == 0) zero_row16(xtile + (kFront + cur.shift) / 2, a.w, lane);
    if (cur.r1 == a.h) zero_row16(xtile + (kFront + cur.shift + (cur.r1 - cur.r0 + 1) * a.w) / 2, a.w, lane);
    const bool more_bands = cur.band + 1 < a.bands;
    const int next_plane = more_bands ? cur.plane : cur.plane + step;
    const bool more = next_plane < a.planes;
    const FlatUnit nxt = flat_unit<T>(a, more ? next_plane : cur.plane, more_bands ? cur.band + 1 : 0, true);
    const FlatUnit gnxt = flat_unit<T>(a, more ? next_plane : cur.plane, more_bands ? cur.band + 1 : 0, false);
    if (more) {
      xl.issue(x, total, nxt, lane);
      gl.issue(gout, total, gnxt, lane);
    }
    lds_sync();
    const unsigned* band = xtile + (kFront + cur.shift - 2) / 2;
    const unsigned* gband = gtile + (kFront + gcur.shift) / 2;
    const int items = (cur.r1 - cur.r0) / PR * strips;
    int orow = lane / strips, os = lane - orow * strips;
    for (int item = lane; item < items; item += kWave) {
      const int oc = os * kStrip;
      unsigned xv[PR + 2][4];
      load_rows16<PR>(band + (orow * PR * a.w + oc) / 2, a.w, oc, xv);
      unsigned gv[PR][2];
#pragma unroll
      for (int pr = 0; pr < PR; ++pr)
#pragma unroll
        for (int p = 0; p < 2; ++p) gv[pr][p] = gband[((orow * PR + pr) * a.w + oc) / 2 + p];
#pragma unroll
      for (int r = 0; r < PR + 2; ++r) {
        // pairs of the row for the taps' three columns, for the strip's columns (0, 1) and (2, 3)
        const unsigned l0 = __builtin_amdgcn_alignbit(xv[r][1], xv[r][0], 16), l1 = __builtin_amdgcn_alignbit(xv[r][2], xv[r][1], 16);
        const unsigned r1_ = __builtin_amdgcn_alignbit(xv[r][3], xv[r][2], 16);
        const unsigned p0[3] = {l0, xv[r][1], l1}, p1[3] = {l1, xv[r][2], r1_};
#pragma unroll
        for (int i = 0; i < 3; ++i) {
          const int pr = r - i;  // the output row that reads staged row r through tap row i
          if (pr < 0 || pr >= PR) continue;
#pragma unroll
          for (int j = 0; j < 3; ++j)
            sum[i * 3 + j] = dot2(gv[pr][1], p1[j], dot2(gv[pr][0], p0[j], sum[i * 3 + j], x), x);
        }
      }
      orow += dro;
      os += dso;
      if (os >= strips) {
        os -= strips;
        ++orow;
      }
    }
    if (!more_bands) {  // the plane is done
      float mine = 0.f;
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        const float total_ = wave_sum(sum[t]);
        mine = lane == t ? total_ : mine;
        sum[t] = 0.f;
      }
      if (lane < 9)
        st(gweight + (cur.plane / a.channel) * a.wl.n + (cur.plane % a.channel) * a.wl.c + tap_offset(a.wl, lane), mine);
    }
    if (!more) break;
    lds_sync();
    cur = nxt;
    gcur = gnxt;
  }
}

// ---- host side of the flat kernels ----------------------------------------------------------

constexpr int kFlatElems = 2048;       // largest staged range of the convolution (elements, halo rows included)
constexpr int kFlatElemsGrad = 1024;   // of the kernel gradient, which stages two tensors

template <typename T>
bool flat_plan(FlatConv& a, const Geo& g, const long* ws, int budget, const void* p0, const void* p1) {
  if constexpr (std::is_same<T, double>::value) return false;
  if (g.k_h != 3 || g.k_w != 3 || g.stride_h != 1 || g.stride_w != 1 || g.dil_h != 1 || g.dil_w != 1 || g.pad_h != 1 ||
      g.pad_w != 1)
    return false;
  const long bytes = (long)g.batch * g.channel * g.in_h * g.in_w * (long)sizeof(T);
  if (bytes >= (1L << 31) || bytes % 16 != 0 || g.in_w < 2) return false;
  // the loads are 16-byte loads at multiples of 16 bytes from the tensor's start
  if (reinterpret_cast<uintptr_t>(p0) % 16 != 0 || reinterpret_cast<uintptr_t>(p1) % 16 != 0) return false;
  const int max_rows = (budget - (kPer<T> - 1)) / g.in_w - 2;
  if (max_rows < 1) return false;
  a.planes = g.batch * g.channel, a.channel = g.channel;
  a.wl = ws ? WLayout{ws[0], ws[1], ws[2], ws[3]} : WLayout{(long)g.channel * 9, 9L, 3L, 1L};
  a.h = g.in_h, a.w = g.in_w, a.hw = g.in_h * g.in_w;
  a.bands = (g.in_h + max_rows - 1) / max_rows;
  a.band_rows = (g.in_h + a.bands - 1) / a.bands;
  // bands of a multiple of four rows where the plane allows it: the kernels then work on 4 x 4 patches
  if (g.in_h % 4 == 0 && (a.band_rows + 3) / 4 * 4 <= max_rows) a.band_rows = (a.band_rows + 3) / 4 * 4;
  a.bands = (g.in_h + a.band_rows - 1) / a.band_rows;
  a.flip = 0;
  return true;
}

// chunks a lane holds for the largest range of the plan (1, 2, 4 or 8)
template <typename T>
int flat_chunks_per_lane(const FlatConv& a) {
  const int elems = (kPer<T> - 1) + (a.band_rows + 2) * a.w;
  const int chunks = (elems + kPer<T> - 1) / kPer<T>;
  int nch = 1;
  while (nch * kWave < chunks) nch *= 2;
  return nch;
}

int flat_grid(const FlatConv& a) {
  // enough waves to fill the GPU several times over, each walking a few planes so that its loads overlap its arithmetic
  const long waves = std::min<long>(a.planes, 256L * 32);
  return (int)((waves + kWaves - 1) / kWaves);
}

template <typename T>
bool launch_flat_conv(const Geo& g, const long* ws, bool flip, const T* src, const T* weight, T* dst, hipStream_t stream) {
  if constexpr (std::is_same<T, double>::value) {
    return false;
  } else {
    FlatConv a{};
    if (!flat_plan<T>(a, g, ws, kFlatElems, src, src)) return false;
    a.flip = flip;
    a.vec_ok = aligned_rows(dst, a.w, sizeof(T));
    const int nch = flat_chunks_per_lane<T>(a);
    if (nch > 8) return false;
    a.tile_elems = kFront + nch * kWave * kPer<T> + 8;
    const size_t lds = (size_t)kWaves * a.tile_elems * sizeof(float);
    const dim3 grid(flat_grid(a)), block(kWave * kWaves);
    const bool w4 = a.vec_ok != 0;  // whole, aligned strips: one vector store each
    const bool patches = w4 && a.h % 4 == 0 && a.band_rows % 4 == 0;
    if constexpr (sizeof(T) == 2) {
      // 16-bit tensors with rows of a multiple of 4 elements: the packed kernels
      if (w4 && a.w % kStrip == 0 && a.w >= kStrip && !path_disabled(kNoImagePacked)) {
#define DK_FLAT16(NN)                                                                                                      \
  if (patches) hipLaunchKernelGGL((image_conv3_flat16_kernel<T, NN, 4>), grid, block, lds, stream, a, src, weight, dst);      \
  else hipLaunchKernelGGL((image_conv3_flat16_kernel<T, NN, 1>), grid, block, lds, stream, a, src, weight, dst)
        if (nch == 1) { DK_FLAT16(1); }
        else if (nch == 2) { DK_FLAT16(2); }
        else if (nch == 4) { DK_FLAT16(4); }
        else { DK_FLAT16(8); }
#undef DK_FLAT16
        return true;
      }
    }
#define DK_FLAT(NN)                                                                                                        \
  if (patches) hipLaunchKernelGGL((image_conv3_flat_kernel<T, NN, true, 4>), grid, block, lds, stream, a, src, weight, dst);  \
  else if (w4) hipLaunchKernelGGL((image_conv3_flat_kernel<T, NN, true, 1>), grid, block, lds, stream, a, src, weight, dst);  \
  else hipLaunchKernelGGL((image_conv3_flat_kernel<T, NN, false, 1>), grid, block, lds, stream, a, src, weight, dst)
    if (nch == 1) { DK_FLAT(1); }
    else if (nch == 2) { DK_FLAT(2); }
    else if (nch == 4) { DK_FLAT(4); }
    else { DK_FLAT(8); }
#undef DK_FLAT
    return true;
  }
}

template <typename T>
bool launch_flat_grad_weight(const Geo& g, const long* ws, const T* gout, const T* x, T* gweight, hipStream_t stream) {
  if constexpr (std::is_same<T, double>::value) {
    return false;
  } else {
    FlatConv a{};
    if (!flat_plan<T>(a, g, ws, kFlatElemsGrad, x, gout)) return false;
    const int nch = flat_chunks_per_lane<T>(a);
    if (nch > 4) return false;
    a.tile_elems = kFront + nch * kWave * kPer<T> + 8;
    const size_t lds = (size_t)kWaves * 2 * a.tile_elems * sizeof(float);
    const dim3 grid(flat_grid(a)), block(kWave * kWaves);
    const bool w4 = a.w % kStrip == 0;
    const bool patches = w4 && a.h % 4 == 0 && a.band_rows % 4 == 0;
    if constexpr (sizeof(T) == 2) {
      if (w4 && a.w >= kStrip && !path_disabled(kNoImagePacked)) {
#define DK_FLAT16(NN)                                                                                                                  \
  if (patches) hipLaunchKernelGGL((image_conv3_flat16_grad_weight_kernel<T, NN, 4>), grid, block, lds, stream, a, gout, x, gweight);   \
  else hipLaunchKernelGGL((image_conv3_flat16_grad_weight_kernel<T, NN, 1>), grid, block, lds, stream, a, gout, x, gweight)
        if (nch == 1) { DK_FLAT16(1); }
        else if (nch == 2) { DK_FLAT16(2); }
        else { DK_FLAT16(4); }
#undef DK_FLAT16
        return true;
      }
    }
#define DK_FLAT(NN)                                                                                                                    \
  if (patches) hipLaunchKernelGGL((image_conv3_flat_grad_weight_kernel<T, NN, true, 4>), grid, block, lds, stream, a, gout, x, gweight); \
  else if (w4) hipLaunchKernelGGL((image_conv3_flat_grad_weight_kernel<T, NN, true, 1>), grid, block, lds, stream, a, gout, x, gweight); \
  else hipLaunchKernelGGL((image_conv3_flat_grad_weight_kernel<T, NN, false, 1>), grid, block, lds, stream, a, gout, x, gweight)
    if (nch == 1) { DK_FLAT(1); }
    else if (nch == 2) { DK_FLAT(2); }
    else { DK_FLAT(4); }
#undef DK_FLAT
    return true;
  }
}

template <typename T>
size_t lds_bytes(const ImgConv& a, bool run_time_taps) {
  return (size_t)kWaves * (a.tile_elems + (run_time_taps ? kMaxTaps : 0)) * sizeof(compute_t<T>);
}

template <typename T>
bool launch_conv(ImgConv a, const T* src, const T* weight, T* dst, hipStream_t stream) {
  if (!plan(a, sizeof(compute_t<T>))) return false;
  a.vec_ok = aligned_rows(dst, a.dst_w, sizeof(T));
  const bool unit = a.stride_h == 1 && a.stride_w == 1 && a.dil_h == 1 && a.dil_w == 1;
  const int k = a.k_h == a.k_w ? a.k_h : 0;
  const dim3 grid((a.planes + kWaves - 1) / kWaves), block(kWave * kWaves);
#define DK_IMG_CONV(KK, UU) \
  hipLaunchKernelGGL((image_conv_kernel<T, KK, UU>), grid, block, lds_bytes<T>(a, KK == 0), stream, a, src, weight, dst)
  if (k == 3 && unit) DK_IMG_CONV(3, true);
  else if (k == 3) DK_IMG_CONV(3, false);
  else if (k == 1) DK_IMG_CONV(1, false);
  else if (k == 5 && unit) DK_IMG_CONV(5, true);
  else DK_IMG_CONV(0, false);
#undef DK_IMG_CONV
  return true;
}

ImgConv forward_args(const Geo& g, const long* ws) {
  ImgConv a{};
  a.planes = g.batch * g.channel;
  a.channel = g.channel;
  a.wl = ws ? WLayout{ws[0], ws[1], ws[2], ws[3]}
            : WLayout{(long)g.channel * g.k_h * g.k_w, (long)g.k_h * g.k_w, (long)g.k_w, 1L};
  a.src_h = g.in_h, a.src_w = g.in_w, a.dst_h = g.out_h, a.dst_w = g.out_w;
  a.k_h = g.k_h, a.k_w = g.k_w, a.stride_h = g.stride_h, a.stride_w = g.stride_w, a.dil_h = g.dil_h, a.dil_w = g.dil_w;
  a.org_h = -g.pad_h, a.org_w = -g.pad_w;
  return a;
}

}  // namespace

bool image_conv_supported(const Geo& g, int dtype) {
  ImgConv a = forward_args(g, nullptr);
  const size_t eb = dtype == DK_F64 ? 8 : 4;
  if (!plan(a, eb)) return false;
  if (g.stride_h == 1 && g.stride_w == 1) {  // the input gradient runs as a convolution over out_grad
    ImgConv b = forward_args(g, nullptr);
    b.src_h = g.out_h, b.src_w = g.out_w, b.dst_h = g.in_h, b.dst_w = g.in_w;
    if (!plan(b, eb)) return false;
  }
  return true;
}

template <typename T>
bool image_conv_forward(const Geo& g, const long* wstrides, const T* x, const T* weight, T* out, hipStream_t stream) {
  if (!path_disabled(kNoImageFlat) && launch_flat_conv<T>(g, wstrides, false, x, weight, out, stream)) return true;
  return launch_conv<T>(forward_args(g, wstrides), x, weight, out, stream);
}

template <typename T>
bool image_conv_grad_input(const Geo& g, const long* wstrides, const T* gout, const T* weight, T* gin,
                           hipStream_t stream) {
  if (!path_disabled(kNoImageFlat) && launch_flat_conv<T>(g, wstrides, true, gout, weight, gin, stream)) return true;
  ImgConv a = forward_args(g, wstrides);
  if (g.stride_h == 1 && g.stride_w == 1) {
    a.src_h = g.out_h, a.src_w = g.out_w, a.dst_h = g.in_h, a.dst_w = g.in_w;
    a.org_h = g.pad_h - (g.k_h - 1) * g.dil_h, a.org_w = g.pad_w - (g.k_w - 1) * g.dil_w;
    a.flip = 1;
    return launch_conv<T>(a, gout, weight, gin, stream);
  }
  if ((long)g.k_h * g.k_w > kMaxTaps) return false;
  const long total = (long)a.planes * g.in_h * g.in_w;
  const int blocks = (int)std::min<long>((total + 255) / 256, 1 << 20);
  hipLaunchKernelGGL((image_conv_grad_input_strided_kernel<T>), dim3(blocks), dim3(256), 0, stream, a, g.pad_h, g.pad_w,
                     gout, weight, gin);
  return true;
}

template <typename T>
bool image_conv_grad_weight(const Geo& g, const long* wstrides, const T* gout, const T* x, T* gweight,
                            hipStream_t stream) {
  if (!path_disabled(kNoImageFlat) && launch_flat_grad_weight<T>(g, wstrides, gout, x, gweight, stream)) return true;
  ImgConv a = forward_args(g, wstrides);
  if (!plan(a, sizeof(compute_t<T>))) return false;
  a.vec_ok = aligned_rows(gout, a.dst_w, sizeof(T));
  const bool unit = a.stride_h == 1 && a.stride_w == 1 && a.dil_h == 1 && a.dil_w == 1;
  const int k = a.k_h == a.k_w ? a.k_h : 0;
  const dim3 grid((a.planes + kWaves - 1) / kWaves), block(kWave * kWaves);
#define DK_IMG_WGRAD(KK, UU)                                                                                       \
  hipLaunchKernelGGL((image_conv_grad_weight_kernel<T, KK, UU>), grid, block, lds_bytes<T>(a, KK == 0), stream, a, \
                     gout, x, gweight)
  if (k == 3 && unit) DK_IMG_WGRAD(3, true);
  else if (k == 3) DK_IMG_WGRAD(3, false);
  else if (k == 1) DK_IMG_WGRAD(1, false);
  else DK_IMG_WGRAD(0, false);
#undef DK_IMG_WGRAD
  return true;
}

#define DK_INSTANTIATE(T)                                                                              \
  template bool image_conv_forward<T>(const Geo&, const long*, const T*, const T*, T*, hipStream_t);    \
  template bool image_conv_grad_input<T>(const Geo&, const long*, const T*, const T*, T*, hipStream_t); \
  template bool image_conv_grad_weight<T>(const Geo&, const long*, const T*, const T*, T*, hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
DK_INSTANTIATE(double)
#undef DK_INSTANTIATE

}  // namespace dk
