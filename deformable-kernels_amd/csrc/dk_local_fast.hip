// Local deformable kernel (kernel-space offsets only), tuned path for gfx950: 3x3 taps, scope
// 3x3 / 4x4 / 5x5 / 7x7, fp32 / fp16 / bf16.  Everything else runs on dk_generic.hip.
//
// One lane owns one pixel and walks the channels of its rotation group.  What depends only on
// (pixel, tap) -- the scope cell and the fractional position inside it -- is computed once and
// held in registers; per channel and tap the lane then needs one 16-byte read from the channel's
// corner-expanded scope table in LDS (dk_scope_table.h) and four FMAs.  Consecutive lanes hold
// consecutive pixels, so every input / gradient access of a wave is one contiguous run of a plane.
//
// Reference kernels covered (K.cu =
// deformable_kernels/ops/deform_kernel/csrc/filter_sample_depthwise_cuda_kernel.cu):
//   forward        K.cu:270-386   -> local_gather_rows_kernel<.., false> (stride 1, same width),
//                                    local_forward_s2_kernel (stride 2), local_gather_kernel<.., false, 9>
//   grad input     K.cu:577-669   -> local_gather_rows_kernel<.., true>, local_grad_input_s2_kernel (stride 2),
//                                    local_gather_kernel<.., true, 9 | 4>
//   grad rotation  K.cu:1285-1370 -> local_grad_rotation_kernel<.., MODE> (+ reduce_few_parts_kernel)
//   grad filter    K.cu:836-955   -> local_grad_filter_mfma_kernel<.., S2> | local_grad_filter_kernel<.., MODE>
//                                    + reduce_partials_kernel
#include <cstdlib>

#include <algorithm>
#include <type_traits>

#include "dk_kernels.h"
#include "dk_scope_table.h"

namespace dk {

namespace {

constexpr int kBlock = 256;

// Geometry of tap (f_h, f_w) for the pixel this lane owns.
//   forward (TRANSPOSED = false): the lane owns OUTPUT pixel (ph, pw); the tap reads input
//     (ph*s - pad + f*d) and the rotation of the lane's own pixel (K.cu:315-336).
//   grad input (TRANSPOSED = true): the lane owns INPUT pixel (ph, pw); the tap is fed by output
//     pixel (ph + pad - f*d) / s when that division is exact and in range, and uses that output
//     pixel's rotation (K.cu:611-651).
// Returns false when the tap does not contribute; `src` is the element offset inside the
// source plane, `rpix` the pixel offset inside a rotation plane.
template <bool TRANSPOSED>
__device__ __forceinline__ bool tap_geometry(const Geo& g, int ph, int pw, int f_h, int f_w,
                                             int& src, int& rpix) {
  if (!TRANSPOSED) {
    const int ih = ph * g.stride_h - g.pad_h + f_h * g.dil_h;
    const int iw = pw * g.stride_w - g.pad_w + f_w * g.dil_w;
    const bool ok = ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
    src = ok ? ih * g.in_w + iw : 0;
    rpix = ph * g.out_w + pw;
    return ok;
  } else {
    const int th = ph + g.pad_h - f_h * g.dil_h;
    const int tw = pw + g.pad_w - f_w * g.dil_w;
    bool ok = th >= 0 && tw >= 0;
    int oh = 0, ow = 0;
    if (g.stride_h == 1 && g.stride_w == 1) {
      oh = th;
      ow = tw;
    } else {
      oh = th / g.stride_h;
      ow = tw / g.stride_w;
      ok = ok && (oh * g.stride_h == th) && (ow * g.stride_w == tw);
    }
    ok = ok && oh < g.out_h && ow < g.out_w;
    src = ok ? oh * g.out_w + ow : 0;
    rpix = src;
    return ok;
  }
}

// ---------------------------------------------------------------------------
// forward and grad-input: dst[n, c, p] = sum_t src[n, c, tap_t(p)] * B_t(p; Wt[c])
// grid = (pixel tiles, channel splits, batch * groups)
//
// Channels are walked kUnroll at a time: the 9 * kUnroll input loads of a block are
// issued first (buffer loads, offsets fixed per lane), then each channel's 9 taps take
// one ds_read_b128 each at an immediate offset from one per-tap LDS address.
// ---------------------------------------------------------------------------
constexpr int kUnroll = 2;
constexpr int kRowStages = 2;  // register stages of the rows kernel's load pipeline (3 and 4 measured slower)

template <typename T, int KH, int KW, int SH, int SW, bool TRANSPOSED, int NT>
__global__ __launch_bounds__(kBlock, 2) void local_gather_kernel(Geo g, const T* __restrict__ src,
                                                                 const T* __restrict__ rot,
                                                                 const T* __restrict__ filter,
                                                                 T* __restrict__ dst, int ch_per_block) {
  using Tb = WideTable<SH, SW>;
  constexpr int K = KH * KW;
  extern __shared__ __align__(16) float tbl[];

  const int cpg = g.channel / g.groups;  // channels per rotation group
  const int out_plane = g.out_h * g.out_w, in_plane = g.in_h * g.in_w;
  const int dst_plane = TRANSPOSED ? in_plane : out_plane;
  const int src_plane = TRANSPOSED ? out_plane : in_plane;
  const int dst_w = TRANSPOSED ? g.in_w : g.out_w;
  // logical block = (tile, channel split, image * group), tile fastest: one XCD gets whole images
  const int tiles = ceil_div(dst_plane, kBlock), splits = ceil_div(cpg, ch_per_block);
  const int total = tiles * splits * g.batch * g.groups;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int bx = lb % tiles, by = lb / tiles % splits, bz = lb / tiles / splits;
  const int n = bz / g.groups, grp = bz % g.groups;
  const int j0 = by * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, grp + g.groups * j0, g.groups, nch);

  const int p = bx * kBlock + threadIdx.x;
  const bool active = p < dst_plane;
  const int pc = active ? p : 0;
  const int ph = pc / dst_w, pw = pc % dst_w;

  static_assert(NT == K || (TRANSPOSED && NT == 4 && KH == 3 && KW == 3), "tap slots: all taps, or the stride-2 subset");
  LiteTap tap[NT];
  unsigned soff[NT];  // byte offset of the tap's source element in a source plane
  const rsrc_t rr = plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K * 2) * out_plane, K * 2 * out_plane);
#pragma unroll
  for (int slot = 0; slot < NT; ++slot) {
    // NT == 4: stride 2 x 2, undilated.  An input pixel is fed only by the taps with
    // f = (p + pad) mod 2 (+ 2), at most two per direction; the slots enumerate those.
    const int f_h = NT == K ? slot / KW : ((ph + g.pad_h) & 1) + 2 * (slot >> 1);
    const int f_w = NT == K ? slot % KW : ((pw + g.pad_w) & 1) + 2 * (slot & 1);
    const int t = NT == K ? slot : min(f_h, KH - 1) * KW + min(f_w, KW - 1);
    int s_el, rpix;
    const bool ok = f_h < KH && f_w < KW && tap_geometry<TRANSPOSED>(g, ph, pw, f_h, f_w, s_el, rpix) && active;
    soff[slot] = ok ? (unsigned)s_el * (unsigned)sizeof(T) : kOutOfRange;
    const unsigned ro = ok ? (unsigned)((2 * t) * out_plane + rpix) * (unsigned)sizeof(T) : kOutOfRange;
    const float r_h = buf_ld(rr, ro, rot);
    const float r_w = buf_ld(rr, ro + (unsigned)out_plane * (unsigned)sizeof(T), rot);
    tap[slot] = make_lite_tap<SH, SW>(scope_coord<float>(g, f_h, r_h, g.centre_h),
                                   scope_coord<float>(g, f_w, r_w, g.centre_w), ok);
  }
  __syncthreads();

  const size_t chan0 = (size_t)n * g.channel + grp + (size_t)g.groups * j0;
  const T* sp = src + chan0 * src_plane;
  T* dp = dst + chan0 * dst_plane;
  const size_t s_step = (size_t)g.groups * src_plane, d_step = (size_t)g.groups * dst_plane;
  const unsigned doff = active ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  // Two register stages of kUnroll channels each: the loads of the next stage are in flight
  // while the current one is computed, so a wave always has input loads outstanding.
  // Channels beyond nch load through a zero-length resource (hardware returns 0) and
  // store to an out-of-range offset (dropped), which keeps the loop free of branches.
  auto load_stage = [&](float (&xv)[kUnroll][NT], int jb) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const rsrc_t rs = plane_rsrc(sp + (size_t)(jb + u) * s_step, (jb + u) < nch ? src_plane : 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) xv[u][t] = buf_ld(rs, soff[t], src);
    }
  };
  auto compute_stage = [&](const float (&xv)[kUnroll][NT], int jb) {
    const float* tb = tbl + jb * Tb::SIZE;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float acc = 0.f;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const float4 q = *reinterpret_cast<const float4*>(tb + tap[t].cell + u * Tb::SIZE);
        acc = fmaf(xv[u][t], lite_weight(tap[t], q), acc);
      }
      buf_st(plane_rsrc(dp + (size_t)(jb + u) * d_step, (jb + u) < nch ? dst_plane : 0), doff, acc, dst);
    }
  };

  float xa[kUnroll][NT], xb[kUnroll][NT];
  load_stage(xa, 0);
  for (int j = 0; j < nch; j += 2 * kUnroll) {
    load_stage(xb, j + kUnroll);
    compute_stage(xa, j);
    load_stage(xa, j + 2 * kUnroll);
    compute_stage(xb, j + kUnroll);
  }
}

// ---------------------------------------------------------------------------
// forward and grad-input for "same" geometries (stride 1, 3 taps per row at unit spacing,
// pad_w = 1, so input and output planes have the same width).
//
// In that case the nine taps of a pixel are three runs of three consecutive plane elements,
// and lane l's left / right element is lane l -+ 1's centre element.  A wave therefore covers
// 62 pixels with lanes 1..62 plus one halo lane at each end; every lane loads only the
// centre element of each of the three tap rows (3 loads per channel instead of 9 -- the
// vector-memory address unit was the busiest unit of the general kernel) and takes the
// side elements from its neighbours with one DPP move each.  Rows above / below the plane
// fall outside the buffer range and read 0; taps whose column wraps to the neighbouring row
// get zero coefficients.
// grid = (pixel tiles of kRowPix, channel splits, batch * groups)
// ---------------------------------------------------------------------------
constexpr int kRowLanes = 62;                          // pixels per wave
constexpr int kRowPix = kRowLanes * (kBlock / 64);     // pixels per workgroup

template <typename T, int KH, int SH, int SW, bool TRANSPOSED>
__global__ __launch_bounds__(kBlock, 2) void local_gather_rows_kernel(Geo g, const T* __restrict__ src,
                                                                      const T* __restrict__ rot,
                                                                      const T* __restrict__ filter,
                                                                      T* __restrict__ dst,
                                                                      int ch_per_block) {
  using Tb = WideTable<SH, SW>;
  constexpr int KW = 3, K = KH * KW;
  extern __shared__ __align__(16) float tbl[];

  const int cpg = g.channel / g.groups;
  const int W = g.in_w;  // == out_w
  const int out_plane = g.out_h * W, in_plane = g.in_h * W;
  const int dst_plane = TRANSPOSED ? in_plane : out_plane;
  const int src_plane = TRANSPOSED ? out_plane : in_plane;
  // logical block = (tile, channel split, image * group), tile fastest: one XCD gets whole images
  const int tiles = ceil_div(dst_plane, kRowPix), splits = ceil_div(cpg, ch_per_block);
  const int total = tiles * splits * g.batch * g.groups;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int bx = lb % tiles, by = lb / tiles % splits, bz = lb / tiles / splits;
  const int n = bz / g.groups, grp = bz % g.groups;
  const int j0 = by * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, grp + g.groups * j0, g.groups, nch);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int p = bx * kRowPix + wave * kRowLanes + lane - 1;  // lanes 0 and 63 are halo
  const bool owns = lane >= 1 && lane <= kRowLanes && p < dst_plane;  // p >= 0 whenever lane >= 1
  const int pc = owns ? p : 0;
  const int ph = pc / W, pw = pc % W;

  // centre element of tap row f_h, as a byte offset into a source plane (out of range -> reads 0)
  unsigned roff[KH];
#pragma unroll
  for (int r = 0; r < KH; ++r) {
    const int dr = TRANSPOSED ? g.pad_h - r * g.dil_h : r * g.dil_h - g.pad_h;
    const long e = (long)p + (long)dr * W;
    roff[r] = (e >= 0 && e < src_plane) ? (unsigned)e * (unsigned)sizeof(T) : kOutOfRange;
  }

  LiteTap tap[K];
  const rsrc_t rr = plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K * 2) * out_plane, K * 2 * out_plane);
#pragma unroll
  for (int t = 0; t < K; ++t) {
    const int f_h = t / KW, f_w = t % KW;
    int s_el, rpix;
    const bool ok = tap_geometry<TRANSPOSED>(g, ph, pw, f_h, f_w, s_el, rpix) && owns;
    const unsigned ro = ok ? (unsigned)((2 * t) * out_plane + rpix) * (unsigned)sizeof(T) : kOutOfRange;
    const float r_h = buf_ld(rr, ro, rot);
    const float r_w = buf_ld(rr, ro + (unsigned)out_plane * (unsigned)sizeof(T), rot);
    tap[t] = make_lite_tap<SH, SW>(scope_coord<float>(g, f_h, r_h, g.centre_h),
                                   scope_coord<float>(g, f_w, r_w, g.centre_w), ok);  // !ok: tap in the padding
  }
  __syncthreads();

  const size_t chan0 = (size_t)n * g.channel + grp + (size_t)g.groups * j0;
  const T* sp = src + chan0 * src_plane;
  T* dp = dst + chan0 * dst_plane;
  const size_t s_step = (size_t)g.groups * src_plane, d_step = (size_t)g.groups * dst_plane;
  const unsigned doff = owns ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  auto load_stage = [&](float (&xc)[kUnroll][KH], int jb) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const rsrc_t rs = plane_rsrc(sp + (size_t)(jb + u) * s_step, (jb + u) < nch ? src_plane : 0);
#pragma unroll
      for (int r = 0; r < KH; ++r) xc[u][r] = buf_ld(rs, roff[r], src);
    }
  };
  auto compute_stage = [&](const float (&xc)[kUnroll][KH], int jb) {
    const float* tb = tbl + jb * Tb::SIZE;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < KH; ++r) {
        // elements at columns -1, 0, +1 of this row; the tap that reads column dc is
        // f_w = dc + 1 (forward) or f_w = 1 - dc (grad input)
#pragma unroll
        for (int f_w = 0; f_w < KW; ++f_w) {
          const int t = r * KW + f_w;
          const int dc = TRANSPOSED ? 1 - f_w : f_w - 1;
          const float4 q = *reinterpret_cast<const float4*>(tb + tap[t].cell + u * Tb::SIZE);
          const float wt = lite_weight(tap[t], q);
          // columns -1 / +1 of the row are the neighbouring lanes' centre elements
          acc = dc < 0 ? fma_lane_below(xc[u][r], wt, acc) : dc == 0 ? fmaf(xc[u][r], wt, acc)
                                                                     : fma_lane_above(xc[u][r], wt, acc);
        }
      }
      buf_st(plane_rsrc(dp + (size_t)(jb + u) * d_step, (jb + u) < nch ? dst_plane : 0), doff, acc, dst);
    }
  };

  constexpr int S = kRowStages;
  float xs[S][kUnroll][KH];
#pragma unroll
  for (int s = 0; s + 1 < S; ++s) load_stage(xs[s], s * kUnroll);
  for (int j = 0; j < nch; j += S * kUnroll) {
#pragma unroll
    for (int s = 0; s < S; ++s) {
      load_stage(xs[(s + S - 1) % S], j + (s + S - 1) * kUnroll);
      compute_stage(xs[s], j + s * kUnroll);
    }
  }
}

// ---------------------------------------------------------------------------
// forward for stride 2 (3 x 3 taps, undilated, padding 1, even input width): the three taps of a
// row read input columns 2 ow - 1, 2 ow, 2 ow + 1.  A lane loads the PAIR (2 ow, 2 ow + 1) of each
// tap row with one 8-byte load (4-byte for the 16-bit types) and takes column 2 ow - 1 from the
// previous lane's pair through the DPP-fused multiply-add: 3 loads per channel instead of 9
// strided ones.  A wave covers 63 pixels with lanes 1..63 plus the halo lane 0.  Taps in the
// padding (row -1, column -1) get the zero scope block; their loads are redirected to element 0.
// grid = (pixel tiles of kS2Pix, channel splits, batch * groups)
// ---------------------------------------------------------------------------
constexpr int kS2Lanes = 63;
constexpr int kS2Pix = kS2Lanes * (kBlock / 64);

template <typename T> struct Pair;
template <> struct Pair<float> {
  typedef float raw __attribute__((ext_vector_type(2), aligned(4)));
  static __device__ __forceinline__ float get(const raw& v, int k) { return v[k]; }
  static __device__ __forceinline__ raw make(float a, float b) { return raw{a, b}; }
};
template <> struct Pair<__half> {
  typedef _Float16 raw __attribute__((ext_vector_type(2), aligned(2)));
  static __device__ __forceinline__ float get(const raw& v, int k) { return static_cast<float>(v[k]); }
  static __device__ __forceinline__ raw make(float a, float b) { return raw{static_cast<_Float16>(a), static_cast<_Float16>(b)}; }
};
template <> struct Pair<bf16_t> {
  typedef unsigned short raw __attribute__((ext_vector_type(2), aligned(2)));
  static __device__ __forceinline__ float get(const raw& v, int k) { return __uint_as_float(static_cast<uint32_t>(v[k]) << 16); }
  static __device__ __forceinline__ raw make(float a, float b) {
    bf16_t x, y;
    st(&x, a);
    st(&y, b);
    return raw{x.bits, y.bits};
  }
};

template <typename T, int SH, int SW>
__global__ __launch_bounds__(kBlock, 2) void local_forward_s2_kernel(Geo g, const T* __restrict__ x,
                                                                     const T* __restrict__ rot,
                                                                     const T* __restrict__ filter,
                                                                     T* __restrict__ out, int ch_per_block) {
  using Tb = WideTable<SH, SW>;
  constexpr int KH = 3, KW = 3, K = 9;
  extern __shared__ __align__(16) float tbl[];

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = g.in_h * g.in_w;
  const int tiles = ceil_div(out_plane, kS2Pix), splits = ceil_div(cpg, ch_per_block);
  const int total = tiles * splits * g.batch * g.groups;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int bx = lb % tiles, by = lb / tiles % splits, bz = lb / tiles / splits;
  const int n = bz / g.groups, grp = bz % g.groups;
  const int j0 = by * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, grp + g.groups * j0, g.groups, nch);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int p = bx * kS2Pix + wave * kS2Lanes + lane - 1;  // lane 0 is the halo: the pixel before the wave's first
  const bool owns = lane >= 1 && p < out_plane;
  const int pc = min(max(p, 0), out_plane - 1);  // halo and tail lanes load some valid pixel's pairs
  const int ph = pc / g.out_w, pw = pc % g.out_w;

  // first element of the pair of tap row r (element 0 when the row is in the padding)
  int pe[KH];
#pragma unroll
  for (int r = 0; r < KH; ++r) {
    const int ih = 2 * ph - 1 + r;
    pe[r] = (ih >= 0 && ih < g.in_h) ? ih * g.in_w + 2 * pw : 0;
  }

  LiteTap tap[K];
  const rsrc_t rr = plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K * 2) * out_plane, K * 2 * out_plane);
#pragma unroll
  for (int t = 0; t < K; ++t) {
    const int f_h = t / KW, f_w = t % KW;
    int s_el, rpix;
    const bool ok = tap_geometry<false>(g, ph, pw, f_h, f_w, s_el, rpix) && owns;
    const unsigned ro = ok ? (unsigned)((2 * t) * out_plane + rpix) * (unsigned)sizeof(T) : kOutOfRange;
    const float r_h = buf_ld(rr, ro, rot);
    const float r_w = buf_ld(rr, ro + (unsigned)out_plane * (unsigned)sizeof(T), rot);
    tap[t] = make_lite_tap<SH, SW>(scope_coord<float>(g, f_h, r_h, g.centre_h),
                                   scope_coord<float>(g, f_w, r_w, g.centre_w), ok);
  }
  __syncthreads();

  const size_t chan0 = (size_t)n * g.channel + grp + (size_t)g.groups * j0;
  const T* sp = x + chan0 * in_plane;
  T* dp = out + chan0 * out_plane;
  const size_t s_step = (size_t)g.groups * in_plane, d_step = (size_t)g.groups * out_plane;
  const unsigned doff = owns ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  typedef typename Pair<T>::raw pair_t;
  auto load_stage = [&](pair_t (&xc)[kUnroll][KH], int jb) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const T* plane = sp + (size_t)min(jb + u, nch - 1) * s_step;  // past the last channel: reload it, the store is dropped
#pragma unroll
      for (int r = 0; r < KH; ++r) xc[u][r] = *reinterpret_cast<const pair_t*>(plane + pe[r]);
    }
  };
  auto compute_stage = [&](const pair_t (&xc)[kUnroll][KH], int jb) {
    const float* tb = tbl + jb * Tb::SIZE;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < KH; ++r) {
        const float x0 = Pair<T>::get(xc[u][r], 0), x1 = Pair<T>::get(xc[u][r], 1);
#pragma unroll
        for (int f_w = 0; f_w < KW; ++f_w) {
          const int t = r * KW + f_w;
          const float4 q = *reinterpret_cast<const float4*>(tb + tap[t].cell + u * Tb::SIZE);
          const float wt = lite_weight(tap[t], q);
          // column 2 ow - 1 is the previous lane's second element
          acc = f_w == 0 ? fma_lane_below(x1, wt, acc) : f_w == 1 ? fmaf(x0, wt, acc) : fmaf(x1, wt, acc);
        }
      }
      buf_st(plane_rsrc(dp + (size_t)(jb + u) * d_step, (jb + u) < nch ? out_plane : 0), doff, acc, out);
    }
  };

  pair_t xa[kUnroll][KH], xb[kUnroll][KH];
  load_stage(xa, 0);
  for (int j = 0; j < nch; j += 2 * kUnroll) {
    load_stage(xb, j + kUnroll);
    compute_stage(xa, j);
    load_stage(xa, j + 2 * kUnroll);
    compute_stage(xb, j + kUnroll);
  }
}

// ---------------------------------------------------------------------------
// grad input for the same stride-2 geometry.  The 2 x 2 input quad (2 qh .. + 1, 2 qw .. + 1) is fed
// by exactly nine (output pixel, tap) pairs of the four output pixels P00 = (qh, qw), P01 = (qh, qw + 1),
// P10 = (qh + 1, qw), P11 = (qh + 1, qw + 1):
//   (even, even)  P00 (1,1)
//   (even, odd)   P00 (1,2)  P01 (1,0)
//   (odd, even)   P00 (2,1)  P10 (0,1)
//   (odd, odd)    P00 (2,2)  P01 (2,0)  P10 (0,2)  P11 (0,0)
// so a lane that owns the quad of output pixel P00 does the forward kernel's nine weights per
// channel, from two gout loads (its own pixel and the one a row below; the right-hand neighbours
// come from the next lane through the DPP-fused multiply-add), and every lane has the same work.
// A gather over input pixels has 1, 2 or 4 taps per lane depending on the pixel's parities
// (local_gather_kernel<.., true, 4>: 16 tap slots per quad instead of 9).  A wave covers 63 quads
// with lanes 0 .. 62 plus the halo lane 63.
// grid = (quad tiles of kS2Pix, channel splits, batch * groups)
// ---------------------------------------------------------------------------
template <typename T, int SH, int SW>
__global__ __launch_bounds__(kBlock, 2) void local_grad_input_s2_kernel(Geo g, const T* __restrict__ gout,
                                                                        const T* __restrict__ rot,
                                                                        const T* __restrict__ filter,
                                                                        T* __restrict__ gin, int ch_per_block) {
  using Tb = WideTable<SH, SW>;
  constexpr int K = 9;
  extern __shared__ __align__(16) float tbl[];

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = g.in_h * g.in_w;
  const int tiles = ceil_div(out_plane, kS2Pix), splits = ceil_div(cpg, ch_per_block);
  const int total = tiles * splits * g.batch * g.groups;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int bx = lb % tiles, by = lb / tiles % splits, bz = lb / tiles / splits;
  const int n = bz / g.groups, grp = bz % g.groups;
  const int j0 = by * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, grp + g.groups * j0, g.groups, nch);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int p = bx * kS2Pix + wave * kS2Lanes + lane;  // lane 63 is the halo: the quad after the wave's last
  const bool exists = p < out_plane;
  const bool owns = lane < kS2Lanes && exists;
  const int pc = exists ? p : 0;
  const int qh = pc / g.out_w, qw = pc % g.out_w;
  const bool right = qw + 1 < g.out_w, below = qh + 1 < g.out_h;

  // the nine (output pixel, tap) pairs in the order of the table above
  constexpr int kDh[K] = {0, 0, 0, 0, 1, 0, 0, 1, 1}, kDw[K] = {0, 0, 1, 0, 0, 0, 1, 0, 1};
  constexpr int kTap[K] = {4, 5, 3, 7, 1, 8, 6, 2, 0};
  LiteTap tap[K];
  const rsrc_t rr = plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K * 2) * out_plane, K * 2 * out_plane);
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const bool ok = exists && (kDh[k] == 0 || below) && (kDw[k] == 0 || right);
    const int rp = pc + kDh[k] * g.out_w + kDw[k];
    const unsigned ro = ok ? (unsigned)((2 * kTap[k]) * out_plane + rp) * (unsigned)sizeof(T) : kOutOfRange;
    const float r_h = buf_ld(rr, ro, rot);
    const float r_w = buf_ld(rr, ro + (unsigned)out_plane * (unsigned)sizeof(T), rot);
    tap[k] = make_lite_tap<SH, SW>(scope_coord<float>(g, kTap[k] / 3, r_h, g.centre_h),
                                   scope_coord<float>(g, kTap[k] % 3, r_w, g.centre_w), ok);
  }
  __syncthreads();

  const size_t chan0 = (size_t)n * g.channel + grp + (size_t)g.groups * j0;
  const T* sp = gout + chan0 * out_plane;
  T* dp = gin + chan0 * in_plane;
  const size_t s_step = (size_t)g.groups * out_plane, d_step = (size_t)g.groups * in_plane;
  // gout of the lane's pixel (halo lane included: its pixel is the next wave's first) and of the one below
  const unsigned g0off = exists ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;
  const unsigned g1off = (exists && below) ? (unsigned)(p + g.out_w) * (unsigned)sizeof(T) : kOutOfRange;
  // the quad's elements: the pairs of rows 2 qh and 2 qh + 1 (the latter may lie past an odd-height plane)
  typedef typename Pair<T>::raw pair_t;
  const int d0 = 2 * qh * g.in_w + 2 * qw;
  const bool row1 = 2 * qh + 1 < g.in_h;

  auto load_stage = [&](float (&gc)[kUnroll][2], int jb) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const rsrc_t rs = plane_rsrc(sp + (size_t)(jb + u) * s_step, (jb + u) < nch ? out_plane : 0);
      gc[u][0] = buf_ld(rs, g0off, gout);
      gc[u][1] = buf_ld(rs, g1off, gout);
    }
  };
  auto compute_stage = [&](const float (&gc)[kUnroll][2], int jb) {
    const float* tb = tbl + jb * Tb::SIZE;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float w[K];
#pragma unroll
      for (int k = 0; k < K; ++k)
        w[k] = lite_weight(tap[k], *reinterpret_cast<const float4*>(tb + tap[k].cell + u * Tb::SIZE));
      const float g0 = gc[u][0], g1 = gc[u][1];
      const float v00 = g0 * w[0];
      const float v01 = fma_lane_above(g0, w[2], g0 * w[1]);
      const float v10 = fmaf(g1, w[4], g0 * w[3]);
      const float v11 = fma_lane_above(g1, w[8], fmaf(g1, w[7], fma_lane_above(g0, w[6], g0 * w[5])));
      // one store per row pair (the wave writes 63 contiguous pairs); non-temporal like the other results
      if (owns && jb + u < nch) {
        T* plane = dp + (size_t)(jb + u) * d_step + d0;
        __builtin_nontemporal_store(Pair<T>::make(v00, v01), reinterpret_cast<pair_t*>(plane));
        if (row1) __builtin_nontemporal_store(Pair<T>::make(v10, v11), reinterpret_cast<pair_t*>(plane + g.in_w));
      }
    }
  };

  float ga[kUnroll][2], gb[kUnroll][2];
  load_stage(ga, 0);
  for (int j = 0; j < nch; j += 2 * kUnroll) {
    load_stage(gb, j + kUnroll);
    compute_stage(ga, j);
    load_stage(ga, j + 2 * kUnroll);
    compute_stage(gb, j + kUnroll);
  }
}

// ---------------------------------------------------------------------------
// grad rotation: the lane owns output pixel p of (n, group) and sums over channels.
// With the block in difference form {a, b, c, d} the derivatives of the bilinear read are
// d/dh = c + lw * d and d/dw = b + lh * d (K.cu:137-158 in corner form), with channel-independent
// lh, lw, so the lane only accumulates
//   S_b[t], S_c[t], S_d[t] = sum_c x_t[c] * gout[c] * {b, c, d}[c]
// and combines the three sums per tap once at the end;
// the fractional parts needed for that are recomputed from the rotation rather than kept
// in registers across the channel loop.
//
// ROWS = true is the "same"-geometry form (see local_gather_rows_kernel): 62 pixels per
// wave, centre-column loads and DPP neighbours; ROWS = false loads every tap.
// The scope tables of the group's channels are staged in passes of ch_per_pass channels.
// Small planes give too few (tile, image) blocks to fill the GPU: the channels of a group are
// then split over `splits` blocks, each writing an fp32 partial [split][image * group][18][pixel]
// to the workspace, and reduce_partials_kernel adds the splits in order.  splits == 1 writes the
// result directly.
// grid = (pixel tiles, splits, batch * groups)
// ---------------------------------------------------------------------------
// OCC: waves per SIMD the register allocation leaves room for.  The 27 sums make this the
// register-heaviest gather kernel; with 96 registers (five waves) it is slower per wave but faster
// where the grid has more than four workgroups per CU to offer (112 x 112 C=32: 125 -> 96 us).
template <typename T, int KH, int KW, int SH, int SW, int MODE, int OCC = 2, bool PAIR = false>
__global__ __launch_bounds__(kBlock, OCC) void local_grad_rotation_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ rot,
    const T* __restrict__ filter, T* __restrict__ grot, float* __restrict__ partial, int splits,
    int ch_per_pass) {
  using Tb = WideTable<SH, SW>;
  constexpr int K = KH * KW;
  constexpr bool ROWS = MODE == 1, S2 = MODE == 2;  // MODE 0: one load per tap
  constexpr int NLOAD = MODE == 0 ? K : KH;          // input loads per channel
  constexpr int PIX = ROWS ? kRowPix : S2 ? kS2Pix : kBlock;  // pixels per workgroup
  // 16-bit tensors: two channels per step, bfloat16 products (PAIR: the host asks for it when a group has
  // at least 16 channels; with a few channels the products' rounding shows in the result: 1.2e-2 of the
  // largest element was seen with one channel per group)
  constexpr bool PAIRS = PAIR && ROWS && sizeof(T) == 2;
  extern __shared__ __align__(16) float tbl[];

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = g.in_h * g.in_w;
  // logical block = (tile, channel split, image * group), tile fastest
  const int tiles = ceil_div(out_plane, PIX);
  const int total = tiles * splits * g.batch * g.groups;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int bx = lb % tiles, split = lb / tiles % splits, bz = lb / tiles / splits;
  const int n = bz / g.groups, grp = bz % g.groups;
  const int per_split = ceil_div(cpg, splits);
  const int c_begin = split * per_split, c_end = min(cpg, c_begin + per_split);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int p = ROWS ? bx * kRowPix + wave * kRowLanes + lane - 1
                : S2 ? bx * kS2Pix + wave * kS2Lanes + lane - 1 : bx * kBlock + threadIdx.x;
  const bool owns = (ROWS ? (lane >= 1 && lane <= kRowLanes) : S2 ? lane >= 1 : true) && p < out_plane;
  const int pc = owns ? p : 0;
  const int ph = pc / g.out_w, pw = pc % g.out_w;

  int cell[K];
  unsigned soff[NLOAD];
  unsigned inside = 0, live = 0;
  const size_t rplane0 = (size_t)(n * g.groups + grp) * (K * 2) * out_plane;
  const rsrc_t rr = plane_rsrc(rot + rplane0, K * 2 * out_plane);
#pragma unroll
  for (int t = 0; t < K; ++t) {
    const int f_h = t / KW, f_w = t % KW;
    int s_el, rpix;
    const bool ok = tap_geometry<false>(g, ph, pw, f_h, f_w, s_el, rpix) && owns;
    if (MODE == 0) soff[t] = ok ? (unsigned)s_el * (unsigned)sizeof(T) : kOutOfRange;
    const unsigned ro = owns ? (unsigned)((2 * t) * out_plane + pc) * (unsigned)sizeof(T) : kOutOfRange;
    const float h = scope_coord<float>(g, f_h, buf_ld(rr, ro, rot), g.centre_h);
    const float w = scope_coord<float>(g, f_w, buf_ld(rr, ro + (unsigned)out_plane * (unsigned)sizeof(T), rot),
                                       g.centre_w);
    const bool in = (h > -1.f) && (w > -1.f) && (h < float(SH)) && (w < float(SW));
    cell[t] = Tb::slot(in ? (static_cast<int>(floorf(h)) + 1) * Tb::RS + static_cast<int>(floorf(w)) + 1 : 0) * 4;
    inside |= (in && ok) ? (1u << t) : 0u;
    live |= ok ? (1u << t) : 0u;
  }
  if (ROWS) {
#pragma unroll
    for (int r = 0; r < KH; ++r) {
      const long e = (long)p + (long)(r * g.dil_h - g.pad_h) * g.in_w;
      soff[r] = (e >= 0 && e < in_plane) ? (unsigned)e * (unsigned)sizeof(T) : kOutOfRange;
    }
  }
  // S2: first element of the pair (columns 2 ow, 2 ow + 1) of tap row r, for the lane's pixel or,
  // on halo and tail lanes, for some valid pixel (see local_forward_s2_kernel)
  int pe[KH];
  if (S2) {
    const int pl = min(max(p, 0), out_plane - 1);
    const int plh = pl / g.out_w, plw = pl % g.out_w;
#pragma unroll
    for (int r = 0; r < KH; ++r) {
      const int ih = 2 * plh - 1 + r;
      pe[r] = (ih >= 0 && ih < g.in_h) ? ih * g.in_w + 2 * plw : 0;
    }
  }
  const unsigned goff = owns ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  float sb[K], sc[K], sd[K];
#pragma unroll
  for (int t = 0; t < K; ++t) sb[t] = sc[t] = sd[t] = 0.f;

  for (int j0 = c_begin; j0 < c_end; j0 += ch_per_pass) {
    const int nch = min(ch_per_pass, c_end - j0);
    __syncthreads();
    if constexpr (PAIRS)
      stage_pair_tables<T, SH, SW>(tbl, filter, g.channel, grp + g.groups * j0, g.groups, nch);
    else
      stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, grp + g.groups * j0, g.groups, nch);
    __syncthreads();
    const size_t chan0 = (size_t)n * g.channel + grp + (size_t)g.groups * j0;
    const T* xp = x + chan0 * in_plane;
    const T* gp = gout + chan0 * out_plane;
    const size_t x_step = (size_t)g.groups * in_plane, g_step = (size_t)g.groups * out_plane;

    typedef typename Pair<T>::raw pair_t;
    // loads run DEPTH - 1 channels ahead of the arithmetic: with one channel ahead the bytes a CU has
    // in flight (about 1.5 KB per wave) cover the memory latency only up to 3 TB/s
    constexpr int DEPTH = (ROWS && OCC < 5) ? 4 : 2;
    float xv[DEPTH][NLOAD], gv[DEPTH];
    pair_t xq[DEPTH][KH];
    // one descriptor per tensor for the whole pass, up to the end of its last channel's plane: a lane's
    // offset is either inside a plane or kOutOfRange, the channel is a scalar offset kept to the pass's
    // channels (what a load past the last channel returns is never accumulated)
    const rsrc_t rg = plane_rsrc(gp, (int)((nch - 1) * g_step) + out_plane);
    const rsrc_t rx = plane_rsrc(xp, (int)((nch - 1) * x_step) + in_plane);
    const int g_bytes = (int)(g_step * sizeof(T)), x_bytes = (int)(x_step * sizeof(T));
    auto load = [&](int s, int j) {
      const int jc = min(j, nch - 1);
      gv[s] = buf_ld2(rg, goff, jc * g_bytes, gout);
      if (S2) {
        const T* plane = xp + (size_t)jc * x_step;
#pragma unroll
        for (int r = 0; r < KH; ++r) xq[s][r] = *reinterpret_cast<const pair_t*>(plane + pe[r]);
      } else {
#pragma unroll
        for (int t = 0; t < NLOAD; ++t) xv[s][t] = buf_ld2(rx, soff[t], jc * x_bytes, x);
      }
    };
    auto accumulate = [&](int s, int j) {
      const float* tb = tbl + j * Tb::SIZE;
#pragma unroll
      for (int t = 0; t < K; ++t) {
        float xt;
        if (ROWS) {
          const int r = t / KW, f_w = t % KW;
          xt = f_w == 0 ? from_lane_below(xv[s][r]) : f_w == 1 ? xv[s][r] : from_lane_above(xv[s][r]);
        } else if (S2) {
          const int r = t / KW, f_w = t % KW;
          const float x0 = Pair<T>::get(xq[s][r], 0), x1 = Pair<T>::get(xq[s][r], 1);
          xt = f_w == 0 ? from_lane_below(x1) : f_w == 1 ? x0 : x1;
        } else {
          xt = xv[s][t];
        }
        // gv is 0 on lanes that own no pixel, and taps in the padding are masked at the end
        const float ps = xt * gv[s];
        const float4 q = lds_read4(tb + cell[t]);
        sb[t] = fmaf(ps, q.y, sb[t]);
        sc[t] = fmaf(ps, q.z, sc[t]);
        sd[t] = fmaf(ps, q.w, sd[t]);
      }
    };
    if constexpr (PAIRS) {
      // two channels per step: their products, rounded to bfloat16, are one operand of three
      // v_dot2c_f32_bf16 against the pair table's {b, c, d} (fp32 sums) -- six vector instructions and one
      // table read per tap and channel pair where the fp32 form takes eight and two.  The second channel
      // of an odd count's last pair is the last channel again, against a table of zeros.
      float xw[2][2][KH], gw[2][2];
      auto load_pair = [&](int s, int jp) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int jc = min(2 * jp + h, nch - 1);
          gw[s][h] = buf_ld2(rg, goff, jc * g_bytes, gout);
#pragma unroll
          for (int r_ = 0; r_ < KH; ++r_) xw[s][h][r_] = buf_ld2(rx, soff[r_], jc * x_bytes, x);
        }
      };
      auto accumulate_pair = [&](int s, int jp) {
        const float* tb = tbl + jp * Tb::SIZE;
#pragma unroll
        for (int t = 0; t < K; ++t) {
          const int r_ = t / KW, f_w = t % KW;
          float ps[2];
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const float xt = f_w == 0 ? from_lane_below(xw[s][h][r_]) : f_w == 1 ? xw[s][h][r_] : from_lane_above(xw[s][h][r_]);
            ps[h] = xt * gw[s][h];
          }
          typedef __bf16 b2 __attribute__((ext_vector_type(2)));
          const b2 pk = __builtin_bit_cast(b2, pack_bf16(ps[0], ps[1]));
          const float4 q = lds_read4(tb + cell[t]);
          sb[t] = __builtin_amdgcn_fdot2_f32_bf16(pk, __builtin_bit_cast(b2, q.x), sb[t], false);
          sc[t] = __builtin_amdgcn_fdot2_f32_bf16(pk, __builtin_bit_cast(b2, q.y), sc[t], false);
          sd[t] = __builtin_amdgcn_fdot2_f32_bf16(pk, __builtin_bit_cast(b2, q.z), sd[t], false);
        }
      };
      const int npair = (nch + 1) / 2;
      load_pair(0, 0);
      for (int jp = 0; jp < npair; jp += 2) {
        load_pair(1, jp + 1);
        accumulate_pair(0, jp);
        load_pair(0, jp + 2);
        if (jp + 1 < npair) accumulate_pair(1, jp + 1);
      }
    } else {
#pragma unroll
      for (int u = 0; u < DEPTH - 1; ++u) load(u, u);
      for (int j = 0; j < nch; j += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
          load((u + DEPTH - 1) % DEPTH, j + u + DEPTH - 1);
          if (j + u < nch) accumulate(u, j + u);
        }
      }
    }
  }

  const rsrc_t ro_ = plane_rsrc(grot + rplane0, K * 2 * out_plane);
#pragma unroll
  for (int t = 0; t < K; ++t) {
    const int f_h = t / KW, f_w = t % KW;
    const unsigned ro = owns ? (unsigned)((2 * t) * out_plane + pc) * (unsigned)sizeof(T) : kOutOfRange;
    bool open_h, open_w;  // false: the offset was clamped, its gradient is zero
    const float h = scope_coord<float>(g, f_h, buf_ld(rr, ro, rot), g.centre_h, &open_h);
    const float w = scope_coord<float>(g, f_w, buf_ld(rr, ro + (unsigned)out_plane * (unsigned)sizeof(T), rot),
                                       g.centre_w, &open_w);
    const float lh = h - floorf(h), lw = w - floorf(w);
    float gh = fmaf(lw, sd[t], sc[t]);
    float gw = fmaf(lh, sd[t], sb[t]);
    if (!(inside >> t & 1u)) gh = gw = 0.f;
    if (!open_h) gh = 0.f;
    if (!open_w) gw = 0.f;
    if (splits == 1) {
      buf_st(ro_, ro, gh, grot);
      buf_st(ro_, ro + (unsigned)out_plane * (unsigned)sizeof(T), gw, grot);
    } else if (owns) {
      float* dst = partial + (((size_t)split * g.batch * g.groups + bz) * (K * 2) + 2 * t) * out_plane + pc;
      dst[0] = gh;
      dst[out_plane] = gw;
    }
  }
  (void)live;
}

// ---------------------------------------------------------------------------
// grad filter: gW[c][i][j] = sum over (image, pixel, tap) of x_t * gout * hat(h_t - i) * hat(w_t - j).
//
// LDS float atomics serialise per lane on this hardware, and a scatter by cell is data
// dependent, so the sum is kept DENSE and in registers: a lane owns a pixel, holds for each
// tap the SH + SW hat-function weights (channel independent), and per channel adds
// ps * a_i * b_j into SH*SW private accumulators -- static register indices, no atomics.
// After each channel the 64 lanes' accumulators are folded through a per-wave LDS
// transpose (write [lane][cell], read back [cell] over 16 lanes, two cross-row
// exchanges) and lanes 0..CELLS-1 add the wave's sum into a per-wave LDS accumulator that
// persists over all the (image, tile) items the workgroup walks.  One partial per
// workgroup goes to the workspace; reduce_partials_kernel adds the partials in order.
// grid = (parts, channel splits, groups)
// ---------------------------------------------------------------------------
// accumulator slots per channel and floats per lane of the fold's transpose scratch (16-byte
// aligned, bank-skewed) for a scope of `cells` cells
constexpr int filter_slots(int cells) { return cells <= 16 ? 16 : 32; }
constexpr int filter_pitch(int cells) { return cells <= 16 ? 20 : 36; }

template <typename T, int KH, int KW, int SH, int SW, int MODE>
__global__ __launch_bounds__(kBlock, (SH * SW <= 16 ? 2 : 1)) void local_grad_filter_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ rot,
    float* __restrict__ partial, int tiles, int ch_per_block, int parts) {
  constexpr int K = KH * KW;
  constexpr int CELLS = SH * SW;
  constexpr bool ROWS = MODE == 1, S2 = MODE == 2;  // as in local_grad_rotation_kernel
  constexpr int NLOAD = MODE == 0 ? K : KH;
  constexpr int PIX = ROWS ? kRowPix : S2 ? kS2Pix : kBlock;  // pixels per (image, tile) item
  static_assert(CELLS <= 32, "the fold below handles up to two cells per lane of a 16-lane row");
  constexpr int CP = filter_slots(CELLS), kPitch = filter_pitch(CELLS);
  constexpr int kWaves = kBlock / 64;
  extern __shared__ __align__(16) float lds[];
  float* wacc = lds;                                  // [kWaves][ch_per_block][CP]
  float* scratch = lds + kWaves * ch_per_block * CP;  // [kWaves][64][kPitch]

  // logical block = (channel split, part, group), split fastest: the splits of one
  // (image, tile) item and the items of one image share an XCD
  const int cpg = g.channel / g.groups;
  const int splits = ceil_div(cpg, ch_per_block);
  const int total = splits * parts * g.groups;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int by = lb % splits, bx = lb / splits % parts, grp = lb / splits / parts;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int e = threadIdx.x; e < kWaves * ch_per_block * CP; e += blockDim.x) wacc[e] = 0.f;
  __syncthreads();

  const int j0 = by * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  const int out_plane = g.out_h * g.out_w, in_plane = g.in_h * g.in_w;
  const int items = g.batch * tiles;
  float* my_acc = wacc + wave * ch_per_block * CP;
  float* my_scr = scratch + wave * 64 * kPitch;
  // read-back pattern of the fold: lane (row = lane / 16, m = lane % 16) sums cell m over the
  // 16 lanes of its row, starting 4 * row lanes in so the four rows hit disjoint banks
  const int row = lane >> 4, m = lane & 15;

  for (int item = bx; item < items; item += parts) {
    const int n = item / tiles, tile = item % tiles;
    const int p = ROWS ? tile * PIX + wave * kRowLanes + lane - 1
                  : S2 ? tile * PIX + wave * kS2Lanes + lane - 1 : tile * PIX + (int)threadIdx.x;
    const bool owns = (ROWS ? (lane >= 1 && lane <= kRowLanes) : S2 ? lane >= 1 : true) && p < out_plane;
    const int pc = owns ? p : 0;
    const int ph = pc / g.out_w, pw = pc % g.out_w;

    float ah[K][SH], bw[K][SW];
    unsigned soff[NLOAD];
    const rsrc_t rr = plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K * 2) * out_plane, K * 2 * out_plane);
#pragma unroll
    for (int t = 0; t < K; ++t) {
      const int f_h = t / KW, f_w = t % KW;
      int s_el, rpix;
      const bool ok = tap_geometry<false>(g, ph, pw, f_h, f_w, s_el, rpix) && owns;
      if (MODE == 0) soff[t] = ok ? (unsigned)s_el * (unsigned)sizeof(T) : kOutOfRange;
      const unsigned ro = ok ? (unsigned)((2 * t) * out_plane + rpix) * (unsigned)sizeof(T) : kOutOfRange;
      const float h = scope_coord<float>(g, f_h, buf_ld(rr, ro, rot), g.centre_h);
      const float w = scope_coord<float>(g, f_w, buf_ld(rr, ro + (unsigned)out_plane * (unsigned)sizeof(T), rot),
                                         g.centre_w);
      // hat(h - i) = lh at i = floor(h) + 1, 1 - lh at i = floor(h), else 0: the same products
      // (hh, lh) x (hw, lw) as K.cu:101-112, laid out densely; all zero outside (-1, S) and for
      // taps in the padding.
      const bool in = ok && (h > -1.f) && (w > -1.f) && (h < float(SH)) && (w < float(SW));
      const float hf = floorf(h), wf = floorf(w);
      const int hl = in ? (int)hf : -8, wl = in ? (int)wf : -8;
      const float lh = h - hf, lw = w - wf;
#pragma unroll
      for (int i = 0; i < SH; ++i) ah[t][i] = (i == hl) ? 1.f - lh : (i == hl + 1) ? lh : 0.f;
#pragma unroll
      for (int i = 0; i < SW; ++i) bw[t][i] = (i == wl) ? 1.f - lw : (i == wl + 1) ? lw : 0.f;
    }
    if (ROWS) {
#pragma unroll
      for (int r = 0; r < KH; ++r) {
        const long e = (long)p + (long)(r * g.dil_h - g.pad_h) * g.in_w;
        soff[r] = (e >= 0 && e < in_plane) ? (unsigned)e * (unsigned)sizeof(T) : kOutOfRange;
      }
    }
    int pe[KH];  // S2: first element of the pair of tap row r (see local_forward_s2_kernel)
    if (S2) {
      const int pl = min(max(p, 0), out_plane - 1);
      const int plh = pl / g.out_w, plw = pl % g.out_w;
#pragma unroll
      for (int r = 0; r < KH; ++r) {
        const int ih = 2 * plh - 1 + r;
        pe[r] = (ih >= 0 && ih < g.in_h) ? ih * g.in_w + 2 * plw : 0;
      }
    }
    const unsigned goff = owns ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

    const size_t chan0 = (size_t)n * g.channel + grp + (size_t)g.groups * j0;
    const T* xp = x + chan0 * in_plane;
    const T* gp = gout + chan0 * out_plane;
    const size_t x_step = (size_t)g.groups * in_plane, g_step = (size_t)g.groups * out_plane;

    typedef typename Pair<T>::raw pair_t;
    float xv[2][NLOAD], gv[2];
    pair_t xq[2][KH];
    auto load = [&](int s, int j) {
      const rsrc_t rg = plane_rsrc(gp + (size_t)j * g_step, j < nch ? out_plane : 0);
      gv[s] = buf_ld(rg, goff, gout);
      if (S2) {
        const T* plane = xp + (size_t)min(j, nch - 1) * x_step;  // past the last channel gv is 0
#pragma unroll
        for (int r = 0; r < KH; ++r) xq[s][r] = *reinterpret_cast<const pair_t*>(plane + pe[r]);
      } else {
        const rsrc_t rx = plane_rsrc(xp + (size_t)j * x_step, j < nch ? in_plane : 0);
#pragma unroll
        for (int t = 0; t < NLOAD; ++t) xv[s][t] = buf_ld(rx, soff[t], x);
      }
    };
    auto accumulate = [&](int s, int j) {
      float acc[SH][SW];
#pragma unroll
      for (int i = 0; i < SH; ++i)
#pragma unroll
        for (int k = 0; k < SW; ++k) acc[i][k] = 0.f;
#pragma unroll
      for (int t = 0; t < K; ++t) {
        float xt;
        if (ROWS) {
          const int r = t / KW, f_w = t % KW;
          xt = f_w == 0 ? from_lane_below(xv[s][r]) : f_w == 1 ? xv[s][r] : from_lane_above(xv[s][r]);
        } else if (S2) {
          const int r = t / KW, f_w = t % KW;
          const float x0 = Pair<T>::get(xq[s][r], 0), x1 = Pair<T>::get(xq[s][r], 1);
          xt = f_w == 0 ? from_lane_below(x1) : f_w == 1 ? x0 : x1;
        } else {
          xt = xv[s][t];
        }
        const float ps = xt * gv[s];
        float u[SW];
#pragma unroll
        for (int k = 0; k < SW; ++k) u[k] = ps * bw[t][k];
#pragma unroll
        for (int i = 0; i < SH; ++i)
#pragma unroll
          for (int k = 0; k < SW; ++k) acc[i][k] += ah[t][i] * u[k];
      }
      // fold the wave: transpose through the wave's scratch
      float* mine = my_scr + lane * kPitch;
#pragma unroll
      for (int i = 0; i < SH; ++i)
#pragma unroll
        for (int k = 0; k < SW; ++k) mine[i * SW + k] = acc[i][k];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      float sum[CP / 16];
#pragma unroll
      for (int h = 0; h < CP / 16; ++h) {  // cells m and (scopes of more than 16 cells) m + 16
        sum[h] = 0.f;
        if (m + 16 * h < CELLS) {
#pragma unroll
          for (int q = 0; q < 16; ++q) sum[h] += my_scr[(row * 16 + ((q + 4 * row) & 15)) * kPitch + m + 16 * h];
        }
        sum[h] += __shfl_xor(sum[h], 16, 64);
        sum[h] += __shfl_xor(sum[h], 32, 64);
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int h = 0; h < CP / 16; ++h)
        if (lane < 16 && lane + 16 * h < CELLS && j < nch) my_acc[j * CP + lane + 16 * h] += sum[h];
    };

    load(0, 0);
    for (int j = 0; j < nch; j += 2) {
      load(1, j + 1);
      accumulate(0, j);
      load(0, j + 2);
      accumulate(1, j + 1);
    }
  }
  __syncthreads();

  for (int e = threadIdx.x; e < nch * CELLS; e += blockDim.x) {
    const int j = e / CELLS, r = e % CELLS;
    float s_ = 0.f;
#pragma unroll
    for (int wv = 0; wv < kWaves; ++wv) s_ += wacc[(wv * ch_per_block + j) * CP + r];
    const int c = grp + g.groups * (j0 + j);
    partial[((size_t)bx * g.channel + c) * CELLS + r] = s_;
  }
}

}  // namespace

// ---------------------------------------------------------------------------
// grad filter on the matrix cores, for "same" geometries (see local_gather_rows_kernel).
//
// With k = (pixel, tap) the reduction is a matrix product per block of 16 channels,
//   gW[cell][c] = sum_k A[cell][k] * P[k][c],
//   A[cell = (i, j)][k] = hat(h_k - i) * hat(w_k - j)      (channel independent),
//   P[k][c] = x_k[c] * gout[c],
// and v_mfma_f32_16x16x4_f32 adds a 16 (cells) x 16 (channels) block over four k per issue in
// full fp32: lane l supplies A[l % 16][l / 16] and P[l / 16][l % 16].  So a lane stands for
// cell l % 16 on the A side and for channel l % 16 on the P side, and for pixel quad l / 16.
//
// A unit of work is (image, 128-pixel tile, channel block); a workgroup of 8 waves walks a
// contiguous range of units, channel block fastest, so that all workgroups (two per CU, all
// resident) carry the same load.  Wave w owns pixels 16 w .. 16 w + 15 of the tile.
//   * per tile: the scope coordinates (h, w) of every (pixel, tap) go to LDS (taps in the
//     padding and coordinates outside the scope band as (-2, -2), where every hat is 0) and
//     every lane derives its 36 A values (4 pixels x 9 taps), kept in registers for all the
//     channel blocks of the tile;
//   * per unit: the 16 channels' tiles of gout and of x with its halo rows are staged
//     channel-major in LDS from loads coalesced along pixels; a lane reads its channel's
//     4 gout and 3 x 6 input values and issues 36 MFMAs (fp32 inputs: v_mfma_f32_16x16x4_f32;
//     16-bit inputs: 9 v_mfma_f32_16x16x16_bf16 on operands rounded to bfloat16, fp32 sums).
//     The loads of the next unit are issued before the MFMAs and land in registers while they run.
//   * the 8 waves' 16 x 16 results of a unit are added into a per-channel-block accumulator in
//     LDS (by a fixed owner thread, in wave order), piggybacked on the next unit's barriers.
// One partial per workgroup goes to the workspace; reduce_partials_kernel adds them in order.
// grid = (workgroups, channel splits, groups); a channel split is at most kMfMaxBlk blocks
// ---------------------------------------------------------------------------
constexpr int kMfPix = 128;            // output pixels per tile
constexpr int kMfCh = 16;              // channels per unit
constexpr int kMfBlock = 512;          // threads per workgroup
constexpr int kMfPitchG = kMfPix + 4;  // floats per channel of the gout tile (16-byte reads, bank skew)
constexpr int kMfX = 6;                // at most this many input elements per lane and channel: tile + halo rows <= 64 * kMfX
constexpr int kMfMaxBlk = 16;          // channel blocks accumulated by one workgroup
constexpr int kMfXS2 = 9;              // stride 2: staged input elements per lane and channel
constexpr int kMfMaxBlkS2 = 12;        // stride 2: channel blocks per workgroup (two workgroups' LDS fit a CU)

typedef float mf4 __attribute__((ext_vector_type(4)));
typedef __bf16 mfb4 __attribute__((ext_vector_type(4)));

// First float of channel j's row in the staged input tile.  The rows are a multiple of 64 floats
// apart plus a skew: in the MFMA phase lane (channel q, pixel quad kg) reads row q at
// 4 * kg + const, and (q % 4) + 16 * (q / 4) + 4 * kg covers the 64 banks exactly once.
__device__ __forceinline__ int mf_row(int j, int pitch_x) { return j * pitch_x + (j & 3) + 16 * (j >> 2); }

__device__ __forceinline__ float hat(float d) { return __builtin_amdgcn_fmed3f(1.f - fabsf(d), 0.f, 1.f); }

// CELL0: the kernel sums the scope cells CELL0 .. CELL0 + 15 (the 16 rows of one MFMA block); a
// scope of more than 16 cells takes further launches (5 x 5: CELL0 = 16; 7 x 7: 16, 32, 48).
// S2: the stride-2 geometry of local_forward_s2_kernel.  A tile is then `th` whole output rows (at
// most 128 pixels), so that the input rows its taps read, 2 oh0 - 1 .. 2 (oh0 + th - 1) + 1, are
// one contiguous range of the plane like the stride-1 tile with its halo rows; a lane's four
// pixels may sit in different rows, so each reads its own 3 x 3 inputs.
// SPLIT (float32 tensors): both operands as bfloat16 pairs, A = Ah + Al and P = Ph + Pl (hi = the
// value rounded to bfloat16, lo = the rounded remainder: together 16 significand bits), and three
// products Ah Ph + Ah Pl + Al Ph on v_mfma_f32_16x16x16_bf16 with fp32 sums instead of one on
// v_mfma_f32_16x16x4_f32.  The fp32 instruction takes 32 clk of the SIMD's issue slots for 4 k and
// does not overlap with vector ALU work, not even of other waves; a bfloat16 one covers 16 k in
// 16 clk of the matrix pipe and runs beside other waves' vector ALU work (measured: it adds about
// 6 clk to a SIMD busy with FMAs).  A unit is then 27 matrix instructions instead of 36 and pays
// 12 more vector ALU instructions per tap for the split of P.  The dropped Al Pl and the rounding
// of the lo parts leave a relative error of about 2^-16 per product -- the filter gradient is held
// to 1e-4 of its largest element and sums thousands of products of either sign.
// CL: channels-last tensors (x and gout as [image][pixel][channel], rotation as [image][pixel][tap][2];
// one group).  Only the staging differs: a thread loads four consecutive channels of a pixel (the unit's
// sixteen channels are 64 contiguous bytes per pixel) and stores them into the same channel-major tiles
// in LDS, so the products run as for planar tensors.
template <typename T, int SH, int SW, int CELL0, int NX, bool S2, bool BF = false, bool SPLIT = false, bool CL = false>
__global__ __launch_bounds__(kMfBlock, 4) void local_grad_filter_mfma_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ rot,
    float* __restrict__ partial, int tiles, int nwg, int csplits, int pitch_x, int th) {
  constexpr int K = 9, CELLS = SH * SW;
  constexpr int kWaves = kMfBlock / 64;
  static_assert(CELL0 % 16 == 0 && CELL0 < CELLS, "the cells come in slices of 16, the rows of one MFMA block");
  static_assert(kMfPix == 16 * kWaves, "one 16-pixel group per wave");
  extern __shared__ __align__(16) float lds[];
  float* xs = lds;                                                  // [kMfCh][pitch_x]
  float* gs = xs + kMfCh * pitch_x;                                 // [kMfCh][kMfPitchG]
  float2* hw = reinterpret_cast<float2*>(gs + kMfCh * kMfPitchG);   // [K][kMfPix]
  float* red = reinterpret_cast<float*>(hw + K * kMfPix);           // [kWaves][256]
  float* accs = red + kWaves * 256;                                 // [blocks of this split][256]

  const int cpg = g.channel / g.groups;
  const int nblk_all = ceil_div(cpg, kMfCh);
  const int total = nwg * csplits * g.groups;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int wg = lb % nwg, cs = lb / nwg % csplits, grp = lb / nwg / csplits;
  const int blk_per = ceil_div(nblk_all, csplits);
  const int cb_lo = cs * blk_per, nblk = min(blk_per, nblk_all - cb_lo);

  const int W = g.in_w;  // == out_w unless S2
  const int OW = g.out_w;
  const int out_plane = g.out_h * OW, in_plane = g.in_h * W;
  const int tile_pix = S2 ? th * OW : kMfPix;  // pixels of a tile (pixel slots past them carry zero weights)
  // the wave index picks channel planes (buffer resources): tell the compiler it is uniform
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int q = lane & 15, kg = lane >> 4;
  const int row_step = g.dil_h * W;               // elements between two tap rows
  const int lo = -g.pad_h * W - 1;                // first staged input element, relative to the tile
  // rows past the last cell (9..15 of a 3 x 3 scope, 25..31 of a 5 x 5 one) stay 0
  const float ci = CELL0 + q < CELLS ? float((CELL0 + q) / SW) : 64.f, cj = float((CELL0 + q) % SW);

  for (int e = threadIdx.x; e < nblk * 256; e += kMfBlock) accs[e] = 0.f;

  // This workgroup's share of the (tile, channel block) units of its group and channel split, as
  // segments (tile, first block, end block).  Whole tiles are dealt out round-robin, tile t to
  // workgroup t % nwg, so that neighbouring workgroups (same XCD, same pace) hold neighbouring
  // tiles of the same channel block at the same time and the halo rows they share are fetched
  // from memory once (a contiguous range of tiles per workgroup re-fetches them: 1.5 x the reads).
  // The units of the last items % nwg tiles -- all of them when the tiles are fewer than the
  // workgroups -- are dealt out as contiguous ranges in (tile, block) order, cut at the tile
  // boundaries, so that a tile's set-up (scope coordinates, hat products) is paid once per
  // workgroup and not once per unit.
  const int items = g.batch * tiles;
  const int whole = items / nwg;                      // whole tiles per workgroup
  const long rest_units = (long)(items - whole * nwg) * nblk;
  const long r_lo = rest_units * wg / nwg, r_hi = rest_units * (wg + 1) / nwg;
  const int rest_lo = (int)(r_lo / nblk), rest_hi = r_hi > r_lo ? (int)((r_hi - 1) / nblk) : rest_lo - 1;
  const int nseg = whole + (rest_hi - rest_lo + 1);
  auto segment = [&](int k, int& item, int& cb_begin, int& cb_end) {
    if (k < whole) {
      item = wg + k * nwg;
      cb_begin = 0;
      cb_end = nblk;
    } else {
      const int t = rest_lo + (k - whole);
      item = whole * nwg + t;
      cb_begin = t == rest_lo ? (int)(r_lo % nblk) : 0;
      cb_end = t == rest_hi ? (int)((r_hi - 1) % nblk) + 1 : nblk;
    }
  };

  // Register stage of one unit: what this thread loads (the rotation values of its pixel for
  // its share of the taps when the unit starts a tile; kMfX input and 2 gout values of each of
  // its wave's 2 channels).
  constexpr int kChW = kMfCh / kWaves;                                  // channels staged per wave
  constexpr int kTapsT = (K + kMfBlock / kMfPix - 1) / (kMfBlock / kMfPix);  // taps staged per thread
  const int pix = threadIdx.x % kMfPix;                                 // pixel whose coordinates this thread stages
  const int tapq = __builtin_amdgcn_readfirstlane(threadIdx.x / kMfPix);  // ... for taps tapq + 4 k
  float r_rot[2 * kTapsT], r_x[kChW][NX], r_g[kChW][kMfPix / 64];
  // CL: thread (pixel slot cl_p, channel quad cl_q) stages four channels of NX / 2 input pixels and of one gout pixel
  static_assert(!CL || (!S2 && NX % 2 == 0 && kMfBlock == 4 * kMfPix), "channels-last staging: four threads per pixel");
  const int cl_p = threadIdx.x >> 2, cl_q = threadIdx.x & 3;
  typename std::conditional<sizeof(T) == 4, nhwc_u4, nhwc_u2>::type c_x[NX / 2], c_g;
  auto issue_loads = [&](int item, int cbi, bool with_rot) {
    const int cb = cb_lo + cbi;
    const int n = item / tiles, p0 = (item % tiles) * tile_pix;
    // first staged input element: the tile's first pixel minus the halo; S2: one element before
    // input row 2 oh0 - 1 (so that column -1 of a row's first pixel is a valid, unused slot)
    const int x0 = S2 ? (2 * (item % tiles) * th - 1) * W - 1 : p0 + lo;
    if (with_rot) {
      const int p = p0 + pix;
      if constexpr (CL) {
        const rsrc_t rr = plane_rsrc(rot + (size_t)n * (K * 2) * out_plane, K * 2 * out_plane);
        const unsigned ro = p < out_plane ? (unsigned)(p * (K * 2)) * (unsigned)sizeof(T) : kOutOfRange;
#pragma unroll
        for (int k = 0; k < kTapsT; ++k) {
          const int t = tapq + (kMfBlock / kMfPix) * k;
          const unsigned o = t < K ? ro + (unsigned)(2 * t) * (unsigned)sizeof(T) : kOutOfRange;
          r_rot[2 * k] = buf_ld(rr, o, rot);
          r_rot[2 * k + 1] = buf_ld(rr, o + (unsigned)sizeof(T), rot);
        }
      } else {
      const rsrc_t rr = plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K * 2) * out_plane, K * 2 * out_plane);
      const unsigned ro = p < out_plane ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;
#pragma unroll
      for (int k = 0; k < kTapsT; ++k) {
        const int t = tapq + (kMfBlock / kMfPix) * k;
        const unsigned o = t < K ? ro + (unsigned)(2 * t * out_plane) * (unsigned)sizeof(T) : kOutOfRange;
        r_rot[2 * k] = buf_ld(rr, o, rot);
        r_rot[2 * k + 1] = buf_ld(rr, o + (unsigned)out_plane * (unsigned)sizeof(T), rot);
      }
      }
    }
    if constexpr (CL) {
      // one image's pixels; a quad past the last channel, an element before the plane: zeros (the host
      // admits channel counts that are a multiple of 4 only, so a quad is inside or outside as a whole)
      const int C = g.channel;
      const rsrc_t rx = plane_rsrc(x + (size_t)n * in_plane * C, in_plane * C);
      const rsrc_t rg = plane_rsrc(gout + (size_t)n * out_plane * C, out_plane * C);
      const int c4 = cb * kMfCh + 4 * cl_q;
      const bool quad = c4 < C;
      const unsigned co = (unsigned)c4 * (unsigned)sizeof(T);
#pragma unroll
      for (int k = 0; k < NX / 2; ++k) {
        const int e = x0 + cl_p + kMfPix * k;
        c_x[k] = raw_ld4(rx, e < 0 || !quad ? kOutOfRange : (unsigned)(e * C) * (unsigned)sizeof(T) + co, x);
      }
      c_g = raw_ld4(rg, quad ? (unsigned)((p0 + cl_p) * C) * (unsigned)sizeof(T) + co : kOutOfRange, gout);
      return;
    }
#pragma unroll
    for (int jj = 0; jj < kChW; ++jj) {
      const int cj_ = cb * kMfCh + wave + jj * kWaves;
      const bool chan = cj_ < cpg;
      const size_t c = (size_t)n * g.channel + grp + (size_t)g.groups * (chan ? cj_ : 0);
      const rsrc_t rx = plane_rsrc(x + c * in_plane, chan ? in_plane : 0);
      const rsrc_t rg = plane_rsrc(gout + c * out_plane, chan ? out_plane : 0);
      // Elements past the plane's end fail the buffer's range check and read 0; the 64 * NX staged
      // elements may run past the tile's halo (never read).  Elements BEFORE the plane (the first
      // tile's top halo row) get the out-of-range offset explicitly: left as negative offsets they
      // are huge unsigned numbers and also fail the check, but the compiler then addresses the
      // loads of one lane as one base register plus immediates, and with a negative base the
      // first three elements of the plane came back as 0 on planes 64 and 112 columns wide.
#pragma unroll
      for (int k = 0; k < NX; ++k) {
        const int e = x0 + lane + 64 * k;
        r_x[jj][k] = buf_ld(rx, e < 0 ? kOutOfRange : (unsigned)e * (unsigned)sizeof(T), x);
      }
#pragma unroll
      for (int k = 0; k < kMfPix / 64; ++k)
        r_g[jj][k] = buf_ld(rg, (unsigned)(p0 + lane + 64 * k) * (unsigned)sizeof(T), gout);
    }
  };
  // Register stage -> LDS.  Scope coordinates: K.cu:338-341 and the band test of K.cu:59.
  auto store_unit = [&](int item, bool with_rot) {
    if (with_rot) {
      const int p = (item % tiles) * tile_pix + pix;
      const bool live = pix < tile_pix && p < out_plane;
      const int pc = live ? p : 0;
      const int ph = pc / OW, pw = pc % OW;
#pragma unroll
      for (int k = 0; k < kTapsT; ++k) {
        const int t = tapq + (kMfBlock / kMfPix) * k;
        if (t < K) {
          const int f_h = t / 3, f_w = t % 3;
          const int ih = S2 ? 2 * ph - 1 + f_h : ph + f_h * g.dil_h - g.pad_h, iw = S2 ? 2 * pw - 1 + f_w : pw + f_w - 1;
          const bool ok = live && ih >= 0 && ih < g.in_h && iw >= 0 && iw < W;
          const float h = scope_coord<float>(g, f_h, r_rot[2 * k], g.centre_h);
          const float w = scope_coord<float>(g, f_w, r_rot[2 * k + 1], g.centre_w);
          const bool in = ok && (h > -1.f) && (w > -1.f) && (h < float(SH)) && (w < float(SW));
          hw[t * kMfPix + pix] = in ? make_float2(h, w) : make_float2(-2.f, -2.f);
        }
      }
    }
    if constexpr (CL) {
      // channel 4 cl_q + i of pixel slot cl_p: over a wave's sixteen pixels and four quads the 64 banks once
      float gv[4];
      raw_cvt4(c_g, gv, gout);
#pragma unroll
      for (int i = 0; i < 4; ++i) gs[(4 * cl_q + i) * kMfPitchG + cl_p] = gv[i];
#pragma unroll
      for (int k = 0; k < NX / 2; ++k) {
        float xv[4];
        raw_cvt4(c_x[k], xv, x);
#pragma unroll
        for (int i = 0; i < 4; ++i) xs[mf_row(4 * cl_q + i, pitch_x) + cl_p + kMfPix * k] = xv[i];
      }
      return;
    }
#pragma unroll
    for (int jj = 0; jj < kChW; ++jj) {
      const int j = wave + jj * kWaves;
#pragma unroll
      for (int k = 0; k < NX; ++k) xs[mf_row(j, pitch_x) + lane + 64 * k] = r_x[jj][k];
#pragma unroll
      for (int k = 0; k < kMfPix / 64; ++k) gs[j * kMfPitchG + lane + 64 * k] = r_g[jj][k];
    }
  };

  const int px = wave * 16 + 4 * kg;  // first of this lane's four pixels in the tile
  // S2: pixel (dh, pw) of the tile reads the staged elements (2 dh + r) W + 2 pw + f_w (pixel slots
  // past the tile read the last pixel's: their weights are zero)
  int xb[4] = {0, 0, 0, 0};
  if constexpr (S2) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) {
      const int pi = min(px + ii, tile_pix - 1), dh = pi / OW, pw = pi - dh * OW;
      xb[ii] = 2 * dh * W + 2 * pw;
    }
  }
  // 16-bit inputs: the four pixels a lane holds per tap become the four k of one
  // v_mfma_f32_16x16x16_bf16 (k = 4 kg + ii), hat products and x * gout products rounded to
  // bfloat16 (for fp16 inputs too: the products can leave fp16's range), fp32 accumulation --
  // 9 matrix instructions of 16 clk per unit instead of 36 of 32 clk.
  // Against the result's largest element the rounding noise is about 3e-3 when a group has many
  // (channel, cell) results, but with a handful of results that largest element can itself be
  // small (one channel, 3 x 3 scope: 1.1e-2 seen), so groups of fewer than 16 channels keep the
  // fp32 instructions (template parameter BF, chosen by the host).
  static_assert(!BF || sizeof(T) == 2, "bfloat16 matrix instructions are for 16-bit inputs");
  static_assert(!SPLIT || (sizeof(T) == 4 && !BF), "the split is for float32 inputs");
  constexpr bool kHalfIn = BF;
  float A[(kHalfIn || SPLIT) ? 1 : 4][K];
  mfb4 Ab[(kHalfIn || SPLIT) ? K : 1];  // SPLIT: the hi parts
  mfb4 Al[SPLIT ? K : 1];               // ... and the lo parts
  mf4 acc = {0.f, 0.f, 0.f, 0.f};
  int done_cb = -1;  // channel block (within the split) whose result `acc` holds

  // stage the unit whose loads are in flight, hand the previous unit's result to its owner
  // threads, start the next unit's loads (n_item < 0: there is none)
  auto begin_unit = [&](int item, bool new_tile, int n_item, int n_cbi, bool n_new_tile) {
    __syncthreads();  // the previous unit's reads of the tiles (and of `red`) are done
    store_unit(item, new_tile);
    if (done_cb >= 0) *reinterpret_cast<mf4*>(red + (wave * 64 + lane) * 4) = acc;
    __syncthreads();
    if (n_item >= 0) issue_loads(n_item, n_cbi, n_new_tile);
    if (done_cb >= 0 && threadIdx.x < 256) {
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) s += red[w * 256 + threadIdx.x];
      accs[done_cb * 256 + threadIdx.x] += s;
    }
  };
  auto multiply_unit = [&](int cbi) {
    mf4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    const float4 gv = *reinterpret_cast<const float4*>(gs + q * kMfPitchG + px);
    const float gq[4] = {gv.x, gv.y, gv.z, gv.w};
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      float xv[4][3];  // the inputs of tap row r: pixel ii, column f_w
      if constexpr (S2) {
#pragma unroll
        for (int ii = 0; ii < 4; ++ii) {
          const float* xr = xs + mf_row(q, pitch_x) + xb[ii] + r * W;
#pragma unroll
          for (int f_w = 0; f_w < 3; ++f_w) xv[ii][f_w] = xr[f_w];
        }
      } else {
        // columns -1 .. +4 of tap row r around the four pixels
        const float* xr = xs + mf_row(q, pitch_x) + px + r * row_step;
        float x6[6];
#pragma unroll
        for (int k = 0; k < 6; ++k) x6[k] = xr[k];
#pragma unroll
        for (int ii = 0; ii < 4; ++ii)
#pragma unroll
          for (int f_w = 0; f_w < 3; ++f_w) xv[ii][f_w] = x6[ii + f_w];
      }
#pragma unroll
      for (int f_w = 0; f_w < 3; ++f_w) {
        const int t = r * 3 + f_w;
        if constexpr (SPLIT) {
          // every instruction adds into a live accumulator, so its result registers cannot be
          // given to one of its operands (see dk_local_mfma.hip for what happens when they can)
          // two values per conversion instruction (v_cvt_pk_bf16_f32 leaves them packed as the matrix operand wants
          // them; converted one by one they cost a conversion and half a byte permute each, six vector
          // instructions per product instead of four)
          float pr[4];
#pragma unroll
          for (int ii = 0; ii < 4; ++ii) {
            pr[ii] = xv[ii][f_w] * gq[ii];
            asm volatile("" : "+v"(pr[ii]));  // one fp32 value for both parts: no contraction into the conversions
          }
          const unsigned h01 = pack_bf16(pr[0], pr[1]), h23 = pack_bf16(pr[2], pr[3]);
          const unsigned l01 = pack_bf16(pr[0] - bf16_lo(h01), pr[1] - bf16_hi(h01));
          const unsigned l23 = pack_bf16(pr[2] - bf16_lo(h23), pr[3] - bf16_hi(h23));
          const mfb4 bh = __builtin_bit_cast(mfb4, make_uint2(h01, h23));
          const mfb4 bl = __builtin_bit_cast(mfb4, make_uint2(l01, l23));
          if (t & 1) {
            acc1 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(Ab[t], bh, acc1, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(Ab[t], bl, acc1, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(Al[t], bh, acc1, 0, 0, 0);
          } else {
            acc0 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(Ab[t], bh, acc0, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(Ab[t], bl, acc0, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(Al[t], bh, acc0, 0, 0, 0);
          }
        } else if constexpr (kHalfIn) {
          const mfb4 b = __builtin_bit_cast(mfb4, make_uint2(pack_bf16(xv[0][f_w] * gq[0], xv[1][f_w] * gq[1]),
                                                             pack_bf16(xv[2][f_w] * gq[2], xv[3][f_w] * gq[3])));
          if (t & 1)
            acc1 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(Ab[t], b, acc1, 0, 0, 0);
          else
            acc0 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(Ab[t], b, acc0, 0, 0, 0);
        } else {
#pragma unroll
          for (int ii = 0; ii < 4; ++ii) {
            const float b = xv[ii][f_w] * gq[ii];
            if ((ii + t) & 1)
              acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(A[ii][t], b, acc1, 0, 0, 0);
            else
              acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(A[ii][t], b, acc0, 0, 0, 0);
          }
        }
      }
    }
    acc = acc0 + acc1;
    done_cb = cbi;
  };

  int item = 0, cb_begin = 0, cb_end = 0;
  if (nseg > 0) {
    segment(0, item, cb_begin, cb_end);
    issue_loads(item, cb_begin, true);
  }
  for (int k = 0; k < nseg; ++k) {
    int n_item = -1, n_begin = 0, n_end = 0;  // the next segment, whose first unit follows this one's last
    if (k + 1 < nseg) segment(k + 1, n_item, n_begin, n_end);
    const bool single = cb_begin + 1 == cb_end;
    begin_unit(item, true, single ? n_item : item, single ? n_begin : cb_begin + 1, single);
#pragma unroll
    for (int t = 0; t < K; ++t) {
      const float4 hw01 = *reinterpret_cast<const float4*>(hw + t * kMfPix + px);
      const float4 hw23 = *reinterpret_cast<const float4*>(hw + t * kMfPix + px + 2);
      const float a0 = hat(hw01.x - ci) * hat(hw01.y - cj), a1 = hat(hw01.z - ci) * hat(hw01.w - cj);
      const float a2 = hat(hw23.x - ci) * hat(hw23.y - cj), a3 = hat(hw23.z - ci) * hat(hw23.w - cj);
      if constexpr (SPLIT) {
        float av[4] = {a0, a1, a2, a3};
#pragma unroll
        for (int ii = 0; ii < 4; ++ii) asm volatile("" : "+v"(av[ii]));
        const unsigned h01 = pack_bf16(av[0], av[1]), h23 = pack_bf16(av[2], av[3]);
        Ab[t] = __builtin_bit_cast(mfb4, make_uint2(h01, h23));
        Al[t] = __builtin_bit_cast(mfb4, make_uint2(pack_bf16(av[0] - bf16_lo(h01), av[1] - bf16_hi(h01)),
                                                    pack_bf16(av[2] - bf16_lo(h23), av[3] - bf16_hi(h23))));
      } else if constexpr (kHalfIn) {
        Ab[t] = __builtin_bit_cast(mfb4, make_uint2(pack_bf16(a0, a1), pack_bf16(a2, a3)));
      } else {
        A[0][t] = a0;
        A[1][t] = a1;
        A[2][t] = a2;
        A[3][t] = a3;
      }
    }
    multiply_unit(cb_begin);
    for (int cbi = cb_begin + 1; cbi < cb_end; ++cbi) {
      const bool last = cbi + 1 == cb_end;
      begin_unit(item, false, last ? n_item : item, last ? n_begin : cbi + 1, last);
      multiply_unit(cbi);
    }
    item = n_item;
    cb_begin = n_begin;
    cb_end = n_end;
  }

  // the last unit's result, then D[cell = 4 * (l / 16) + r][channel = l % 16] (register r of lane l,
  // entry 4 l + r of a block's accumulator) goes out as this workgroup's partial
  __syncthreads();
  if (done_cb >= 0) *reinterpret_cast<mf4*>(red + (wave * 64 + lane) * 4) = acc;
  __syncthreads();
  if (done_cb >= 0 && threadIdx.x < 256) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) s += red[w * 256 + threadIdx.x];
    accs[done_cb * 256 + threadIdx.x] += s;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < nblk * 256; e += kMfBlock) {
    const int b = e / 256, l = (e % 256) / 4, r = e % 4;
    const int cell = CELL0 + 4 * (l / 16) + r, cj_ = (cb_lo + b) * kMfCh + l % 16;
    if (cell < CELLS && cj_ < cpg)
      partial[((size_t)wg * g.channel + grp + (size_t)g.groups * cj_) * CELLS + cell] = accs[e];
  }
}

// out[e] = sum over parts of partial[part][e].  8 elements per workgroup, 32 threads per
// element each summing every 32nd part, combined in a fixed order (run-to-run reproducible).
constexpr int kRedEl = 8, kRedSlices = 32;

template <typename CT, typename T>
__global__ __launch_bounds__(kRedEl * kRedSlices) void reduce_partials_kernel(
    const CT* __restrict__ partial, int parts, int count, T* __restrict__ out) {
  __shared__ CT part_sum[kRedSlices][kRedEl];
  const int el = threadIdx.x % kRedEl, slice = threadIdx.x / kRedEl;
  const int e = blockIdx.x * kRedEl + el;
  CT s = 0;
  if (e < count) {
#pragma unroll 4
    for (int q = slice; q < parts; q += kRedSlices) s += partial[(size_t)q * count + e];
  }
  part_sum[slice][el] = s;
  __syncthreads();
  if (slice == 0 && e < count) {
    CT t = 0;
#pragma unroll
    for (int k = 0; k < kRedSlices; ++k) t += part_sum[k][el];
    st(out + e, t);
  }
}

// The same sum for few parts of many elements (channel splits of a gradient image): one
// element per thread, parts added in order, coalesced.
template <typename CT, typename T>
__global__ __launch_bounds__(kBlock) void reduce_few_parts_kernel(const CT* __restrict__ partial, int parts,
                                                                  long count, T* __restrict__ out) {
  const long e = (long)blockIdx.x * kBlock + threadIdx.x;
  if (e >= count) return;
  CT s = partial[e];
  for (int q = 1; q < parts; ++q) s += partial[(size_t)q * count + e];
  st(out + e, s);
}

template <typename CT, typename T>
void launch_reduce_partials(const CT* partial, int parts, long count, T* out, hipStream_t stream) {
  // parts == 0 (an empty batch) takes the second kernel, which then writes zeros and reads nothing
  if (parts > 0 && parts <= kRedSlices && count >= 16384)
    reduce_few_parts_kernel<CT, T><<<(unsigned)((count + kBlock - 1) / kBlock), kBlock, 0, stream>>>(partial, parts, count, out);
  else
    reduce_partials_kernel<CT, T><<<(unsigned)((count + kRedEl - 1) / kRedEl), kRedEl * kRedSlices, 0, stream>>>(partial, parts, (int)count, out);
}
template void launch_reduce_partials<float, float>(const float*, int, long, float*, hipStream_t);
template void launch_reduce_partials<float, __half>(const float*, int, long, __half*, hipStream_t);
template void launch_reduce_partials<float, bf16_t>(const float*, int, long, bf16_t*, hipStream_t);
template void launch_reduce_partials<double, double>(const double*, int, long, double*, hipStream_t);

// ---------------------------------------------------------------------------
// host-side dispatch of the tuned path
// ---------------------------------------------------------------------------
namespace {

constexpr int kMaxLdsTables = 60 * 1024;  // bytes of LDS a workgroup may spend on scope tables (64 KB launch limit)

// stride 1, unit column spacing and pad_w = 1: input and output planes share their width and a
// pixel's taps are three runs of three consecutive elements
bool same_width_geometry(const Geo& g) {
  return g.stride_h == 1 && g.stride_w == 1 && g.dil_w == 1 && g.pad_w == 1 && g.k_w == 3 &&
         g.in_w == g.out_w && !path_disabled(kNoRows);
}

template <int SH, int SW>
int channels_per_block(int cpg, int wanted_splits) {
  const int fit = kMaxLdsTables / (WideTable<SH, SW>::SIZE * 4) - std::max(2, kRowStages) * kUnroll;
  int per = ceil_div(cpg, wanted_splits);
  if (per > fit) per = fit;
  if (per < 1) per = 1;
  return per;
}

// How many channel splits give the forward / grad-input grid enough waves to fill 256 CUs.  A plane of up to
// 62 pixels is one wave per workgroup (row_block), so it takes four times the splits of a four-wave plane.
int pick_splits(const Geo& g, int planes_pixels) {
  const int waves_per_block = std::min(kBlock / 64, ceil_div(planes_pixels, 62));
  const long waves = (long)ceil_div(planes_pixels, kBlock) * waves_per_block * g.batch * g.groups;
  const int cpg = g.channel / g.groups;
  const int least = waves_per_block == 1 ? 8 : 16;  // channels per split
  int splits = 1;
  while (waves * splits < 8192 && cpg / (splits * 2) >= least) splits *= 2;
  return splits;
}

// stride 2 x 2, 3 x 3 undilated taps, padding 1, even input width: the pair-load kernels apply
bool stride2_geometry(const Geo& g) {
  return g.stride_h == 2 && g.stride_w == 2 && g.dil_h == 1 && g.dil_w == 1 && g.pad_h == 1 && g.pad_w == 1 &&
         g.k_h == 3 && g.k_w == 3 && g.in_w % 2 == 0 && !path_disabled(kNoRows);
}
int rotation_tile(const Geo& g) { return same_width_geometry(g) ? kRowPix : stride2_geometry(g) ? kS2Pix : kBlock; }

// Threads of a workgroup of the row kernels: whole waves, no more than the plane needs (a 7 x 7
// plane fits the 62 pixels of one wave; three more waves would only walk the channels idle).
unsigned row_block(int pixels, int lanes_per_wave) {
  return 64u * (unsigned)std::min(kBlock / 64, ceil_div(pixels, lanes_per_wave));
}

template <typename T, int SH, int SW>
bool run_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                hipStream_t stream) {
  const int cpg = g.channel / g.groups;
  const int pixels = transposed ? g.in_h * g.in_w : g.out_h * g.out_w;
  if (same_width_geometry(g)) {
    const int per = channels_per_block<SH, SW>(cpg, pick_splits(g, pixels));
    const unsigned grid = (unsigned)xcd_grid_size((long)ceil_div(pixels, kRowPix) * ceil_div(cpg, per) * g.batch * g.groups);
    const size_t lds = (size_t)(per + kRowStages * kUnroll) * WideTable<SH, SW>::SIZE * sizeof(float);
    if (transposed)
      local_gather_rows_kernel<T, 3, SH, SW, true><<<grid, row_block(pixels, kRowLanes), lds, stream>>>(g, src, rot, filter, dst, per);
    else
      local_gather_rows_kernel<T, 3, SH, SW, false><<<grid, row_block(pixels, kRowLanes), lds, stream>>>(g, src, rot, filter, dst, per);
    return true;
  }
  if (transposed && stride2_geometry(g) && !path_disabled(kNoS2Quads)) {
    // lanes own 2 x 2 input quads, one per output pixel
    const int quads = g.out_h * g.out_w;
    const int perq = channels_per_block<SH, SW>(cpg, pick_splits(g, quads));
    const unsigned gridq = (unsigned)xcd_grid_size((long)ceil_div(quads, kS2Pix) * ceil_div(cpg, perq) * g.batch * g.groups);
    const size_t ldsq = (size_t)(perq + 2 * kUnroll) * WideTable<SH, SW>::SIZE * sizeof(float);
    local_grad_input_s2_kernel<T, SH, SW><<<gridq, row_block(quads, kS2Lanes), ldsq, stream>>>(g, src, rot, filter, dst, perq);
    return true;
  }
  const int per = channels_per_block<SH, SW>(cpg, pick_splits(g, pixels));
  if (!transposed && stride2_geometry(g)) {
    const unsigned grid2 = (unsigned)xcd_grid_size((long)ceil_div(pixels, kS2Pix) * ceil_div(cpg, per) * g.batch * g.groups);
    const size_t lds2 = (size_t)(per + 2 * kUnroll) * WideTable<SH, SW>::SIZE * sizeof(float);
    local_forward_s2_kernel<T, SH, SW><<<grid2, row_block(pixels, kS2Lanes), lds2, stream>>>(g, src, rot, filter, dst, per);
    return true;
  }
  const unsigned grid = (unsigned)xcd_grid_size((long)ceil_div(pixels, kBlock) * ceil_div(cpg, per) * g.batch * g.groups);
  // stages past the last channel still read (and discard) table entries: pad to whole stages
  const size_t lds = (size_t)(per + 2 * kUnroll) * WideTable<SH, SW>::SIZE * sizeof(float);
  if (transposed && g.stride_h == 2 && g.stride_w == 2 && g.dil_h == 1 && g.dil_w == 1)
    local_gather_kernel<T, 3, 3, SH, SW, true, 4><<<grid, kBlock, lds, stream>>>(g, src, rot, filter, dst, per);
  else if (transposed)
    local_gather_kernel<T, 3, 3, SH, SW, true, 9><<<grid, kBlock, lds, stream>>>(g, src, rot, filter, dst, per);
  else
    local_gather_kernel<T, 3, 3, SH, SW, false, 9><<<grid, kBlock, lds, stream>>>(g, src, rot, filter, dst, per);
  return true;
}

// Channel splits of the grad-rotation grid: enough for about four blocks per CU with at least
// 16 channels per split.  (One-wave blocks -- planes of up to 62 pixels -- were tried with four times
// the splits: N=128 C=960 7 x 7 59 -> 66 us, the partial sums cost more than the fuller grid gains.)
int rotation_splits(const Geo& g) {
  const int cpg = g.channel / g.groups;
  const long base = std::max(1L, (long)ceil_div(g.out_h * g.out_w, rotation_tile(g)) * g.batch * g.groups);  // batch may be 0
  const long want = 1024 / base;  // measured: about four blocks per CU is the best grid
  return (int)std::max<long>(1, std::min<long>(want, cpg / 16));
}

template <typename T, int SH, int SW>
bool run_grad_rotation(const Geo& g, const T* gout, const T* x, const T* rot, const T* filter,
                       T* grot, float* ws, hipStream_t stream) {
  using Tb = WideTable<SH, SW>;
  const int cpg = g.channel / g.groups;
  const int splits = rotation_splits(g);
  // channels staged per pass; their planes stay within the 2 GiB a scalar byte offset reaches
  const long step_bytes = (long)g.groups * std::max(g.in_h * g.in_w, g.out_h * g.out_w) * (long)sizeof(T);
  const int per = (int)std::max(1L, std::min<long>(std::min(ceil_div(cpg, splits), 36), ((1L << 31) - 1) / step_bytes));
  const size_t lds = (size_t)per * Tb::SIZE * sizeof(float);
  const unsigned grid = (unsigned)xcd_grid_size((long)ceil_div(g.out_h * g.out_w, rotation_tile(g)) * splits * g.batch * g.groups);
  if (same_width_geometry(g)) {
    // Channel pairs on bfloat16 dot products, for bfloat16 tensors: the products' and the table's rounding
    // (2^-9 each) comes to about what the result's own rounding to bfloat16 is, 6.5e-3 of the largest
    // element at worst over random shapes against 4e-3 without.  float16 tensors would lose three of
    // their eleven bits (5e-4 -> 6e-3) and keep the fp32 multiply-adds.
    constexpr bool k16 = std::is_same<T, bf16_t>::value;
    const unsigned block = row_block(g.out_h * g.out_w, kRowLanes);
    if (k16 && cpg >= 16) {
      if (grid > 5 * 256)
        local_grad_rotation_kernel<T, 3, 3, SH, SW, 1, 5, k16><<<grid, block, lds, stream>>>(g, gout, x, rot, filter, grot, ws, splits, per);
      else
        local_grad_rotation_kernel<T, 3, 3, SH, SW, 1, 2, k16><<<grid, block, lds, stream>>>(g, gout, x, rot, filter, grot, ws, splits, per);
    } else if (grid > 5 * 256) {
      local_grad_rotation_kernel<T, 3, 3, SH, SW, 1, 5><<<grid, block, lds, stream>>>(g, gout, x, rot, filter, grot, ws, splits, per);
    } else {
      local_grad_rotation_kernel<T, 3, 3, SH, SW, 1><<<grid, block, lds, stream>>>(g, gout, x, rot, filter, grot, ws, splits, per);
    }
  } else if (stride2_geometry(g))
    local_grad_rotation_kernel<T, 3, 3, SH, SW, 2><<<grid, row_block(g.out_h * g.out_w, kS2Lanes), lds, stream>>>(g, gout, x, rot, filter, grot, ws, splits, per);
  else
    local_grad_rotation_kernel<T, 3, 3, SH, SW, 0><<<grid, kBlock, lds, stream>>>(g, gout, x, rot, filter, grot, ws, splits, per);
  if (splits > 1)
    launch_reduce_partials<float, T>(ws, splits, (long)g.batch * g.groups * 18 * g.out_h * g.out_w, grot, stream);
  return true;
}

// grad-filter launch shape: channel splits of at most kFilterChPerBlock channels, and enough
// (image, tile) parts that the grid has a few workgroups per CU.
constexpr int kFilterChPerBlock = 36;

struct FilterGrid {
  int per, splits, parts, tiles;
  bool mfma;       // matrix-core kernel: 16 channels per workgroup, 256-pixel tiles
  int pitch_x;     // its floats per channel of the staged input tile
  int nx;          // its staged input elements per lane and channel (4 or 6; 9 for stride 2)
  int th;          // stride 2: output rows per tile
  size_t lds;      // its LDS bytes
};

FilterGrid filter_grid(const Geo& g) {
  FilterGrid f;
  const int cpg = g.channel / g.groups;
  f.mfma = false;
  f.pitch_x = 0;
  f.nx = 0;
  f.th = 0;
  f.lds = 0;
  if (same_width_geometry(g) && !path_disabled(kNoMfma)) {
    const long xt = kMfPix + 2 + 2L * g.dil_h * g.in_w;
    // a row holds 64 * nx staged elements (nx = 4 or 6 per lane) plus the skew of mf_row() (at most 51)
    const long pitch = (xt <= 256 ? 256 : 64 * kMfX) + 64;
    const int nblk = ceil_div(cpg, kMfCh);
    const int csplits = ceil_div(nblk, kMfMaxBlk);
    const long lds = ((long)kMfCh * pitch + (long)kMfCh * kMfPitchG) * 4 + 9L * kMfPix * 8 +
                     (long)(kMfBlock / 64) * 256 * 4 + (long)ceil_div(nblk, csplits) * 256 * 4;
    if (lds <= 64 * 1024 && xt <= 64 * kMfX) {
      f.mfma = true;
      f.pitch_x = (int)pitch;
      f.nx = xt <= 256 ? 4 : kMfX;
      f.lds = (size_t)lds;
      f.per = kMfCh;
      f.splits = csplits;
      f.tiles = ceil_div(g.out_h * g.out_w, kMfPix);
      // two workgroups of 8 waves fit a CU: launch at most that many, all resident at once,
      // each walking an equal share of the (tile, channel block) units
      const long units = (long)g.batch * f.tiles * ceil_div(nblk, csplits);
      const long slots = std::max(1, 2 * 256 / (csplits * g.groups));
      f.parts = (int)std::max(1L, std::min(units, slots));
      return f;
    }
  }
  if (stride2_geometry(g) && !path_disabled(kNoMfma) && !path_disabled(kNoMfmaS2) && g.out_w <= kMfPix) {
    // tiles of whole output rows whose input rows (2 th + 1 of them, plus one element) fit the stage
    int th = std::min(kMfPix / g.out_w, g.out_h);
    while (th > 1 && (2L * th + 1) * g.in_w + 1 > 64 * kMfXS2) --th;
    const long xt = (2L * th + 1) * g.in_w + 1;
    const long pitch = 64 * kMfXS2 + 64;
    const int nblk = ceil_div(cpg, kMfCh);
    const int csplits = ceil_div(nblk, kMfMaxBlkS2);
    const long lds = ((long)kMfCh * pitch + (long)kMfCh * kMfPitchG) * 4 + 9L * kMfPix * 8 +
                     (long)(kMfBlock / 64) * 256 * 4 + (long)ceil_div(nblk, csplits) * 256 * 4;
    const int tiles = ceil_div(g.out_h, th);
    const bool countable = (long)g.batch * tiles * ceil_div(nblk, csplits) < (1L << 30);
    if (xt <= 64 * kMfXS2 && lds <= 80 * 1024 && countable) {
      f.mfma = true;
      f.pitch_x = (int)pitch;
      f.nx = kMfXS2;
      f.th = th;
      f.lds = (size_t)lds;
      f.per = kMfCh;
      f.splits = csplits;
      f.tiles = tiles;
      const long units = (long)g.batch * f.tiles * ceil_div(nblk, csplits);
      const long slots = std::max(1, 2 * 256 / (csplits * g.groups));
      f.parts = (int)std::max(1L, std::min(units, slots));
      return f;
    }
  }
  f.splits = ceil_div(cpg, kFilterChPerBlock);
  f.per = ceil_div(cpg, f.splits);
  f.tiles = ceil_div(g.out_h * g.out_w, rotation_tile(g));
  const int items = g.batch * f.tiles;
  // one (image, tile) item per workgroup while that keeps the partial buffer small; many more
  // workgroups than the GPU holds at once, so the dispatcher evens out the load
  f.parts = items < 1024 ? items : 1024;
  if (f.parts < 1) f.parts = 1;
  return f;
}

// CL: channels-last tensors, matrix-core kernel at stride 1 only (false otherwise)
template <typename T, int SH, int SW, bool CL = false>
bool run_grad_filter(const Geo& g, const T* gout, const T* x, const T* rot, T* gfilter, float* ws,
                     hipStream_t stream) {
  {
    const FilterGrid f = filter_grid(g);
    const unsigned grid = (unsigned)xcd_grid_size((long)f.parts * f.splits * g.groups);
    if (f.mfma) {
#define DK_LAUNCH_BF(CELL0, BF, SP)                                                                                 \
  if (f.th > 0) {                                                                                                \
    if constexpr (CL) return false;                                                                              \
    else {                                                                                                       \
    auto kernel = local_grad_filter_mfma_kernel<T, SH, SW, CELL0, kMfXS2, true, BF, SP>;                                                           \
    if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel)))                                                           \
      return false;                                                                                              \
    kernel<<<grid, kMfBlock, f.lds, stream>>>(g, gout, x, rot, ws, f.tiles, f.parts, f.splits, f.pitch_x, f.th); \
    }                                                                                                            \
  } else if (f.nx == 4)                                                                                          \
    local_grad_filter_mfma_kernel<T, SH, SW, CELL0, 4, false, BF, SP, CL><<<grid, kMfBlock, f.lds, stream>>>(g, gout, x, rot, ws, f.tiles, f.parts, f.splits, f.pitch_x, 0); \
  else                                                                                                           \
    local_grad_filter_mfma_kernel<T, SH, SW, CELL0, kMfX, false, BF, SP, CL><<<grid, kMfBlock, f.lds, stream>>>(g, gout, x, rot, ws, f.tiles, f.parts, f.splits, f.pitch_x, 0);
      // 16-bit inputs with at least one full block of 16 channels per group: bfloat16 matrix instructions
      // float32 inputs: bfloat16 pairs (three products) unless switched off, at stride 2 as well (N=64: 96 x 112^2
      // 98 -> 90 us, 144 x 56^2 46 -> 41, 192 x 28^2 25.9 -> 24.3, 576 x 14^2 32.8 -> 30.1)
      const bool split = !path_disabled(kNoFilterSplit);
#define DK_LAUNCH(CELL0)                                                    \
  if constexpr (sizeof(T) == 2) {                                           \
    if (g.channel / g.groups >= kMfCh) { DK_LAUNCH_BF(CELL0, true, false) } \
    else { DK_LAUNCH_BF(CELL0, false, false) }                              \
  } else if (split) { DK_LAUNCH_BF(CELL0, false, true) }                    \
  else { DK_LAUNCH_BF(CELL0, false, false) }
      DK_LAUNCH(0)
      // the further 16-cell slices of a larger scope, into the same partials
      if constexpr (SH * SW > 16) DK_LAUNCH(16)
      if constexpr (SH * SW > 32) DK_LAUNCH(32)
      if constexpr (SH * SW > 48) DK_LAUNCH(48)
#undef DK_LAUNCH
#undef DK_LAUNCH_BF
      launch_reduce_partials<float, T>(ws, f.parts, g.channel * SH * SW, gfilter, stream);
      return true;
    }
    if constexpr (CL || SH * SW > 32) {
      return false;  // the dense kernel's fold holds two cells per lane: a 7 x 7 scope goes to the generic kernel
    } else {
    const size_t lds = ((size_t)(kBlock / 64) * f.per * filter_slots(SH * SW) +
                        (size_t)(kBlock / 64) * 64 * filter_pitch(SH * SW)) * sizeof(float);
    if (same_width_geometry(g))
      local_grad_filter_kernel<T, 3, 3, SH, SW, 1><<<grid, row_block(g.out_h * g.out_w, kRowLanes), lds, stream>>>(g, gout, x, rot, ws, f.tiles, f.per, f.parts);
    else if (stride2_geometry(g))
      local_grad_filter_kernel<T, 3, 3, SH, SW, 2><<<grid, row_block(g.out_h * g.out_w, kS2Lanes), lds, stream>>>(g, gout, x, rot, ws, f.tiles, f.per, f.parts);
    else
      local_grad_filter_kernel<T, 3, 3, SH, SW, 0><<<grid, kBlock, lds, stream>>>(g, gout, x, rot, ws, f.tiles, f.per, f.parts);
    launch_reduce_partials<float, T>(ws, f.parts, g.channel * SH * SW, gfilter, stream);
    return true;
    }
  }
}

bool fast_shape(const Geo& g) {
  const long plane_limit = (1L << 31) / 4 / 32;  // byte offsets inside a plane (x 18 for rotation) stay below 2^31
  // every grid is 1-D with at most tiles * channels * batch blocks, indexed in 32 bits
  const long max_plane = std::max((long)g.in_h * g.in_w, (long)g.out_h * g.out_w);
  const long max_blocks = ((max_plane + kRowPix - 1) / kRowPix) * g.channel * g.batch;
  return g.k_h == 3 && g.k_w == 3 && max_blocks < (1L << 31) - 8 &&
         (long)g.in_h * g.in_w < plane_limit && (long)g.out_h * g.out_w < plane_limit &&
         ((g.scope_h == 4 && g.scope_w == 4) || (g.scope_h == 3 && g.scope_w == 3) ||
          (g.scope_h == 5 && g.scope_w == 5) || (g.scope_h == 7 && g.scope_w == 7));
}

}  // namespace

#define DK_DISPATCH_SCOPE(g, CALL)                                   \
  if ((g).scope_h == 4) return CALL(4, 4);                           \
  if ((g).scope_h == 3) return CALL(3, 3);                           \
  if ((g).scope_h == 5) return CALL(5, 5);                           \
  return CALL(7, 7);

template <typename T>
bool fast_local_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter,
                       T* dst, hipStream_t stream) {
  if (!fast_shape(g)) return false;
  if (lanes_local_gather<T>(g, transposed, src, rot, filter, dst, stream)) return true;
  if (mfma_local_gather<T>(g, transposed, src, rot, filter, dst, stream)) return true;
#define CALL(SH, SW) run_gather<T, SH, SW>(g, transposed, src, rot, filter, dst, stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

template <typename T>
bool fast_local_grad_rotation(const Geo& g, const T* gout, const T* x, const T* rot,
                              const T* filter, T* grot, void* ws, hipStream_t stream) {
  if (!fast_shape(g)) return false;
#define CALL(SH, SW) run_grad_rotation<T, SH, SW>(g, gout, x, rot, filter, grot, static_cast<float*>(ws), stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

size_t fast_local_grad_rotation_workspace(const Geo& g) {
  if (!fast_shape(g)) return 0;
  const int splits = rotation_splits(g);
  return splits > 1 ? (size_t)splits * g.batch * g.groups * 18 * g.out_h * g.out_w * sizeof(float) : 0;
}

size_t fast_local_grad_filter_workspace(const Geo& g) {
  if (!fast_shape(g)) return 0;
  const FilterGrid f = filter_grid(g);
  // more than 32 cells outside the matrix-core kernel's geometry: run_grad_filter() declines, and
  // the caller sizes the workspace for the generic kernel
  if (!f.mfma && g.scope_h * g.scope_w > 32) return 0;
  return (size_t)f.parts * g.channel * g.scope_h * g.scope_w * sizeof(float);
}

template <typename T>
bool fast_local_grad_filter(const Geo& g, const T* gout, const T* x, const T* rot, T* gfilter,
                            void* ws, hipStream_t stream) {
  if (!fast_shape(g)) return false;
#define CALL(SH, SW) run_grad_filter<T, SH, SW>(g, gout, x, rot, gfilter, static_cast<float*>(ws), stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

// Channels-last tensors on the matrix-core grad filter (its staging reads four consecutive channels per
// thread): one group, a multiple of 4 channels, stride-1 same-width geometry, 16-byte (16-bit types: 8-byte)
// aligned tensors, an image's tensor within 2 GB.
bool fast_local_grad_filter_cl_shape(const Geo& g, size_t elem) {
  if (!fast_shape(g) || g.groups != 1 || g.channel % 4 != 0 || path_disabled(kNoNhwcStaged)) return false;
  if ((long)std::max(g.in_h * g.in_w, g.out_h * g.out_w) * g.channel * (long)elem >= (1L << 31)) return false;
  const FilterGrid f = filter_grid(g);
  return f.mfma && f.th == 0;
}

size_t fast_local_grad_filter_cl_workspace(const Geo& g) {
  // (queried without the element size: the 4-byte bound covers the 2-byte types)
  if (!fast_local_grad_filter_cl_shape(g, 4)) return 0;
  return (size_t)filter_grid(g).parts * g.channel * g.scope_h * g.scope_w * sizeof(float);
}

template <typename T>
bool fast_local_grad_filter_cl(const Geo& g, const T* gout, const T* x, const T* rot, T* gfilter, void* ws,
                               hipStream_t stream) {
  if (!fast_local_grad_filter_cl_shape(g, 4)) return false;
  if (reinterpret_cast<uintptr_t>(gout) % (4 * sizeof(T)) != 0 || reinterpret_cast<uintptr_t>(x) % (4 * sizeof(T)) != 0)
    return false;
#define CALL(SH, SW) run_grad_filter<T, SH, SW, true>(g, gout, x, rot, gfilter, static_cast<float*>(ws), stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

#define DK_INSTANTIATE(T)                                                                           \
  template bool fast_local_grad_filter_cl<T>(const Geo&, const T*, const T*, const T*, T*, void*,   \
                                             hipStream_t);                                          \
  template bool fast_local_gather<T>(const Geo&, bool, const T*, const T*, const T*, T*, hipStream_t); \
  template bool fast_local_grad_rotation<T>(const Geo&, const T*, const T*, const T*, const T*, T*, void*,  \
                                            hipStream_t);                                           \
  template bool fast_local_grad_filter<T>(const Geo&, const T*, const T*, const T*, T*, void*,      \
                                          hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
#undef DK_INSTANTIATE

}  // namespace dk
