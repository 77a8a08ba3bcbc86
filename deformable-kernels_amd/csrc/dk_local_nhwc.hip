// Local deformable kernel on channels-last tensors: input [N][H][W][C], rotation
// [N][Ho][Wo][G * k * k * 2], output [N][Ho][Wo][C] in memory (the logical shapes and the channel
// order of the rotation tensor are those of the planar operator, K.cu:270-386 forward, K.cu:577-669
// grad input, K.cu:836-955 grad rotation, K.cu:1285-1370 grad filter); the filter stays [C][S_h][S_w].
// A network whose 1 x 1 convolutions run channels-last can then call the operator without a
// layout change on either side.
//
// With the channels innermost, everything that depends on (pixel, rotation group, tap) only -- the
// scope coordinate, its four cells and bilinear weights, the source pixel -- is wave-uniform work:
// a workgroup computes it once into a table in LDS (one thread per entry), and the channel work
// runs with lanes over channels, every global access a contiguous run.
//   forward / grad input : table entry = 4 cells + 4 weights + source pixel; the channel chunk's
//                          filter sits in LDS as [cell][channel]; a lane handles 1 or 4 channels.
//   grad rotation        : one wave per (pixel, group, tap), lanes over the group's channels,
//                          two wave sums.
//   grad filter          : a thread owns a channel and keeps its S_h * S_w sums in registers (scope
//                          up to 5 x 5; other scopes: a column of LDS); the table holds the
//                          dense row of hat products of each (pixel, tap); per-workgroup partial sums
//                          are added in a fixed order by reduce_partials.
#include "dk_kernels.h"

namespace dk {
namespace {

constexpr int kNBlock = 256;

template <typename CT>
struct NhwcTap {
  int cell[4];  // scope cells of the four corners (clamped into the scope)
  CT w[4];      // their weights; 0 for a corner outside the scope or a tap that contributes nothing
  long src;     // element offset of the sampled pixel's channel 0 in the source tensor; < 0: no contribution
};

// Scope part of a table entry: cells and bilinear weights of the coordinate (sh, sw), as
// planar_bilinear reads them (K.cu:51-83).
template <typename CT>
__device__ __forceinline__ void scope_corners(const Geo& g, CT sh, CT sw, int (&cell)[4], CT (&w)[4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) cell[i] = 0, w[i] = CT(0);
  if (!(sh > CT(-1) && sw > CT(-1) && sh < CT(g.scope_h) && sw < CT(g.scope_w))) return;
  const CT hf = floor(sh), wf = floor(sw);
  const int hl = (int)hf, wl = (int)wf, hi = hl + 1, wi = wl + 1;
  const CT lh = sh - hf, lw = sw - wf, hh = CT(1) - lh, hw = CT(1) - lw;
  const bool h0 = hl >= 0, h1 = hi <= g.scope_h - 1, w0 = wl >= 0, w1 = wi <= g.scope_w - 1;
  if (h0 && w0) cell[0] = hl * g.scope_w + wl, w[0] = hh * hw;
  if (h0 && w1) cell[1] = hl * g.scope_w + wi, w[1] = hh * lw;
  if (h1 && w0) cell[2] = hi * g.scope_w + wl, w[2] = lh * hw;
  if (h1 && w1) cell[3] = hi * g.scope_w + wi, w[3] = lh * lw;
}

// Rotation element (image b, output pixel opix, group grp, tap t, direction dir) of the channels-last tensor.
__device__ __forceinline__ size_t rot_index_nhwc(const Geo& g, int b, int opix, int grp, int t, int dir) {
  const int taps = g.k_h * g.k_w;
  return ((size_t)b * g.out_h * g.out_w + opix) * ((size_t)g.groups * taps * 2) + (size_t)(grp * taps + t) * 2 + dir;
}

// The output pixel and validity of tap t for destination pixel `pix`:
// forward: destination = output pixel, source = the input pixel the tap reads;
// transposed: destination = input pixel, source = the output pixel whose tap t reads it.
template <bool TRANSPOSED>
__device__ __forceinline__ bool tap_pixels(const Geo& g, int pix, int t, int& opix, long& src_pix) {
  const int f_h = t / g.k_w, f_w = t % g.k_w;
  if (!TRANSPOSED) {
    const int oh = pix / g.out_w, ow = pix % g.out_w;
    const int ih = oh * g.stride_h - g.pad_h + f_h * g.dil_h, iw = ow * g.stride_w - g.pad_w + f_w * g.dil_w;
    opix = pix;
    src_pix = (long)ih * g.in_w + iw;
    return ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
  } else {
    const int h = pix / g.in_w, w = pix % g.in_w;
    const int hh = h + g.pad_h - f_h * g.dil_h, ww = w + g.pad_w - f_w * g.dil_w;
    if (hh < 0 || ww < 0 || hh % g.stride_h != 0 || ww % g.stride_w != 0) return false;
    const int oh = hh / g.stride_h, ow = ww / g.stride_w;
    if (oh >= g.out_h || ow >= g.out_w) return false;
    opix = oh * g.out_w + ow;
    src_pix = opix;
    return true;
  }
}

template <typename T, typename CT, bool TRANSPOSED>
__device__ __forceinline__ NhwcTap<CT> make_tap(const Geo& g, const T* __restrict__ rot, int b, int pix, int grp, int t) {
  NhwcTap<CT> e;
  int opix = 0;
  long src_pix = 0;
  const bool hit = tap_pixels<TRANSPOSED>(g, pix, t, opix, src_pix);
#pragma unroll
  for (int i = 0; i < 4; ++i) e.cell[i] = 0, e.w[i] = CT(0);
  e.src = -1;
  if (hit) {
    const size_t ri = rot_index_nhwc(g, b, opix, grp, t, 0);
    const CT sh = scope_coord<CT>(g, t / g.k_w, (CT)ld(rot + ri), g.centre_h);
    const CT sw = scope_coord<CT>(g, t % g.k_w, (CT)ld(rot + ri + 1), g.centre_w);
    scope_corners<CT>(g, sh, sw, e.cell, e.w);
    const long plane = TRANSPOSED ? (long)g.out_h * g.out_w : (long)g.in_h * g.in_w;
    e.src = ((long)b * plane + src_pix) * g.channel;
  }
  return e;
}

struct NhwcLaunch {
  int dst_pixels;  // pixels of a destination plane
  int pb;          // destination pixels per workgroup
  int cc;          // channels per chunk (blockIdx.y)
  int pblocks;     // workgroups per image
};

// forward (TRANSPOSED = false) and grad input (true); VEC channels per lane (4 needs one rotation
// group, channels a multiple of 4 and 16-byte aligned tensors)
template <typename T, int VEC, bool TRANSPOSED>
__global__ __launch_bounds__(kNBlock) void nhwc_gather_kernel(Geo g, NhwcLaunch L, const T* __restrict__ src,
                                                              const T* __restrict__ rot,
                                                              const T* __restrict__ filter, T* __restrict__ dst) {
  using CT = compute_t<T>;
  extern __shared__ __align__(16) unsigned char nhwc_lds[];
  const int cells = g.scope_h * g.scope_w, taps = g.k_h * g.k_w;
  CT* wt = reinterpret_cast<CT*>(nhwc_lds);  // [cells][cc]
  NhwcTap<CT>* table =
      reinterpret_cast<NhwcTap<CT>*>(nhwc_lds + (((size_t)cells * L.cc * sizeof(CT) + 15) & ~(size_t)15));  // [pb][groups][taps]
  const int b = blockIdx.x / L.pblocks, p0 = (blockIdx.x % L.pblocks) * L.pb;
  const int c0 = blockIdx.y * L.cc;
  const int cc = min(L.cc, g.channel - c0);
  const int npix = min(L.pb, L.dst_pixels - p0);
  for (int i = threadIdx.x; i < cells * cc; i += kNBlock) {
    const int ch = i / cells, cell = i - ch * cells;
    wt[cell * L.cc + ch] = (CT)ld(filter + (size_t)(c0 + ch) * cells + cell);
  }
  const int entries = npix * g.groups * taps;
  for (int i = threadIdx.x; i < entries; i += kNBlock) {
    const int t = i % taps, grp = i / taps % g.groups, pl = i / taps / g.groups;
    table[i] = make_tap<T, CT, TRANSPOSED>(g, rot, b, p0 + pl, grp, t);
  }
  __syncthreads();
  const int ccv = (cc + VEC - 1) / VEC;
  for (int i = threadIdx.x; i < npix * ccv; i += kNBlock) {
    const int pl = i / ccv, cl = (i - pl * ccv) * VEC;
    const int c = c0 + cl;
    CT acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = CT(0);
    const NhwcTap<CT>* row = table + (size_t)(pl * g.groups + (VEC == 1 ? c % g.groups : 0)) * taps;
    for (int t = 0; t < taps; ++t) {
      const NhwcTap<CT> e = row[t];
      if (e.src < 0) continue;
      CT xv[VEC];
      if constexpr (VEC == 4) {
        struct alignas(sizeof(T) * 4) Pack { T v[4]; };
        const Pack pk = *reinterpret_cast<const Pack*>(src + e.src + c);
#pragma unroll
        for (int v = 0; v < 4; ++v) xv[v] = (CT)ld(pk.v + v);
      } else {
        xv[0] = (CT)ld(src + e.src + c);
      }
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        CT wv = CT(0);
#pragma unroll
        for (int k = 0; k < 4; ++k) wv += e.w[k] * wt[e.cell[k] * L.cc + cl + v];
        acc[v] += xv[v] * wv;
      }
    }
    T* out = dst + ((size_t)b * L.dst_pixels + p0 + pl) * g.channel + c;
    if constexpr (VEC == 4) {
      struct alignas(sizeof(T) * 4) Pack { T v[4]; } pk;
#pragma unroll
      for (int v = 0; v < 4; ++v) st(pk.v + v, acc[v]);
      *reinterpret_cast<Pack*>(out) = pk;
    } else {
      st(out, acc[0]);
    }
  }
}

__device__ __forceinline__ float group_sum(float v) { return wave_sum(v); }
__device__ __forceinline__ double group_sum(double v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

// grad rotation: grot[pixel][(grp, t, dir)] = sum over the group's channels of
// out_grad * input(tap) * d/d(dir) of the bilinear scope read (planar_bilinear_backward_coord, K.cu:116-163)
template <typename T>
__global__ __launch_bounds__(kNBlock) void nhwc_grad_rotation_kernel(Geo g, const T* __restrict__ gout,
                                                                     const T* __restrict__ x,
                                                                     const T* __restrict__ rot,
                                                                     const T* __restrict__ filter,
                                                                     T* __restrict__ grot, int wt_in_lds) {
  using CT = compute_t<T>;
  extern __shared__ __align__(16) unsigned char nhwc_lds[];
  const int cells = g.scope_h * g.scope_w, taps = g.k_h * g.k_w;
  CT* wt = reinterpret_cast<CT*>(nhwc_lds);  // [cells][channel] when it fits
  if (wt_in_lds) {
    for (int i = threadIdx.x; i < cells * g.channel; i += kNBlock) {
      const int ch = i / cells, cell = i - ch * cells;
      wt[(size_t)cell * g.channel + ch] = (CT)ld(filter + i);
    }
    __syncthreads();
  }
  const int lane = threadIdx.x & 63;
  const int oplane = g.out_h * g.out_w;
  const long items = (long)g.batch * oplane * g.groups * taps;
  const long waves = (long)gridDim.x * (kNBlock / 64);
  const int cpg = g.channel / g.groups;
  for (long it = (long)blockIdx.x * (kNBlock / 64) + (threadIdx.x >> 6); it < items; it += waves) {
    const int t = (int)(it % taps), grp = (int)(it / taps % g.groups);
    const int pix = (int)(it / taps / g.groups % oplane), b = (int)(it / taps / g.groups / oplane);
    int opix;
    long src_pix;
    const bool hit = tap_pixels<false>(g, pix, t, opix, src_pix);
    const size_t ri = rot_index_nhwc(g, b, pix, grp, t, 0);
    CT gh = CT(0), gw = CT(0);
    bool open_h = true, open_w = true;
    const CT sh = scope_coord<CT>(g, t / g.k_w, (CT)ld(rot + ri), g.centre_h, &open_h);
    const CT sw = scope_coord<CT>(g, t % g.k_w, (CT)ld(rot + ri + 1), g.centre_w, &open_w);
    if (hit && sh > CT(-1) && sw > CT(-1) && sh < CT(g.scope_h) && sw < CT(g.scope_w)) {
      const CT hf = floor(sh), wf = floor(sw);
      const int hl = (int)hf, wl = (int)wf, hi = hl + 1, wi = wl + 1;
      const CT lh = sh - hf, lw = sw - wf, hh = CT(1) - lh, hw = CT(1) - lw;
      const bool c00 = hl >= 0 && wl >= 0, c01 = hl >= 0 && wi <= g.scope_w - 1;
      const bool c10 = hi <= g.scope_h - 1 && wl >= 0, c11 = hi <= g.scope_h - 1 && wi <= g.scope_w - 1;
      const int i00 = c00 ? hl * g.scope_w + wl : 0, i01 = c01 ? hl * g.scope_w + wi : 0;
      const int i10 = c10 ? hi * g.scope_w + wl : 0, i11 = c11 ? hi * g.scope_w + wi : 0;
      // d/dh and d/dw weights of the four corners
      const CT dh[4] = {c00 ? -hw : CT(0), c01 ? -lw : CT(0), c10 ? hw : CT(0), c11 ? lw : CT(0)};
      const CT dw[4] = {c00 ? -hh : CT(0), c01 ? hh : CT(0), c10 ? -lh : CT(0), c11 ? lh : CT(0)};
      const int ci[4] = {i00, i01, i10, i11};
      const T* gp = gout + ((size_t)b * oplane + pix) * g.channel;
      const T* xp = x + ((size_t)b * g.in_h * g.in_w + src_pix) * g.channel;
      for (int j = lane; j < cpg; j += 64) {
        const int c = grp + g.groups * j;
        const CT pv = (CT)ld(gp + c) * (CT)ld(xp + c);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const CT f = wt_in_lds ? wt[(size_t)ci[k] * g.channel + c] : (CT)ld(filter + (size_t)c * cells + ci[k]);
          gh += pv * dh[k] * f;
          gw += pv * dw[k] * f;
        }
      }
    }
    gh = group_sum(gh);
    gw = group_sum(gw);
    if (lane == 0) {
      st(grot + ri, open_h ? gh : CT(0));
      st(grot + ri + 1, open_w ? gw : CT(0));
    }
  }
}

// grad filter.  CELLS > 0: the scope's cell count, sums in registers; CELLS == 0: any scope, sums in
// the thread's own column of LDS.
template <typename T, int CELLS>
__global__ __launch_bounds__(kNBlock) void nhwc_grad_filter_kernel(Geo g, const T* __restrict__ gout,
                                                                   const T* __restrict__ x,
                                                                   const T* __restrict__ rot,
                                                                   compute_t<T>* __restrict__ partial, int pix_per_block,
                                                                   int pb) {
  using CT = compute_t<T>;
  extern __shared__ __align__(16) unsigned char nhwc_lds[];
  const int cells = g.scope_h * g.scope_w, taps = g.k_h * g.k_w;
  const int oplane = g.out_h * g.out_w;
  // table: per (pixel of the batch, group, tap) the dense row of hat products and the source offset
  long* srcs = reinterpret_cast<long*>(nhwc_lds);                                // [pb * groups * taps]
  CT* hats = reinterpret_cast<CT*>(srcs + (size_t)pb * g.groups * taps);         // [pb * groups * taps][cells]
  CT* col = hats + (size_t)pb * g.groups * taps * cells;                         // CELLS == 0: [cells][kNBlock]
  const int c = blockIdx.y * kNBlock + threadIdx.x;
  const bool live = c < g.channel;
  const int grp = live ? c % g.groups : 0;
  const long total_pix = (long)g.batch * oplane;
  const long q0 = (long)blockIdx.x * pix_per_block, q1 = min(total_pix, q0 + pix_per_block);
  CT acc[CELLS > 0 ? CELLS : 1];
#pragma unroll
  for (int k = 0; k < (CELLS > 0 ? CELLS : 1); ++k) acc[k] = CT(0);
  if constexpr (CELLS == 0)
    for (int k = 0; k < cells; ++k) col[k * kNBlock + threadIdx.x] = CT(0);
  for (long qb = q0; qb < q1; qb += pb) {
    const int npix = (int)min((long)pb, q1 - qb);
    __syncthreads();  // the previous batch's table has been read
    for (int i = threadIdx.x; i < npix * g.groups * taps; i += kNBlock) {
      const int t = i % taps, gi = i / taps % g.groups, pl = i / taps / g.groups;
      const long q = qb + pl;
      const NhwcTap<CT> e = make_tap<T, CT, false>(g, rot, (int)(q / oplane), (int)(q % oplane), gi, t);
      for (int k = 0; k < cells; ++k) hats[(size_t)i * cells + k] = CT(0);
      if (e.src >= 0)
#pragma unroll
        for (int k = 0; k < 4; ++k) hats[(size_t)i * cells + e.cell[k]] += e.w[k];  // absent corners add 0 to cell 0
      srcs[i] = e.src;
    }
    __syncthreads();
    if (live) {
      for (int pl = 0; pl < npix; ++pl) {
        const CT gv = (CT)ld(gout + (size_t)(qb + pl) * g.channel + c);
        const int base = (pl * g.groups + grp) * taps;
        for (int t = 0; t < taps; ++t) {
          const long s = srcs[base + t];
          if (s < 0) continue;
          const CT pv = gv * (CT)ld(x + s + c);
          const CT* h = hats + (size_t)(base + t) * cells;
          if constexpr (CELLS > 0) {
#pragma unroll
            for (int k = 0; k < CELLS; ++k) acc[k] += h[k] * pv;
          } else {
            for (int k = 0; k < cells; ++k) col[k * kNBlock + threadIdx.x] += h[k] * pv;
          }
        }
      }
    }
  }
  if (live) {
    CT* out = partial + ((size_t)blockIdx.x * g.channel + c) * cells;
    if constexpr (CELLS > 0) {
#pragma unroll
      for (int k = 0; k < CELLS; ++k) out[k] = acc[k];
    } else {
      for (int k = 0; k < cells; ++k) out[k] = col[k * kNBlock + threadIdx.x];
    }
  }
}

// ---- host side --------------------------------------------------------------------------

constexpr int kFilterPixPerBlock = 512;
constexpr int kFilterBatch = 16;  // pixels per table batch of the grad filter

template <typename T>
NhwcLaunch gather_launch(const Geo& g, bool transposed, size_t& lds) {
  using CT = compute_t<T>;
  NhwcLaunch L;
  const int cells = g.scope_h * g.scope_w, taps = g.k_h * g.k_w;
  L.dst_pixels = transposed ? g.in_h * g.in_w : g.out_h * g.out_w;
  L.cc = std::min(g.channel, std::max(4, std::min(256, (int)(32768 / sizeof(CT)) / cells) & ~3));
  L.pb = std::max(1, std::min(32, 512 / (g.groups * taps)));
  L.pblocks = ceil_div(L.dst_pixels, L.pb);
  lds = (((size_t)cells * L.cc * sizeof(CT) + 15) & ~(size_t)15) + (size_t)L.pb * g.groups * taps * sizeof(NhwcTap<CT>);
  return L;
}

template <typename T>
bool vec4_ok(const Geo& g, const void* a, const void* b) {
  return g.groups == 1 && g.channel % 4 == 0 && reinterpret_cast<uintptr_t>(a) % (4 * sizeof(T)) == 0 &&
         reinterpret_cast<uintptr_t>(b) % (4 * sizeof(T)) == 0;
}

}  // namespace

bool nhwc_supported(const Geo& g, int dtype) {
  const size_t ct = dtype == DK_F64 ? 8 : 4;
  const long cells = (long)g.scope_h * g.scope_w, taps = (long)g.k_h * g.k_w;
  if (cells > 1024 || taps * g.groups > 4096) return false;
  // forward / grad input: a chunk of at least 4 channels of the filter and one pixel's table
  if (cells * 4 * ct + (size_t)g.groups * taps * (32 + 4 * ct) > 60 * 1024) return false;
  // grad filter: one pixel's dense table (and a column of sums for scopes other than 3x3 / 4x4 / 5x5)
  const bool reg = cells == 9 || cells == 16 || cells == 25;
  if ((size_t)g.groups * taps * (cells * ct + 8) > 40 * 1024 || (reg ? 0 : cells * kNBlock * ct) > 100 * 1024) return false;
  return true;
}

template <typename T>
void nhwc_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                 hipStream_t stream) {
  size_t lds;
  const NhwcLaunch L = gather_launch<T>(g, transposed, lds);
  const dim3 grid((unsigned)(g.batch * L.pblocks), (unsigned)ceil_div(g.channel, L.cc));
  const bool v4 = vec4_ok<T>(g, src, dst) && L.cc % 4 == 0;
#define DK_NHWC_GATHER(VV, TT) \
  hipLaunchKernelGGL((nhwc_gather_kernel<T, VV, TT>), grid, dim3(kNBlock), lds, stream, g, L, src, rot, filter, dst)
  if (transposed) {
    if (v4) DK_NHWC_GATHER(4, true);
    else DK_NHWC_GATHER(1, true);
  } else {
    if (v4) DK_NHWC_GATHER(4, false);
    else DK_NHWC_GATHER(1, false);
  }
#undef DK_NHWC_GATHER
}

template <typename T>
void nhwc_grad_rotation(const Geo& g, const T* gout, const T* x, const T* rot, const T* filter, T* grot,
                        hipStream_t stream) {
  using CT = compute_t<T>;
  const size_t wt_bytes = (size_t)g.scope_h * g.scope_w * g.channel * sizeof(CT);
  const int in_lds = wt_bytes <= 48 * 1024;
  const long items = (long)g.batch * g.out_h * g.out_w * g.groups * g.k_h * g.k_w;
  const long blocks = std::min<long>((items + 3) / 4, 256L * 32);
  hipLaunchKernelGGL((nhwc_grad_rotation_kernel<T>), dim3((unsigned)blocks), dim3(kNBlock), in_lds ? wt_bytes : 0, stream,
                     g, gout, x, rot, filter, grot, in_lds);
}

size_t nhwc_grad_filter_workspace(const Geo& g, int dtype) {
  const long parts = ceil_div((long)g.batch * g.out_h * g.out_w, (long)kFilterPixPerBlock);
  return (size_t)parts * g.channel * g.scope_h * g.scope_w * (dtype == DK_F64 ? 8 : 4);
}

template <typename T>
void nhwc_grad_filter(const Geo& g, const T* gout, const T* x, const T* rot, T* gfilter, void* ws,
                      hipStream_t stream) {
  using CT = compute_t<T>;
  const int cells = g.scope_h * g.scope_w, taps = g.k_h * g.k_w;
  const long total_pix = (long)g.batch * g.out_h * g.out_w;
  const int parts = (int)ceil_div(total_pix, (long)kFilterPixPerBlock);
  const bool reg = cells == 9 || cells == 16 || cells == 25;
  const size_t per_pixel = (size_t)g.groups * taps * (cells * sizeof(CT) + sizeof(long));
  const size_t colb = reg ? 0 : (size_t)cells * kNBlock * sizeof(CT);
  const int pb = (int)std::max<size_t>(1, std::min<size_t>(kFilterBatch, 40 * 1024 / per_pixel));
  const size_t lds = pb * per_pixel + colb;  // at most 40 KB of table and 100 KB of sums
  CT* partial = static_cast<CT*>(ws);
  const dim3 grid((unsigned)parts, (unsigned)ceil_div(g.channel, kNBlock));
#define DK_NHWC_GF(CC)                                                                                                        \
  if (lds <= 64 * 1024 || allow_dynamic_lds(reinterpret_cast<const void*>(&nhwc_grad_filter_kernel<T, CC>), 144 * 1024))   \
  hipLaunchKernelGGL((nhwc_grad_filter_kernel<T, CC>), grid, dim3(kNBlock), lds, stream, g, gout, x, rot, partial, kFilterPixPerBlock, pb)
  if (cells == 9) { DK_NHWC_GF(9); }
  else if (cells == 16) { DK_NHWC_GF(16); }
  else if (cells == 25) { DK_NHWC_GF(25); }
  else { DK_NHWC_GF(0); }
#undef DK_NHWC_GF
  launch_reduce_partials<CT, T>(partial, parts, (long)g.channel * cells, gfilter, stream);
}

#define DK_INSTANTIATE(T)                                                                                  \
  template void nhwc_gather<T>(const Geo&, bool, const T*, const T*, const T*, T*, hipStream_t);           \
  template void nhwc_grad_rotation<T>(const Geo&, const T*, const T*, const T*, const T*, T*, hipStream_t); \
  template void nhwc_grad_filter<T>(const Geo&, const T*, const T*, const T*, T*, void*, hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
DK_INSTANTIATE(double)
#undef DK_INSTANTIATE

}  // namespace dk
