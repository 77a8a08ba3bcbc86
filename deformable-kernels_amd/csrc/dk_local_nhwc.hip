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
// Layers of one rotation group with 3 x 3 taps -- the shapes networks use -- take matrix-core kernels instead:
//   forward / grad input : nhwc_gather_mfma16_kernel (scopes of up to 16 cells): the effective weights of 16 channels
//                          x 16 pixels per matrix instruction, landing as the four consecutive channels a 16-byte
//                          load of the source pixel delivers;
//   grad rotation        : nhwc_grad_rotation_mfma16_kernel: out_grad * input of 32 channels from the loads'
//                          registers as the matrix operand, nine 16 x 16 accumulators per 16 pixels;
//   grad filter          : the planar operator's matrix-core kernel (dk_local_fast.hip) with a staging that
//                          reads four consecutive channels per thread (stride-1 layers);
// and, where those do not apply, nhwc_grad_filter_mfma_kernel / nhwc_grad_rotation_mfma_kernel on fp32
// matrix instructions with dense hat-product tables.
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

// cell_pitch: what a cell index is multiplied with in the entry (the gather kernels store the cell's
// offset in their [cell][channel chunk] copy of the filter, so that no lane multiplies)
template <typename T, typename CT, bool TRANSPOSED>
__device__ __forceinline__ NhwcTap<CT> make_tap(const Geo& g, const T* __restrict__ rot, int b, int pix, int grp, int t,
                                                int cell_pitch = 1) {
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
#pragma unroll
    for (int i = 0; i < 4; ++i) e.cell[i] *= cell_pitch;
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
// TAPS: the tap count when it is known at compile time (9: a lane's nine source loads are issued
// before the first is used), 0: any.
template <typename T, int VEC, bool TRANSPOSED, int TAPS>
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
    table[i] = make_tap<T, CT, TRANSPOSED>(g, rot, b, p0 + pl, grp, t, L.cc);
  }
  __syncthreads();
  const int ccv = (cc + VEC - 1) / VEC;
  const unsigned ccv_magic = 0xffffffffu / (unsigned)ccv + 1u;  // i / ccv for i < 2^16 (a workgroup has at most 32 * 256 items)
  for (int i = threadIdx.x; i < npix * ccv; i += kNBlock) {
    const int pl = (int)__umulhi((unsigned)i, ccv_magic), cl = (i - pl * ccv) * VEC;
    const int c = c0 + cl;
    CT acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = CT(0);
    const NhwcTap<CT>* row = table + (size_t)(pl * g.groups + (VEC == 1 ? c % g.groups : 0)) * taps;
    struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
    struct alignas(sizeof(CT) * VEC) WVec { CT v[VEC]; };
    if constexpr (TAPS > 0) {
      Pack pk[TAPS];
      bool on[TAPS];
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        const long so = row[t].src;
        on[t] = so >= 0;
        pk[t] = *reinterpret_cast<const Pack*>(src + (on[t] ? so : 0) + c);  // a dead tap reads element c of the tensor: valid, unused
      }
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        int cell[4];
        CT w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) cell[k] = row[t].cell[k], w[k] = row[t].w[k];
        // the lane's VEC channels of a cell in one LDS read (a read per channel has the lanes VEC banks apart)
        WVec f[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) f[k] = *reinterpret_cast<const WVec*>(wt + cell[k] + cl);
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          CT wv = CT(0);
#pragma unroll
          for (int k = 0; k < 4; ++k) wv += w[k] * f[k].v[v];
          const CT xv = on[t] ? (CT)ld(pk[t].v + v) : CT(0);
          acc[v] += xv * wv;
        }
      }
    } else {
      for (int t = 0; t < taps; ++t) {
        const NhwcTap<CT> e = row[t];
        if (e.src < 0) continue;
        const Pack pk = *reinterpret_cast<const Pack*>(src + e.src + c);
        WVec f[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) f[k] = *reinterpret_cast<const WVec*>(wt + e.cell[k] + cl);
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          CT wv = CT(0);
#pragma unroll
          for (int k = 0; k < 4; ++k) wv += e.w[k] * f[k].v[v];
          acc[v] += (CT)ld(pk.v + v) * wv;
        }
      }
    }
    T* out = dst + ((size_t)b * L.dst_pixels + p0 + pl) * g.channel + c;
    Pack res;
#pragma unroll
    for (int v = 0; v < VEC; ++v) st(res.v + v, acc[v]);
    if constexpr (sizeof(Pack) == 16) {
      __builtin_nontemporal_store(__builtin_bit_cast(nhwc_u4, res), reinterpret_cast<nhwc_u4*>(out));
    } else {
      *reinterpret_cast<Pack*>(out) = res;
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

// grad rotation for 3 x 3 taps with the filter in LDS: the derivative weights of each (pixel, group,
// tap) are computed once into a table (one thread per entry); a wave then takes a (pixel, group),
// walks the group's channels with lanes over channels -- out_grad and the nine tap inputs loaded
// first -- and keeps 18 running sums, added up over the wave at the end and written as one
// contiguous run of 18 values.
template <typename CT>
struct NhwcRotTap {
  int cell[4];
  CT dh[4], dw[4];
  long src;
  int open;  // bit 0 / 1: the h / w offset was not clamped (its gradient passes)
};

template <typename T>
__global__ __launch_bounds__(kNBlock) void nhwc_grad_rotation9_kernel(Geo g, const T* __restrict__ gout,
                                                                      const T* __restrict__ x,
                                                                      const T* __restrict__ rot,
                                                                      const T* __restrict__ filter,
                                                                      T* __restrict__ grot, int pb) {
  using CT = compute_t<T>;
  constexpr int TAPS = 9;
  extern __shared__ __align__(16) unsigned char nhwc_lds[];
  const int cells = g.scope_h * g.scope_w;
  CT* wt = reinterpret_cast<CT*>(nhwc_lds);  // [cells][channel]
  NhwcRotTap<CT>* table =
      reinterpret_cast<NhwcRotTap<CT>*>(nhwc_lds + (((size_t)cells * g.channel * sizeof(CT) + 15) & ~(size_t)15));
  const int oplane = g.out_h * g.out_w;
  const long total_pix = (long)g.batch * oplane;
  const long q0 = (long)blockIdx.x * pb;
  const int npix = (int)min((long)pb, total_pix - q0);
  for (int i = threadIdx.x; i < cells * g.channel; i += kNBlock) {
    const int ch = i / cells, cell = i - ch * cells;
    wt[(size_t)cell * g.channel + ch] = (CT)ld(filter + i);
  }
  for (int i = threadIdx.x; i < npix * g.groups * TAPS; i += kNBlock) {
    const int t = i % TAPS, grp = i / TAPS % g.groups, pl = i / TAPS / g.groups;
    const long q = q0 + pl;
    const int b = (int)(q / oplane), pix = (int)(q % oplane);
    NhwcRotTap<CT> e;
#pragma unroll
    for (int k = 0; k < 4; ++k) e.cell[k] = 0, e.dh[k] = CT(0), e.dw[k] = CT(0);
    e.src = -1;
    int opix;
    long src_pix;
    const bool hit = tap_pixels<false>(g, pix, t, opix, src_pix);
    const size_t ri = rot_index_nhwc(g, b, pix, grp, t, 0);
    bool open_h = true, open_w = true;
    const CT sh = scope_coord<CT>(g, t / 3, (CT)ld(rot + ri), g.centre_h, &open_h);
    const CT sw = scope_coord<CT>(g, t % 3, (CT)ld(rot + ri + 1), g.centre_w, &open_w);
    e.open = (open_h ? 1 : 0) | (open_w ? 2 : 0);
    if (hit && sh > CT(-1) && sw > CT(-1) && sh < CT(g.scope_h) && sw < CT(g.scope_w)) {
      const CT hf = floor(sh), wf = floor(sw);
      const int hl = (int)hf, wl = (int)wf, hi = hl + 1, wi = wl + 1;
      const CT lh = sh - hf, lw = sw - wf, hh = CT(1) - lh, hw = CT(1) - lw;
      const bool c00 = hl >= 0 && wl >= 0, c01 = hl >= 0 && wi <= g.scope_w - 1;
      const bool c10 = hi <= g.scope_h - 1 && wl >= 0, c11 = hi <= g.scope_h - 1 && wi <= g.scope_w - 1;
      e.cell[0] = c00 ? hl * g.scope_w + wl : 0, e.cell[1] = c01 ? hl * g.scope_w + wi : 0;
      e.cell[2] = c10 ? hi * g.scope_w + wl : 0, e.cell[3] = c11 ? hi * g.scope_w + wi : 0;
      e.dh[0] = c00 ? -hw : CT(0), e.dh[1] = c01 ? -lw : CT(0), e.dh[2] = c10 ? hw : CT(0), e.dh[3] = c11 ? lw : CT(0);
      e.dw[0] = c00 ? -hh : CT(0), e.dw[1] = c01 ? hh : CT(0), e.dw[2] = c10 ? -lh : CT(0), e.dw[3] = c11 ? lh : CT(0);
      e.src = ((long)b * g.in_h * g.in_w + src_pix) * g.channel;
    }
    table[i] = e;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int cpg = g.channel / g.groups;
  for (int item = wave; item < npix * g.groups; item += kNBlock / 64) {
    const int grp = item % g.groups, pl = item / g.groups;
    const long q = q0 + pl;
    const NhwcRotTap<CT>* row = table + (size_t)item * TAPS;
    CT ph[TAPS], pw[TAPS];
#pragma unroll
    for (int t = 0; t < TAPS; ++t) ph[t] = CT(0), pw[t] = CT(0);
    for (int j = lane; j < cpg; j += 64) {
      const int c = grp + g.groups * j;
      const T graw = gout[(size_t)q * g.channel + c];
      T xraw[TAPS];
      bool on[TAPS];
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        const long so = row[t].src;
        on[t] = so >= 0;
        xraw[t] = x[(on[t] ? so : 0) + c];
      }
      const CT gv = (CT)ld(&graw);
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        const CT pv = on[t] ? gv * (CT)ld(&xraw[t]) : CT(0);
        CT fh = CT(0), fw = CT(0);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const CT f = wt[(size_t)row[t].cell[k] * g.channel + c];
          fh += row[t].dh[k] * f;
          fw += row[t].dw[k] * f;
        }
        ph[t] += pv * fh;
        pw[t] += pv * fw;
      }
    }
    CT mine = CT(0);
#pragma unroll
    for (int t = 0; t < TAPS; ++t) {
      const CT sh_ = group_sum(ph[t]), sw_ = group_sum(pw[t]);
      const int open = row[t].open;
      mine = lane == 2 * t ? ((open & 1) ? sh_ : CT(0)) : mine;
      mine = lane == 2 * t + 1 ? ((open & 2) ? sw_ : CT(0)) : mine;
    }
    if (lane < 2 * TAPS)
      st(grot + rot_index_nhwc(g, (int)(q / oplane), (int)(q % oplane), grp, 0, 0) + lane, mine);
  }
}

// grad filter.  CELLS > 0: the scope's cell count, sums in registers; CELLS == 0: any scope, sums in
// the thread's own column of LDS.
template <typename T, int CELLS, int TAPS>
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
        const int base = (pl * g.groups + grp) * taps;
        if constexpr (TAPS > 0 && CELLS > 0) {
          // the pixel's ten loads first
          const T graw = gout[(size_t)(qb + pl) * g.channel + c];
          T xraw[TAPS];
          bool on[TAPS];
#pragma unroll
          for (int t = 0; t < TAPS; ++t) {
            const long so = srcs[base + t];
            on[t] = so >= 0;
            xraw[t] = x[(on[t] ? so : 0) + c];
          }
          const CT gv = (CT)ld(&graw);
#pragma unroll
          for (int t = 0; t < TAPS; ++t) {
            const CT pv = on[t] ? gv * (CT)ld(&xraw[t]) : CT(0);
            const CT* h = hats + (size_t)(base + t) * cells;
#pragma unroll
            for (int k = 0; k < CELLS; ++k) acc[k] += h[k] * pv;
          }
        } else {
          const CT gv = (CT)ld(gout + (size_t)(qb + pl) * g.channel + c);
          for (int t = 0; t < taps; ++t) {
            const long so = srcs[base + t];
            if (so < 0) continue;
            const CT pv = gv * (CT)ld(x + so + c);
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

// ---------------------------------------------------------------------------
// grad filter and grad rotation on the matrix cores (one rotation group, scopes of up to 32 cells,
// 16- and 32-bit types).  With k = (pixel, tap) and P[k][c] = out_grad[pixel][c] * input(tap)[c]:
//   grad filter    gW[cell][c]  = sum_k A[k][cell] * P[k][c]       A: the hat products of (pixel, tap)
//   grad rotation  R[k][cell]   = sum_c P[k][c] * W[c][cell]       then  grot[k][dir] = sum_cell dA_dir[k][cell] * R[k][cell]
// Channels-last is the natural layout for both: P's rows are contiguous over c.  Both use
// v_mfma_f32_16x16x4_f32 (fp32 products and sums): lane l supplies A[l % 16][l / 16] and
// B[l / 16][l % 16] and holds D[4 * (l / 16) + i][l % 16].  The tables of a batch of pixels (dense
// rows of A or dA over the cells, source offsets) are written by one thread per row.
// ---------------------------------------------------------------------------
typedef float nhwc_f4 __attribute__((ext_vector_type(4)));
constexpr int kMfRows = 144;  // table rows ((pixel, tap) pairs) per batch; a multiple of 16

struct NhwcRow {
  unsigned src;   // byte offset of the tap's input pixel (channel 0) in the input tensor
  unsigned gsrc;  // byte offset of the pixel's out_grad (channel 0)
  unsigned rix;   // element index of the row's h entry in the rotation tensor (the w entry follows)
  unsigned pad_;
};                // a row that contributes nothing has both at kOutOfRange: its buffer loads return zeros

// One element / four consecutive elements at a byte offset of a buffer resource, as stored (converted when used:
// a conversion next to the load would wait for it).
template <typename T> struct RawOf { using type = unsigned; };
template <> struct RawOf<__half> { using type = unsigned short; };
template <> struct RawOf<bf16_t> { using type = unsigned short; };
__device__ __forceinline__ unsigned raw_ld(rsrc_t r, unsigned off, const float*) { return __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0); }
__device__ __forceinline__ unsigned short raw_ld(rsrc_t r, unsigned off, const __half*) { return __builtin_amdgcn_raw_buffer_load_b16(r, (int)off, 0, 0); }
__device__ __forceinline__ unsigned short raw_ld(rsrc_t r, unsigned off, const bf16_t*) { return __builtin_amdgcn_raw_buffer_load_b16(r, (int)off, 0, 0); }
__device__ __forceinline__ float raw_cvt(unsigned v, const float*) { return __uint_as_float(v); }
__device__ __forceinline__ float raw_cvt(unsigned short v, const __half*) { return static_cast<float>(__builtin_bit_cast(_Float16, v)); }
__device__ __forceinline__ float raw_cvt(unsigned short v, const bf16_t*) { return __uint_as_float((unsigned)v << 16); }

// Sum over the 16 lanes of a DPP row, in every lane of the row.
__device__ __forceinline__ float row16_sum(float v) {
#define DK_DPP_ADD(ctrl) \
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true))
  DK_DPP_ADD(0xB1);   // quad_perm [1,0,3,2]
  DK_DPP_ADD(0x4E);   // quad_perm [2,3,0,1]
  DK_DPP_ADD(0x141);  // row_half_mirror
  DK_DPP_ADD(0x140);  // row_mirror
#undef DK_DPP_ADD
  return v;
}

// Rows of a batch: row r = (pixel q0 + r / taps, tap r % taps).  Writes the row's offsets and its dense
// cell rows: MODE 0: hat products (grad filter); MODE 1: d/dh and d/dw of them, zero where the offset is
// clamped (grad rotation; planar_bilinear_backward_coord, K.cu:116-163).
template <typename T, int MODE, int NCT>
__device__ __forceinline__ void nhwc_build_rows(const Geo& g, const T* __restrict__ rot, long q0, int nrows, int rows_padded,
                                                NhwcRow* rows, float* dense_a, float* dense_b) {
  constexpr int ROW = 16 * NCT;
  const int taps = g.k_h * g.k_w, oplane = g.out_h * g.out_w;
  for (int r = threadIdx.x; r < rows_padded; r += blockDim.x) {
    // the dense rows start as zeros; the (at most four) corners are then stored over them by the same thread
#pragma unroll
    for (int k = 0; k < ROW; k += 4) {
      *reinterpret_cast<nhwc_f4*>(dense_a + (size_t)r * ROW + k) = nhwc_f4{0.f, 0.f, 0.f, 0.f};
      if (MODE == 1) *reinterpret_cast<nhwc_f4*>(dense_b + (size_t)r * ROW + k) = nhwc_f4{0.f, 0.f, 0.f, 0.f};
    }
    NhwcRow row{kOutOfRange, kOutOfRange, 0u, 0u};
    if (r < nrows) {
      const long q = q0 + r / taps;
      const int t = r % taps, b = (int)(q / oplane), pix = (int)(q % oplane);
      int opix;
      long src_pix;
      const bool hit = tap_pixels<false>(g, pix, t, opix, src_pix);
      const size_t ri = rot_index_nhwc(g, b, pix, 0, t, 0);
      row.rix = (unsigned)ri;
      bool open_h = true, open_w = true;
      const float sh = scope_coord<float>(g, t / g.k_w, (float)ld(rot + ri), g.centre_h, &open_h);
      const float sw = scope_coord<float>(g, t % g.k_w, (float)ld(rot + ri + 1), g.centre_w, &open_w);
      if (hit && sh > -1.f && sw > -1.f && sh < (float)g.scope_h && sw < (float)g.scope_w) {
        row.src = (unsigned)((((long)b * g.in_h * g.in_w + src_pix) * g.channel) * (long)sizeof(T));
        row.gsrc = (unsigned)(q * g.channel * (long)sizeof(T));
        const float hf = floorf(sh), wf = floorf(sw);
        const int hl = (int)hf, wl = (int)wf, hi = hl + 1, wi = wl + 1;
        const float lh = sh - hf, lw = sw - wf, hh = 1.f - lh, hw = 1.f - lw;
        const bool cok[4] = {hl >= 0 && wl >= 0, hl >= 0 && wi <= g.scope_w - 1, hi <= g.scope_h - 1 && wl >= 0,
                             hi <= g.scope_h - 1 && wi <= g.scope_w - 1};
        const int ci[4] = {hl * g.scope_w + wl, hl * g.scope_w + wi, hi * g.scope_w + wl, hi * g.scope_w + wi};
        const float w0[4] = {hh * hw, hh * lw, lh * hw, lh * lw};
        const float dh[4] = {-hw, -lw, hw, lw}, dw[4] = {-hh, hh, -lh, lh};
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");  // the zeros above go first
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (!cok[k]) continue;
          if (MODE == 0) dense_a[(size_t)r * ROW + ci[k]] = w0[k];
          if (MODE == 1) {
            dense_a[(size_t)r * ROW + ci[k]] = open_h ? dh[k] : 0.f;
            dense_b[(size_t)r * ROW + ci[k]] = open_w ? dw[k] : 0.f;
          }
        }
      }
    }
    rows[r] = row;
  }
}

// grad filter: a workgroup owns a range of pixels and up to 16 tiles of 16 channels, one per wave, so the
// table of a batch is built once for all of them and every tile's loads are in flight together
constexpr int kMfTiles = 1;
template <typename T, int NCT>
__global__ __launch_bounds__(1024) void nhwc_grad_filter_mfma_kernel(Geo g, const T* __restrict__ gout,
                                                                        const T* __restrict__ x,
                                                                        const T* __restrict__ rot,
                                                                        float* __restrict__ partial, int pix_per_block) {
  constexpr int ROW = 16 * NCT;
  __shared__ NhwcRow rows[kMfRows];
  __shared__ __align__(16) float hats[kMfRows * ROW];
  const int taps = g.k_h * g.k_w, cells = g.scope_h * g.scope_w;
  const int oplane = g.out_h * g.out_w;
  const long total_pix = (long)g.batch * oplane;
  const long q_lo = (long)blockIdx.x * pix_per_block, q_hi = min(total_pix, q_lo + pix_per_block);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kg = lane >> 4, n = lane & 15;
  const int tile0 = blockIdx.y * (blockDim.x >> 6) + wave;  // this wave's tile
  const rsrc_t rg = plane_rsrc(gout, (int)(total_pix * g.channel)), rx = plane_rsrc(x, g.batch * g.in_h * g.in_w * g.channel);
  const int pb = kMfRows / taps;                      // pixels per batch (taps <= kMfRows, checked by the host)
  nhwc_f4 acc[kMfTiles][NCT];
#pragma unroll
  for (int j = 0; j < kMfTiles; ++j)
#pragma unroll
    for (int t = 0; t < NCT; ++t) acc[j][t] = nhwc_f4{0.f, 0.f, 0.f, 0.f};
  for (long qb = q_lo; qb < q_hi; qb += pb) {
    const int nrows = (int)min((long)pb, q_hi - qb) * taps;
    __syncthreads();
    nhwc_build_rows<T, 0, NCT>(g, rot, qb, nrows, kMfRows, rows, hats, nullptr);  // rows past nrows: dead, zero hats
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kMfTiles; ++j) {
      const int c0 = (tile0 + 4 * j) * 16;
      if (c0 >= g.channel) continue;              // uniform over the wave
      const int c = min(c0 + n, g.channel - 1);   // columns past the last channel repeat it; they are not stored
      // half a batch's loads first, then its products (a dead row loads zeros: no select anywhere)
      constexpr int STEPS = kMfRows / 8;  // (the whole batch at once needs 126 registers and is slower: 268 against 189 us)
      const unsigned cb_ = (unsigned)c * (unsigned)sizeof(T);
      for (int k0 = 0; 4 * k0 < nrows; k0 += STEPS) {
        typename RawOf<T>::type graw[STEPS], xraw[STEPS];
#pragma unroll
        for (int k = 0; k < STEPS; ++k) {
          const NhwcRow rw = rows[4 * (k0 + k) + kg];
          graw[k] = raw_ld(rg, rw.gsrc + cb_, gout);
          xraw[k] = raw_ld(rx, rw.src + cb_, x);
        }
#pragma unroll
        for (int k = 0; k < STEPS; ++k) {
          if (4 * (k0 + k) < nrows) {  // uniform over the wave
            const float pv = raw_cvt(graw[k], gout) * raw_cvt(xraw[k], x);
#pragma unroll
            for (int t = 0; t < NCT; ++t)
              acc[j][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(hats[(size_t)(4 * (k0 + k) + kg) * ROW + t * 16 + n], pv,
                                                               acc[j][t], 0, 0, 0);
          }
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < kMfTiles; ++j) {
    const int c0 = (tile0 + 4 * j) * 16;
    if (c0 + n < g.channel) {
      float* out = partial + ((size_t)blockIdx.x * g.channel + c0 + n) * cells;
#pragma unroll
      for (int t = 0; t < NCT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int cell = t * 16 + 4 * kg + i;
          if (cell < cells) out[cell] = acc[j][t][i];
        }
    }
  }
}

// grad rotation: a workgroup takes batches of pixels; a wave takes 16 rows ((pixel, tap) pairs) at a time and
// walks the channels 16 at a time, each lane loading four consecutive channels of its row.  The filter
// sits in LDS as [channel][16 * NCT] (zero rows up to a multiple of 16 channels).
template <typename T, int NCT>
__global__ __launch_bounds__(kNBlock) void nhwc_grad_rotation_mfma_kernel(Geo g, const T* __restrict__ gout,
                                                                          const T* __restrict__ x,
                                                                          const T* __restrict__ rot,
                                                                          const T* __restrict__ filter,
                                                                          T* __restrict__ grot, int batches_per_block) {
  constexpr int ROW = 16 * NCT;
  extern __shared__ __align__(16) unsigned char nhwc_lds[];
  __shared__ NhwcRow rows[kMfRows];
  __shared__ __align__(16) float dah[kMfRows * ROW];
  __shared__ __align__(16) float daw[kMfRows * ROW];
  // filter rows 4 floats apart from a multiple of 16: lane (kg, m) reads row 4 kg + j at column m, and
  // 4 * WROW = 16 mod 64 puts the four kg groups on four different sets of 16 banks
  constexpr int WROW = ROW + 4;
  float* wl = reinterpret_cast<float*>(nhwc_lds);  // [channels rounded up to 16][WROW]
  const int taps = g.k_h * g.k_w, cells = g.scope_h * g.scope_w;
  const int oplane = g.out_h * g.out_w;
  const long total_pix = (long)g.batch * oplane;
  const int cpad = (g.channel + 15) & ~15;
  for (int i = threadIdx.x; i < cpad * WROW; i += kNBlock) {
    const int ch = i / WROW, cell = i - ch * WROW;
    wl[i] = ch < g.channel && cell < cells ? (float)ld(filter + (size_t)ch * cells + cell) : 0.f;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kg = lane >> 4, m = lane & 15;
  const int pb = kMfRows / taps;
  const rsrc_t rg = plane_rsrc(gout, (int)(total_pix * g.channel)), rx = plane_rsrc(x, g.batch * g.in_h * g.in_w * g.channel);
  for (int bi = 0; bi < batches_per_block; ++bi) {
    const long qb = ((long)blockIdx.x * batches_per_block + bi) * pb;
    if (qb >= total_pix) break;  // uniform over the workgroup
    const int nrows = (int)min((long)pb, total_pix - qb) * taps;
    __syncthreads();
    nhwc_build_rows<T, 1, NCT>(g, rot, qb, nrows, (nrows + 15) & ~15, rows, dah, daw);
    __syncthreads();
    for (int rt = wave * 16; rt < nrows; rt += 64) {
      const NhwcRow rw = rows[rt + m];  // rows past nrows were written as dead rows
      nhwc_f4 acc[NCT];
#pragma unroll
      for (int t = 0; t < NCT; ++t) acc[t] = nhwc_f4{0.f, 0.f, 0.f, 0.f};
      const float* wlane = wl + 4 * kg * WROW + m;
      for (int cb = 0; cb < cpad; cb += 64) {  // four 16-channel blocks at a time, their loads first
        const float* wcb = wlane + cb * WROW;
        decltype(raw_ld4(rg, 0u, gout)) gp[4], xp[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          // channels past the last one: out of the resource's range for the last row, a neighbour's values for
          // the others -- multiplied by the filter's zero rows either way
          const unsigned cc = (unsigned)min(cb + 16 * u + 4 * kg, g.channel - 4) * (unsigned)sizeof(T);
          gp[u] = raw_ld4(rg, rw.gsrc + cc, gout);
          xp[u] = raw_ld4(rx, rw.src + cc, x);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (cb + 16 * u < cpad) {  // uniform
            const bool inside = cpad == g.channel || cb + 16 * u + 4 * kg < g.channel;
            float gv[4], xv[4];
            raw_cvt4(gp[u], gv, gout);
            raw_cvt4(xp[u], xv, x);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const float pv = inside ? gv[j] * xv[j] : 0.f;
#pragma unroll
              for (int t = 0; t < NCT; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(pv, wcb[(16 * u + j) * WROW + t * 16], acc[t], 0, 0, 0);
            }
          }
        }
      }
      // lane (kg, m) holds R[row rt + 4 kg + i][cell t * 16 + m]
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = rt + 4 * kg + i;
        float sh_ = 0.f, sw_ = 0.f;
#pragma unroll
        for (int t = 0; t < NCT; ++t) {
          sh_ += dah[(size_t)r * ROW + t * 16 + m] * acc[t][i];
          sw_ += daw[(size_t)r * ROW + t * 16 + m] * acc[t][i];
        }
        sh_ = row16_sum(sh_);
        sw_ = row16_sum(sw_);
        if (m == 0 && r < nrows) {
          const unsigned ri = rows[r].rix;
          st(grot + ri, sh_);
          st(grot + ri + 1, sw_);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// grad rotation with 32 channels per matrix instruction (3 x 3 taps, one group, a multiple of 8 channels).
// A wave owns 16 consecutive output pixels and all nine taps.  Per step of 32 channels, lane
// (pixel m = l % 16, k group kg = l / 16) loads channels 8 kg .. 8 kg + 7 of its pixel's out_grad once and of
// each tap's input pixel -- exactly the A operand of v_mfma_f32_16x16x32_bf16 (16 rows x 32 k, eight
// consecutive k per lane), so P = out_grad * input goes from the loads' registers into the instruction:
//   R_t[pixel][cell] = sum_c P_t[pixel][c] * W[c][cell]          (nine accumulators of 16 x 16 per 16 cells)
// The filter sits in LDS as [cell][channel] bfloat16, read 16 bytes per lane as the B operand.
// float32 / float16 tensors: P = Ph + Pl and W = Wh + Wl as bfloat16 (hi, lo) pairs and three products
// Ph Wh + Pl Wh + Ph Wl (16 significand bits; fp32 sums); bfloat16 tensors: W = Wh is exact and so is
// P = Ph + Pl (a product of two 8-bit significands), two products.
// Then  grot[pixel][t][dir] = sum_cell dA_dir[cell] * R_t[pixel][cell]  touches the four corner cells of the
// tap's scope coordinate only (planar_bilinear_backward_coord, K.cu:116-163): R_t goes to a wave-private
// LDS tile, three taps at a time, and lane (tap, pixel) reads its four corners.
// Invalid rows (pixels past the tensor's end, taps in the padding) and channel groups past the last
// channel get load offsets outside the buffer's range and load zeros: bit 31 for a row, bit 30 for a
// channel group, so that their sum stays out of range (the host admits tensors below 2^30 bytes).
// ---------------------------------------------------------------------------
typedef __bf16 nhwc_b8 __attribute__((ext_vector_type(8)));
constexpr int kR16Waves = 4;
constexpr int kR16TilesPerWave = 1;

// Orders a wave's LDS writes before its LDS reads and the other way round (its LDS operations execute in
// program order: only the compiler has to be kept from moving them across this point).
__device__ __forceinline__ void lds_fence_wave() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
}
constexpr unsigned kNoChannels = 0x40000000u;

template <typename T, int NCT, bool WLO>
__global__ __launch_bounds__(64 * kR16Waves, NCT == 1 ? 4 : 3) void nhwc_grad_rotation_mfma16_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ rot,
    const T* __restrict__ filter, T* __restrict__ grot, int tiles_per_wave, int wpitch, int tile_blocks, int csplits,
    float* __restrict__ partial) {
  constexpr int ROW = 16 * NCT, ROWP = ROW + 4, TAPS = 9;
  constexpr int NL = 2, HALF = 4;  // two loads of four channels for a lane's eight
  using Raw = typename std::conditional<sizeof(T) == 4, nhwc_u4, nhwc_u2>::type;
  extern __shared__ __align__(16) unsigned char nhwc_lds[];
  unsigned short* wh = reinterpret_cast<unsigned short*>(nhwc_lds);  // [ROW][wpitch] hi parts, then the lo parts
  unsigned short* wlo = wh + ROW * wpitch;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  float* rl = reinterpret_cast<float*>(nhwc_lds + (size_t)ROW * wpitch * 2 * (WLO ? 2 : 1)) + wave * (3 * 16 * ROWP);
  const int C = g.channel, cells = g.scope_h * g.scope_w;
  const int cpad = (C + 31) & ~31;
  const int lb_all = logical_block(tile_blocks * csplits);
  if (lb_all >= tile_blocks * csplits) return;
  // csplits > 1 (few tiles, many channels): this workgroup sums the steps s_lo .. s_hi - 1 of 32 channels into an
  // fp32 partial result of its own; reduce_few_parts_kernel adds the splits in order
  const int lb = lb_all % tile_blocks, split = lb_all / tile_blocks;
  const int nsteps_all = cpad / 32, per_split = (nsteps_all + csplits - 1) / csplits;
  const int s_lo = split * per_split, s_hi = min(nsteps_all, s_lo + per_split);

  // (eight loads at a time, all issued before the first is used: one at a time every workgroup began with a
  // chain of dependent trips to L2 that took longer than its products)
  for (int i0 = threadIdx.x + ROW * 32 * s_lo; i0 < ROW * 32 * s_hi; i0 += 8 * 64 * kR16Waves) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * 64 * kR16Waves;
      const int ch = i / ROW, cell = i - ch * ROW;
      v[u] = i < ROW * 32 * s_hi && ch < C && cell < cells ? (float)ld(filter + (size_t)ch * cells + cell) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * 64 * kR16Waves;
      if (i < ROW * 32 * s_hi) {
        const int ch = i / ROW, cell = i - ch * ROW;
        const unsigned hi = pack_bf16(v[u], 0.f) & 0xffffu;
        wh[cell * wpitch + ch] = (unsigned short)hi;
        if (WLO) wlo[cell * wpitch + ch] = (unsigned short)(pack_bf16(v[u] - bf16_lo(hi), 0.f) & 0xffffu);
      }
    }
  }
  __syncthreads();

  const int m = lane & 15, kg = lane >> 4;
  const int oplane = g.out_h * g.out_w;
  const long total_pix = (long)g.batch * oplane;
  const rsrc_t rg = plane_rsrc(gout, (int)(total_pix * C));
  const rsrc_t rx = plane_rsrc(x, g.batch * g.in_h * g.in_w * C);

  for (int tk = 0; tk < tiles_per_wave; ++tk) {
    const long q0 = (((long)lb * kR16Waves + wave) * tiles_per_wave + tk) * 16;
    if (q0 >= total_pix) break;  // uniform over the wave
    const long q = q0 + m;
    const bool live = q < total_pix;
    const long qc = live ? q : 0;
    const int b = (int)(qc / oplane), pix = (int)(qc - (long)b * oplane);
    const int oh = pix / g.out_w, ow = pix - oh * g.out_w;
    const unsigned goff = live ? (unsigned)(qc * C) * (unsigned)sizeof(T) : kOutOfRange;
    unsigned xoff[TAPS];
#pragma unroll
    for (int t = 0; t < TAPS; ++t) {
      const int ih = oh * g.stride_h - g.pad_h + (t / 3) * g.dil_h, iw = ow * g.stride_w - g.pad_w + (t % 3) * g.dil_w;
      const bool ok = live && ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
      xoff[t] = ok ? (unsigned)((((long)b * g.in_h + ih) * g.in_w + iw) * C) * (unsigned)sizeof(T) : kOutOfRange;
    }
    // byte offset of the lane's eight channels in a step, or kNoChannels
    auto chan_off = [&](int step) {
      const int c8 = step * 32 + 8 * kg;
      return c8 < C && step < s_hi ? (unsigned)c8 * (unsigned)sizeof(T) : kNoChannels;
    };

    nhwc_f4 acc[TAPS][NCT];
#pragma unroll
    for (int t = 0; t < TAPS; ++t)
#pragma unroll
      for (int n = 0; n < NCT; ++n) acc[t][n] = nhwc_f4{0.f, 0.f, 0.f, 0.f};
    Raw xr[3][NL], gcur[NL];  // a ring of three taps' loads: three taps ahead of the split and the products
    auto issue_x = [&](Raw (&buf)[NL], int t, unsigned co) {
#pragma unroll
      for (int h = 0; h < NL; ++h) buf[h] = raw_ld4(rx, xoff[t] + co + (unsigned)(HALF * sizeof(T)) * h, x);
    };
    auto issue_g = [&](Raw (&buf)[NL], unsigned co) {
#pragma unroll
      for (int h = 0; h < NL; ++h) buf[h] = raw_ld4(rg, goff + co + (unsigned)(HALF * sizeof(T)) * h, gout);
    };
    unsigned co = chan_off(s_lo);
    issue_g(gcur, co);
    issue_x(xr[0], 0, co);
    issue_x(xr[1], 1, co);
    issue_x(xr[2], 2, co);
    for (int step = s_lo; step < s_hi; ++step) {
      const unsigned co_next = chan_off(step + 1);  // past the last step: no channels, the loads return zeros
      // this step's filter operands
      uint4 bh[NCT], bl[NCT];
#pragma unroll
      for (int n = 0; n < NCT; ++n) {
        bh[n] = *reinterpret_cast<const uint4*>(wh + (n * 16 + m) * wpitch + step * 32 + 8 * kg);
        if (WLO) bl[n] = *reinterpret_cast<const uint4*>(wlo + (n * 16 + m) * wpitch + step * 32 + 8 * kg);
      }
      float gv[8];
#pragma unroll
      for (int h = 0; h < NL; ++h) {
        float f[4];
        raw_cvt4(gcur[h], f, gout);
#pragma unroll
        for (int i = 0; i < 4; ++i) gv[HALF * h + i] = f[i];
      }
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        float xv[8];
#pragma unroll
        for (int h = 0; h < NL; ++h) {
          float f[4];
          raw_cvt4(xr[t % 3][h], f, x);
#pragma unroll
          for (int i = 0; i < 4; ++i) xv[HALF * h + i] = f[i];
        }
        float pr[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          pr[i] = gv[i] * xv[i];
          asm volatile("" : "+v"(pr[i]));  // one fp32 value for both parts: no contraction into the conversions
        }
        // the tap's registers are free again: the load three taps ahead goes into them
        if (t + 3 < TAPS) issue_x(xr[t % 3], t + 3, co);
        else issue_x(xr[t % 3], t + 3 - TAPS, co_next);
        if (t == TAPS - 1) issue_g(gcur, co_next);  // out_grad of the next step, once this step's is used up
        unsigned hi[4], lo[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          hi[i] = pack_bf16(pr[2 * i], pr[2 * i + 1]);
          lo[i] = pack_bf16(pr[2 * i] - bf16_lo(hi[i]), pr[2 * i + 1] - bf16_hi(hi[i]));
        }
        const nhwc_b8 ph = __builtin_bit_cast(nhwc_b8, uint4{hi[0], hi[1], hi[2], hi[3]});
        const nhwc_b8 pl = __builtin_bit_cast(nhwc_b8, uint4{lo[0], lo[1], lo[2], lo[3]});
#pragma unroll
        for (int n = 0; n < NCT; ++n) {
          const nhwc_b8 wb = __builtin_bit_cast(nhwc_b8, bh[n]);
          acc[t][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph, wb, acc[t][n], 0, 0, 0);
          acc[t][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl, wb, acc[t][n], 0, 0, 0);
          if (WLO) acc[t][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph, __builtin_bit_cast(nhwc_b8, bl[n]), acc[t][n], 0, 0, 0);
        }
      }
      co = co_next;
    }

    // lane (kg, m) holds R_t[pixel 4 kg + i][cell 16 n + m]; lane (tap tt = l / 16 < 3, pixel m) finishes a row
#pragma unroll
    for (int ph_ = 0; ph_ < 3; ++ph_) {
      lds_fence_wave();
#pragma unroll
      for (int tt = 0; tt < 3; ++tt)
#pragma unroll
        for (int n = 0; n < NCT; ++n)
#pragma unroll
          for (int i = 0; i < 4; ++i) rl[(tt * 16 + 4 * kg + i) * ROWP + 16 * n + m] = acc[3 * ph_ + tt][n][i];
      lds_fence_wave();
      if (lane < 48 && live) {
        const int tt = kg, t = 3 * ph_ + tt;
        const int ih = oh * g.stride_h - g.pad_h + ph_ * g.dil_h, iw = ow * g.stride_w - g.pad_w + tt * g.dil_w;
        const bool hit = ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
        const size_t ri = (size_t)q * (TAPS * 2) + 2 * t;
        bool open_h = true, open_w = true;
        const float sh = scope_coord<float>(g, ph_, (float)ld(rot + ri), g.centre_h, &open_h);
        const float sw = scope_coord<float>(g, tt, (float)ld(rot + ri + 1), g.centre_w, &open_w);
        float gh = 0.f, gw = 0.f;
        if (hit && sh > -1.f && sw > -1.f && sh < (float)g.scope_h && sw < (float)g.scope_w) {
          const float hf = floorf(sh), wf = floorf(sw);
          const int hl = (int)hf, wl = (int)wf, hi_ = hl + 1, wi = wl + 1;
          const float lh = sh - hf, lw = sw - wf, hh = 1.f - lh, hw = 1.f - lw;
          const bool top = hl >= 0, bot = hi_ <= g.scope_h - 1, lft = wl >= 0, rgt = wi <= g.scope_w - 1;
          const float* row = rl + (tt * 16 + m) * ROWP;
          const int c00 = max(hl, 0) * g.scope_w + max(wl, 0), c01 = max(hl, 0) * g.scope_w + min(wi, g.scope_w - 1);
          const int c10 = min(hi_, g.scope_h - 1) * g.scope_w + max(wl, 0), c11 = min(hi_, g.scope_h - 1) * g.scope_w + min(wi, g.scope_w - 1);
          const float r00 = top && lft ? row[c00] : 0.f, r01 = top && rgt ? row[c01] : 0.f;
          const float r10 = bot && lft ? row[c10] : 0.f, r11 = bot && rgt ? row[c11] : 0.f;
          gh = hw * (r10 - r00) + lw * (r11 - r01);
          gw = hh * (r01 - r00) + lh * (r11 - r10);
        }
        if (partial) {
          float* dst = partial + (size_t)split * ((size_t)total_pix * (TAPS * 2)) + ri;
          dst[0] = open_h ? gh : 0.f;
          dst[1] = open_w ? gw : 0.f;
        } else {
          st(grot + ri, open_h ? gh : 0.f);
          st(grot + ri + 1, open_w ? gw : 0.f);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// forward / grad input on the matrix cores (3 x 3 taps, one group, scopes of up to 16 cells, a multiple of 4
// channels).  The bilinear read of a channel's scope is the dense contraction
//   w_eff[c][(pixel, tap)] = sum_cell W[c][cell] * A[cell][(pixel, tap)],   A = hat(h - i) * hat(w - j),
// and with the channels on the rows of v_mfma_f32_16x16x32_{f16,bf16} and 16 destination pixels on its columns
// the result lands as lane (kg, n) <- channels 4 kg .. 4 kg + 3 of pixel n: the four consecutive channels a
// 16-byte load of the tap's source pixel delivers, so the sources go from global memory to registers to
// four multiply-adds per tap with no staging, and the four results leave as one 16-byte store.
// Split precision as in the planar matrix-core kernel: A = Ah + Al in the matrix type; float32 tensors
// W * s = Wh + Wl in fp16 (s a power of two per channel that brings the channel's largest weight into [0.5, 1)),
// products Ah Wh + Al Wh (one K = 32 instruction: k = the lane group's four cells' hi parts, then their lo
// parts, against [Wh ; Wh]) and Ah Wl ([Wl ; 0]); 16-bit tensors: W is exact, one instruction.
// A wave owns 16 consecutive destination pixels: per tile the lane groups share the work on the nine taps'
// scope coordinates and source offsets through a wave-private LDS table, every lane derives its 36 operand
// registers, then the wave walks the channel blocks with the sources of two tap rows in flight.
// grad input is the same kernel on the transposed geometry (tap t of input pixel q is fed by the output
// pixel that reads q through t, with that pixel's rotation; K.cu:611-651).
// ---------------------------------------------------------------------------
template <typename E> struct NhwcMx;
template <> struct NhwcMx<_Float16> {
  typedef _Float16 v4 __attribute__((ext_vector_type(4)));
  typedef _Float16 v8 __attribute__((ext_vector_type(8)));
  // d_i = w0 * h_i (+ w1 * h_i): rows = 16 channels, columns = 16 pixels.  From inline assembly with
  // early-clobber results: a result of these instructions must not share registers with an operand,
  // which the compiler otherwise arranges at an operand's last use.  The second product on a result
  // follows two independent instructions; s_nop 7 covers the wait states before the vector ALU may read.
  template <bool SECOND>
  static __device__ __forceinline__ void rows3(nhwc_f4& d0, nhwc_f4& d1, nhwc_f4& d2, v8 w0, v8 w1, v8 h0, v8 h1, v8 h2) {
    if constexpr (SECOND)
      asm volatile(
          "s_nop 1\n\t"
          "v_mfma_f32_16x16x32_f16 %0, %3, %5, 0\n\t"
          "v_mfma_f32_16x16x32_f16 %1, %3, %6, 0\n\t"
          "v_mfma_f32_16x16x32_f16 %2, %3, %7, 0\n\t"
          "v_mfma_f32_16x16x32_f16 %0, %4, %5, %0\n\t"
          "v_mfma_f32_16x16x32_f16 %1, %4, %6, %1\n\t"
          "v_mfma_f32_16x16x32_f16 %2, %4, %7, %2\n\t"
          "s_nop 7"
          : "=&v"(d0), "=&v"(d1), "=&v"(d2)
          : "v"(w0), "v"(w1), "v"(h0), "v"(h1), "v"(h2));
    else
      asm volatile(
          "s_nop 1\n\t"
          "v_mfma_f32_16x16x32_f16 %0, %3, %4, 0\n\t"
          "v_mfma_f32_16x16x32_f16 %1, %3, %5, 0\n\t"
          "v_mfma_f32_16x16x32_f16 %2, %3, %6, 0\n\t"
          "s_nop 7"
          : "=&v"(d0), "=&v"(d1), "=&v"(d2)
          : "v"(w0), "v"(h0), "v"(h1), "v"(h2));
  }
};
template <> struct NhwcMx<__bf16> {
  typedef __bf16 v4 __attribute__((ext_vector_type(4)));
  typedef __bf16 v8 __attribute__((ext_vector_type(8)));
  template <bool SECOND>
  static __device__ __forceinline__ void rows3(nhwc_f4& d0, nhwc_f4& d1, nhwc_f4& d2, v8 w0, v8 w1, v8 h0, v8 h1, v8 h2) {
    static_assert(!SECOND, "bfloat16 tensors need no second product");
    asm volatile(
        "s_nop 1\n\t"
        "v_mfma_f32_16x16x32_bf16 %0, %3, %4, 0\n\t"
        "v_mfma_f32_16x16x32_bf16 %1, %3, %5, 0\n\t"
        "v_mfma_f32_16x16x32_bf16 %2, %3, %6, 0\n\t"
        "s_nop 7"
        : "=&v"(d0), "=&v"(d1), "=&v"(d2)
        : "v"(w0), "v"(h0), "v"(h1), "v"(h2));
  }
};
template <typename T> struct NhwcMxOf { using type = _Float16; };  // float, __half
template <> struct NhwcMxOf<bf16_t> { using type = __bf16; };

__device__ __forceinline__ float nhwc_hat(float d) { return __builtin_amdgcn_fmed3f(1.f - fabsf(d), 0.f, 1.f); }

template <int AUX = 0>
__device__ __forceinline__ void raw_st4(rsrc_t r, unsigned off, const float (&v)[4], float*) {
  __builtin_amdgcn_raw_buffer_store_b128(nhwc_u4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])}, r, (int)off, 0, AUX);
}
template <int AUX = 0, typename T>
__device__ __forceinline__ void raw_st4(rsrc_t r, unsigned off, const float (&v)[4], T*) {
  struct { T e[4]; } pk;
#pragma unroll
  for (int i = 0; i < 4; ++i) st(pk.e + i, v[i]);
  __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(nhwc_u2, pk), r, (int)off, 0, AUX);
}

constexpr int kG16Waves = 4;  // (two: 75.9 us on benchmark configuration 2, four: 74, six: 95)
// One tile per wave: workgroups that live as long as one tile keep the tail of the grid short (two tiles per wave
// measured 85.8 against 81.4 us on benchmark configuration 2, four 96).
constexpr int kG16TilesPerWave = 1;

template <typename T, int SH, int SW, bool TRANSPOSED>
__global__ __launch_bounds__(64 * kG16Waves) void nhwc_gather_mfma16_kernel(
    Geo g, const T* __restrict__ src, const T* __restrict__ rot, const T* __restrict__ filter, T* __restrict__ dst,
    int tiles_per_wave, int total_blocks) {
  using E = typename NhwcMxOf<T>::type;
  using M = NhwcMx<E>;
  using Raw = typename std::conditional<sizeof(T) == 4, nhwc_u4, nhwc_u2>::type;
  constexpr bool kThird = sizeof(T) == 4;  // float32 tensors: the filter has a low part
  constexpr int TAPS = 9, CELLS = SH * SW;
  static_assert(CELLS <= 16, "one block of sixteen cells");
  extern __shared__ __align__(16) unsigned char nhwc_lds[];
  const int C = g.channel, nblk = (C + 15) >> 4;
  uint4* wsp = reinterpret_cast<uint4*>(nhwc_lds);                // [nblk][64]: Wh (2 words), Wl (2 words) of lane (channel, cells 4 kg ..)
  float* unscale = reinterpret_cast<float*>(wsp + nblk * 64);     // [nblk][16]: 1 / s of the channel
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  float2* cw = reinterpret_cast<float2*>(unscale + nblk * 16) + wave * (TAPS * 16);             // [tap][pixel]: scope coordinates
  unsigned* xo = reinterpret_cast<unsigned*>(reinterpret_cast<float2*>(unscale + nblk * 16) + kG16Waves * TAPS * 16) +
                 wave * (TAPS * 16);                                                             // [tap][pixel]: source offsets
  const int lb = logical_block(total_blocks);
  if (lb >= total_blocks) return;

  // ---- per workgroup: the split filter operands of every channel block.  An entry is lane l of its wave, so the
  // channel's largest weight is the maximum over the four lanes l % 16 + 16 k of what each holds: one load per lane
  // instead of the channel's sixteen (a workgroup lives about as long as a dozen trips to L2, and every thread
  // waits for this table: forward 80 -> 75 us on benchmark configuration 2).  Issuing several entries' loads
  // together measured slower (83 us).
  for (int e = threadIdx.x; e < nblk * 64; e += 64 * kG16Waves) {
    const int b = e >> 6, l = e & 63, cj = b * 16 + (l & 15), c0 = 4 * (l >> 4);
    float v[4] = {0.f, 0.f, 0.f, 0.f}, s = 1.f;
    if (cj < C) {
      const T* f = filter + (size_t)cj * CELLS;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (c0 + k < CELLS) v[k] = (float)ld(f + c0 + k);
    }
    if constexpr (kThird) {
      float mx = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      int ex = 0;
      if (mx > 0.f && mx < __builtin_inff()) (void)frexpf(mx, &ex);
      ex = min(max(ex, -100), 100);
      s = ldexpf(1.f, -ex);
      if ((l >> 4) == 0) unscale[b * 16 + (l & 15)] = cj < C ? ldexpf(1.f, ex) : 0.f;
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] *= s;
    }
    typename M::v4 h4, l4;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float vv = v[k];
      asm volatile("" : "+v"(vv));  // one fp32 value for both parts
      const E hi = static_cast<E>(vv);
      h4[k] = hi;
      l4[k] = static_cast<E>(vv - static_cast<float>(hi));
    }
    const uint2 hb = __builtin_bit_cast(uint2, h4), lb2 = __builtin_bit_cast(uint2, l4);
    wsp[e] = make_uint4(hb.x, hb.y, lb2.x, lb2.y);
  }
  __syncthreads();

  const int n = lane & 15, kg = lane >> 4;
  const int oplane = g.out_h * g.out_w, iplane = g.in_h * g.in_w;
  const int dplane = TRANSPOSED ? iplane : oplane, splane = TRANSPOSED ? oplane : iplane;
  const long total_pix = (long)g.batch * dplane;
  const rsrc_t rs = plane_rsrc(src, g.batch * splane * C);
  const rsrc_t rd = plane_rsrc(dst, g.batch * dplane * C);
  // the lane group's four cells: rows past the last cell never match a coordinate
  float crow[4], ccol[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int c = 4 * kg + k;
    crow[k] = c < CELLS ? (float)(c / SW) : 64.f;
    ccol[k] = (float)(c % SW);
  }

  for (int tk = 0; tk < tiles_per_wave; ++tk) {
    const long q0 = (((long)lb * kG16Waves + wave) * tiles_per_wave + tk) * 16;
    if (q0 >= total_pix) break;  // uniform over the wave
    const long q = q0 + n;
    const bool live = q < total_pix;
    const long qc = live ? q : 0;
    const int b = (int)(qc / dplane), pix = (int)(qc - (long)b * dplane);

    // ---- the nine taps of the sixteen pixels: lane group kg takes taps kg, kg + 4, kg + 8
    lds_fence_wave();
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const int t = kg + 4 * k;
      if (t < TAPS) {
        int opix = 0;
        long src_pix = 0;
        const bool hit = tap_pixels<TRANSPOSED>(g, pix, t, opix, src_pix) && live;
        float2 c = make_float2(-2.f, -2.f);
        unsigned so = kOutOfRange;
        if (hit) {
          const size_t ri = ((size_t)b * oplane + opix) * (TAPS * 2) + 2 * t;
          const float h = scope_coord<float>(g, t / 3, (float)ld(rot + ri), g.centre_h);
          const float w = scope_coord<float>(g, t % 3, (float)ld(rot + ri + 1), g.centre_w);
          if (h > -1.f && w > -1.f && h < (float)SH && w < (float)SW) {
            c = make_float2(h, w);
            so = (unsigned)(((long)b * splane + src_pix) * C) * (unsigned)sizeof(T);
          }
        }
        cw[t * 16 + n] = c;
        xo[t * 16 + n] = so;
      }
    }
    lds_fence_wave();
    typename M::v8 A[TAPS];
    unsigned xoff[TAPS];
#pragma unroll
    for (int t = 0; t < TAPS; ++t) {
      const float2 c = cw[t * 16 + n];
      xoff[t] = xo[t * 16 + n];
      typedef float f2v __attribute__((ext_vector_type(2)));
      typedef E e2v __attribute__((ext_vector_type(2)));
      float v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        v[k] = nhwc_hat(c.x - crow[k]) * nhwc_hat(c.y - ccol[k]);
        asm volatile("" : "+v"(v[k]));  // one fp32 value for both parts
      }
      const e2v h01 = __builtin_convertvector(f2v{v[0], v[1]}, e2v), h23 = __builtin_convertvector(f2v{v[2], v[3]}, e2v);
      const f2v b01 = __builtin_convertvector(h01, f2v), b23 = __builtin_convertvector(h23, f2v);
      const e2v l01 = __builtin_convertvector(f2v{v[0] - b01[0], v[1] - b01[1]}, e2v);
      const e2v l23 = __builtin_convertvector(f2v{v[2] - b23[0], v[3] - b23[1]}, e2v);
      A[t] = typename M::v8{h01[0], h01[1], h23[0], h23[1], l01[0], l01[1], l23[0], l23[1]};
    }

    // ---- the channel blocks
    const unsigned doff = live ? (unsigned)(qc * C) * (unsigned)sizeof(T) : kOutOfRange;
    auto chan_off = [&](int blk) {
      const int c4 = blk * 16 + 4 * kg;
      return c4 < C ? (unsigned)c4 * (unsigned)sizeof(T) : kNoChannels;
    };
    Raw xr[3][3];  // [tap row][tap]: two tap rows ahead of the arithmetic
    auto issue_row = [&](Raw (&buf)[3], int r, unsigned co) {
#pragma unroll
      for (int tt = 0; tt < 3; ++tt) buf[tt] = raw_ld4(rs, xoff[3 * r + tt] + co, src);
    };
    unsigned co = chan_off(0);
    issue_row(xr[0], 0, co);
    issue_row(xr[1], 1, co);
    for (int blk = 0; blk < nblk; ++blk) {
      const unsigned co_next = chan_off(blk + 1);  // past the last block: no channels, zeros
      const uint4 wv = wsp[blk * 64 + lane];
      const typename M::v4 wh = __builtin_bit_cast(typename M::v4, make_uint2(wv.x, wv.y));
      const typename M::v4 wl = __builtin_bit_cast(typename M::v4, make_uint2(wv.z, wv.w));
      const typename M::v8 whh = __builtin_shufflevector(wh, wh, 0, 1, 2, 3, 0, 1, 2, 3);
      const typename M::v4 zero4 = {E(0), E(0), E(0), E(0)};
      const typename M::v8 wl0 = __builtin_shufflevector(wl, zero4, 0, 1, 2, 3, 4, 5, 6, 7);
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < 3; ++r) {
        if (r == 0) issue_row(xr[2], 2, co);
        else issue_row(xr[r - 1], r - 1, co_next);
        nhwc_f4 d[3];
        M::template rows3<kThird>(d[0], d[1], d[2], whh, wl0, A[3 * r], A[3 * r + 1], A[3 * r + 2]);
#pragma unroll
        for (int tt = 0; tt < 3; ++tt) {
          float xv[4];
          raw_cvt4(xr[r][tt], xv, src);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] = fmaf(xv[i], d[tt][i], acc[i]);
        }
      }
      if constexpr (kThird) {
        const nhwc_f4 us = *reinterpret_cast<const nhwc_f4*>(unscale + blk * 16 + 4 * kg);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] *= us[i];
      }
      // non-temporal: written with the default policy the result pushes the operands of the next kernel out of
      // the memory-side cache (the step of benchmark configuration 2 took 0.425 instead of 0.363 ms)
      raw_st4<kStreamingStore>(rd, doff + co, acc, dst);
      co = co_next;
    }
  }
}

// ---- host side --------------------------------------------------------------------------

constexpr int kFilterPixPerBlock = 128;
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

// The matrix-core forward / grad input; false where it does not apply.
template <typename T, int SH, int SW>
bool launch_gather_mfma16(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                          hipStream_t stream) {
  const int nblk = ceil_div(g.channel, 16);
  const size_t lds = (size_t)nblk * 64 * 16 + (size_t)nblk * 16 * 4 + (size_t)kG16Waves * 9 * 16 * (8 + 4);
  const long pixels = (long)g.batch * (transposed ? g.in_h * g.in_w : g.out_h * g.out_w);
  const long tiles = ceil_div(pixels, 16L);
  const int blocks = (int)ceil_div(tiles, (long)kG16Waves * kG16TilesPerWave);
  auto kernel = transposed ? nhwc_gather_mfma16_kernel<T, SH, SW, true> : nhwc_gather_mfma16_kernel<T, SH, SW, false>;
  if (lds > 64 * 1024 && !(lds <= 120 * 1024 && allow_dynamic_lds(reinterpret_cast<const void*>(kernel), 120 * 1024))) return false;
  hipLaunchKernelGGL(kernel, dim3((unsigned)xcd_grid_size(blocks)), dim3(64 * kG16Waves), lds, stream, g, src, rot, filter, dst,
                     kG16TilesPerWave, blocks);
  return true;
}

template <typename T>
bool nhwc_gather_mfma16(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                        hipStream_t stream) {
  if constexpr (std::is_same<T, double>::value) {
    return false;
  } else {
    const long bytes = (long)g.batch * g.channel * std::max((long)g.in_h * g.in_w, (long)g.out_h * g.out_w) * (long)sizeof(T);
    if (g.groups != 1 || g.k_h != 3 || g.k_w != 3 || g.channel % 4 != 0 || g.channel < 16 || bytes >= (1L << 30) ||
        reinterpret_cast<uintptr_t>(src) % (4 * sizeof(T)) != 0 || reinterpret_cast<uintptr_t>(dst) % (4 * sizeof(T)) != 0 ||
        path_disabled(kNoNhwcMfma) || path_disabled(kNoNhwcStaged))
      return false;
    // Where it is the faster kernel (step-level measurements on the MobileNetV2-DK layer shapes, batch 64, float32;
    // this kernel against the table kernel): its per-tile set-up (a third of its instructions at 144 channels) and
    // its one-tile-per-wave grid want many channels and many tiles.  Forward 144 x 56^2: 80 against 103 us, but
    // 32 x 112^2 136 / 109, 192 x 28^2 50 / 39, 960 x 7^2 58 / 22.  Grad input at stride 2, where the table kernel
    // tests every tap of every input pixel against the stride's grid: 96 x 112^2 166 / 262, 144 x 56^2 61 / 96,
    // 192 x 28^2 28 / 38.  DK_FORCE_NHWC_GATHER_MFMA takes it wherever it applies (the tests).
    const long tiles = ((long)g.batch * (transposed ? g.in_h * g.in_w : g.out_h * g.out_w) + 15) / 16;
    const bool strided = g.stride_h > 1 || g.stride_w > 1;
    const bool faster = (g.channel >= 128 && tiles >= 8192) || (transposed && strided && g.channel >= 64 && tiles >= 3000);
    if (!faster && !path_disabled(kForceNhwcGatherMfma)) return false;
    if (g.scope_h == 4 && g.scope_w == 4) return launch_gather_mfma16<T, 4, 4>(g, transposed, src, rot, filter, dst, stream);
    if (g.scope_h == 3 && g.scope_w == 3) return launch_gather_mfma16<T, 3, 3>(g, transposed, src, rot, filter, dst, stream);
    return false;
  }
}

template <typename T>
void nhwc_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                 hipStream_t stream) {
  if (nhwc_gather_mfma16<T>(g, transposed, src, rot, filter, dst, stream)) return;
  size_t lds;
  const NhwcLaunch L = gather_launch<T>(g, transposed, lds);
  const dim3 grid((unsigned)(g.batch * L.pblocks), (unsigned)ceil_div(g.channel, L.cc));
  const bool v4 = vec4_ok<T>(g, src, dst) && L.cc % 4 == 0;
  const bool nine = g.k_h * g.k_w == 9;
#define DK_NHWC_GATHER(VV, TT)                                                                                             \
  if (nine) hipLaunchKernelGGL((nhwc_gather_kernel<T, VV, TT, 9>), grid, dim3(kNBlock), lds, stream, g, L, src, rot, filter, dst); \
  else hipLaunchKernelGGL((nhwc_gather_kernel<T, VV, TT, 0>), grid, dim3(kNBlock), lds, stream, g, L, src, rot, filter, dst)
  if (transposed) {
    if (v4) { DK_NHWC_GATHER(4, true); }
    else { DK_NHWC_GATHER(1, true); }
  } else {
    if (v4) { DK_NHWC_GATHER(4, false); }
    else { DK_NHWC_GATHER(1, false); }
  }
#undef DK_NHWC_GATHER
}

// Shape test and channel splits of the 32-channel matrix-core grad rotation (0: it does not apply).  Few tiles of 16
// pixels and many channels (960 x 7 x 7 at batch 64: 196 tiles, 30 steps of 32 channels) leave most of the GPU idle:
// the steps are then split over workgroups, at least two steps each, for about four waves per SIMD.
int nhwc_rotation16_splits(const Geo& g, size_t elem) {
  const int nct = (g.scope_h * g.scope_w + 15) / 16;
  const long bytes = (long)g.batch * g.channel * std::max((long)g.in_h * g.in_w, (long)g.out_h * g.out_w) * (long)elem;
  if (g.groups != 1 || nct > 2 || g.k_h != 3 || g.k_w != 3 || g.channel % 8 != 0 || bytes >= (1L << 30) ||
      path_disabled(kNoNhwcMfma) || path_disabled(kNoNhwcStaged))
    return 0;
  const long tiles = ceil_div((long)g.batch * g.out_h * g.out_w, 16L);
  const int nsteps = (g.channel + 31) / 32;
  const long want = ceil_div(4096L, std::max(1L, tiles));
  return (int)std::max(1L, std::min<long>(want, nsteps / 2));
}

size_t nhwc_grad_rotation_workspace(const Geo& g, int dtype) {
  if (dtype == DK_F64) return 0;
  const int splits = nhwc_rotation16_splits(g, dtype == DK_F32 ? 4 : 2);
  return splits > 1 ? (size_t)splits * g.batch * g.out_h * g.out_w * 18 * sizeof(float) : 0;
}

template <typename T>
void nhwc_grad_rotation(const Geo& g, const T* gout, const T* x, const T* rot, const T* filter, T* grot, void* ws,
                        hipStream_t stream) {
  using CT = compute_t<T>;
  const int cells_ = g.scope_h * g.scope_w, taps_ = g.k_h * g.k_w;
  if constexpr (!std::is_same<T, double>::value) {
    const int nct = (cells_ + 15) / 16;
    const size_t wl_bytes = (size_t)((g.channel + 15) & ~15) * (16 * nct + 4) * sizeof(float);
    const bool aligned = g.channel % 4 == 0 && reinterpret_cast<uintptr_t>(gout) % (4 * sizeof(T)) == 0 &&
                         reinterpret_cast<uintptr_t>(x) % (4 * sizeof(T)) == 0;
    const bool small = (long)g.batch * g.channel * std::max((long)g.in_h * g.in_w, (long)g.out_h * g.out_w) * (long)sizeof(T) < (1L << 31);
    // 3 x 3 taps, a multiple of 8 channels: 32 channels per matrix instruction
    const int splits = nhwc_rotation16_splits(g, sizeof(T));
    if (splits > 0 && aligned) {
      constexpr bool wlo = !std::is_same<T, bf16_t>::value;
      const int wpitch = ((g.channel + 31) & ~31) + 8;
      const size_t lds = (size_t)16 * nct * wpitch * 2 * (wlo ? 2 : 1) + (size_t)kR16Waves * 48 * (16 * nct + 4) * sizeof(float);
      const long tiles = ceil_div((long)g.batch * g.out_h * g.out_w, 16L);
      const int blocks = (int)ceil_div(tiles, (long)kR16Waves * kR16TilesPerWave);
      auto kernel = nct == 1 ? nhwc_grad_rotation_mfma16_kernel<T, 1, wlo> : nhwc_grad_rotation_mfma16_kernel<T, 2, wlo>;
      if (lds <= 64 * 1024 || (lds <= 120 * 1024 && allow_dynamic_lds(reinterpret_cast<const void*>(kernel), 120 * 1024))) {
        float* partial = splits > 1 ? static_cast<float*>(ws) : nullptr;
        hipLaunchKernelGGL(kernel, dim3((unsigned)xcd_grid_size((long)blocks * splits)), dim3(64 * kR16Waves), lds, stream, g, gout,
                           x, rot, filter, grot, kR16TilesPerWave, wpitch, blocks, splits, partial);
        if (splits > 1) launch_reduce_partials<float, T>(partial, splits, (long)g.batch * g.out_h * g.out_w * 18, grot, stream);
        return;
      }
    }
    if (g.groups == 1 && nct <= 2 && taps_ <= kMfRows && aligned && small && wl_bytes <= 96 * 1024 && !path_disabled(kNoNhwcMfma)) {
      const int pb = kMfRows / taps_;
      const long batches = ceil_div((long)g.batch * g.out_h * g.out_w, (long)pb);
      const int per_block = 4;
      const dim3 grid((unsigned)ceil_div(batches, (long)per_block));
      if (nct == 1) {
        if (wl_bytes <= 40 * 1024 || allow_dynamic_lds(reinterpret_cast<const void*>(&nhwc_grad_rotation_mfma_kernel<T, 1>), 96 * 1024))
          hipLaunchKernelGGL((nhwc_grad_rotation_mfma_kernel<T, 1>), grid, dim3(kNBlock), wl_bytes, stream, g, gout, x, rot,
                             filter, grot, per_block);
      } else {
        if (wl_bytes <= 24 * 1024 || allow_dynamic_lds(reinterpret_cast<const void*>(&nhwc_grad_rotation_mfma_kernel<T, 2>), 96 * 1024))
          hipLaunchKernelGGL((nhwc_grad_rotation_mfma_kernel<T, 2>), grid, dim3(kNBlock), wl_bytes, stream, g, gout, x, rot,
                             filter, grot, per_block);
      }
      return;
    }
  }
  const size_t wt_bytes = (size_t)g.scope_h * g.scope_w * g.channel * sizeof(CT);
  const int in_lds = wt_bytes <= 48 * 1024;
  if (in_lds && g.k_h == 3 && g.k_w == 3) {
    const size_t entry = sizeof(NhwcRotTap<CT>) * g.groups * 9;
    const int pb = (int)std::max<size_t>(1, std::min<size_t>(16, 12 * 1024 / entry));
    const long total_pix = (long)g.batch * g.out_h * g.out_w;
    const size_t lds = ((wt_bytes + 15) & ~(size_t)15) + pb * entry;
    hipLaunchKernelGGL((nhwc_grad_rotation9_kernel<T>), dim3((unsigned)ceil_div(total_pix, (long)pb)), dim3(kNBlock), lds,
                       stream, g, gout, x, rot, filter, grot, pb);
    return;
  }
  const long items = (long)g.batch * g.out_h * g.out_w * g.groups * g.k_h * g.k_w;
  const long blocks = std::min<long>((items + 3) / 4, 256L * 32);
  hipLaunchKernelGGL((nhwc_grad_rotation_kernel<T>), dim3((unsigned)blocks), dim3(kNBlock), in_lds ? wt_bytes : 0, stream,
                     g, gout, x, rot, filter, grot, in_lds);
}

size_t nhwc_grad_filter_workspace(const Geo& g, int dtype) {
  const long parts = ceil_div((long)g.batch * g.out_h * g.out_w, (long)kFilterPixPerBlock);
  const size_t own = (size_t)parts * g.channel * g.scope_h * g.scope_w * (dtype == DK_F64 ? 8 : 4);
  // (the kernel that stages planar tiles is chosen by the tensors' alignment as well: room for either)
  return std::max(own, dtype == DK_F64 ? (size_t)0 : fast_local_grad_filter_cl_workspace(g));
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
  if constexpr (!std::is_same<T, double>::value) {
    // stride-1 layers of one group: the planar operator's matrix-core kernel, its tiles staged from channels-last rows
    if (fast_local_grad_filter_cl<T>(g, gout, x, rot, gfilter, ws, stream)) return;
    const int nct = (cells + 15) / 16;
    const bool small = (long)g.batch * g.channel * std::max((long)g.in_h * g.in_w, (long)g.out_h * g.out_w) * (long)sizeof(T) < (1L << 31);
    if (g.groups == 1 && nct <= 2 && taps <= kMfRows && small && !path_disabled(kNoNhwcMfma)) {
      const int ntiles = ceil_div(g.channel, 16), wpb = std::min(ntiles, 16);
      const dim3 mgrid((unsigned)parts, (unsigned)ceil_div(ntiles, wpb));
      if (nct == 1)
        hipLaunchKernelGGL((nhwc_grad_filter_mfma_kernel<T, 1>), mgrid, dim3(64 * wpb), 0, stream, g, gout, x, rot, partial,
                           kFilterPixPerBlock);
      else
        hipLaunchKernelGGL((nhwc_grad_filter_mfma_kernel<T, 2>), mgrid, dim3(64 * wpb), 0, stream, g, gout, x, rot, partial,
                           kFilterPixPerBlock);
      launch_reduce_partials<CT, T>(partial, parts, (long)g.channel * cells, gfilter, stream);
      return;
    }
  }
  const dim3 grid((unsigned)parts, (unsigned)ceil_div(g.channel, kNBlock));
  const bool nine = taps == 9;
#define DK_NHWC_GF1(CC, TT)                                                                                                    \
  if (lds <= 64 * 1024 || allow_dynamic_lds(reinterpret_cast<const void*>(&nhwc_grad_filter_kernel<T, CC, TT>), 144 * 1024))   \
  hipLaunchKernelGGL((nhwc_grad_filter_kernel<T, CC, TT>), grid, dim3(kNBlock), lds, stream, g, gout, x, rot, partial, kFilterPixPerBlock, pb)
#define DK_NHWC_GF(CC) \
  if (nine) { DK_NHWC_GF1(CC, 9); } else { DK_NHWC_GF1(CC, 0); }
  if (cells == 9) { DK_NHWC_GF(9); }
  else if (cells == 16) { DK_NHWC_GF(16); }
  else if (cells == 25) { DK_NHWC_GF(25); }
  else { DK_NHWC_GF(0); }
#undef DK_NHWC_GF
#undef DK_NHWC_GF1
  launch_reduce_partials<CT, T>(partial, parts, (long)g.channel * cells, gfilter, stream);
}

#define DK_INSTANTIATE(T)                                                                                  \
  template void nhwc_gather<T>(const Geo&, bool, const T*, const T*, const T*, T*, hipStream_t);           \
  template void nhwc_grad_rotation<T>(const Geo&, const T*, const T*, const T*, const T*, T*, void*, hipStream_t); \
  template void nhwc_grad_filter<T>(const Geo&, const T*, const T*, const T*, T*, void*, hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
DK_INSTANTIATE(double)
#undef DK_INSTANTIATE

}  // namespace dk
