// Generic kernels: any tap count, scope size, stride, padding, dilation,
// rotation-group count and dtype (fp32, fp16, bf16 with fp32 arithmetic; fp64
// with fp64 arithmetic), for the local and the deformable variant.  They keep
// the reference's one-thread-per-element decomposition but none of its global
// atomics except in the deformable grad-input scatter, where the target of a
// contribution is data dependent.  The tuned kernels take over for the shapes
// they cover; these are the fallback and the fp64 path.
//
// K.cu = deformable_kernels/ops/deform_kernel/csrc/filter_sample_depthwise_cuda_kernel.cu
#include "dk_kernels.h"

namespace dk {

namespace {

constexpr int kBlock = 256;

inline int grid_for(long total) {
  long b = (total + kBlock - 1) / kBlock;
  if (b > 1048576) b = 1048576;  // grid-stride beyond this
  if (b < 1) b = 1;
  return (int)b;
}

// Kernel-space offset at element `i` of the rotation tensor; a null tensor stands for all zeros
// (the deformable operator without kernel-space offsets).
template <typename T>
__device__ __forceinline__ compute_t<T> rot_at(const T* rot, size_t i) {
  return rot ? static_cast<compute_t<T>>(ld(rot + i)) : compute_t<T>(0);
}

// planar_bilinear, K.cu:51-83, on a tile in global memory.
template <typename T, typename CT>
__device__ __forceinline__ CT tile_bilinear(const T* tile, int S_h, int S_w, CT h, CT w) {
  if (!(h > CT(-1) && w > CT(-1) && h < CT(S_h) && w < CT(S_w))) return CT(0);
  const CT hf = floor(h), wf = floor(w);
  const int hl = (int)hf, wl = (int)wf, hi = hl + 1, wi = wl + 1;
  const CT lh = h - hf, lw = w - wf, hh = CT(1) - lh, hw = CT(1) - lw;
  CT v = 0;
  if (hl >= 0 && wl >= 0) v += hh * hw * ld(tile + hl * S_w + wl);
  if (hl >= 0 && wi <= S_w - 1) v += hh * lw * ld(tile + hl * S_w + wi);
  if (hi <= S_h - 1 && wl >= 0) v += lh * hw * ld(tile + hi * S_w + wl);
  if (hi <= S_h - 1 && wi <= S_w - 1) v += lh * lw * ld(tile + hi * S_w + wi);
  return v;
}

// planar_bilinear_backward_coord, K.cu:116-163, both directions at once (without
// the partial_sum factor).
template <typename T, typename CT>
__device__ __forceinline__ void tile_bilinear_dcoord(const T* tile, int S_h, int S_w, CT h, CT w,
                                                     CT& dh, CT& dw) {
  dh = dw = CT(0);
  if (!(h > CT(-1) && w > CT(-1) && h < CT(S_h) && w < CT(S_w))) return;
  const CT hf = floor(h), wf = floor(w);
  const int hl = (int)hf, wl = (int)wf, hi = hl + 1, wi = wl + 1;
  const CT lh = h - hf, lw = w - wf, hh = CT(1) - lh, hw = CT(1) - lw;
  if (hl >= 0 && wl >= 0) {
    const CT f = ld(tile + hl * S_w + wl);
    dh -= hw * f;
    dw -= hh * f;
  }
  if (hl >= 0 && wi <= S_w - 1) {
    const CT f = ld(tile + hl * S_w + wi);
    dh -= lw * f;
    dw += hh * f;
  }
  if (hi <= S_h - 1 && wl >= 0) {
    const CT f = ld(tile + hi * S_w + wl);
    dh += hw * f;
    dw -= lh * f;
  }
  if (hi <= S_h - 1 && wi <= S_w - 1) {
    const CT f = ld(tile + hi * S_w + wi);
    dh += lw * f;
    dw += lh * f;
  }
}

// deformable_im2col_bilinear, K.cu:165-199 (caller has checked the open box).
template <typename T, typename CT>
__device__ __forceinline__ CT image_bilinear(const T* plane, int H, int W, CT h, CT w) {
  const CT hf = floor(h), wf = floor(w);
  const int hl = (int)hf, wl = (int)wf, hi = hl + 1, wi = wl + 1;
  const CT lh = h - hf, lw = w - wf, hh = CT(1) - lh, hw = CT(1) - lw;
  CT v1 = 0, v2 = 0, v3 = 0, v4 = 0;
  if (hl >= 0 && wl >= 0) v1 = ld(plane + hl * W + wl);
  if (hl >= 0 && wi <= W - 1) v2 = ld(plane + hl * W + wi);
  if (hi <= H - 1 && wl >= 0) v3 = ld(plane + hi * W + wl);
  if (hi <= H - 1 && wi <= W - 1) v4 = ld(plane + hi * W + wi);
  return hh * hw * v1 + hh * lw * v2 + lh * hw * v3 + lh * lw * v4;
}

// get_coordinate_weight, K.cu:231-268, both directions at once.
template <typename T, typename CT>
__device__ __forceinline__ void image_bilinear_dcoord(const T* plane, int H, int W, CT h, CT w,
                                                      CT& dh, CT& dw) {
  const CT hf = floor(h), wf = floor(w);
  const int hl = (int)hf, wl = (int)wf, hi = hl + 1, wi = wl + 1;
  const CT wr = (wf + CT(1)) - w, wq = w - wf;  // (w_low + 1 - w), (w - w_low)
  const CT hr = (hf + CT(1)) - h, hq = h - hf;
  dh = dw = CT(0);
  if (hl >= 0 && wl >= 0) {
    const CT v = ld(plane + hl * W + wl);
    dh -= wr * v;
    dw -= hr * v;
  }
  if (hl >= 0 && wi <= W - 1) {
    const CT v = ld(plane + hl * W + wi);
    dh -= wq * v;
    dw += hr * v;
  }
  if (hi <= H - 1 && wl >= 0) {
    const CT v = ld(plane + hi * W + wl);
    dh += wr * v;
    dw -= hq * v;
  }
  if (hi <= H - 1 && wi <= W - 1) {
    const CT v = ld(plane + hi * W + wi);
    dh += wq * v;
    dw += hq * v;
  }
}

struct TapCoords {
  size_t rot_h;  // element offset of the h rotation of this (b, g, tap, pixel); w is one plane on
  size_t off_h;  // same for the image-space offset
};

__device__ __forceinline__ size_t rot_index(const Geo& g, int b, int grp, int t, int pix) {
  return ((size_t)(b * g.groups + grp) * (g.k_h * g.k_w) + t) * 2 * ((size_t)g.out_h * g.out_w) + pix;
}
__device__ __forceinline__ size_t off_index(const Geo& g, int b, int t, int pix) {
  return ((size_t)b * (g.k_h * g.k_w) + t) * 2 * ((size_t)g.out_h * g.out_w) + pix;
}

// Value the tap (f_h, f_w) of output pixel (oh, ow) reads from channel plane `xp`
// (local: the input element, zero in the padding; deformable: the bilinear sample,
// zero outside the image band).  `hit` is false where the reference skips the tap.
template <typename T, typename CT, bool DEFORM>
__device__ __forceinline__ CT tap_input(const Geo& g, const T* xp, const T* off, int b, int t,
                                        int f_h, int f_w, int oh, int ow, bool& hit, CT& ih_f,
                                        CT& iw_f) {
  const int ih = oh * g.stride_h - g.pad_h + f_h * g.dil_h;
  const int iw = ow * g.stride_w - g.pad_w + f_w * g.dil_w;
  if (!DEFORM) {
    hit = ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
    ih_f = CT(ih);
    iw_f = CT(iw);
    return (hit && xp) ? ld(xp + ih * g.in_w + iw) : CT(0);
  } else {
    const size_t oi = off_index(g, b, t, oh * g.out_w + ow);
    ih_f = CT(ih) + ld(off + oi);
    iw_f = CT(iw) + ld(off + oi + (size_t)g.out_h * g.out_w);
    hit = ih_f > CT(-1) && iw_f > CT(-1) && ih_f < CT(g.in_h) && iw_f < CT(g.in_w);
    return (hit && xp) ? image_bilinear<T, CT>(xp, g.in_h, g.in_w, ih_f, iw_f) : CT(0);
  }
}

// ---- forward: K.cu:270-386 (local), K.cu:433-528 (deformable) -----------------------------
template <typename T, bool DEFORM>
__global__ __launch_bounds__(kBlock) void generic_forward_kernel(
    Geo g, const T* __restrict__ x, const T* __restrict__ off, const T* __restrict__ rot,
    const T* __restrict__ filter, T* __restrict__ out, long total) {
  using CT = compute_t<T>;
  const int plane = g.out_h * g.out_w;
  for (long id = (long)blockIdx.x * kBlock + threadIdx.x; id < total; id += (long)gridDim.x * kBlock) {
    const int pix = (int)(id % plane);
    const int c = (int)((id / plane) % g.channel);
    const int b = (int)(id / plane / g.channel);
    const int oh = pix / g.out_w, ow = pix % g.out_w;
    const int grp = c % g.groups;
    const T* xp = x + ((size_t)b * g.channel + c) * g.in_h * g.in_w;
    const T* tile = filter + (size_t)c * g.scope_h * g.scope_w;
    CT sum = 0;
    for (int f_h = 0; f_h < g.k_h; ++f_h)
      for (int f_w = 0; f_w < g.k_w; ++f_w) {
        const int t = f_h * g.k_w + f_w;
        bool hit;
        CT ihf, iwf;
        const CT xv = tap_input<T, CT, DEFORM>(g, xp, off, b, t, f_h, f_w, oh, ow, hit, ihf, iwf);
        if (hit) {
          const size_t ri = rot_index(g, b, grp, t, pix);
          const CT h = scope_coord<CT>(g, f_h, rot_at(rot, ri), g.centre_h);
          const CT w = scope_coord<CT>(g, f_w, rot_at(rot, ri + plane), g.centre_w);
          sum += xv * tile_bilinear<T, CT>(tile, g.scope_h, g.scope_w, h, w);
        }
      }
    st(out + id, sum);
  }
}

// ---- local grad input: K.cu:577-669 -------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void generic_local_grad_input_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ rot, const T* __restrict__ filter,
    T* __restrict__ gin, long total) {
  using CT = compute_t<T>;
  const int iplane = g.in_h * g.in_w, oplane = g.out_h * g.out_w;
  for (long id = (long)blockIdx.x * kBlock + threadIdx.x; id < total; id += (long)gridDim.x * kBlock) {
    const int pix = (int)(id % iplane);
    const int c = (int)((id / iplane) % g.channel);
    const int b = (int)(id / iplane / g.channel);
    const int ih = pix / g.in_w, iw = pix % g.in_w;
    const int grp = c % g.groups;
    const T* gp = gout + ((size_t)b * g.channel + c) * oplane;
    const T* tile = filter + (size_t)c * g.scope_h * g.scope_w;
    CT sum = 0;
    for (int f_h = 0; f_h < g.k_h; ++f_h) {
      const int th = ih + g.pad_h - f_h * g.dil_h;
      if (th < 0 || th % g.stride_h != 0) continue;
      const int oh = th / g.stride_h;
      if (oh >= g.out_h) continue;
      for (int f_w = 0; f_w < g.k_w; ++f_w) {
        const int tw = iw + g.pad_w - f_w * g.dil_w;
        if (tw < 0 || tw % g.stride_w != 0) continue;
        const int ow = tw / g.stride_w;
        if (ow >= g.out_w) continue;
        const int t = f_h * g.k_w + f_w, opix = oh * g.out_w + ow;
        const size_t ri = rot_index(g, b, grp, t, opix);
        const CT h = scope_coord<CT>(g, f_h, rot_at(rot, ri), g.centre_h);
        const CT w = scope_coord<CT>(g, f_w, rot_at(rot, ri + oplane), g.centre_w);
        sum += ld(gp + opix) * tile_bilinear<T, CT>(tile, g.scope_h, g.scope_w, h, w);
      }
    }
    st(gin + id, sum);
  }
}

// ---- deformable grad input: K.cu:704-795, scatter with hardware float atomics -------------
template <typename T, typename CT>
__global__ __launch_bounds__(kBlock) void generic_deform_grad_input_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ off, const T* __restrict__ rot,
    const T* __restrict__ filter, CT* __restrict__ gin_acc, long total) {
  const int oplane = g.out_h * g.out_w, K = g.k_h * g.k_w;
  const int H = g.in_h, W = g.in_w;
  for (long id = (long)blockIdx.x * kBlock + threadIdx.x; id < total; id += (long)gridDim.x * kBlock) {
    const int pix = (int)(id % oplane);
    const int c = (int)((id / oplane) % g.channel);
    const int t = (int)((id / oplane / g.channel) % K);
    const int b = (int)(id / oplane / g.channel / K);
    const int oh = pix / g.out_w, ow = pix % g.out_w;
    const int f_h = t / g.k_w, f_w = t % g.k_w;
    bool hit;
    CT h, w;
    tap_input<T, CT, true>(g, (const T*)nullptr, off, b, t, f_h, f_w, oh, ow, hit, h, w);
    if (!hit) continue;
    const int grp = c % g.groups;
    const size_t ri = rot_index(g, b, grp, t, pix);
    const CT sh = scope_coord<CT>(g, f_h, rot_at(rot, ri), g.centre_h);
    const CT sw = scope_coord<CT>(g, f_w, rot_at(rot, ri + oplane), g.centre_w);
    const CT ps = tile_bilinear<T, CT>(filter + (size_t)c * g.scope_h * g.scope_w, g.scope_h,
                                       g.scope_w, sh, sw) *
                  ld(gout + ((size_t)b * g.channel + c) * oplane + pix);
    CT* dp = gin_acc + ((size_t)b * g.channel + c) * H * W;
    const CT hf = floor(h), wf = floor(w);
    const int hl = (int)hf, wl = (int)wf, hi = hl + 1, wi = wl + 1;
    const CT lh = h - hf, lw = w - wf, hh = CT(1) - lh, hw = CT(1) - lw;
    if (hl >= 0 && wl >= 0) atomicAdd(dp + hl * W + wl, hh * hw * ps);
    if (hl >= 0 && wi <= W - 1) atomicAdd(dp + hl * W + wi, hh * lw * ps);
    if (hi <= H - 1 && wl >= 0) atomicAdd(dp + hi * W + wl, lh * hw * ps);
    if (hi <= H - 1 && wi <= W - 1) atomicAdd(dp + hi * W + wi, lh * lw * ps);
  }
}

template <typename CT>
__global__ void fill_zero_kernel(CT* p, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    p[i] = CT(0);
}

template <typename CT, typename T>
__global__ void convert_kernel(const CT* __restrict__ a, T* __restrict__ out, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    st(out + i, a[i]);
}

// ---- grad rotation: K.cu:1285-1370 (local), K.cu:1410-1507 (deformable) ------------------
// one thread per (b, group, tap, pixel), both directions
template <typename T, bool DEFORM>
__global__ __launch_bounds__(kBlock) void generic_grad_rotation_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ off,
    const T* __restrict__ rot, const T* __restrict__ filter, T* __restrict__ grot, long total) {
  using CT = compute_t<T>;
  const int oplane = g.out_h * g.out_w, iplane = g.in_h * g.in_w, K = g.k_h * g.k_w;
  for (long id = (long)blockIdx.x * kBlock + threadIdx.x; id < total; id += (long)gridDim.x * kBlock) {
    const int pix = (int)(id % oplane);
    const int t = (int)((id / oplane) % K);
    const int grp = (int)((id / oplane / K) % g.groups);
    const int b = (int)(id / oplane / K / g.groups);
    const int oh = pix / g.out_w, ow = pix % g.out_w;
    const int f_h = t / g.k_w, f_w = t % g.k_w;
    const size_t ri = rot_index(g, b, grp, t, pix);
    bool open_h, open_w;  // false: the offset was clamped, its gradient is zero
    const CT h = scope_coord<CT>(g, f_h, rot_at(rot, ri), g.centre_h, &open_h);
    const CT w = scope_coord<CT>(g, f_w, rot_at(rot, ri + oplane), g.centre_w, &open_w);
    CT gh = 0, gw = 0;
    bool hit;
    CT ihf, iwf;
    tap_input<T, CT, DEFORM>(g, (const T*)nullptr, off, b, t, f_h, f_w, oh, ow, hit, ihf, iwf);
    if (hit) {
      for (int c = grp; c < g.channel; c += g.groups) {
        const T* xp = x + ((size_t)b * g.channel + c) * iplane;
        bool hit2;
        const CT xv = tap_input<T, CT, DEFORM>(g, xp, off, b, t, f_h, f_w, oh, ow, hit2, ihf, iwf);
        const CT ps = xv * ld(gout + ((size_t)b * g.channel + c) * oplane + pix);
        CT dh, dw;
        tile_bilinear_dcoord<T, CT>(filter + (size_t)c * g.scope_h * g.scope_w, g.scope_h, g.scope_w,
                                    h, w, dh, dw);
        gh += ps * dh;
        gw += ps * dw;
      }
    }
    st(grot + ri, open_h ? gh : CT(0));
    st(grot + ri + oplane, open_w ? gw : CT(0));
  }
}

// ---- grad offset: K.cu:1147-1243; one thread per (b, tap, pixel), both directions --------
template <typename T>
__global__ __launch_bounds__(kBlock) void generic_grad_offset_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ off,
    const T* __restrict__ rot, const T* __restrict__ filter, T* __restrict__ goff, long total) {
  using CT = compute_t<T>;
  const int oplane = g.out_h * g.out_w, iplane = g.in_h * g.in_w, K = g.k_h * g.k_w;
  for (long id = (long)blockIdx.x * kBlock + threadIdx.x; id < total; id += (long)gridDim.x * kBlock) {
    const int pix = (int)(id % oplane);
    const int t = (int)((id / oplane) % K);
    const int b = (int)(id / oplane / K);
    const int oh = pix / g.out_w, ow = pix % g.out_w;
    const int f_h = t / g.k_w, f_w = t % g.k_w;
    bool hit;
    CT h, w;
    tap_input<T, CT, true>(g, (const T*)nullptr, off, b, t, f_h, f_w, oh, ow, hit, h, w);
    CT gh = 0, gw = 0;
    if (hit) {
      for (int c = 0; c < g.channel; ++c) {
        const int grp = c % g.groups;
        const size_t ri = rot_index(g, b, grp, t, pix);
        const CT sh = scope_coord<CT>(g, f_h, rot_at(rot, ri), g.centre_h);
        const CT sw = scope_coord<CT>(g, f_w, rot_at(rot, ri + oplane), g.centre_w);
        const CT ps = tile_bilinear<T, CT>(filter + (size_t)c * g.scope_h * g.scope_w, g.scope_h,
                                           g.scope_w, sh, sw) *
                      ld(gout + ((size_t)b * g.channel + c) * oplane + pix);
        CT dh, dw;
        image_bilinear_dcoord<T, CT>(x + ((size_t)b * g.channel + c) * iplane, g.in_h, g.in_w, h, w,
                                     dh, dw);
        gh += dh * ps;
        gw += dw * ps;
      }
    }
    const size_t oi = off_index(g, b, t, pix);
    st(goff + oi, gh);
    st(goff + oi + oplane, gw);
  }
}

// ---- grad filter: K.cu:836-955 (local), K.cu:1002-1097 (deformable) ----------------------
// A workgroup owns one channel and every `parts`-th image; contributions go to a replicated
// LDS accumulator (replica = lane id mod R), folded at the end into partial[part][c][cell].
template <typename T, bool DEFORM>
__global__ __launch_bounds__(kBlock) void generic_grad_filter_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ off,
    const T* __restrict__ rot, compute_t<T>* __restrict__ partial, int reps) {
  using CT = compute_t<T>;
  extern __shared__ unsigned char smem_raw[];
  CT* acc = reinterpret_cast<CT*>(smem_raw);
  const int cells = g.scope_h * g.scope_w;
  for (int e = threadIdx.x; e < cells * reps; e += kBlock) acc[e] = CT(0);
  __syncthreads();

  const int c = blockIdx.y, grp = c % g.groups;
  const int oplane = g.out_h * g.out_w, iplane = g.in_h * g.in_w;
  const int rep = threadIdx.x % reps;
  const int S_h = g.scope_h, S_w = g.scope_w;
  for (int b = blockIdx.x; b < g.batch; b += gridDim.x) {
    const T* xp = x + ((size_t)b * g.channel + c) * iplane;
    const T* gp = gout + ((size_t)b * g.channel + c) * oplane;
    for (int pix = threadIdx.x; pix < oplane; pix += kBlock) {
      const int oh = pix / g.out_w, ow = pix % g.out_w;
      const CT go = ld(gp + pix);
      for (int f_h = 0; f_h < g.k_h; ++f_h)
        for (int f_w = 0; f_w < g.k_w; ++f_w) {
          const int t = f_h * g.k_w + f_w;
          bool hit;
          CT ihf, iwf;
          const CT xv = tap_input<T, CT, DEFORM>(g, xp, off, b, t, f_h, f_w, oh, ow, hit, ihf, iwf);
          if (!hit) continue;
          const size_t ri = rot_index(g, b, grp, t, pix);
          const CT h = scope_coord<CT>(g, f_h, rot_at(rot, ri), g.centre_h);
          const CT w = scope_coord<CT>(g, f_w, rot_at(rot, ri + oplane), g.centre_w);
          if (!(h > CT(-1) && w > CT(-1) && h < CT(S_h) && w < CT(S_w))) continue;
          const CT ps = xv * go;
          const CT hf = floor(h), wf = floor(w);
          const int hl = (int)hf, wl = (int)wf, hi = hl + 1, wi = wl + 1;
          const CT lh = h - hf, lw = w - wf, hh = CT(1) - lh, hw = CT(1) - lw;
          if (hl >= 0 && wl >= 0) atomicAdd(acc + (hl * S_w + wl) * reps + rep, hh * hw * ps);
          if (hl >= 0 && wi <= S_w - 1) atomicAdd(acc + (hl * S_w + wi) * reps + rep, hh * lw * ps);
          if (hi <= S_h - 1 && wl >= 0) atomicAdd(acc + (hi * S_w + wl) * reps + rep, lh * hw * ps);
          if (hi <= S_h - 1 && wi <= S_w - 1)
            atomicAdd(acc + (hi * S_w + wi) * reps + rep, lh * lw * ps);
        }
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < cells; e += kBlock) {
    CT s = 0;
    for (int q = 0; q < reps; ++q) s += acc[e * reps + (q + threadIdx.x) % reps];
    partial[((size_t)blockIdx.x * g.channel + c) * cells + e] = s;
  }
}

int filter_reps(const Geo& g, size_t elt) {
  const size_t cells = (size_t)g.scope_h * g.scope_w;
  size_t r = (48 * 1024) / (cells * elt);
  if (r > 32) r = 32;
  if (r < 1) r = 1;
  return (int)r;
}

int filter_parts(const Geo& g) {
  int parts = ceil_div(1024, g.channel);
  if (parts > g.batch) parts = g.batch;
  if (parts < 1) parts = 1;
  return parts;
}

}  // namespace

template <typename T>
void generic_forward(const Geo& g, bool deform, const T* x, const T* off, const T* rot,
                     const T* filter, T* out, hipStream_t stream) {
  const long total = (long)g.batch * g.channel * g.out_h * g.out_w;
  if (deform)
    generic_forward_kernel<T, true><<<grid_for(total), kBlock, 0, stream>>>(g, x, off, rot, filter, out, total);
  else
    generic_forward_kernel<T, false><<<grid_for(total), kBlock, 0, stream>>>(g, x, off, rot, filter, out, total);
}

template <typename T>
void generic_local_grad_input(const Geo& g, const T* gout, const T* rot, const T* filter, T* gin,
                              hipStream_t stream) {
  const long total = (long)g.batch * g.channel * g.in_h * g.in_w;
  generic_local_grad_input_kernel<T><<<grid_for(total), kBlock, 0, stream>>>(g, gout, rot, filter, gin, total);
}

size_t generic_deform_grad_input_workspace(const Geo& g, int dtype) {
  // fp16 / bf16 gradients are scattered into an fp32 image first
  if (dtype == DK_F16 || dtype == DK_BF16)
    return (size_t)g.batch * g.channel * g.in_h * g.in_w * sizeof(float);
  return 0;
}

template <typename T>
void generic_deform_grad_input(const Geo& g, const T* gout, const T* off, const T* rot,
                               const T* filter, T* gin, void* ws, hipStream_t stream) {
  using CT = compute_t<T>;
  const long n_in = (long)g.batch * g.channel * g.in_h * g.in_w;
  const long total = (long)g.batch * g.k_h * g.k_w * g.channel * g.out_h * g.out_w;
  constexpr bool direct = sizeof(T) == sizeof(CT);
  CT* acc = direct ? reinterpret_cast<CT*>(gin) : static_cast<CT*>(ws);
  fill_zero_kernel<CT><<<grid_for(n_in), kBlock, 0, stream>>>(acc, n_in);
  generic_deform_grad_input_kernel<T, CT><<<grid_for(total), kBlock, 0, stream>>>(g, gout, off, rot, filter, acc, total);
  if (!direct) convert_kernel<CT, T><<<grid_for(n_in), kBlock, 0, stream>>>(acc, gin, n_in);
}

template <typename T>
void generic_grad_rotation(const Geo& g, bool deform, const T* gout, const T* x, const T* off,
                           const T* rot, const T* filter, T* grot, hipStream_t stream) {
  const long total = (long)g.batch * g.groups * g.k_h * g.k_w * g.out_h * g.out_w;
  if (deform)
    generic_grad_rotation_kernel<T, true><<<grid_for(total), kBlock, 0, stream>>>(g, gout, x, off, rot, filter, grot, total);
  else
    generic_grad_rotation_kernel<T, false><<<grid_for(total), kBlock, 0, stream>>>(g, gout, x, off, rot, filter, grot, total);
}

template <typename T>
void generic_grad_offset(const Geo& g, const T* gout, const T* x, const T* off, const T* rot,
                         const T* filter, T* goff, hipStream_t stream) {
  const long total = (long)g.batch * g.k_h * g.k_w * g.out_h * g.out_w;
  generic_grad_offset_kernel<T><<<grid_for(total), kBlock, 0, stream>>>(g, gout, x, off, rot, filter, goff, total);
}

size_t generic_grad_filter_workspace(const Geo& g, int dtype) {
  const size_t elt = dtype == DK_F64 ? sizeof(double) : sizeof(float);
  return (size_t)filter_parts(g) * g.channel * g.scope_h * g.scope_w * elt;
}

template <typename T>
void generic_grad_filter(const Geo& g, bool deform, const T* gout, const T* x, const T* off,
                         const T* rot, T* gfilter, void* ws, hipStream_t stream) {
  using CT = compute_t<T>;
  const int parts = filter_parts(g), reps = filter_reps(g, sizeof(CT));
  const size_t lds = (size_t)g.scope_h * g.scope_w * reps * sizeof(CT);
  const dim3 grid(parts, g.channel);
  CT* partial = static_cast<CT*>(ws);
  if (deform)
    generic_grad_filter_kernel<T, true><<<grid, kBlock, lds, stream>>>(g, gout, x, off, rot, partial, reps);
  else
    generic_grad_filter_kernel<T, false><<<grid, kBlock, lds, stream>>>(g, gout, x, off, rot, partial, reps);
  launch_reduce_partials<CT, T>(partial, parts, g.channel * g.scope_h * g.scope_w, gfilter, stream);
}

#define DK_INSTANTIATE(T)                                                                            \
  template void generic_forward<T>(const Geo&, bool, const T*, const T*, const T*, const T*, T*,      \
                                   hipStream_t);                                                     \
  template void generic_local_grad_input<T>(const Geo&, const T*, const T*, const T*, T*, hipStream_t); \
  template void generic_deform_grad_input<T>(const Geo&, const T*, const T*, const T*, const T*, T*,  \
                                             void*, hipStream_t);                                    \
  template void generic_grad_rotation<T>(const Geo&, bool, const T*, const T*, const T*, const T*,    \
                                         const T*, T*, hipStream_t);                                 \
  template void generic_grad_offset<T>(const Geo&, const T*, const T*, const T*, const T*, const T*,  \
                                       T*, hipStream_t);                                             \
  template void generic_grad_filter<T>(const Geo&, bool, const T*, const T*, const T*, const T*, T*,  \
                                       void*, hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(double)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
#undef DK_INSTANTIATE

}  // namespace dk
