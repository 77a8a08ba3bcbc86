// Local deformable kernel (kernel-space offsets only), tuned path for gfx950.
//
// One lane owns one pixel and walks the channels of its rotation group.  What
// depends only on (pixel, tap) -- the scope cell and the four bilinear
// coefficients -- is computed once and held in registers; per channel the
// lane then needs four reads from the channel's zero-padded scope tile in LDS
// and five FMAs per tap.  Consecutive lanes hold consecutive pixels, so every
// input / gradient access of a wave is one contiguous run of a plane.
//
// Reference kernels covered (K.cu =
// deformable_kernels/ops/deform_kernel/csrc/filter_sample_depthwise_cuda_kernel.cu):
//   forward        K.cu:270-386   -> local_gather_kernel<.., false>
//   grad input     K.cu:577-669   -> local_gather_kernel<.., true>
//   grad rotation  K.cu:1285-1370 -> local_grad_rotation_kernel
//   grad filter    K.cu:836-955   -> local_grad_filter_kernel + reduce_partials_kernel
#include "dk_kernels.h"

namespace dk {

namespace {

constexpr int kBlock = 256;

// Zero-padded scope table of one channel: (SH + 2) rows of (SW + 2) entries.
template <int SH, int SW>
struct Table {
  static constexpr int RS = SW + 2;
  static constexpr int SIZE = (SH + 2) * RS;
};

template <typename T, int SH, int SW>
__device__ __forceinline__ void stage_tables(float* tbl, const T* filter, int c_first, int c_step,
                                             int nch) {
  using Tb = Table<SH, SW>;
  for (int e = threadIdx.x; e < nch * Tb::SIZE; e += blockDim.x) {
    const int j = e / Tb::SIZE, r = e % Tb::SIZE;
    const int i = r / Tb::RS - 1, k = r % Tb::RS - 1;
    float v = 0.f;
    if (i >= 0 && i < SH && k >= 0 && k < SW)
      v = ld(filter + (size_t)(c_first + j * c_step) * (SH * SW) + i * SW + k);
    tbl[e] = v;
  }
}

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
// ---------------------------------------------------------------------------
template <typename T, int KH, int KW, int SH, int SW, bool TRANSPOSED>
__global__ __launch_bounds__(kBlock) void local_gather_kernel(Geo g, const T* __restrict__ src,
                                                              const T* __restrict__ rot,
                                                              const T* __restrict__ filter,
                                                              T* __restrict__ dst, int ch_per_block) {
  using Tb = Table<SH, SW>;
  constexpr int K = KH * KW;
  extern __shared__ float tbl[];

  const int n = blockIdx.z / g.groups, grp = blockIdx.z % g.groups;
  const int cpg = g.channel / g.groups;  // channels per rotation group
  const int j0 = blockIdx.y * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  stage_tables<T, SH, SW>(tbl, filter, grp + g.groups * j0, g.groups, nch);

  const int out_plane = g.out_h * g.out_w, in_plane = g.in_h * g.in_w;
  const int dst_plane = TRANSPOSED ? in_plane : out_plane;
  const int src_plane = TRANSPOSED ? out_plane : in_plane;
  const int dst_w = TRANSPOSED ? g.in_w : g.out_w;
  const int p = blockIdx.x * kBlock + threadIdx.x;
  const bool active = p < dst_plane;
  const int pc = active ? p : 0;
  const int ph = pc / dst_w, pw = pc % dst_w;

  ScopeTap<float> tap[K];
  int soff[K];
  unsigned live = 0;
  const T* rbase = rot + (size_t)(n * g.groups + grp) * (K * 2) * out_plane;
#pragma unroll
  for (int t = 0; t < K; ++t) {
    const int f_h = t / KW, f_w = t % KW;
    int rpix;
    const bool ok = tap_geometry<TRANSPOSED>(g, ph, pw, f_h, f_w, soff[t], rpix) && active;
    float r_h = 0.f, r_w = 0.f;
    if (ok) {
      r_h = ld(rbase + (size_t)(2 * t) * out_plane + rpix);
      r_w = ld(rbase + (size_t)(2 * t + 1) * out_plane + rpix);
    }
    tap[t] = make_scope_tap<float>(scope_coord<float>(f_h, r_h, g.centre_h),
                                   scope_coord<float>(f_w, r_w, g.centre_w), SH, SW, Tb::RS);
    live |= ok ? (1u << t) : 0u;
  }
  __syncthreads();
  if (!active) return;

  const size_t chan0 = (size_t)n * g.channel + grp + (size_t)g.groups * j0;
  const T* sp = src + chan0 * src_plane;
  T* dp = dst + chan0 * dst_plane + p;
  const size_t s_step = (size_t)g.groups * src_plane, d_step = (size_t)g.groups * dst_plane;
#pragma unroll 2
  for (int j = 0; j < nch; ++j) {
    const float* tb = tbl + j * Tb::SIZE;
    float acc = 0.f;
#pragma unroll
    for (int t = 0; t < K; ++t) {
      const float xv = (live >> t & 1u) ? ld(sp + soff[t]) : 0.f;
      const float* q = tb + tap[t].cell;
      const float b = tap[t].c00 * q[0] + tap[t].c01 * q[1] + tap[t].c10 * q[Tb::RS] +
                      tap[t].c11 * q[Tb::RS + 1];
      acc += xv * b;
    }
    st(dp, acc);
    sp += s_step;
    dp += d_step;
  }
}

// ---------------------------------------------------------------------------
// grad rotation: the lane owns output pixel p of (n, group) and sums over the
// group's channels.  d/dh and d/dw of the bilinear read are linear in the four
// corner weights with channel-independent coefficients, so the lane only
// accumulates  S_k[t] = sum_c x_t[c] * gout[c] * corner_k[c]  and combines the
// four sums per tap once at the end (K.cu:137-158 gives the combination).
// grid = (pixel tiles, 1, batch * groups)
// ---------------------------------------------------------------------------
template <typename T, int KH, int KW, int SH, int SW>
__global__ __launch_bounds__(kBlock) void local_grad_rotation_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ rot,
    const T* __restrict__ filter, T* __restrict__ grot, int ch_per_pass) {
  using Tb = Table<SH, SW>;
  constexpr int K = KH * KW;
  extern __shared__ float tbl[];

  const int n = blockIdx.z / g.groups, grp = blockIdx.z % g.groups;
  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = g.in_h * g.in_w;
  const int p = blockIdx.x * kBlock + threadIdx.x;
  const bool active = p < out_plane;
  const int pc = active ? p : 0;
  const int ph = pc / g.out_w, pw = pc % g.out_w;

  int cell[K], soff[K];
  float lh[K], lw[K];
  unsigned live = 0, inside = 0;
  const size_t rplane0 = (size_t)(n * g.groups + grp) * (K * 2) * out_plane;
#pragma unroll
  for (int t = 0; t < K; ++t) {
    const int f_h = t / KW, f_w = t % KW;
    int rpix;
    const bool ok = tap_geometry<false>(g, ph, pw, f_h, f_w, soff[t], rpix) && active;
    float r_h = 0.f, r_w = 0.f;
    if (active) {
      r_h = ld(rot + rplane0 + (size_t)(2 * t) * out_plane + pc);
      r_w = ld(rot + rplane0 + (size_t)(2 * t + 1) * out_plane + pc);
    }
    const float h = scope_coord<float>(f_h, r_h, g.centre_h);
    const float w = scope_coord<float>(f_w, r_w, g.centre_w);
    const bool in = (h > -1.f) && (w > -1.f) && (h < float(SH)) && (w < float(SW));
    const float hf = floorf(h), wf = floorf(w);
    lh[t] = h - hf;
    lw[t] = w - wf;
    cell[t] = in ? (static_cast<int>(hf) + 1) * Tb::RS + static_cast<int>(wf) + 1 : 0;
    live |= ok ? (1u << t) : 0u;
    inside |= (in && ok) ? (1u << t) : 0u;
  }

  float s00[K], s01[K], s10[K], s11[K];
#pragma unroll
  for (int t = 0; t < K; ++t) s00[t] = s01[t] = s10[t] = s11[t] = 0.f;

  for (int j0 = 0; j0 < cpg; j0 += ch_per_pass) {
    const int nch = min(ch_per_pass, cpg - j0);
    __syncthreads();
    stage_tables<T, SH, SW>(tbl, filter, grp + g.groups * j0, g.groups, nch);
    __syncthreads();
    if (active) {
      const size_t chan0 = (size_t)n * g.channel + grp + (size_t)g.groups * j0;
      const T* xp = x + chan0 * in_plane;
      const T* gp = gout + chan0 * out_plane + p;
#pragma unroll 2
      for (int j = 0; j < nch; ++j) {
        const float* tb = tbl + j * Tb::SIZE;
        const float go = ld(gp);
#pragma unroll
        for (int t = 0; t < K; ++t) {
          const float xv = (live >> t & 1u) ? ld(xp + soff[t]) : 0.f;
          const float ps = xv * go;
          const float* q = tb + cell[t];
          s00[t] += ps * q[0];
          s01[t] += ps * q[1];
          s10[t] += ps * q[Tb::RS];
          s11[t] += ps * q[Tb::RS + 1];
        }
        xp += (size_t)g.groups * in_plane;
        gp += (size_t)g.groups * out_plane;
      }
    }
  }
  if (!active) return;
#pragma unroll
  for (int t = 0; t < K; ++t) {
    const float hh = 1.f - lh[t], hw = 1.f - lw[t];
    float gh = hw * (s10[t] - s00[t]) + lw[t] * (s11[t] - s01[t]);
    float gw = hh * (s01[t] - s00[t]) + lh[t] * (s11[t] - s10[t]);
    if (!(inside >> t & 1u)) gh = gw = 0.f;
    st(grot + rplane0 + (size_t)(2 * t) * out_plane + p, gh);
    st(grot + rplane0 + (size_t)(2 * t + 1) * out_plane + p, gw);
  }
}

// ---------------------------------------------------------------------------
// grad filter: a workgroup owns CCH channels of one rotation group and walks
// (image, pixel tile) work items.  Contributions x_t * gout * coef_k go into an
// LDS accumulator of the padded table shape, replicated 32 times with the
// replica chosen by lane id so that a wave's 64 adds fall on 32 distinct banks
// whatever cells they address.  Each workgroup finally writes one partial
// [CCH][SH*SW] to the workspace; reduce_partials_kernel sums the partials in a
// fixed order.  No global atomics.
// grid = (parts, channel chunks, groups)
// ---------------------------------------------------------------------------
constexpr int kRep = 32;

template <typename T, int KH, int KW, int SH, int SW, int CCH>
__global__ __launch_bounds__(kBlock) void local_grad_filter_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ rot,
    float* __restrict__ partial, int tiles) {
  using Tb = Table<SH, SW>;
  constexpr int K = KH * KW;
  __shared__ float acc[CCH * Tb::SIZE * kRep];

  for (int e = threadIdx.x; e < CCH * Tb::SIZE * kRep; e += kBlock) acc[e] = 0.f;
  __syncthreads();

  const int grp = blockIdx.z;
  const int cpg = g.channel / g.groups;
  const int j0 = blockIdx.y * CCH;
  const int nch = min(CCH, cpg - j0);
  const int out_plane = g.out_h * g.out_w, in_plane = g.in_h * g.in_w;
  const int rep = threadIdx.x & (kRep - 1);
  const int items = g.batch * tiles;

  for (int item = blockIdx.x; item < items; item += gridDim.x) {
    const int n = item / tiles, tile = item % tiles;
    const int p = tile * kBlock + threadIdx.x;
    if (p >= out_plane) continue;
    const int ph = p / g.out_w, pw = p % g.out_w;

    ScopeTap<float> tap[K];
    int soff[K];
    unsigned live = 0;
    const T* rbase = rot + (size_t)(n * g.groups + grp) * (K * 2) * out_plane + p;
#pragma unroll
    for (int t = 0; t < K; ++t) {
      const int f_h = t / KW, f_w = t % KW;
      int rpix;
      const bool ok = tap_geometry<false>(g, ph, pw, f_h, f_w, soff[t], rpix);
      float r_h = 0.f, r_w = 0.f;
      if (ok) {
        r_h = ld(rbase + (size_t)(2 * t) * out_plane);
        r_w = ld(rbase + (size_t)(2 * t + 1) * out_plane);
      }
      tap[t] = make_scope_tap<float>(scope_coord<float>(f_h, r_h, g.centre_h),
                                     scope_coord<float>(f_w, r_w, g.centre_w), SH, SW, Tb::RS);
      live |= ok ? (1u << t) : 0u;
    }

    const size_t chan0 = (size_t)n * g.channel + grp + (size_t)g.groups * j0;
    const T* xp = x + chan0 * in_plane;
    const T* gp = gout + chan0 * out_plane + p;
    for (int j = 0; j < nch; ++j) {
      const float go = ld(gp);
      float* a = acc + (j * Tb::SIZE) * kRep + rep;
#pragma unroll
      for (int t = 0; t < K; ++t) {
        if (live >> t & 1u) {
          const float ps = ld(xp + soff[t]) * go;
          float* q = a + tap[t].cell * kRep;
          atomicAdd(q, ps * tap[t].c00);
          atomicAdd(q + kRep, ps * tap[t].c01);
          atomicAdd(q + Tb::RS * kRep, ps * tap[t].c10);
          atomicAdd(q + (Tb::RS + 1) * kRep, ps * tap[t].c11);
        }
      }
      xp += (size_t)g.groups * in_plane;
      gp += (size_t)g.groups * out_plane;
    }
  }
  __syncthreads();

  // fold the replicas; lane-rotated start keeps the 32 reads of a step on 32 banks
  for (int e = threadIdx.x; e < nch * SH * SW; e += kBlock) {
    const int j = e / (SH * SW), r = e % (SH * SW);
    const int i = r / SW, k = r % SW;
    const float* a = acc + (j * Tb::SIZE + (i + 1) * Tb::RS + (k + 1)) * kRep;
    float s = 0.f;
    for (int q = 0; q < kRep; ++q) s += a[(q + threadIdx.x) & (kRep - 1)];
    const int c = grp + g.groups * (j0 + j);
    partial[((size_t)blockIdx.x * g.channel + c) * (SH * SW) + r] = s;
  }
}

}  // namespace

// out[e] = sum over parts of partial[part][e], in part order.
template <typename CT, typename T>
__global__ void reduce_partials_kernel(const CT* __restrict__ partial, int parts, int count,
                                       T* __restrict__ out) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= count) return;
  CT s = 0;
  for (int q = 0; q < parts; ++q) s += partial[(size_t)q * count + e];
  st(out + e, s);
}

template <typename CT, typename T>
void launch_reduce_partials(const CT* partial, int parts, int count, T* out, hipStream_t stream) {
  reduce_partials_kernel<CT, T><<<ceil_div(count, 256), 256, 0, stream>>>(partial, parts, count, out);
}
template void launch_reduce_partials<float, float>(const float*, int, int, float*, hipStream_t);
template void launch_reduce_partials<float, __half>(const float*, int, int, __half*, hipStream_t);
template void launch_reduce_partials<float, bf16_t>(const float*, int, int, bf16_t*, hipStream_t);
template void launch_reduce_partials<double, double>(const double*, int, int, double*, hipStream_t);

// ---------------------------------------------------------------------------
// host-side dispatch of the tuned path
// ---------------------------------------------------------------------------
namespace {

constexpr int kFilterCch = 8;        // channels per grad-filter workgroup
constexpr int kMaxLdsTables = 96 * 1024;  // bytes of LDS a workgroup may spend on scope tables

template <int SH, int SW>
int channels_per_block(int cpg, int wanted_splits) {
  const int fit = kMaxLdsTables / (Table<SH, SW>::SIZE * 4);
  int per = ceil_div(cpg, wanted_splits);
  if (per > fit) per = fit;
  if (per < 1) per = 1;
  return per;
}

// How many channel splits give the forward / grad-input grid enough waves to fill 256 CUs.
int pick_splits(const Geo& g, int planes_pixels) {
  const long waves = (long)ceil_div(planes_pixels, kBlock) * (kBlock / 64) * g.batch * g.groups;
  const int cpg = g.channel / g.groups;
  int splits = 1;
  while (waves * splits < 8192 && cpg / (splits * 2) >= 16) splits *= 2;
  return splits;
}

template <typename T, int SH, int SW>
bool run_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                hipStream_t stream) {
  const int cpg = g.channel / g.groups;
  const int pixels = transposed ? g.in_h * g.in_w : g.out_h * g.out_w;
  const int per = channels_per_block<SH, SW>(cpg, pick_splits(g, pixels));
  const dim3 grid(ceil_div(pixels, kBlock), ceil_div(cpg, per), g.batch * g.groups);
  const size_t lds = (size_t)per * Table<SH, SW>::SIZE * sizeof(float);
  if (transposed)
    local_gather_kernel<T, 3, 3, SH, SW, true><<<grid, kBlock, lds, stream>>>(g, src, rot, filter, dst, per);
  else
    local_gather_kernel<T, 3, 3, SH, SW, false><<<grid, kBlock, lds, stream>>>(g, src, rot, filter, dst, per);
  return true;
}

template <typename T, int SH, int SW>
bool run_grad_rotation(const Geo& g, const T* gout, const T* x, const T* rot, const T* filter,
                       T* grot, hipStream_t stream) {
  const int cpg = g.channel / g.groups;
  const int per = channels_per_block<SH, SW>(cpg, 1);
  const dim3 grid(ceil_div(g.out_h * g.out_w, kBlock), 1, g.batch * g.groups);
  const size_t lds = (size_t)per * Table<SH, SW>::SIZE * sizeof(float);
  local_grad_rotation_kernel<T, 3, 3, SH, SW><<<grid, kBlock, lds, stream>>>(g, gout, x, rot, filter, grot, per);
  return true;
}

int filter_parts(const Geo& g) {
  const int tiles = ceil_div(g.out_h * g.out_w, kBlock);
  const int items = g.batch * tiles;
  const int chunks = ceil_div(g.channel / g.groups, kFilterCch) * g.groups;
  int parts = ceil_div(2048, chunks);  // ~8 workgroups per CU in total
  if (parts > items) parts = items;
  if (parts < 1) parts = 1;
  return parts;
}

template <typename T, int SH, int SW>
bool run_grad_filter(const Geo& g, const T* gout, const T* x, const T* rot, T* gfilter, float* ws,
                     hipStream_t stream) {
  const int tiles = ceil_div(g.out_h * g.out_w, kBlock);
  const int parts = filter_parts(g);
  const dim3 grid(parts, ceil_div(g.channel / g.groups, kFilterCch), g.groups);
  local_grad_filter_kernel<T, 3, 3, SH, SW, kFilterCch><<<grid, kBlock, 0, stream>>>(g, gout, x, rot, ws, tiles);
  launch_reduce_partials<float, T>(ws, parts, g.channel * SH * SW, gfilter, stream);
  return true;
}

bool fast_shape(const Geo& g) {
  return g.k_h == 3 && g.k_w == 3 && (long)g.batch * g.groups <= 65535 &&
         ((g.scope_h == 4 && g.scope_w == 4) || (g.scope_h == 3 && g.scope_w == 3) ||
          (g.scope_h == 5 && g.scope_w == 5));
}

}  // namespace

#define DK_DISPATCH_SCOPE(g, CALL)                                   \
  if ((g).scope_h == 4) return CALL(4, 4);                           \
  if ((g).scope_h == 3) return CALL(3, 3);                           \
  return CALL(5, 5);

template <typename T>
bool fast_local_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter,
                       T* dst, hipStream_t stream) {
  if (!fast_shape(g)) return false;
#define CALL(SH, SW) run_gather<T, SH, SW>(g, transposed, src, rot, filter, dst, stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

template <typename T>
bool fast_local_grad_rotation(const Geo& g, const T* gout, const T* x, const T* rot,
                              const T* filter, T* grot, hipStream_t stream) {
  if (!fast_shape(g)) return false;
#define CALL(SH, SW) run_grad_rotation<T, SH, SW>(g, gout, x, rot, filter, grot, stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

size_t fast_local_grad_filter_workspace(const Geo& g) {
  if (!fast_shape(g)) return 0;
  return (size_t)filter_parts(g) * g.channel * g.scope_h * g.scope_w * sizeof(float);
}

template <typename T>
bool fast_local_grad_filter(const Geo& g, const T* gout, const T* x, const T* rot, T* gfilter,
                            void* ws, hipStream_t stream) {
  if (!fast_shape(g)) return false;
#define CALL(SH, SW) run_grad_filter<T, SH, SW>(g, gout, x, rot, gfilter, static_cast<float*>(ws), stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

#define DK_INSTANTIATE(T)                                                                           \
  template bool fast_local_gather<T>(const Geo&, bool, const T*, const T*, const T*, T*, hipStream_t); \
  template bool fast_local_grad_rotation<T>(const Geo&, const T*, const T*, const T*, const T*, T*,  \
                                            hipStream_t);                                           \
  template bool fast_local_grad_filter<T>(const Geo&, const T*, const T*, const T*, T*, void*,      \
                                          hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
#undef DK_INSTANTIATE

}  // namespace dk
