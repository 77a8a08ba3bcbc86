// Tuned gfx950 kernels of the DEFORMABLE variant (the input taps are themselves sampled
// bilinearly at image-space offsets) for 3x3 taps, scope 3x3 / 4x4 / 5x5, fp32 / fp16 / bf16,
// input planes up to 64 columns wide that fit LDS.  Everything else runs on dk_generic.hip.
//
// Reference kernels covered (K.cu =
// deformable_kernels/ops/deform_kernel/csrc/filter_sample_depthwise_cuda_kernel.cu):
//   forward        K.cu:433-528   -> deform_forward_kernel
//   grad input     K.cu:704-795   -> deform_grad_input_kernel
//   grad offset    K.cu:1147-1243 -> deform_grad_coord_kernel<.., OFFSET>
//   grad rotation  K.cu:1410-1508 -> deform_grad_coord_kernel<.., ROTATION>
//   grad filter    K.cu:1002-1097 -> deform_grad_filter_kernel
//
// Common structure: a lane owns an output pixel and walks the channels of a chunk.  What depends
// only on (pixel, tap) -- where the tap samples the image and the scope tile -- is computed once
// per lane.  The reference gathers the four image corners of every (pixel, tap, channel) from
// global memory; here the workgroup stages each channel's input plane in LDS, ZERO-PADDED by one
// element on every side, so that a sample anywhere in the open box (-1, H) x (-1, W) reads its four
// corners at idx, idx + 1, idx + RS, idx + RS + 1 with no range tests (K.cu:182-193 tests each
// corner).  Planes are double buffered: the next channel's plane is loaded into registers before
// the current channel is computed and written to the other buffer afterwards (one barrier per
// channel).  The scope tiles of the chunk sit in LDS in the corner-expanded difference form.
#include <algorithm>
#include <cstdlib>

#include "dk_kernels.h"
#include "dk_scope_table.h"

namespace dk {

namespace {

constexpr int kDBlock = 256;
constexpr int K9 = 9;

// Where tap t of the lane's pixel samples the padded image plane: index of the top-left corner
// and the fractional position.  A sample outside (-1, H) x (-1, W) (K.cu:500), or a lane without
// a pixel, points at the padding corner with lh = lw = 0 and so reads 0.
struct ImgTap {
  int pidx;
  float lh, lw;
};

template <typename T, int SH, int SW>
__device__ __forceinline__ void deform_taps(const Geo& g, const T* off, const T* rot, int n, int grp, int p,
                                            bool live, int RS, ImgTap (&it)[K9], LiteTap (&st)[K9]) {
  const int out_plane = g.out_h * g.out_w;
  const int pc = live ? p : 0;
  const int oh = pc / g.out_w, ow = pc % g.out_w;
  const rsrc_t ro = plane_rsrc(off + (size_t)n * (K9 * 2) * out_plane, K9 * 2 * out_plane);
  const rsrc_t rr = plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K9 * 2) * out_plane, K9 * 2 * out_plane);
  const unsigned step = (unsigned)out_plane * (unsigned)sizeof(T);
#pragma unroll
  for (int t = 0; t < K9; ++t) {
    const int f_h = t / 3, f_w = t % 3;
    const unsigned o = live ? (unsigned)((2 * t) * out_plane + pc) * (unsigned)sizeof(T) : kOutOfRange;
    // K.cu:486-499: tap position plus the learned offset
    const float h = float(oh * g.stride_h - g.pad_h + f_h * g.dil_h) + buf_ld(ro, o, off);
    const float w = float(ow * g.stride_w - g.pad_w + f_w * g.dil_w) + buf_ld(ro, o + step, off);
    const bool hit = live && (h > -1.f) && (w > -1.f) && (h < float(g.in_h)) && (w < float(g.in_w));
    const float hf = floorf(h), wf = floorf(w);
    it[t].pidx = hit ? (static_cast<int>(hf) + 1) * RS + static_cast<int>(wf) + 1 : 0;
    it[t].lh = hit ? h - hf : 0.f;
    it[t].lw = hit ? w - wf : 0.f;
    st[t] = make_lite_tap<SH, SW>(scope_coord<float>(f_h, buf_ld(rr, o, rot), g.centre_h),
                                  scope_coord<float>(f_w, buf_ld(rr, o + step, rot), g.centre_w), hit);
  }
}

// The four corners of a sample in the padded plane, and their bilinear combination.
struct Corners {
  float a, b, c, d;  // top-left, top-right, bottom-left, bottom-right
};
__device__ __forceinline__ Corners read_corners(const float* plane, int pidx, int RS) {
  Corners q;
  q.a = plane[pidx];
  q.b = plane[pidx + 1];
  q.c = plane[pidx + RS];
  q.d = plane[pidx + RS + 1];
  return q;
}
__device__ __forceinline__ float lerp2(const Corners& q, float lh, float lw) {
  const float top = fmaf(lw, q.b - q.a, q.a), bot = fmaf(lw, q.d - q.c, q.c);
  return fmaf(lh, bot - top, top);
}

// Cooperative load of one H x W plane into the padded LDS layout.  A row takes 2^shift lanes
// (the smallest power of two >= W), so a thread's (row, column) needs no division; NPASS passes
// of blockDim / 2^shift rows cover the plane.  load() fills the register stage, store() writes it.
template <typename T, int NPASS>
struct PlaneStage {
  float v[NPASS];
  __device__ __forceinline__ void load(const T* plane, bool on, int H, int W, int shift) {
    const int col = threadIdx.x & ((1 << shift) - 1), sub = threadIdx.x >> shift;
    const int rpp = (int)blockDim.x >> shift;
    const rsrc_t r = plane_rsrc(plane, on ? H * W : 0);
#pragma unroll
    for (int k = 0; k < NPASS; ++k) {
      const int row = k * rpp + sub;
      v[k] = buf_ld(r, (col < W && row < H) ? (unsigned)(row * W + col) * (unsigned)sizeof(T) : kOutOfRange, plane);
    }
  }
  __device__ __forceinline__ void store(float* lds_plane, int H, int W, int shift) const {
    const int col = threadIdx.x & ((1 << shift) - 1), sub = threadIdx.x >> shift;
    const int rpp = (int)blockDim.x >> shift;
    const int RS = W + 2;
#pragma unroll
    for (int k = 0; k < NPASS; ++k) {
      const int row = k * rpp + sub;
      if (col < W && row < H) lds_plane[(row + 1) * RS + 1 + col] = v[k];
    }
  }
};

// logical block = (pixel tile, channel chunk, image * group), tile fastest (see logical_block())
struct BlockId {
  int tile, chunk, n, grp;
  bool valid;
};
__device__ __forceinline__ BlockId decode_block(const Geo& g, int tiles, int chunks) {
  BlockId b;
  const int total = tiles * chunks * g.batch * g.groups;
  const int lb = logical_block(total);
  b.valid = lb < total;
  b.tile = lb % tiles;
  b.chunk = lb / tiles % chunks;
  const int z = lb / tiles / chunks;
  b.n = z / g.groups;
  b.grp = z % g.groups;
  return b;
}

// ---------------------------------------------------------------------------
// forward: out[n, c, p] = sum_t sample(x[n, c], h_t, w_t) * B(Wt[c], sh_t, sw_t)
// ---------------------------------------------------------------------------
template <typename T, int SH, int SW, int NPASS>
__global__ __launch_bounds__(kDBlock, 2) void deform_forward_kernel(
    Geo g, const T* __restrict__ x, const T* __restrict__ off, const T* __restrict__ rot,
    const T* __restrict__ filter, T* __restrict__ out, int ch_per_block, int shift) {
  using Tb = WideTable<SH, SW>;
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int PS = ((H + 2) * RS + 3) & ~3;
  float* planes = lds;           // [2][PS]
  float* tbl = lds + 2 * PS;     // [ch_per_block][Tb::SIZE]

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const BlockId b = decode_block(g, ceil_div(out_plane, kDBlock), ceil_div(cpg, ch_per_block));
  if (!b.valid) return;
  const int j0 = b.chunk * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);

  for (int e = threadIdx.x; e < 2 * PS; e += kDBlock) planes[e] = 0.f;
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, b.grp + g.groups * j0, g.groups, nch);

  const int p = b.tile * kDBlock + threadIdx.x;
  const bool live = p < out_plane;
  ImgTap it[K9];
  LiteTap st[K9];
  deform_taps<T, SH, SW>(g, off, rot, b.n, b.grp, p, live, RS, it, st);

  const size_t chan0 = (size_t)b.n * g.channel + b.grp + (size_t)g.groups * j0;
  const T* xp = x + chan0 * in_plane;
  T* op = out + chan0 * out_plane;
  const size_t x_step = (size_t)g.groups * in_plane, o_step = (size_t)g.groups * out_plane;
  const unsigned ooff = live ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  PlaneStage<T, NPASS> stage;
  stage.load(xp, true, H, W, shift);
  __syncthreads();  // the zero fill is done
  stage.store(planes, H, W, shift);
  __syncthreads();
  for (int j = 0; j < nch; ++j) {
    if (j + 1 < nch) stage.load(xp + (size_t)(j + 1) * x_step, true, H, W, shift);
    const float* pl = planes + (j & 1) * PS;
    const float* tb = tbl + j * Tb::SIZE;
    float acc = 0.f;
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      const float v = lerp2(read_corners(pl, it[t].pidx, RS), it[t].lh, it[t].lw);
      const float4 q = *reinterpret_cast<const float4*>(tb + st[t].cell);
      acc = fmaf(v, lite_weight(st[t], q), acc);
    }
    buf_st(plane_rsrc(op + (size_t)j * o_step, out_plane), ooff, acc, out);
    if (j + 1 < nch) stage.store(planes + ((j + 1) & 1) * PS, H, W, shift);
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct DeformPlan {
  bool ok;
  int shift;   // log2 of the lanes a plane row takes
  int npass;   // register stage size: 4, 8 or 16
  int PS;      // floats of a padded plane
  int per;     // channels per block
  int chunks;  // channel chunks per group
  int tiles;   // pixel tiles
  size_t lds;
};

// table_floats: LDS floats per channel beyond the two planes; plane_floats: LDS floats per plane
DeformPlan deform_plan(const Geo& g, int table_floats, int planes, int block) {
  DeformPlan d{};
  d.ok = false;
  if (getenv("DK_NO_DEFORM_FAST")) return d;
  if (g.k_h != 3 || g.k_w != 3 || g.in_w > 64) return d;
  if (!((g.scope_h == 3 && g.scope_w == 3) || (g.scope_h == 4 && g.scope_w == 4) ||
        (g.scope_h == 5 && g.scope_w == 5)))
    return d;
  if ((long)g.out_h * g.out_w * 18 * 4 >= (1L << 31)) return d;
  d.shift = 0;
  while ((1 << d.shift) < g.in_w) ++d.shift;
  const int rpp = block >> d.shift;
  const int np = ceil_div(g.in_h, rpp);
  if (np > 16) return d;
  d.npass = np <= 4 ? 4 : np <= 8 ? 8 : 16;
  d.PS = ((g.in_h + 2) * (g.in_w + 2) + 3) & ~3;
  const int cpg = g.channel / g.groups;
  d.tiles = ceil_div(g.out_h * g.out_w, block);
  const long plane_bytes = (long)planes * d.PS * 4;
  const long room = 64 * 1024 - plane_bytes;
  if (room < (long)table_floats * 4 * 4) return d;
  const int fit = (int)std::min<long>(room / ((long)table_floats * 4), cpg);
  // enough blocks for two per CU, chunks of at least 8 channels
  const long base = (long)d.tiles * g.batch * g.groups;
  int chunks = (int)std::max<long>(1, (2 * 256 + base - 1) / base);
  chunks = std::min(chunks, std::max(1, cpg / 8));
  chunks = std::max(chunks, ceil_div(cpg, fit));
  d.per = ceil_div(cpg, chunks);
  d.chunks = ceil_div(cpg, d.per);
  d.lds = (size_t)plane_bytes + (size_t)d.per * table_floats * 4;
  if ((long)d.tiles * d.chunks * g.batch * g.groups >= (1L << 31) - 8) return d;
  d.ok = true;
  return d;
}

template <typename T, int SH, int SW>
bool run_deform_forward(const Geo& g, const T* x, const T* off, const T* rot, const T* filter, T* out,
                        hipStream_t stream) {
  const DeformPlan d = deform_plan(g, WideTable<SH, SW>::SIZE, 2, kDBlock);
  if (!d.ok) return false;
  const unsigned grid = (unsigned)xcd_grid_size((long)d.tiles * d.chunks * g.batch * g.groups);
#define DK_LAUNCH(NP) \
  deform_forward_kernel<T, SH, SW, NP><<<grid, kDBlock, d.lds, stream>>>(g, x, off, rot, filter, out, d.per, d.shift)
  if (d.npass == 4) DK_LAUNCH(4);
  else if (d.npass == 8) DK_LAUNCH(8);
  else DK_LAUNCH(16);
#undef DK_LAUNCH
  return true;
}

}  // namespace

#define DK_DISPATCH_SCOPE(g, CALL)    \
  if ((g).scope_h == 4) return CALL(4, 4); \
  if ((g).scope_h == 3) return CALL(3, 3); \
  if ((g).scope_h == 5) return CALL(5, 5); \
  return false;

template <typename T>
bool fast_deform_forward(const Geo& g, const T* x, const T* off, const T* rot, const T* filter, T* out,
                         hipStream_t stream) {
#define CALL(SH, SW) run_deform_forward<T, SH, SW>(g, x, off, rot, filter, out, stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

#define DK_INSTANTIATE(T)                                                                              \
  template bool fast_deform_forward<T>(const Geo&, const T*, const T*, const T*, const T*, T*, hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
#undef DK_INSTANTIATE

}  // namespace dk
