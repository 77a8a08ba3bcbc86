// Tuned gfx950 kernels of the DEFORMABLE variant (the input taps are themselves sampled
// bilinearly at image-space offsets) for 3x3 taps, scope 3x3 / 4x4 / 5x5, fp32 / fp16 / bf16,
// input planes whose zero-padded copy fits LDS twice (up to about 130 x 130 in a workgroup of its own).
// Everything else runs on dk_generic.hip.
//
// Reference kernels covered (K.cu =
// deformable_kernels/ops/deform_kernel/csrc/filter_sample_depthwise_cuda_kernel.cu):
//   forward        K.cu:433-528   -> deform_forward_ch_kernel | deform_forward_kernel
//   grad input     K.cu:704-795   -> deform_grad_input_kernel | deform_grad_input_tiled_kernel
//   grad offset    K.cu:1147-1243 -> deform_grad_coord_ch_kernel | deform_grad_coord_kernel <.., OFFSET>
//   grad rotation  K.cu:1410-1508 -> deform_grad_coord_ch_kernel | deform_grad_coord_kernel <.., ROTATION>
//   grad filter    K.cu:1002-1097 -> deform_grad_filter_mfma_kernel | deform_grad_filter_kernel
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
// Forward, grad offset and grad rotation interleave four channel planes, element e of channel c at
// [e][c]: the corner gathers at per-lane addresses bound these kernels, and one 16-byte read per
// corner then serves four channels.  Planes up to about 30 x 30 run that form in workgroups of 256
// threads, several per CU; larger ones (up to 64 x 64) in one workgroup of 1024 threads per CU that
// takes most of the CU's LDS for the two interleaved buffers.  Wider or taller planes (112 x 112) run the
// one-plane forms of forward, the coordinate gradients and grad filter in workgroups of 512 threads that
// stage only the plane rows the tile's samples touch, and grad input with fewer planes per workgroup.
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

// Scope coordinates of tap t; (-2, -2), outside every scope band, where the tap samples nothing.
struct ScopeCoord {
  float h, w;
};

template <typename T>
__device__ __forceinline__ void deform_taps(const Geo& g, const T* off, const T* rot, int n, int grp, int p,
                                            bool live, int RS, ImgTap (&it)[K9], ScopeCoord (&sc)[K9],
                                            unsigned* hits = nullptr) {
  const int out_plane = g.out_h * g.out_w;
  const int pc = live ? p : 0;
  const int oh = pc / g.out_w, ow = pc % g.out_w;
  const rsrc_t ro = plane_rsrc(off + (size_t)n * (K9 * 2) * out_plane, K9 * 2 * out_plane);
  // no rotation tensor (the caller's offsets in kernel space are all zero): a resource of no bytes reads as zeros
  const rsrc_t rr = rot ? plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K9 * 2) * out_plane, K9 * 2 * out_plane)
                        : plane_rsrc(rot, 0);
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
    const float sh = scope_coord<float>(g, f_h, buf_ld(rr, o, rot), g.centre_h);
    const float sw = scope_coord<float>(g, f_w, buf_ld(rr, o + step, rot), g.centre_w);
    sc[t].h = hit ? sh : -2.f;
    sc[t].w = hit ? sw : -2.f;
    if (hits) *hits |= hit ? (1u << t) : 0u;  // bit t: tap t samples the image
  }
}

template <typename T, int SH, int SW>
__device__ __forceinline__ void deform_taps(const Geo& g, const T* off, const T* rot, int n, int grp, int p,
                                            bool live, int RS, ImgTap (&it)[K9], LiteTap (&st)[K9],
                                            unsigned* hits = nullptr) {
  ScopeCoord sc[K9];
  deform_taps<T>(g, off, rot, n, grp, p, live, RS, it, sc, hits);
#pragma unroll
  for (int t = 0; t < K9; ++t) st[t] = make_lite_tap<SH, SW>(sc[t].h, sc[t].w, true);
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
// WINDOW: only the plane rows row0 .. row0 + nrows - 1 are staged, in as many passes as they take
// (the LDS layout stays that of the whole plane: rows outside the window keep what they held).
struct RowWindow {
  int row0, nrows;
};
template <typename T, int NPASS>
struct PlaneStage {
  float v[NPASS];
  template <bool WINDOW = false>
  __device__ __forceinline__ void load(const T* plane, bool on, int H, int W, int shift, RowWindow rw = RowWindow{0, 0}) {
    const int col = threadIdx.x & ((1 << shift) - 1), sub = threadIdx.x >> shift;
    const int rpp = (int)blockDim.x >> shift;
    const rsrc_t r = plane_rsrc(plane, on ? H * W : 0);
#pragma unroll
    for (int k = 0; k < NPASS; ++k) {
      const int row = k * rpp + sub;
      if constexpr (WINDOW) {
        if (k * rpp < rw.nrows)  // uniform
          v[k] = buf_ld(r, (col < W && row < rw.nrows) ? (unsigned)((rw.row0 + row) * W + col) * (unsigned)sizeof(T) : kOutOfRange, plane);
      } else {
        v[k] = buf_ld(r, (col < W && row < H) ? (unsigned)(row * W + col) * (unsigned)sizeof(T) : kOutOfRange, plane);
      }
    }
  }
  template <bool WINDOW = false>
  __device__ __forceinline__ void store(float* lds_plane, int H, int W, int shift, RowWindow rw = RowWindow{0, 0}) const {
    const int col = threadIdx.x & ((1 << shift) - 1), sub = threadIdx.x >> shift;
    const int rpp = (int)blockDim.x >> shift;
    const int RS = W + 2;
#pragma unroll
    for (int k = 0; k < NPASS; ++k) {
      const int row = k * rpp + sub;
      if constexpr (WINDOW) {
        if (k * rpp < rw.nrows)
          if (col < W && row < rw.nrows) lds_plane[(rw.row0 + row + 1) * RS + 1 + col] = v[k];
      } else {
        if (col < W && row < H) lds_plane[(row + 1) * RS + 1 + col] = v[k];
      }
    }
  }
};

// The rows of the input plane that the workgroup's samples read: the taps' descriptors point at
// the top-left corner in the padded plane (row r of the plane is padded row r + 1), a sample reads
// that padded row and the next.  Two barriers; every thread of the workgroup must call it.
__device__ __forceinline__ RowWindow sample_rows(const ImgTap (&it)[K9], unsigned hits, int RS, int H) {
  __shared__ int s_lo[16], s_hi[16];
  int lo = H + 2, hi = -1;  // padded rows
#pragma unroll
  for (int t = 0; t < K9; ++t) {
    if (hits >> t & 1u) {
      const int pr = it[t].pidx / RS;
      lo = min(lo, pr);
      hi = max(hi, pr + 1);
    }
  }
  for (int s = 32; s > 0; s >>= 1) {
    lo = min(lo, __shfl_xor(lo, s));
    hi = max(hi, __shfl_xor(hi, s));
  }
  if ((threadIdx.x & 63) == 0) {
    s_lo[threadIdx.x >> 6] = lo;
    s_hi[threadIdx.x >> 6] = hi;
  }
  __syncthreads();
  for (int w = 0; w < (int)blockDim.x / 64; ++w) {
    lo = min(lo, s_lo[w]);
    hi = max(hi, s_hi[w]);
  }
  __syncthreads();
  const int first = max(lo - 1, 0), last = min(hi - 1, H - 1);
  return RowWindow{first, max(last - first + 1, 0)};
}

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
// BLOCK > kDBlock: the form for planes that the others do not take (wider than 64 columns, or taller than their
// staging passes cover): one workgroup per CU, and only the plane rows that the tile's samples touch are staged.
template <typename T, int SH, int SW, int NPASS, int BLOCK = kDBlock>
__global__ __launch_bounds__(BLOCK, 2) void deform_forward_kernel(
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
  const BlockId b = decode_block(g, ceil_div(out_plane, BLOCK), ceil_div(cpg, ch_per_block));
  if (!b.valid) return;
  const int j0 = b.chunk * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);

  for (int e = threadIdx.x; e < 2 * PS; e += BLOCK) planes[e] = 0.f;
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, b.grp + g.groups * j0, g.groups, nch);

  const int p = b.tile * BLOCK + threadIdx.x;
  const bool live = p < out_plane;
  ImgTap it[K9];
  LiteTap st[K9];
  constexpr bool WINDOW = BLOCK != kDBlock;
  unsigned hits = 0;
  deform_taps<T, SH, SW>(g, off, rot, b.n, b.grp, p, live, RS, it, st, &hits);
  RowWindow rw{0, H};
  if constexpr (WINDOW) rw = sample_rows(it, hits, RS, H);

  const size_t chan0 = (size_t)b.n * g.channel + b.grp + (size_t)g.groups * j0;
  const T* xp = x + chan0 * in_plane;
  T* op = out + chan0 * out_plane;
  const size_t x_step = (size_t)g.groups * in_plane, o_step = (size_t)g.groups * out_plane;
  const unsigned ooff = live ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  PlaneStage<T, NPASS> stage;
  stage.template load<WINDOW>(xp, true, H, W, shift, rw);
  __syncthreads();  // the zero fill is done
  stage.template store<WINDOW>(planes, H, W, shift, rw);
  __syncthreads();
  for (int j = 0; j < nch; ++j) {
    if (j + 1 < nch) stage.template load<WINDOW>(xp + (size_t)(j + 1) * x_step, true, H, W, shift, rw);
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
    if (j + 1 < nch) stage.template store<WINDOW>(planes + ((j + 1) & 1) * PS, H, W, shift, rw);
    __syncthreads();
  }
}

// The same with CH channel planes interleaved in LDS, element e of channel c at [e][c]: a corner
// of a sample is one 16-byte read for CH = 4 channels instead of four 4-byte reads, and the
// gathers at per-lane addresses are what bounds these kernels.
template <typename T, int NPASS, int CH>
struct PlaneStageN {
  float v[CH][NPASS];
  __device__ __forceinline__ void load(const T* plane0, size_t step, int live_channels, int H, int W, int shift) {
    const int col = threadIdx.x & ((1 << shift) - 1), sub = threadIdx.x >> shift;
    const int rpp = (int)blockDim.x >> shift;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const bool on = c < live_channels;
      const rsrc_t r = plane_rsrc(plane0 + (on ? (size_t)c * step : 0), on ? H * W : 0);
#pragma unroll
      for (int k = 0; k < NPASS; ++k) {
        const int row = k * rpp + sub;
        v[c][k] = buf_ld(r, (col < W && row < H) ? (unsigned)(row * W + col) * (unsigned)sizeof(T) : kOutOfRange, plane0);
      }
    }
  }
  __device__ __forceinline__ void store(float* lds_planes, int H, int W, int shift) const {
    const int col = threadIdx.x & ((1 << shift) - 1), sub = threadIdx.x >> shift;
    const int rpp = (int)blockDim.x >> shift;
    const int RS = W + 2;
#pragma unroll
    for (int k = 0; k < NPASS; ++k) {
      const int row = k * rpp + sub;
      if (col < W && row < H) {
        float* dst = lds_planes + ((row + 1) * RS + 1 + col) * CH;
        if constexpr (CH == 4) {
          *reinterpret_cast<float4*>(dst) = make_float4(v[0][k], v[1][k], v[2][k], v[3][k]);
        } else {
#pragma unroll
          for (int c = 0; c < CH; ++c) dst[c] = v[c][k];
        }
      }
    }
  }
};

template <int CH>
struct CornersN {
  float a[CH], b[CH], c[CH], d[CH];
};
template <int CH>
__device__ __forceinline__ CornersN<CH> read_corners_n(const float* planes, int pidx_ch, int RS) {
  CornersN<CH> q;
  const float* p0 = planes + pidx_ch;
  const float* p1 = p0 + RS * CH;
  static_assert(CH == 4 || CH == 2, "16-byte or 8-byte corner reads");
  if constexpr (CH == 4) {
    const float4 a = *reinterpret_cast<const float4*>(p0), b = *reinterpret_cast<const float4*>(p0 + 4);
    const float4 c = *reinterpret_cast<const float4*>(p1), d = *reinterpret_cast<const float4*>(p1 + 4);
    q.a[0] = a.x; q.a[1] = a.y; q.a[2] = a.z; q.a[3] = a.w;
    q.b[0] = b.x; q.b[1] = b.y; q.b[2] = b.z; q.b[3] = b.w;
    q.c[0] = c.x; q.c[1] = c.y; q.c[2] = c.z; q.c[3] = c.w;
    q.d[0] = d.x; q.d[1] = d.y; q.d[2] = d.z; q.d[3] = d.w;
  } else {
    const float2 a = *reinterpret_cast<const float2*>(p0), b = *reinterpret_cast<const float2*>(p0 + 2);
    const float2 c = *reinterpret_cast<const float2*>(p1), d = *reinterpret_cast<const float2*>(p1 + 2);
    q.a[0] = a.x; q.a[1] = a.y; q.b[0] = b.x; q.b[1] = b.y;
    q.c[0] = c.x; q.c[1] = c.y; q.d[0] = d.x; q.d[1] = d.y;
  }
  return q;
}

template <typename T, int SH, int SW, int NPASS, int CH, int BLOCK = kDBlock>
__global__ __launch_bounds__(BLOCK, BLOCK == kDBlock ? 2 : 1) void deform_forward_ch_kernel(
    Geo g, const T* __restrict__ x, const T* __restrict__ off, const T* __restrict__ rot,
    const T* __restrict__ filter, T* __restrict__ out, int ch_per_block, int shift, int tile_pix) {
  using Tb = WideTable<SH, SW>;
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int PS = ((H + 2) * RS + 3) & ~3;
  float* planes = lds;                // [2][PS][CH]
  float* tbl = lds + 2 * PS * CH;     // [ch_per_block rounded up to CH][Tb::SIZE]

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const BlockId b = decode_block(g, ceil_div(out_plane, tile_pix), ceil_div(cpg, ch_per_block));
  if (!b.valid) return;
  const int j0 = b.chunk * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  const int nq = ceil_div(nch, CH);

  for (int e = threadIdx.x; e < 2 * PS * CH; e += BLOCK) planes[e] = 0.f;
  // the tables of the channels that pad the last CH-tuple are read (their products discarded)
  for (int e = nch * Tb::SIZE + threadIdx.x; e < nq * CH * Tb::SIZE; e += BLOCK) tbl[e] = 0.f;
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, b.grp + g.groups * j0, g.groups, nch);

  const int p = b.tile * tile_pix + threadIdx.x;
  const bool live = (int)threadIdx.x < tile_pix && p < out_plane;
  ImgTap it[K9];
  LiteTap st[K9];
  deform_taps<T, SH, SW>(g, off, rot, b.n, b.grp, p, live, RS, it, st);
#pragma unroll
  for (int t = 0; t < K9; ++t) it[t].pidx *= CH;

  const size_t chan0 = (size_t)b.n * g.channel + b.grp + (size_t)g.groups * j0;
  const T* xp = x + chan0 * in_plane;
  T* op = out + chan0 * out_plane;
  const size_t x_step = (size_t)g.groups * in_plane, o_step = (size_t)g.groups * out_plane;
  const unsigned ooff = live ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  PlaneStageN<T, NPASS, CH> stage;
  stage.load(xp, x_step, nch, H, W, shift);
  __syncthreads();  // the zero fill is done
  stage.store(planes, H, W, shift);
  __syncthreads();
  for (int jq = 0; jq < nq; ++jq) {
    if (jq + 1 < nq) stage.load(xp + (size_t)(jq + 1) * CH * x_step, x_step, nch - (jq + 1) * CH, H, W, shift);
    const float* pl = planes + (jq & 1) * PS * CH;
    const float* tb = tbl + jq * CH * Tb::SIZE;
    float acc[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) acc[c] = 0.f;
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      const CornersN<CH> q = read_corners_n<CH>(pl, it[t].pidx, RS);
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const float top = fmaf(it[t].lw, q.b[c] - q.a[c], q.a[c]), bot = fmaf(it[t].lw, q.d[c] - q.c[c], q.c[c]);
        const float v = fmaf(it[t].lh, bot - top, top);
        const float4 w = *reinterpret_cast<const float4*>(tb + c * Tb::SIZE + st[t].cell);
        acc[c] = fmaf(v, lite_weight(st[t], w), acc[c]);
      }
    }
#pragma unroll
    for (int c = 0; c < CH; ++c)
      buf_st(plane_rsrc(op + (size_t)(jq * CH + c) * o_step, jq * CH + c < nch ? out_plane : 0), ooff, acc[c], out);
    if (jq + 1 < nq) stage.store(planes + ((jq + 1) & 1) * PS * CH, H, W, shift);
    __syncthreads();
  }
}


// ---------------------------------------------------------------------------
// grad offset / grad rotation: the lane owns output pixel p and sums over the channels of its
// chunk; one fp32 partial per chunk goes to the workspace and reduce_partials_kernel adds the
// chunks in order.
//   rotation (K.cu:1410-1508): with the scope block in difference form the derivatives of the
//     scope read are c + lw * d and b + lh * d, so the lane accumulates
//     S_{b,c,d}[t] = sum_c sample_t[c] * gout[c] * {b, c, d}[c] and combines at the end;
//   offset (K.cu:1147-1243, get_coordinate_weight K.cu:231-268): d sample / dh =
//     (1 - lw) (bl - tl) + lw (br - tr), d sample / dw = (1 - lh) (tr - tl) + lh (br - bl), the
//     zero padding standing for the reference's per-corner range tests; times gout * B(Wt[c]).
// partial layout: [part][image (* group for rotation)][2 t + dir][pixel], part = chunk for
// rotation and group * chunks + chunk for offset (which sums over the groups as well).
// ---------------------------------------------------------------------------
template <typename T, int SH, int SW, int NPASS, bool ROTATION, int BLOCK = kDBlock>
__global__ __launch_bounds__(BLOCK, 2) void deform_grad_coord_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ off,
    const T* __restrict__ rot, const T* __restrict__ filter, float* __restrict__ partial,
    int ch_per_block, int shift) {
  using Tb = WideTable<SH, SW>;
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int PS = ((H + 2) * RS + 3) & ~3;
  float* planes = lds;
  float* tbl = lds + 2 * PS;

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const int chunks = ceil_div(cpg, ch_per_block);
  const BlockId b = decode_block(g, ceil_div(out_plane, BLOCK), chunks);
  if (!b.valid) return;
  const int j0 = b.chunk * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);

  for (int e = threadIdx.x; e < 2 * PS; e += BLOCK) planes[e] = 0.f;
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, b.grp + g.groups * j0, g.groups, nch);

  const int p = b.tile * BLOCK + threadIdx.x;
  const bool live = p < out_plane;
  ImgTap it[K9];
  LiteTap st[K9];
  constexpr bool WINDOW = BLOCK != kDBlock;
  unsigned hits = 0;
  deform_taps<T, SH, SW>(g, off, rot, b.n, b.grp, p, live, RS, it, st, &hits);
  RowWindow rw{0, H};
  if constexpr (WINDOW) rw = sample_rows(it, hits, RS, H);

  const size_t chan0 = (size_t)b.n * g.channel + b.grp + (size_t)g.groups * j0;
  const T* xp = x + chan0 * in_plane;
  const T* gp = gout + chan0 * out_plane;
  const size_t x_step = (size_t)g.groups * in_plane, g_step = (size_t)g.groups * out_plane;
  const unsigned goff = live ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  float s0[K9], s1[K9], s2[K9];
#pragma unroll
  for (int t = 0; t < K9; ++t) s0[t] = s1[t] = s2[t] = 0.f;

  PlaneStage<T, NPASS> stage;
  stage.template load<WINDOW>(xp, true, H, W, shift, rw);
  float gv = buf_ld(plane_rsrc(gp, out_plane), goff, gout);
  __syncthreads();
  stage.template store<WINDOW>(planes, H, W, shift, rw);
  __syncthreads();
  for (int j = 0; j < nch; ++j) {
    float gv_next = 0.f;
    if (j + 1 < nch) {
      stage.template load<WINDOW>(xp + (size_t)(j + 1) * x_step, true, H, W, shift, rw);
      gv_next = buf_ld(plane_rsrc(gp + (size_t)(j + 1) * g_step, out_plane), goff, gout);
    }
    const float* pl = planes + (j & 1) * PS;
    const float* tb = tbl + j * Tb::SIZE;
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      const Corners cq = read_corners(pl, it[t].pidx, RS);
      if (ROTATION) {
        const float ps = lerp2(cq, it[t].lh, it[t].lw) * gv;
        const float4 q = lds_read4(tb + st[t].cell);
        s0[t] = fmaf(ps, q.y, s0[t]);
        s1[t] = fmaf(ps, q.z, s1[t]);
        s2[t] = fmaf(ps, q.w, s2[t]);
      } else {
        const float4 q = *reinterpret_cast<const float4*>(tb + st[t].cell);
        const float gw = gv * lite_weight(st[t], q);
        const float ca = cq.c - cq.a, ba = cq.b - cq.a;
        const float dh = fmaf(it[t].lw, (cq.d - cq.b) - ca, ca);
        const float dw = fmaf(it[t].lh, (cq.d - cq.c) - ba, ba);
        s0[t] = fmaf(dh, gw, s0[t]);
        s1[t] = fmaf(dw, gw, s1[t]);
      }
    }
    gv = gv_next;
    if (j + 1 < nch) stage.template store<WINDOW>(planes + ((j + 1) & 1) * PS, H, W, shift, rw);
    __syncthreads();
  }

  if (live) {
    const size_t part = ROTATION ? (size_t)b.chunk : (size_t)b.grp * chunks + b.chunk;
    const size_t img = ROTATION ? (size_t)(b.n * g.groups + b.grp) : (size_t)b.n;
    const size_t imgs = ROTATION ? (size_t)g.batch * g.groups : (size_t)g.batch;
    float* dst = partial + ((part * imgs + img) * (K9 * 2)) * out_plane + p;
    const T* rp = rot + (size_t)(b.n * g.groups + b.grp) * (K9 * 2) * out_plane + p;
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      float dh = ROTATION ? fmaf(st[t].lw, s2[t], s1[t]) : s0[t];
      float dw = ROTATION ? fmaf(st[t].lh, s2[t], s0[t]) : s1[t];
      if (ROTATION && g.clip_mode != kClipNone) {  // a clamped offset has no gradient
        bool open_h, open_w;
        scope_coord<float>(g, t / 3, ld(rp + (size_t)(2 * t) * out_plane), g.centre_h, &open_h);
        scope_coord<float>(g, t % 3, ld(rp + (size_t)(2 * t + 1) * out_plane), g.centre_w, &open_w);
        dh = open_h ? dh : 0.f;
        dw = open_w ? dw : 0.f;
      }
      dst[(size_t)(2 * t) * out_plane] = dh;
      dst[(size_t)(2 * t + 1) * out_plane] = dw;
    }
  }
}

// The same with CH channel planes interleaved in LDS (see deform_forward_ch_kernel).
// MODE 0: grad offset, 1: grad rotation, 2: both from one pass over the staged planes (the corner gathers and
// the table reads, which bound these kernels, are shared; the rotation partials go to `partial`, the offset
// partials to `partial_off`).
template <typename T, int SH, int SW, int NPASS, int MODE, int CH, int BLOCK = kDBlock>
__global__ __launch_bounds__(BLOCK, BLOCK == kDBlock ? 2 : 1) void deform_grad_coord_ch_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ off,
    const T* __restrict__ rot, const T* __restrict__ filter, float* __restrict__ partial,
    int ch_per_block, int shift, int tile_pix, float* __restrict__ partial_off) {
  constexpr bool ROTATION = MODE != 0, OFFSET = MODE != 1;
  using Tb = WideTable<SH, SW>;
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int PS = ((H + 2) * RS + 3) & ~3;
  float* planes = lds;               // [2][PS][CH]
  float* tbl = lds + 2 * PS * CH;    // [ch_per_block rounded up to CH][Tb::SIZE]

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const int chunks = ceil_div(cpg, ch_per_block);
  const BlockId b = decode_block(g, ceil_div(out_plane, tile_pix), chunks);
  if (!b.valid) return;
  const int j0 = b.chunk * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  const int nq = ceil_div(nch, CH);

  for (int e = threadIdx.x; e < 2 * PS * CH; e += BLOCK) planes[e] = 0.f;
  // the padding channels of the last CH-tuple have gout = 0; their tables must be finite
  for (int e = nch * Tb::SIZE + threadIdx.x; e < nq * CH * Tb::SIZE; e += BLOCK) tbl[e] = 0.f;
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, b.grp + g.groups * j0, g.groups, nch);

  const int p = b.tile * tile_pix + threadIdx.x;
  const bool live = (int)threadIdx.x < tile_pix && p < out_plane;
  ImgTap it[K9];
  LiteTap st[K9];
  deform_taps<T, SH, SW>(g, off, rot, b.n, b.grp, p, live, RS, it, st);
#pragma unroll
  for (int t = 0; t < K9; ++t) it[t].pidx *= CH;

  const size_t chan0 = (size_t)b.n * g.channel + b.grp + (size_t)g.groups * j0;
  const T* xp = x + chan0 * in_plane;
  const T* gp = gout + chan0 * out_plane;
  const size_t x_step = (size_t)g.groups * in_plane, g_step = (size_t)g.groups * out_plane;
  const unsigned goff = live ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  float s0[K9], s1[K9], s2[K9];                    // rotation: sums of sample * gout * {b, c, d}
  float o0[OFFSET ? K9 : 1], o1[OFFSET ? K9 : 1];  // offset: sums of d sample / d{h, w} * gout * B
#pragma unroll
  for (int t = 0; t < K9; ++t) s0[t] = s1[t] = s2[t] = 0.f;
#pragma unroll
  for (int t = 0; t < (OFFSET ? K9 : 1); ++t) o0[t] = o1[t] = 0.f;

  PlaneStageN<T, NPASS, CH> stage;
  float gv[CH], gv_next[CH];
  stage.load(xp, x_step, nch, H, W, shift);
#pragma unroll
  for (int c = 0; c < CH; ++c) gv[c] = buf_ld(plane_rsrc(gp + (size_t)c * g_step, c < nch ? out_plane : 0), goff, gout);
  __syncthreads();
  stage.store(planes, H, W, shift);
  __syncthreads();
  for (int jq = 0; jq < nq; ++jq) {
#pragma unroll
    for (int c = 0; c < CH; ++c) gv_next[c] = 0.f;
    if (jq + 1 < nq) {
      const int jn = (jq + 1) * CH;
      stage.load(xp + (size_t)jn * x_step, x_step, nch - jn, H, W, shift);
#pragma unroll
      for (int c = 0; c < CH; ++c)
        gv_next[c] = buf_ld(plane_rsrc(gp + (size_t)(jn + c) * g_step, jn + c < nch ? out_plane : 0), goff, gout);
    }
    const float* pl = planes + (jq & 1) * PS * CH;
    const float* tb = tbl + jq * CH * Tb::SIZE;
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      const CornersN<CH> cq = read_corners_n<CH>(pl, it[t].pidx, RS);
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const float4 q = MODE == 1 ? lds_read4(tb + c * Tb::SIZE + st[t].cell)
                                   : *reinterpret_cast<const float4*>(tb + c * Tb::SIZE + st[t].cell);
        if constexpr (ROTATION) {
          const float top = fmaf(it[t].lw, cq.b[c] - cq.a[c], cq.a[c]), bot = fmaf(it[t].lw, cq.d[c] - cq.c[c], cq.c[c]);
          const float ps = fmaf(it[t].lh, bot - top, top) * gv[c];
          s0[t] = fmaf(ps, q.y, s0[t]);
          s1[t] = fmaf(ps, q.z, s1[t]);
          s2[t] = fmaf(ps, q.w, s2[t]);
        }
        if constexpr (OFFSET) {
          const float gw = gv[c] * lite_weight(st[t], q);
          const float ca = cq.c[c] - cq.a[c], ba = cq.b[c] - cq.a[c];
          const float dh = fmaf(it[t].lw, (cq.d[c] - cq.b[c]) - ca, ca);
          const float dw = fmaf(it[t].lh, (cq.d[c] - cq.c[c]) - ba, ba);
          o0[t] = fmaf(dh, gw, o0[t]);
          o1[t] = fmaf(dw, gw, o1[t]);
        }
      }
      // keeps the compiler from issuing every tap's reads first (8 x 16 bytes per tap: registers)
      // the tap's sums are complete here: without this the compiler sinks the arithmetic of all nine
      // taps below the plane store and keeps their 9 x 32 loaded values in registers meanwhile
      if constexpr (ROTATION) asm volatile("" : "+v"(s0[t]), "+v"(s1[t]), "+v"(s2[t])::"memory");
      if constexpr (OFFSET) asm volatile("" : "+v"(o0[t]), "+v"(o1[t])::"memory");
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) gv[c] = gv_next[c];
    if (jq + 1 < nq) stage.store(planes + ((jq + 1) & 1) * PS * CH, H, W, shift);
    __syncthreads();
  }

  if (live) {
    if constexpr (ROTATION) {
      float* dst = partial + (((size_t)b.chunk * g.batch * g.groups + (size_t)(b.n * g.groups + b.grp)) * (K9 * 2)) * out_plane + p;
      const T* rp = rot + (size_t)(b.n * g.groups + b.grp) * (K9 * 2) * out_plane + p;
#pragma unroll
      for (int t = 0; t < K9; ++t) {
        float dh = fmaf(st[t].lw, s2[t], s1[t]);
        float dw = fmaf(st[t].lh, s2[t], s0[t]);
        if (g.clip_mode != kClipNone) {  // a clamped offset has no gradient
          bool open_h, open_w;
          scope_coord<float>(g, t / 3, ld(rp + (size_t)(2 * t) * out_plane), g.centre_h, &open_h);
          scope_coord<float>(g, t % 3, ld(rp + (size_t)(2 * t + 1) * out_plane), g.centre_w, &open_w);
          dh = open_h ? dh : 0.f;
          dw = open_w ? dw : 0.f;
        }
        dst[(size_t)(2 * t) * out_plane] = dh;
        dst[(size_t)(2 * t + 1) * out_plane] = dw;
      }
    }
    if constexpr (OFFSET) {
      float* base = MODE == 2 ? partial_off : partial;
      float* dst = base + ((((size_t)b.grp * chunks + b.chunk) * g.batch + (size_t)b.n) * (K9 * 2)) * out_plane + p;
#pragma unroll
      for (int t = 0; t < K9; ++t) {
        dst[(size_t)(2 * t) * out_plane] = o0[t];
        dst[(size_t)(2 * t + 1) * out_plane] = o1[t];
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The channel-interleaved kernels for planes whose padded copy does not fit LDS twice four at a time (wider than
// 64 columns, or larger than 64 x 64): LDS holds a WINDOW of `wr` rows of the padded planes -- the rows the
// tile's samples touch, from a block-wide minimum / maximum over the taps that hit the image -- followed by
// RS + 2 zero positions, where the taps that contribute nothing point.  When the samples span more rows than the
// window holds, the tile takes several passes over consecutive windows, each sample counted in the pass that holds
// its two rows: any offsets are served, at one staging per pass and channel tuple.
// ---------------------------------------------------------------------------
constexpr int kDWinCh = 4;                                 // interleaved planes (kDeformCh of the host side)
constexpr int kDWinFwdBlock = 1024, kDWinFwdPass = 4;      // forward: 128 registers per lane suffice
constexpr int kDWinCoordBlock = 512, kDWinCoordPass = 8;   // coordinate gradients: up to 45 sums per lane

// Block-wide range [lo, hi] of the padded rows that hold the top-left corners of the workgroup's samples
// (hi < lo: no tap samples the image).  Two barriers; every thread of the workgroup must call it.
__device__ __forceinline__ void sample_top_rows(const ImgTap (&it)[K9], unsigned hits, int RS, int& lo, int& hi) {
  __shared__ int s_lo[16], s_hi[16];
  lo = 1 << 30, hi = -1;
#pragma unroll
  for (int t = 0; t < K9; ++t) {
    if (hits >> t & 1u) {
      const int pr = it[t].pidx / RS;
      lo = min(lo, pr);
      hi = max(hi, pr);
    }
  }
  for (int s = 32; s > 0; s >>= 1) {
    lo = min(lo, __shfl_xor(lo, s));
    hi = max(hi, __shfl_xor(hi, s));
  }
  if ((threadIdx.x & 63) == 0) {
    s_lo[threadIdx.x >> 6] = lo;
    s_hi[threadIdx.x >> 6] = hi;
  }
  __syncthreads();
  for (int w = 0; w < (int)blockDim.x / 64; ++w) {
    lo = min(lo, s_lo[w]);
    hi = max(hi, s_hi[w]);
  }
  __syncthreads();
}

// Cooperative load of window rows of CH planes: window row w (w < wr) is padded plane row wlo + w, i.e. plane row
// wlo + w - 1; rows outside the plane and the columns beside it load zeros, and every position of the window is
// written, so that a later pass leaves nothing of an earlier one.
template <typename T, int NPASS, int CH>
struct WindowStageN {
  float v[CH][NPASS];
  __device__ __forceinline__ void load(const T* plane0, size_t step, int live_channels, int H, int W, int shift,
                                       int wlo, int wr) {
    const int col = threadIdx.x & ((1 << shift) - 1), sub = threadIdx.x >> shift;
    const int rpp = (int)blockDim.x >> shift;
    unsigned so[NPASS];
#pragma unroll
    for (int k = 0; k < NPASS; ++k) {
      const int w = k * rpp + sub, row = wlo + w - 1;
      so[k] = (col < W && w < wr && row >= 0 && row < H) ? (unsigned)(row * W + col) * (unsigned)sizeof(T) : kOutOfRange;
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const bool on = c < live_channels;
      const rsrc_t r = plane_rsrc(plane0 + (on ? (size_t)c * step : 0), on ? H * W : 0);
#pragma unroll
      for (int k = 0; k < NPASS; ++k) v[c][k] = buf_ld(r, so[k], plane0);
    }
  }
  __device__ __forceinline__ void store(float* lds_planes, int W, int shift, int wr) const {
    static_assert(CH == 4, "16-byte stores");
    const int col = threadIdx.x & ((1 << shift) - 1), sub = threadIdx.x >> shift;
    const int rpp = (int)blockDim.x >> shift;
    const int RS = W + 2;
#pragma unroll
    for (int k = 0; k < NPASS; ++k) {
      const int w = k * rpp + sub;
      if (w < wr && col + 1 < RS)
        *reinterpret_cast<float4*>(lds_planes + (w * RS + 1 + col) * CH) = make_float4(v[0][k], v[1][k], v[2][k], v[3][k]);
    }
  }
};

// Descriptors of a pass: element offset (times CH) of each tap's top-left corner inside the window that starts at
// padded row wlo, or the zero area behind the window for a tap that is not in this pass.
template <int CH>
__device__ __forceinline__ void window_taps(const ImgTap (&it)[K9], unsigned hits, int RS, int wlo, int wr, int (&rel)[K9]) {
#pragma unroll
  for (int t = 0; t < K9; ++t) {
    const bool in = (hits >> t & 1u) && it[t].pidx >= wlo * RS && it[t].pidx < (wlo + wr - 1) * RS;
    rel[t] = (in ? it[t].pidx - wlo * RS : wr * RS) * CH;
  }
}

template <typename T, int SH, int SW>
__global__ __launch_bounds__(kDWinFwdBlock, 1) void deform_forward_chw_kernel(
    Geo g, const T* __restrict__ x, const T* __restrict__ off, const T* __restrict__ rot,
    const T* __restrict__ filter, T* __restrict__ out, int ch_per_block, int shift, int wr) {
  constexpr int CH = kDWinCh, BLOCK = kDWinFwdBlock;
  using Tb = WideTable<SH, SW>;
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int WP = wr * RS + RS + 2;    // positions of a buffer: the window, then the zero area
  float* planes = lds;                // [2][WP][CH]
  float* tbl = lds + 2 * WP * CH;     // [ch_per_block rounded up to CH][Tb::SIZE]

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const BlockId b = decode_block(g, ceil_div(out_plane, BLOCK), ceil_div(cpg, ch_per_block));
  if (!b.valid) return;
  const int j0 = b.chunk * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  const int nq = ceil_div(nch, CH);

  for (int e = threadIdx.x; e < 2 * WP * CH; e += BLOCK) planes[e] = 0.f;
  for (int e = nch * Tb::SIZE + threadIdx.x; e < nq * CH * Tb::SIZE; e += BLOCK) tbl[e] = 0.f;
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, b.grp + g.groups * j0, g.groups, nch);

  const int p = b.tile * BLOCK + threadIdx.x;
  const bool live = p < out_plane;
  ImgTap it[K9];
  LiteTap st[K9];
  unsigned hits = 0;
  deform_taps<T, SH, SW>(g, off, rot, b.n, b.grp, p, live, RS, it, st, &hits);
  int lo, hi;
  sample_top_rows(it, hits, RS, lo, hi);  // (its barriers also end the zero fill)
  const int npass = hi < lo ? 1 : ceil_div(hi - lo + 1, wr - 1);
  if (hi < lo) lo = 0;

  const size_t chan0 = (size_t)b.n * g.channel + b.grp + (size_t)g.groups * j0;
  const T* xp = x + chan0 * in_plane;
  T* op = out + chan0 * out_plane;
  const size_t x_step = (size_t)g.groups * in_plane, o_step = (size_t)g.groups * out_plane;
  const unsigned ooff = live ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  WindowStageN<T, kDWinFwdPass, CH> stage;
  for (int k = 0; k < npass; ++k) {
    const int wlo = lo + k * (wr - 1);
    int rel[K9];
    window_taps<CH>(it, hits, RS, wlo, wr, rel);
    stage.load(xp, x_step, nch, H, W, shift, wlo, wr);
    __syncthreads();  // the previous pass's reads are done
    stage.store(planes, W, shift, wr);
    __syncthreads();
    for (int jq = 0; jq < nq; ++jq) {
      if (jq + 1 < nq) stage.load(xp + (size_t)(jq + 1) * CH * x_step, x_step, nch - (jq + 1) * CH, H, W, shift, wlo, wr);
      const float* pl = planes + (jq & 1) * WP * CH;
      const float* tb = tbl + jq * CH * Tb::SIZE;
      float acc[CH];
#pragma unroll
      for (int c = 0; c < CH; ++c) acc[c] = 0.f;
#pragma unroll
      for (int t = 0; t < K9; ++t) {
        const CornersN<CH> q = read_corners_n<CH>(pl, rel[t], RS);
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          const float top = fmaf(it[t].lw, q.b[c] - q.a[c], q.a[c]), bot = fmaf(it[t].lw, q.d[c] - q.c[c], q.c[c]);
          const float v = fmaf(it[t].lh, bot - top, top);
          const float4 w = *reinterpret_cast<const float4*>(tb + c * Tb::SIZE + st[t].cell);
          acc[c] = fmaf(v, lite_weight(st[t], w), acc[c]);
        }
      }
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const rsrc_t ro = plane_rsrc(op + (size_t)(jq * CH + c) * o_step, jq * CH + c < nch ? out_plane : 0);
        if (k > 0) acc[c] += buf_ld(ro, ooff, out);  // the taps of the earlier passes
        buf_st(ro, ooff, acc[c], out);
      }
      if (jq + 1 < nq) stage.store(planes + ((jq + 1) & 1) * WP * CH, W, shift, wr);
      __syncthreads();
    }
  }
}

// MODE as in deform_grad_coord_ch_kernel.  A tap's sums collect in the one pass that holds its sample.
template <typename T, int SH, int SW, int MODE>
__global__ __launch_bounds__(kDWinCoordBlock, 1) void deform_grad_coord_chw_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ off,
    const T* __restrict__ rot, const T* __restrict__ filter, float* __restrict__ partial,
    int ch_per_block, int shift, int wr, float* __restrict__ partial_off) {
  constexpr bool ROTATION = MODE != 0, OFFSET = MODE != 1;
  constexpr int CH = kDWinCh, BLOCK = kDWinCoordBlock;
  using Tb = WideTable<SH, SW>;
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int WP = wr * RS + RS + 2;
  float* planes = lds;               // [2][WP][CH]
  float* tbl = lds + 2 * WP * CH;    // [ch_per_block rounded up to CH][Tb::SIZE]

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const int chunks = ceil_div(cpg, ch_per_block);
  const BlockId b = decode_block(g, ceil_div(out_plane, BLOCK), chunks);
  if (!b.valid) return;
  const int j0 = b.chunk * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  const int nq = ceil_div(nch, CH);

  for (int e = threadIdx.x; e < 2 * WP * CH; e += BLOCK) planes[e] = 0.f;
  for (int e = nch * Tb::SIZE + threadIdx.x; e < nq * CH * Tb::SIZE; e += BLOCK) tbl[e] = 0.f;
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, b.grp + g.groups * j0, g.groups, nch);

  const int p = b.tile * BLOCK + threadIdx.x;
  const bool live = p < out_plane;
  ImgTap it[K9];
  LiteTap st[K9];
  unsigned hits = 0;
  deform_taps<T, SH, SW>(g, off, rot, b.n, b.grp, p, live, RS, it, st, &hits);
  int lo, hi;
  sample_top_rows(it, hits, RS, lo, hi);
  const int npass = hi < lo ? 1 : ceil_div(hi - lo + 1, wr - 1);
  if (hi < lo) lo = 0;

  const size_t chan0 = (size_t)b.n * g.channel + b.grp + (size_t)g.groups * j0;
  const T* xp = x + chan0 * in_plane;
  const T* gp = gout + chan0 * out_plane;
  const size_t x_step = (size_t)g.groups * in_plane, g_step = (size_t)g.groups * out_plane;
  const unsigned goff = live ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  float s0[K9], s1[K9], s2[K9];                    // rotation: sums of sample * gout * {b, c, d}
  float o0[OFFSET ? K9 : 1], o1[OFFSET ? K9 : 1];  // offset: sums of d sample / d{h, w} * gout * B
#pragma unroll
  for (int t = 0; t < K9; ++t) s0[t] = s1[t] = s2[t] = 0.f;
#pragma unroll
  for (int t = 0; t < (OFFSET ? K9 : 1); ++t) o0[t] = o1[t] = 0.f;

  WindowStageN<T, kDWinCoordPass, CH> stage;
  for (int k = 0; k < npass; ++k) {
    const int wlo = lo + k * (wr - 1);
    int rel[K9];
    window_taps<CH>(it, hits, RS, wlo, wr, rel);
    float gv[CH], gv_next[CH];
    stage.load(xp, x_step, nch, H, W, shift, wlo, wr);
#pragma unroll
    for (int c = 0; c < CH; ++c) gv[c] = buf_ld(plane_rsrc(gp + (size_t)c * g_step, c < nch ? out_plane : 0), goff, gout);
    __syncthreads();
    stage.store(planes, W, shift, wr);
    __syncthreads();
    for (int jq = 0; jq < nq; ++jq) {
#pragma unroll
      for (int c = 0; c < CH; ++c) gv_next[c] = 0.f;
      if (jq + 1 < nq) {
        const int jn = (jq + 1) * CH;
        stage.load(xp + (size_t)jn * x_step, x_step, nch - jn, H, W, shift, wlo, wr);
#pragma unroll
        for (int c = 0; c < CH; ++c)
          gv_next[c] = buf_ld(plane_rsrc(gp + (size_t)(jn + c) * g_step, jn + c < nch ? out_plane : 0), goff, gout);
      }
      const float* pl = planes + (jq & 1) * WP * CH;
      const float* tb = tbl + jq * CH * Tb::SIZE;
#pragma unroll
      for (int t = 0; t < K9; ++t) {
        const CornersN<CH> cq = read_corners_n<CH>(pl, rel[t], RS);
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          const float4 q = *reinterpret_cast<const float4*>(tb + c * Tb::SIZE + st[t].cell);
          if constexpr (ROTATION) {
            const float top = fmaf(it[t].lw, cq.b[c] - cq.a[c], cq.a[c]), bot = fmaf(it[t].lw, cq.d[c] - cq.c[c], cq.c[c]);
            const float ps = fmaf(it[t].lh, bot - top, top) * gv[c];
            s0[t] = fmaf(ps, q.y, s0[t]);
            s1[t] = fmaf(ps, q.z, s1[t]);
            s2[t] = fmaf(ps, q.w, s2[t]);
          }
          if constexpr (OFFSET) {
            const float gw = gv[c] * lite_weight(st[t], q);
            const float ca = cq.c[c] - cq.a[c], ba = cq.b[c] - cq.a[c];
            const float dh = fmaf(it[t].lw, (cq.d[c] - cq.b[c]) - ca, ca);
            const float dw = fmaf(it[t].lh, (cq.d[c] - cq.c[c]) - ba, ba);
            o0[t] = fmaf(dh, gw, o0[t]);
            o1[t] = fmaf(dw, gw, o1[t]);
          }
        }
        // the tap's sums are complete here: keeps the arithmetic of all nine taps from sinking below the plane store
        if constexpr (ROTATION) asm volatile("" : "+v"(s0[t]), "+v"(s1[t]), "+v"(s2[t])::"memory");
        if constexpr (OFFSET) asm volatile("" : "+v"(o0[t]), "+v"(o1[t])::"memory");
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int c = 0; c < CH; ++c) gv[c] = gv_next[c];
      if (jq + 1 < nq) stage.store(planes + ((jq + 1) & 1) * WP * CH, W, shift, wr);
      __syncthreads();
    }
  }

  if (live) {
    if constexpr (ROTATION) {
      float* dst = partial + (((size_t)b.chunk * g.batch * g.groups + (size_t)(b.n * g.groups + b.grp)) * (K9 * 2)) * out_plane + p;
      const T* rp = rot + (size_t)(b.n * g.groups + b.grp) * (K9 * 2) * out_plane + p;
#pragma unroll
      for (int t = 0; t < K9; ++t) {
        float dh = fmaf(st[t].lw, s2[t], s1[t]);
        float dw = fmaf(st[t].lh, s2[t], s0[t]);
        if (g.clip_mode != kClipNone) {  // a clamped offset has no gradient
          bool open_h, open_w;
          scope_coord<float>(g, t / 3, ld(rp + (size_t)(2 * t) * out_plane), g.centre_h, &open_h);
          scope_coord<float>(g, t % 3, ld(rp + (size_t)(2 * t + 1) * out_plane), g.centre_w, &open_w);
          dh = open_h ? dh : 0.f;
          dw = open_w ? dw : 0.f;
        }
        dst[(size_t)(2 * t) * out_plane] = dh;
        dst[(size_t)(2 * t + 1) * out_plane] = dw;
      }
    }
    if constexpr (OFFSET) {
      float* base = MODE == 2 ? partial_off : partial;
      float* dst = base + ((((size_t)b.grp * chunks + b.chunk) * g.batch + (size_t)b.n) * (K9 * 2)) * out_plane + p;
#pragma unroll
      for (int t = 0; t < K9; ++t) {
        dst[(size_t)(2 * t) * out_plane] = o0[t];
        dst[(size_t)(2 * t + 1) * out_plane] = o1[t];
      }
    }
  }
}

// ---------------------------------------------------------------------------
// grad input (K.cu:704-795): every (pixel, tap, channel) adds gout * B(Wt[c]) * corner weight to
// the four input elements around its sample -- a scatter with data-dependent targets, done by
// the reference with global float atomics.  LDS float atomics are slow on gfx950 (about 190 clk
// per wave instruction) but 64-bit integer ones are not (about 15 clk), so the workgroup, which
// owns the whole output plane of its channels, accumulates the input-gradient planes in LDS in
// FIXED POINT, two channels per 64-bit add: each term becomes a signed 32-bit integer
// round(v * 2^s), and the pair travels as b * 2^32 + a (decoded after the sum: a is the low
// word read as signed, b the high word plus the borrow a negative a took).  s is chosen per
// channel from max|gout| (over the tensor, computed by a small kernel into the workspace),
// max|Wt[c]| and M, the largest number of samples touching one input element of this image
// (counted by the workgroup with a 32-bit LDS histogram), so that a term stays below
// 2^(30 - ceil(log2 M)) and no sum overflows.  This is used for M <= 64, where the grid is
// 2^-24 of the largest possible term or finer; an image with more samples on one element falls
// back to one channel per 64-bit sum on a 2^-44 grid.  Either sum is exact on its grid and
// independent of the order of the additions (run-to-run reproducible, which float atomics are not).
// Corners outside the image fall on the plane's zero padding, which is never read back.
// One block per (image, group, channel chunk); blockDim = output pixels rounded up to a wave.
// The kernel for planes of more than 1024 output pixels further down always uses the 2^-44 grid.
// ---------------------------------------------------------------------------
// max |p[i]| over a workgroup's share into out[blockIdx.x], as the bits of a non-negative float,
// which order like unsigned integers -- and the maximum is taken on those bits, so that an
// infinity (0x7f800000) or a NaN (anything above) in p wins and reaches the consumer, where a
// float maximum would drop a NaN; the consumer takes the maximum of the kAbsParts words
// (one atomic maximum per workgroup on a single word cost more than the reads: the atomics on one
// address serialise).  16-byte loads, four in flight per thread; p must be 16-byte aligned (the
// host checks).
template <typename T>
__global__ __launch_bounds__(256) void absmax_kernel(const T* __restrict__ p, long n, unsigned* __restrict__ out) {
  __shared__ unsigned wave_max[4];
  constexpr int V = 16 / (int)sizeof(T);
  struct alignas(16) Vec {
    T e[V];
  };
  const long nv = n / V, stride = (long)gridDim.x * blockDim.x, tid = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const Vec* pv = reinterpret_cast<const Vec*>(p);
  unsigned m = 0u;
  auto absbits = [](float v) { return __float_as_uint(v) & 0x7fffffffu; };
  constexpr int kInFlight = 4;
  for (long i = tid; i < nv; i += kInFlight * stride) {
    Vec q[kInFlight];
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) q[k] = pv[min(i + k * stride, nv - 1)];  // a repeated element does not change a maximum
#pragma unroll
    for (int k = 0; k < kInFlight; ++k)
#pragma unroll
      for (int e = 0; e < V; ++e) m = max(m, absbits(ld(&q[k].e[e])));
  }
  for (long i = nv * V + tid; i < n; i += stride) m = max(m, absbits(ld(p + i)));
  for (int s = 32; s > 0; s >>= 1) m = max(m, (unsigned)__shfl_xor((int)m, s));
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = max(max(wave_max[0], wave_max[1]), max(wave_max[2], wave_max[3]));
}
constexpr int kAbsParts = 512;  // workgroups of absmax_kernel = words the consumers reduce

// The maximum of absmax_kernel's words, for every thread of the workgroup (two barriers).
__device__ __forceinline__ float block_absmax(const unsigned* __restrict__ parts) {
  __shared__ unsigned s_max;
  if (threadIdx.x == 0) s_max = 0u;
  __syncthreads();
  unsigned m = 0u;
  for (int i = threadIdx.x; i < kAbsParts; i += blockDim.x) m = max(m, parts[i]);
  for (int s = 32; s > 0; s >>= 1) m = max(m, (unsigned)__shfl_xor((int)m, s));
  if ((threadIdx.x & 63) == 0) atomicMax(&s_max, m);
  __syncthreads();
  return __uint_as_float(s_max);
}

// The fixed-point sums need a finite bound gmax * wmax[c] on a term.  With an infinity or a NaN in
// out_grad (gmax is then that value: the maximum is taken on bit patterns) or in a channel's filter
// there is none, and the conversions to integers would turn such terms into zeros or wrapped numbers:
// the workgroup then writes NaN to the planes it owns instead (all of grad_input for a non-finite
// out_grad).  The reference's float atomics carry a non-finite term to the elements it touches;
// what a caller tests -- any non-finite value in the gradient, as loss scaling does -- gives the
// same answer.  Uniform over the workgroup; must be called by all its threads after wmax is visible.
template <typename T>
__device__ __forceinline__ bool write_nan_if_unbounded(float gmax, const float* wmax, int nch, T* planes0, size_t step,
                                                       int plane) {
  bool bounded = true;
  for (int j = 0; j < nch; ++j) bounded = bounded && (fabsf(gmax * wmax[j]) < __builtin_inff());  // false for NaN
  if (bounded) return false;
  for (int j = 0; j < nch; ++j)
    for (int e = threadIdx.x; e < plane; e += blockDim.x) dk::st(planes0 + (size_t)j * step + e, __builtin_nanf(""));
  return true;
}

// A result element that is not read again by the operator: non-temporal for 4-byte elements (a wave writes whole
// lines), the plain store for 2-byte ones (as partial lines they reach memory one by one).
__device__ __forceinline__ void st_stream(float* p, float v) { __builtin_nontemporal_store(v, p); }
template <typename T>
__device__ __forceinline__ void st_stream(T* p, float v) { dk::st(p, v); }

// Two channels share a 64-bit sum while at most 2^kPairHead samples touch one input element: a term is then
// rounded on a grid of 2^-(31 - kPairHead) = 2^-24 of the largest possible term or finer.  (3 x 3 taps at stride 1
// put 36 samples on an element on average and about 65 on the fullest element of a large plane.)
constexpr int kPairHead = 7;

// floor(v + 0.5) as a signed 32-bit integer, one instruction
__device__ __forceinline__ int round_half_up(float v) {
  int r;
  asm("v_cvt_rpi_i32_f32 %0, %1" : "=v"(r) : "v"(v));
  return r;
}

template <typename T, int SH, int SW>
__global__ __launch_bounds__(1024) void deform_grad_input_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ off, const T* __restrict__ rot,
    const T* __restrict__ filter, T* __restrict__ gin, const unsigned* __restrict__ gmax_bits,
    int ch_per_block, int shift) {
  using Tb = WideTable<SH, SW>;
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int PS = ((H + 2) * RS + 3) & ~3;
  unsigned long long* planes = reinterpret_cast<unsigned long long*>(lds);  // [2][PS]
  float* tbl = lds + 4 * PS;                                                // [ch_per_block][Tb::SIZE]
  float* wmax = tbl + ch_per_block * Tb::SIZE;                              // [ch_per_block]

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const BlockId b = decode_block(g, 1, ceil_div(cpg, ch_per_block));
  if (!b.valid) return;
  const int j0 = b.chunk * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);

  for (int e = threadIdx.x; e < 2 * PS; e += blockDim.x) planes[e] = 0ull;
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, b.grp + g.groups * j0, g.groups, nch);
  for (int j = threadIdx.x; j < nch; j += blockDim.x) {
    const T* f = filter + (size_t)(b.grp + g.groups * (j0 + j)) * (SH * SW);
    unsigned m = 0u;  // on bit patterns, so that a NaN is not dropped
    for (int e = 0; e < SH * SW; ++e) m = max(m, __float_as_uint(ld(f + e)) & 0x7fffffffu);
    wmax[j] = __uint_as_float(m);
  }

  const int p = threadIdx.x;
  const bool live = p < out_plane;
  ImgTap it[K9];
  LiteTap st[K9];
  unsigned hits = 0;  // taps that sample the image inside the scope band: the others add nothing
  {
    ScopeCoord sc[K9];
    deform_taps<T>(g, off, rot, b.n, b.grp, p, live, RS, it, sc);
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      st[t] = make_lite_tap<SH, SW>(sc[t].h, sc[t].w, true);
      const bool in = (sc[t].h > -1.f) && (sc[t].w > -1.f) && (sc[t].h < float(SH)) && (sc[t].w < float(SW));
      hits |= (live && in) ? (1u << t) : 0u;
    }
  }
  __syncthreads();  // planes are zero

  // The largest number of samples that touch one input element, M: a 32-bit histogram over the
  // (still empty) planes.  A plane element then sums at most M terms, so terms scaled below
  // 2^(30 - ceil(log2 M)) cannot overflow a signed 32-bit sum.
  __shared__ unsigned wave_most[16];
  {
    unsigned* count = reinterpret_cast<unsigned*>(planes);
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      if (hits >> t & 1u) {
        atomicAdd(count + it[t].pidx, 1u);
        atomicAdd(count + it[t].pidx + 1, 1u);
        atomicAdd(count + it[t].pidx + RS, 1u);
        atomicAdd(count + it[t].pidx + RS + 1, 1u);
      }
    }
    __syncthreads();
    unsigned most = 1u;
    for (int e = threadIdx.x; e < PS; e += blockDim.x) {
      most = max(most, count[e]);
      count[e] = 0u;
    }
    for (int sft = 32; sft > 0; sft >>= 1) most = max(most, (unsigned)__shfl_xor((int)most, sft));
    if ((threadIdx.x & 63) == 0) wave_most[threadIdx.x >> 6] = most;
    __syncthreads();
  }
  unsigned most = 1u;
  for (int w = 0; w < (int)blockDim.x / 64; ++w) most = max(most, wave_most[w]);
  const int head = most <= 1u ? 0 : 32 - __builtin_clz(most - 1u);  // ceil(log2(most))

  const size_t chan0 = (size_t)b.n * g.channel + b.grp + (size_t)g.groups * j0;
  const T* gp = gout + chan0 * out_plane;
  T* ip = gin + chan0 * in_plane;
  const size_t g_step = (size_t)g.groups * out_plane, i_step = (size_t)g.groups * in_plane;
  const unsigned goff = live ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;
  const float gmax = block_absmax(gmax_bits);
  if (write_nan_if_unbounded(gmax, wmax, nch, ip, i_step, in_plane)) return;
  const int col = threadIdx.x & ((1 << shift) - 1), sub = threadIdx.x >> shift;
  const int rpp = (int)blockDim.x >> shift;

  if (head > kPairHead) {
    // many samples on one element: one channel per 64-bit sum, on a 2^-44 grid through the
    // "add 1.5 * 2^52 in double" trick (the low mantissa bits of the sum are the rounded integer)
    float gv = buf_ld(plane_rsrc(gp, out_plane), goff, gout);
    for (int j = 0; j < nch; ++j) {
      const float gv_next = buf_ld(plane_rsrc(gp + (size_t)(j + 1) * g_step, j + 1 < nch ? out_plane : 0), goff, gout);
      unsigned long long* pl = planes + (j & 1) * PS;
      const float* tb = tbl + j * Tb::SIZE;
      int e;  // a term is at most gmax * wmax < 2^e: scale 2^(44 - e), the plane's sum stays below 2^62
      (void)frexpf(gmax * wmax[j], &e);
      const double scale = ldexp(1.0, 44 - e), unscale = ldexp(1.0, e - 44);
      constexpr double kMagic = 6755399441055744.0;  // 1.5 * 2^52
#pragma unroll
      for (int t = 0; t < K9; ++t) {
        if (hits >> t & 1u) {
          const float gw = gv * lite_weight(st[t], *reinterpret_cast<const float4*>(tb + st[t].cell));
          const float lh = it[t].lh, lw = it[t].lw, hh = 1.f - lh, hw = 1.f - lw;
          const float term[4] = {hh * hw * gw, hh * lw * gw, lh * hw * gw, lh * lw * gw};  // K.cu:776-789
          const int at[4] = {it[t].pidx, it[t].pidx + 1, it[t].pidx + RS, it[t].pidx + RS + 1};
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const double d = fma((double)term[k], scale, kMagic);
            // bits(d) - bits(kMagic): the magic's low word is 0, so only the high word changes
            atomicAdd(pl + at[k], (unsigned long long)__double_as_longlong(d) - 0x4338000000000000ull);
          }
        }
      }
      gv = gv_next;
      __syncthreads();
      T* dst = ip + (size_t)j * i_step;
      for (int row = sub; row < H; row += rpp) {
        if (col < W) {
          unsigned long long* cell = pl + (row + 1) * RS + 1 + col;
          const long long v = (long long)*cell;
          *cell = 0ull;
          dk::st(dst + row * W + col, (float)((double)v * unscale));
        }
      }
    }
    return;
  }

  float gva = buf_ld(plane_rsrc(gp, out_plane), goff, gout);
  float gvb = buf_ld(plane_rsrc(gp + g_step, 1 < nch ? out_plane : 0), goff, gout);
  for (int j = 0; j < nch; j += 2) {
    const bool pair = j + 1 < nch;
    const float ga_next = buf_ld(plane_rsrc(gp + (size_t)(j + 2) * g_step, j + 2 < nch ? out_plane : 0), goff, gout);
    const float gb_next = buf_ld(plane_rsrc(gp + (size_t)(j + 3) * g_step, j + 3 < nch ? out_plane : 0), goff, gout);
    unsigned long long* pl = planes + ((j >> 1) & 1) * PS;
    const float* ta = tbl + j * Tb::SIZE;
    const float* tb = tbl + (pair ? j + 1 : j) * Tb::SIZE;
    // a term of channel c is below gmax * wmax[c] < 2^e: scale 2^(30 - head - e)
    int ea, eb;
    (void)frexpf(gmax * wmax[j], &ea);
    (void)frexpf(gmax * wmax[pair ? j + 1 : j], &eb);
    const int sa = min(max(30 - head - ea, -100), 100), sb = min(max(30 - head - eb, -100), 100);
    const float ga_s = gva * ldexpf(1.f, sa), gb_s = pair ? gvb * ldexpf(1.f, sb) : 0.f;
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      if (hits >> t & 1u) {
        const float wa = ga_s * lite_weight(st[t], *reinterpret_cast<const float4*>(ta + st[t].cell));
        const float wb = gb_s * lite_weight(st[t], *reinterpret_cast<const float4*>(tb + st[t].cell));
        const float lh = it[t].lh, lw = it[t].lw, hh = 1.f - lh, hw = 1.f - lw;
        const float cw[4] = {hh * hw, hh * lw, lh * hw, lh * lw};  // K.cu:776-789
        const int at[4] = {it[t].pidx, it[t].pidx + 1, it[t].pidx + RS, it[t].pidx + RS + 1};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          // two signed 32-bit fixed-point terms in one 64-bit add: b * 2^32 + a
          const int ia = round_half_up(cw[k] * wa), ib = round_half_up(cw[k] * wb);
          const unsigned long long both =
              ((unsigned long long)(unsigned)(ib + (ia >> 31)) << 32) | (unsigned long long)(unsigned)ia;
          atomicAdd(pl + at[k], both);
        }
      }
    }
    gva = ga_next;
    gvb = gb_next;
    __syncthreads();
    // read the pair's plane back, clear it for the pair after next
    const float ua = ldexpf(1.f, -sa), ub = ldexpf(1.f, -sb);
    T* dst = ip + (size_t)j * i_step;
    for (int row = sub; row < H; row += rpp) {
      if (col < W) {
        unsigned long long* cell = pl + (row + 1) * RS + 1 + col;
        const unsigned long long v = *cell;
        *cell = 0ull;
        const int lo = (int)(unsigned)v;
        const int hi = (int)(unsigned)(v >> 32) + (lo < 0 ? 1 : 0);
        st_stream(dst + row * W + col, (float)lo * ua);
        if (pair) st_stream(dst + i_step + row * W + col, (float)hi * ub);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The input rows a tile of 1024 output pixels samples, for the band form of the tiled grad input below:
// table[(image * tiles + tile) * 2] = least, [.. + 1] = largest padded row (image row + 1) of the top corners of
// the tile's samples that hit the image (K.cu:486-500); a tile without such samples gets an empty range.
// The offsets belong to the image, not to the rotation group.  grid = image * tiles
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(1024) void deform_tile_rows_kernel(Geo g, const T* __restrict__ off, int* __restrict__ table,
                                                                int ntiles, unsigned* __restrict__ most_img) {
  __shared__ int wave_lo[16], wave_hi[16];
  const int out_plane = g.out_h * g.out_w;
  const int tile = blockIdx.x % ntiles, n = blockIdx.x / ntiles;
  const int p = tile * 1024 + threadIdx.x;
  const bool live = p < out_plane;
  const int pc = live ? p : 0;
  const int oh = pc / g.out_w, ow = pc % g.out_w;
  const rsrc_t ro = plane_rsrc(off + (size_t)n * (K9 * 2) * out_plane, K9 * 2 * out_plane);
  const unsigned step = (unsigned)out_plane * (unsigned)sizeof(T);
  int lo = 0x7fffffff, hi = -1;
#pragma unroll
  for (int t = 0; t < K9; ++t) {
    const int f_h = t / 3, f_w = t % 3;
    const unsigned o = live ? (unsigned)((2 * t) * out_plane + pc) * (unsigned)sizeof(T) : kOutOfRange;
    const float h = float(oh * g.stride_h - g.pad_h + f_h * g.dil_h) + buf_ld(ro, o, off);
    const float w = float(ow * g.stride_w - g.pad_w + f_w * g.dil_w) + buf_ld(ro, o + step, off);
    const bool hit = live && (h > -1.f) && (w > -1.f) && (h < float(g.in_h)) && (w < float(g.in_w));
    const int pr = static_cast<int>(floorf(h)) + 1;
    lo = hit ? min(lo, pr) : lo;
    hi = hit ? max(hi, pr) : hi;
  }
  for (int sft = 32; sft > 0; sft >>= 1) {
    lo = min(lo, __shfl_xor(lo, sft));
    hi = max(hi, __shfl_xor(hi, sft));
  }
  if ((threadIdx.x & 63) == 0) {
    wave_lo[threadIdx.x >> 6] = lo;
    wave_hi[threadIdx.x >> 6] = hi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; ++w) {
      lo = min(lo, wave_lo[w]);
      hi = max(hi, wave_hi[w]);
    }
    table[(size_t)blockIdx.x * 2] = lo;
    table[(size_t)blockIdx.x * 2 + 1] = hi;
    if (tile == 0) most_img[n] = 0u;  // deform_sample_count_kernel, next on the stream, takes maxima into it
  }
}

// ---------------------------------------------------------------------------
// most_img[image] = an upper bound of the number of samples whose bilinear footprint covers one input element
// (every sample that hits the image counts, also where its scope coordinate leaves the scope band and the
// operator adds nothing).  A workgroup holds a 32-bit histogram of a band of `band_rows` image rows in LDS
// (the whole plane where it fits), walks the tiles that touch it and sends the band's maximum.
// grid = image * bands
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(1024) void deform_sample_count_kernel(Geo g, const T* __restrict__ off,
                                                                   const int* __restrict__ tile_rows,
                                                                   unsigned* __restrict__ most_img, int ntiles,
                                                                   int band_rows) {
  extern __shared__ __align__(16) float lds[];
  unsigned* count = reinterpret_cast<unsigned*>(lds);
  __shared__ unsigned wave_most[16];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int out_plane = g.out_h * g.out_w;
  const int nbands = ceil_div(H, band_rows);
  const int band = blockIdx.x % nbands, n = blockIdx.x / nbands;
  const int r_lo = band * band_rows, r_hi = min(H, r_lo + band_rows);
  const int lo_idx = (r_lo + 1) * RS, hi_idx = (r_hi + 1) * RS;
  const int cells = band_rows * RS;
  for (int e = threadIdx.x; e < cells; e += 1024) count[e] = 0u;
  __syncthreads();
  const rsrc_t ro = plane_rsrc(off + (size_t)n * (K9 * 2) * out_plane, K9 * 2 * out_plane);
  const unsigned step = (unsigned)out_plane * (unsigned)sizeof(T);
  for (int tile = 0; tile < ntiles; ++tile) {
    const int* tr = tile_rows + ((size_t)n * ntiles + tile) * 2;
    if (!(tr[0] - 1 < r_hi && tr[1] >= r_lo)) continue;  // uniform over the workgroup
    const int p = tile * 1024 + threadIdx.x;
    const bool live = p < out_plane;
    const int pc = live ? p : 0;
    const int oh = pc / g.out_w, ow = pc % g.out_w;
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      const int f_h = t / 3, f_w = t % 3;
      const unsigned o = live ? (unsigned)((2 * t) * out_plane + pc) * (unsigned)sizeof(T) : kOutOfRange;
      const float h = float(oh * g.stride_h - g.pad_h + f_h * g.dil_h) + buf_ld(ro, o, off);
      const float w = float(ow * g.stride_w - g.pad_w + f_w * g.dil_w) + buf_ld(ro, o + step, off);
      const bool hit = live && (h > -1.f) && (w > -1.f) && (h < float(H)) && (w < float(W));
      if (hit) {
        const int pidx = (static_cast<int>(floorf(h)) + 1) * RS + static_cast<int>(floorf(w)) + 1;
        const int at = pidx - lo_idx;
        if (pidx >= lo_idx && pidx < hi_idx) {
          atomicAdd(count + at, 1u);
          atomicAdd(count + at + 1, 1u);
        }
        if (pidx + RS >= lo_idx && pidx + RS < hi_idx) {
          atomicAdd(count + at + RS, 1u);
          atomicAdd(count + at + RS + 1, 1u);
        }
      }
    }
  }
  __syncthreads();
  unsigned most = 0u;
  for (int e = threadIdx.x; e < cells; e += 1024) most = max(most, count[e]);
  for (int sft = 32; sft > 0; sft >>= 1) most = max(most, (unsigned)__shfl_xor((int)most, sft));
  if ((threadIdx.x & 63) == 0) wave_most[threadIdx.x >> 6] = most;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; ++w) most = max(most, wave_most[w]);
    atomicMax(most_img + n, most);
  }
}

// ---------------------------------------------------------------------------
// grad input for output planes of more than 1024 pixels, or input planes the kernel above has no room for.  The
// same fixed-point LDS accumulation, but the workgroup (1024 threads) owns 2 NP channels of an image and NP 64-bit
// planes; it walks the output plane in tiles of 1024 pixels, computes a tile's tap descriptors once and adds the
// tile's contributions for each of its channels.  M, the largest number of samples on one input element (as above),
// comes per image from deform_sample_count_kernel -- every workgroup of an image repeating that walk took 9 % of
// this kernel on 56 x 56 planes and 28 - 38 % of its band form: while M <= 2^kPairHead two channels share a plane,
// each as a signed 32-bit term in its half of the 64-bit sum, and one walk serves all 2 NP channels; otherwise
// every channel gets a plane of its own on the 2^-44 grid and the channels take two walks.  The planes are read
// back at the end of a walk.
// BAND: input planes that do not fit LDS even once (224 x 224).  A workgroup owns a band of `band_rows` image rows
// (of all columns) instead of the whole plane: it walks the tiles whose samples touch the band -- found in a table of
// each tile's least and largest sample row, written by deform_tile_rows_kernel -- and adds the corner pairs that lie
// in its rows; the other pairs are added by the band that owns theirs, so every input element is still summed in
// one workgroup's LDS, exactly, and written once.
// grid = ([bands,] channel chunks of 2 NP, image * group)
// ---------------------------------------------------------------------------
template <typename T, int SH, int SW, int NP, bool BAND = false>
__global__ __launch_bounds__(1024) void deform_grad_input_tiled_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ off, const T* __restrict__ rot,
    const T* __restrict__ filter, T* __restrict__ gin, const unsigned* __restrict__ gmax_bits, int shift,
    int band_rows, const int* __restrict__ tile_rows, const unsigned* __restrict__ most_img) {
  using Tb = WideTable<SH, SW>;
  constexpr int NC = 2 * NP;  // channels per workgroup
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int PS = ((BAND ? band_rows : H + 2) * RS + 3) & ~3;
  unsigned long long* planes = reinterpret_cast<unsigned long long*>(lds);  // [NP][PS]
  float* tbl = lds + 2 * NP * PS;                                           // [NC][Tb::SIZE]
  float* wmax = tbl + NC * Tb::SIZE;                                        // [NC]

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const BlockId b = decode_block(g, BAND ? ceil_div(H, band_rows) : 1, ceil_div(cpg, NC));
  if (!b.valid) return;
  const int j0 = b.chunk * NC;
  const int nch = min(NC, cpg - j0);
  // BAND: the image rows r_lo .. r_hi - 1 are this workgroup's; row r sits in LDS row r - r_lo (no padding rows),
  // and an index `pidx` of the whole padded plane lies in one of its rows when lo_idx <= pidx < hi_idx
  const int r_lo = BAND ? b.tile * band_rows : 0, r_hi = BAND ? min(H, r_lo + band_rows) : H;
  const int lo_idx = BAND ? (r_lo + 1) * RS : 0, hi_idx = BAND ? (r_hi + 1) * RS : 0x7fffffff;
  constexpr int ROWOFF = BAND ? 0 : 1;  // LDS row of the first image row

  for (int e = threadIdx.x; e < NP * PS; e += blockDim.x) planes[e] = 0ull;
  stage_wide_tables<T, SH, SW>(tbl, filter, g.channel, b.grp + g.groups * j0, g.groups, nch);
  if (threadIdx.x < nch) {
    const T* f = filter + (size_t)(b.grp + g.groups * (j0 + threadIdx.x)) * (SH * SW);
    unsigned m = 0u;  // on bit patterns, so that a NaN is not dropped
    for (int e = 0; e < SH * SW; ++e) m = max(m, __float_as_uint(ld(f + e)) & 0x7fffffffu);
    wmax[threadIdx.x] = __uint_as_float(m);
  }
  __syncthreads();

  const float gmax = block_absmax(gmax_bits);
  constexpr double kMagic = 6755399441055744.0;  // 1.5 * 2^52
  const size_t chan0 = (size_t)b.n * g.channel + b.grp + (size_t)g.groups * j0;
  const T* gp = gout + chan0 * out_plane;
  T* ip = gin + chan0 * in_plane;
  const size_t g_step = (size_t)g.groups * out_plane, i_step = (size_t)g.groups * in_plane;
  if (write_nan_if_unbounded(gmax, wmax, nch, ip, i_step, in_plane)) return;

  // a tile's descriptors; bit t of the result: tap t samples the image inside the scope band
  auto tile_taps = [&](int tile, ImgTap (&it)[K9], LiteTap (&st)[K9], unsigned& goff) {
    const int p = tile * (int)blockDim.x + threadIdx.x;
    const bool live = p < out_plane;
    ScopeCoord sc[K9];
    deform_taps<T>(g, off, rot, b.n, b.grp, p, live, RS, it, sc);
    unsigned hits = 0;
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      st[t] = make_lite_tap<SH, SW>(sc[t].h, sc[t].w, true);
      const bool in = (sc[t].h > -1.f) && (sc[t].w > -1.f) && (sc[t].h < float(SH)) && (sc[t].w < float(SW));
      hits |= in ? (1u << t) : 0u;
    }
    goff = live ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;
    return hits;
  };
  const int ntiles = ceil_div(out_plane, (int)blockDim.x);
  // BAND: the tiles whose samples touch this band's rows (tile_rows: least and largest padded row of a tile's
  // top corners, per image), and per sample whether its upper / lower corner pair lies in the band
  auto tile_in_band = [&](int tile) {
    const int* tr = tile_rows + ((size_t)b.n * ntiles + tile) * 2;
    return tr[0] - 1 < r_hi && tr[1] >= r_lo;  // image rows tr[0] - 1 .. tr[1] (a tile without samples: none)
  };
  auto top_in = [&](int pidx) { return !BAND || (pidx >= lo_idx && pidx < hi_idx); };
  auto bot_in = [&](int pidx) { return !BAND || (pidx + RS >= lo_idx && pidx + RS < hi_idx); };

  // M: an upper bound of the number of samples on one input element of this image (deform_sample_count_kernel)
  const unsigned most = max(1u, most_img[b.n]);
  const int head = most <= 1u ? 0 : 32 - __builtin_clz(most - 1u);  // ceil(log2(most))
  const int col = threadIdx.x & ((1 << shift) - 1), sub = threadIdx.x >> shift;
  const int rpp = (int)blockDim.x >> shift;

  if (head <= kPairHead) {
    // two channels per plane: channel 2 q in the low half, 2 q + 1 in the high half (see deform_grad_input_kernel)
    for (int tile = 0; tile < ntiles; ++tile) {
      if (!tile_in_band(tile)) continue;
      ImgTap it[K9];
      LiteTap st[K9];
      unsigned goff;
      const unsigned hits = tile_taps(tile, it, st, goff);
      for (int j = 0; j < nch; j += 2) {
        const bool pair = j + 1 < nch;
        const float gva = buf_ld(plane_rsrc(gp + (size_t)j * g_step, out_plane), goff, gout);
        const float gvb = buf_ld(plane_rsrc(gp + (size_t)(j + 1) * g_step, pair ? out_plane : 0), goff, gout);
        unsigned long long* pl = planes + (j >> 1) * PS;
        const float* ta = tbl + j * Tb::SIZE;
        const float* tb = tbl + (pair ? j + 1 : j) * Tb::SIZE;
        int ea, eb;  // a term of channel c is below gmax * wmax[c] < 2^e: scale 2^(30 - head - e)
        (void)frexpf(gmax * wmax[j], &ea);
        (void)frexpf(gmax * wmax[pair ? j + 1 : j], &eb);
        const int sa = min(max(30 - head - ea, -100), 100), sb = min(max(30 - head - eb, -100), 100);
        const float ga_s = gva * ldexpf(1.f, sa), gb_s = pair ? gvb * ldexpf(1.f, sb) : 0.f;
#pragma unroll
        for (int t = 0; t < K9; ++t) {
          if (hits >> t & 1u) {
            const float wa = ga_s * lite_weight(st[t], *reinterpret_cast<const float4*>(ta + st[t].cell));
            const float wb = gb_s * lite_weight(st[t], *reinterpret_cast<const float4*>(tb + st[t].cell));
            const float lh = it[t].lh, lw = it[t].lw, hh = 1.f - lh, hw = 1.f - lw;
            const float cw[4] = {hh * hw, hh * lw, lh * hw, lh * lw};  // K.cu:776-789
            const int a0 = it[t].pidx - lo_idx;
            const int at[4] = {a0, a0 + 1, a0 + RS, a0 + RS + 1};
            const bool in[2] = {top_in(it[t].pidx), bot_in(it[t].pidx)};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              if (BAND && !in[k >> 1]) continue;
              const int ia = round_half_up(cw[k] * wa), ib = round_half_up(cw[k] * wb);
              const unsigned long long both =
                  ((unsigned long long)(unsigned)(ib + (ia >> 31)) << 32) | (unsigned long long)(unsigned)ia;
              atomicAdd(pl + at[k], both);
            }
          }
        }
      }
    }
    __syncthreads();
    for (int j = 0; j < nch; j += 2) {
      const bool pair = j + 1 < nch;
      int ea, eb;
      (void)frexpf(gmax * wmax[j], &ea);
      (void)frexpf(gmax * wmax[pair ? j + 1 : j], &eb);
      const int sa = min(max(30 - head - ea, -100), 100), sb = min(max(30 - head - eb, -100), 100);
      const float ua = ldexpf(1.f, -sa), ub = ldexpf(1.f, -sb);
      const unsigned long long* pl = planes + (j >> 1) * PS;
      T* dst = ip + (size_t)j * i_step;
      for (int row = sub; row < r_hi - r_lo; row += rpp) {
        if (col < W) {
          const unsigned long long v = pl[(row + ROWOFF) * RS + 1 + col];
          const int lo = (int)(unsigned)v;
          const int hi = (int)(unsigned)(v >> 32) + (lo < 0 ? 1 : 0);
          st_stream(dst + (r_lo + row) * W + col, (float)lo * ua);
          if (pair) st_stream(dst + i_step + (r_lo + row) * W + col, (float)hi * ub);
        }
      }
    }
    return;
  }

  // many samples on one element: a plane per channel on the 2^-44 grid, NP channels per walk over the tiles
  for (int c0 = 0; c0 < nch; c0 += NP) {
    const int nc = min(NP, nch - c0);
    for (int tile = 0; tile < ntiles; ++tile) {
      if (!tile_in_band(tile)) continue;
      ImgTap it[K9];
      LiteTap st[K9];
      unsigned goff;
      const unsigned hits = tile_taps(tile, it, st, goff);
      for (int jj = 0; jj < nc; ++jj) {
        const int j = c0 + jj;
        const float gv = buf_ld(plane_rsrc(gp + (size_t)j * g_step, out_plane), goff, gout);
        unsigned long long* pl = planes + jj * PS;
        const float* tb = tbl + j * Tb::SIZE;
        int e;
        (void)frexpf(gmax * wmax[j], &e);
        const double scale = ldexp(1.0, 44 - e);
#pragma unroll
        for (int t = 0; t < K9; ++t) {
          if (hits >> t & 1u) {
            const float4 q = *reinterpret_cast<const float4*>(tb + st[t].cell);
            const float gw = gv * lite_weight(st[t], q);
            const float lh = it[t].lh, lw = it[t].lw, hh = 1.f - lh, hw = 1.f - lw;
            const float term[4] = {hh * hw * gw, hh * lw * gw, lh * hw * gw, lh * lw * gw};
            const int a0 = it[t].pidx - lo_idx;
            const int at[4] = {a0, a0 + 1, a0 + RS, a0 + RS + 1};
            const bool in[2] = {top_in(it[t].pidx), bot_in(it[t].pidx)};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              if (BAND && !in[k >> 1]) continue;
              const double d = fma((double)term[k], scale, kMagic);
              atomicAdd(pl + at[k], (unsigned long long)__double_as_longlong(d) - 0x4338000000000000ull);
            }
          }
        }
      }
    }
    __syncthreads();
    for (int jj = 0; jj < nc; ++jj) {
      const int j = c0 + jj;
      int e;
      (void)frexpf(gmax * wmax[j], &e);
      const double unscale = ldexp(1.0, e - 44);
      unsigned long long* pl = planes + jj * PS;
      T* dst = ip + (size_t)j * i_step;
      for (int row = sub; row < r_hi - r_lo; row += rpp) {
        if (col < W) {
          unsigned long long* cell = pl + (row + ROWOFF) * RS + 1 + col;
          dk::st(dst + (r_lo + row) * W + col, (float)((double)(long long)*cell * unscale));
          *cell = 0ull;  // for the next walk
        }
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// grad filter (K.cu:1002-1097): gW[c][i][j] = sum over (image, pixel, tap) of
// sample_t * gout * hat(sh_t - i) * hat(sw_t - j).  As in the local operator the sum is kept
// dense and in registers (per tap the lane holds the SH + SW hat weights, per channel it adds
// ps * a_i * b_j into SH * SW accumulators); after each channel the 64 lanes are summed with DPP
// wave reductions and lane `cell` adds the wave's total to a per-wave LDS accumulator.  One
// partial per (image, tile) workgroup; reduce_partials_kernel adds them in order.
// ---------------------------------------------------------------------------
template <typename T, int SH, int SW, int NPASS, int BLOCK = kDBlock>
__global__ __launch_bounds__(BLOCK, 2) void deform_grad_filter_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ off,
    const T* __restrict__ rot, float* __restrict__ partial, int ch_per_block, int shift) {
  constexpr int CELLS = SH * SW;
  constexpr int kWaves = BLOCK / 64;
  constexpr bool WINDOW = BLOCK != kDBlock;
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int PS = ((H + 2) * RS + 3) & ~3;
  float* planes = lds;
  float* wacc = lds + 2 * PS;  // [kWaves][ch_per_block][CELLS]

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const int tiles = ceil_div(out_plane, BLOCK);
  const BlockId b = decode_block(g, tiles, ceil_div(cpg, ch_per_block));
  if (!b.valid) return;
  const int j0 = b.chunk * ch_per_block;
  const int nch = min(ch_per_block, cpg - j0);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  for (int e = threadIdx.x; e < 2 * PS; e += BLOCK) planes[e] = 0.f;
  for (int e = threadIdx.x; e < kWaves * ch_per_block * CELLS; e += BLOCK) wacc[e] = 0.f;

  const int p = b.tile * BLOCK + threadIdx.x;
  const bool live = p < out_plane;
  ImgTap it[K9];
  float ah[K9][SH], bw[K9][SW];
  unsigned hits = 0;
  {
    ScopeCoord sc[K9];
    deform_taps<T>(g, off, rot, b.n, b.grp, p, live, RS, it, sc, &hits);
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      // outside the open box (-1, S) every hat below is 0 by itself, NaN coordinates excepted
      const bool in = (sc[t].h > -1.f) && (sc[t].w > -1.f) && (sc[t].h < float(SH)) && (sc[t].w < float(SW));
#pragma unroll
      for (int i = 0; i < SH; ++i) ah[t][i] = in ? fmaxf(1.f - fabsf(sc[t].h - float(i)), 0.f) : 0.f;
#pragma unroll
      for (int i = 0; i < SW; ++i) bw[t][i] = in ? fmaxf(1.f - fabsf(sc[t].w - float(i)), 0.f) : 0.f;
    }
  }

  const size_t chan0 = (size_t)b.n * g.channel + b.grp + (size_t)g.groups * j0;
  const T* xp = x + chan0 * in_plane;
  const T* gp = gout + chan0 * out_plane;
  const size_t x_step = (size_t)g.groups * in_plane, g_step = (size_t)g.groups * out_plane;
  const unsigned goff = live ? (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;

  RowWindow rw{0, H};
  if constexpr (WINDOW) rw = sample_rows(it, hits, RS, H);
  PlaneStage<T, NPASS> stage;
  stage.template load<WINDOW>(xp, true, H, W, shift, rw);
  float gv = buf_ld(plane_rsrc(gp, out_plane), goff, gout);
  __syncthreads();
  stage.template store<WINDOW>(planes, H, W, shift, rw);
  __syncthreads();
  for (int j = 0; j < nch; ++j) {
    float gv_next = 0.f;
    if (j + 1 < nch) {
      stage.template load<WINDOW>(xp + (size_t)(j + 1) * x_step, true, H, W, shift, rw);
      gv_next = buf_ld(plane_rsrc(gp + (size_t)(j + 1) * g_step, out_plane), goff, gout);
    }
    const float* pl = planes + (j & 1) * PS;
    float acc[SH][SW];
#pragma unroll
    for (int i = 0; i < SH; ++i)
#pragma unroll
      for (int k = 0; k < SW; ++k) acc[i][k] = 0.f;
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      const float ps = lerp2(read_corners(pl, it[t].pidx, RS), it[t].lh, it[t].lw) * gv;
#pragma unroll
      for (int i = 0; i < SH; ++i) {
        const float a = ah[t][i] * ps;
#pragma unroll
        for (int k = 0; k < SW; ++k) acc[i][k] = fmaf(a, bw[t][k], acc[i][k]);
      }
    }
    float mine = 0.f;
#pragma unroll
    for (int i = 0; i < SH; ++i)
#pragma unroll
      for (int k = 0; k < SW; ++k) {
        const float s = wave_sum(acc[i][k]);
        if (lane == i * SW + k) mine = s;
      }
    if (lane < CELLS) wacc[(wave * ch_per_block + j) * CELLS + lane] += mine;
    gv = gv_next;
    if (j + 1 < nch) stage.template store<WINDOW>(planes + ((j + 1) & 1) * PS, H, W, shift, rw);
    __syncthreads();
  }

  const size_t part = (size_t)b.n * tiles + b.tile;
  for (int e = threadIdx.x; e < nch * CELLS; e += BLOCK) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) s += wacc[w * ch_per_block * CELLS + e];
    const int c = b.grp + g.groups * (j0 + e / CELLS);
    partial[(part * g.channel + c) * CELLS + e % CELLS] = s;
  }
}

// ---------------------------------------------------------------------------
// grad filter on the matrix cores, for input planes small enough that 16 of them fit LDS.
//
// With k = (pixel, tap) the sum is a matrix product per block of 16 channels,
//   gW[cell][c] = sum_k A[cell][k] * P[k][c],
//   A[cell = (i, j)][k] = hat(sh_k - i) * hat(sw_k - j)          (channel independent),
//   P[k][c] = sample(x[c], h_k, w_k) * gout[c][pixel_k],
// and v_mfma_f32_16x16x4_f32 adds a 16 (cells) x 16 (channels) block over four k per issue in
// full fp32: lane l supplies A[l % 16][l / 16] and P[l / 16][l % 16].  A workgroup of 16 waves owns
// (image, tile of 256 output pixels) and walks a range of channel blocks; wave w owns pixels
// 16 w .. 16 w + 15, lane l the four pixels 16 w + 4 (l / 16) .. + 3 on the A side (its 36 hat
// products stay in registers for all channel blocks) and channel l % 16 on the P side.
//   * set-up: per (pixel, tap) where the tap samples the padded plane (byte offset, lh, lw) goes to
//     LDS, read back as one 16-byte broadcast per (lane, pixel, tap);
//   * per channel block: the 16 input planes are staged zero-padded and channel-interleaved,
//     position e of channel c at [e][c] with 20 floats per position (a thread owns a position and
//     writes its 16 channels as four 16-byte stores; with the pitch of 20 the 16 positions of one
//     store pass hit distinct banks), so the corner reads of the 16 lanes of a pixel quad are 64
//     contiguous bytes; the gout tile is staged channel-major.  The next block's loads are issued
//     before the MFMAs and land in registers while they run;
//   * the waves' 16 x 16 results are added in wave order by 256 owner threads and go out as the
//     partial of (image, tile): reduce_partials_kernel adds those in order.
// CELL0: the launch covers the scope cells CELL0 .. CELL0 + 15 (a 5 x 5 scope takes two).
// ---------------------------------------------------------------------------
// The value that lane II of the caller's quad (four consecutive lanes) holds; the compiler folds the lane
// selection into the instruction that uses the value where that instruction has a DPP form.
template <int II>
__device__ __forceinline__ float quad_lane(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), II * 0x55, 0xf, 0xf, true));
}
template <int II>
__device__ __forceinline__ unsigned quad_lane(unsigned v) {
  return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, II * 0x55, 0xf, 0xf, true);
}

// The planes of one block of channels of an image behind one descriptor each (input, gout): a channel of the
// block is selected by the scalar part of the address, `channel * x_cs` bytes, so that a load costs the scalar
// unit two instructions and not the twenty of a descriptor of its own (the 64-bit address, the size, the
// selects).  The range check compares the lane's offset with the descriptor's size less the scalar part, so the
// scalar part has to stay inside: channels past the block's last one (`last_`) re-read that one -- their columns
// of the product are never written -- and the host keeps sixteen channels' span below 2^31 bytes.
#define DK_GF_BLOCK_PLANES(cb)                                                                       \
  const int last_ = min(kGfCh, cpg - (cb) * kGfCh) - 1;                                              \
  const size_t c0_ = (size_t)n * g.channel + grp + (size_t)g.groups * ((cb) * kGfCh);                \
  const rsrc_t rx_ = plane_rsrc(x + c0_ * in_plane, last_ * g.groups * in_plane + in_plane);         \
  const rsrc_t rg_ = plane_rsrc(gout + c0_ * out_plane, last_ * g.groups * out_plane + out_plane);
template <typename T>
bool block_planes_fit(const Geo& g) {  // what DK_GF_BLOCK_PLANES asks of the shape
  const long plane = std::max<long>((long)g.in_h * g.in_w, (long)g.out_h * g.out_w);
  return 16L * g.groups * plane * (long)sizeof(T) < (1L << 31);
}

constexpr int kGfBlock = 1024;            // threads per workgroup
constexpr int kGfPix = 256;               // output pixels per tile
constexpr int kGfCh = 16;                 // channels per block
constexpr int kGfPitch = 20;              // floats per position of the interleaved planes
constexpr int kGfPitchG = kGfPix + 4;     // floats per channel of the gout tile

typedef float gf4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float hat1(float d) { return __builtin_amdgcn_fmed3f(1.f - fabsf(d), 0.f, 1.f); }

template <typename T, int SH, int SW, int CELL0>
__global__ __launch_bounds__(kGfBlock, 1) void deform_grad_filter_mfma_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ off,
    const T* __restrict__ rot, float* __restrict__ partial, int tiles, int csplits, int shift) {
  constexpr int CELLS = SH * SW;
  constexpr int kWaves = kGfBlock / 64;
  static_assert(CELL0 % 16 == 0 && CELL0 < CELLS, "the cells come in slices of 16, the rows of one MFMA block");
  static_assert(kGfPix == 16 * kWaves, "one 16-pixel group per wave");
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int PS = (H + 2) * RS;
  float* planes = lds;                                               // [PS][kGfPitch]
  float* gs = planes + PS * kGfPitch;                                // [kGfCh][kGfPitchG]
  float4* hwd = reinterpret_cast<float4*>(gs + kGfCh * kGfPitchG);   // [K9][kGfPix] {byte offset, lh, lw, -}
  float* red = reinterpret_cast<float*>(hwd + K9 * kGfPix);          // [kWaves][256]; set-up: scope coordinates [K9][kGfPix][2]
  float2* sc = reinterpret_cast<float2*>(red);

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const int x_cs = g.groups * in_plane * (int)sizeof(T), g_cs = g.groups * out_plane * (int)sizeof(T);  // bytes from a channel of the group to the next
  const int nblk_all = ceil_div(cpg, kGfCh);
  const int total = tiles * csplits * g.batch * g.groups;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int tile = lb % tiles, cs = lb / tiles % csplits;
  const int n = lb / tiles / csplits / g.groups, grp = lb / tiles / csplits % g.groups;
  const int blk_per = ceil_div(nblk_all, csplits);
  const int cb_lo = cs * blk_per, nblk = min(blk_per, nblk_all - cb_lo);
  if (nblk <= 0) return;

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int q = lane & 15, kg = lane >> 4;
  const int p0 = tile * kGfPix;
  const int live_pixels = min(kGfPix, out_plane - p0);
  const int live_waves = ceil_div(live_pixels, 16);
  const bool wave_live = wave < live_waves;

  // register stage of a channel block: the 16 channels of this thread's plane position, and four
  // channels of gout at its pixel
  const int s_col = threadIdx.x & ((1 << shift) - 1), s_row = threadIdx.x >> shift;
  const bool s_on = s_col < W && s_row < H;
  const unsigned s_off = s_on ? (unsigned)(s_row * W + s_col) * (unsigned)sizeof(T) : kOutOfRange;
  const int g_pix = threadIdx.x % kGfPix, g_cq = __builtin_amdgcn_readfirstlane(threadIdx.x / kGfPix);
  const unsigned g_off = p0 + g_pix < out_plane ? (unsigned)(p0 + g_pix) * (unsigned)sizeof(T) : kOutOfRange;
  float r_x[kGfCh], r_g[4];
#define DK_GF_ISSUE(cb)                                                                              \
  {                                                                                                  \
    DK_GF_BLOCK_PLANES(cb)                                                                           \
    _Pragma("unroll") for (int c = 0; c < kGfCh; ++c)                                                \
      r_x[c] = buf_ld2(rx_, s_off, min(c, last_) * x_cs, x);                                         \
    _Pragma("unroll") for (int c = 0; c < 4; ++c)                                                    \
      r_g[c] = buf_ld2(rg_, g_off, min(g_cq * 4 + c, last_) * g_cs, gout);                           \
  }
#define DK_GF_STORE()                                                                                \
  {                                                                                                  \
    if (s_on) {                                                                                      \
      float* dst = planes + ((s_row + 1) * RS + 1 + s_col) * kGfPitch;                               \
      _Pragma("unroll") for (int c = 0; c < kGfCh; c += 4)                                           \
        *reinterpret_cast<float4*>(dst + c) = make_float4(r_x[c], r_x[c + 1], r_x[c + 2], r_x[c + 3]); \
    }                                                                                                \
    _Pragma("unroll") for (int c = 0; c < 4; ++c) gs[(g_cq * 4 + c) * kGfPitchG + g_pix] = r_g[c];   \
  }

  DK_GF_ISSUE(cb_lo)

  for (int e = threadIdx.x; e < PS * kGfPitch; e += kGfBlock) planes[e] = 0.f;

  // set-up: this thread's pixel, taps g_cq, g_cq + 4, g_cq + 8 (K.cu:486-500 and 338-341)
  {
    const int p = p0 + g_pix;
    const bool live = p < out_plane;
    const int pc = live ? p : 0;
    const int oh = pc / g.out_w, ow = pc % g.out_w;
    const rsrc_t ro = plane_rsrc(off + (size_t)n * (K9 * 2) * out_plane, K9 * 2 * out_plane);
    const rsrc_t rr = rot ? plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K9 * 2) * out_plane, K9 * 2 * out_plane)
                          : plane_rsrc(rot, 0);  // no rotation tensor: reads as zeros
    const unsigned step = (unsigned)out_plane * (unsigned)sizeof(T);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const int t = g_cq + 4 * k;
      if (t < K9) {
        const int f_h = t / 3, f_w = t % 3;
        const unsigned o = live ? (unsigned)((2 * t) * out_plane + pc) * (unsigned)sizeof(T) : kOutOfRange;
        const float h = float(oh * g.stride_h - g.pad_h + f_h * g.dil_h) + buf_ld(ro, o, off);
        const float w = float(ow * g.stride_w - g.pad_w + f_w * g.dil_w) + buf_ld(ro, o + step, off);
        const bool hit = live && (h > -1.f) && (w > -1.f) && (h < float(H)) && (w < float(W));
        const float hf = floorf(h), wf = floorf(w);
        const int pidx = hit ? (static_cast<int>(hf) + 1) * RS + static_cast<int>(wf) + 1 : 0;
        const float sh = scope_coord<float>(g, f_h, buf_ld(rr, o, rot), g.centre_h);
        const float sw = scope_coord<float>(g, f_w, buf_ld(rr, o + step, rot), g.centre_w);
        const bool in = hit && (sh > -1.f) && (sw > -1.f) && (sh < float(SH)) && (sw < float(SW));
        hwd[t * kGfPix + g_pix] =
            make_float4(__int_as_float(pidx * kGfPitch * 4), hit ? h - hf : 0.f, hit ? w - wf : 0.f, 0.f);
        sc[t * kGfPix + g_pix] = in ? make_float2(sh, sw) : make_float2(-2.f, -2.f);
      }
    }
  }
  __syncthreads();

  const int px = wave * 16 + 4 * kg;  // first of this lane's four pixels in the tile
  // rows past the last cell stay 0
  const float ci = CELL0 + q < CELLS ? float((CELL0 + q) / SW) : 64.f, cj = float((CELL0 + q) % SW);
  float A[4][K9];
#pragma unroll
  for (int t = 0; t < K9; ++t) {
    const float4 s01 = *reinterpret_cast<const float4*>(sc + t * kGfPix + px);
    const float4 s23 = *reinterpret_cast<const float4*>(sc + t * kGfPix + px + 2);
    A[0][t] = hat1(s01.x - ci) * hat1(s01.y - cj);
    A[1][t] = hat1(s01.z - ci) * hat1(s01.w - cj);
    A[2][t] = hat1(s23.x - ci) * hat1(s23.y - cj);
    A[3][t] = hat1(s23.z - ci) * hat1(s23.w - cj);
  }
  // a lane keeps the descriptors of one of its four pixels, the one of its place in its quad of lanes; a sample's
  // descriptor comes out of the quad's lane of that pixel (quad_lane)
  unsigned d_off[K9];
  float d_lh[K9], d_lw[K9];
#pragma unroll
  for (int t = 0; t < K9; ++t) {
    const float4 d = hwd[t * kGfPix + px + (q & 3)];
    d_off[t] = __float_as_uint(d.x), d_lh[t] = d.y, d_lw[t] = d.z;
  }

  const size_t part = (size_t)n * tiles + tile;
  // owner threads: entry e of a block's result is D[cell = CELL0 + 4 * (l / 16) + r][channel l % 16]
  // with l = e / 4, r = e % 4 (register r of lane l)
#define DK_GF_FLUSH(cb)                                                                              \
  if (threadIdx.x < 256) {                                                                           \
    float s_ = 0.f;                                                                                  \
    for (int w_ = 0; w_ < live_waves; ++w_) s_ += red[w_ * 256 + threadIdx.x];                       \
    const int l_ = threadIdx.x / 4, r_ = threadIdx.x % 4;                                            \
    const int cell_ = CELL0 + 4 * (l_ / 16) + r_, cj_ = (cb) * kGfCh + l_ % 16;                      \
    if (cell_ < CELLS && cj_ < cpg)                                                                  \
      partial[(part * g.channel + grp + (size_t)g.groups * cj_) * CELLS + cell_] = s_;               \
  }

  gf4 acc = {0.f, 0.f, 0.f, 0.f};
  const unsigned row_bytes = (unsigned)RS * kGfPitch * 4;
  const char* plane_q = reinterpret_cast<const char*>(planes) + q * 4;
  for (int i = 0; i < nblk; ++i) {
    __syncthreads();  // the previous block's reads of the planes, the gout tile and `red` are done
    DK_GF_STORE()
    if (i > 0 && wave_live) *reinterpret_cast<gf4*>(red + (wave * 64 + lane) * 4) = acc;
    __syncthreads();
    if (i + 1 < nblk) DK_GF_ISSUE(cb_lo + i + 1)
    if (i > 0) DK_GF_FLUSH(cb_lo + i - 1)
    if (wave_live) {
      gf4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
      const float4 gv = *reinterpret_cast<const float4*>(gs + q * kGfPitchG + px);
      const float gq[4] = {gv.x, gv.y, gv.z, gv.w};
#define DK_GF_SAMPLE(t, ii)                                                                          \
  {                                                                                                  \
    const char* c0 = plane_q + quad_lane<ii>(d_off[t]);                                              \
    const char* c1 = c0 + row_bytes;                                                                 \
    const float ca = *reinterpret_cast<const float*>(c0), cb_ = *reinterpret_cast<const float*>(c0 + kGfPitch * 4); \
    const float cc = *reinterpret_cast<const float*>(c1), cd = *reinterpret_cast<const float*>(c1 + kGfPitch * 4);  \
    const float lh = quad_lane<ii>(d_lh[t]), lw = quad_lane<ii>(d_lw[t]);                            \
    const float top = fmaf(lw, cb_ - ca, ca), bot = fmaf(lw, cd - cc, cc);                           \
    const float b = fmaf(lh, bot - top, top) * gq[ii];                                               \
    if (((ii) + (t)) & 1)                                                                            \
      acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(A[ii][t], b, acc1, 0, 0, 0);                       \
    else                                                                                             \
      acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(A[ii][t], b, acc0, 0, 0, 0);                       \
  }
#pragma unroll
      for (int t = 0; t < K9; ++t) { DK_GF_SAMPLE(t, 0) DK_GF_SAMPLE(t, 1) DK_GF_SAMPLE(t, 2) DK_GF_SAMPLE(t, 3) }
#undef DK_GF_SAMPLE
      acc = acc0 + acc1;
    }
  }
  __syncthreads();
  if (wave_live) *reinterpret_cast<gf4*>(red + (wave * 64 + lane) * 4) = acc;
  __syncthreads();
  DK_GF_FLUSH(cb_lo + nblk - 1)
#undef DK_GF_ISSUE
#undef DK_GF_STORE
#undef DK_GF_FLUSH
}

// ---------------------------------------------------------------------------
// The same product for input planes of up to 64 columns that do not fit LDS sixteen at a time (56 x 56):
// a workgroup of 8 waves owns (image, tile of 128 output pixels) and stages, per block of 16 channels, only a
// window of `wr` rows of the padded planes -- the rows its tile's samples touch, found by a block-wide minimum /
// maximum over the taps that hit the image.  Descriptors are relative to the window; a tap that contributes
// nothing points at a zero area behind it.  When the samples span more rows than the window holds (offsets of
// many rows), the tile takes several passes over consecutive windows, each sample counted in the pass that holds
// its two rows: any offsets are served, at the cost of one staging per pass and block.
// ---------------------------------------------------------------------------
constexpr int kGwBlock = 512;
constexpr int kGwPix = 128;
constexpr int kGwPitchG = kGwPix + 4;
constexpr int kGwStage = 3;  // plane positions a thread stages per block
constexpr int kGwGrid = 256; // resident workgroups: one per CU (the window takes most of a CU's LDS)

// Persistent workgroups: workgroup w of `nwg` walks the units [units * w / nwg, units * (w + 1) / nwg) of the
// order (image, group, tile) x channel block, so every CU gets the same number of channel blocks and a tile's
// set-up (descriptors, hat products) is paid once per run of blocks, not once per launched workgroup.
template <typename T, int SH, int SW, int CELL0>
__global__ __launch_bounds__(kGwBlock, 1) void deform_grad_filter_win_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ off,
    const T* __restrict__ rot, float* __restrict__ partial, int tiles, int nwg, int shift, int wr) {
  constexpr int CELLS = SH * SW;
  constexpr int kWaves = kGwBlock / 64;
  static_assert(CELL0 % 16 == 0 && CELL0 < CELLS, "the cells come in slices of 16, the rows of one MFMA block");
  static_assert(kGwPix == 16 * kWaves, "one 16-pixel group per wave");
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w, RS = W + 2;
  const int wpos = wr * RS;                                          // positions of the window; then RS + 2 zeros
  float* planes = lds;                                               // [wpos + RS + 2][kGfPitch]
  float* gs = planes + (wpos + RS + 2) * kGfPitch;                   // [kGfCh][kGwPitchG]
  float4* hwd = reinterpret_cast<float4*>(gs + kGfCh * kGwPitchG);   // [K9][kGwPix] {byte offset, lh, lw, -}
  float* red = reinterpret_cast<float*>(hwd + K9 * kGwPix);          // [kWaves][256]; set-up: scope coordinates [K9][kGwPix][2]
  float2* sc = reinterpret_cast<float2*>(red);
  int* mm = reinterpret_cast<int*>(red + (kWaves * 256 > 2 * K9 * kGwPix ? kWaves * 256 : 2 * K9 * kGwPix));  // {min, max} row

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const int x_cs = g.groups * in_plane * (int)sizeof(T), g_cs = g.groups * out_plane * (int)sizeof(T);  // bytes from a channel of the group to the next
  const int nblk_all = ceil_div(cpg, kGfCh);
  const long units = (long)tiles * g.batch * g.groups * nblk_all;
  const int wg = logical_block(nwg);
  if (wg >= nwg) return;
  long u = units * wg / nwg;
  const long u_end = units * (wg + 1) / nwg;

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int q = lane & 15, kg = lane >> 4;
  const int px = wave * 16 + 4 * kg;  // first of this lane's four pixels in the tile
  // rows past the last cell stay 0
  const float ci = CELL0 + q < CELLS ? float((CELL0 + q) / SW) : 64.f, cj = float((CELL0 + q) % SW);
  const int g_pix = threadIdx.x % kGwPix, g_cq = __builtin_amdgcn_readfirstlane(threadIdx.x / kGwPix);
  const int rpp = kGwBlock >> shift;  // window rows one sweep of the workgroup's threads covers
  const int s_col = threadIdx.x & ((1 << shift) - 1), s_row = threadIdx.x >> shift;
  const unsigned row_bytes = (unsigned)RS * kGfPitch * 4;
  const unsigned zero_off = (unsigned)wpos * kGfPitch * 4;
  const char* plane_q = reinterpret_cast<const char*>(planes) + q * 4;

  // column 0 of the window's rows and the area behind it stay zero from here on: the staging writes columns 1..W + 1
  for (int e = threadIdx.x; e < (wpos + RS + 2) * kGfPitch; e += kGwBlock) planes[e] = 0.f;

  while (u < u_end) {  // a run of channel blocks of one (image, group, tile)
    const int tg = (int)(u / nblk_all), cb_lo = (int)(u % nblk_all);
    const int nblk = (int)(u_end - u < (long)(nblk_all - cb_lo) ? u_end - u : (long)(nblk_all - cb_lo));
    u += nblk;
    const int tile = tg % tiles, grp = tg / tiles % g.groups, n = tg / tiles / g.groups;
    const int p0 = tile * kGwPix;
    const int live_pixels = min(kGwPix, out_plane - p0);
    const int live_waves = ceil_div(live_pixels, 16);
    const bool wave_live = wave < live_waves;

    __syncthreads();  // the previous run's last reads of `red` (which `sc` shares) are done; the zero fill
    if (threadIdx.x == 0) mm[0] = 1 << 30, mm[1] = -1;

    // set-up: this thread's pixel, taps g_cq, g_cq + 4, g_cq + 8 (K.cu:486-500 and 338-341)
    int t_row[3], t_col[3];   // padded row / column of the sample's top-left corner; row -1: no contribution
    float t_lh[3], t_lw[3];
    __syncthreads();          // mm is initialised
    {
      const int p = p0 + g_pix;
      const bool live = p < out_plane;
      const int pc = live ? p : 0;
      const int oh = pc / g.out_w, ow = pc % g.out_w;
      const rsrc_t ro = plane_rsrc(off + (size_t)n * (K9 * 2) * out_plane, K9 * 2 * out_plane);
      const rsrc_t rr = rot ? plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K9 * 2) * out_plane, K9 * 2 * out_plane)
                            : plane_rsrc(rot, 0);  // no rotation tensor: reads as zeros
      const unsigned step = (unsigned)out_plane * (unsigned)sizeof(T);
      int lo_row = 1 << 30, hi_row = -1;
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        const int t = g_cq + 4 * k;
        t_row[k] = -1, t_col[k] = 0, t_lh[k] = 0.f, t_lw[k] = 0.f;
        if (t < K9) {
          const int f_h = t / 3, f_w = t % 3;
          const unsigned o = live ? (unsigned)((2 * t) * out_plane + pc) * (unsigned)sizeof(T) : kOutOfRange;
          const float h = float(oh * g.stride_h - g.pad_h + f_h * g.dil_h) + buf_ld(ro, o, off);
          const float w = float(ow * g.stride_w - g.pad_w + f_w * g.dil_w) + buf_ld(ro, o + step, off);
          const bool hit = live && (h > -1.f) && (w > -1.f) && (h < float(H)) && (w < float(W));
          const float hf = floorf(h), wf = floorf(w);
          const float sh = scope_coord<float>(g, f_h, buf_ld(rr, o, rot), g.centre_h);
          const float sw = scope_coord<float>(g, f_w, buf_ld(rr, o + step, rot), g.centre_w);
          const bool in = hit && (sh > -1.f) && (sw > -1.f) && (sh < float(SH)) && (sw < float(SW));
          sc[t * kGwPix + g_pix] = in ? make_float2(sh, sw) : make_float2(-2.f, -2.f);
          if (hit) {
            t_row[k] = static_cast<int>(hf) + 1, t_col[k] = static_cast<int>(wf) + 1;
            t_lh[k] = h - hf, t_lw[k] = w - wf;
            lo_row = min(lo_row, t_row[k]), hi_row = max(hi_row, t_row[k]);
          }
        }
      }
      // one atomic per wave and bound: 512 lanes on one LDS address take their turns one by one
      lo_row = wave_min(lo_row), hi_row = wave_max(hi_row);
      if (lane == 0 && hi_row >= 0) {
        atomicMin(&mm[0], lo_row);
        atomicMax(&mm[1], hi_row);
      }
    }
    __syncthreads();
    const int row_hi = mm[1], row_lo = row_hi < 0 ? 0 : mm[0];
    // a window holds the samples whose top row lies in its first wr - 1 rows
    const int npass = row_hi < 0 ? 1 : ceil_div(row_hi - row_lo + 1, wr - 1);

    // register stage of a (channel block, pass): the 16 channels of this thread's window positions, and four
    // channels of gout at its pixel
    const unsigned g_off = p0 + g_pix < out_plane ? (unsigned)(p0 + g_pix) * (unsigned)sizeof(T) : kOutOfRange;
    float r_x[kGwStage][kGfCh], r_g[4];
#define DK_GW_ISSUE(cb, lo_k, with_gout)                                                             \
  {                                                                                                  \
    unsigned so_[kGwStage];                                                                          \
    _Pragma("unroll") for (int j = 0; j < kGwStage; ++j) {                                           \
      const int urow_ = (lo_k) + s_row + rpp * j - 1;  /* plane row of window row s_row + rpp j */    \
      /* (plane rows past the lowest sample's bottom row are not read: row_hi is a padded row) */    \
      const bool ok_ = s_row + rpp * j < wr && urow_ >= 0 && urow_ < H && urow_ <= row_hi && s_col < W; \
      so_[j] = ok_ ? (unsigned)(urow_ * W + s_col) * (unsigned)sizeof(T) : kOutOfRange;              \
    }                                                                                                \
    DK_GF_BLOCK_PLANES(cb)                                                                           \
    _Pragma("unroll") for (int c = 0; c < kGfCh; ++c) {                                              \
      const int sc_ = min(c, last_) * x_cs;                                                          \
      _Pragma("unroll") for (int j = 0; j < kGwStage; ++j) r_x[j][c] = buf_ld2(rx_, so_[j], sc_, x); \
    }                                                                                                \
    if (with_gout) {                                                                                 \
      _Pragma("unroll") for (int c = 0; c < 4; ++c)                                                  \
        r_g[c] = buf_ld2(rg_, g_off, min(g_cq * 4 + c, last_) * g_cs, gout);                         \
    }                                                                                                \
  }

    float A[4][K9];
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      const float4 s01 = *reinterpret_cast<const float4*>(sc + t * kGwPix + px);
      const float4 s23 = *reinterpret_cast<const float4*>(sc + t * kGwPix + px + 2);
      A[0][t] = hat1(s01.x - ci) * hat1(s01.y - cj);
      A[1][t] = hat1(s01.z - ci) * hat1(s01.w - cj);
      A[2][t] = hat1(s23.x - ci) * hat1(s23.y - cj);
      A[3][t] = hat1(s23.z - ci) * hat1(s23.w - cj);
    }

    const size_t part = (size_t)n * tiles + tile;
    // owner threads: entry e of a block's result is D[cell = CELL0 + 4 * (l / 16) + r][channel l % 16]
    // with l = e / 4, r = e % 4 (register r of lane l)
    // ... in two halves: the reads of the waves' partial sums are asked for in front of a block's arithmetic and
    // added and written behind it, so that the four owner waves do not keep the other four waiting at the barrier
#define DK_GW_FLUSH_READ()                                                                           \
  if (threadIdx.x < 256) {                                                                           \
    _Pragma("unroll") for (int w_ = 0; w_ < kWaves; ++w_)                                            \
      fl[w_] = w_ < live_waves ? red[w_ * 256 + threadIdx.x] : 0.f;                                  \
  }
#define DK_GW_FLUSH(cb)                                                                              \
  if (threadIdx.x < 256) {                                                                           \
    float s_ = 0.f;                                                                                  \
    _Pragma("unroll") for (int w_ = 0; w_ < kWaves; ++w_) s_ += fl[w_];                              \
    const int l_ = threadIdx.x / 4, r_ = threadIdx.x % 4;                                            \
    const int cell_ = CELL0 + 4 * (l_ / 16) + r_, cj_ = (cb) * kGfCh + l_ % 16;                      \
    if (cell_ < CELLS && cj_ < cpg)                                                                  \
      partial[(part * g.channel + grp + (size_t)g.groups * cj_) * CELLS + cell_] = s_;               \
  }

    DK_GW_ISSUE(cb_lo, row_lo, true)

    gf4 acc = {0.f, 0.f, 0.f, 0.f};
    float fl[kWaves];            // the waves' partial sums of one entry of a block's result, on their way to `partial`
    unsigned d_off[K9];          // per tap, of pixel px + (q & 3): byte offset of the sample's top-left corner in the window
    float d_lh[K9], d_lw[K9];    // ... and its bilinear fractions
    const int steps = nblk * npass;
    for (int it = 0; it < steps; ++it) {
      const int i = it / npass, k = it % npass;
      const int lo_k = row_lo + k * (wr - 1);
      __syncthreads();  // the previous step's reads of the planes, the gout tile, the descriptors and `red` are done
      if (it == 0 || npass > 1) {
#pragma unroll
        for (int kk = 0; kk < 3; ++kk) {
          const int t = g_cq + 4 * kk;
          if (t < K9) {
            const bool in_pass = t_row[kk] >= lo_k && t_row[kk] <= lo_k + wr - 2;  // (row -1: never)
            const unsigned o = in_pass ? (unsigned)((t_row[kk] - lo_k) * RS + t_col[kk]) * (kGfPitch * 4) : zero_off;
            hwd[t * kGwPix + g_pix] = make_float4(__uint_as_float(o), t_lh[kk], t_lw[kk], 0.f);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < kGwStage; ++j) {
        const int wrow = s_row + rpp * j;
        if (wrow < wr && wrow <= row_hi + 1 - lo_k && s_col + 1 < RS) {  // (a row outside the image or the column right of it: zeros were loaded; rows below every sample: not read)
          float* dst = planes + (wrow * RS + 1 + s_col) * kGfPitch;
#pragma unroll
          for (int c = 0; c < kGfCh; c += 4)
            *reinterpret_cast<float4*>(dst + c) = make_float4(r_x[j][c], r_x[j][c + 1], r_x[j][c + 2], r_x[j][c + 3]);
        }
      }
      if (k == 0) {
#pragma unroll
        for (int c = 0; c < 4; ++c) gs[(g_cq * 4 + c) * kGwPitchG + g_pix] = r_g[c];
        if (it > 0 && wave_live) *reinterpret_cast<gf4*>(red + (wave * 64 + lane) * 4) = acc;
      }
      __syncthreads();
      if (it + 1 < steps) {
        const int i1 = (it + 1) / npass, k1 = (it + 1) % npass;
        if (k1 == 0) DK_GW_ISSUE(cb_lo + i1, row_lo, true)
        else DK_GW_ISSUE(cb_lo + i1, row_lo + k1 * (wr - 1), false)
      }
      const bool flush = k == 0 && it > 0;
      if (flush) DK_GW_FLUSH_READ()
      if (k == 0) acc = gf4{0.f, 0.f, 0.f, 0.f};
      if (it == 0 || npass > 1) {  // a lane keeps the descriptors of one of its four pixels, the one of its place in its quad
#pragma unroll
        for (int t = 0; t < K9; ++t) {
          const float4 d = hwd[t * kGwPix + px + (q & 3)];
          d_off[t] = __float_as_uint(d.x), d_lh[t] = d.y, d_lw[t] = d.z;
        }
      }
      if (wave_live) {
        gf4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
        const float4 gv = *reinterpret_cast<const float4*>(gs + q * kGwPitchG + px);
        const float gq[4] = {gv.x, gv.y, gv.z, gv.w};
        // Two stages kept apart by hand (the reads of LDS return in order): the corner reads of tap t + 1's four
        // samples, the arithmetic of tap t.  Left to itself the compiler waits for every sample's corners right
        // after asking for them.  The descriptor of sample (tap, pixel ii) comes out of the quad's lane ii.
        float cr[2][4][4];
#define DK_GW_CORNER(t, b, ii)                                                                       \
  {                                                                                                  \
    const char* c0 = plane_q + quad_lane<ii>(d_off[t]);                                              \
    const char* c1 = c0 + row_bytes;                                                                 \
    cr[b][ii][0] = *reinterpret_cast<const float*>(c0);                                              \
    cr[b][ii][1] = *reinterpret_cast<const float*>(c0 + kGfPitch * 4);                               \
    cr[b][ii][2] = *reinterpret_cast<const float*>(c1);                                              \
    cr[b][ii][3] = *reinterpret_cast<const float*>(c1 + kGfPitch * 4);                               \
  }
#define DK_GW_CORNERS(t, b) DK_GW_CORNER(t, b, 0) DK_GW_CORNER(t, b, 1) DK_GW_CORNER(t, b, 2) DK_GW_CORNER(t, b, 3)
#define DK_GW_SAMPLE(t, ii)                                                                          \
  {                                                                                                  \
    const float lh = quad_lane<ii>(d_lh[t]), lw = quad_lane<ii>(d_lw[t]);                            \
    const float ca = cr[(t) & 1][ii][0], cb_ = cr[(t) & 1][ii][1], cc = cr[(t) & 1][ii][2], cd = cr[(t) & 1][ii][3]; \
    const float top = fmaf(lw, cb_ - ca, ca), bot = fmaf(lw, cd - cc, cc);                           \
    const float b = fmaf(lh, bot - top, top) * gq[ii];                                               \
    if (((ii) + (t)) & 1)                                                                            \
      acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(A[ii][t], b, acc1, 0, 0, 0);                       \
    else                                                                                             \
      acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(A[ii][t], b, acc0, 0, 0, 0);                       \
  }
        DK_GW_CORNERS(0, 0)
#pragma unroll
        for (int t = 0; t < K9; ++t) {
          if (t + 1 < K9) DK_GW_CORNERS(t + 1, (t + 1) & 1)
          __builtin_amdgcn_sched_barrier(0);
          DK_GW_SAMPLE(t, 0) DK_GW_SAMPLE(t, 1) DK_GW_SAMPLE(t, 2) DK_GW_SAMPLE(t, 3)
          __builtin_amdgcn_sched_barrier(0);
        }
#undef DK_GW_CORNER
#undef DK_GW_CORNERS
#undef DK_GW_SAMPLE
        acc += acc0 + acc1;
      }
      if (flush) DK_GW_FLUSH(cb_lo + i - 1)
    }
    __syncthreads();
    if (wave_live) *reinterpret_cast<gf4*>(red + (wave * 64 + lane) * 4) = acc;
    __syncthreads();
    DK_GW_FLUSH_READ()
    DK_GW_FLUSH(cb_lo + nblk - 1)
#undef DK_GW_ISSUE
#undef DK_GW_FLUSH_READ
#undef DK_GW_FLUSH
  }
}

// ---------------------------------------------------------------------------
// ... and for planes of any width: the tile is a block of kG2Th x kG2Tw output pixels and the window a rectangle
// of `wr` rows x 32 columns of the padded planes (rows and columns from block-wide minima / maxima over the taps
// that hit the image), so its size depends on the offsets and not on the plane; passes over consecutive windows
// in both directions where the samples span more.
// ---------------------------------------------------------------------------
constexpr int kG2Tw = 8, kG2Th = kGwPix / kG2Tw;  // 16 rows of 8 pixels: a wave owns two rows
constexpr int kG2Wc = 32;                         // window columns (a power of two: the staging threads' mapping)

template <typename T, int SH, int SW, int CELL0>
__global__ __launch_bounds__(kGwBlock, 1) void deform_grad_filter_win2_kernel(
    Geo g, const T* __restrict__ gout, const T* __restrict__ x, const T* __restrict__ off,
    const T* __restrict__ rot, float* __restrict__ partial, int tiles_x, int tiles, int nwg, int wr) {
  constexpr int CELLS = SH * SW;
  constexpr int kWaves = kGwBlock / 64;
  constexpr int WC = kG2Wc;
  static_assert(CELL0 % 16 == 0 && CELL0 < CELLS, "the cells come in slices of 16, the rows of one MFMA block");
  static_assert(kGwPix == 16 * kWaves, "one 16-pixel group per wave");
  extern __shared__ __align__(16) float lds[];
  const int H = g.in_h, W = g.in_w;
  const int wpos = wr * WC;                                          // positions of the window; then WC + 2 zeros
  float* planes = lds;                                               // [wpos + WC + 2][kGfPitch]
  float* gs = planes + (wpos + WC + 2) * kGfPitch;                   // [kGfCh][kGwPitchG]
  float4* hwd = reinterpret_cast<float4*>(gs + kGfCh * kGwPitchG);   // [K9][kGwPix] {byte offset, lh, lw, -}
  float* red = reinterpret_cast<float*>(hwd + K9 * kGwPix);          // [kWaves][256]; set-up: scope coordinates [K9][kGwPix][2]
  float2* sc = reinterpret_cast<float2*>(red);
  int* mm = reinterpret_cast<int*>(red + (kWaves * 256 > 2 * K9 * kGwPix ? kWaves * 256 : 2 * K9 * kGwPix));  // min / max row, column

  const int cpg = g.channel / g.groups;
  const int out_plane = g.out_h * g.out_w, in_plane = H * W;
  const int x_cs = g.groups * in_plane * (int)sizeof(T), g_cs = g.groups * out_plane * (int)sizeof(T);  // bytes from a channel of the group to the next
  const int nblk_all = ceil_div(cpg, kGfCh);
  // persistent workgroups with equal shares of the (image, group, tile) x channel block units, as in the
  // row-window form
  const long units = (long)tiles * g.batch * g.groups * nblk_all;
  const int wg = logical_block(nwg);
  if (wg >= nwg) return;
  long u = units * wg / nwg;
  const long u_end = units * (wg + 1) / nwg;

  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int q = lane & 15, kg = lane >> 4;
  // every wave computes (a pixel outside the plane has gout = 0 and descriptors in the zero area)
  const int px = wave * 16 + 4 * kg;  // first of this lane's four pixels in the tile
  // rows past the last cell stay 0
  const float ci = CELL0 + q < CELLS ? float((CELL0 + q) / SW) : 64.f, cj = float((CELL0 + q) % SW);
  const int g_pix = threadIdx.x % kGwPix, g_cq = __builtin_amdgcn_readfirstlane(threadIdx.x / kGwPix);
  constexpr int rpp = kGwBlock / WC;  // window rows one sweep of the workgroup's threads covers
  const int s_col = threadIdx.x & (WC - 1), s_row = threadIdx.x / WC;
  const unsigned row_bytes = (unsigned)WC * kGfPitch * 4;
  const unsigned zero_off = (unsigned)wpos * kGfPitch * 4;
  const char* plane_q = reinterpret_cast<const char*>(planes) + q * 4;

  // the zero area (every position of the window that a pass reads is written by its staging)
  for (int e = threadIdx.x; e < (WC + 2) * kGfPitch; e += kGwBlock) planes[wpos * kGfPitch + e] = 0.f;

  while (u < u_end) {  // a run of channel blocks of one (image, group, tile)
    const int tg = (int)(u / nblk_all), cb_lo = (int)(u % nblk_all);
    const int nblk = (int)(u_end - u < (long)(nblk_all - cb_lo) ? u_end - u : (long)(nblk_all - cb_lo));
    u += nblk;
    const int tile = tg % tiles, grp = tg / tiles % g.groups, n = tg / tiles / g.groups;
    const int oy0 = tile / tiles_x * kG2Th, ox0 = tile % tiles_x * kG2Tw;

    __syncthreads();  // the previous run's last reads of `red` (which `sc` shares) are done; the zero fill
    if (threadIdx.x == 0) mm[0] = 1 << 30, mm[1] = -1, mm[2] = 1 << 30, mm[3] = -1;

    // set-up: this thread's pixel (index i of the tile: row i / kG2Tw, column i % kG2Tw), taps g_cq, g_cq + 4, g_cq + 8
    const int g_oy = oy0 + g_pix / kG2Tw, g_ox = ox0 + g_pix % kG2Tw;
    const bool g_live = g_oy < g.out_h && g_ox < g.out_w;
    const int g_p = g_live ? g_oy * g.out_w + g_ox : 0;
    int t_row[3], t_col[3];   // padded row / column of the sample's top-left corner; row -1: no contribution
    float t_lh[3], t_lw[3];
    __syncthreads();          // mm is initialised
    {
      const rsrc_t ro = plane_rsrc(off + (size_t)n * (K9 * 2) * out_plane, K9 * 2 * out_plane);
      const rsrc_t rr = rot ? plane_rsrc(rot + (size_t)(n * g.groups + grp) * (K9 * 2) * out_plane, K9 * 2 * out_plane)
                            : plane_rsrc(rot, 0);  // no rotation tensor: reads as zeros
      const unsigned step = (unsigned)out_plane * (unsigned)sizeof(T);
      int lo_row = 1 << 30, hi_row = -1, lo_col = 1 << 30, hi_col = -1;
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        const int t = g_cq + 4 * k;
        t_row[k] = -1, t_col[k] = 0, t_lh[k] = 0.f, t_lw[k] = 0.f;
        if (t < K9) {
          const int f_h = t / 3, f_w = t % 3;
          const unsigned o = g_live ? (unsigned)((2 * t) * out_plane + g_p) * (unsigned)sizeof(T) : kOutOfRange;
          const float h = float(g_oy * g.stride_h - g.pad_h + f_h * g.dil_h) + buf_ld(ro, o, off);
          const float w = float(g_ox * g.stride_w - g.pad_w + f_w * g.dil_w) + buf_ld(ro, o + step, off);
          const bool hit = g_live && (h > -1.f) && (w > -1.f) && (h < float(H)) && (w < float(W));
          const float hf = floorf(h), wf = floorf(w);
          const float sh = scope_coord<float>(g, f_h, buf_ld(rr, o, rot), g.centre_h);
          const float sw = scope_coord<float>(g, f_w, buf_ld(rr, o + step, rot), g.centre_w);
          const bool in = hit && (sh > -1.f) && (sw > -1.f) && (sh < float(SH)) && (sw < float(SW));
          sc[t * kGwPix + g_pix] = in ? make_float2(sh, sw) : make_float2(-2.f, -2.f);
          if (hit) {
            t_row[k] = static_cast<int>(hf) + 1, t_col[k] = static_cast<int>(wf) + 1;
            t_lh[k] = h - hf, t_lw[k] = w - wf;
            lo_row = min(lo_row, t_row[k]), hi_row = max(hi_row, t_row[k]);
            lo_col = min(lo_col, t_col[k]), hi_col = max(hi_col, t_col[k]);
          }
        }
      }
      // one atomic per wave and bound: 512 lanes on one LDS address take their turns one by one
      lo_row = wave_min(lo_row), hi_row = wave_max(hi_row), lo_col = wave_min(lo_col), hi_col = wave_max(hi_col);
      if (lane == 0 && hi_row >= 0) {
        atomicMin(&mm[0], lo_row);
        atomicMax(&mm[1], hi_row);
        atomicMin(&mm[2], lo_col);
        atomicMax(&mm[3], hi_col);
      }
    }
    __syncthreads();
    const bool any = mm[1] >= 0;
    const int row_lo = any ? mm[0] : 0, col_lo = any ? mm[2] : 0, row_hi = mm[1];
    // a window holds the samples whose corner lies in its first wr - 1 rows and WC - 1 columns
    const int npr = any ? ceil_div(mm[1] - row_lo + 1, wr - 1) : 1, npc = any ? ceil_div(mm[3] - col_lo + 1, WC - 1) : 1;
    const int npass = npr * npc;

    float A[4][K9];
#pragma unroll
    for (int t = 0; t < K9; ++t) {
      const float4 s01 = *reinterpret_cast<const float4*>(sc + t * kGwPix + px);
      const float4 s23 = *reinterpret_cast<const float4*>(sc + t * kGwPix + px + 2);
      A[0][t] = hat1(s01.x - ci) * hat1(s01.y - cj);
      A[1][t] = hat1(s01.z - ci) * hat1(s01.w - cj);
      A[2][t] = hat1(s23.x - ci) * hat1(s23.y - cj);
      A[3][t] = hat1(s23.z - ci) * hat1(s23.w - cj);
    }

    // register stage of a (channel block, pass): the 16 channels of this thread's window positions, and four
    // channels of gout at its pixel
    const unsigned g_off = g_live ? (unsigned)g_p * (unsigned)sizeof(T) : kOutOfRange;
    float r_x[kGwStage][kGfCh], r_g[4];
#define DK_GW_ISSUE(cb, lo_r, lo_c, with_gout)                                                       \
  {                                                                                                  \
    unsigned so_[kGwStage];                                                                          \
    const int ucol_ = (lo_c) + s_col - 1;  /* plane column of window column s_col */                 \
    _Pragma("unroll") for (int j = 0; j < kGwStage; ++j) {                                           \
      const int urow_ = (lo_r) + s_row + rpp * j - 1;                                                \
      /* (plane rows past the lowest sample's bottom row are not read: row_hi is a padded row) */    \
      const bool ok_ = s_row + rpp * j < wr && urow_ >= 0 && urow_ < H && urow_ <= row_hi && ucol_ >= 0 && ucol_ < W; \
      so_[j] = ok_ ? (unsigned)(urow_ * W + ucol_) * (unsigned)sizeof(T) : kOutOfRange;              \
    }                                                                                                \
    DK_GF_BLOCK_PLANES(cb)                                                                           \
    _Pragma("unroll") for (int c = 0; c < kGfCh; ++c) {                                              \
      const int sc_ = min(c, last_) * x_cs;                                                          \
      _Pragma("unroll") for (int j = 0; j < kGwStage; ++j) r_x[j][c] = buf_ld2(rx_, so_[j], sc_, x); \
    }                                                                                                \
    if (with_gout) {                                                                                 \
      _Pragma("unroll") for (int c = 0; c < 4; ++c)                                                  \
        r_g[c] = buf_ld2(rg_, g_off, min(g_cq * 4 + c, last_) * g_cs, gout);                         \
    }                                                                                                \
  }

    const size_t part = (size_t)n * tiles + tile;
    // owner threads: entry e of a block's result is D[cell = CELL0 + 4 * (l / 16) + r][channel l % 16]
    // with l = e / 4, r = e % 4 (register r of lane l)
    // ... in two halves, as in the row-window form
#define DK_GW_FLUSH_READ()                                                                           \
  if (threadIdx.x < 256) {                                                                           \
    _Pragma("unroll") for (int w_ = 0; w_ < kWaves; ++w_) fl[w_] = red[w_ * 256 + threadIdx.x];      \
  }
#define DK_GW_FLUSH(cb)                                                                              \
  if (threadIdx.x < 256) {                                                                           \
    float s_ = 0.f;                                                                                  \
    _Pragma("unroll") for (int w_ = 0; w_ < kWaves; ++w_) s_ += fl[w_];                              \
    const int l_ = threadIdx.x / 4, r_ = threadIdx.x % 4;                                            \
    const int cell_ = CELL0 + 4 * (l_ / 16) + r_, cj_ = (cb) * kGfCh + l_ % 16;                      \
    if (cell_ < CELLS && cj_ < cpg)                                                                  \
      partial[(part * g.channel + grp + (size_t)g.groups * cj_) * CELLS + cell_] = s_;               \
  }

    DK_GW_ISSUE(cb_lo, row_lo, col_lo, true)

    gf4 acc = {0.f, 0.f, 0.f, 0.f};
    float fl[kWaves];            // the waves' partial sums of one entry of a block's result, on their way to `partial`
    unsigned d_off[K9];          // per tap, of pixel px + (q & 3): byte offset of the sample's top-left corner in the window
    float d_lh[K9], d_lw[K9];    // ... and its bilinear fractions
    const int steps = nblk * npass;
    for (int it = 0; it < steps; ++it) {
      const int i = it / npass, k = it % npass;
      const int lo_r = row_lo + (k / npc) * (wr - 1), lo_c = col_lo + (k % npc) * (WC - 1);
      __syncthreads();  // the previous step's reads of the planes, the gout tile, the descriptors and `red` are done
      if (it == 0 || npass > 1) {
#pragma unroll
        for (int kk = 0; kk < 3; ++kk) {
          const int t = g_cq + 4 * kk;
          if (t < K9) {
            const bool in_pass = t_row[kk] >= lo_r && t_row[kk] <= lo_r + wr - 2 && t_col[kk] >= lo_c &&
                                 t_col[kk] <= lo_c + WC - 2;  // (row -1: never)
            const unsigned o = in_pass ? (unsigned)((t_row[kk] - lo_r) * WC + t_col[kk] - lo_c) * (kGfPitch * 4) : zero_off;
            hwd[t * kGwPix + g_pix] = make_float4(__uint_as_float(o), t_lh[kk], t_lw[kk], 0.f);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < kGwStage; ++j) {
        const int wrow = s_row + rpp * j;
        if (wrow < wr && wrow <= row_hi + 1 - lo_r) {  // (a position outside the image: zeros were loaded; rows below every sample: not read)
          float* dst = planes + (wrow * WC + s_col) * kGfPitch;
#pragma unroll
          for (int c = 0; c < kGfCh; c += 4)
            *reinterpret_cast<float4*>(dst + c) = make_float4(r_x[j][c], r_x[j][c + 1], r_x[j][c + 2], r_x[j][c + 3]);
        }
      }
      if (k == 0) {
#pragma unroll
        for (int c = 0; c < 4; ++c) gs[(g_cq * 4 + c) * kGwPitchG + g_pix] = r_g[c];
        if (it > 0) *reinterpret_cast<gf4*>(red + (wave * 64 + lane) * 4) = acc;
      }
      __syncthreads();
      if (it + 1 < steps) {
        const int i1 = (it + 1) / npass, k1 = (it + 1) % npass;
        if (k1 == 0) DK_GW_ISSUE(cb_lo + i1, row_lo, col_lo, true)
        else DK_GW_ISSUE(cb_lo + i1, row_lo + (k1 / npc) * (wr - 1), col_lo + (k1 % npc) * (WC - 1), false)
      }
      const bool flush = k == 0 && it > 0;
      if (flush) DK_GW_FLUSH_READ()
      if (k == 0) acc = gf4{0.f, 0.f, 0.f, 0.f};
      if (it == 0 || npass > 1) {  // a lane keeps the descriptors of one of its four pixels, the one of its place in its quad
#pragma unroll
        for (int t = 0; t < K9; ++t) {
          const float4 d = hwd[t * kGwPix + px + (q & 3)];
          d_off[t] = __float_as_uint(d.x), d_lh[t] = d.y, d_lw[t] = d.z;
        }
      }
      {
        gf4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
        const float4 gv = *reinterpret_cast<const float4*>(gs + q * kGwPitchG + px);
        const float gq[4] = {gv.x, gv.y, gv.z, gv.w};
        // corner reads of tap t + 1 ahead of the arithmetic of tap t, descriptors out of the quad's lanes: as in
        // the row-window form
        float cr[2][4][4];
#define DK_GW_CORNER(t, b, ii)                                                                       \
  {                                                                                                  \
    const char* c0 = plane_q + quad_lane<ii>(d_off[t]);                                              \
    const char* c1 = c0 + row_bytes;                                                                 \
    cr[b][ii][0] = *reinterpret_cast<const float*>(c0);                                              \
    cr[b][ii][1] = *reinterpret_cast<const float*>(c0 + kGfPitch * 4);                               \
    cr[b][ii][2] = *reinterpret_cast<const float*>(c1);                                              \
    cr[b][ii][3] = *reinterpret_cast<const float*>(c1 + kGfPitch * 4);                               \
  }
#define DK_GW_CORNERS(t, b) DK_GW_CORNER(t, b, 0) DK_GW_CORNER(t, b, 1) DK_GW_CORNER(t, b, 2) DK_GW_CORNER(t, b, 3)
#define DK_GW_SAMPLE(t, ii)                                                                          \
  {                                                                                                  \
    const float lh = quad_lane<ii>(d_lh[t]), lw = quad_lane<ii>(d_lw[t]);                            \
    const float ca = cr[(t) & 1][ii][0], cb_ = cr[(t) & 1][ii][1], cc = cr[(t) & 1][ii][2], cd = cr[(t) & 1][ii][3]; \
    const float top = fmaf(lw, cb_ - ca, ca), bot = fmaf(lw, cd - cc, cc);                           \
    const float b = fmaf(lh, bot - top, top) * gq[ii];                                               \
    if (((ii) + (t)) & 1)                                                                            \
      acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(A[ii][t], b, acc1, 0, 0, 0);                       \
    else                                                                                             \
      acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(A[ii][t], b, acc0, 0, 0, 0);                       \
  }
        DK_GW_CORNERS(0, 0)
#pragma unroll
        for (int t = 0; t < K9; ++t) {
          if (t + 1 < K9) DK_GW_CORNERS(t + 1, (t + 1) & 1)
          __builtin_amdgcn_sched_barrier(0);
          DK_GW_SAMPLE(t, 0) DK_GW_SAMPLE(t, 1) DK_GW_SAMPLE(t, 2) DK_GW_SAMPLE(t, 3)
          __builtin_amdgcn_sched_barrier(0);
        }
#undef DK_GW_CORNER
#undef DK_GW_CORNERS
#undef DK_GW_SAMPLE
        acc += acc0 + acc1;
      }
      if (flush) DK_GW_FLUSH(cb_lo + i - 1)
    }
    __syncthreads();
    *reinterpret_cast<gf4*>(red + (wave * 64 + lane) * 4) = acc;
    __syncthreads();
    DK_GW_FLUSH_READ()
    DK_GW_FLUSH(cb_lo + nblk - 1)
#undef DK_GW_ISSUE
#undef DK_GW_FLUSH_READ
#undef DK_GW_FLUSH
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
  int block;   // threads of a workgroup
  int tile_pix;  // output pixels of a tile (<= block)
  int wr;        // rows of the LDS window (the row-window forms)
  size_t lds;
};

// table_floats: LDS floats per channel beyond the two planes; plane_floats: LDS floats per plane
// blocks_per_cu: how many workgroups per CU the channel chunking aims at (measured per kernel on
// N=64 C=512 28x28 -> 14x14: grad input 4, grad filter 3, the channel-interleaved kernels 3; the
// one-plane forward 4, grad offset 3, grad rotation 2)
DeformPlan deform_plan(const Geo& g, int table_floats, int planes, int block, int blocks_per_cu,
                       long lds_budget = 64 * 1024, int max_w = 64, int max_passes = 16) {
  DeformPlan d{};
  d.ok = false;
  if (path_disabled(kNoDeformFast)) return d;
  if (g.k_h != 3 || g.k_w != 3 || g.in_w > max_w) return d;
  if (!((g.scope_h == 3 && g.scope_w == 3) || (g.scope_h == 4 && g.scope_w == 4) ||
        (g.scope_h == 5 && g.scope_w == 5)))
    return d;
  if ((long)g.out_h * g.out_w * 18 * 4 >= (1L << 31)) return d;
  d.shift = 0;
  while ((1 << d.shift) < g.in_w) ++d.shift;
  const int rpp = block >> d.shift;
  if (rpp < 1) return d;
  const int np = ceil_div(g.in_h, rpp);
  if (np > max_passes) return d;
  d.npass = np <= 4 ? 4 : np <= 8 ? 8 : np <= 16 ? 16 : 32;
  d.PS = ((g.in_h + 2) * (g.in_w + 2) + 3) & ~3;
  const int cpg = g.channel / g.groups;
  d.tiles = ceil_div(g.out_h * g.out_w, block);
  d.block = d.tile_pix = block;
  const long plane_bytes = (long)planes * d.PS * 4;
  const long room = lds_budget - plane_bytes;
  if (room < (long)table_floats * 4 * 4) return d;
  const int fit = (int)std::min<long>(room / ((long)table_floats * 4), cpg);
  // enough blocks for blocks_per_cu per CU, chunks of at least 8 channels
  const long base = std::max(1L, (long)d.tiles * g.batch * g.groups);  // batch may be 0
  int chunks = (int)std::max<long>(1, (blocks_per_cu * 256L + base - 1) / base);
  chunks = std::min(chunks, std::max(1, cpg / 8));
  chunks = std::max(chunks, ceil_div(cpg, fit));
  d.per = ceil_div(cpg, chunks);
  d.chunks = ceil_div(cpg, d.per);
  d.lds = (size_t)plane_bytes + (size_t)d.per * table_floats * 4;
  if ((long)d.tiles * d.chunks * g.batch * g.groups >= (1L << 31) - 8) return d;
  d.ok = true;
  return d;
}

// Plan of the kernels that interleave kDeformCh channel planes in LDS; ok only when the two
// interleaved buffers, the tables and a four-pass register stage fit.
constexpr int kDeformCh = 4;
static_assert(kDeformCh == kDWinCh, "the row-window kernels interleave as many planes");
constexpr int kDBigBlock = 1024;
constexpr int kDBigBlocksPerCu = 1;
constexpr long kDBigLds = 150 * 1024;

DeformPlan deform_plan_ch(const Geo& g, int table_floats, int blocks_per_cu) {
  DeformPlan d{};
  d.ok = false;
  if (path_disabled(kNoDeformCh)) return d;
  d = deform_plan(g, table_floats, 2 * kDeformCh, kDBlock, blocks_per_cu);
  if (d.ok) {
    d.lds += (size_t)(kDeformCh - 1) * table_floats * 4;  // tables of the channels that pad the last tuple
    d.ok = d.npass == 4 && d.lds <= 64 * 1024;
    if (d.ok) return d;
  }
  // Larger planes (up to 64 x 64): one workgroup of kDBigBlock threads per CU with most of the CU's LDS (its
  // sixteen waves hide the gathers' latency: 512 threads were 25 % slower, more than one channel chunk per
  // CU's worth of workgroups no faster), and tiles of equal size (a plane of 56 x 56 is 4 tiles of 13 waves).
  if (path_disabled(kNoDeformChBig)) { d.ok = false; return d; }
  d = deform_plan(g, table_floats, 2 * kDeformCh, kDBigBlock, kDBigBlocksPerCu,
                  kDBigLds - (long)(kDeformCh - 1) * table_floats * 4);
  if (!d.ok) return d;
  d.lds += (size_t)(kDeformCh - 1) * table_floats * 4;
  d.tile_pix = ceil_div(ceil_div(g.out_h * g.out_w, d.tiles), 64) * 64;
  d.ok = d.npass == 4 && d.lds <= (size_t)kDBigLds;
  return d;
}

// Planes that neither form above takes -- wider than 64 columns, or taller than sixteen staging passes of a
// 256-thread workgroup -- while two padded copies fit a CU's LDS (112 x 112, 130 x 130 in fp32): the one-plane
// kernels in workgroups of kDWideBlock threads, one per CU, staging only the rows a tile's samples touch.
constexpr int kDWideBlock = 512;
constexpr int kDWidePasses = 32;

DeformPlan deform_plan_wide(const Geo& g, int table_floats) {
  return deform_plan(g, table_floats, 2, kDWideBlock, 1, kDBigLds, 1 << 30, kDWidePasses);
}

// The same planes on the channel-interleaved kernels with a row window in LDS: two buffers of `wr` rows of four
// interleaved planes beside the tables of at most 64 channels.  ok only when the window holds the rows a tile's own
// taps span plus a margin for the offsets (otherwise every tile would take several passes and the one-plane
// kernels above are the better choice).
DeformPlan deform_plan_chw(const Geo& g, int table_floats, int block, int npass) {
  DeformPlan d{};
  d.ok = false;
  if (path_disabled(kNoDeformCh) || path_disabled(kNoDeformWindow)) return d;
  // the family's limits, the row mapping and the channel chunks (tables in at most 26 KB)
  d = deform_plan(g, table_floats, 0, block, 1, 26 * 1024, 1 << 30, 1 << 30);
  if (!d.ok) return d;
  d.ok = false;
  const int RS = g.in_w + 2, rpp = block >> d.shift;
  const long table_bytes = (long)(d.per + kDeformCh - 1) * table_floats * 4;
  const long positions = (kDBigLds - table_bytes) / 2 / (kDeformCh * 4) - (RS + 2);
  const long wr = std::min<long>({(long)g.in_h + 2, positions / RS, (long)npass * rpp});
  const long own = (long)(ceil_div(block, g.out_w) + 1) * g.stride_h + 2L * g.dil_h + 2;  // rows without offsets
  // (planes the one-plane kernels cannot take either -- 224 x 224: two padded copies do not fit LDS -- settle
  // for a smaller margin: the alternative there is the generic kernel)
  const long margin = deform_plan_wide(g, table_floats).ok ? 8 : 2;
  if (wr < std::min<long>(g.in_h + 2, own + margin)) return d;
  d.wr = (int)wr;
  d.lds = (size_t)(2 * (wr * RS + RS + 2) * kDeformCh * 4 + table_bytes);
  d.ok = true;
  return d;
}

template <typename T, int SH, int SW>
bool run_deform_forward(const Geo& g, const T* x, const T* off, const T* rot, const T* filter, T* out,
                        hipStream_t stream) {
  // four channel planes interleaved in LDS while a double buffer of them leaves room for the tables
  const DeformPlan d4 = deform_plan_ch(g, WideTable<SH, SW>::SIZE, 3);
  if (d4.ok) {
    const unsigned grid = (unsigned)xcd_grid_size((long)d4.tiles * d4.chunks * g.batch * g.groups);
    if (d4.block == kDBlock) {
      deform_forward_ch_kernel<T, SH, SW, 4, kDeformCh><<<grid, kDBlock, d4.lds, stream>>>(g, x, off, rot, filter, out, d4.per, d4.shift, d4.tile_pix);
      return true;
    }
    auto kernel = deform_forward_ch_kernel<T, SH, SW, 4, kDeformCh, kDBigBlock>;
    if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel)))
      return false;
    kernel<<<grid, kDBigBlock, d4.lds, stream>>>(g, x, off, rot, filter, out, d4.per, d4.shift, d4.tile_pix);
    return true;
  }
  const DeformPlan d = deform_plan(g, WideTable<SH, SW>::SIZE, 2, kDBlock, 4);
  if (!d.ok) {
    const DeformPlan cw = deform_plan_chw(g, WideTable<SH, SW>::SIZE, kDWinFwdBlock, kDWinFwdPass);
    if (cw.ok) {
      auto kernel = deform_forward_chw_kernel<T, SH, SW>;
      if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel))) return false;
      const unsigned cgrid = (unsigned)xcd_grid_size((long)cw.tiles * cw.chunks * g.batch * g.groups);
      kernel<<<cgrid, kDWinFwdBlock, cw.lds, stream>>>(g, x, off, rot, filter, out, cw.per, cw.shift, cw.wr);
      return true;
    }
    const DeformPlan w = deform_plan_wide(g, WideTable<SH, SW>::SIZE);
    if (!w.ok) return false;
    auto kernel = deform_forward_kernel<T, SH, SW, kDWidePasses, kDWideBlock>;
    if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel))) return false;
    const unsigned wgrid = (unsigned)xcd_grid_size((long)w.tiles * w.chunks * g.batch * g.groups);
    kernel<<<wgrid, kDWideBlock, w.lds, stream>>>(g, x, off, rot, filter, out, w.per, w.shift);
    return true;
  }
  const unsigned grid = (unsigned)xcd_grid_size((long)d.tiles * d.chunks * g.batch * g.groups);
#define DK_LAUNCH(NP) \
  deform_forward_kernel<T, SH, SW, NP><<<grid, kDBlock, d.lds, stream>>>(g, x, off, rot, filter, out, d.per, d.shift)
  if (d.npass == 4) DK_LAUNCH(4);
  else if (d.npass == 8) DK_LAUNCH(8);
  else DK_LAUNCH(16);
#undef DK_LAUNCH
  return true;
}


template <typename T, int SH, int SW>
bool run_deform_grad_coord(const Geo& g, bool rotation, const T* gout, const T* x, const T* off, const T* rot,
                           const T* filter, T* result, float* ws, hipStream_t stream) {
  const DeformPlan d4 = deform_plan_ch(g, WideTable<SH, SW>::SIZE, 3);
  DeformPlan d = d4.ok ? d4 : deform_plan(g, WideTable<SH, SW>::SIZE, 2, kDBlock, rotation ? 2 : 3);
  const bool wide = !d.ok;
  bool window = false;
  if (wide) {
    d = deform_plan_chw(g, WideTable<SH, SW>::SIZE, kDWinCoordBlock, kDWinCoordPass);
    window = d.ok;
    if (!window) d = deform_plan_wide(g, WideTable<SH, SW>::SIZE);
  }
  if (!d.ok) return false;
  const unsigned grid = (unsigned)xcd_grid_size((long)d.tiles * d.chunks * g.batch * g.groups);
  if (window) {
    auto kernel = rotation ? deform_grad_coord_chw_kernel<T, SH, SW, 1> : deform_grad_coord_chw_kernel<T, SH, SW, 0>;
    if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel))) return false;
    kernel<<<grid, kDWinCoordBlock, d.lds, stream>>>(g, gout, x, off, rot, filter, ws, d.per, d.shift, d.wr, nullptr);
  } else if (wide) {
    auto kernel = rotation ? deform_grad_coord_kernel<T, SH, SW, kDWidePasses, true, kDWideBlock>
                           : deform_grad_coord_kernel<T, SH, SW, kDWidePasses, false, kDWideBlock>;
    if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel))) return false;
    kernel<<<grid, kDWideBlock, d.lds, stream>>>(g, gout, x, off, rot, filter, ws, d.per, d.shift);
  } else if (d4.ok && d.block == kDBigBlock) {
    auto kernel = rotation ? deform_grad_coord_ch_kernel<T, SH, SW, 4, 1, kDeformCh, kDBigBlock>
                           : deform_grad_coord_ch_kernel<T, SH, SW, 4, 0, kDeformCh, kDBigBlock>;
    if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel)))
      return false;
    kernel<<<grid, kDBigBlock, d.lds, stream>>>(g, gout, x, off, rot, filter, ws, d.per, d.shift, d.tile_pix, nullptr);
  } else if (d4.ok) {
    if (rotation)
      deform_grad_coord_ch_kernel<T, SH, SW, 4, 1, kDeformCh><<<grid, kDBlock, d.lds, stream>>>(g, gout, x, off, rot, filter, ws, d.per, d.shift, d.tile_pix, nullptr);
    else
      deform_grad_coord_ch_kernel<T, SH, SW, 4, 0, kDeformCh><<<grid, kDBlock, d.lds, stream>>>(g, gout, x, off, rot, filter, ws, d.per, d.shift, d.tile_pix, nullptr);
  } else {
#define DK_LAUNCH(NP, ROT)                                                                          \
  deform_grad_coord_kernel<T, SH, SW, NP, ROT><<<grid, kDBlock, d.lds, stream>>>(g, gout, x, off, rot, filter, ws, \
                                                                                 d.per, d.shift)
  if (rotation) {
    if (d.npass == 4) DK_LAUNCH(4, true);
    else if (d.npass == 8) DK_LAUNCH(8, true);
    else DK_LAUNCH(16, true);
  } else {
    if (d.npass == 4) DK_LAUNCH(4, false);
    else if (d.npass == 8) DK_LAUNCH(8, false);
    else DK_LAUNCH(16, false);
  }
#undef DK_LAUNCH
  }
  const int plane18 = 18 * g.out_h * g.out_w;
  if (rotation)
    launch_reduce_partials<float, T>(ws, d.chunks, g.batch * g.groups * plane18, result, stream);
  else
    launch_reduce_partials<float, T>(ws, d.chunks * g.groups, g.batch * plane18, result, stream);
  return true;
}

// Plan of the one-pass offset + rotation gradient: the 256-thread channel-interleaved form, or, for planes up to
// 64 x 64, workgroups of 512 threads (the 45 sums do not fit the 128 registers of the 1024-thread form).
constexpr int kDCoordsBlock = 512;
DeformPlan coords_plan(const Geo& g, int table_floats) {
  DeformPlan d = deform_plan_ch(g, table_floats, 3);
  if (d.ok && d.block == kDBlock) return d;
  if (!d.ok) return d;
  d = deform_plan(g, table_floats, 2 * kDeformCh, kDCoordsBlock, kDBigBlocksPerCu,
                  kDBigLds - (long)(kDeformCh - 1) * table_floats * 4);
  if (!d.ok) return d;
  d.lds += (size_t)(kDeformCh - 1) * table_floats * 4;
  d.tile_pix = ceil_div(ceil_div(g.out_h * g.out_w, d.tiles), 64) * 64;
  d.ok = d.npass <= 8 && d.lds <= (size_t)kDBigLds;
  return d;
}

// ... and its row-window form for the planes that neither of those takes: *d is that plan when it applies
bool coords_window(const Geo& g, int table_floats, DeformPlan* d) {
  // only where no other channel-interleaved or one-plane 256-thread form serves the shape (as in run_deform_grad_coord)
  if (deform_plan_ch(g, table_floats, 3).ok || deform_plan(g, table_floats, 2, kDBlock, 2).ok) return false;
  const DeformPlan w = deform_plan_chw(g, table_floats, kDWinCoordBlock, kDWinCoordPass);
  if (w.ok) *d = w;
  return w.ok;
}

// Offset and rotation gradient from one pass (MODE 2 of the channel-interleaved kernel in 256-thread workgroups: its
// 45 sums fit their register budget, not that of the 1024-thread form); false where that form does not apply.
// Workspace: the rotation partials, then the offset partials (the same number of floats).
template <typename T, int SH, int SW>
bool run_deform_grad_coords(const Geo& g, const T* gout, const T* x, const T* off, const T* rot, const T* filter,
                            T* goff, T* grot, float* ws, hipStream_t stream) {
  DeformPlan d = coords_plan(g, WideTable<SH, SW>::SIZE);
  const bool window = !d.ok && coords_window(g, WideTable<SH, SW>::SIZE, &d);
  if (!d.ok) return false;
  const int plane18 = 18 * g.out_h * g.out_w;
  float* ws_off = ws + (size_t)d.chunks * g.groups * g.batch * plane18;
  const unsigned grid = (unsigned)xcd_grid_size((long)d.tiles * d.chunks * g.batch * g.groups);
  if (window) {
    auto kernel = deform_grad_coord_chw_kernel<T, SH, SW, 2>;
    if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel))) return false;
    kernel<<<grid, kDWinCoordBlock, d.lds, stream>>>(g, gout, x, off, rot, filter, ws, d.per, d.shift, d.wr, ws_off);
  } else if (d.block == kDBlock) {
    deform_grad_coord_ch_kernel<T, SH, SW, 4, 2, kDeformCh><<<grid, kDBlock, d.lds, stream>>>(g, gout, x, off, rot, filter, ws, d.per, d.shift, d.tile_pix, ws_off);
  } else {
    auto kernel = deform_grad_coord_ch_kernel<T, SH, SW, 8, 2, kDeformCh, kDCoordsBlock>;
    if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel))) return false;
    kernel<<<grid, kDCoordsBlock, d.lds, stream>>>(g, gout, x, off, rot, filter, ws, d.per, d.shift, d.tile_pix, ws_off);
  }
  launch_reduce_partials<float, T>(ws, d.chunks, g.batch * g.groups * plane18, grot, stream);
  launch_reduce_partials<float, T>(ws_off, d.chunks * g.groups, g.batch * plane18, goff, stream);
  return true;
}

// blockDim of the grad-input kernel: it owns a whole output plane
int grad_input_block(const Geo& g) { return ceil_div(g.out_h * g.out_w, 64) * 64; }

template <int SH, int SW>
DeformPlan grad_input_plan(const Geo& g) {
  DeformPlan d{};
  d.ok = false;
  if (g.out_h * g.out_w > 1024) return d;
  // 4 floats of LDS per plane element (two 64-bit planes), one more float per channel for max|Wt[c]|
  return deform_plan(g, WideTable<SH, SW>::SIZE + 1, 4, grad_input_block(g), 4);
}

// 64-bit planes per workgroup of the tiled grad input (it owns twice as many channels): 4, 2 or 1, as many as fit
// LDS; 0 if not even one.
template <int SH, int SW>
int tiled_planes(const DeformPlan& basic, size_t* lds) {
  for (int np = 4; np >= 1; np >>= 1) {
    *lds = ((size_t)2 * np * basic.PS + (size_t)2 * np * WideTable<SH, SW>::SIZE + 2 * np) * sizeof(float);
    if (*lds <= 150 * 1024) return np;
  }
  return 0;
}

// Band form of the tiled grad input: 64-bit planes per workgroup (4, 2 or 1) and rows per band, the largest
// plane count that leaves bands of at least kBandRows rows (fewer rows: every tile is walked by many bands); 0 if
// not even one plane of 8 rows fits.
constexpr int kBandRows = 20;
template <int SH, int SW>
int band_planes(const Geo& g, int* rows, size_t* lds) {
  const long RS = g.in_w + 2;
  for (int np = 4; np >= 1; np >>= 1) {
    const long fixed = ((long)2 * np * WideTable<SH, SW>::SIZE + 2 * np) * 4 + 64;
    const long r = std::min<long>(g.in_h, (150L * 1024 - fixed) / (np * RS * 8) - 1);
    if (r >= std::min<long>(g.in_h, np == 1 ? 8 : kBandRows)) {
      *rows = (int)r;
      *lds = (size_t)(2 * np * (((r * RS + 3) & ~3L)) * 4 + fixed);
      return np;
    }
  }
  return 0;
}

template <typename T, int SH, int SW>
bool run_deform_grad_input(const Geo& g, const T* gout, const T* off, const T* rot, const T* filter, T* gin,
                           void* ws, hipStream_t stream) {
  const DeformPlan d = grad_input_plan<SH, SW>(g);
  const bool tiled = !d.ok;  // output planes of more than 1024 pixels, input planes wider than 64 columns
  size_t tiled_lds = 0;
  int tiled_shift = 0, tiled_ch = 0;
  if (tiled) {
    // the basic limits of the tuned family (any width: the read-back loop walks the rows), then room for the 64-bit planes
    const DeformPlan basic = deform_plan(g, WideTable<SH, SW>::SIZE, 0, 1024, 2, 64 * 1024, 1 << 30, 1 << 30);
    if (!basic.ok) return false;
    tiled_shift = basic.shift;
    tiled_ch = tiled_planes<SH, SW>(basic, &tiled_lds);
  }
  if (reinterpret_cast<uintptr_t>(gout) % 16 != 0) return false;  // absmax_kernel reads 16-byte vectors
  unsigned* gmax = static_cast<unsigned*>(ws);
  const long n = (long)g.batch * g.channel * g.out_h * g.out_w;
  if (tiled) {
    // workspace: the maxima of |gout|, the images' sample counts, the tiles' rows
    unsigned* most_img = gmax + kAbsParts;
    int* table = reinterpret_cast<int*>(most_img + g.batch);
    const int ntiles = ceil_div(g.out_h * g.out_w, 1024), cpg = g.channel / g.groups;
    // the counting kernel's bands: about 512 workgroups, of at least 8 rows, of at most what fits as 32-bit counters
    const long cfit = (150L * 1024 / 4) / (g.in_w + 2) - 1;
    const int cbands = std::max(1, std::min(g.in_h / 8, ceil_div(512, std::max(1, g.batch))));
    const int crows = (int)std::min<long>(cfit, ceil_div(g.in_h, cbands));
    auto count_kernel = deform_sample_count_kernel<T>;
    if (crows < 1 || !allow_max_dynamic_lds(reinterpret_cast<const void*>(count_kernel))) return false;
    // not even one 64-bit plane fits, or only one (two channels per workgroup and walk): bands of rows
    size_t blds = 0;
    int brows = 0;
    const int bnp = tiled_ch <= 1 && !path_disabled(kNoDeformWindow) ? band_planes<SH, SW>(g, &brows, &blds) : 0;
    const bool band = bnp >= 2 || (tiled_ch == 0 && bnp == 1);
    if (!band && tiled_ch == 0) return false;
    const int np = band ? bnp : tiled_ch;
    const size_t lds = band ? blds : tiled_lds;
    const unsigned tgrid = (unsigned)xcd_grid_size((long)(band ? ceil_div(g.in_h, brows) : 1) * ceil_div(cpg, 2 * np) * g.batch * g.groups);
#define DK_LAUNCH(CH, BAND)                                                                                       \
  {                                                                                                               \
    auto kernel = deform_grad_input_tiled_kernel<T, SH, SW, CH, BAND>;                                            \
    if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel))) return false;                              \
    absmax_kernel<T><<<kAbsParts, 256, 0, stream>>>(gout, n, gmax);                                               \
    deform_tile_rows_kernel<T><<<(unsigned)(g.batch * ntiles), 1024, 0, stream>>>(g, off, table, ntiles, most_img); \
    count_kernel<<<(unsigned)(g.batch * ceil_div(g.in_h, crows)), 1024, (size_t)crows * (g.in_w + 2) * 4, stream>>>( \
        g, off, table, most_img, ntiles, crows);                                                                  \
    kernel<<<tgrid, 1024, lds, stream>>>(g, gout, off, rot, filter, gin, gmax, tiled_shift, brows, table, most_img); \
  }
    if (band) {
      if (np == 4) DK_LAUNCH(4, true) else if (np == 2) DK_LAUNCH(2, true) else DK_LAUNCH(1, true)
    } else {
      if (np == 4) DK_LAUNCH(4, false) else if (np == 2) DK_LAUNCH(2, false) else DK_LAUNCH(1, false)
    }
#undef DK_LAUNCH
    return true;
  }
  absmax_kernel<T><<<kAbsParts, 256, 0, stream>>>(gout, n, gmax);
  const unsigned grid = (unsigned)xcd_grid_size((long)d.chunks * g.batch * g.groups);
  deform_grad_input_kernel<T, SH, SW><<<grid, grad_input_block(g), d.lds, stream>>>(g, gout, off, rot, filter, gin, gmax,
                                                                                   d.per, d.shift);
  return true;
}

// Launch shape of the matrix-core grad filter, ok when the geometry fits it.
struct GradFilterMfma {
  bool ok;
  int tiles, csplits, shift;
  size_t lds;
};
GradFilterMfma grad_filter_mfma_plan(const Geo& g) {
  GradFilterMfma m{};
  m.ok = false;
  if (path_disabled(kNoDeformMfma)) return m;
  const DeformPlan basic = deform_plan(g, 64, 0, kGfBlock, 1);  // the family's limits and the row mapping only
  if (!basic.ok) return m;
  m.shift = basic.shift;
  if (g.in_h > (kGfBlock >> m.shift)) return m;  // a thread per plane position
  const long PS = (long)(g.in_h + 2) * (g.in_w + 2);
  const long floats = PS * kGfPitch + (long)kGfCh * kGfPitchG + 4L * K9 * kGfPix +
                      std::max((kGfBlock / 64) * 256, 2 * K9 * kGfPix);
  if (floats * 4 > 150 * 1024) return m;
  m.lds = (size_t)floats * 4;
  m.tiles = ceil_div(g.out_h * g.out_w, kGfPix);
  const int nblk = ceil_div(g.channel / g.groups, kGfCh);
  const long base = std::max(1L, (long)m.tiles * g.batch * g.groups);  // batch may be 0
  // one workgroup per CU, all resident at once: the set-up of a workgroup (descriptors, hat products,
  // zero fill) costs about as much as two channel blocks (measured: 256 workgroups 73 us, 512: 79, 1024: 93)
  m.csplits = (int)std::max<long>(1, std::min<long>(nblk, (256 + base - 1) / base));
  if (base * m.csplits >= (1L << 31) - 8) return m;
  m.ok = true;
  return m;
}

// Launch shape of its row-window form (planes of up to 64 columns that the form above does not hold)
struct GradFilterWin {
  bool ok;
  int tiles, nwg, shift, wr;
  size_t lds;
};
GradFilterWin grad_filter_win_plan(const Geo& g) {
  GradFilterWin m{};
  m.ok = false;
  if (path_disabled(kNoDeformMfma) || path_disabled(kNoDeformWindow)) return m;
  const DeformPlan basic = deform_plan(g, 64, 0, kGwBlock, 1);  // the family's limits and the row mapping only
  if (!basic.ok) return m;
  m.shift = basic.shift;
  const int RS = g.in_w + 2, rpp = kGwBlock >> m.shift;
  const long fixed = (long)kGfCh * kGwPitchG + 4L * K9 * kGwPix + std::max((kGwBlock / 64) * 256, 2 * K9 * kGwPix) + 4;
  const long positions = (150L * 1024 / 4 - fixed) / kGfPitch - (RS + 2);  // window positions that fit beside the tables
  const long wr = std::min<long>({(long)g.in_h + 2, positions / RS, (long)kGwStage * rpp});
  if (wr < 8) return m;
  m.wr = (int)wr;
  m.lds = (size_t)((wr * RS + RS + 2) * kGfPitch + fixed) * 4;
  m.tiles = ceil_div(g.out_h * g.out_w, kGwPix);
  const int nblk = ceil_div(g.channel / g.groups, kGfCh);
  const long base = std::max(1L, (long)m.tiles * g.batch * g.groups);  // batch may be 0
  if (base >= (1L << 31) - 8) return m;
  m.nwg = (int)std::min<long>(base * nblk, kGwGrid);  // persistent workgroups, one per CU, equal shares of the channel blocks
  m.ok = true;
  return m;
}

// ... and of the form with a window in rows and columns (any plane of the family)
struct GradFilterWin2 {
  bool ok;
  int tiles_x, tiles, nwg, wr;
  size_t lds;
};
GradFilterWin2 grad_filter_win2_plan(const Geo& g) {
  GradFilterWin2 m{};
  m.ok = false;
  if (path_disabled(kNoDeformMfma) || path_disabled(kNoDeformWindow)) return m;
  const DeformPlan basic = deform_plan(g, 64, 0, kGwBlock, 1, 64 * 1024, 1 << 30, 1 << 30);  // the family's limits only
  if (!basic.ok) return m;
  // the window must hold a tile's own taps and a margin for the offsets, or every tile takes several passes
  if ((kG2Tw - 1) * g.stride_w + 2 * g.dil_w + 2 + 8 > kG2Wc) return m;
  const long own = (long)(kG2Th - 1) * g.stride_h + 2L * g.dil_h + 2;
  const long fixed = (long)kGfCh * kGwPitchG + 4L * K9 * kGwPix + std::max((kGwBlock / 64) * 256, 2 * K9 * kGwPix) + 4;
  const long positions = (150L * 1024 / 4 - fixed) / kGfPitch - (kG2Wc + 2);
  const long wr = std::min<long>({(long)g.in_h + 2, positions / kG2Wc, (long)kGwStage * (kGwBlock / kG2Wc)});
  if (wr < std::min<long>(g.in_h + 2, own + 8)) return m;
  m.wr = (int)wr;
  m.lds = (size_t)((wr * kG2Wc + kG2Wc + 2) * kGfPitch + fixed) * 4;
  m.tiles_x = ceil_div(g.out_w, kG2Tw);
  m.tiles = m.tiles_x * ceil_div(g.out_h, kG2Th);
  const int nblk = ceil_div(g.channel / g.groups, kGfCh);
  const long base = std::max(1L, (long)m.tiles * g.batch * g.groups);  // batch may be 0
  if (base >= (1L << 31) - 8) return m;
  m.nwg = (int)std::min<long>(base * nblk, kGwGrid);  // persistent workgroups, one per CU, equal shares of the channel blocks
  m.ok = true;
  return m;
}

template <typename T, int SH, int SW, int CELL0>
bool launch_deform_grad_filter_win2(const Geo& g, const GradFilterWin2& m, const T* gout, const T* x, const T* off,
                                    const T* rot, float* ws, hipStream_t stream) {
  auto kernel = deform_grad_filter_win2_kernel<T, SH, SW, CELL0>;
  if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel))) return false;
  const unsigned grid = (unsigned)xcd_grid_size(m.nwg);
  kernel<<<grid, kGwBlock, m.lds, stream>>>(g, gout, x, off, rot, ws, m.tiles_x, m.tiles, m.nwg, m.wr);
  return true;
}

template <typename T, int SH, int SW, int CELL0>
bool launch_deform_grad_filter_win(const Geo& g, const GradFilterWin& m, const T* gout, const T* x, const T* off,
                                   const T* rot, float* ws, hipStream_t stream) {
  const unsigned grid = (unsigned)xcd_grid_size(m.nwg);
  auto kernel = deform_grad_filter_win_kernel<T, SH, SW, CELL0>;
  if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel))) return false;
  kernel<<<grid, kGwBlock, m.lds, stream>>>(g, gout, x, off, rot, ws, m.tiles, m.nwg, m.shift, m.wr);
  return true;
}

template <typename T, int SH, int SW, int CELL0>
bool launch_deform_grad_filter_mfma(const Geo& g, const GradFilterMfma& m, const T* gout, const T* x, const T* off,
                                    const T* rot, float* ws, hipStream_t stream) {
  auto kernel = deform_grad_filter_mfma_kernel<T, SH, SW, CELL0>;
  if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel)))
    return false;
  const unsigned grid = (unsigned)xcd_grid_size((long)m.tiles * m.csplits * g.batch * g.groups);
  kernel<<<grid, kGfBlock, m.lds, stream>>>(g, gout, x, off, rot, ws, m.tiles, m.csplits, m.shift);
  return true;
}

template <typename T, int SH, int SW>
bool run_deform_grad_filter(const Geo& g, const T* gout, const T* x, const T* off, const T* rot, T* gfilter,
                            float* ws, hipStream_t stream) {
  const bool fit = block_planes_fit<T>(g);  // (the matrix-core forms address a block's channels through one descriptor)
  const GradFilterMfma m = grad_filter_mfma_plan(g);
  if (m.ok && fit) {
    if (!launch_deform_grad_filter_mfma<T, SH, SW, 0>(g, m, gout, x, off, rot, ws, stream)) return false;
    if constexpr (SH * SW > 16)
      if (!launch_deform_grad_filter_mfma<T, SH, SW, 16>(g, m, gout, x, off, rot, ws, stream)) return false;
    launch_reduce_partials<float, T>(ws, g.batch * m.tiles, g.channel * SH * SW, gfilter, stream);
    return true;
  }
  const GradFilterWin2 w2 = grad_filter_win2_plan(g);
  const GradFilterWin wn = grad_filter_win_plan(g);
  if (fit && w2.ok && (!wn.ok || path_disabled(kForceWin2))) {
    if (!launch_deform_grad_filter_win2<T, SH, SW, 0>(g, w2, gout, x, off, rot, ws, stream)) return false;
    if constexpr (SH * SW > 16)
      if (!launch_deform_grad_filter_win2<T, SH, SW, 16>(g, w2, gout, x, off, rot, ws, stream)) return false;
    launch_reduce_partials<float, T>(ws, g.batch * w2.tiles, g.channel * SH * SW, gfilter, stream);
    return true;
  }
  if (fit && wn.ok) {
    if (!launch_deform_grad_filter_win<T, SH, SW, 0>(g, wn, gout, x, off, rot, ws, stream)) return false;
    if constexpr (SH * SW > 16)
      if (!launch_deform_grad_filter_win<T, SH, SW, 16>(g, wn, gout, x, off, rot, ws, stream)) return false;
    launch_reduce_partials<float, T>(ws, g.batch * wn.tiles, g.channel * SH * SW, gfilter, stream);
    return true;
  }
  if constexpr (SH * SW > 16) {
    return false;  // 25 dense accumulators and 90 hat weights per lane do not fit the register budget
  } else {
    const DeformPlan d = deform_plan(g, (kDBlock / 64) * SH * SW, 2, kDBlock, 3);
    if (!d.ok) {
      const DeformPlan w = deform_plan_wide(g, (kDWideBlock / 64) * SH * SW);
      if (!w.ok) return false;
      auto kernel = deform_grad_filter_kernel<T, SH, SW, kDWidePasses, kDWideBlock>;
      if (!allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel))) return false;
      const unsigned wgrid = (unsigned)xcd_grid_size((long)w.tiles * w.chunks * g.batch * g.groups);
      kernel<<<wgrid, kDWideBlock, w.lds, stream>>>(g, gout, x, off, rot, ws, w.per, w.shift);
      launch_reduce_partials<float, T>(ws, g.batch * w.tiles, g.channel * SH * SW, gfilter, stream);
      return true;
    }
    const unsigned grid = (unsigned)xcd_grid_size((long)d.tiles * d.chunks * g.batch * g.groups);
#define DK_LAUNCH(NP) \
  deform_grad_filter_kernel<T, SH, SW, NP><<<grid, kDBlock, d.lds, stream>>>(g, gout, x, off, rot, ws, d.per, d.shift)
    if (d.npass == 4) DK_LAUNCH(4);
    else if (d.npass == 8) DK_LAUNCH(8);
    else DK_LAUNCH(16);
#undef DK_LAUNCH
    launch_reduce_partials<float, T>(ws, g.batch * d.tiles, g.channel * SH * SW, gfilter, stream);
    return true;
  }
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


template <typename T>
bool fast_deform_grad_coord(const Geo& g, bool rotation, const T* gout, const T* x, const T* off, const T* rot,
                            const T* filter, T* result, void* ws, hipStream_t stream) {
#define CALL(SH, SW) \
  run_deform_grad_coord<T, SH, SW>(g, rotation, gout, x, off, rot, filter, result, static_cast<float*>(ws), stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

size_t fast_deform_grad_coord_workspace(const Geo& g, bool rotation) {
  const int table = g.scope_h == 3 ? WideTable<3, 3>::SIZE : g.scope_h == 4 ? WideTable<4, 4>::SIZE : WideTable<5, 5>::SIZE;
  const DeformPlan d4 = deform_plan_ch(g, table, 3);
  DeformPlan d = d4.ok ? d4 : deform_plan(g, table, 2, kDBlock, rotation ? 2 : 3);
  if (!d.ok) d = deform_plan_chw(g, table, kDWinCoordBlock, kDWinCoordPass);
  if (!d.ok) d = deform_plan_wide(g, table);
  if (!d.ok) return 0;
  // both lay out chunks * groups * batch planes of 18 * out pixels
  return (size_t)d.chunks * g.groups * g.batch * 18 * g.out_h * g.out_w * sizeof(float);
}

size_t fast_deform_grad_coords_workspace(const Geo& g) {
  const int table = g.scope_h == 3 ? WideTable<3, 3>::SIZE : g.scope_h == 4 ? WideTable<4, 4>::SIZE : WideTable<5, 5>::SIZE;
  DeformPlan d = coords_plan(g, table);
  if (!d.ok) coords_window(g, table, &d);
  if (!d.ok) return 0;
  return 2 * (size_t)d.chunks * g.groups * g.batch * 18 * g.out_h * g.out_w * sizeof(float);
}

template <typename T>
bool fast_deform_grad_coords(const Geo& g, const T* gout, const T* x, const T* off, const T* rot, const T* filter,
                             T* goff, T* grot, void* ws, hipStream_t stream) {
#define CALL(SH, SW) \
  run_deform_grad_coords<T, SH, SW>(g, gout, x, off, rot, filter, goff, grot, static_cast<float*>(ws), stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

template <typename T>
bool fast_deform_grad_input(const Geo& g, const T* gout, const T* off, const T* rot, const T* filter, T* gin,
                            void* ws, hipStream_t stream) {
#define CALL(SH, SW) run_deform_grad_input<T, SH, SW>(g, gout, off, rot, filter, gin, ws, stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

size_t fast_deform_grad_input_workspace(const Geo& g) {
  // absmax_kernel's per-workgroup maxima of |gout|, then the tiled form's sample count per image and its table of
  // two rows per (image, tile)
  return (size_t)kAbsParts * sizeof(unsigned) + (size_t)g.batch * sizeof(unsigned) +
         (size_t)g.batch * ceil_div(g.out_h * g.out_w, 1024) * 2 * sizeof(int);
}

template <typename T>
bool fast_deform_grad_filter(const Geo& g, const T* gout, const T* x, const T* off, const T* rot, T* gfilter,
                             void* ws, hipStream_t stream) {
#define CALL(SH, SW) run_deform_grad_filter<T, SH, SW>(g, gout, x, off, rot, gfilter, static_cast<float*>(ws), stream)
  DK_DISPATCH_SCOPE(g, CALL)
#undef CALL
}

size_t fast_deform_grad_filter_workspace(const Geo& g) {  // one partial per (image, tile); the form with the most tiles
  const long tiles = std::max<long>(ceil_div(g.out_h * g.out_w, kGwPix), (long)ceil_div(g.out_w, kG2Tw) * ceil_div(g.out_h, kG2Th));
  return (size_t)g.batch * tiles * g.channel * g.scope_h * g.scope_w * sizeof(float);
}

#define DK_INSTANTIATE(T)                                                                              \
  template bool fast_deform_forward<T>(const Geo&, const T*, const T*, const T*, const T*, T*, hipStream_t);      \
  template bool fast_deform_grad_coord<T>(const Geo&, bool, const T*, const T*, const T*, const T*, const T*, T*,  \
                                          void*, hipStream_t);                                                     \
  template bool fast_deform_grad_coords<T>(const Geo&, const T*, const T*, const T*, const T*, const T*, T*, T*,    \
                                           void*, hipStream_t);                                                    \
  template bool fast_deform_grad_input<T>(const Geo&, const T*, const T*, const T*, const T*, T*, void*,           \
                                          hipStream_t);                                                            \
  template bool fast_deform_grad_filter<T>(const Geo&, const T*, const T*, const T*, const T*, T*, void*,          \
                                           hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
#undef DK_INSTANTIATE

}  // namespace dk
