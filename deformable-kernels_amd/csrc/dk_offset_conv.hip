// The offset branch of a deformable-kernel layer: the 3x3 convolution that predicts the
// kernel-space offsets ("rotation_conv", reference modules/deform_kernel.py:165-168 and :214-216:
// nn.Conv2d(in_planes, rotation_groups * k * k * 2, k, stride, padding, dilation, bias=True)).
// It has many input channels and only 18 output channels per rotation group, a shape on which
// the library convolution spends twice the time of the deformable-kernel operator itself.
//
// Forward as a shift-GEMM on the matrix cores, full fp32 (v_mfma_f32_16x16x4_f32):
//   out[o][p] = bias[o] + sum over taps t, channels c of W[o][c][t] * x[c][p + shift_t].
// A workgroup owns a tile of TH rows of one image (up to 448 pixels = 28 groups of 16 pixels,
// seven per wave) and walks the input channels in chunks of 16, staged zero-padded in LDS.
// Per tap and 4 channels one MFMA per pixel group multiplies the 16 x 4 block of weights
// (outputs 0..15; A operand, from the chunk's slice of the packed copy [tap][c][16] in LDS) with
// the 4 x 16 block of shifted inputs (B operand, one LDS read per lane: lane = (channel k,
// pixel n); the channel pitch is 16 mod 64 words so the four channels of a read hit disjoint
// banks).  The outputs beyond the 16th (two of the 18) are summed on the vector ALU, their
// weights staged in LDS per chunk and read as broadcasts.  Stride 1, padding 1, no dilation; other cases are left
// to the caller's library convolution.  16-bit tensors (fp16 / bf16) take the same kernels: their elements are
// converted to fp32 on the way into LDS, the products and sums are fp32, the results are rounded once.
#include <algorithm>

#include "dk_kernels.h"

namespace dk {

namespace {

constexpr int kCvBlock = 256;
constexpr int kCvChunk = 16;     // input channels staged per pass
constexpr int kCvGroups = 7;     // 16-pixel groups per wave
constexpr int kCvTilePix = kCvGroups * 16 * (kCvBlock / 64);  // 448

typedef float v4f __attribute__((ext_vector_type(4)));

struct ConvGeo {
  int batch, cin, cout, h;
  int tiles;  // row tiles per image
};

// The plane width is a template constant, so that every LDS offset of the unrolled tap / channel
// loops is an immediate: rows per tile, 64-column segments per staged row, floats per staged
// row and per staged channel (rounded up to 16 mod 64).
template <int W>
struct ConvTile {
  static constexpr int TH = W <= 56 ? 8 : 4;  // (4 and 2 rows at width 56 measured slower: more halo rows staged)
  static constexpr int SEGS = (W + 63) / 64;
  static constexpr int RS = W + 2;
  static constexpr int PS = ((TH + 2) * RS + 47) / 64 * 64 + 16;
  static_assert(TH * W <= kCvTilePix && PS >= (TH + 2) * RS && PS % 64 == 16, "tile does not fit the workgroup");
};

// weights [cout][cin][3][3] -> w16 [9][cin][16] (outputs 0..15, zero where cout < 16) and
// wrest [9][cin][rest] (outputs 16..)
template <typename T>
__global__ void conv_pack_weights_kernel(const T* __restrict__ w, int cout, int cin, int rest,
                                         float* __restrict__ w16, float* __restrict__ wrest) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < 9 * cin * 16) {
    const int m = idx % 16, c = idx / 16 % cin, t = idx / 16 / cin;
    w16[idx] = m < cout ? ld(w + ((size_t)m * cin + c) * 9 + t) : 0.f;
  }
  if (idx < 9 * cin * rest) {
    const int o = 16 + idx % rest, c = idx / rest % cin, t = idx / rest / cin;
    wrest[idx] = ld(w + ((size_t)o * cin + c) * 9 + t);
  }
}

template <typename T, int W, int REST>
__global__ __launch_bounds__(kCvBlock, 2) void offset_conv_forward_kernel(
    ConvGeo g, const T* __restrict__ x, const float* __restrict__ w16, const float* __restrict__ wrest,
    const T* __restrict__ bias, T* __restrict__ out, float* __restrict__ partial, int ksplit) {
  extern __shared__ __align__(16) float xs[];  // [kCvChunk][PS], the chunk's VALU-path weights [kCvChunk][9][REST], its MFMA weights [9][256]
  constexpr int TH = ConvTile<W>::TH, SEGS = ConvTile<W>::SEGS, RS = ConvTile<W>::RS, PS = ConvTile<W>::PS;
  constexpr int kStage = (kCvChunk / 4) * (TH + 2) * SEGS;  // row segments of 64 columns a wave stages per chunk
  constexpr int kPixPerThread = (kCvTilePix + kCvBlock - 1) / kCvBlock;  // of the VALU path

  // logical block = (input-channel split, row tile, image), split fastest.  With ksplit > 1 (small
  // planes, where (image, tile) alone gives too few workgroups) a workgroup sums a share of the
  // channel chunks and writes partial[split][...]; the splits are added afterwards, in order.
  const int total = g.batch * g.tiles * ksplit;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int split = lb % ksplit, n = lb / ksplit / g.tiles, r0 = (lb / ksplit % g.tiles) * TH;
  // the wave index enters scalar offsets and loop bounds: tell the compiler it is uniform
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int tile_pix = TH * W, groups = (tile_pix + 15) / 16;
  constexpr int GPW = (groups + 3) / 4;  // pixel groups per wave; a wave with fewer repeats its last pixel (not stored)

  // LDS float index of the lane's pixel of each group (padded coordinates), plus the lane's
  // channel of a 4-channel step
  int base[GPW];
#pragma unroll
  for (int i = 0; i < GPW; ++i) {
    const int q = min((wave + 4 * i) * 16 + (lane & 15), tile_pix - 1);
    base[i] = (q / W + 1) * RS + q % W + 1 + (lane >> 4) * PS;
  }
  int rbase[kPixPerThread];
#pragma unroll
  for (int j = 0; j < kPixPerThread; ++j) {
    const int q = min((int)threadIdx.x + kCvBlock * j, tile_pix - 1);
    rbase[j] = (q / W + 1) * RS + q % W + 1;
  }

  for (int e = threadIdx.x; e < kCvChunk * PS; e += kCvBlock) xs[e] = 0.f;  // the padding stays zero

  v4f acc[GPW];
#pragma unroll
  for (int i = 0; i < GPW; ++i) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
  float racc[kPixPerThread][REST > 0 ? REST : 1];
#pragma unroll
  for (int j = 0; j < kPixPerThread; ++j)
#pragma unroll
    for (int o = 0; o < (REST > 0 ? REST : 1); ++o) racc[j][o] = 0.f;

  // staging: wave w takes channels w, w + 4, w + 8, w + 12 of the chunk; its i-th row segment is
  // (channel w + 4 * (i / rows), staged row, 64-column segment).  Buffer loads: the lane part of
  // the address is one register per segment, the (channel, row) part a scalar offset (which
  // the hardware's range check does not see, so it must stay inside the chunk), and rows or
  // columns outside the image read 0 through an out-of-range lane offset.
  const int plane = g.h * W;
  unsigned vcol[SEGS];
#pragma unroll
  for (int sg = 0; sg < SEGS; ++sg)
    vcol[sg] = sg * 64 + lane < W ? (unsigned)((sg * 64 + lane) * sizeof(T)) : kOutOfRange;
  const int lds_row0 = wave * PS + 1 + lane;  // + immediate per row segment
  float stage[kStage];
  // the chunk's weights of the outputs beyond the 16th go through LDS as well: read as scalars
  // from memory they cost a round trip per (channel, tap)
  constexpr int kRestW = kCvChunk * 9 * REST, kRestPerThread = (kRestW + kCvBlock - 1) / kCvBlock;
  float* wl = xs + kCvChunk * PS;
  float wstage[kRestPerThread > 0 ? kRestPerThread : 1];
  // The chunk's matrix-core weights [9][16 channels][16 outputs] travel through LDS too, loaded
  // with the next chunk's inputs, so that the multiply loop holds LDS reads and MFMAs only.
  float* wa = wl + kCvChunk * 9 * REST;
  float astage[9];
#define DK_LOAD_CHUNK(CK)                                                                                  \
  {                                                                                                        \
    _Pragma("unroll") for (int t = 0; t < 9; ++t)                                                          \
      astage[t] = w16[((size_t)t * g.cin + (size_t)(CK) * kCvChunk) * 16 + threadIdx.x];                   \
    _Pragma("unroll") for (int u = 0; u < kRestPerThread; ++u) {                                           \
      const int e = (int)threadIdx.x + kCvBlock * u; /* = (c * 9 + t) * REST + o */                        \
      const int o = e % (REST > 0 ? REST : 1), t = e / (REST > 0 ? REST : 1) % 9, c = e / (REST > 0 ? REST : 1) / 9; \
      wstage[u] = e < kRestW ? wrest[((size_t)t * g.cin + (CK) * kCvChunk + c) * REST + o] : 0.f;          \
    }                                                                                                      \
    const rsrc_t rx = plane_rsrc(x + ((size_t)n * g.cin + (size_t)(CK) * kCvChunk) * plane, kCvChunk * plane); \
    _Pragma("unroll") for (int i = 0; i < kStage; ++i) {                                                   \
      const int chq = i / ((TH + 2) * SEGS), ry = i / SEGS % (TH + 2), sg = i % SEGS;                      \
      const int row = r0 - 1 + ry;                                                                         \
      const bool ok = row >= 0 && row < g.h;                                                               \
      const int soff = ok ? ((wave + 4 * chq) * g.h + row) * W * (int)sizeof(T) : 0;                       \
      stage[i] = buf_ld2(rx, ok ? vcol[sg] : kOutOfRange, soff, x);                                        \
    }                                                                                                      \
  }

  const int per_split = ceil_div(g.cin / kCvChunk, ksplit);
  const int ck_begin = split * per_split, nchunks = min(g.cin / kCvChunk, ck_begin + per_split);
  if (ck_begin < nchunks) DK_LOAD_CHUNK(ck_begin)
  for (int ck = ck_begin; ck < nchunks; ++ck) {
    __syncthreads();  // every wave is done with the previous chunk
#pragma unroll
    for (int i = 0; i < kStage; ++i) {
      const int chq = i / ((TH + 2) * SEGS), ry = i / SEGS % (TH + 2), sg = i % SEGS;
      if (sg * 64 + lane < W) xs[lds_row0 + 4 * chq * PS + ry * RS + sg * 64] = stage[i];
    }
#pragma unroll
    for (int u = 0; u < kRestPerThread; ++u)
      if ((int)threadIdx.x + kCvBlock * u < kRestW) wl[threadIdx.x + kCvBlock * u] = wstage[u];
#pragma unroll
    for (int t = 0; t < 9; ++t) wa[t * 256 + threadIdx.x] = astage[t];
    __syncthreads();
    if (ck + 1 < nchunks) DK_LOAD_CHUNK(ck + 1)

    // matrix-core part: outputs 0..15
    // A operand of (tap t, channels 4 cs .. 4 cs + 3): wa[t][4 cs + k][m], lane = 16 k + m
    // 36 steps (tap, 4 channels); the B operands of the next step are read from LDS before the
    // MFMAs of the current one are issued, and a scheduling barrier per step keeps the compiler
    // from hoisting the reads of all steps to the front (252 registers)
    float bcur[GPW], bnext[GPW];
#pragma unroll
    for (int i = 0; i < GPW; ++i) bcur[i] = xs[base[i] - RS - 1];
    float acur = wa[lane], anext = 0.f;
#pragma unroll
    for (int st = 0; st < 36; ++st) {
      if (st + 1 < 36) {
        const int t2 = (st + 1) / 4, cs2 = (st + 1) % 4;
        const int off2 = 4 * cs2 * PS + (t2 / 3 - 1) * RS + (t2 % 3 - 1);
        anext = wa[t2 * 256 + cs2 * 64 + lane];
#pragma unroll
        for (int i = 0; i < GPW; ++i) bnext[i] = xs[base[i] + off2];
      }
#pragma unroll
      for (int i = 0; i < GPW; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(acur, bcur[i], acc[i], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < GPW; ++i) bcur[i] = bnext[i];
      acur = anext;
      __builtin_amdgcn_sched_barrier(0);
    }

    // vector part: the outputs beyond the 16th; the weights are LDS broadcast reads
    if (REST > 0) {
#pragma unroll 4
      for (int c = 0; c < kCvChunk; ++c) {
        float wv[9][REST > 0 ? REST : 1];
#pragma unroll
        for (int t = 0; t < 9; ++t)
#pragma unroll
          for (int o = 0; o < REST; ++o) wv[t][o] = wl[(c * 9 + t) * REST + o];
#pragma unroll
        for (int t = 0; t < 9; ++t) {
          const int shift = (t / 3 - 1) * RS + (t % 3 - 1);
#pragma unroll
          for (int j = 0; j < kPixPerThread; ++j) {
            const float xv = xs[c * PS + rbase[j] + shift];
#pragma unroll
            for (int o = 0; o < REST; ++o) racc[j][o] = fmaf(wv[t][o], xv, racc[j][o]);
          }
        }
      }
    }
  }

#undef DK_LOAD_CHUNK
  // results: lane holds outputs 4 * (lane / 16) + j of pixel lane % 16 of each of its groups.  One split: the
  // result with its bias, in the tensor's type; several: fp32 partial sums (the bias with split 0), added afterwards.
  float* pn = partial + ((size_t)split * g.batch + n) * g.cout * plane;
  T* on = out + (size_t)n * g.cout * plane;
  const bool add_bias = split == 0;
  auto put = [&](int o, int at, float v) {
    v += add_bias ? ld(bias + o) : 0.f;
    if (ksplit > 1)
      pn[(size_t)o * plane + at] = v;
    else
      st(on + (size_t)o * plane + at, v);
  };
#pragma unroll
  for (int i = 0; i < GPW; ++i) {
    const int q = (wave + 4 * i) * 16 + (lane & 15);
    const int row = r0 + q / W;
    if (q < tile_pix && row < g.h) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int o = 4 * (lane >> 4) + j;
        if (o < g.cout) put(o, row * W + q % W, acc[i][j]);
      }
    }
  }
  if (REST > 0) {
#pragma unroll
    for (int j = 0; j < kPixPerThread; ++j) {
      const int q = (int)threadIdx.x + kCvBlock * j;
      const int row = r0 + q / W;
      if (q < tile_pix && row < g.h) {
#pragma unroll
        for (int o = 0; o < REST; ++o) put(16 + o, row * W + q % W, racc[j][o]);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Weight gradient: gW[o][c][t] = sum over images n and pixels p of gout[n][o][p] * x[n][c][p + shift_t].
// With q = p + shift_t this is a sum over the positions q of the zero-padded input tile,
//   gW[o][c][t] = sum_q G[o][q - shift_t] * X[c][q],
// G being the output-gradient tile, zero outside the tile: a matrix product whose rows are the
// cout * 9 pairs (o, t), whose columns are the channels and whose inner dimension is the padded
// position -- the (o, t) rows of a tile of 16 read G at 16 different (plane, shift) offsets, the
// 16 channels read X unshifted, and neither operand needs a per-tap pass.  18 outputs are 162
// rows = 11 MFMA tiles, 92 % of them useful, with no special case for the outputs beyond 16.
// A workgroup of 8 waves owns one chunk of 16 input channels and walks its share of the
// (image, row tile) items: both tiles staged in LDS (X channel pitch and row count chosen
// 4 mod 64 words, so 16 channels x 4 positions hit 64 banks), the waves split the positions in
// steps of 4, each accumulating the 11 tiles in registers over all items; at the end the waves'
// sums are added in a fixed order and one partial per workgroup goes to the workspace.
// ---------------------------------------------------------------------------
constexpr int kWgBlock = 512;
constexpr int kWgWaves = kWgBlock / 64;

template <int W>
struct WgradTile {
  static constexpr int TH = ConvTile<W>::TH, RS = W + 2, ROWS = TH + 2;
  static constexpr int PSX = (ROWS * RS + 59) / 64 * 64 + 4;  // positions per channel, 4 mod 64
  static constexpr int KSTEPS = PSX / 4;
  static constexpr int MARGIN = RS + 1;                         // the largest |shift|
  static constexpr int GP = (PSX + 2 * MARGIN + 31) / 64 * 64 + 32;  // floats per output plane of G, 32 mod 64
  static constexpr int SEGS = ConvTile<W>::SEGS;
  static_assert(PSX >= ROWS * RS && PSX % 64 == 4 && GP >= PSX + 2 * MARGIN, "tile layout");
};

template <typename T, int W, int NT>
__global__ __launch_bounds__(kWgBlock, 1) void offset_conv_wgrad_kernel(
    ConvGeo g, const T* __restrict__ x, const T* __restrict__ gout, float* __restrict__ partial, int parts) {
  using Tl = WgradTile<W>;
  constexpr int TH = Tl::TH, RS = Tl::RS, PSX = Tl::PSX, GP = Tl::GP, SEGS = Tl::SEGS;
  extern __shared__ __align__(16) float lds[];
  float* xs = lds;                      // [kCvChunk][PSX]
  float* gs = lds + kCvChunk * PSX;     // [cout][GP], position q at gs[o * GP + MARGIN + q]

  const int nchunks = g.cin / kCvChunk;
  const int chunk = blockIdx.x % nchunks, part = blockIdx.x / nchunks;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int m = lane & 15, k = lane >> 4;
  const int plane = g.h * W, items = g.batch * g.tiles;

  for (int e = threadIdx.x; e < kCvChunk * PSX + g.cout * GP; e += kWgBlock) lds[e] = 0.f;  // padding and margins

  // A operand of row tile j: row v = 16 j + m = (o, t); G[o][q - shift_t] at q = 4 ks + k
  int offa[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int v = 16 * j + m;
    const int o = v / 9, t = v % 9;
    const int shift = (t / 3 - 1) * RS + (t % 3 - 1);
    offa[j] = v < g.cout * 9 ? o * GP + Tl::MARGIN - shift + k : k;  // rows past cout * 9: any valid address
  }
  const bool last_rows_real = 16 * (NT - 1) + m < g.cout * 9;  // the last row tile may be partial
  const int offb = m * PSX + k;  // B operand: X[c = m][q]
  const float* xs_w = xs + 4 * wave;  // the wave's first step
  const float* gs_w = gs + 4 * wave;

  v4f acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) acc[j] = v4f{0.f, 0.f, 0.f, 0.f};

  // staging, as in the forward kernel: wave w takes channels w and w + 8 of the chunk (TH + 2 rows
  // each) and output planes w, w + 8, w + 16 (TH rows each)
  constexpr int kXStage = (kCvChunk / kWgWaves) * (TH + 2) * SEGS;
  constexpr int kGPlanes = 3;  // ceil(20 / 8)
  constexpr int kGStage = kGPlanes * TH * SEGS;
  unsigned vcol[SEGS];
#pragma unroll
  for (int sg = 0; sg < SEGS; ++sg) vcol[sg] = sg * 64 + lane < W ? (unsigned)((sg * 64 + lane) * sizeof(T)) : kOutOfRange;
  float xst[kXStage], gst[kGStage];
#define DK_LOAD_ITEM(ITEM)                                                                                     \
  {                                                                                                            \
    const int n_ = (ITEM) / g.tiles, r0_ = (ITEM) % g.tiles * TH;                                              \
    const rsrc_t rx = plane_rsrc(x + ((size_t)n_ * g.cin + (size_t)chunk * kCvChunk) * plane, kCvChunk * plane); \
    const rsrc_t rg = plane_rsrc(gout + (size_t)n_ * g.cout * plane, g.cout * plane);                          \
    _Pragma("unroll") for (int i = 0; i < kXStage; ++i) {                                                      \
      const int chq = i / ((TH + 2) * SEGS), ry = i / SEGS % (TH + 2), sg = i % SEGS;                          \
      const int row = r0_ - 1 + ry;                                                                            \
      const bool ok = row >= 0 && row < g.h;                                                                   \
      const int soff = ok ? ((wave + kWgWaves * chq) * g.h + row) * W * (int)sizeof(T) : 0;                    \
      xst[i] = buf_ld2(rx, ok ? vcol[sg] : kOutOfRange, soff, x);                                              \
    }                                                                                                          \
    _Pragma("unroll") for (int i = 0; i < kGStage; ++i) {                                                      \
      const int pq = i / (TH * SEGS), ry = i / SEGS % TH, sg = i % SEGS;                                       \
      const int o = wave + kWgWaves * pq, row = r0_ + ry;                                                      \
      const bool ok = o < g.cout && row < g.h;                                                                 \
      const int soff = ok ? (o * g.h + row) * W * (int)sizeof(T) : 0;                                          \
      gst[i] = buf_ld2(rg, ok ? vcol[sg] : kOutOfRange, soff, gout);                                           \
    }                                                                                                          \
  }

  int item = part;
  if (item < items) DK_LOAD_ITEM(item)
  for (; item < items; item += parts) {
    __syncthreads();  // the previous item's products are done (and, the first time, the zero fill)
#pragma unroll
    for (int i = 0; i < kXStage; ++i) {
      const int chq = i / ((TH + 2) * SEGS), ry = i / SEGS % (TH + 2), sg = i % SEGS;
      if (sg * 64 + lane < W) xs[(wave + kWgWaves * chq) * PSX + ry * RS + 1 + sg * 64 + lane] = xst[i];
    }
#pragma unroll
    for (int i = 0; i < kGStage; ++i) {
      const int pq = i / (TH * SEGS), ry = i / SEGS % TH, sg = i % SEGS;
      const int o = wave + kWgWaves * pq;
      // tile row ry is row ry + 1 of the padded geometry
      if (o < g.cout && sg * 64 + lane < W) gs[o * GP + Tl::MARGIN + (ry + 1) * RS + 1 + sg * 64 + lane] = gst[i];
    }
    __syncthreads();
    if (item + parts < items) DK_LOAD_ITEM(item + parts)

    // wave w takes the steps w, w + 8, ...: the wave part of the LDS address sits in the base
    // registers, the rest is an immediate of the unrolled loop
    constexpr int kTrips = (Tl::KSTEPS + kWgWaves - 1) / kWgWaves;
#pragma unroll 3
    for (int i = 0; i < kTrips; ++i) {
      if (wave + kWgWaves * i < Tl::KSTEPS) {  // wave-uniform; false only in the last trip
        const float b = xs_w[offb + 4 * kWgWaves * i];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          float a = gs_w[offa[j] + 4 * kWgWaves * i];
          if (j == NT - 1 && !last_rows_real) a = 0.f;
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[j], 0, 0, 0);
        }
      }
    }
  }
#undef DK_LOAD_ITEM

  // add the waves' sums in wave order into red[NT][256] (entry 4 * lane + r of a tile), then out
  __syncthreads();
  float* red = lds;
  for (int w = 0; w < kWgWaves; ++w) {
    if (wave == w) {
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        v4f* dst = reinterpret_cast<v4f*>(red + j * 256 + lane * 4);
        *dst = w == 0 ? acc[j] : *dst + acc[j];
      }
    }
    __syncthreads();
  }
  // D[row 4 * (l / 16) + r][channel l % 16] sits at red[j * 256 + 4 * l + r]
  float* dst = partial + (size_t)(part * nchunks + chunk) * (NT * 256);
  for (int e = threadIdx.x; e < NT * 256; e += kWgBlock) dst[e] = red[e];
}

// gW[o][c][t] = sum over parts of partial[part][chunk(c)][row tile][...], parts added in order
template <typename T>
__global__ __launch_bounds__(256) void offset_conv_wgrad_reduce_kernel(const float* __restrict__ partial, int parts,
                                                                       int nchunks, int nt, int cout, int cin,
                                                                       T* __restrict__ gw) {
  const int idx = blockIdx.x * 256 + threadIdx.x;  // = (o * cin + c) * 9 + t
  if (idx >= cout * cin * 9) return;
  const int t = idx % 9, c = idx / 9 % cin, o = idx / 9 / cin;
  const int v = o * 9 + t, j = v / 16, mrow = v % 16;
  // row mrow = 4 * (l / 16) + r, column c % 16 = l % 16
  const int l = (mrow / 4) * 16 + c % 16, r = mrow % 4;
  const float* p = partial + (size_t)(c / kCvChunk) * (nt * 256) + j * 256 + 4 * l + r;
  float s = 0.f;
  for (int q = 0; q < parts; ++q) s += p[(size_t)q * nchunks * (nt * 256)];
  st(gw + idx, s);
}

size_t round256(size_t n) { return (n + 255) / 256 * 256; }

// Bias gradient: partial[n][o] = sum over the pixels of gout[n][o]; one workgroup per plane.
template <typename T>
__global__ __launch_bounds__(kCvBlock) void conv_bias_grad_kernel(const T* __restrict__ gout, int plane,
                                                                  float* __restrict__ partial) {
  __shared__ float wave_sums[kCvBlock / 64];
  const T* p = gout + (size_t)blockIdx.x * plane;
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  for (int i = threadIdx.x; i < plane; i += 4 * kCvBlock) {
#pragma unroll
    for (int u = 0; u < 4; ++u) s[u] += i + u * kCvBlock < plane ? ld(p + i + u * kCvBlock) : 0.f;
  }
  const float t = wave_sum((s[0] + s[1]) + (s[2] + s[3]));
  if ((threadIdx.x & 63) == 0) wave_sums[threadIdx.x >> 6] = t;
  __syncthreads();
  if (threadIdx.x == 0) partial[blockIdx.x] = (wave_sums[0] + wave_sums[1]) + (wave_sums[2] + wave_sums[3]);
}

}  // namespace

// gbias[o] = sum over images and pixels of gout[n][o][.]; workspace: batch * cout floats
size_t offset_conv_bias_grad_workspace(int batch, int cout) { return (size_t)batch * cout * sizeof(float); }

template <typename T>
void offset_conv_bias_grad(int batch, int cout, int plane, const T* gout, T* gbias, void* ws, hipStream_t stream) {
  float* partial = static_cast<float*>(ws);
  if (batch > 0) conv_bias_grad_kernel<T><<<batch * cout, kCvBlock, 0, stream>>>(gout, plane, partial);
  launch_reduce_partials<float, T>(partial, batch, cout, gbias, stream);  // the images, added in order
}

bool offset_conv_supported(int cin, int cout, int h, int w) {
  const bool outputs_ok = (cout >= 1 && cout <= 16) || cout == 18 || cout == 20;  // the instantiated VALU widths
  return cin >= kCvChunk && cin % kCvChunk == 0 && outputs_ok && (w == 7 || w == 14 || w == 28 || w == 56 || w == 112) && h >= 1 &&
         (long)cin * h * w < (1L << 31) / 4 && (long)cout * h * w < (1L << 31) / 4;  // 32-bit byte offsets per image
}

// Input-channel splits of the forward: enough for about two workgroups per CU, at least two
// chunks of 16 channels per split
int forward_splits(int batch, int cin, int h, int w) {
  const int th = w <= 56 ? 8 : 4;
  const long base = std::max(1L, (long)batch * ceil_div(h, th));  // batch may be 0
  if (base >= 384) return 1;
  return (int)std::max<long>(1, std::min<long>((512 + base - 1) / base, cin / kCvChunk / 2));
}

// Whether the kernels are also the faster choice (measured against the library convolution on
// MI355X, forward + backward): float32, batch 64: on planes 28 wide and wider (56 and 112: by 30-40 %)
// once the grid -- (image, row tile) items times the input-channel splits -- gives about a
// workgroup per CU; on the 14- and 7-wide planes the two are within 10 % of each other either way.
// (16-bit tensors have forward and input gradient on 16-bit matrix instructions, dk_offset_conv16.hip, and a
// rule of their own in dk_offset_conv_worthwhile(); these kernels serve them where those do not apply.)
bool offset_conv_worthwhile(int batch, int cin, int cout, int h, int w) {
  if (!offset_conv_supported(cin, cout, h, w) || w < 28) return false;
  const int th = w <= 56 ? 8 : 4;
  return (long)batch * ceil_div(h, th) * forward_splits(batch, cin, h, w) >= 192;
}

// packed weights: w16 [9][cin][16] and wrest [9][cin][cout - 16]; then the splits' partial outputs
size_t offset_conv_workspace(int batch, int cin, int cout, int h, int w) {
  const int ks = forward_splits(batch, cin, h, w);
  return round256((size_t)9 * cin * 16 * sizeof(float)) + round256((size_t)9 * cin * std::max(0, cout - 16) * sizeof(float)) +
         (ks > 1 ? (size_t)ks * batch * cout * h * w * sizeof(float) : 0);
}

template <typename T>
bool offset_conv_forward(int batch, int cin, int cout, int h, int w, const T* x, const T* weight, const T* bias, T* out,
                         void* ws, hipStream_t stream) {
  if (!offset_conv_supported(cin, cout, h, w)) return false;
  if (batch == 0) return true;
  const int rest = std::max(0, cout - 16);
  float* w16 = static_cast<float*>(ws);
  char* after16 = static_cast<char*>(ws) + round256((size_t)9 * cin * 16 * sizeof(float));
  float* wrest = reinterpret_cast<float*>(after16);
  float* partial = reinterpret_cast<float*>(after16 + round256((size_t)9 * cin * rest * sizeof(float)));
  const int ksplit = forward_splits(batch, cin, h, w);
  conv_pack_weights_kernel<T><<<ceil_div(9 * cin * 16, 256), 256, 0, stream>>>(weight, cout, cin, rest, w16, wrest);
  ConvGeo g;
  g.batch = batch, g.cin = cin, g.cout = cout, g.h = h;
#define DK_LAUNCH(WW, REST)                                                                             \
  {                                                                                                     \
    g.tiles = ceil_div(h, ConvTile<WW>::TH);                                                            \
    const size_t lds = (size_t)(kCvChunk * (ConvTile<WW>::PS + 9 * REST) + 9 * 256) * sizeof(float);    \
    const unsigned grid = (unsigned)xcd_grid_size((long)batch * g.tiles * ksplit);                      \
    offset_conv_forward_kernel<T, WW, REST><<<grid, kCvBlock, lds, stream>>>(g, x, w16, wrest, bias, out, \
                                                                            partial, ksplit);            \
  }
#define DK_WIDTH(REST)                       \
  switch (w) {                               \
    case 7: DK_LAUNCH(7, REST) break;        \
    case 14: DK_LAUNCH(14, REST) break;      \
    case 28: DK_LAUNCH(28, REST) break;      \
    case 56: DK_LAUNCH(56, REST) break;      \
    case 112: DK_LAUNCH(112, REST) break;    \
    default: return false;                   \
  }
  switch (rest) {
    case 0: DK_WIDTH(0) break;
    case 2: DK_WIDTH(2) break;
    case 4: DK_WIDTH(4) break;
    default: return false;
  }
#undef DK_WIDTH
#undef DK_LAUNCH
  if (ksplit > 1) launch_reduce_partials<float, T>(partial, ksplit, (long)batch * cout * h * w, out, stream);
  return true;
}

// parts of the (image, row tile) items a chunk's workgroups split: about one workgroup per CU
int wgrad_parts(int batch, int cin, int h, int w) {
  const int th = w <= 56 ? 8 : 4;
  const int items = batch * ceil_div(h, th), nchunks = cin / kCvChunk;
  return std::max(1, std::min(items, 256 / nchunks));
}

// The weight gradient's 16-row blocks of (output, tap) pairs are instantiated for 9, 11 and 12 blocks:
// 15 or 16, 18 and 20 outputs.  0 bytes: not covered.
size_t offset_conv_wgrad_workspace(int batch, int cin, int cout, int h, int w) {
  const int nt = ceil_div(cout * 9, 16);
  if (nt != 9 && nt != 11 && nt != 12) return 0;
  return (size_t)wgrad_parts(batch, cin, h, w) * (cin / kCvChunk) * nt * 256 * sizeof(float);
}

template <typename T>
bool offset_conv_wgrad(int batch, int cin, int cout, int h, int w, const T* x, const T* gout, T* gweight, void* ws,
                       hipStream_t stream) {
  if (!offset_conv_supported(cin, cout, h, w)) return false;
  const int nt = ceil_div(cout * 9, 16), nchunks = cin / kCvChunk;
  const int parts = wgrad_parts(batch, cin, h, w);
  float* partial = static_cast<float*>(ws);
  ConvGeo g;
  g.batch = batch, g.cin = cin, g.cout = cout, g.h = h;
  bool ok = true;
#define DK_LAUNCH(WW, NT)                                                                                      \
  {                                                                                                            \
    auto kernel = offset_conv_wgrad_kernel<T, WW, NT>;                                                            \
    g.tiles = ceil_div(h, WgradTile<WW>::TH);                                                                  \
    const size_t lds = (size_t)(kCvChunk * WgradTile<WW>::PSX + cout * WgradTile<WW>::GP) * sizeof(float);     \
    const size_t lds_red = (size_t)NT * 256 * sizeof(float);                                                   \
    const size_t bytes = std::max(lds, lds_red);                                                               \
    if (bytes > (size_t)kMaxDynamicLds ||                                                                                  \
        !allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel)))                                                         \
      ok = false;                                                                                              \
    else if (batch > 0)                                                                                        \
      kernel<<<parts * nchunks, kWgBlock, bytes, stream>>>(g, x, gout, partial, parts);                        \
  }
#define DK_WIDTH(NT)                       \
  switch (w) {                             \
    case 7: DK_LAUNCH(7, NT) break;        \
    case 14: DK_LAUNCH(14, NT) break;      \
    case 28: DK_LAUNCH(28, NT) break;      \
    case 56: DK_LAUNCH(56, NT) break;      \
    case 112: DK_LAUNCH(112, NT) break;    \
    default: ok = false;                   \
  }
  switch (nt) {
    case 9: DK_WIDTH(9) break;    // 16 outputs
    case 11: DK_WIDTH(11) break;  // 18 outputs
    case 12: DK_WIDTH(12) break;  // 20 outputs
    default: ok = false;
  }
#undef DK_WIDTH
#undef DK_LAUNCH
  if (!ok) return false;
  const int total = cout * cin * 9;
  offset_conv_wgrad_reduce_kernel<T><<<ceil_div(total, 256), 256, 0, stream>>>(partial, batch > 0 ? parts : 0, nchunks,
                                                                              nt, cout, cin, gweight);
  return true;
}

#define DK_INSTANTIATE(T)                                                                                          \
  template void offset_conv_bias_grad<T>(int, int, int, const T*, T*, void*, hipStream_t);                         \
  template bool offset_conv_forward<T>(int, int, int, int, int, const T*, const T*, const T*, T*, void*, hipStream_t); \
  template bool offset_conv_wgrad<T>(int, int, int, int, int, const T*, const T*, T*, void*, hipStream_t);
DK_INSTANTIATE(float)
DK_INSTANTIATE(__half)
DK_INSTANTIATE(bf16_t)
#undef DK_INSTANTIATE

}  // namespace dk
