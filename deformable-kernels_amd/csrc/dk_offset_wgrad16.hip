// Weight gradient of the offset branch's 3x3 convolution (reference modules/deform_kernel.py:165-168; what
// autograd derives for the call at :214) on the 16-bit matrix instructions, padding 1, stride 1 or 2:
//   gW[o][c][t] = sum over images n and output pixels p of gout[n][o][p] * x[n][c][s p + shift_t].
// The sum runs over pixels, so both operands of v_mfma_f32_16x16x32_{bf16,f16} want eight consecutive pixels of
// one plane per lane: per tap t the product D_t[o][c] += G[o][q .. q + 31] * X_t[q .. q + 31][c] takes the output
// gradient tile G as the A operand (rows = output channels, two blocks of 16 for the branch's 18) and the input
// tile, read at the tap's shift, as the B operand (columns = the 16 channels of a chunk).  Both tiles sit in LDS
// plane by plane with a row pitch that is a multiple of 8 elements and at least one zero element between rows:
// G's window is one aligned 16-byte read; X's window at a row shift (dy) is aligned too, and the three column
// shifts (dx) come from that read plus the 32-bit words before and after it through v_alignbit -- 11 LDS reads and
// 24 vector instructions per 18 matrix instructions and 32 positions.  At stride 2 the input tile is staged as
// four planes by the parity of (row, column), X_{py,px}[j][i] = x[2 j + py][2 i + px], in which every tap is again a
// fixed shift of the output position.  float32 tensors: every element as a bfloat16 (hi, lo) pair in planes of
// their own, the four products hi*hi + hi*lo + lo*hi + lo*lo added (as in dk_offset_conv16.hip: about 3e-6 of the
// result's scale).
// A workgroup of four waves owns a chunk of 16 input channels and walks its share of the (image, row tile)
// items; the waves split a tile's steps of 32 positions and keep the 18 accumulator blocks in registers over all
// items; the next item's loads are in flight behind the products.  At the end the waves' sums are added in wave
// order, one partial per workgroup goes to the workspace, and a second kernel adds the partials in order:
// reproducible run to run, no atomics.
#include <algorithm>
#include <type_traits>

#include "dk_kernels.h"

namespace dk {

namespace {

constexpr int kW16Block = 256;
constexpr int kW16Waves = kW16Block / 64;
constexpr int kW16Chunk = 16;   // input channels per workgroup
constexpr int kW16Blocks = 2;   // blocks of 16 output channels
constexpr int kW16Tiles = 9 * kW16Blocks;

typedef float w16f4 __attribute__((ext_vector_type(4)));
typedef __bf16 w16b8 __attribute__((ext_vector_type(8)));
typedef _Float16 w16h8 __attribute__((ext_vector_type(8)));

template <typename T>
constexpr int kW16Parts = sizeof(T) == 4 ? 2 : 1;  // planes per tensor: the elements, or hi and lo parts

template <typename T>
__device__ __forceinline__ w16f4 w16_mma(const uint4& a, const uint4& b, w16f4 acc) {
  if constexpr (std::is_same<T, __half>::value)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(w16h8, a), __builtin_bit_cast(w16h8, b), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(w16b8, a), __builtin_bit_cast(w16b8, b), acc, 0, 0, 0);
}

// Geometry of the staged tiles, in elements of 2 bytes.  W: width of the output plane (= of the input plane at
// stride 1); TH: output rows per tile; S: stride.
//   G plane o:  position q = ry * RS + col, ry < TH, at gs[o * GP + q]; GP covers the steps (zeros beyond the tile)
//   X planes:   stride 1: one plane per channel, tile row ry (input row r0 - 1 + ry) at xs[... + XOFF + ry * RS + col];
//               tap (dy, dx) of position q reads XOFF + q + dy * RS + dx - 1.
//               stride 2: four planes per channel, plane (py, px) row j (input row 2 (r0 - 1 + j) + py) column i
//               (input column 2 i + px) at XOFF + j * RS + i; tap (dy, dx) of q reads plane ((dy + 1) & 1, (dx + 1) & 1)
//               at XOFF + q + (dy == 0 ? 0 : RS) + (dx == 0 ? -1 : 0).
// Plane pitches are 8 mod 128 elements: the 16 lanes of a read (16 planes, one 16-byte window each) hit all banks.
template <int W, int TH, int S>
struct W16Tile {
  static constexpr int RS = (W + 1 + 7) / 8 * 8;
  static constexpr int KSTEPS = (TH * RS + 31) / 32;
  static constexpr int XOFF = 8;
  static constexpr int XROWS = S == 1 ? TH + 2 : TH + 1;
  static constexpr int XNEED = XOFF + std::max(XROWS * RS, KSTEPS * 32 + (S == 1 ? 2 : 1) * RS) + 8;
  static constexpr int XP = (XNEED - 8 + 127) / 128 * 128 + 8;
  static constexpr int GP = (KSTEPS * 32 - 8 + 127) / 128 * 128 + 8;
  static constexpr int XPLANES = S == 1 ? 1 : 4;
};

// The 16 bits to stage for a loaded element; float32: part 0 = hi, 1 = lo of the pair
template <typename T>
__device__ __forceinline__ unsigned short w16_part(unsigned raw, int part) {
  if constexpr (sizeof(T) == 4) {
    const float v = __uint_as_float(raw);
    const unsigned hi = pack_bf16(v, 0.f) & 0xffffu;
    return (unsigned short)(part == 0 ? hi : pack_bf16(v - bf16_lo(hi), 0.f) & 0xffffu);
  } else {
    return (unsigned short)raw;
  }
}

template <typename T>
__device__ __forceinline__ unsigned w16_load(rsrc_t r, unsigned lane_off, int scalar_off) {
  if constexpr (sizeof(T) == 4)
    return __builtin_amdgcn_raw_buffer_load_b32(r, (int)lane_off, scalar_off, 0);
  else
    return __builtin_amdgcn_raw_buffer_load_b16(r, (int)lane_off, scalar_off, 0);
}

// x [batch][cin][h][S * W], gout [batch][cout][ho][W]; partial [parts][chunks][18][256]
template <typename T, int W, int TH, int S>
__global__ __launch_bounds__(kW16Block, 2) void offset_wgrad16_kernel(int batch, int cin, int cout, int h, int ho,
                                                                      int tiles, const T* __restrict__ x,
                                                                      const T* __restrict__ gout,
                                                                      float* __restrict__ partial, int parts) {
  using Tl = W16Tile<W, TH, S>;
  constexpr int RS = Tl::RS, KSTEPS = Tl::KSTEPS, XOFF = Tl::XOFF, XP = Tl::XP, GP = Tl::GP;
  constexpr int XPL = Tl::XPLANES, XROWS = Tl::XROWS, WIN = S * W;
  constexpr int P = kW16Parts<T>;
  extern __shared__ __align__(16) unsigned short lds16[];
  unsigned short* xs = lds16;                                // [part][channel][plane][XP]
  unsigned short* gs = lds16 + P * kW16Chunk * XPL * XP;     // [part][cout + 1][GP]; plane `cout` stays zero
  const int gplanes = cout + 1;

  const int nchunks = cin / kW16Chunk;
  const int chunk = blockIdx.x % nchunks, part = blockIdx.x / nchunks;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int m = lane & 15, kg = lane >> 4;
  const int plane_in = h * WIN, plane_out = ho * W, items = batch * tiles;

  {
    unsigned* z = reinterpret_cast<unsigned*>(lds16);
    const int words = (P * kW16Chunk * XPL * XP + P * gplanes * GP) / 2;
    for (int e = threadIdx.x; e < words; e += kW16Block) z[e] = 0u;  // margins, gaps between rows, the zero plane
  }

  // element offsets of the lane's operand windows at step 0
  int offa[kW16Blocks];
#pragma unroll
  for (int b = 0; b < kW16Blocks; ++b) offa[b] = min(16 * b + m, cout) * GP + 8 * kg;
  const int offb = m * XPL * XP + XOFF + 8 * kg;

  w16f4 acc[kW16Tiles];
#pragma unroll
  for (int j = 0; j < kW16Tiles; ++j) acc[j] = w16f4{0.f, 0.f, 0.f, 0.f};

  // staging: wave w takes channels w, w + 4, .. of the chunk and output planes w, w + 4, ..; the rows a tile needs
  // are one contiguous range of a plane, walked 64 elements at a time (out-of-image rows: offsets that fail the
  // range check and load zeros, which overwrite what the previous item left)
  constexpr int kInRows = S == 1 ? XROWS : 2 * XROWS;  // input rows per channel: r0 - 1 .. (stride 2: 2 (r0 - 1) ..)
  constexpr int kXLoads = (kInRows * WIN + 63) / 64, kGLoads = (TH * W + 63) / 64;
  constexpr int kXStage = (kW16Chunk / kW16Waves) * kXLoads;
  constexpr int kGPlanesPerWave = 5;  // output planes per wave: up to 20 outputs
  constexpr int kGStage = kGPlanesPerWave * kGLoads;
  unsigned xst[kXStage], gst[kGStage];
#define DK_LOAD_ITEM(ITEM)                                                                                          \
  {                                                                                                                 \
    const int n_ = (ITEM) / tiles, r0_ = (ITEM) % tiles * TH;                                                       \
    const rsrc_t rx = plane_rsrc(x + ((size_t)n_ * cin + (size_t)chunk * kW16Chunk) * plane_in, kW16Chunk * plane_in); \
    const rsrc_t rg = plane_rsrc(gout + (size_t)n_ * cout * plane_out, cout * plane_out);                           \
    const int xrow0 = S == 1 ? r0_ - 1 : 2 * (r0_ - 1);                                                             \
    _Pragma("unroll") for (int i = 0; i < kXStage; ++i) {                                                           \
      const int chq = i / kXLoads, e = i % kXLoads * 64 + lane;                                                     \
      const int row = xrow0 + e / WIN;                                                                              \
      const bool ok = e < kInRows * WIN && row >= 0 && row < h;                                                     \
      xst[i] = w16_load<T>(rx, ok ? (unsigned)((xrow0 * WIN + e) * (int)sizeof(T)) : kOutOfRange,                   \
                           (wave + kW16Waves * chq) * plane_in * (int)sizeof(T));                                   \
    }                                                                                                               \
    _Pragma("unroll") for (int i = 0; i < kGStage; ++i) {                                                           \
      const int o = wave + kW16Waves * (i / kGLoads), e = i % kGLoads * 64 + lane;                                  \
      const bool ok = o < cout && e < TH * W && r0_ + e / W < ho;                                                   \
      gst[i] = w16_load<T>(rg, ok ? (unsigned)((r0_ * W + e) * (int)sizeof(T)) : kOutOfRange,                       \
                           ok ? o * plane_out * (int)sizeof(T) : 0);                                                \
    }                                                                                                               \
  }

  int item = part;
  if (item < items) DK_LOAD_ITEM(item)
  for (; item < items; item += parts) {
    __syncthreads();  // the previous item's products are done (and, the first time, the zero fill)
#pragma unroll
    for (int i = 0; i < kXStage; ++i) {
      const int chq = i / kXLoads, e = i % kXLoads * 64 + lane;
      if (e < kInRows * WIN) {
        const int ry = e / WIN, col = e % WIN;
        // stride 1: plane 0, row ry; stride 2: plane (ry & 1, col & 1), row ry / 2, column col / 2
        const int pl = S == 1 ? 0 : (ry & 1) * 2 + (col & 1);
        const int at = S == 1 ? ry * RS + col : (ry >> 1) * RS + (col >> 1);
#pragma unroll
        for (int p = 0; p < P; ++p)
          xs[((p * kW16Chunk + wave + kW16Waves * chq) * XPL + pl) * XP + XOFF + at] = w16_part<T>(xst[i], p);
      }
    }
#pragma unroll
    for (int i = 0; i < kGStage; ++i) {
      const int o = wave + kW16Waves * (i / kGLoads), e = i % kGLoads * 64 + lane;
      if (o < cout && e < TH * W) {
#pragma unroll
        for (int p = 0; p < P; ++p) gs[(p * gplanes + o) * GP + e / W * RS + e % W] = w16_part<T>(gst[i], p);
      }
    }
    __syncthreads();
    if (item + parts < items) DK_LOAD_ITEM(item + parts)

    // wave w takes the steps w, w + 4, ..
    for (int ks = wave; ks < KSTEPS; ks += kW16Waves) {
      uint4 a[kW16Blocks][P];
#pragma unroll
      for (int b = 0; b < kW16Blocks; ++b)
#pragma unroll
        for (int p = 0; p < P; ++p)
          a[b][p] = *reinterpret_cast<const uint4*>(gs + p * gplanes * GP + offa[b] + 32 * ks);
#pragma unroll
      for (int dy = 0; dy < 3; ++dy) {
        uint4 bt[3][P];
        if constexpr (S == 1) {
#pragma unroll
          for (int p = 0; p < P; ++p) {
            const unsigned short* w0 = xs + p * kW16Chunk * XP + offb + 32 * ks + dy * RS;
            const uint4 d = *reinterpret_cast<const uint4*>(w0);
            const unsigned prev = *reinterpret_cast<const unsigned*>(w0 - 2);
            const unsigned next = *reinterpret_cast<const unsigned*>(w0 + 8);
            bt[0][p] = make_uint4(__builtin_amdgcn_alignbit(d.x, prev, 16), __builtin_amdgcn_alignbit(d.y, d.x, 16),
                                  __builtin_amdgcn_alignbit(d.z, d.y, 16), __builtin_amdgcn_alignbit(d.w, d.z, 16));
            bt[1][p] = d;
            bt[2][p] = make_uint4(__builtin_amdgcn_alignbit(d.y, d.x, 16), __builtin_amdgcn_alignbit(d.z, d.y, 16),
                                  __builtin_amdgcn_alignbit(d.w, d.z, 16), __builtin_amdgcn_alignbit(next, d.w, 16));
          }
        } else {
          // rows: dy = 0 -> plane row parity 1 at row j, dy = 1 -> parity 0 at j + 1, dy = 2 -> parity 1 at j + 1
          // (tile row j is input row pair r0 - 1 + j); columns: dx = 0 -> parity 1 at i - 1, dx = 1 -> parity 0
          // at i, dx = 2 -> parity 1 at i
          const int py = dy == 1 ? 0 : 1;
          const int rowoff = dy == 0 ? 0 : RS;
#pragma unroll
          for (int p = 0; p < P; ++p) {
            const unsigned short* odd = xs + (p * kW16Chunk * XPL + py * 2 + 1) * XP + offb + 32 * ks + rowoff;
            const unsigned short* even = xs + (p * kW16Chunk * XPL + py * 2 + 0) * XP + offb + 32 * ks + rowoff;
            const uint4 d = *reinterpret_cast<const uint4*>(odd);
            const unsigned prev = *reinterpret_cast<const unsigned*>(odd - 2);
            bt[0][p] = make_uint4(__builtin_amdgcn_alignbit(d.x, prev, 16), __builtin_amdgcn_alignbit(d.y, d.x, 16),
                                  __builtin_amdgcn_alignbit(d.z, d.y, 16), __builtin_amdgcn_alignbit(d.w, d.z, 16));
            bt[1][p] = *reinterpret_cast<const uint4*>(even);
            bt[2][p] = d;
          }
        }
#pragma unroll
        for (int dx = 0; dx < 3; ++dx)
#pragma unroll
          for (int b = 0; b < kW16Blocks; ++b)
#pragma unroll
            for (int pa = 0; pa < P; ++pa)
#pragma unroll
              for (int pb = 0; pb < P; ++pb)
                acc[(dy * 3 + dx) * kW16Blocks + b] = w16_mma<T>(a[b][pa], bt[dx][pb], acc[(dy * 3 + dx) * kW16Blocks + b]);
      }
    }
  }
#undef DK_LOAD_ITEM

  // add the waves' sums in wave order into red[18][256] (entry 4 * lane + r of a block), then out
  __syncthreads();
  float* red = reinterpret_cast<float*>(lds16);
  for (int w = 0; w < kW16Waves; ++w) {
    if (wave == w) {
#pragma unroll
      for (int j = 0; j < kW16Tiles; ++j) {
        w16f4* dst = reinterpret_cast<w16f4*>(red + j * 256 + lane * 4);
        *dst = w == 0 ? acc[j] : *dst + acc[j];
      }
    }
    __syncthreads();
  }
  float* dst = partial + (size_t)(part * nchunks + chunk) * (kW16Tiles * 256);
  for (int e = threadIdx.x; e < kW16Tiles * 256; e += kW16Block) dst[e] = red[e];
}

// gW[o][c][t] = sum over parts of partial[part][chunk(c)][t][block(o)][...], parts added in order.
// D[row 4 (l / 16) + r][column l % 16] of a block sits at entry 4 l + r: row = o % 16, column = c % 16.
template <typename T>
__global__ __launch_bounds__(256) void offset_wgrad16_reduce_kernel(const float* __restrict__ partial, int parts,
                                                                    int nchunks, int cout, int cin, T* __restrict__ gw) {
  const int idx = blockIdx.x * 256 + threadIdx.x;  // = (o * cin + c) * 9 + t
  if (idx >= cout * cin * 9) return;
  const int t = idx % 9, c = idx / 9 % cin, o = idx / 9 / cin;
  const int row = o % 16, l = (row / 4) * 16 + c % 16, r = row % 4;
  const float* p = partial + ((size_t)(c / kW16Chunk) * kW16Tiles + t * kW16Blocks + o / 16) * 256 + 4 * l + r;
  const size_t step = (size_t)nchunks * (kW16Tiles * 256);
  // eight loads in flight, added in part order
  float s = 0.f;
  int q = 0;
  for (; q + 8 <= parts; q += 8) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = p[(size_t)(q + j) * step];
#pragma unroll
    for (int j = 0; j < 8; ++j) s += v[j];
  }
  for (; q < parts; ++q) s += p[(size_t)q * step];
  st(gw + idx, s);
}

// output rows per tile by output width, stride and element size (float32 stages two planes per tensor)
constexpr int w16_rows(int wo, int stride, bool pairs) {
  if (stride == 1) return wo >= 112 ? (pairs ? 2 : 4) : wo >= 56 ? (pairs ? 4 : 8) : wo >= 28 ? (pairs ? 8 : 16) : wo >= 14 ? 14 : 7;
  return wo >= 56 ? 2 : wo >= 28 ? 4 : 7;  // (more rows: more staging registers than a lane has)
}

template <int W, int TH, int S>
size_t w16_lds_bytes(int parts_per_tensor, int cout) {
  using Tl = W16Tile<W, TH, S>;
  const size_t tiles = (size_t)parts_per_tensor * (kW16Chunk * Tl::XPLANES * Tl::XP + (cout + 1) * Tl::GP) * 2;
  return std::max(tiles, (size_t)kW16Tiles * 256 * sizeof(float));
}

// parts of the (image, row tile) items a chunk's workgroups split: about two workgroups per CU
int w16_parts(int batch, int cin, int ho, int wo, int stride, bool pairs) {
  const int items = batch * ceil_div(ho, w16_rows(wo, stride, pairs)), nchunks = cin / kW16Chunk;
  return std::max(1, std::min(items, 512 / nchunks));
}

}  // namespace

// stride 1: planes 7 .. 112 wide; stride 2: input planes 14 .. 112 wide (output planes 7 .. 56)
bool offset_wgrad16_supported(int cin, int cout, int h, int w, int stride) {
  if (cin < kW16Chunk || cin % kW16Chunk != 0 || cout < 1 || cout > 20 || h < 1) return false;  // (20: the output planes a wave stages)
  if ((long)cin * h * w >= (1L << 31) / 4 || (long)cout * h * w >= (1L << 31) / 4) return false;
  if (stride == 2) return w == 14 || w == 28 || w == 56 || w == 112;
  return w == 7 || w == 14 || w == 28 || w == 56 || w == 112;
}

size_t offset_wgrad16_workspace(int batch, int cin, int cout, int h, int w, int stride, bool pairs) {
  if (!offset_wgrad16_supported(cin, cout, h, w, stride)) return 0;
  const int ho = stride == 2 ? (h - 1) / 2 + 1 : h, wo = stride == 2 ? w / 2 : w;
  return (size_t)w16_parts(batch, cin, ho, wo, stride, pairs) * (cin / kW16Chunk) * kW16Tiles * 256 * sizeof(float);
}

template <typename T>
bool offset_wgrad16(int batch, int cin, int cout, int h, int w, int stride, const T* x, const T* gout, T* gweight,
                    void* ws, hipStream_t stream) {
  if (!offset_wgrad16_supported(cin, cout, h, w, stride)) return false;
  constexpr bool pairs = sizeof(T) == 4;
  const int ho = stride == 2 ? (h - 1) / 2 + 1 : h, wo = stride == 2 ? w / 2 : w;
  const int nchunks = cin / kW16Chunk;
  const int parts = w16_parts(batch, cin, ho, wo, stride, pairs);
  float* partial = static_cast<float*>(ws);
  bool ok = true;
#define DK_LAUNCH(WO, S)                                                                                          \
  {                                                                                                               \
    constexpr int TH = w16_rows(WO, S, pairs);                                                                      \
    auto kernel = offset_wgrad16_kernel<T, WO, TH, S>;                                                            \
    const int tiles = ceil_div(ho, TH);                                                                           \
    const size_t bytes = w16_lds_bytes<WO, TH, S>(kW16Parts<T>, cout);                                            \
    if (bytes > (size_t)kMaxDynamicLds || !allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel)))          \
      ok = false;                                                                                                 \
    else if (batch > 0)                                                                                           \
      kernel<<<parts * nchunks, kW16Block, bytes, stream>>>(batch, cin, cout, h, ho, tiles, x, gout, partial, parts); \
  }
  if (stride == 2) {
    switch (wo) {
      case 7: DK_LAUNCH(7, 2) break;
      case 14: DK_LAUNCH(14, 2) break;
      case 28: DK_LAUNCH(28, 2) break;
      case 56: DK_LAUNCH(56, 2) break;
      default: ok = false;
    }
  } else {
    switch (wo) {
      case 7: DK_LAUNCH(7, 1) break;
      case 14: DK_LAUNCH(14, 1) break;
      case 28: DK_LAUNCH(28, 1) break;
      case 56: DK_LAUNCH(56, 1) break;
      case 112: DK_LAUNCH(112, 1) break;
      default: ok = false;
    }
  }
#undef DK_LAUNCH
  if (!ok) return false;
  const int total = cout * cin * 9;
  offset_wgrad16_reduce_kernel<T><<<ceil_div(total, 256), 256, 0, stream>>>(partial, batch > 0 ? parts : 0, nchunks,
                                                                           cout, cin, gweight);
  return true;
}

#define DK_INST(T) \
  template bool offset_wgrad16<T>(int, int, int, int, int, int, const T*, const T*, T*, void*, hipStream_t);
DK_INST(__half)
DK_INST(bf16_t)
DK_INST(float)
#undef DK_INST

}  // namespace dk
