// The offset branch's 3x3 convolution (reference modules/deform_kernel.py:165-168, applied at :214)
// on 16-bit tensors: forward and input gradient on the 16-bit matrix instructions
// (v_mfma_f32_16x16x32_bf16 / _f16: the tensors' elements are the operands as they are, the products
// exact, the sums fp32, one rounding of the result).  Padding 1, no dilation; stride 1 on planes 7, 14, 28, 56
// or 112 wide, stride 2 (kernels of their own, further down) on input planes 14, 28, 56 or 112 wide.
//
// At stride 1 both passes are the same shift-GEMM, out[m][p] = sum over taps t, channels k of A_t[m][k] * in[k][p + shift_t]:
//   forward          in = x (Cin channels),   m = output channel,  A_t[m][k] = W[m][k][t], + bias;
//   input gradient   in = gout (Cout channels), m = input channel, A_t[m][k] = W[k][m][8 - t]  (the taps flipped).
// A workgroup of four waves owns 448 pixels (whole rows) of one image and walks the `in` channels in chunks
// of 32, staged zero-padded and channel-interleaved in LDS: position e holds the chunk's 32 elements in 64
// bytes of an 80-byte slot, so that the B operand of a lane -- pixel l % 16, channels 8 (l / 16) .. + 7 -- is
// one 16-byte read, and the 16 lanes of a pass (20 words apart) hit disjoint banks.  The A operands come
// packed per (tap, chunk, 16-row block) as the instruction wants them, one coalesced 16-byte load per lane.
// A wave holds seven pixel groups x MTB row blocks of accumulators; row blocks beyond MTB go to further
// workgroups that stage the same tile (the input gradient: 18 channels in, one chunk, three workgroups of
// three blocks for 144 channels out).
#include <algorithm>
#include <type_traits>

#include "dk_kernels.h"

namespace dk {

namespace {

constexpr int kC16Block = 256;
constexpr int kC16Chunk = 32;     // channels per matrix instruction
constexpr int kC16Pitch = 20;     // 32-bit words per staged position: 16 of data, 4 of bank skew
constexpr int kC16Pix = 448;      // pixels per workgroup: 28 groups of 16, seven per wave
constexpr int kC16Gpw = kC16Pix / 16 / (kC16Block / 64);

template <int W>
struct Tile16 {
  static constexpr int TH = kC16Pix / W;
  static constexpr int RS = W + 2;
  static constexpr int POS = (TH + 2) * RS;
  static_assert(TH * W == kC16Pix, "whole rows");
};

typedef float c16f4 __attribute__((ext_vector_type(4)));
typedef __bf16 c16b8 __attribute__((ext_vector_type(8)));
typedef _Float16 c16h8 __attribute__((ext_vector_type(8)));

// v rounded to T, as the 16 bits of the element
template <typename T>
__device__ __forceinline__ unsigned bits16(float v) {
  T t;
  st(&t, v);
  unsigned short b;
  __builtin_memcpy(&b, &t, sizeof(b));
  return b;
}

template <typename T>
__device__ __forceinline__ c16f4 mma16(const uint4& a, const uint4& b, c16f4 acc) {
  if constexpr (std::is_same<T, bf16_t>::value)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(c16b8, a), __builtin_bit_cast(c16b8, b), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(c16h8, a), __builtin_bit_cast(c16h8, b), acc, 0, 0, 0);
}

// wp[t][chunk][block][lane] = the eight elements A_t[16 block + lane % 16][32 chunk + 8 (lane / 16) .. + 7], zeros
// past the tensor.  weight is [O][C][3][3]; forward: rows = O, k = C; transposed: rows = C, k = O, taps flipped.
template <typename T>
__global__ void conv16_pack_kernel(const T* __restrict__ weight, int O, int C, int transposed, int chunks, int blocks,
                                   uint4* __restrict__ wp) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= 9 * chunks * blocks * 64) return;
  const int lane = idx % 64, mb = idx / 64 % blocks, ch = idx / 64 / blocks % chunks, t = idx / 64 / blocks / chunks;
  const int m = 16 * mb + (lane & 15), k0 = kC16Chunk * ch + 8 * (lane >> 4);
  const unsigned short* w = reinterpret_cast<const unsigned short*>(weight);
  unsigned v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int k = k0 + j;
    const int o = transposed ? k : m, c = transposed ? m : k;
    v[j] = (o < O && c < C) ? w[((size_t)o * C + c) * 9 + (transposed ? 8 - t : t)] : 0u;
  }
  wp[idx] = make_uint4(v[0] | v[1] << 16, v[2] | v[3] << 16, v[4] | v[5] << 16, v[6] | v[7] << 16);
}

// in [batch][kin][h][W] -> out [batch][mout][h][W]; wp as packed above with `chunks` = ceil(kin / 32) and
// `blocks` = ceil(mout / 16); bias [mout] or null.
// grid = (image, row tile, walk of MTB row blocks)
template <typename T, int W, int MTB>
__global__ __launch_bounds__(kC16Block, 2) void conv16_kernel(int batch, int kin, int mout, int h, int tiles, int chunks,
                                                              int blocks, const T* __restrict__ in,
                                                              const uint4* __restrict__ wp, const T* __restrict__ bias,
                                                              T* __restrict__ out, float* __restrict__ partial,
                                                              int ksplit) {
  using Tl = Tile16<W>;
  constexpr int TH = Tl::TH, RS = Tl::RS, POS = Tl::POS;
  extern __shared__ __align__(16) unsigned tile[];  // [POS][kC16Pitch]

  // logical block = (walk over MTB row blocks, row tile, image), walk fastest: the workgroups that share an
  // input tile run side by side
  // With ksplit > 1 (small planes with many channels, where (image, tile) gives too few workgroups) a workgroup
  // sums a share of the chunks and writes partial[split][...] in fp32; the splits are added afterwards, in order.
  const int walks = (blocks + MTB - 1) / MTB;
  const int total = batch * tiles * walks * ksplit;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int split = lb % ksplit, lw = lb / ksplit;
  const int mb0 = (lw % walks) * MTB, n = lw / walks / tiles, r0 = (lw / walks % tiles) * TH;
  const int per_split = (chunks + ksplit - 1) / ksplit;
  const int ch_lo = split * per_split, ch_hi = min(chunks, ch_lo + per_split);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int plane = h * W;

  // rows of the tile that lie in the image (a plane lower than the tile: 14 x 14 and 7 x 7 planes are one tile
  // of 32 / 64 rows), and the pixel groups that hold any of their pixels
  const int rows = min(TH, h - r0);
  const int live_groups = (rows * W + 15) / 16;
  for (int e = threadIdx.x; e < (rows + 2) * RS * kC16Pitch; e += kC16Block) tile[e] = 0u;  // the padding stays zero

  // word index of the lane's B operand for each of its pixel groups (tap shifts are immediates)
  int bword[kC16Gpw];
#pragma unroll
  for (int i = 0; i < kC16Gpw; ++i) {
    const int q = min((wave + 4 * i) * 16 + (lane & 15), rows * W - 1);  // (a pixel below the image: not stored)
    bword[i] = ((q / W + 1) * RS + q % W + 1) * kC16Pitch + (lane >> 4) * 4;
  }

  {
    c16f4 acc[kC16Gpw][MTB];
#pragma unroll
    for (int i = 0; i < kC16Gpw; ++i)
#pragma unroll
      for (int m = 0; m < MTB; ++m) acc[i][m] = c16f4{0.f, 0.f, 0.f, 0.f};

    for (int ch = ch_lo; ch < ch_hi; ++ch) {
      {
        __syncthreads();  // the previous chunk's reads are done
        // one buffer over the chunk's planes: channels past the tensor and rows outside the image fail
        // the range check and read zero
        const int kc = min(kC16Chunk, kin - ch * kC16Chunk);
        const rsrc_t rs = plane_rsrc(in + ((size_t)n * kin + (size_t)ch * kC16Chunk) * plane, kc * plane);
        for (int e = threadIdx.x; e < (rows + 2) * 4 * W; e += kC16Block) {
          const int col = e % W, ry = e / W % (rows + 2), oct = e / W / (rows + 2);
          const int row = r0 - 1 + ry;
          const bool live = row >= 0 && row < h;
          unsigned v[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const unsigned o = live ? (unsigned)((oct * 8 + j) * plane + row * W + col) * 2u : kOutOfRange;
            v[j] = __builtin_amdgcn_raw_buffer_load_b16(rs, (int)o, 0, 0);
          }
          *reinterpret_cast<uint4*>(tile + (ry * RS + col + 1) * kC16Pitch + oct * 4) =
              make_uint4(v[0] | v[1] << 16, v[2] | v[3] << 16, v[4] | v[5] << 16, v[6] | v[7] << 16);
        }
        __syncthreads();
      }
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        const int shift = ((t / 3 - 1) * RS + (t % 3 - 1)) * kC16Pitch;
        uint4 a[MTB];
#pragma unroll
        for (int m = 0; m < MTB; ++m) {
          const int mb = min(mb0 + m, blocks - 1);  // a block past the last repeats it; its results are not stored
          a[m] = wp[((size_t)(t * chunks + ch) * blocks + mb) * 64 + lane];
        }
#pragma unroll
        for (int i = 0; i < kC16Gpw; ++i) {
          // planes lower than the tile (uniform: the wave's remaining groups lie below the image)
          if constexpr (W <= 14)
            if (wave + 4 * i >= live_groups) break;
          const uint4 b = *reinterpret_cast<const uint4*>(tile + bword[i] + shift);
#pragma unroll
          for (int m = 0; m < MTB; ++m) acc[i][m] = mma16<T>(a[m], b, acc[i][m]);
        }
      }
    }

    // lane (pixel l % 16, rows 4 (l / 16) .. + 3 of each block)
#pragma unroll
    for (int m = 0; m < MTB; ++m) {
      if (mb0 + m >= blocks) break;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int o = 16 * (mb0 + m) + 4 * (lane >> 4) + r;
        if (o >= mout) continue;
        const float bv = bias && split == 0 ? ld(bias + o) : 0.f;
        const size_t at = ((size_t)n * mout + o) * plane + (size_t)r0 * W;
#pragma unroll
        for (int i = 0; i < kC16Gpw; ++i) {
          const int q = (wave + 4 * i) * 16 + (lane & 15);
          if (r0 * W + q < plane) {
            if (ksplit > 1)
              partial[(size_t)split * batch * mout * plane + at + q] = acc[i][m][r] + bv;
            else
              st(out + at + q, acc[i][m][r] + bv);
          }
        }
      }
    }
  }
}


// ---- stride 2, forward --------------------------------------------------------------------------------------
// out[m][(oy, ox)] = sum over taps, channels of A_t[m][k] * in[k][(2 oy + dy - 1, 2 ox + dx - 1)].  A tile of 448
// output pixels needs 2 TH + 1 input rows of the full width, so the chunk is 16 channels (v_mfma_f32_16x16x16):
// a position's 16 elements in 32 bytes of a 40-byte slot (17 rows of a 112-wide plane: 77 KB, two workgroups per
// CU); a lane's B operand -- output pixel l % 16, channels 4 (l / 16) .. + 3 -- is one 8-byte read at the input
// position (2 r, 2 c) + (dy, dx) of the zero-padded tile, and the 16 lanes of a pass, 20 words apart, hit
// disjoint banks.
constexpr int kS2Chunk = 16;
constexpr int kS2Pitch = 10;  // 32-bit words per staged position: 8 of data, 2 of bank skew

typedef __bf16 c16b4 __attribute__((ext_vector_type(4)));
typedef _Float16 c16h4 __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ c16f4 mma16k16(const uint2& a, const uint2& b, c16f4 acc) {
  if constexpr (std::is_same<T, bf16_t>::value)
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(c16b4, a), __builtin_bit_cast(c16b4, b), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(c16h4, a), __builtin_bit_cast(c16h4, b), acc, 0, 0, 0);
}

// wp[t][chunk][block][lane] = the four elements W[16 block + lane % 16][16 chunk + 4 (lane / 16) .. + 3][t]
template <typename T>
__global__ void conv16_s2_pack_kernel(const T* __restrict__ weight, int O, int C, int chunks, int blocks,
                                      uint2* __restrict__ wp) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= 9 * chunks * blocks * 64) return;
  const int lane = idx % 64, mb = idx / 64 % blocks, ch = idx / 64 / blocks % chunks, t = idx / 64 / blocks / chunks;
  const int o = 16 * mb + (lane & 15), c0 = kS2Chunk * ch + 4 * (lane >> 4);
  const unsigned short* w = reinterpret_cast<const unsigned short*>(weight);
  unsigned v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = (o < O && c0 + j < C) ? w[((size_t)o * C + c0 + j) * 9 + t] : 0u;
  wp[idx] = make_uint2(v[0] | v[1] << 16, v[2] | v[3] << 16);
}

// in [batch][kin][h][WIN] -> out [batch][mout][ho][WIN / 2], ho = (h - 1) / 2 + 1 (padding 1, 3 x 3 taps)
// grid = (image, tile of output rows, chunk split)
template <typename T, int WIN, int MTB>
__global__ __launch_bounds__(kC16Block, 2) void conv16_s2_kernel(int batch, int kin, int mout, int h, int ho, int tiles,
                                                                 int chunks, int blocks, const T* __restrict__ in,
                                                                 const uint2* __restrict__ wp,
                                                                 const T* __restrict__ bias, T* __restrict__ out,
                                                                 float* __restrict__ partial, int ksplit) {
  constexpr int W = WIN / 2, TH = kC16Pix / W, RS = WIN + 2;
  static_assert(WIN % 2 == 0 && TH * W == kC16Pix, "whole output rows");
  extern __shared__ __align__(16) unsigned tile[];  // [2 rows + 1][RS][kS2Pitch]

  const int total = batch * tiles * ksplit;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int split = lb % ksplit, n = lb / ksplit / tiles, r0 = (lb / ksplit % tiles) * TH;
  const int per_split = (chunks + ksplit - 1) / ksplit;
  const int ch_lo = split * per_split, ch_hi = min(chunks, ch_lo + per_split);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int plane_in = h * WIN, plane = ho * W;

  const int rows = min(TH, ho - r0);  // output rows of the tile inside the image
  const int rows_in = 2 * rows + 1;   // input rows 2 r0 - 1 .. 2 (r0 + rows - 1) + 1
  const int live_groups = (rows * W + 15) / 16;
  for (int e = threadIdx.x; e < rows_in * RS * kS2Pitch; e += kC16Block) tile[e] = 0u;  // the padding stays zero

  int bword[kC16Gpw];
#pragma unroll
  for (int i = 0; i < kC16Gpw; ++i) {
    const int q = min((wave + 4 * i) * 16 + (lane & 15), rows * W - 1);  // (a pixel below the image: not stored)
    bword[i] = (2 * (q / W) * RS + 2 * (q % W)) * kS2Pitch + (lane >> 4) * 2;
  }

  c16f4 acc[kC16Gpw][MTB];
#pragma unroll
  for (int i = 0; i < kC16Gpw; ++i)
#pragma unroll
    for (int m = 0; m < MTB; ++m) acc[i][m] = c16f4{0.f, 0.f, 0.f, 0.f};

  for (int ch = ch_lo; ch < ch_hi; ++ch) {
    __syncthreads();  // the previous chunk's reads are done
    const int kc = min(kS2Chunk, kin - ch * kS2Chunk);
    const rsrc_t rs = plane_rsrc(in + ((size_t)n * kin + (size_t)ch * kS2Chunk) * plane_in, kc * plane_in);
    for (int e = threadIdx.x; e < rows_in * 2 * WIN; e += kC16Block) {
      const int col = e % WIN, ry = e / WIN % rows_in, oct = e / WIN / rows_in;
      const int row = 2 * r0 - 1 + ry;
      const bool live = row >= 0 && row < h;
      unsigned v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const unsigned o = live ? (unsigned)((oct * 8 + j) * plane_in + row * WIN + col) * 2u : kOutOfRange;
        v[j] = __builtin_amdgcn_raw_buffer_load_b16(rs, (int)o, 0, 0);
      }
      uint2* dst = reinterpret_cast<uint2*>(tile + (ry * RS + col + 1) * kS2Pitch + oct * 4);
      dst[0] = make_uint2(v[0] | v[1] << 16, v[2] | v[3] << 16);
      dst[1] = make_uint2(v[4] | v[5] << 16, v[6] | v[7] << 16);
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 9; ++t) {
      const int shift = ((t / 3) * RS + t % 3) * kS2Pitch;
      uint2 a[MTB];
#pragma unroll
      for (int m = 0; m < MTB; ++m) a[m] = wp[((size_t)(t * chunks + ch) * blocks + min(m, blocks - 1)) * 64 + lane];
#pragma unroll
      for (int i = 0; i < kC16Gpw; ++i) {
        if constexpr (W <= 14)
          if (wave + 4 * i >= live_groups) break;
        const uint2 b = *reinterpret_cast<const uint2*>(tile + bword[i] + shift);
#pragma unroll
        for (int m = 0; m < MTB; ++m) acc[i][m] = mma16k16<T>(a[m], b, acc[i][m]);
      }
    }
  }

#pragma unroll
  for (int m = 0; m < MTB; ++m) {
    if (m >= blocks) break;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int o = 16 * m + 4 * (lane >> 4) + r;
      if (o >= mout) continue;
      const float bv = bias && split == 0 ? ld(bias + o) : 0.f;
      const size_t at = ((size_t)n * mout + o) * plane + (size_t)r0 * W;
#pragma unroll
      for (int i = 0; i < kC16Gpw; ++i) {
        const int q = (wave + 4 * i) * 16 + (lane & 15);
        if (r0 * W + q < plane) {
          if (ksplit > 1)
            partial[(size_t)split * batch * mout * plane + at + q] = acc[i][m][r] + bv;
          else
            st(out + at + q, acc[i][m][r] + bv);
        }
      }
    }
  }
}


// ---- stride 2, input gradient ---------------------------------------------------------------------------------
// gin[c][y][x] = sum over outputs o and the taps (th, tw) with y + 1 - th and x + 1 - tw even of
//                W[o][c][th][tw] * gout[o][(y + 1 - th) / 2][(x + 1 - tw) / 2].
// The input pixels fall into four parity classes: y = 2 j + py takes th = 1 (gout row j) when py = 0 and
// th = 0, 2 (rows j + 1, j) when py = 1, and x = 2 i + px likewise -- 1, 2, 2 and 4 taps, nine matrix
// instructions per 2 x 2 quad of input pixels, each against the gout tile at a fixed offset (dj, di) from the
// quad's (j, i).  The gout tile (at most 32 channels: one chunk) is staged channel-interleaved as in the stride-1
// kernel, with a zero row below and a zero column to the right; a lane holds the sums of both px of its quads
// and writes them as one 4-byte pair.  A workgroup owns 448 quads (whole j rows) of an image and MTB blocks of
// 16 channels; further blocks go to further workgroups on the same tile.
// grid = (image, tile of j rows, walk of MTB row blocks)
template <typename T, int WIN, int MTB>
__global__ __launch_bounds__(kC16Block, 2) void conv16_s2_bwd_kernel(int batch, int kin, int mout, int h, int ho,
                                                                     int tiles, int blocks,
                                                                     const T* __restrict__ gout,
                                                                     const uint4* __restrict__ wp, T* __restrict__ gin) {
  constexpr int WO = WIN / 2, TJ = kC16Pix / WO, RS = WO + 1;
  static_assert(WIN % 2 == 0 && TJ * WO == kC16Pix, "whole rows of quads");
  extern __shared__ __align__(16) unsigned tile[];  // [rows + 1][RS][kC16Pitch]

  const int walks = (blocks + MTB - 1) / MTB;
  const int total = batch * tiles * walks;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int mb0 = (lb % walks) * MTB, n = lb / walks / tiles, j0 = (lb / walks % tiles) * TJ;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int plane_o = ho * WO;

  const int rows = min(TJ, ho - j0);  // j rows of the tile; gout rows j0 .. j0 + rows are staged (the last may be zero)
  const int live_groups = (rows * WO + 15) / 16;
  for (int e = threadIdx.x; e < (rows + 1) * RS * kC16Pitch; e += kC16Block) tile[e] = 0u;
  __syncthreads();
  {
    const rsrc_t rs = plane_rsrc(gout + (size_t)n * kin * plane_o, kin * plane_o);
    for (int e = threadIdx.x; e < (rows + 1) * 4 * WO; e += kC16Block) {
      const int col = e % WO, jr = e / WO % (rows + 1), oct = e / WO / (rows + 1);
      const int row = j0 + jr;
      unsigned v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const unsigned o = row < ho ? (unsigned)((oct * 8 + k) * plane_o + row * WO + col) * 2u : kOutOfRange;
        v[k] = __builtin_amdgcn_raw_buffer_load_b16(rs, (int)o, 0, 0);
      }
      *reinterpret_cast<uint4*>(tile + (jr * RS + col) * kC16Pitch + oct * 4) =
          make_uint4(v[0] | v[1] << 16, v[2] | v[3] << 16, v[4] | v[5] << 16, v[6] | v[7] << 16);
    }
  }
  __syncthreads();

  int bword[kC16Gpw];
#pragma unroll
  for (int i = 0; i < kC16Gpw; ++i) {
    const int q = min((wave + 4 * i) * 16 + (lane & 15), rows * WO - 1);
    bword[i] = ((q / WO) * RS + q % WO) * kC16Pitch + (lane >> 4) * 4;
  }

#pragma unroll
  for (int py = 0; py < 2; ++py) {
    c16f4 acc[2][kC16Gpw][MTB];
#pragma unroll
    for (int px = 0; px < 2; ++px)
#pragma unroll
      for (int i = 0; i < kC16Gpw; ++i)
#pragma unroll
        for (int m = 0; m < MTB; ++m) acc[px][i][m] = c16f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int th = 0; th < 3; ++th) {
      if ((th == 1) != (py == 0)) continue;  // py = 0: th = 1; py = 1: th = 0, 2
      const int dj = th == 0 ? 1 : 0;
#pragma unroll
      for (int tw = 0; tw < 3; ++tw) {
        const int px = tw == 1 ? 0 : 1, di = tw == 0 ? 1 : 0;
        const int shift = (dj * RS + di) * kC16Pitch;
        uint4 a[MTB];
#pragma unroll
        for (int m = 0; m < MTB; ++m)  // the packed copy holds tap 8 - t at index t
          a[m] = wp[((size_t)(8 - (th * 3 + tw)) * blocks + min(mb0 + m, blocks - 1)) * 64 + lane];
#pragma unroll
        for (int i = 0; i < kC16Gpw; ++i) {
          if constexpr (WO <= 14)
            if (wave + 4 * i >= live_groups) break;
          const uint4 b = *reinterpret_cast<const uint4*>(tile + bword[i] + shift);
#pragma unroll
          for (int m = 0; m < MTB; ++m) acc[px][i][m] = mma16<T>(a[m], b, acc[px][i][m]);
        }
      }
    }
    // lane (quad l % 16 of each group, channels 4 (l / 16) .. + 3 of each block): the pair (x = 2 i, 2 i + 1)
#pragma unroll
    for (int m = 0; m < MTB; ++m) {
      if (mb0 + m >= blocks) break;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int c = 16 * (mb0 + m) + 4 * (lane >> 4) + r;
        if (c >= mout) continue;
        T* plane = gin + ((size_t)n * mout + c) * h * WIN;
#pragma unroll
        for (int i = 0; i < kC16Gpw; ++i) {
          const int q = (wave + 4 * i) * 16 + (lane & 15);
          const int y = 2 * (j0 + q / WO) + py;
          if (q < rows * WO && y < h) {
            const unsigned pair = bits16<T>(acc[0][i][m][r]) | bits16<T>(acc[1][i][m][r]) << 16;
            *reinterpret_cast<unsigned*>(plane + (size_t)y * WIN + 2 * (q % WO)) = pair;  // (x even, rows of even length)
          }
        }
      }
    }
  }
}

size_t round_up_256(size_t n) { return (n + 255) / 256 * 256; }
size_t pack_bytes(int kin, int mout) {
  return (size_t)9 * ceil_div(kin, kC16Chunk) * ceil_div(mout, 16) * 64 * sizeof(uint4);
}

// Chunk splits of a pass: enough for about two workgroups per CU, at least four chunks per split
int conv16_splits(int batch, int kin, int mout, int h, int w, int mtb) {
  const long base = std::max(1L, (long)batch * ceil_div(h, kC16Pix / w) * ceil_div(ceil_div(mout, 16), mtb));
  if (base >= 256) return 1;
  return (int)std::max<long>(1, std::min<long>((512 + base - 1) / base, ceil_div(kin, kC16Chunk) / 4));
}

template <typename T, int MTB>
bool launch_conv16(int batch, int kin, int mout, int h, int w, const T* in, const uint4* wp, const T* bias, T* out,
                   float* partial, hipStream_t stream) {
  const int chunks = ceil_div(kin, kC16Chunk), blocks = ceil_div(mout, 16);
  const int ksplit = conv16_splits(batch, kin, mout, h, w, MTB);
#define DK_C16(WW)                                                                                                     \
  {                                                                                                                    \
    const int tiles = ceil_div(h, Tile16<WW>::TH);                                                                     \
    const size_t lds = (size_t)Tile16<WW>::POS * kC16Pitch * sizeof(unsigned);                                         \
    const long wgs = (long)batch * tiles * ceil_div(blocks, MTB) * ksplit;                                             \
    conv16_kernel<T, WW, MTB><<<(unsigned)xcd_grid_size(wgs), kC16Block, lds, stream>>>(                               \
        batch, kin, mout, h, tiles, chunks, blocks, in, wp, bias, out, partial, ksplit);                               \
  }
  switch (w) {
    case 7: DK_C16(7) break;
    case 14: DK_C16(14) break;
    case 28: DK_C16(28) break;
    case 56: DK_C16(56) break;
    case 112: DK_C16(112) break;
    default: return false;
  }
#undef DK_C16
  if (ksplit > 1) launch_reduce_partials<float, T>(partial, ksplit, (long)batch * mout * h * w, out, stream);
  return true;
}

}  // namespace

bool offset_conv16_supported(int cin, int cout, int h, int w) {
  return cin >= 1 && cout >= 1 && cout <= 32 && h >= 1 && (w == 7 || w == 14 || w == 28 || w == 56 || w == 112) &&
         (long)kC16Chunk * h * w * 2 < (1L << 31) && (long)cin * h * w < (1L << 31) && (long)cout * h * w < (1L << 31);
}

// packed weights of either pass, then the forward's partial outputs (the input gradient has one chunk: no splits)
size_t offset_conv16_workspace(int batch, int cin, int cout, int h, int w) {
  const int mtb = ceil_div(cout, 16) == 1 ? 1 : 2;
  const int ks = conv16_splits(batch, cin, cout, h, w, mtb);
  return round_up_256(std::max(pack_bytes(cin, cout), pack_bytes(cout, cin))) +
         (ks > 1 ? (size_t)ks * batch * cout * h * w * sizeof(float) : 0);
}

template <typename T>
bool offset_conv16_forward(int batch, int cin, int cout, int h, int w, const T* x, const T* weight, const T* bias,
                           T* out, void* ws, hipStream_t stream) {
  if (!offset_conv16_supported(cin, cout, h, w)) return false;
  if (batch == 0) return true;
  uint4* wp = static_cast<uint4*>(ws);
  float* partial = reinterpret_cast<float*>(static_cast<char*>(ws) +
                                            round_up_256(std::max(pack_bytes(cin, cout), pack_bytes(cout, cin))));
  const int chunks = ceil_div(cin, kC16Chunk), blocks = ceil_div(cout, 16);
  conv16_pack_kernel<T><<<ceil_div(9 * chunks * blocks * 64, 256), 256, 0, stream>>>(weight, cout, cin, 0, chunks, blocks, wp);
  return blocks == 1 ? launch_conv16<T, 1>(batch, cin, cout, h, w, x, wp, bias, out, partial, stream)
                     : launch_conv16<T, 2>(batch, cin, cout, h, w, x, wp, bias, out, partial, stream);
}

template <typename T>
bool offset_conv16_backward_input(int batch, int cin, int cout, int h, int w, const T* gout, const T* weight, T* gin,
                                  void* ws, hipStream_t stream) {
  if (!offset_conv16_supported(cin, cout, h, w)) return false;
  if (batch == 0) return true;
  uint4* wp = static_cast<uint4*>(ws);
  const int chunks = ceil_div(cout, kC16Chunk), blocks = ceil_div(cin, 16);
  conv16_pack_kernel<T><<<ceil_div(9 * chunks * blocks * 64, 256), 256, 0, stream>>>(weight, cout, cin, 1, chunks, blocks, wp);
  return launch_conv16<T, 3>(batch, cout, cin, h, w, gout, wp, static_cast<const T*>(nullptr), gin,
                             static_cast<float*>(nullptr), stream);
}


// stride 2: input planes 14, 28, 56 or 112 wide (even), at most 32 outputs
bool offset_conv16_s2_supported(int cin, int cout, int h, int w) {
  return cin >= 1 && cout >= 1 && cout <= 32 && h >= 1 && (w == 14 || w == 28 || w == 56 || w == 112) &&
         (long)kS2Chunk * h * w * 2 < (1L << 31) && (long)cin * h * w < (1L << 31) && (long)cout * h * w < (1L << 31);
}

static int s2_splits(int batch, int cin, int ho, int wo) {
  const long base = std::max(1L, (long)batch * ceil_div(ho, kC16Pix / wo));
  if (base >= 256) return 1;
  return (int)std::max<long>(1, std::min<long>((512 + base - 1) / base, ceil_div(cin, kS2Chunk) / 4));
}

static size_t s2_pack_bytes(int cin, int cout) {
  return (size_t)9 * ceil_div(cin, kS2Chunk) * ceil_div(cout, 16) * 64 * sizeof(uint2);
}

size_t offset_conv16_s2_workspace(int batch, int cin, int cout, int h, int w) {
  const int ho = (h - 1) / 2 + 1, wo = w / 2;
  const int ks = s2_splits(batch, cin, ho, wo);
  return (s2_pack_bytes(cin, cout) + 255) / 256 * 256 + (ks > 1 ? (size_t)ks * batch * cout * ho * wo * sizeof(float) : 0);
}

template <typename T, int MTB>
static bool launch_conv16_s2(int batch, int cin, int cout, int h, int w, const T* x, const uint2* wp, const T* bias,
                             T* out, float* partial, hipStream_t stream) {
  const int ho = (h - 1) / 2 + 1, wo = w / 2;
  const int chunks = ceil_div(cin, kS2Chunk), blocks = ceil_div(cout, 16);
  const int ksplit = s2_splits(batch, cin, ho, wo);
  bool ok = true;
#define DK_S2(WW)                                                                                                      \
  {                                                                                                                    \
    auto kernel = conv16_s2_kernel<T, WW, MTB>;                                                                        \
    constexpr int TH = kC16Pix / (WW / 2);                                                                             \
    const int tiles = ceil_div(ho, TH);                                                                                \
    const size_t lds = (size_t)(2 * std::min(TH, ho) + 1) * (WW + 2) * kS2Pitch * sizeof(unsigned);                    \
    if (lds > (size_t)kMaxDynamicLds || !allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel)))                 \
      ok = false;                                                                                                      \
    else                                                                                                               \
      kernel<<<(unsigned)xcd_grid_size((long)batch * tiles * ksplit), kC16Block, lds, stream>>>(                       \
          batch, cin, cout, h, ho, tiles, chunks, blocks, x, wp, bias, out, partial, ksplit);                          \
  }
  switch (w) {
    case 14: DK_S2(14) break;
    case 28: DK_S2(28) break;
    case 56: DK_S2(56) break;
    case 112: DK_S2(112) break;
    default: ok = false;
  }
#undef DK_S2
  if (ok && ksplit > 1) launch_reduce_partials<float, T>(partial, ksplit, (long)batch * cout * ho * wo, out, stream);
  return ok;
}

template <typename T>
bool offset_conv16_s2_forward(int batch, int cin, int cout, int h, int w, const T* x, const T* weight, const T* bias,
                              T* out, void* ws, hipStream_t stream) {
  if (!offset_conv16_s2_supported(cin, cout, h, w)) return false;
  if (batch == 0) return true;
  uint2* wp = static_cast<uint2*>(ws);
  float* partial = reinterpret_cast<float*>(static_cast<char*>(ws) + (s2_pack_bytes(cin, cout) + 255) / 256 * 256);
  const int chunks = ceil_div(cin, kS2Chunk), blocks = ceil_div(cout, 16);
  conv16_s2_pack_kernel<T><<<ceil_div(9 * chunks * blocks * 64, 256), 256, 0, stream>>>(weight, cout, cin, chunks, blocks, wp);
  return blocks == 1 ? launch_conv16_s2<T, 1>(batch, cin, cout, h, w, x, wp, bias, out, partial, stream)
                     : launch_conv16_s2<T, 2>(batch, cin, cout, h, w, x, wp, bias, out, partial, stream);
}


size_t offset_conv16_s2_backward_input_workspace(int cin, int cout) { return pack_bytes(cout, cin); }

template <typename T>
bool offset_conv16_s2_backward_input(int batch, int cin, int cout, int h, int w, const T* gout, const T* weight,
                                     T* gin, void* ws, hipStream_t stream) {
  if (!offset_conv16_s2_supported(cin, cout, h, w) || cout > kC16Chunk) return false;
  if (batch == 0) return true;
  uint4* wp = static_cast<uint4*>(ws);
  const int ho = (h - 1) / 2 + 1, blocks = ceil_div(cin, 16);
  conv16_pack_kernel<T><<<ceil_div(9 * blocks * 64, 256), 256, 0, stream>>>(weight, cout, cin, 1, 1, blocks, wp);
  constexpr int MTB = 2;
  bool ok = true;
#define DK_S2B(WW)                                                                                                     \
  {                                                                                                                    \
    auto kernel = conv16_s2_bwd_kernel<T, WW, MTB>;                                                                    \
    constexpr int TJ = kC16Pix / (WW / 2);                                                                             \
    const int tiles = ceil_div(ho, TJ);                                                                                \
    const size_t lds = (size_t)(std::min(TJ, ho) + 1) * (WW / 2 + 1) * kC16Pitch * sizeof(unsigned);                   \
    if (lds > (size_t)kMaxDynamicLds || !allow_max_dynamic_lds(reinterpret_cast<const void*>(kernel)))                 \
      ok = false;                                                                                                      \
    else                                                                                                               \
      kernel<<<(unsigned)xcd_grid_size((long)batch * tiles * ceil_div(blocks, MTB)), kC16Block, lds, stream>>>(        \
          batch, cout, cin, h, ho, tiles, blocks, gout, wp, gin);                                                      \
  }
  switch (w) {
    case 14: DK_S2B(14) break;
    case 28: DK_S2B(28) break;
    case 56: DK_S2B(56) break;
    case 112: DK_S2B(112) break;
    default: ok = false;
  }
#undef DK_S2B
  return ok;
}

#define DK_INST(T)                                                                                                      \
  template bool offset_conv16_forward<T>(int, int, int, int, int, const T*, const T*, const T*, T*, void*, hipStream_t); \
  template bool offset_conv16_backward_input<T>(int, int, int, int, int, const T*, const T*, T*, void*, hipStream_t);  \
  template bool offset_conv16_s2_forward<T>(int, int, int, int, int, const T*, const T*, const T*, T*, void*, hipStream_t); \
  template bool offset_conv16_s2_backward_input<T>(int, int, int, int, int, const T*, const T*, T*, void*, hipStream_t);
DK_INST(__half)
DK_INST(bf16_t)
#undef DK_INST

}  // namespace dk
