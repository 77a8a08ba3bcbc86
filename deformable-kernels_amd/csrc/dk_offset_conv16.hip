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
//
// float32 tensors take the same kernels with every element as a bfloat16 (hi, lo) pair, hi = bf16(v),
// lo = bf16(v - hi): a chunk then holds half as many channels, an operand octet is four channels' hi parts
// followed by their lo parts, and the A operands come twice over the same octet, [Wh Wh] and [Wl Wl], so two
// instructions add all four products (Wh + Wl)(xh + xl).  A pair represents its float to 2^-18, the sums are
// fp32: the error against the float64 convolution is about 1e-6 of the result's scale (the fp32 matrix
// instructions: 2e-7 .. 1.3e-6), at half their matrix time.  An infinite element gives NaN (lo = inf - inf).
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

// float32 tensors: bfloat16 pairs (see the head of the file)
template <typename T>
constexpr bool kPairs = sizeof(T) == 4;
template <typename T>
constexpr int kParts = kPairs<T> ? 2 : 1;  // A operands per (tap, chunk, row block)
template <typename T>
constexpr int kChunkOf = kC16Chunk / kParts<T>;  // channels per K = 32 chunk
template <typename T>
constexpr int kOctOf = 8 / kParts<T>;  // channels per operand octet

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
  if constexpr (std::is_same<T, __half>::value)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(c16h8, a), __builtin_bit_cast(c16h8, b), acc, 0, 0, 0);
  else  // bfloat16 tensors, and the bfloat16 pairs of float32 ones
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(c16b8, a), __builtin_bit_cast(c16b8, b), acc, 0, 0, 0);
}

// The 16 bits of weight element `at` as an operand: the element itself, or part 0 (hi) / 1 (lo) of a float's pair
template <typename T>
__device__ __forceinline__ unsigned weight_bits(const T* w, size_t at, int part) {
  if constexpr (kPairs<T>) {
    const float v = w[at];
    const unsigned hi = pack_bf16(v, 0.f) & 0xffffu;
    return part == 0 ? hi : pack_bf16(v - bf16_lo(hi), 0.f) & 0xffffu;
  } else {
    return reinterpret_cast<const unsigned short*>(w)[at];
  }
}

// One operand octet of a staged position: channels c .. c + kOctOf - 1 of the buffer, `elem` the index of channel
// c's element and `plane` the channel stride (elements).  16-bit tensors: the eight elements; float32: four hi
// parts, then the four lo parts.  !live: zeros (the offset fails the range check).
template <typename T>
__device__ __forceinline__ uint4 load_octet(rsrc_t rs, bool live, unsigned elem, unsigned plane) {
  if constexpr (kPairs<T>) {
    float f[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      f[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                           rs, (int)(live ? (elem + j * plane) * 4u : kOutOfRange), 0, 0));
    const unsigned h01 = pack_bf16(f[0], f[1]), h23 = pack_bf16(f[2], f[3]);
    return make_uint4(h01, h23, pack_bf16(f[0] - bf16_lo(h01), f[1] - bf16_hi(h01)),
                      pack_bf16(f[2] - bf16_lo(h23), f[3] - bf16_hi(h23)));
  } else {
    unsigned v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      v[j] = __builtin_amdgcn_raw_buffer_load_b16(rs, (int)(live ? (elem + j * plane) * 2u : kOutOfRange), 0, 0);
    return make_uint4(v[0] | v[1] << 16, v[2] | v[3] << 16, v[4] | v[5] << 16, v[6] | v[7] << 16);
  }
}

// wp[t][chunk][block][part][lane] = the lane's eight operand elements of A_t, rows 16 block + lane % 16, zeros past
// the tensor.  16-bit tensors (one part): k = 32 chunk + 8 (lane / 16) .. + 7.  float32 (parts hi, lo): the part
// of k = 16 chunk + 4 (lane / 16) .. + 3, twice.  weight is [O][C][3][3]; forward: rows = O, k = C; transposed:
// rows = C, k = O, taps flipped.
template <typename T>
__global__ void conv16_pack_kernel(const T* __restrict__ weight, int O, int C, int transposed, int chunks, int blocks,
                                   uint4* __restrict__ wp) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= 9 * chunks * blocks * kParts<T> * 64) return;
  const int lane = idx % 64, part = idx / 64 % kParts<T>, rest = idx / 64 / kParts<T>;
  const int mb = rest % blocks, ch = rest / blocks % chunks, t = rest / blocks / chunks;
  const int m = 16 * mb + (lane & 15), k0 = kChunkOf<T> * ch + kOctOf<T> * (lane >> 4);
  unsigned v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int k = k0 + j % kOctOf<T>;
    const int o = transposed ? k : m, c = transposed ? m : k;
    v[j] = (o < O && c < C) ? weight_bits<T>(weight, ((size_t)o * C + c) * 9 + (transposed ? 8 - t : t), part) : 0u;
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
        const int kc = min(kChunkOf<T>, kin - ch * kChunkOf<T>);
        const rsrc_t rs = plane_rsrc(in + ((size_t)n * kin + (size_t)ch * kChunkOf<T>) * plane, kc * plane);
        for (int e = threadIdx.x; e < (rows + 2) * 4 * W; e += kC16Block) {
          const int col = e % W, ry = e / W % (rows + 2), oct = e / W / (rows + 2);
          const int row = r0 - 1 + ry;
          *reinterpret_cast<uint4*>(tile + (ry * RS + col + 1) * kC16Pitch + oct * 4) = load_octet<T>(
              rs, row >= 0 && row < h, (unsigned)(oct * kOctOf<T> * plane + row * W + col), (unsigned)plane);
        }
        __syncthreads();
      }
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        const int shift = ((t / 3 - 1) * RS + (t % 3 - 1)) * kC16Pitch;
        uint4 a[MTB][kParts<T>];
#pragma unroll
        for (int m = 0; m < MTB; ++m) {
          const int mb = min(mb0 + m, blocks - 1);  // a block past the last repeats it; its results are not stored
#pragma unroll
          for (int p = 0; p < kParts<T>; ++p)
            a[m][p] = wp[(((size_t)(t * chunks + ch) * blocks + mb) * kParts<T> + p) * 64 + lane];
        }
#pragma unroll
        for (int i = 0; i < kC16Gpw; ++i) {
          // planes lower than the tile (uniform: the wave's remaining groups lie below the image)
          if constexpr (W <= 14)
            if (wave + 4 * i >= live_groups) break;
          const uint4 b = *reinterpret_cast<const uint4*>(tile + bword[i] + shift);
#pragma unroll
          for (int m = 0; m < MTB; ++m)
#pragma unroll
            for (int p = 0; p < kParts<T>; ++p) acc[i][m] = mma16<T>(a[m][p], b, acc[i][m]);
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
  if constexpr (std::is_same<T, __half>::value)
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(c16h4, a), __builtin_bit_cast(c16h4, b), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(c16b4, a), __builtin_bit_cast(c16b4, b), acc, 0, 0, 0);
}

template <typename T>
constexpr int kS2ChunkOf = kS2Chunk / kParts<T>;  // channels per K = 16 chunk

// wp[t][chunk][block][part][lane] = the lane's four operand elements of W[16 block + lane % 16][.][t]: 16-bit
// tensors, channels 16 chunk + 4 (lane / 16) .. + 3; float32, the part (hi, lo) of channels 8 chunk + 2 (lane / 16),
// + 1, twice
template <typename T>
__global__ void conv16_s2_pack_kernel(const T* __restrict__ weight, int O, int C, int chunks, int blocks,
                                      uint2* __restrict__ wp) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= 9 * chunks * blocks * kParts<T> * 64) return;
  const int lane = idx % 64, part = idx / 64 % kParts<T>, rest = idx / 64 / kParts<T>;
  const int mb = rest % blocks, ch = rest / blocks % chunks, t = rest / blocks / chunks;
  constexpr int kQuad = 4 / kParts<T>;  // channels per operand quad
  const int o = 16 * mb + (lane & 15), c0 = kS2ChunkOf<T> * ch + kQuad * (lane >> 4);
  unsigned v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = c0 + j % kQuad;
    v[j] = (o < O && c < C) ? weight_bits<T>(weight, ((size_t)o * C + c) * 9 + t, part) : 0u;
  }
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
    const int kc = min(kS2ChunkOf<T>, kin - ch * kS2ChunkOf<T>);
    const rsrc_t rs = plane_rsrc(in + ((size_t)n * kin + (size_t)ch * kS2ChunkOf<T>) * plane_in, kc * plane_in);
    for (int e = threadIdx.x; e < rows_in * 2 * WIN; e += kC16Block) {
      const int col = e % WIN, ry = e / WIN % rows_in, oct = e / WIN / rows_in;
      const int row = 2 * r0 - 1 + ry;
      const uint4 v = load_octet<T>(rs, row >= 0 && row < h, (unsigned)(oct * kOctOf<T> * plane_in + row * WIN + col),
                                    (unsigned)plane_in);
      // two operand quads: four elements each, or two channels' hi parts and their lo parts
      uint2* dst = reinterpret_cast<uint2*>(tile + (ry * RS + col + 1) * kS2Pitch + oct * 4);
      dst[0] = kPairs<T> ? make_uint2(v.x, v.z) : make_uint2(v.x, v.y);
      dst[1] = kPairs<T> ? make_uint2(v.y, v.w) : make_uint2(v.z, v.w);
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < 9; ++t) {
      const int shift = ((t / 3) * RS + t % 3) * kS2Pitch;
      uint2 a[MTB][kParts<T>];
#pragma unroll
      for (int m = 0; m < MTB; ++m)
#pragma unroll
        for (int p = 0; p < kParts<T>; ++p)
          a[m][p] = wp[(((size_t)(t * chunks + ch) * blocks + min(m, blocks - 1)) * kParts<T> + p) * 64 + lane];
#pragma unroll
      for (int i = 0; i < kC16Gpw; ++i) {
        if constexpr (W <= 14)
          if (wave + 4 * i >= live_groups) break;
        const uint2 b = *reinterpret_cast<const uint2*>(tile + bword[i] + shift);
#pragma unroll
        for (int m = 0; m < MTB; ++m)
#pragma unroll
          for (int p = 0; p < kParts<T>; ++p) acc[i][m] = mma16k16<T>(a[m][p], b, acc[i][m]);
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
// quad's (j, i).  The gout tile (at most 32 channels: one chunk of 16-bit elements, two of float32 pairs, each with a
// tile of its own) is staged channel-interleaved as in the stride-1 kernel, with a zero row below and a zero column
// to the right; a lane holds the sums of both px of its quads
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
  extern __shared__ __align__(16) unsigned tile[];  // [chunk][rows + 1][RS][kC16Pitch]

  const int walks = (blocks + MTB - 1) / MTB;
  const int total = batch * tiles * walks;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int mb0 = (lb % walks) * MTB, n = lb / walks / tiles, j0 = (lb / walks % tiles) * TJ;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int plane_o = ho * WO;

  const int rows = min(TJ, ho - j0);  // j rows of the tile; gout rows j0 .. j0 + rows are staged (the last may be zero)
  const int live_groups = (rows * WO + 15) / 16;
  // one staged tile per chunk of gout channels (16-bit tensors: one chunk; float32 pairs, 18 channels: two)
  const int chunks = (kin + kChunkOf<T> - 1) / kChunkOf<T>;
  const int tile_words = (rows + 1) * RS * kC16Pitch;
  for (int e = threadIdx.x; e < chunks * tile_words; e += kC16Block) tile[e] = 0u;
  __syncthreads();
  for (int ch = 0; ch < chunks; ++ch) {
    const int kc = min(kChunkOf<T>, kin - ch * kChunkOf<T>);
    const rsrc_t rs = plane_rsrc(gout + ((size_t)n * kin + (size_t)ch * kChunkOf<T>) * plane_o, kc * plane_o);
    for (int e = threadIdx.x; e < (rows + 1) * 4 * WO; e += kC16Block) {
      const int col = e % WO, jr = e / WO % (rows + 1), oct = e / WO / (rows + 1);
      const int row = j0 + jr;
      *reinterpret_cast<uint4*>(tile + ch * tile_words + (jr * RS + col) * kC16Pitch + oct * 4) =
          load_octet<T>(rs, row < ho, (unsigned)(oct * kOctOf<T> * plane_o + row * WO + col), (unsigned)plane_o);
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
        for (int ch = 0; ch < chunks; ++ch) {
          uint4 a[MTB][kParts<T>];
#pragma unroll
          for (int m = 0; m < MTB; ++m)  // the packed copy holds tap 8 - t at index t
#pragma unroll
            for (int p = 0; p < kParts<T>; ++p)
              a[m][p] = wp[((((size_t)(8 - (th * 3 + tw)) * chunks + ch) * blocks + min(mb0 + m, blocks - 1)) * kParts<T> + p) * 64 + lane];
#pragma unroll
          for (int i = 0; i < kC16Gpw; ++i) {
            if constexpr (WO <= 14)
              if (wave + 4 * i >= live_groups) break;
            const uint4 b = *reinterpret_cast<const uint4*>(tile + ch * tile_words + bword[i] + shift);
#pragma unroll
            for (int m = 0; m < MTB; ++m)
#pragma unroll
              for (int p = 0; p < kParts<T>; ++p) acc[px][i][m] = mma16<T>(a[m][p], b, acc[px][i][m]);
          }
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
          if (q < rows * WO && y < h) {  // (x even, rows of even length: the pair is aligned)
            if constexpr (kPairs<T>) {
              *reinterpret_cast<float2*>(plane + (size_t)y * WIN + 2 * (q % WO)) = make_float2(acc[0][i][m][r], acc[1][i][m][r]);
            } else {
              const unsigned pair = bits16<T>(acc[0][i][m][r]) | bits16<T>(acc[1][i][m][r]) << 16;
              *reinterpret_cast<unsigned*>(plane + (size_t)y * WIN + 2 * (q % WO)) = pair;
            }
          }
        }
      }
    }
  }
}

size_t round_up_256(size_t n) { return (n + 255) / 256 * 256; }
// pairs: float32 tensors (two A operands per block, 16 channels per chunk)
size_t pack_bytes(int kin, int mout, bool pairs) {
  return (size_t)9 * ceil_div(kin, pairs ? kC16Chunk / 2 : kC16Chunk) * ceil_div(mout, 16) * (pairs ? 2 : 1) * 64 * sizeof(uint4);
}

// Chunk splits of a pass: enough for about two workgroups per CU, at least four chunks per split
int conv16_splits(int batch, int kin, int mout, int h, int w, int mtb, bool pairs) {
  const long base = std::max(1L, (long)batch * ceil_div(h, kC16Pix / w) * ceil_div(ceil_div(mout, 16), mtb));
  if (base >= 256) return 1;
  return (int)std::max<long>(1, std::min<long>((512 + base - 1) / base, ceil_div(kin, pairs ? kC16Chunk / 2 : kC16Chunk) / 4));
}

template <typename T, int MTB>
bool launch_conv16(int batch, int kin, int mout, int h, int w, const T* in, const uint4* wp, const T* bias, T* out,
                   float* partial, hipStream_t stream) {
  const int chunks = ceil_div(kin, kChunkOf<T>), blocks = ceil_div(mout, 16);
  const int ksplit = conv16_splits(batch, kin, mout, h, w, MTB, kPairs<T>);
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

// packed weights of either pass, then the forward's partial outputs (the input gradient has few chunks: no splits)
size_t offset_conv16_workspace(int batch, int cin, int cout, int h, int w, bool pairs) {
  const int mtb = ceil_div(cout, 16) == 1 ? 1 : 2;
  const int ks = conv16_splits(batch, cin, cout, h, w, mtb, pairs);
  return round_up_256(std::max(pack_bytes(cin, cout, pairs), pack_bytes(cout, cin, pairs))) +
         (ks > 1 ? (size_t)ks * batch * cout * h * w * sizeof(float) : 0);
}

template <typename T>
bool offset_conv16_forward(int batch, int cin, int cout, int h, int w, const T* x, const T* weight, const T* bias,
                           T* out, void* ws, hipStream_t stream) {
  if (!offset_conv16_supported(cin, cout, h, w)) return false;
  if (batch == 0) return true;
  uint4* wp = static_cast<uint4*>(ws);
  float* partial = reinterpret_cast<float*>(
      static_cast<char*>(ws) + round_up_256(std::max(pack_bytes(cin, cout, kPairs<T>), pack_bytes(cout, cin, kPairs<T>))));
  const int chunks = ceil_div(cin, kChunkOf<T>), blocks = ceil_div(cout, 16);
  conv16_pack_kernel<T><<<ceil_div(9 * chunks * blocks * kParts<T> * 64, 256), 256, 0, stream>>>(weight, cout, cin, 0, chunks, blocks, wp);
  return blocks == 1 ? launch_conv16<T, 1>(batch, cin, cout, h, w, x, wp, bias, out, partial, stream)
                     : launch_conv16<T, 2>(batch, cin, cout, h, w, x, wp, bias, out, partial, stream);
}

template <typename T>
bool offset_conv16_backward_input(int batch, int cin, int cout, int h, int w, const T* gout, const T* weight, T* gin,
                                  void* ws, hipStream_t stream) {
  if (!offset_conv16_supported(cin, cout, h, w)) return false;
  if (batch == 0) return true;
  uint4* wp = static_cast<uint4*>(ws);
  const int chunks = ceil_div(cout, kChunkOf<T>), blocks = ceil_div(cin, 16);
  conv16_pack_kernel<T><<<ceil_div(9 * chunks * blocks * kParts<T> * 64, 256), 256, 0, stream>>>(weight, cout, cin, 1, chunks, blocks, wp);
  return launch_conv16<T, 3>(batch, cout, cin, h, w, gout, wp, static_cast<const T*>(nullptr), gin,
                             static_cast<float*>(nullptr), stream);
}


// stride 2: input planes 14, 28, 56 or 112 wide (even), at most 32 outputs
bool offset_conv16_s2_supported(int cin, int cout, int h, int w) {
  return cin >= 1 && cout >= 1 && cout <= 32 && h >= 1 && (w == 14 || w == 28 || w == 56 || w == 112) &&
         (long)kS2Chunk * h * w * 2 < (1L << 31) && (long)cin * h * w < (1L << 31) && (long)cout * h * w < (1L << 31);
}

static int s2_splits(int batch, int cin, int ho, int wo, bool pairs) {
  const long base = std::max(1L, (long)batch * ceil_div(ho, kC16Pix / wo));
  if (base >= 256) return 1;
  return (int)std::max<long>(1, std::min<long>((512 + base - 1) / base, ceil_div(cin, pairs ? kS2Chunk / 2 : kS2Chunk) / 4));
}

static size_t s2_pack_bytes(int cin, int cout, bool pairs) {
  return (size_t)9 * ceil_div(cin, pairs ? kS2Chunk / 2 : kS2Chunk) * ceil_div(cout, 16) * (pairs ? 2 : 1) * 64 * sizeof(uint2);
}

size_t offset_conv16_s2_workspace(int batch, int cin, int cout, int h, int w, bool pairs) {
  const int ho = (h - 1) / 2 + 1, wo = w / 2;
  const int ks = s2_splits(batch, cin, ho, wo, pairs);
  return round_up_256(s2_pack_bytes(cin, cout, pairs)) + (ks > 1 ? (size_t)ks * batch * cout * ho * wo * sizeof(float) : 0);
}

template <typename T, int MTB>
static bool launch_conv16_s2(int batch, int cin, int cout, int h, int w, const T* x, const uint2* wp, const T* bias,
                             T* out, float* partial, hipStream_t stream) {
  const int ho = (h - 1) / 2 + 1, wo = w / 2;
  const int chunks = ceil_div(cin, kS2ChunkOf<T>), blocks = ceil_div(cout, 16);
  const int ksplit = s2_splits(batch, cin, ho, wo, kPairs<T>);
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
  float* partial = reinterpret_cast<float*>(static_cast<char*>(ws) + round_up_256(s2_pack_bytes(cin, cout, kPairs<T>)));
  const int chunks = ceil_div(cin, kS2ChunkOf<T>), blocks = ceil_div(cout, 16);
  conv16_s2_pack_kernel<T><<<ceil_div(9 * chunks * blocks * kParts<T> * 64, 256), 256, 0, stream>>>(weight, cout, cin, chunks, blocks, wp);
  return blocks == 1 ? launch_conv16_s2<T, 1>(batch, cin, cout, h, w, x, wp, bias, out, partial, stream)
                     : launch_conv16_s2<T, 2>(batch, cin, cout, h, w, x, wp, bias, out, partial, stream);
}


size_t offset_conv16_s2_backward_input_workspace(int cin, int cout, bool pairs) { return pack_bytes(cout, cin, pairs); }

template <typename T>
bool offset_conv16_s2_backward_input(int batch, int cin, int cout, int h, int w, const T* gout, const T* weight,
                                     T* gin, void* ws, hipStream_t stream) {
  if (!offset_conv16_s2_supported(cin, cout, h, w) || cout > kC16Chunk) return false;
  if (kPairs<T> && reinterpret_cast<uintptr_t>(gin) % 8 != 0) return false;  // pairs of floats leave as 8-byte stores
  if (batch == 0) return true;
  uint4* wp = static_cast<uint4*>(ws);
  const int ho = (h - 1) / 2 + 1, blocks = ceil_div(cin, 16), chunks = ceil_div(cout, kChunkOf<T>);
  conv16_pack_kernel<T><<<ceil_div(9 * chunks * blocks * kParts<T> * 64, 256), 256, 0, stream>>>(weight, cout, cin, 1, chunks, blocks, wp);
  constexpr int MTB = 2;
  bool ok = true;
#define DK_S2B(WW)                                                                                                     \
  {                                                                                                                    \
    auto kernel = conv16_s2_bwd_kernel<T, WW, MTB>;                                                                    \
    constexpr int TJ = kC16Pix / (WW / 2);                                                                             \
    const int tiles = ceil_div(ho, TJ);                                                                                \
    const size_t lds = (size_t)chunks * (std::min(TJ, ho) + 1) * (WW / 2 + 1) * kC16Pitch * sizeof(unsigned);          \
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
DK_INST(float)
#undef DK_INST

}  // namespace dk
