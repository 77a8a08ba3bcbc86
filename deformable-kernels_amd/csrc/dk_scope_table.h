// Scope tables in LDS for the tuned kernels: the corner-expanded, difference-form table of a
// channel's scope tile, its staging, and the per-(pixel, tap) descriptor that addresses it.
// Shared by the local (dk_local_fast.hip) and the deformable (dk_deform_fast.hip) kernels.
#pragma once

#include "dk_common.h"

namespace dk {

// Corner-expanded scope table of one channel: one float4 per 2x2 block {tl, tr, bl, br} of the
// zero-padded tile, (SH + 1) x (SW + 1) blocks, so a tap needs a single 16-byte LDS read.
// The float4 holds the block in difference form
//   a = tl,  b = tr - tl,  c = bl - tl,  d = br - tr - bl + tl,
// which turns the bilinear read at fractional position (lh, lw) into three fused multiply-adds,
//   a + lw * b + lh * (c + lw * d),
// with only (lh, lw) per tap in registers, and makes its derivatives c + lw * d and b + lh * d.
//
// gfx950 serves a ds_read_b128 at 256 B/clk from 64 banks, so two float4 blocks collide when
// their block slots are congruent mod 16.  For the 5 x 5 blocks of a 4 x 4 scope the slots are
// permuted so that colliding pairs are blocks at opposite borders of the tile (4 apart in a
// coordinate, or a far corner against the opposite inner corner), which the lanes of one wave
// rarely address together; a row-major order would pair blocks only (3, 1) apart.
template <int SH, int SW>
struct WideTable {
  static constexpr int RS = SW + 1;
  static constexpr int BLOCKS = (SH + 1) * RS;
  static constexpr int SIZE = BLOCKS * 4;
  __host__ __device__ static constexpr int slot(int block) { return block; }
};

template <>
struct WideTable<4, 4> {
  static constexpr int RS = 5;
  static constexpr int BLOCKS = 25;
  static constexpr int SIZE = BLOCKS * 4;
  // block (r, c) = r * 5 + c  ->  slot; slots s and s + 16 share banks
  __host__ __device__ static constexpr int slot(int block) {
    constexpr signed char lut[25] = {
        /* r=0 */ 24, 0, 1, 2, 3,
        /* r=1 */ 4, 7, 9, 10, 20,
        /* r=2 */ 5, 11, 12, 13, 21,
        /* r=3 */ 6, 14, 15, 8, 22,
        /* r=4 */ 16, 17, 18, 19, 23};
    return lut[block];
  }
};

// Stage the tables of channels c_first + j * c_step, j < nch.  A thread owns one block of the
// tile for every (256 / 32)-th channel: which corners exist, their offsets in a channel's
// filter and the destination slot are fixed per thread, so a channel costs four range-checked
// loads (missing corners read 0), three subtractions and one 16-byte LDS write.
template <typename T, int SH, int SW>
__device__ __forceinline__ void stage_wide_tables(float* tbl, const T* filter, int channels, int c_first,
                                                  int c_step, int nch) {
  using Tb = WideTable<SH, SW>;
  constexpr int CB = Tb::BLOCKS <= 32 ? 32 : 64;  // threads per channel
  const int m = threadIdx.x % CB;
  if (m >= Tb::BLOCKS) return;
  const int i = m / Tb::RS - 1, k = m % Tb::RS - 1;
  unsigned off[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int ii = i + (q >> 1), kk = k + (q & 1);
    off[q] = (ii >= 0 && ii < SH && kk >= 0 && kk < SW) ? (unsigned)(ii * SW + kk) * (unsigned)sizeof(T) : kOutOfRange;
  }
  const rsrc_t rf = plane_rsrc(filter, channels * SH * SW);
  float* dst = tbl + Tb::slot(m) * 4;
  const int CPP = (int)blockDim.x / CB;  // channels per sweep of the workgroup
  constexpr int kSweeps = 4;        // sweeps whose loads are issued together
  for (int jb = threadIdx.x / CB; jb < nch; jb += kSweeps * CPP) {
    float tl[kSweeps], tr[kSweeps], bl[kSweeps], br[kSweeps];
#pragma unroll
    for (int u = 0; u < kSweeps; ++u) {
      const int j = jb + u * CPP;
      const unsigned cb = j < nch ? (unsigned)(c_first + j * c_step) * (unsigned)(SH * SW * sizeof(T)) : kOutOfRange;
      tl[u] = buf_ld(rf, off[0] + cb, filter);
      tr[u] = buf_ld(rf, off[1] + cb, filter);
      bl[u] = buf_ld(rf, off[2] + cb, filter);
      br[u] = buf_ld(rf, off[3] + cb, filter);
    }
#pragma unroll
    for (int u = 0; u < kSweeps; ++u) {
      const int j = jb + u * CPP;
      if (j < nch)
        *reinterpret_cast<float4*>(dst + j * Tb::SIZE) =
            make_float4(tl[u], tr[u] - tl[u], bl[u] - tl[u], (br[u] - tr[u]) - (bl[u] - tl[u]));
    }
  }
}

// Pair tables for kernels that need the derivatives only and take two channels per step: block m of
// channels (2 jp, 2 jp + 1) is {b, c, d} as three bfloat16 pairs (the even channel in the lower half)
// and an unused word, in the slot order of the wide table; table jp starts at tbl + jp * SIZE.  A
// channel past the last one leaves zeros.
template <typename T, int SH, int SW>
__device__ __forceinline__ void stage_pair_tables(float* tbl, const T* filter, int channels, int c_first,
                                                  int c_step, int nch) {
  using Tb = WideTable<SH, SW>;
  constexpr int CB = Tb::BLOCKS <= 32 ? 32 : 64;  // threads per table
  const int m = threadIdx.x % CB;
  if (m >= Tb::BLOCKS) return;
  const int i = m / Tb::RS - 1, k = m % Tb::RS - 1;
  unsigned off[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int ii = i + (q >> 1), kk = k + (q & 1);
    off[q] = (ii >= 0 && ii < SH && kk >= 0 && kk < SW) ? (unsigned)(ii * SW + kk) * (unsigned)sizeof(T) : kOutOfRange;
  }
  const rsrc_t rf = plane_rsrc(filter, channels * SH * SW);
  float* dst = tbl + Tb::slot(m) * 4;
  const int npair = (nch + 1) / 2;
  for (int jp = threadIdx.x / CB; jp < npair; jp += (int)blockDim.x / CB) {
    float d[2][3];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int j = 2 * jp + h;
      const unsigned cb = (unsigned)(c_first + min(j, nch - 1) * c_step) * (unsigned)(SH * SW * sizeof(T));
      const float tl = buf_ld(rf, off[0] + cb, filter), tr = buf_ld(rf, off[1] + cb, filter);
      const float bl = buf_ld(rf, off[2] + cb, filter), br = buf_ld(rf, off[3] + cb, filter);
      // (two out-of-range parts of an offset add up to an offset in range: the zeros are written out)
      d[h][0] = j < nch ? tr - tl : 0.f;
      d[h][1] = j < nch ? bl - tl : 0.f;
      d[h][2] = j < nch ? (br - tr) - (bl - tl) : 0.f;
    }
    *reinterpret_cast<uint4*>(dst + jp * Tb::SIZE) =
        make_uint4(pack_bf16(d[0][0], d[1][0]), pack_bf16(d[0][1], d[1][1]), pack_bf16(d[0][2], d[1][2]), 0u);
  }
}

// One 16-byte LDS read for a caller that uses only some components: the empty asm counts as
// a use of all four, so the compiler keeps the single wide read instead of two narrower ones
// (two LDS issues).
__device__ __forceinline__ float4 lds_read4(const float* p) {
  const float4 q = *reinterpret_cast<const float4*>(p);
  asm volatile("" ::"v"(q.x), "v"(q.y), "v"(q.z), "v"(q.w));
  return q;
}

// (pixel, tap) descriptor for the difference-form table: the LDS float index of the tap's
// block and the fractional position inside it.  A tap that contributes nothing (outside the
// scope band, in the padding, or not owned) points at block (-1, -1) with lh = lw = 0, which
// evaluates to that block's `a` entry: a padding zero.
struct LiteTap {
  int cell;
  float lh, lw;
};

template <int SH, int SW>
__device__ __forceinline__ LiteTap make_lite_tap(float h, float w, bool ok) {
  using Tb = WideTable<SH, SW>;
  const bool in = ok && (h > -1.f) && (w > -1.f) && (h < float(SH)) && (w < float(SW));
  const float hf = floorf(h), wf = floorf(w);
  LiteTap t;
  t.lh = in ? h - hf : 0.f;
  t.lw = in ? w - wf : 0.f;
  t.cell = Tb::slot(in ? (static_cast<int>(hf) + 1) * Tb::RS + static_cast<int>(wf) + 1 : 0) * 4;
  return t;
}

__device__ __forceinline__ float lite_weight(const LiteTap& t, const float4& q) {
  return fmaf(t.lh, fmaf(t.lw, q.w, q.z), fmaf(t.lw, q.y, q.x));
}

}  // namespace dk
