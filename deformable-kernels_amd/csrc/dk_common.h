// Shared device-side building blocks of the gfx950 deformable-kernel library:
// element I/O for the four dtypes, the geometry block passed to every kernel,
// the XCD-aware block order, wave-level reductions and buffer-addressed plane access.
//
// Semantics follow the reference's device helpers in
// deformable_kernels/ops/deform_kernel/csrc/filter_sample_depthwise_cuda_kernel.cu
// (cited as K.cu): planar_bilinear K.cu:51-83, its two backward forms
// K.cu:85-163, deformable_im2col_bilinear K.cu:165-229 and
// get_coordinate_weight K.cu:231-268.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/dk_hip.h"

namespace dk {

// ---------------------------------------------------------------------------
// element I/O: tensors are T in memory, arithmetic is compute_t<T>
// ---------------------------------------------------------------------------
struct bf16_t { uint16_t bits; };

template <typename T> struct compute { using type = float; };
template <> struct compute<double> { using type = double; };
template <typename T> using compute_t = typename compute<T>::type;

__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ double ld(const double* p) { return *p; }
__device__ __forceinline__ float ld(const __half* p) { return __half2float(*p); }
__device__ __forceinline__ float ld(const bf16_t* p) {
  return __uint_as_float(static_cast<uint32_t>(p->bits) << 16);
}
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(double* p, double v) { *p = v; }
__device__ __forceinline__ void st(__half* p, float v) { *p = __float2half_rn(v); }
__device__ __forceinline__ void st(bf16_t* p, float v) {
  // the hardware conversion (v_cvt_pk_bf16_f32): round to nearest even, a NaN stays a NaN
  p->bits = __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
}

// ---------------------------------------------------------------------------
// geometry handed to every kernel by value
// ---------------------------------------------------------------------------
struct Geo {
  int batch, channel, in_h, in_w;
  int k_h, k_w, stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
  int out_h, out_w;
  int scope_h, scope_w, groups;
  double centre_h, centre_w;  // (scope - k) / 2.0, the double literal of K.cu:338-341
  int clip_mode;              // kClipNone / kClipRotation / kClipCoord
  float clip_lo, clip_hi;
};

// Clamp of the kernel-space offsets, folded into the operator.  The reference clamps the rotation
// tensor in its module before the operator runs (modules/deform_kernel.py:185-212): a plain
// range on the offsets (kClipRotation), or "scope", a range on the scope coordinate
// f + r + centre (kClipCoord, with [0, scope_h - 1] for both axes as written there).  The
// gradient with respect to a clamped offset is zero, as torch.clamp's is.
enum { kClipNone = 0, kClipRotation = 1, kClipCoord = 2 };

// Scope coordinate of tap f with kernel-space offset r.  The reference writes
// `f + r + (scope - k) / 2.0`: int + scalar_t in scalar_t, then + double in
// double, rounded to scalar_t on assignment.  Reproduced operation by
// operation so the floor below lands on the same cell as the reference's.
// For float the detour through double is a single correctly rounded float
// addition: the centre is a multiple of 0.5, so float(t) + centre is exact in
// double (or leaves t unchanged when t is huge) and its rounding to float is
// what the float addition returns.
template <typename CT>
__device__ __forceinline__ CT scope_coord(int f, CT r, double centre) {
  CT t = static_cast<CT>(f) + r;
  if constexpr (sizeof(CT) == 4)
    return t + static_cast<CT>(centre);
  else
    return static_cast<CT>(static_cast<double>(t) + centre);
}

// The same with the descriptor's clamp applied; `open` tells whether the offset was inside the
// range (its gradient passes) or clamped (gradient zero).
template <typename CT>
__device__ __forceinline__ CT scope_coord(const Geo& g, int f, CT r, double centre, bool* open = nullptr) {
  bool inside = true;
  if (g.clip_mode == kClipRotation) {
    inside = r >= static_cast<CT>(g.clip_lo) && r <= static_cast<CT>(g.clip_hi);
    r = r < static_cast<CT>(g.clip_lo) ? static_cast<CT>(g.clip_lo) : r;
    r = r > static_cast<CT>(g.clip_hi) ? static_cast<CT>(g.clip_hi) : r;
  }
  CT c = scope_coord<CT>(f, r, centre);
  if (g.clip_mode == kClipCoord) {
    inside = c >= static_cast<CT>(g.clip_lo) && c <= static_cast<CT>(g.clip_hi);
    c = c < static_cast<CT>(g.clip_lo) ? static_cast<CT>(g.clip_lo) : c;
    c = c > static_cast<CT>(g.clip_hi) ? static_cast<CT>(g.clip_hi) : c;
  }
  if (open) *open = inside;
  return c;
}

__host__ __device__ __forceinline__ int ceil_div(int a, int b) { return (a + b - 1) / b; }

// ---------------------------------------------------------------------------
// XCD-aware block order.  MI355X has 8 XCDs with one L2 each, and the dispatcher hands
// consecutive workgroups of a grid to consecutive XCDs (block b runs on XCD b % 8).  Work items
// that share data (the tiles of one image, the channel splits of one tile) should therefore not
// be consecutive blocks but blocks congruent mod 8.  Grids are launched 1-D with
// xcd_grid_size(total) blocks; logical_block() gives block b the logical index
//   (b % 8) * ceil(total / 8) + b / 8,
// so each XCD walks one contiguous eighth of the logical order.  Indices >= total (at most 7)
// are padding and must exit.
// ---------------------------------------------------------------------------
constexpr int kXcds = 8;
__host__ __device__ __forceinline__ long xcd_grid_size(long total) { return (total + kXcds - 1) / kXcds * kXcds; }
__device__ __forceinline__ int logical_block(int total) {
  const int chunk = (total + kXcds - 1) / kXcds;
  return (int)(blockIdx.x % kXcds) * chunk + (int)(blockIdx.x / kXcds);
}

// Sum of v over the 64 lanes of the wave, returned in every lane: six DPP adds and one readlane
// (no LDS crossbar traffic, unlike a shuffle-based butterfly).
__device__ __forceinline__ float wave_sum(float v) {
#define DK_DPP_ADD(ctrl, row_mask)                                                              \
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, row_mask, 0xf, true))
  DK_DPP_ADD(0xB1, 0xf);   // quad_perm [1,0,3,2]
  DK_DPP_ADD(0x4E, 0xf);   // quad_perm [2,3,0,1]
  DK_DPP_ADD(0x141, 0xf);  // row_half_mirror
  DK_DPP_ADD(0x140, 0xf);  // row_mirror: every lane now holds its 16-lane row's sum
  DK_DPP_ADD(0x142, 0xa);  // row_bcast15 into rows 1 and 3
  DK_DPP_ADD(0x143, 0xc);  // row_bcast31 into rows 2 and 3: lane 63 holds the total
#undef DK_DPP_ADD
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Least / largest v over the 64 lanes of the wave, returned in every lane: the same six DPP steps (a lane that a
// step's row mask leaves out, or that has no source lane, compares with its own value).
__device__ __forceinline__ int wave_min(int v) {
#define DK_DPP_MIN(ctrl, row_mask) v = min(v, __builtin_amdgcn_update_dpp(v, v, ctrl, row_mask, 0xf, false))
  DK_DPP_MIN(0xB1, 0xf);
  DK_DPP_MIN(0x4E, 0xf);
  DK_DPP_MIN(0x141, 0xf);
  DK_DPP_MIN(0x140, 0xf);
  DK_DPP_MIN(0x142, 0xa);
  DK_DPP_MIN(0x143, 0xc);
#undef DK_DPP_MIN
  return __builtin_amdgcn_readlane(v, 63);
}
__device__ __forceinline__ int wave_max(int v) { return -wave_min(-v); }

// Value held by the previous / next lane of the wave (0 at the wave's ends): one DPP move.
__device__ __forceinline__ float from_lane_below(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x138 /* wave_shr:1 */, 0xf, 0xf, true));
}
__device__ __forceinline__ float from_lane_above(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x130 /* wave_shl:1 */, 0xf, 0xf, true));
}

// acc + (value of x held by the previous / next lane) * w in one instruction: the multiply-add
// takes its first operand through the DPP lane shift (0 at the wave's ends).  The s_nop covers
// the two idle states a DPP read needs after a vector write of its operand, in case the
// compiler schedules such a write directly in front.
__device__ __forceinline__ float fma_lane_below(float x, float w, float acc) {
  asm("s_nop 1\n\tv_fmac_f32_dpp %0, %1, %2 wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(x), "v"(w));
  return acc;
}
__device__ __forceinline__ float fma_lane_above(float x, float w, float acc) {
  asm("s_nop 1\n\tv_fmac_f32_dpp %0, %1, %2 wave_shl:1 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(x), "v"(w));
  return acc;
}

// ---------------------------------------------------------------------------
// Buffer-addressed plane access.  A plane (one image channel) is described by a
// 128-bit buffer resource whose num_records is the plane's size in bytes; every
// access gives a 32-bit byte offset in a VGPR.  The hardware range-checks the
// offset: a load beyond num_records returns 0 and a store is dropped.  Taps that
// fall in the zero padding and lanes beyond the end of a plane are therefore
// expressed as the offset kOutOfRange, with no branch, exec masking or select,
// and no 64-bit address arithmetic is spent on the vector ALU.
// ---------------------------------------------------------------------------
constexpr unsigned kOutOfRange = 0x80000000u;
constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format (gfx9 family)

using rsrc_t = __amdgpu_buffer_rsrc_t;
// Cache policy of the result stores: non-temporal.  Results (an output or input-gradient tensor
// of the layer's size) are not read again by the operator, and written with the default policy
// they push the operands of the next kernel out of the 256 MB memory-side cache
// (measured: 6 % of a forward + backward step on a 245 MB layer).
constexpr int kStreamingStore = 2;  // "nt" bit of the buffer instruction's cache-policy field
// 2-byte stores keep the default policy: a wave's 2-byte stores cover half a cache line or less, and
// written non-temporally they reached memory as partial lines (WRITE_SIZE 47 % above the tensor's
// size on a 58 MB bfloat16 result; forward and grad input 4-6 % slower than with this policy).
constexpr int kMergedStore = 0;

template <typename T>
__device__ __forceinline__ rsrc_t plane_rsrc(const T* base, int elems) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(base), 0, elems * (int)sizeof(T), kRsrcFlags);
}

__device__ __forceinline__ float buf_ld(rsrc_t r, unsigned byte_off, const float*) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)byte_off, 0, 0));
}
__device__ __forceinline__ float buf_ld(rsrc_t r, unsigned byte_off, const __half*) {
  const unsigned short b = __builtin_amdgcn_raw_buffer_load_b16(r, (int)byte_off, 0, 0);
  return static_cast<float>(__builtin_bit_cast(_Float16, b));
}
__device__ __forceinline__ float buf_ld(rsrc_t r, unsigned byte_off, const bf16_t*) {
  const unsigned short b = __builtin_amdgcn_raw_buffer_load_b16(r, (int)byte_off, 0, 0);
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}
// Four consecutive elements at a byte offset of a buffer resource, as stored (converted when they are used: a
// conversion next to the load would wait for it).
typedef unsigned nhwc_u4 __attribute__((ext_vector_type(4)));
typedef unsigned nhwc_u2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ nhwc_u4 raw_ld4(rsrc_t r, unsigned off, const float*) { return __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0); }
__device__ __forceinline__ nhwc_u2 raw_ld4(rsrc_t r, unsigned off, const __half*) { return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0); }
__device__ __forceinline__ nhwc_u2 raw_ld4(rsrc_t r, unsigned off, const bf16_t*) { return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0); }
__device__ __forceinline__ void raw_cvt4(nhwc_u4 v, float (&f)[4], const float*) {
  const unsigned u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(u[i]);
}
__device__ __forceinline__ void raw_cvt4(nhwc_u2 v, float (&f)[4], const __half*) {
  const unsigned u[2] = {v.x, v.y};
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    f[2 * i] = static_cast<float>(__builtin_bit_cast(_Float16, (unsigned short)(u[i] & 0xffffu)));
    f[2 * i + 1] = static_cast<float>(__builtin_bit_cast(_Float16, (unsigned short)(u[i] >> 16)));
  }
}
__device__ __forceinline__ void raw_cvt4(nhwc_u2 v, float (&f)[4], const bf16_t*) {
  const unsigned u[2] = {v.x, v.y};
#pragma unroll
  for (int i = 0; i < 2; ++i) f[2 * i] = __uint_as_float(u[i] << 16), f[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
}

// The same with a scalar part of the address.  The range check compares the lane's offset with the buffer's
// size less the scalar part, so the descriptor must cover every position the scalar part selects.
__device__ __forceinline__ float buf_ld2(rsrc_t r, unsigned lane_off, int scalar_off, const float*) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)lane_off, scalar_off, 0));
}
__device__ __forceinline__ float buf_ld2(rsrc_t r, unsigned lane_off, int scalar_off, const __half*) {
  const unsigned short b = __builtin_amdgcn_raw_buffer_load_b16(r, (int)lane_off, scalar_off, 0);
  return static_cast<float>(__builtin_bit_cast(_Float16, b));
}
__device__ __forceinline__ float buf_ld2(rsrc_t r, unsigned lane_off, int scalar_off, const bf16_t*) {
  const unsigned short b = __builtin_amdgcn_raw_buffer_load_b16(r, (int)lane_off, scalar_off, 0);
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}
__device__ __forceinline__ void buf_st(rsrc_t r, unsigned byte_off, float v, float*) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, (int)byte_off, 0, kStreamingStore);
}
__device__ __forceinline__ void buf_st(rsrc_t r, unsigned byte_off, float v, __half*) {
  const _Float16 h = static_cast<_Float16>(v);
  __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, h), r, (int)byte_off, 0, kMergedStore);
}
__device__ __forceinline__ void buf_st(rsrc_t r, unsigned byte_off, float v, bf16_t*) {
  bf16_t t;
  st(&t, v);
  __builtin_amdgcn_raw_buffer_store_b16(t.bits, r, (int)byte_off, 0, kMergedStore);
}

// Two floats rounded to bfloat16 by one instruction (v_cvt_pk_bf16_f32), a in the lower half; and the two halves
// of such a pair back as floats.
__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
  typedef float f2 __attribute__((ext_vector_type(2)));
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(unsigned, __builtin_convertvector(f2{a, b}, b2));
}
__device__ __forceinline__ float bf16_lo(unsigned pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(unsigned pair) { return __uint_as_float(pair & 0xffff0000u); }

}  // namespace dk
