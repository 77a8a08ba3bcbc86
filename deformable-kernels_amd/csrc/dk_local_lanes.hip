// Local deformable kernel with the pixels on the lanes of the matrix instruction: forward and grad
// input (K.cu:270-386, 577-669; K.cu =
// deformable_kernels/ops/deform_kernel/csrc/filter_sample_depthwise_cuda_kernel.cu) for "same-width"
// geometries (3 x 3 taps, stride 1, unit column spacing, pad_w = 1) and scopes of at most 16 cells.
//
// The bilinear read of a channel's scope tile is a contraction over the tile's cells,
//   w_eff[c][(pixel, tap)] = sum_cell Wt[c][cell] * A[cell][(pixel, tap)],
//   A[cell = (i, j)][(p, t)] = hat(h_pt - i) * hat(w_pt - j)            (channel independent),
// and K.cu:51-83 writes the same sum corner by corner.  Here it is one v_mfma_f32_32x32x16 per tap
// with the CHANNELS on the rows and the PIXELS on the columns: the result leaves lane l holding
// pixel l % 32 of the tile and sixteen channels, which is exactly how a plain coalesced load of a
// channel plane hands a wave its data -- half a wave reads 32 consecutive pixels (128 bytes) of one
// plane -- so the source tensor goes from memory to registers to the multiply-add with no staging
// in LDS and no workgroup barrier in the loop.  The left / right taps take the neighbouring lane's
// element through the DPP shift folded into the multiply-add, so a tile is 30 pixels (columns
// 1..30) with a halo column at each end of the half wave.
//
// Split precision (fp32 tensors): A = Ah + Al, Wt * s = Wh + Wl in fp16 (s a power of two per
// channel), three products Wh Ah + Wh Al + Wl Ah with fp32 sums -- the dropped term is below
// 2^-22 of the channel's largest weight.  16-bit tensors: the filter is exact in the type, two products.
//
// A wave owns (image, tile of 30 pixels) and walks the blocks of 32 channels with the tile's A
// operands (72 registers) kept; the rows of the next block are requested while the current one is
// multiplied.  Taps whose source element lies outside the image have A = 0; their source loads are
// redirected out of range (rows above / below the plane) or read the element across the row's end
// (columns -1 / W), which is multiplied by that zero.
#include <algorithm>
#include <type_traits>

#include "dk_kernels.h"

namespace dk {

namespace {

constexpr int kLpThreads = 256;
constexpr int kLpWaves = kLpThreads / 64;
constexpr int kLpPix = 30;  // pixels a wave produces per tile: columns 1..30 of the 32
constexpr int kLpCh = 32;   // channels per block = rows of the matrix instruction

typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));

// The three taps of a source row: d = Wh Bh + Wh Bl (+ Wl Bh) for the left, right and centre tap, nine (six)
// v_mfma_f32_32x32x16 in one assembly statement.  Written out by hand because the multiply-adds that consume
// the results are partly inline assembly themselves (the lane shift folded into v_fmac), which the compiler's
// hazard handling does not look into: it would put no wait between a matrix instruction and such a reader.
// Here the order is fixed -- the three chains interleaved, so that an instruction never follows the one it
// accumulates onto -- and the s_nop after the last instruction covers the 11 wait states an 8-pass matrix
// result needs before a vector instruction may read it (the pipe completes in order, so that covers all
// three).  "=&v": a result never shares registers with an operand.
template <typename E> struct Lmx;
template <> struct Lmx<_Float16> {
  typedef _Float16 v8 __attribute__((ext_vector_type(8)));
  template <bool THIRD>
  static __device__ __forceinline__ void row(f16v& dl, f16v& dr, f16v& dc, v8 wh, v8 wl, v8 hl, v8 ll, v8 hr, v8 lr,
                                             v8 hc, v8 lc) {
    if constexpr (THIRD)
      asm volatile(
          "v_mfma_f32_32x32x16_f16 %0, %3, %5, 0\n\t"
          "v_mfma_f32_32x32x16_f16 %1, %3, %7, 0\n\t"
          "v_mfma_f32_32x32x16_f16 %2, %3, %9, 0\n\t"
          "v_mfma_f32_32x32x16_f16 %0, %3, %6, %0\n\t"
          "v_mfma_f32_32x32x16_f16 %1, %3, %8, %1\n\t"
          "v_mfma_f32_32x32x16_f16 %2, %3, %10, %2\n\t"
          "v_mfma_f32_32x32x16_f16 %0, %4, %5, %0\n\t"
          "v_mfma_f32_32x32x16_f16 %1, %4, %7, %1\n\t"
          "v_mfma_f32_32x32x16_f16 %2, %4, %9, %2\n\t"
          "s_nop 11"
          : "=&v"(dl), "=&v"(dr), "=&v"(dc)
          : "v"(wh), "v"(wl), "v"(hl), "v"(ll), "v"(hr), "v"(lr), "v"(hc), "v"(lc));
    else
      asm volatile(
          "v_mfma_f32_32x32x16_f16 %0, %3, %5, 0\n\t"
          "v_mfma_f32_32x32x16_f16 %1, %3, %7, 0\n\t"
          "v_mfma_f32_32x32x16_f16 %2, %3, %9, 0\n\t"
          "v_mfma_f32_32x32x16_f16 %0, %3, %6, %0\n\t"
          "v_mfma_f32_32x32x16_f16 %1, %3, %8, %1\n\t"
          "v_mfma_f32_32x32x16_f16 %2, %3, %10, %2\n\t"
          "s_nop 11"
          : "=&v"(dl), "=&v"(dr), "=&v"(dc)
          : "v"(wh), "v"(wl), "v"(hl), "v"(ll), "v"(hr), "v"(lr), "v"(hc), "v"(lc));
  }
};
template <> struct Lmx<__bf16> {
  typedef __bf16 v8 __attribute__((ext_vector_type(8)));
  template <bool THIRD>
  static __device__ __forceinline__ void row(f16v& dl, f16v& dr, f16v& dc, v8 wh, v8 wl, v8 hl, v8 ll, v8 hr, v8 lr,
                                             v8 hc, v8 lc) {
    static_assert(!THIRD, "bfloat16 tensors: the filter is exact in the type");
    asm volatile(
        "v_mfma_f32_32x32x16_bf16 %0, %3, %5, 0\n\t"
        "v_mfma_f32_32x32x16_bf16 %1, %3, %7, 0\n\t"
        "v_mfma_f32_32x32x16_bf16 %2, %3, %9, 0\n\t"
        "v_mfma_f32_32x32x16_bf16 %0, %3, %6, %0\n\t"
        "v_mfma_f32_32x32x16_bf16 %1, %3, %8, %1\n\t"
        "v_mfma_f32_32x32x16_bf16 %2, %3, %10, %2\n\t"
        "s_nop 11"
        : "=&v"(dl), "=&v"(dr), "=&v"(dc)
        : "v"(wh), "v"(wl), "v"(hl), "v"(ll), "v"(hr), "v"(lr), "v"(hc), "v"(lc));
  }
};
template <typename T> struct LmxOf { using type = _Float16; };  // float, __half
template <> struct LmxOf<bf16_t> { using type = __bf16; };

// Eight products a[k] * b[k] as fp16 pairs: hi = fp16(a b) with one rounding of the exact product, lo = fp16(a b - hi)
// with the exact product again (v_fma_mix: fp32 factors, fp16 addend and result), two instructions per value where
// multiply, convert, convert back, subtract, convert take four.  The instructions that write one half of a register
// are kept two instructions away from the reader of that register (a half-register write needs one).
__device__ __forceinline__ void lp_split_products(const float (&a)[8], const float (&b)[8], uint4& hi, uint4& lo) {
#define DK_PAIR(H, L, K)                                                                                      \
  asm("v_fma_mixlo_f16 %0, %2, %3, 0\n\t"                                                                     \
      "v_fma_mixhi_f16 %0, %4, %5, 0\n\t"                                                                     \
      "s_nop 0\n\t"                                                                                           \
      "v_fma_mixlo_f16 %1, %2, %3, -%0 op_sel_hi:[0,0,1]\n\t"                                                 \
      "v_fma_mixhi_f16 %1, %4, %5, -%0 op_sel:[0,0,1] op_sel_hi:[0,0,1]\n\t"                                  \
      "s_nop 0"                                                                                               \
      : "=&v"(H), "=&v"(L)                                                                                    \
      : "v"(a[K]), "v"(b[K]), "v"(a[K + 1]), "v"(b[K + 1]))
  DK_PAIR(hi.x, lo.x, 0);
  DK_PAIR(hi.y, lo.y, 2);
  DK_PAIR(hi.z, lo.z, 4);
  DK_PAIR(hi.w, lo.w, 6);
#undef DK_PAIR
}

__device__ __forceinline__ float lp_hat(float d) { return __builtin_amdgcn_fmed3f(1.f - fabsf(d), 0.f, 1.f); }

// acc + (x of the previous / next lane) * w, the lane shift folded into the multiply-add.  No wait
// states in front: x comes from a load or from a conversion that is at least two instructions old.
__device__ __forceinline__ float lp_fma_below(float x, float w, float acc) {
  asm("v_fmac_f32_dpp %0, %1, %2 wave_shr:1 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(x), "v"(w));
  return acc;
}
__device__ __forceinline__ float lp_fma_above(float x, float w, float acc) {
  asm("v_fmac_f32_dpp %0, %1, %2 wave_shl:1 row_mask:0xf bank_mask:0xf bound_ctrl:1" : "+v"(acc) : "v"(x), "v"(w));
  return acc;
}

// Vector-memory operations of the kernel's loop, all from inline assembly: the compiler then neither reorders them
// nor places waits of its own for them (its counting is per loop, and it waited for a whole block's rows where
// the first was needed), and the loop below writes the waits out itself.  A 2-byte load leaves the element
// zero-extended in its register.
typedef unsigned lp_u4 __attribute__((ext_vector_type(4)));
template <typename T>
__device__ __forceinline__ lp_u4 lp_resource(const T* base, int bytes) {
  const unsigned long a = reinterpret_cast<unsigned long>(base);
  return lp_u4{(unsigned)a, (unsigned)(a >> 32) & 0xffffu, (unsigned)bytes, (unsigned)kRsrcFlags};
}
// A group of loads or stores is ONE assembly statement that starts with s_nop 4: an SGPR written by a vector
// instruction (v_readfirstlane, the v_readlane of a spilled SGPR) may be read by a vector-memory instruction
// only five wait states later, the compiler's hazard handling does not look into inline assembly, and it does
// place such writes directly in front of (or between) single-instruction statements.  
// Eight elements of a source row / eight results, each with its own scalar offset (the channel's offset from the
// lane's first channel: constants of the launch, kept in SGPRs, so that a block costs no scalar arithmetic for
// its 64 addresses; the block's own offset is part of the lane offset).
template <int SIZE>
__device__ __forceinline__ void lp_load8(unsigned* x, lp_u4 r, unsigned lane_off, const int* so) {
#define DK_IO8 "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3]), "=&v"(x[4]), "=&v"(x[5]), "=&v"(x[6]), "=&v"(x[7])             \
    : "v"(lane_off), "s"(r), "s"(so[0]), "s"(so[1]), "s"(so[2]), "s"(so[3]), "s"(so[4]), "s"(so[5]), "s"(so[6]), "s"(so[7])
  if constexpr (SIZE == 4)
    asm volatile(
        "s_nop 4\n\t"
        "buffer_load_dword %0, %8, %9, %10 offen\n\t"
        "buffer_load_dword %1, %8, %9, %11 offen\n\t"
        "buffer_load_dword %2, %8, %9, %12 offen\n\t"
        "buffer_load_dword %3, %8, %9, %13 offen\n\t"
        "buffer_load_dword %4, %8, %9, %14 offen\n\t"
        "buffer_load_dword %5, %8, %9, %15 offen\n\t"
        "buffer_load_dword %6, %8, %9, %16 offen\n\t"
        "buffer_load_dword %7, %8, %9, %17 offen"
        : DK_IO8);
  else
    asm volatile(
        "s_nop 4\n\t"
        "buffer_load_ushort %0, %8, %9, %10 offen\n\t"
        "buffer_load_ushort %1, %8, %9, %11 offen\n\t"
        "buffer_load_ushort %2, %8, %9, %12 offen\n\t"
        "buffer_load_ushort %3, %8, %9, %13 offen\n\t"
        "buffer_load_ushort %4, %8, %9, %14 offen\n\t"
        "buffer_load_ushort %5, %8, %9, %15 offen\n\t"
        "buffer_load_ushort %6, %8, %9, %16 offen\n\t"
        "buffer_load_ushort %7, %8, %9, %17 offen"
        : DK_IO8);
#undef DK_IO8
}
template <int SIZE>
__device__ __forceinline__ void lp_store8(const unsigned* v, lp_u4 r, unsigned lane_off, const int* so) {
#define DK_IO8 "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]), "v"(lane_off), "s"(r),     \
    "s"(so[0]), "s"(so[1]), "s"(so[2]), "s"(so[3]), "s"(so[4]), "s"(so[5]), "s"(so[6]), "s"(so[7])
  if constexpr (SIZE == 4)
    asm volatile(
        "s_nop 4\n\t"
        "buffer_store_dword %0, %8, %9, %10 offen\n\t"
        "buffer_store_dword %1, %8, %9, %11 offen\n\t"
        "buffer_store_dword %2, %8, %9, %12 offen\n\t"
        "buffer_store_dword %3, %8, %9, %13 offen\n\t"
        "buffer_store_dword %4, %8, %9, %14 offen\n\t"
        "buffer_store_dword %5, %8, %9, %15 offen\n\t"
        "buffer_store_dword %6, %8, %9, %16 offen\n\t"
        "buffer_store_dword %7, %8, %9, %17 offen"
        :
        : DK_IO8
        : "memory");
  else
    asm volatile(
        "s_nop 4\n\t"
        "buffer_store_short %0, %8, %9, %10 offen\n\t"
        "buffer_store_short %1, %8, %9, %11 offen\n\t"
        "buffer_store_short %2, %8, %9, %12 offen\n\t"
        "buffer_store_short %3, %8, %9, %13 offen\n\t"
        "buffer_store_short %4, %8, %9, %14 offen\n\t"
        "buffer_store_short %5, %8, %9, %15 offen\n\t"
        "buffer_store_short %6, %8, %9, %16 offen\n\t"
        "buffer_store_short %7, %8, %9, %17 offen"
        :
        : DK_IO8
        : "memory");
#undef DK_IO8
}
// Nine values with a lane offset each (the rotation values of one direction), from scalar offset `soff`.
template <int SIZE>
__device__ __forceinline__ void lp_load9(unsigned (&x)[9], lp_u4 r, const unsigned (&lane_off)[9], int soff) {
#define DK_IO9 "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3]), "=&v"(x[4]), "=&v"(x[5]), "=&v"(x[6]), "=&v"(x[7]), "=&v"(x[8]) \
    : "v"(lane_off[0]), "v"(lane_off[1]), "v"(lane_off[2]), "v"(lane_off[3]), "v"(lane_off[4]), "v"(lane_off[5]),                 \
      "v"(lane_off[6]), "v"(lane_off[7]), "v"(lane_off[8]), "s"(r), "s"(soff)
  if constexpr (SIZE == 4)
    asm volatile(
        "s_nop 4\n\t"
        "buffer_load_dword %0, %9, %18, %19 offen\n\t"
        "buffer_load_dword %1, %10, %18, %19 offen\n\t"
        "buffer_load_dword %2, %11, %18, %19 offen\n\t"
        "buffer_load_dword %3, %12, %18, %19 offen\n\t"
        "buffer_load_dword %4, %13, %18, %19 offen\n\t"
        "buffer_load_dword %5, %14, %18, %19 offen\n\t"
        "buffer_load_dword %6, %15, %18, %19 offen\n\t"
        "buffer_load_dword %7, %16, %18, %19 offen\n\t"
        "buffer_load_dword %8, %17, %18, %19 offen"
        : DK_IO9);
  else
    asm volatile(
        "s_nop 4\n\t"
        "buffer_load_ushort %0, %9, %18, %19 offen\n\t"
        "buffer_load_ushort %1, %10, %18, %19 offen\n\t"
        "buffer_load_ushort %2, %11, %18, %19 offen\n\t"
        "buffer_load_ushort %3, %12, %18, %19 offen\n\t"
        "buffer_load_ushort %4, %13, %18, %19 offen\n\t"
        "buffer_load_ushort %5, %14, %18, %19 offen\n\t"
        "buffer_load_ushort %6, %15, %18, %19 offen\n\t"
        "buffer_load_ushort %7, %16, %18, %19 offen\n\t"
        "buffer_load_ushort %8, %17, %18, %19 offen"
        : DK_IO9);
#undef DK_IO9
}
__device__ __forceinline__ float lp_value(unsigned bits, const float*) { return __uint_as_float(bits); }
// (16-bit elements are converted by volatile assembly statements: an ordinary conversion could be moved in front
// of the wait for the load)
__device__ __forceinline__ float lp_value(unsigned bits, const bf16_t*) {
  float v;
  asm volatile("v_lshlrev_b32 %0, 16, %1" : "=v"(v) : "v"(bits));
  return v;
}
__device__ __forceinline__ float lp_value(unsigned bits, const __half*) {
  float v;
  asm volatile("v_cvt_f32_f16 %0, %1" : "=v"(v) : "v"(bits));
  return v;
}
// A result as the bits its store writes.
__device__ __forceinline__ unsigned lp_bits(float v, float*) { return __float_as_uint(v); }
__device__ __forceinline__ unsigned lp_bits(float v, __half*) { return __builtin_bit_cast(unsigned short, static_cast<_Float16>(v)); }
__device__ __forceinline__ unsigned lp_bits(float v, bf16_t*) {
  bf16_t t;
  st(&t, v);
  return t.bits;
}
// Wait until at most N of the wave's vector-memory operations are outstanding.  Assembly statements marked
// volatile keep their order, so what follows a wait there -- the matrix instructions of a row and, through their
// results, the row's multiply-adds -- stays behind it; where ordinary arithmetic reads the loaded registers
// (the rotation values) they are in/out operands of the wait, which keeps those readers behind it as well.
template <int N>
__device__ __forceinline__ void lp_wait() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N));
}
template <int N>
__device__ __forceinline__ void lp_wait(unsigned (&a)[9], unsigned (&b)[9]) {
  asm volatile("s_waitcnt vmcnt(%18)"
               : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]), "+v"(a[8]),
                 "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]), "+v"(b[5]), "+v"(b[6]), "+v"(b[7]), "+v"(b[8])
               : "n"(N));
}

template <typename T, int SH, int SW, bool TRANSPOSED, bool CLIP>
__global__ __launch_bounds__(kLpThreads, 2) void local_pixel_lanes_kernel(
    Geo g, const T* __restrict__ src, const T* __restrict__ rot, const T* __restrict__ filter,
    T* __restrict__ dst, int tiles, int nwg) {
  using E = typename LmxOf<T>::type;
  using M = Lmx<E>;
  using v8 = typename M::v8;
  constexpr bool kThird = sizeof(T) == 4;  // fp32 tensors: the filter has a low part
  constexpr bool kBf = std::is_same<E, __bf16>::value;
  constexpr int K = 9, CELLS = SH * SW;
  static_assert(CELLS <= 16, "one K = 16 block of cells");
  extern __shared__ __align__(16) unsigned dyn[];

  const int cpg = g.channel / g.groups;
  const int nblk = ceil_div(cpg, kLpCh);
  // [nblk][64] lanes x {Wh (16 bytes), Wl (16 bytes)}: lane l of the A side stands for channel l % 32 of the
  // block and cells 8 (l / 32) .. + 7; then [nblk][32] floats 1 / s
  uint4* wtab = reinterpret_cast<uint4*>(dyn);
  float* unscale = reinterpret_cast<float*>(wtab + nblk * 128);

  const int total = nwg * g.groups;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int wg = lb % nwg, grp = lb / nwg;

  const int W = g.in_w;  // == out_w
  const int out_plane = g.out_h * W, in_plane = g.in_h * W;
  const int dst_plane = TRANSPOSED ? in_plane : out_plane, src_plane = TRANSPOSED ? out_plane : in_plane;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 31, hf = lane >> 5;

  // ---- per workgroup: the split filter operands of every channel block
  for (int e = threadIdx.x; e < nblk * 64; e += kLpThreads) {
    const int b = e >> 6, l = e & 63, cj = b * kLpCh + (l & 31), c0 = 8 * (l >> 5);
    float v[8], s = 1.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = 0.f;
    if (cj < cpg) {
      const T* f = filter + (size_t)(grp + g.groups * cj) * CELLS;
      if constexpr (kThird) {
        float m = 0.f;
#pragma unroll
        for (int k = 0; k < CELLS; ++k) m = fmaxf(m, fabsf(ld(f + k)));
        int ex = 0;
        if (m > 0.f && m < __builtin_inff()) (void)frexpf(m, &ex);  // m = fraction * 2^ex, fraction in [0.5, 1)
        ex = min(max(ex, -100), 100);
        s = ldexpf(1.f, -ex);
        if ((l >> 5) == 0) unscale[b * kLpCh + (l & 31)] = ldexpf(1.f, ex);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (c0 + k < CELLS) v[k] = ld(f + c0 + k) * s;
    } else if constexpr (kThird) {
      if ((l >> 5) == 0) unscale[b * kLpCh + (l & 31)] = 0.f;
    }
    v8 h, lw;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      float vk = v[k];
      asm volatile("" : "+v"(vk));  // one fp32 value for both parts (no contraction into the conversions)
      const E a = static_cast<E>(vk);
      h[k] = a;
      lw[k] = static_cast<E>(vk - static_cast<float>(a));
    }
    wtab[2 * e] = __builtin_bit_cast(uint4, h);
    wtab[2 * e + 1] = __builtin_bit_cast(uint4, lw);
  }
  __syncthreads();  // the only workgroup barrier: from here on the waves run on their own

  // ---- this wave's share of the work, as segments (item, range of channel blocks).  Items are (image, tile)
  // pairs; whole rounds of items go round-robin over the wave slots (item i to slot i % slots: neighbouring
  // slots -- the waves of one workgroup, the workgroups of one XCD -- hold neighbouring tiles at the same
  // time, so the rows that vertically adjacent tiles share are fetched from memory once), and the (item,
  // channel block) units of the last, incomplete round are dealt as contiguous ranges cut at the tile boundaries.
  const int slot = wg * kLpWaves + wave, slots = nwg * kLpWaves, items = g.batch * tiles;
  const int whole = items / slots;
  const long rest_units = (long)(items - whole * slots) * nblk;
  const long r_lo = rest_units * slot / slots, r_hi = rest_units * (slot + 1) / slots;
  const int rest_lo = (int)(r_lo / nblk), rest_hi = r_hi > r_lo ? (int)((r_hi - 1) / nblk) : rest_lo - 1;
  const int cb_first = (int)(r_lo % nblk), cb_last = r_hi > r_lo ? (int)((r_hi - 1) % nblk) + 1 : 0;
  const int nseg = whole + (rest_hi - rest_lo + 1);
  if (nseg <= 0) return;
  auto segment = [&](int k, int& item, int& cb_begin, int& cb_end) {
    const int t = rest_lo + (k - whole);
    const bool round_robin = k < whole;
    item = round_robin ? slot + k * slots : whole * slots + t;
    cb_begin = (!round_robin && t == rest_lo) ? cb_first : 0;
    cb_end = (!round_robin && t == rest_hi) ? cb_last : nblk;
  };

  // bytes between two channels of the group; a lane's first channel of a block is 4 hf (the result
  // register r holds row 8 (r / 4) + 4 hf + r % 4)
  const int src_ch = g.groups * src_plane * (int)sizeof(T), dst_ch = g.groups * dst_plane * (int)sizeof(T);
  const unsigned w_magic = (unsigned)(0x100000000ull / (unsigned)W) + 1u;  // floor(p / W) = (p * magic) >> 32 for p < 2^24

  // What a lane knows of a tile: its pixel's offsets into the three source rows and into the result plane.
  struct Tile {
    int n, p0;
    unsigned row[3], out;
  };
  auto make_tile = [&](int item) {
    Tile t;
    t.n = item / tiles;
    t.p0 = (item - t.n * tiles) * kLpPix;
    const int p = t.p0 - 1 + col;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      const int dr = TRANSPOSED ? g.pad_h - r * g.dil_h : r * g.dil_h - g.pad_h;
      const int e = p + dr * W;
      t.row[r] = (e >= 0 && e < src_plane) ? (unsigned)(4 * hf * src_ch) + (unsigned)e * (unsigned)sizeof(T) : kOutOfRange;
    }
    const bool owns = col >= 1 && col <= kLpPix && p < dst_plane;
    t.out = owns ? (unsigned)(4 * hf * dst_ch) + (unsigned)p * (unsigned)sizeof(T) : kOutOfRange;
    return t;
  };
  // an image's channels of this group (the range check drops what a block holds beyond the group's last channel)
  auto src_rsrc = [&](int n) {
    return lp_resource(src + (size_t)(n * g.channel + grp) * src_plane, ((cpg - 1) * g.groups + 1) * src_plane * (int)sizeof(T));
  };
  auto dst_rsrc = [&](int n) {
    return lp_resource(dst + (size_t)(n * g.channel + grp) * dst_plane, ((cpg - 1) * g.groups + 1) * dst_plane * (int)sizeof(T));
  };

  // The nine taps of the lane's pixel: which contribute (forward: the tap's input element lies in the image,
  // K.cu:321-336; grad input: output pixel q + pad - f dil, which feeds input pixel q through tap t, exists,
  // K.cu:611-651) and the pixel whose rotation they use.
  auto tap_pixels = [&](const Tile& tl, bool (&ok)[K], int (&o)[K]) {
    const int p = tl.p0 - 1 + col;
    const bool live = p >= 0 && p < dst_plane;
    const int pc = live ? p : 0;
    const int ph = (int)__umulhi((unsigned)pc, w_magic), pw = pc - ph * W;
#pragma unroll
    for (int t = 0; t < K; ++t) {
      const int f_h = t / 3, f_w = t % 3;
      const int qh = TRANSPOSED ? ph + g.pad_h - f_h * g.dil_h : ph + f_h * g.dil_h - g.pad_h;
      const int qw = TRANSPOSED ? pw + 1 - f_w : pw + f_w - 1;
      ok[t] = live && qw >= 0 && qw < W && qh >= 0 && qh < (TRANSPOSED ? g.out_h : g.in_h);
      o[t] = TRANSPOSED ? qh * W + qw : pc;
    }
  };
  // The rotation values of a tile, requested one block ahead of the tile's first (18 registers in flight).
  unsigned rh[K], rw[K];
  auto load_rotation = [&](const Tile& tl) {
    bool ok[K];
    int o[K];
    tap_pixels(tl, ok, o);
    const lp_u4 rr = lp_resource(rot + (size_t)(tl.n * g.groups + grp) * (K * 2) * out_plane, K * 2 * out_plane * (int)sizeof(T));
    unsigned ro[K];
#pragma unroll
    for (int t = 0; t < K; ++t) ro[t] = ok[t] ? (unsigned)((2 * t) * out_plane + o[t]) * (unsigned)sizeof(T) : kOutOfRange;
    lp_load9<sizeof(T)>(rh, rr, ro, 0);
    lp_load9<sizeof(T)>(rw, rr, ro, out_plane * (int)sizeof(T));
  };
  // The A operands of a tile: lane (column = pixel, hf) holds cells 8 hf .. 8 hf + 7 of its pixel's nine taps.
  // The band test of K.cu:59 is the hats' own: outside (-1, S) every hat(h - i), i = 0 .. S - 1, is 0; a tap that
  // does not contribute gets h = -2.
  v8 Bh[K], Bl[K];
  auto derive_operands = [&](const Tile& tl) {
    bool ok[K];
    int o[K];
    tap_pixels(tl, ok, o);
#pragma unroll
    for (int t = 0; t < K; ++t) {
      float h, w;
      if constexpr (CLIP) {
        h = scope_coord<float>(g, t / 3, lp_value(rh[t], rot), g.centre_h);
        w = scope_coord<float>(g, t % 3, lp_value(rw[t], rot), g.centre_w);
      } else {
        h = scope_coord<float>(t / 3, lp_value(rh[t], rot), g.centre_h);
        w = scope_coord<float>(t % 3, lp_value(rw[t], rot), g.centre_w);
      }
      const float hh = ok[t] ? h : -2.f;
      float ra[8], cb[8];  // the row and the column hat of each of the lane's cells
      if constexpr (SW == 4) {
        // cells 8 hf + k = (row 2 hf + k / 4, column k % 4)
        const float a0 = lp_hat(hh - float(2 * hf)), a1 = lp_hat(hh - float(2 * hf + 1));
        float b[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = lp_hat(w - float(j));
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          ra[k] = k < 4 ? a0 : a1;
          cb[k] = b[k & 3];
        }
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const int cell = 8 * hf + k;
          ra[k] = cell < CELLS ? lp_hat(hh - float(cell / SW)) : 0.f;
          cb[k] = lp_hat(w - float(cell % SW));
        }
      }
      if constexpr (sizeof(E) == 2 && !kBf) {
        uint4 hi, lo;
        lp_split_products(ra, cb, hi, lo);
        Bh[t] = __builtin_bit_cast(v8, hi);
        Bl[t] = __builtin_bit_cast(v8, lo);
      } else {
        typedef float f2v __attribute__((ext_vector_type(2)));
        typedef E e2v __attribute__((ext_vector_type(2)));
        v8 hi, lo;
#pragma unroll
        for (int k = 0; k < 8; k += 2) {
          float v0 = ra[k] * cb[k], v1 = ra[k + 1] * cb[k + 1];
          asm volatile("" : "+v"(v0), "+v"(v1));  // one fp32 value for both parts
          const e2v h2 = __builtin_convertvector(f2v{v0, v1}, e2v);
          const f2v b2 = __builtin_convertvector(h2, f2v);
          const e2v l2 = __builtin_convertvector(f2v{v0 - b2[0], v1 - b2[1]}, e2v);
          hi[k] = h2[0];
          hi[k + 1] = h2[1];
          lo[k] = l2[0];
          lo[k + 1] = l2[1];
        }
        Bh[t] = hi;
        Bl[t] = lo;
      }
    }
  };

  unsigned xs[3][16];
  // scalar offset of result register r's channel from the lane's first: channel 8 (r / 4) + r % 4
  int so_src[16], so_dst[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    so_src[r] = (8 * (r >> 2) + (r & 3)) * src_ch;
    so_dst[r] = (8 * (r >> 2) + (r & 3)) * dst_ch;
  }
  auto load_row = [&](unsigned (&x)[16], lp_u4 rs, unsigned voff, int cb) {
    const unsigned at = voff + (unsigned)(cb * kLpCh * src_ch);  // a row outside the plane stays beyond the range: the block's offset is below 2^31
    lp_load8<sizeof(T)>(x, rs, at, so_src);
    lp_load8<sizeof(T)>(x + 8, rs, at, so_src + 8);
  };

  // ---- the walk.  Vector-memory operations in program order, per block u: [in a tile's last block, after the
  // wait for row 0: the rotation values of the next tile, R = 18 loads], then per source row r = 0, 1, 2 the 16
  // loads L_r(u + 1) of the NEXT block's row, issued right after row r of this block has been used, then the 16
  // result stores S(u).  Loads complete in order, so "row r of block u has landed" is "at most the loads issued
  // after L_r(u) are outstanding": L_{r+1} and L_{r+2}, 32 operations.  The stores in between are not counted on:
  // a store that completes late only makes the wait longer, one that completes early must not make it shorter.
  // The last block of all has no loads behind its rows and waits for everything.  The counter holds 63: a
  // tile's last block waits for 29 before it adds the 18 rotation loads (then 16 row loads), and every block
  // for 47 before its 16 stores.
  // One flat loop over the blocks, with the tile's set-up in a branch: registers with a load in flight must not
  // be copied before the wait for them, and values carried through nested loops invite such copies.
  int seg = 0, item, cb, cb_end;
  segment(0, item, cb, cb_end);
  Tile cur = make_tile(__builtin_amdgcn_readfirstlane(item)), nxt = cur;
  lp_u4 rs_cur = src_rsrc(cur.n), rs_nxt = rs_cur, rd = rs_cur;
  int n_cb = 0, n_cb_end = 0;
  bool more = false;
  load_rotation(cur);
  load_row(xs[0], rs_cur, cur.row[0], cb);
  load_row(xs[1], rs_cur, cur.row[1], cb);
  bool first = true;  // the wave's first tile
  bool fresh = true;  // the coming block is the first of its tile

  while (true) {
    if (fresh) {
      // the rotation values: behind them two rows of the first block (the wave's first tile) or three
      lp_wait<32>(rh, rw);
      derive_operands(cur);
      if (first) {
        load_row(xs[2], rs_cur, cur.row[2], cb);
        first = false;
      }
      // the tile after this one (if any), whose first rows are requested during this tile's last block
      int n_item = 0;
      n_cb = n_cb_end = 0;
      more = seg + 1 < nseg;
      if (more) segment(seg + 1, n_item, n_cb, n_cb_end);
      n_item = __builtin_amdgcn_readfirstlane(n_item);
      n_cb = __builtin_amdgcn_readfirstlane(n_cb);
      n_cb_end = __builtin_amdgcn_readfirstlane(n_cb_end);
      nxt = make_tile(n_item);
      rs_nxt = src_rsrc(nxt.n);
      rd = dst_rsrc(cur.n);
    }
    const bool last = cb + 1 == cb_end;
    // the next block's rows: the same tile's next block, or the next tile's first
    const bool any_next = !last || more;
    const int cb_n = last ? n_cb : cb + 1;
    const uint4 whb = wtab[2 * (cb * 64 + lane)], wlb = wtab[2 * (cb * 64 + lane) + 1];
    const v8 wh = __builtin_bit_cast(v8, whb), wl = __builtin_bit_cast(v8, wlb);
    float acc[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int rr = 0; rr < 3; ++rr) {
      if (!any_next) {
        lp_wait<0>();
      } else if (rr == 0 && last) {
        lp_wait<29>();
        load_rotation(nxt);  // in flight through this tile's last block
      } else {
        lp_wait<32>();
      }
      // the taps of source columns -1, 0, +1 of this row
      // (forward: tap f_w reads column f_w - 1; grad input: output column 1 - f_w feeds the pixel through tap f_w)
      const int tl = TRANSPOSED ? rr * 3 + 2 : rr * 3, tc = rr * 3 + 1, tr = TRANSPOSED ? rr * 3 : rr * 3 + 2;
      f16v dl, dr, dc;
      M::template row<kThird>(dl, dr, dc, wh, wl, Bh[tl], Bl[tl], Bh[tr], Bl[tr], Bh[tc], Bl[tc]);
      float xv[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) xv[r] = lp_value(xs[rr][r], src);
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = fmaf(xv[r], dc[r], acc[r]);
      if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = lp_fma_below(xv[r], dl[r], acc[r]);
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = lp_fma_above(xv[r], dr[r], acc[r]);
      } else {
        // the element was converted by a vector instruction, which a lane-shifted read must follow at a distance
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = fma_lane_below(xv[r], dl[r], acc[r]);
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = fma_lane_above(xv[r], dr[r], acc[r]);
      }
      if (any_next) load_row(xs[rr], last ? rs_nxt : rs_cur, last ? nxt.row[rr] : cur.row[rr], cb_n);
    }
    if constexpr (kThird) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const f4v us = *reinterpret_cast<const f4v*>(unscale + cb * kLpCh + 8 * i + 4 * hf);
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[4 * i + k] *= us[k];
      }
    }
    unsigned res[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) res[r] = lp_bits(acc[r], dst);
    lp_wait<47>();
    {
      const unsigned at = cur.out + (unsigned)(cb * kLpCh * dst_ch);
      lp_store8<sizeof(T)>(res, rd, at, so_dst);
      lp_store8<sizeof(T)>(res + 8, rd, at, so_dst + 8);
    }
    fresh = last;
    if (last) {
      if (!more) break;
      ++seg;
      cur = nxt;
      rs_cur = rs_nxt;
      cb = n_cb;
      cb_end = n_cb_end;
    } else {
      ++cb;
    }
  }
}

struct LanesPlan {
  bool ok;
  int tiles, nwg;
  size_t lds;
};

LanesPlan lanes_plan(const Geo& g, bool transposed, int esize) {
  LanesPlan p{};
  const bool same_width = g.stride_h == 1 && g.stride_w == 1 && g.dil_w == 1 && g.pad_w == 1 && g.k_h == 3 &&
                          g.k_w == 3 && g.in_w == g.out_w;
  if (!same_width || g.scope_h * g.scope_w > 16 || g.in_w < 2 || path_disabled(kNoPixelLanes)) return p;  // in_w >= 2: the division by the width is a multiplication
  const int cpg = g.channel / g.groups, nblk = ceil_div(cpg, kLpCh);
  const long plane = std::max((long)g.in_h * g.in_w, (long)g.out_h * g.out_w);
  // byte offsets inside an image's channels of one group (lane part + scalar part) stay below 2^31
  if ((long)(nblk * kLpCh + 8) * g.groups * plane * esize >= (1L << 31)) return p;
  const long dplane = transposed ? (long)g.in_h * g.in_w : (long)g.out_h * g.out_w;
  p.tiles = (int)((dplane + kLpPix - 1) / kLpPix);
  const long items = (long)g.batch * p.tiles;
  if (items * nblk >= (1L << 30)) return p;
  p.lds = (size_t)nblk * 64 * 32 + (size_t)nblk * kLpCh * 4;
  if (p.lds > 64 * 1024) return p;
  // two workgroups per CU, all resident; fewer where there is less work than that (at least two units per wave)
  const long want = std::max(1L, (items * nblk / 2 + kLpWaves - 1) / kLpWaves);
  p.nwg = (int)std::min(want, (long)std::max(1, 2 * 256 / g.groups));
  p.ok = true;
  return p;
}

template <typename T, int SH, int SW>
bool run_pixel_lanes(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                     hipStream_t stream) {
  const LanesPlan p = lanes_plan(g, transposed, (int)sizeof(T));
  if (!p.ok) return false;
  const unsigned grid = (unsigned)xcd_grid_size((long)p.nwg * g.groups);
#define DK_LAUNCH(TR, CL) \
  local_pixel_lanes_kernel<T, SH, SW, TR, CL><<<grid, kLpThreads, p.lds, stream>>>(g, src, rot, filter, dst, p.tiles, p.nwg)
  const bool clip = g.clip_mode != kClipNone;
  if (transposed) {
    if (clip) DK_LAUNCH(true, true); else DK_LAUNCH(true, false);
  } else {
    if (clip) DK_LAUNCH(false, true); else DK_LAUNCH(false, false);
  }
#undef DK_LAUNCH
  return true;
}

}  // namespace

template <typename T>
bool lanes_local_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                        hipStream_t stream) {
  if (g.k_h != 3 || g.k_w != 3) return false;
  if ((long)g.in_h * g.in_w >= (1L << 24) || (long)g.out_h * g.out_w >= (1L << 24)) return false;  // byte offsets of 18 rotation planes in 31 bits
  if (!path_disabled(kForcePixelLanes)) {
    // A tile's set-up (18 rotation loads, 72 operand registers) is paid once per tile and wave and a block is 32
    // channels: the kernel is for large planes with many channels.  Measured on N=64 C=144 56 x 56, against the
    // kernel that stages its tiles in LDS (dk_local_mfma.hip): called in a loop of its own, where the 256 MB
    // memory-side cache holds most of the 245 MB it touches, it is the faster one for float32 (60 against 63.4 us)
    // and bfloat16 (55 / 57) and level for float16 (54.7 / 53.8); inside a forward + backward step, where the
    // operands come from HBM, its two waves per SIMD with one block of loads in flight hide less of the latency
    // than four waves with two staged tiles do -- float32 step 0.3165 against 0.3005 ms, bfloat16 0.2476
    // against 0.2529 ms.  So on large planes the dispatch takes it for bfloat16 tensors only.  On planes of fewer
    // than 2048 pixels (the 28 x 28, 14 x 14 and 7 x 7 stages of MobileNetV2-DK, 128 to 960 channels) its small
    // per-tile set-up makes it the faster kernel for both 16-bit types -- forward, batch 64 / 128: 28 x 28 C=192
    // 22.8 against 29.4 us / 38.2 against 44.5, 14 x 14 C=576 20.7 against 26.1, 7 x 7 C=960 14.2 against 16.2 /
    // 19.7 against 29.5, the layer's forward + backward step 4 to 16 % shorter -- while float32 gains on two of
    // those shapes (1.6 and 4 % of the step) and loses on the others, and stays where it was.
    const long plane = (long)g.out_h * g.out_w;
    const int cpg = g.channel / g.groups;
    const bool large = plane >= 2048;
    if (cpg < 96 || sizeof(T) == 4 || (large && !std::is_same<T, bf16_t>::value)) return false;
  }
  if (g.scope_h == 4 && g.scope_w == 4) return run_pixel_lanes<T, 4, 4>(g, transposed, src, rot, filter, dst, stream);
  if (g.scope_h == 3 && g.scope_w == 3) return run_pixel_lanes<T, 3, 3>(g, transposed, src, rot, filter, dst, stream);
  return false;
}

template bool lanes_local_gather<float>(const Geo&, bool, const float*, const float*, const float*, float*, hipStream_t);
template bool lanes_local_gather<__half>(const Geo&, bool, const __half*, const __half*, const __half*, __half*, hipStream_t);
template bool lanes_local_gather<bf16_t>(const Geo&, bool, const bf16_t*, const bf16_t*, const bf16_t*, bf16_t*, hipStream_t);

}  // namespace dk
