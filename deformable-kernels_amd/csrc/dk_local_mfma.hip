// Local deformable kernel on the matrix cores, for "same-width" geometries (3 x 3 taps, stride 1,
// unit column spacing, pad_w = 1: input and output planes share their width) and scopes of at
// most 16 cells: forward and grad input (K.cu:270-386, 577-669; K.cu =
// deformable_kernels/ops/deform_kernel/csrc/filter_sample_depthwise_cuda_kernel.cu).
//
// The bilinear read of a channel's scope tile is a dense contraction over the tile's cells,
//   w_eff[(pixel, tap)][c] = sum_cell A[(pixel, tap)][cell] * Wt[cell][c],
//   A[(p, t)][cell = (i, j)] = hat(h_pt - i) * hat(w_pt - j)          (channel independent),
// with at most four non-zero A per row (K.cu:51-83 writes the same sum corner by corner).  On
// the vector ALU the sparse form wins (three FMAs per weight from a 16-byte LDS table gather), but
// those gathers and FMAs are what bounds the gather kernels of dk_local_fast.hip -- LDS pipe and
// VALU issue both sit at the HBM time -- while the matrix pipe idles.  16-bit matrix instructions
// run beside VALU work of other waves (measured: a v_mfma_f32_16x16x32_f16 adds about 6 clk to a
// SIMD that is busy with FMAs; the fp32 instruction takes its 32 clk from the same issue slots), so
// the dense product goes there, in split precision:
//   fp32 tensors   A = Ah + Al, Wt * s = Wh + Wl in fp16 (s a power of two per channel, so that the
//                  tile's largest entry lies in [0.5, 1)), three products Ah Wh + Al Wh + Ah Wl with
//                  fp32 sums -- the dropped terms are below 2^-21 of the channel's largest weight;
//   fp16 / bf16    A = Ah + Al in the tensor's type, Wt as it is: two products.
// Ah Wh + Al Wh is one K = 32 instruction ([Ah | Al] against [Wh ; Wh]), Ah Wl another ([Wl ; 0]).
//
// A unit of work is (image, 128-pixel tile, block of 16 channels); a workgroup of 8 waves walks
// units, channel block fastest; wave w owns pixels 16 w .. 16 w + 15 of the tile.
//   * per workgroup: every channel block's split filter operands go to LDS once;
//   * per tile: the scope coordinates (h, w) of the (pixel, tap) pairs go to LDS and every lane
//     derives the A operands of its pixel (l % 16) and its four cells (4 (l / 16) ..), 36 registers,
//     kept for all channel blocks of the tile;
//   * per unit: the 16 channels' source tiles with their halo rows are staged channel-major in LDS
//     from loads coalesced along pixels (issued one unit ahead, into registers); per tap two or
//     three matrix instructions leave w_eff[pixels 4 kg .. 4 kg + 3][channel q] in lane (kg, q),
//     which holds the same channel's inputs for those pixels: four FMAs per tap.
// grad input is the same kernel on the transposed geometry: the lane owns input pixels, tap t is fed
// by output pixel o = q + pad - f * dil and uses o's rotation (K.cu:611-651), so the coordinate
// table covers the staged range of output pixels instead of the tile.
#include <algorithm>

#include "dk_kernels.h"

namespace dk {

namespace {

constexpr int kPix = 128;     // pixels per tile
constexpr int kCh = 16;       // channels per matrix block; a unit is one block of fp32 channels or two of 16-bit ones
constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int kMaxX = 6;      // staged source elements per lane and channel: tile + halo rows <= 64 * kMaxX

typedef float f4 __attribute__((ext_vector_type(4)));

// The matrix element type of a tensor type and its two instruction shapes.
// Both run as one K = 32 matrix instruction per product pair.  They are issued from inline
// assembly, three taps at a time, because the result registers must not overlap the operands: the
// compiler lets the result of a 4-register MFMA share registers with an operand at the operand's
// last use (`v_mfma_f32_16x16x32_f16 v[156:159], v[32:35], v[154:157], 0` is what the builtin
// produced), and on gfx950 rows 0 and 1 of such a result came out as garbage.  "=&v" (early
// clobber) rules the overlap out.  What the compiler's hazard recogniser would otherwise insert is
// written out: the second instruction on a result follows two independent ones (its SrcC is
// complete by then), and s_nop 7 after the last one covers the 4-pass instruction's 7 wait states
// before a vector ALU instruction may read the result.
template <typename E> struct Mx;
template <> struct Mx<_Float16> {
  typedef _Float16 v4 __attribute__((ext_vector_type(4)));
  typedef _Float16 v8 __attribute__((ext_vector_type(8)));
  // d_i = a_i * b0 (+ a_i * b1): rows = the 16 pixels, columns = the 16 channels
  template <bool SECOND>
  static __device__ __forceinline__ void row(f4& d0, f4& d1, f4& d2, v8 a0, v8 a1, v8 a2, v8 b0, v8 b1) {
    if constexpr (SECOND)
      asm volatile(
          "s_nop 1\n\t"
          "v_mfma_f32_16x16x32_f16 %0, %3, %6, 0\n\t"
          "v_mfma_f32_16x16x32_f16 %1, %4, %6, 0\n\t"
          "v_mfma_f32_16x16x32_f16 %2, %5, %6, 0\n\t"
          "v_mfma_f32_16x16x32_f16 %0, %3, %7, %0\n\t"
          "v_mfma_f32_16x16x32_f16 %1, %4, %7, %1\n\t"
          "v_mfma_f32_16x16x32_f16 %2, %5, %7, %2\n\t"
          "s_nop 7"
          : "=&v"(d0), "=&v"(d1), "=&v"(d2)
          : "v"(a0), "v"(a1), "v"(a2), "v"(b0), "v"(b1));
    else
      asm volatile(
          "s_nop 1\n\t"
          "v_mfma_f32_16x16x32_f16 %0, %3, %6, 0\n\t"
          "v_mfma_f32_16x16x32_f16 %1, %4, %6, 0\n\t"
          "v_mfma_f32_16x16x32_f16 %2, %5, %6, 0\n\t"
          "s_nop 7"
          : "=&v"(d0), "=&v"(d1), "=&v"(d2)
          : "v"(a0), "v"(a1), "v"(a2), "v"(b0));
  }
};
template <> struct Mx<__bf16> {
  typedef __bf16 v4 __attribute__((ext_vector_type(4)));
  typedef __bf16 v8 __attribute__((ext_vector_type(8)));
  template <bool SECOND>
  static __device__ __forceinline__ void row(f4& d0, f4& d1, f4& d2, v8 a0, v8 a1, v8 a2, v8 b0, v8 b1) {
    static_assert(!SECOND, "bfloat16 tensors need no second product");
    asm volatile(
        "s_nop 1\n\t"
        "v_mfma_f32_16x16x32_bf16 %0, %3, %6, 0\n\t"
        "v_mfma_f32_16x16x32_bf16 %1, %4, %6, 0\n\t"
        "v_mfma_f32_16x16x32_bf16 %2, %5, %6, 0\n\t"
        "s_nop 7"
        : "=&v"(d0), "=&v"(d1), "=&v"(d2)
        : "v"(a0), "v"(a1), "v"(a2), "v"(b0));
  }
};
template <typename T> struct MxOf { using type = _Float16; };  // float, __half
template <> struct MxOf<bf16_t> { using type = __bf16; };

// v = hi + lo + (an error below 2^-2p |v| for a p-bit type), both parts in the matrix type.
// The empty asm pins v as one fp32 value: where v is a product the compiler otherwise contracts
// it into the conversions -- hi packed from the fp32-rounded product, lo taken against the once-rounded
// exact product (v_fma_mixlo_f16) -- and the two roundings of hi differ by one unit in the last
// place about once in 4096 values, which leaves a hi + lo that is off by that unit.
template <typename E>
__device__ __forceinline__ void split2(float v, E& hi, E& lo) {
  asm volatile("" : "+v"(v));
  hi = static_cast<E>(v);
  lo = static_cast<E>(v - static_cast<float>(hi));
}

__device__ __forceinline__ float hat(float d) { return __builtin_amdgcn_fmed3f(1.f - fabsf(d), 0.f, 1.f); }

// First slot of channel j's row in the staged source tile.  Rows are a multiple of 64 slots
// apart plus a skew: lane (channel q, pixel quad kg) reads row q at 4 kg + const, and
// (q % 4) + 16 (q / 4) + 4 kg covers the 64 banks exactly once.
__device__ __forceinline__ constexpr int tile_row(int j, int pitch) { return j * pitch + (j & 3) + 16 * (j >> 2); }
// The same for 16-bit tensors, whose tile holds two elements per slot: lane (q, kg) reads rows q and
// q + 16 at 2 kg + const; with a pitch of 8 mod 64 the rows q % 8 start 8 banks apart, and the one
// slot of skew for q / 8 odd fills the gaps between the even 2 kg.
__device__ __forceinline__ constexpr int tile_row16(int j, int pitch) { return j * pitch + ((j >> 3) & 1); }

// A staged element: the tile holds one 32-bit slot per element, written by the buffer load itself
// (a 2-byte load leaves the element zero-extended in its slot).
__device__ __forceinline__ float slot_value(unsigned bits, const float*) { return __uint_as_float(bits); }
__device__ __forceinline__ float slot_value(unsigned bits, const bf16_t*) { return __uint_as_float(bits << 16); }
__device__ __forceinline__ float slot_value(unsigned bits, const __half*) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(bits)));
}

// The two elements of a slot of a 16-bit tile (the lower address in the lower half).
__device__ __forceinline__ float pair_lo(unsigned bits, const float*) { return 0.f; }
__device__ __forceinline__ float pair_hi(unsigned bits, const float*) { return 0.f; }
__device__ __forceinline__ float pair_lo(unsigned bits, const bf16_t*) { return __uint_as_float(bits << 16); }
__device__ __forceinline__ float pair_hi(unsigned bits, const bf16_t*) { return __uint_as_float(bits & 0xffff0000u); }
__device__ __forceinline__ float pair_lo(unsigned bits, const __half*) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(bits)));
}
__device__ __forceinline__ float pair_hi(unsigned bits, const __half*) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(bits >> 16)));
}

typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef unsigned u4 __attribute__((ext_vector_type(4)));

// One buffer load that writes LDS: lane l's element (SIZE bytes at byte offset `off` of the buffer,
// zero if out of range) goes to the 32-bit slot `to + l`.  Issued from inline assembly so that the
// compiler does not see it: it guards every LDS read that might alias an outstanding load of this
// kind with a wait for ALL outstanding loads (it cannot tell the buffers of the rotation below apart
// once the pointers pass through the unit loop), which would take the look-ahead away.  The waits are
// written out instead (wait_barrier): a tile is read only after the wave's own loads of it have
// landed and the workgroup has passed a barrier.
// (The buffer resource as its four words: base address, 48 bits; stride 0; size in bytes; flags.)
template <typename T>
__device__ __forceinline__ u4 resource_words(const T* base, int elems) {
  const unsigned long a = reinterpret_cast<unsigned long>(base);
  return u4{(unsigned)a, (unsigned)(a >> 32) & 0xffffu, (unsigned)elems * (unsigned)sizeof(T), (unsigned)kRsrcFlags};
}
template <int SIZE>
__device__ __forceinline__ void load_to_lds(u4 r, unsigned* to, int off) {
  const unsigned addr = (unsigned)(unsigned long)(lds_void_ptr)to;
  if constexpr (SIZE == 4)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" ::"s"(addr), "v"(off), "s"(r) : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_ushort %1, %2, 0 offen lds" ::"s"(addr), "v"(off), "s"(r) : "memory", "m0");
}

// Wait until at most N of this wave's vector-memory operations are outstanding and its LDS
// operations are done, then the workgroup barrier.  __syncthreads() would do, but it waits for
// ALL outstanding vector-memory operations, and the point of the staging scheme below is that the
// loads of the unit after next stay in flight across the barrier.
template <int N>
__device__ __forceinline__ void wait_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// NX consecutive 64-element runs with one per-lane offset: the steps are the instruction's
// immediate offset, which the hardware adds to the memory address AND to the LDS address, so M0 is
// set once.
template <int SIZE, int NX>
__device__ __forceinline__ void load_run_to_lds(u4 r, unsigned* to, int off) {
  const unsigned addr = (unsigned)(unsigned long)(lds_void_ptr)to;
  static_assert(SIZE == 4, "the LDS side steps by 4 bytes per element, the memory side by SIZE: equal only for 4");
  static_assert(NX == 2 || NX == 3 || NX == 4 || NX == 6, "two, three, four or six runs");
  if constexpr (NX == 2)
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
        "buffer_load_dword %1, %2, 0 offen lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:256 lds" ::"s"(addr), "v"(off), "s"(r)
        : "memory", "m0");
  else if constexpr (NX == 3)
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
        "buffer_load_dword %1, %2, 0 offen lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:256 lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:512 lds" ::"s"(addr), "v"(off), "s"(r)
        : "memory", "m0");
  else if constexpr (NX == 4)
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
        "buffer_load_dword %1, %2, 0 offen lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:256 lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:512 lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:768 lds" ::"s"(addr), "v"(off), "s"(r)
        : "memory", "m0");
  else
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
        "buffer_load_dword %1, %2, 0 offen lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:256 lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:512 lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:768 lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:1024 lds\n\t"
        "buffer_load_dword %1, %2, 0 offen offset:1280 lds" ::"s"(addr), "v"(off), "s"(r)
        : "memory", "m0");
}

// One unit of work, and whether it is the first of its tile that this workgroup handles.
struct Unit {
  int n, p0;            // image and first pixel of the tile (set once per segment: a division by the tile count)
  int cb, seg, cb_end;  // channel block; segment and the end of its channel blocks
  bool first, valid;
};

// Source tiles are staged by buffer loads that write LDS directly (no register stage), two units
// ahead, into three buffers used in rotation.
template <typename T, int SH, int SW, bool TRANSPOSED, int NX>
__global__ __launch_bounds__(kThreads, 4) void local_gather_mfma_kernel(
    Geo g, const T* __restrict__ src, const T* __restrict__ rot, const T* __restrict__ filter,
    T* __restrict__ dst, int tiles, int nwg) {
  using E = typename MxOf<T>::type;
  using M = Mx<E>;
  constexpr bool kThird = sizeof(T) == 4;  // fp32 tensors: the filter has a low part
  constexpr bool kPacked = sizeof(T) == 2; // 16-bit tensors: two elements per slot of the tile, two channel blocks per unit
  constexpr int CHU = kPacked ? 2 * kCh : kCh;  // channels per unit
  constexpr int NRUN = kPacked ? NX / 2 : NX;   // 64-slot runs of a staged row
  constexpr int K = 9, CELLS = SH * SW;
  static_assert(CELLS <= 16, "one K = 16 block of cells");
  constexpr int PITCH = kPacked ? 64 * NRUN + 8 : 64 * NX + 64;
  constexpr int kEntries = (K * kPix + kThreads - 1) / kThreads;  // coordinate entries staged per thread
  constexpr int kChW = CHU / kWaves;                              // channels staged per wave
  constexpr int kDma = kChW * NRUN;                               // staging loads per wave and unit
  __shared__ unsigned xs0[CHU * PITCH], xs1[CHU * PITCH], xs2[CHU * PITCH];
  __shared__ float2 hw[K * kPix];  // scope coordinates (h, w) of (tap, pixel of the tile)
  extern __shared__ __align__(16) unsigned dyn[];

  const int cpg = g.channel / g.groups;
  const int nblk = ceil_div(cpg, CHU);
  uint4* wsp = reinterpret_cast<uint4*>(dyn);                  // [nblk][64]: Wh (2 words), Wl (2 words); 16-bit: W of channel q, W of channel q + 16
  float* unscale = reinterpret_cast<float*>(wsp + nblk * 64);  // [nblk][kCh]: 1 / s of the channel (fp32 tensors)

  const int total = nwg * g.groups;
  const int lb = logical_block(total);
  if (lb >= total) return;
  const int wg = lb % nwg, grp = lb / nwg;

  const int W = g.in_w;  // == out_w
  const int out_plane = g.out_h * W, in_plane = g.in_h * W;
  const int dst_plane = TRANSPOSED ? in_plane : out_plane, src_plane = TRANSPOSED ? out_plane : in_plane;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int q = lane & 15, kg = lane >> 4;
  const int row_step = g.dil_h * W;  // elements between two tap rows
  // first staged source element relative to the tile's first pixel: the lowest tap offset.
  // forward: tap (f_h, f_w) reads p + (f_h dil - pad) W + f_w - 1; grad input: output pixel
  // q + (pad - f_h dil) W + 1 - f_w.  Either way the taps read staged index
  // px + rr * row_step + cc with (rr, cc) = (f_h, f_w), or (2 - f_h, 2 - f_w) for grad input.
  const int lo = TRANSPOSED ? (g.pad_h - 2 * g.dil_h) * W - 1 : -g.pad_h * W - 1;
  const unsigned w_magic = (unsigned)(0x100000000ull / (unsigned)W) + 1u;  // floor(p / W) = (p * magic) >> 32 for p < 2^24

  // ---- per workgroup: the split filter operands of every channel block.  Lane (q, kg) of the
  // B side stands for channel q and cells 4 kg .. 4 kg + 3.
  for (int e = threadIdx.x; e < nblk * 64; e += kThreads) {
    const int b = e >> 6, l = e & 63, cj = b * CHU + (l & 15), c0 = 4 * (l >> 4);
    if constexpr (kPacked) {
      // the filter is exact in the matrix type: the cells 4 kg .. 4 kg + 3 of channel q and of channel q + 16
      typename M::v4 w2[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int ch = cj + h * kCh;
        const T* f = filter + (size_t)(grp + g.groups * (ch < cpg ? ch : 0)) * CELLS;
#pragma unroll
        for (int k = 0; k < 4; ++k) w2[h][k] = static_cast<E>((ch < cpg && c0 + k < CELLS) ? ld(f + c0 + k) : 0.f);
      }
      const uint2 b0 = __builtin_bit_cast(uint2, w2[0]), b1 = __builtin_bit_cast(uint2, w2[1]);
      wsp[e] = make_uint4(b0.x, b0.y, b1.x, b1.y);
      continue;
    }
    float v[4] = {0.f, 0.f, 0.f, 0.f}, s = 1.f;
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
        if ((l >> 4) == 0) unscale[b * kCh + (l & 15)] = ldexpf(1.f, ex);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (c0 + k < CELLS) v[k] = ld(f + c0 + k) * s;
    } else if constexpr (kThird) {
      if ((l >> 4) == 0) unscale[b * kCh + (l & 15)] = 0.f;
    }
    typename M::v4 h, lw;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      E a, bb;
      split2<E>(v[k], a, bb);
      h[k] = a;
      lw[k] = bb;
    }
    uint2 hb = __builtin_bit_cast(uint2, h), lb2 = __builtin_bit_cast(uint2, lw);
    wsp[e] = make_uint4(hb.x, hb.y, lb2.x, lb2.y);
  }

  // ---- this workgroup's share of the (tile, channel block) units: whole tiles round-robin (tile t
  // to workgroup t % nwg: neighbouring workgroups stage neighbouring tiles at the same time and
  // the halo rows they share come from L2), the units of the last items % nwg tiles as contiguous
  // ranges in (tile, block) order cut at the tile boundaries.
  const int items = g.batch * tiles;
  const int whole = items / nwg;
  const long rest_units = (long)(items - whole * nwg) * nblk;
  const long r_lo = rest_units * wg / nwg, r_hi = rest_units * (wg + 1) / nwg;
  const int rest_lo = (int)(r_lo / nblk), rest_hi = r_hi > r_lo ? (int)((r_hi - 1) / nblk) : rest_lo - 1;
  const int nseg = whole + (rest_hi - rest_lo + 1);
  auto segment = [&](int k, int& item, int& cb_begin, int& cb_end) {
    if (k < whole) {
      item = wg + k * nwg;
      cb_begin = 0;
      cb_end = nblk;
    } else {
      const int t = rest_lo + (k - whole);
      item = whole * nwg + t;
      cb_begin = t == rest_lo ? (int)(r_lo % nblk) : 0;
      cb_end = t == rest_hi ? (int)((r_hi - 1) % nblk) + 1 : nblk;
    }
  };
  auto first_of_segment = [&](int seg) {
    Unit u{0, 0, 0, seg, 0, true, seg < nseg};
    if (u.valid) {
      int item;
      segment(seg, item, u.cb, u.cb_end);
      u.n = item / tiles;
      u.p0 = (item - u.n * tiles) * kPix;
    }
    return u;
  };
  auto first_unit = [&]() { return first_of_segment(0); };
  auto next_unit = [&](Unit u) {  // one scalar add and compare except at the end of a segment
    if (!u.valid) return u;
    if (u.cb + 1 < u.cb_end) {
      ++u.cb;
      u.first = false;
      return u;
    }
    return first_of_segment(u.seg + 1);
  };

  // ---- staging
  // bytes between two channels of the group, and this wave's first staged channel of a unit in those terms
  const size_t ch_bytes = (size_t)g.groups * src_plane * sizeof(T);
  const size_t wave_first = (size_t)wave * ch_bytes;
  auto stage_tile = [&](const Unit& u, unsigned* buf) {
    const int n = u.n, x0 = u.p0 + lo;
    // channel u.cb * CHU + wave of the unit: one 64-bit scalar product per unit, an addition per channel
    const char* unit_first = reinterpret_cast<const char*>(src) + (size_t)(n * g.channel + grp) * src_plane * sizeof(T) +
                             (size_t)(u.cb * CHU) * ch_bytes + wave_first;
#pragma unroll
    for (int jj = 0; jj < kChW; ++jj) {
      const int j = wave + jj * kWaves, cj = u.cb * CHU + j;
      const bool chan = cj < cpg;
      const T* plane = reinterpret_cast<const T*>(unit_first + (chan ? (size_t)jj * kWaves * ch_bytes : 0));
      if constexpr (kPacked) {
        // pairs of elements from the even element below x0 (the width is even, so x0 is odd and every
        // plane starts on a 4-byte boundary): slot i of the row holds elements x0 - 1 + 2 i, + 1
        const int x0e = x0 - 1;
        unsigned* row = buf + tile_row16(j, PITCH);
        if (x0e >= 0) {
          const u4 rx = resource_words(plane + x0e, chan ? max(src_plane - x0e, 0) : 0);
          load_run_to_lds<4, NRUN>(rx, row, lane * 4);
        } else {
          const u4 rx = resource_words(plane, chan ? src_plane : 0);
#pragma unroll
          for (int k = 0; k < NRUN; ++k) {
            const int e = x0e + 2 * (lane + 64 * k);  // even: both elements of the pair lie before the plane, or neither
            load_to_lds<4>(rx, row + 64 * k, e < 0 ? (int)kOutOfRange : e * 2);
          }
        }
      } else if (x0 >= 0) {
        // the buffer starts at the first staged element: every lane's offset is its lane number,
        // the 64-element steps are immediates, and what lies past the plane fails the range check
        const u4 rx = resource_words(plane + x0, chan ? max(src_plane - x0, 0) : 0);
        load_run_to_lds<4, NX>(rx, buf + tile_row(j, PITCH), lane * 4);
      } else {
        // the first tile of a plane: the elements before the plane must read as zeros
        const u4 rx = resource_words(plane, chan ? src_plane : 0);
#pragma unroll
        for (int k = 0; k < NX; ++k) {
          const int e = x0 + lane + 64 * k;
          load_to_lds<4>(rx, buf + tile_row(j, PITCH) + 64 * k, e < 0 ? (int)kOutOfRange : e * 4);
        }
      }
    }
  };
  // The rotation pixel of (tap t, pixel idx of the tile), and whether the tap contributes at all.
  // forward: the pixel itself, if the tap's input element lies in the image; grad input: the
  // output pixel q + pad - f dil that feeds input pixel q through tap t, if it exists.
  auto rotation_pixel = [&](int p0, int t, int idx, int& o) {
    const int p = p0 + idx, f_h = t / 3, f_w = t % 3;
    const bool live = p < dst_plane;
    const int pc = live ? p : 0;
    const int ph = (int)__umulhi((unsigned)pc, w_magic), pw = pc - ph * W;  // pc / W, exact below 2^32 / W
    const int rh = TRANSPOSED ? ph + g.pad_h - f_h * g.dil_h : ph + f_h * g.dil_h - g.pad_h;
    const int rw = TRANSPOSED ? pw + 1 - f_w : pw + f_w - 1;
    const bool ok = live && rw >= 0 && rw < W && rh >= 0 && rh < (TRANSPOSED ? g.out_h : g.in_h);
    o = TRANSPOSED ? rh * W + rw : pc;
    return ok;
  };
  // The rotation values of a tile go straight into the coordinate table, again by loads that write
  // LDS (no registers held while they are in flight): entry e = (tap, pixel) is two slots, so a
  // wave-load fills 32 entries, lane l the component l % 2 of entry l / 2; the gather of the
  // rotation pixel is the load's own per-lane offset.  store_coordinates() then turns the
  // values into scope coordinates in place.
  constexpr int kRotLoads = K * kPix / 32;                         // wave-loads per tile
  constexpr int kRotPerWave = (kRotLoads + kWaves - 1) / kWaves;   // ... per wave
  // (The empty asm in these two once-per-tile functions makes the thread's index opaque, so that
  // the per-thread constants derived from it -- tap, pixel, plane offsets of each entry -- are
  // recomputed when needed instead of living in registers through the unit loop, which has none to spare.)
  auto load_rotation = [&](const Unit& u) {
    int lane_ = lane;
    asm volatile("" : "+v"(lane_));
    const int n = u.n, p0 = u.p0;
    const u4 rr = resource_words(rot + (size_t)(n * g.groups + grp) * (K * 2) * out_plane, K * 2 * out_plane);
#pragma unroll
    for (int k = 0; k < kRotPerWave; ++k) {
      const int ld_ = wave + k * kWaves;  // wave-uniform
      if (ld_ < kRotLoads) {
        const int e = ld_ * 32 + (lane_ >> 1);
        const int t = e / kPix, idx = e - t * kPix;
        int o = 0;
        const bool ok = rotation_pixel(p0, t, idx, o);
        const int off = ok ? (int)((unsigned)((2 * t + (lane_ & 1)) * out_plane + o) * (unsigned)sizeof(T)) : (int)kOutOfRange;
        load_to_lds<sizeof(T)>(rr, reinterpret_cast<unsigned*>(hw) + ld_ * 64, off);
      }
    }
  };
  // Scope coordinates: K.cu:338-341 and the band test of K.cu:59; a tap that contributes nothing
  // gets (-2, -2), where every hat is 0.
  auto store_coordinates = [&](const Unit& u) {
    int tid_ = threadIdx.x;
    asm volatile("" : "+v"(tid_));
    const int p0 = u.p0;
#pragma unroll
    for (int k = 0; k < kEntries; ++k) {
      const int e = tid_ + k * kThreads;
      const int t = e / kPix, idx = e - t * kPix;
      if (t < K) {
        int o = 0;
        const bool ok = rotation_pixel(p0, t, idx, o);
        const uint2 raw = *reinterpret_cast<const uint2*>(hw + e);
        const float h = scope_coord<float>(g, t / 3, slot_value(raw.x, rot), g.centre_h);
        const float w = scope_coord<float>(g, t % 3, slot_value(raw.y, rot), g.centre_w);
        const bool in = ok && (h > -1.f) && (w > -1.f) && (h < float(SH)) && (w < float(SW));
        hw[e] = in ? make_float2(h, w) : make_float2(-2.f, -2.f);
      }
    }
  };

  // A side: lane (pixel q of the wave's 16, cells 4 kg .. 4 kg + 3)
  // cell 4 kg + k = (row, column); rows past the last cell stay 0.  With four columns the row is kg
  // and the column k, which costs one register instead of eight.
  auto cell_row = [&](int k) { return SW == 4 ? float(kg) : (4 * kg + k < CELLS ? float((4 * kg + k) / SW) : 64.f); };
  auto cell_col = [&](int k) { return SW == 4 ? float(k) : float((4 * kg + k) % SW); };
  typename M::v8 A[K];
  const int px = wave * 16 + 4 * kg;  // D side: first of this lane's four pixels in the tile

  auto derive_operands = [&]() {
#pragma unroll
    for (int t = 0; t < K; ++t) {
      const float2 c = hw[t * kPix + wave * 16 + q];
      // hi and lo parts, two values per conversion instruction (vector conversions: they also leave the values
      // packed; one at a time a value costs two conversions and two packing moves more)
      typedef float f2v __attribute__((ext_vector_type(2)));
      typedef E e2v __attribute__((ext_vector_type(2)));
      float v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        v[k] = hat(c.x - cell_row(k)) * hat(c.y - cell_col(k));
        asm volatile("" : "+v"(v[k]));  // as in split2: one fp32 value for both parts
      }
      const e2v h01 = __builtin_convertvector(f2v{v[0], v[1]}, e2v), h23 = __builtin_convertvector(f2v{v[2], v[3]}, e2v);
      const f2v b01 = __builtin_convertvector(h01, f2v), b23 = __builtin_convertvector(h23, f2v);
      const e2v l01 = __builtin_convertvector(f2v{v[0] - b01[0], v[1] - b01[1]}, e2v);
      const e2v l23 = __builtin_convertvector(f2v{v[2] - b23[0], v[3] - b23[1]}, e2v);
      A[t] = typename M::v8{h01[0], h01[1], h23[0], h23[1], l01[0], l01[1], l23[0], l23[1]};
    }
  };

  // Where a lane's four results go: a scalar 64-bit part per unit (image, first channel of the unit, tile) and a
  // 32-bit part per lane (its channel within the unit, its pixels within the tile) that never changes.
  const unsigned lane_out = (unsigned)(g.groups * q) * (unsigned)dst_plane + (unsigned)px;
  auto unit_out = [&](const Unit& u) {
    return dst + ((size_t)(u.n * g.channel + grp) + (size_t)g.groups * (u.cb * CHU)) * dst_plane + u.p0;
  };
  auto multiply_unit = [&](const Unit& u, const unsigned* buf) {
    if constexpr (kPacked) {
      // one channel block after the other (block h: channel q + 16 h), each with its own store, so that only
      // one block's sums and filter operand are live
      const int p = u.p0 + px;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // [W ; W] pairs with [Ah | Al]
        const uint2 wbits = reinterpret_cast<const uint2*>(wsp + u.cb * 64 + lane)[h];
        const typename M::v4 w4 = __builtin_bit_cast(typename M::v4, wbits);
        const typename M::v8 wb = __builtin_shufflevector(w4, w4, 0, 1, 2, 3, 0, 1, 2, 3);
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        const unsigned* xr0 = buf + tile_row16(q + h * kCh, PITCH) + (px >> 1);
#pragma unroll
        for (int rr = 0; rr < 3; ++rr) {
          // columns -1 .. +4 around the four pixels: element px + rr * row_step + k of the range that starts at
          // x0 = slot-aligned start + 1, so k = 0 is the upper half of the first slot
          const unsigned* xr = xr0 + ((rr * row_step) >> 1);
          const unsigned u0 = xr[0], u1 = xr[1], u2 = xr[2], u3 = xr[3];
          const float x6[6] = {pair_hi(u0, src), pair_lo(u1, src), pair_hi(u1, src),
                               pair_lo(u2, src), pair_hi(u2, src), pair_lo(u3, src)};
          const int t0 = TRANSPOSED ? (2 - rr) * 3 + 2 : rr * 3, dt = TRANSPOSED ? -1 : 1;
          f4 d[3];
          M::template row<false>(d[0], d[1], d[2], A[t0], A[t0 + dt], A[t0 + 2 * dt], wb, wb);
#pragma unroll
          for (int cc = 0; cc < 3; ++cc)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = fmaf(x6[i + cc], d[cc][i], acc[i]);
        }
        const int cj = u.cb * CHU + h * kCh + q;
        if (cj < cpg && p < dst_plane) {
          // the plane is a multiple of 4 pixels (the host checks), so the four pixels are inside it and 8-byte aligned
          T* out = unit_out(u) + (lane_out + (unsigned)h * (unsigned)(kCh * g.groups * dst_plane));
          struct { T e[4]; } pk;
#pragma unroll
          for (int i = 0; i < 4; ++i) st(pk.e + i, acc[i]);
          *reinterpret_cast<uint2*>(out) = __builtin_bit_cast(uint2, pk);  // default policy: 2-byte runs merge to whole lines in L2
        }
      }
      return;
    }
    const uint4 wv = wsp[u.cb * 64 + lane];
    const typename M::v4 wh = __builtin_bit_cast(typename M::v4, make_uint2(wv.x, wv.y));
    const typename M::v4 wl = __builtin_bit_cast(typename M::v4, make_uint2(wv.z, wv.w));
    // [Wh ; Wh] pairs with [Ah | Al]; [Wl ; 0] adds Ah Wl
    const typename M::v8 whh = __builtin_shufflevector(wh, wh, 0, 1, 2, 3, 0, 1, 2, 3);
    const typename M::v4 zero4 = {E(0), E(0), E(0), E(0)};
    const typename M::v8 wl0 = __builtin_shufflevector(wl, zero4, 0, 1, 2, 3, 4, 5, 6, 7);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    const unsigned* xr0 = buf + tile_row(q, PITCH) + px;
#pragma unroll
    for (int rr = 0; rr < 3; ++rr) {
      float x6[6];  // columns -1 .. +4 of staged tap row rr around the four pixels
#pragma unroll
      for (int k = 0; k < 6; ++k) x6[k] = __uint_as_float(xr0[rr * row_step + k]);
      const int t0 = TRANSPOSED ? (2 - rr) * 3 + 2 : rr * 3, dt = TRANSPOSED ? -1 : 1;  // the taps of columns 0, 1, 2
      f4 d[3];
      M::template row<kThird>(d[0], d[1], d[2], A[t0], A[t0 + dt], A[t0 + 2 * dt], whh, wl0);
#pragma unroll
      for (int cc = 0; cc < 3; ++cc)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = fmaf(x6[i + cc], d[cc][i], acc[i]);
    }
    // lane (kg, q): channel q of the block, pixels px .. px + 3 of the tile
    const int cj = u.cb * kCh + q;
    const int p = u.p0 + px;
    if (cj < cpg && p < dst_plane) {
      const float us = unscale[u.cb * kCh + q];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] *= us;
      T* out = unit_out(u) + lane_out;
      if ((dst_plane & 3) == 0) {
        // p is a multiple of 4, so the four pixels are inside the plane and 16-byte aligned
        f4 v = {acc[0], acc[1], acc[2], acc[3]};
        *reinterpret_cast<f4*>(out) = v;  // default policy: the wave's 64-byte runs merge to whole lines in L2
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (p + i < dst_plane) st(out + i, acc[i]);
      }
    }
  };

  // ---- the walk.  In flight when unit u starts: the tiles of u (issued two units ago) and of
  // u + 1.  Per unit: wait for the own loads of u's tile and for everybody to have left the
  // previous unit; [first unit of a tile: rotation values -> coordinates in place, barrier, operands];
  // multiply and store; start the rotation loads of the next tile where the table is free for them,
  // then the tile loads of unit u + 2 into the buffer the previous unit used (always last, so that
  // "all but the newest kDma operations" is the right thing to wait for).
  // The rotation loads of tile T + 1 go out in the second unit of tile T (the table is read in the
  // first); a tile with a single unit here is followed by a stall on them.
  Unit u0 = first_unit(), u1 = next_unit(u0), u2 = next_unit(u1);
  bool rot_in_flight = false;
  if (u0.valid) {
    load_rotation(u0);
    stage_tile(u0, xs0);
  }
  if (u1.valid) stage_tile(u1, xs1);
  auto step = [&](unsigned* cur, unsigned* free_buf) {
    if (u0.first && !rot_in_flight && u0.seg > 0) {
      // single-unit tile before this one: its loads could not be issued ahead
      wait_barrier<63>();  // everybody is past the previous tile's operands
      load_rotation(u0);
      wait_barrier<0>();
    } else if (u1.valid) {
      wait_barrier<kDma>();  // everything older than the loads of u1's tile has landed
    } else {
      wait_barrier<0>();
    }
    if (u0.first) {
      rot_in_flight = false;
      store_coordinates(u0);
      wait_barrier<63>();  // LDS only: the tile loads stay in flight
      derive_operands();
    }
    const bool table_free = !u0.first;  // read in the first unit of this tile, at least a barrier ago
    multiply_unit(u0, cur);
    // vector-memory operations of this step, oldest first: the result stores, the rotation loads,
    // the tile loads -- so that "all but the newest kDma" at the next step means "all but u2's tile"
    if (table_free && !rot_in_flight) {
      const Unit nx = first_of_segment(u0.seg + 1);
      if (nx.valid) {
        load_rotation(nx);
        rot_in_flight = true;
      }
    }
    if (u2.valid) stage_tile(u2, free_buf);
    u0 = u1;
    u1 = u2;
    u2 = next_unit(u2);
  };
  while (u0.valid) {
    step(xs0, xs2);
    if (!u0.valid) break;
    step(xs1, xs0);
    if (!u0.valid) break;
    step(xs2, xs1);
  }
}

struct GatherPlan {
  bool ok;
  int nx, pitch, tiles, nwg;
  size_t lds;
};

// Static LDS of the kernel: three tiles and the coordinate table.
constexpr long gather_static_lds(bool packed, int nx) {
  return 3L * (packed ? 2 * kCh * (64 * (nx / 2) + 8) : kCh * (64 * nx + 64)) * 4 + 9L * kPix * 8;
}

template <int SH, int SW>
GatherPlan gather_plan(const Geo& g, bool transposed, bool packed) {
  GatherPlan p{};
  p.ok = false;
  const bool same_width = g.stride_h == 1 && g.stride_w == 1 && g.dil_w == 1 && g.pad_w == 1 && g.k_h == 3 &&
                          g.k_w == 3 && g.in_w == g.out_w;
  if (!same_width || SH * SW > 16 || g.in_w < 2 || path_disabled(kNoRows) || path_disabled(kNoGatherMfma)) return p;  // in_w >= 2: the division by the width is a multiplication
  // 16-bit tiles are staged as pairs of elements: rows of an even number of elements keep every plane, every
  // tap row and every lane's four pixels on pair boundaries
  if (packed && (g.in_w & 1)) return p;
  const long xt = kPix + 2 + 2L * g.dil_h * g.in_w + (packed ? 1 : 0);  // tile + halo rows (+ the element below an odd start)
  if (xt > 64 * kMaxX) return p;
  p.nx = xt <= 256 ? 4 : kMaxX;
  const int chu = packed ? 2 * kCh : kCh;
  const int cpg = g.channel / g.groups, nblk = ceil_div(cpg, chu);
  const long plane = transposed ? (long)g.in_h * g.in_w : (long)g.out_h * g.out_w;
  if (packed && (plane & 3)) return p;  // four pixels per 8-byte store
  if ((long)g.groups * 2 * kCh * plane >= (1L << 31)) return p;  // a lane's channel offset within a unit in 32 bits
  p.tiles = (int)ceil_div((int)plane, kPix);
  // dynamic part: the split filter operands
  const long lds = (long)nblk * 64 * 16 + (long)nblk * kCh * 4;
  if (lds + gather_static_lds(packed, p.nx) > 160 * 1024) return p;
  p.lds = (size_t)lds;
  const long units = (long)g.batch * p.tiles * nblk;
  if (units >= (1L << 30)) return p;
  // at most two workgroups per CU, all resident at once, each walking an equal share of the units
  // (with fewer tiles than that, the workgroups share tiles: contiguous ranges of a tile's channel blocks, at least
  // four units each, every range paying the tile's set-up)
  p.nwg = (int)std::max(1L, std::min(std::max((long)g.batch * p.tiles, units / 4), (long)std::max(1, 2 * 256 / g.groups)));
  p.ok = true;
  return p;
}

template <typename T, int SH, int SW>
bool run_gather_mfma(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                     hipStream_t stream) {
  constexpr bool packed = sizeof(T) == 2;
  const GatherPlan p = gather_plan<SH, SW>(g, transposed, packed);
  if (!p.ok) return false;
  if (packed && (reinterpret_cast<uintptr_t>(src) % 4 != 0 || reinterpret_cast<uintptr_t>(dst) % 8 != 0)) return false;
  const unsigned grid = (unsigned)xcd_grid_size((long)p.nwg * g.groups);
#define DK_LAUNCH(TR, NXV)                                                                        \
  {                                                                                               \
    auto kernel = local_gather_mfma_kernel<T, SH, SW, TR, NXV>;                                   \
    const int room = 160 * 1024 - (int)gather_static_lds(packed, NXV);                            \
    if (!allow_dynamic_lds(reinterpret_cast<const void*>(kernel), room)) return false;            \
    kernel<<<grid, kThreads, p.lds, stream>>>(g, src, rot, filter, dst, p.tiles, p.nwg);          \
  }
  if (transposed) {
    if (p.nx == 4) DK_LAUNCH(true, 4) else DK_LAUNCH(true, kMaxX)
  } else {
    if (p.nx == 4) DK_LAUNCH(false, 4) else DK_LAUNCH(false, kMaxX)
  }
#undef DK_LAUNCH
  return true;
}

}  // namespace

template <typename T>
bool mfma_local_gather(const Geo& g, bool transposed, const T* src, const T* rot, const T* filter, T* dst,
                       hipStream_t stream) {
  if (g.k_h != 3 || g.k_w != 3) return false;
  if ((long)g.in_h * g.in_w >= (1L << 24) || (long)g.out_h * g.out_w >= (1L << 24)) return false;  // byte offsets of 18 rotation planes in 31 bits
  // A tile's set-up (coordinates, operands) is paid once per tile and its 128 pixels must be filled: the kernel
  // wins where a plane has many tiles and a group at least six 16-channel blocks (N=64 C=144 56 x 56: 64 against
  // 68 us), and loses to the row kernels on small planes or few channels (fp32, N=64: C=960 7 x 7: 73 against 18 us;
  // C=384 14 x 14: 31 / 19; C=192 28 x 28: 41 / 34; C=32 112 x 112: 122 / 58).  16-bit tensors, whose units hold 32
  // channels, also win on smaller planes once there are enough units to share out (bf16, N=128: C=384 14 x 14
  // 29 against 33 us, C=576 14 x 14 38 / 44, C=192 28 x 28 45 / 54; N=64: 22.8 / 19.1, 29.4 / 27.4, 29.9 / 33.7).
  if (!path_disabled(kForceGatherMfma)) {
    const long plane = (long)g.out_h * g.out_w;
    const int cpg = g.channel / g.groups;
    const long units = (long)g.batch * ceil_div((int)plane, kPix) * ceil_div(cpg, 2 * kCh);
    const bool large = plane >= 2048 || (sizeof(T) == 2 && units >= 2560);
    if (!large || cpg < 96) return false;
  }
  if (g.scope_h == 4 && g.scope_w == 4) return run_gather_mfma<T, 4, 4>(g, transposed, src, rot, filter, dst, stream);
  if (g.scope_h == 3 && g.scope_w == 3) return run_gather_mfma<T, 3, 3>(g, transposed, src, rot, filter, dst, stream);
  return false;
}

template bool mfma_local_gather<float>(const Geo&, bool, const float*, const float*, const float*, float*, hipStream_t);
template bool mfma_local_gather<__half>(const Geo&, bool, const __half*, const __half*, const __half*, __half*, hipStream_t);
template bool mfma_local_gather<bf16_t>(const Geo&, bool, const bf16_t*, const bf16_t*, const bf16_t*, bf16_t*, hipStream_t);

}  // namespace dk
