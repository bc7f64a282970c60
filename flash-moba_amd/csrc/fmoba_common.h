// Shared device helpers for the gfx950 FlashMoBA kernels: element types, MFMA wrappers,
// transposing LDS reads, wave-level utilities and the host-side error plumbing.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>
#include <utility>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/flash_moba_hip.h"

namespace fmoba {

// ------------------------------------------------------------------------------------
// host-side error handling
// ------------------------------------------------------------------------------------
void set_error(const char *fmt, ...);
#define FMOBA_REQUIRE(cond, ...)          \
  do {                                    \
    if (!(cond)) {                        \
      ::fmoba::set_error(__VA_ARGS__);    \
      return 1;                           \
    }                                     \
  } while (0)
#define FMOBA_LAUNCH_CHECK(what)                                                     \
  do {                                                                               \
    hipError_t e__ = hipGetLastError();                                              \
    if (e__ != hipSuccess) {                                                         \
      ::fmoba::set_error("%s: launch failed: %s", what, hipGetErrorString(e__));     \
      return 2;                                                                      \
    }                                                                                \
  } while (0)

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ------------------------------------------------------------------------------------
// element types
// ------------------------------------------------------------------------------------
typedef _Float16 f16_t;
typedef __bf16 bf16_t;

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

template <typename T> struct ElemTraits;
template <> struct ElemTraits<f16_t> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ float to_float(f16_t x) { return (float)x; }
  static __device__ __forceinline__ f16_t from_float(float x) { return (f16_t)x; }
};
template <> struct ElemTraits<bf16_t> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ float to_float(bf16_t x) { return (float)x; }
  static __device__ __forceinline__ bf16_t from_float(float x) { return (bf16_t)x; }
};

// 16 bytes = 8 elements, the unit every kernel moves.
struct alignas(16) Pack8 {
  uint32_t w[4];
};

template <typename T>
__device__ __forceinline__ float elem_to_float(uint16_t bits) {
  T x;
  __builtin_memcpy(&x, &bits, 2);
  return ElemTraits<T>::to_float(x);
}
template <typename T>
__device__ __forceinline__ uint16_t float_to_elem_bits(float f) {
  T x = ElemTraits<T>::from_float(f);
  uint16_t b;
  __builtin_memcpy(&b, &x, 2);
  return b;
}
// Two floats to one 32-bit word of two elements (lo in bits 0..15), round to nearest even:
// the vector conversion compiles to a single packed convert.
template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef T elem2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {lo, hi};
  const elem2_t r = __builtin_convertvector(v, elem2_t);
  uint32_t b;
  __builtin_memcpy(&b, &r, 4);
  return b;
}
template <typename T>
__device__ __forceinline__ void unpack8(const Pack8 &p, float (&f)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = elem_to_float<T>((uint16_t)(p.w[i] & 0xffffu));
    f[2 * i + 1] = elem_to_float<T>((uint16_t)(p.w[i] >> 16));
  }
}

// ------------------------------------------------------------------------------------
// MFMA 32x32x16 (gfx950).  Operand layout, lane l, hh = l / 32:
//   A (32 x 16): lane holds A[l % 32][hh*8 .. hh*8+7]
//   B (16 x 32): lane holds B[hh*8 .. hh*8+7][l % 32]
//   C (32 x 32): lane holds C[8*(i/4) + 4*hh + i%4][l % 32], i = 0..15
// ------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ f32x16 mfma32(const Pack8 &a, const Pack8 &b, f32x16 c);
template <>
__device__ __forceinline__ f32x16 mfma32<bf16_t>(const Pack8 &a, const Pack8 &b, f32x16 c) {
  bf16x8 av, bv;
  __builtin_memcpy(&av, &a, 16);
  __builtin_memcpy(&bv, &b, 16);
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16 mfma32<f16_t>(const Pack8 &a, const Pack8 &b, f32x16 c) {
  f16x8 av, bv;
  __builtin_memcpy(&av, &a, 16);
  __builtin_memcpy(&bv, &b, 16);
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, c, 0, 0, 0);
}

// MFMAs with the register file of every operand named, for kernels whose waves own all 512 registers of their SIMD
// lane: 256 ordinary ones and 256 accumulation registers, which only MFMAs and copies can address.  What fits without
// a copy in the dK/dV pass: dK^T and dV^T (128) and the resident K and V operands (64) in accumulation registers, S
// and dP and every operand that vector instructions produce or consume in ordinary ones.  Left to itself the compiler
// puts every MFMA result of such a kernel into accumulation registers, keeps the resident operands there as spills and
// copies them (and whole accumulator tiles) to and fro around the products: 550 copies per 160 MFMAs of that loop.
// An MFMA in assembly hides from the compiler that its result arrives late: mfma_results_ready() follows the last
// product of a chain whose result vector instructions read.
__device__ __forceinline__ u32x4_t pack8_vec(const Pack8 &p) {
  u32x4_t v;
  __builtin_memcpy(&v, &p, 16);
  return v;
}
// c = a b (FIRST) or c += a b: c and a in ordinary registers, b in accumulation registers
template <typename T, bool FIRST>
__device__ __forceinline__ void mfma32_b_acc(f32x16 &c, const Pack8 &a, const u32x4_t &b) {
#if defined(__HIP_DEVICE_COMPILE__)
  const u32x4_t av = pack8_vec(a);
  if constexpr (std::is_same<T, bf16_t>::value) {
    if constexpr (FIRST)
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(av), "a"(b));
    else
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "a"(b));
  } else {
    if constexpr (FIRST)
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(av), "a"(b));
    else
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "a"(b));
  }
#else
  (void)c, (void)a, (void)b;
#endif
}
// c = a b (FIRST) or c += a b, everything in ordinary registers
template <typename T, bool FIRST>
__device__ __forceinline__ void mfma32_vv(f32x16 &c, const Pack8 &a, const Pack8 &b) {
#if defined(__HIP_DEVICE_COMPILE__)
  const u32x4_t av = pack8_vec(a), bv = pack8_vec(b);
  if constexpr (std::is_same<T, bf16_t>::value) {
    if constexpr (FIRST)
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(av), "v"(bv));
    else
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "v"(bv));
  } else {
    if constexpr (FIRST)
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(av), "v"(bv));
    else
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "v"(bv));
  }
#else
  (void)c, (void)a, (void)b;
#endif
}
// the same with a in accumulation registers and b in ordinary ones
template <typename T, bool FIRST>
__device__ __forceinline__ void mfma32_a_acc(f32x16 &c, const u32x4_t &a, const Pack8 &b) {
#if defined(__HIP_DEVICE_COMPILE__)
  const u32x4_t bv = pack8_vec(b);
  if constexpr (std::is_same<T, bf16_t>::value) {
    if constexpr (FIRST)
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "a"(a), "v"(bv));
    else
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "a"(a), "v"(bv));
  } else {
    if constexpr (FIRST)
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "a"(a), "v"(bv));
    else
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "a"(a), "v"(bv));
  }
#else
  (void)c, (void)a, (void)b;
#endif
}
// c += a b: c in the accumulation registers a[16 SLOT .. 16 SLOT + 15], named so that the sum of a whole walk stays where
// it is (as a value with a free choice of registers it is copied to ordinary registers and back once per turn of the
// loop); a and b in ordinary registers
#define FMOBA_MFMA_SLOT(N, REGS)                                                                                   \
  if constexpr (SLOT == N) {                                                                                       \
    if constexpr (std::is_same<T, bf16_t>::value)                                                                  \
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+{" REGS "}"(c) : "v"(av), "v"(bv));              \
    else                                                                                                           \
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+{" REGS "}"(c) : "v"(av), "v"(bv));               \
  }
template <typename T, int SLOT>
__device__ __forceinline__ void mfma32_c_acc(f32x16 &c, const Pack8 &a, const Pack8 &b) {
#if defined(__HIP_DEVICE_COMPILE__)
  const u32x4_t av = pack8_vec(a), bv = pack8_vec(b);
  static_assert(SLOT >= 0 && SLOT < 8, "eight accumulator tiles");
  FMOBA_MFMA_SLOT(0, "a[0:15]")
  FMOBA_MFMA_SLOT(1, "a[16:31]")
  FMOBA_MFMA_SLOT(2, "a[32:47]")
  FMOBA_MFMA_SLOT(3, "a[48:63]")
  FMOBA_MFMA_SLOT(4, "a[64:79]")
  FMOBA_MFMA_SLOT(5, "a[80:95]")
  FMOBA_MFMA_SLOT(6, "a[96:111]")
  FMOBA_MFMA_SLOT(7, "a[112:127]")
#else
  (void)c, (void)a, (void)b;
#endif
}
#undef FMOBA_MFMA_SLOT
// A 32x32x16 product writes its result eight passes of four clocks after it starts; a vector instruction that reads
// the result has to start at least eleven instruction slots after the product, which the compiler counts for its own
// MFMAs and cannot for these.
__device__ __forceinline__ void mfma_results_ready(f32x16 &x, f32x16 &y) {  // (two different results)
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_nop 7\n\ts_nop 4" : "+v"(x), "+v"(y));
#else
  (void)x, (void)y;
#endif
}
__device__ __forceinline__ void mfma_results_ready(f32x16 &x) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_nop 7\n\ts_nop 4" : "+v"(x));
#else
  (void)x;
#endif
}

// MFMA 16x16x32 (gfx950).  Operand layout, lane l, g = l / 16:
//   A (16 x 32): lane holds A[l % 16][g*8 .. g*8+7]
//   B (32 x 16): lane holds B[g*8 .. g*8+7][l % 16]
//   C (16 x 16): lane holds C[4*g + i][l % 16], i = 0..3
template <typename T>
__device__ __forceinline__ f32x4 mfma16(const Pack8 &a, const Pack8 &b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma16<bf16_t>(const Pack8 &a, const Pack8 &b, f32x4 c) {
  bf16x8 av, bv;
  __builtin_memcpy(&av, &a, 16);
  __builtin_memcpy(&bv, &b, 16);
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma16<f16_t>(const Pack8 &a, const Pack8 &b, f32x4 c) {
  f16x8 av, bv;
  __builtin_memcpy(&av, &a, 16);
  __builtin_memcpy(&bv, &b, 16);
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, c, 0, 0, 0);
}

// Row of a 32x32 accumulator tile that register i of this lane holds.
__device__ __forceinline__ int acc_row(int i, int hh) { return 8 * (i >> 2) + 4 * hh + (i & 3); }

// When accumulator registers 8s..8s+7 (s = 0,1) of a 32x32 tile are packed and fed back
// as the k-operand of the next MFMA, contraction index kappa = hh*8 + v (v = 0..7) of
// k-step s refers to accumulator row 16*s + 8*(v/4) + 4*hh + v%4.
__device__ __forceinline__ int ktile_row(int s, int hh, int v) { return 16 * s + 8 * (v >> 2) + 4 * hh + (v & 3); }

// ------------------------------------------------------------------------------------
// Transposing LDS read (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane i
// receives element (i % 4) of the 8-byte blocks whose addresses were supplied by lanes
// i/4, i/4 + 4, i/4 + 8, i/4 + 12 of the same group.
//
// tr_frag8 builds the 8-element k-operand of a 32x32x16 MFMA for a matrix X stored
// row-major in LDS ([k][n], row stride `ld` elements) such that this lane ends up with
//   X[row(v)][col0 + l % 32],  v = 0..7,
// where row(v) = rows4_lo + v for v < 4 and rows4_hi + (v - 4) for v >= 4 are the rows
// THIS lane's half (hh) needs.  Address supplied by lane l (i = l % 16):
//   &X[rows4_xx + i / 4][col0 + 16 * ((l % 32) / 16) + 4 * (i % 4)].
// ------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
__device__ __forceinline__ s16x4 ds_read_tr16(const void *lds_generic_ptr) {
#if defined(__HIP_DEVICE_COMPILE__)
  // generic -> LDS address space: the low 32 bits of a generic LDS pointer are the LDS offset
  lds_s16x4 *p = (lds_s16x4 *)(uint32_t)(uintptr_t)lds_generic_ptr;
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(p);
#else
  (void)lds_generic_ptr;
  return s16x4{0, 0, 0, 0};
#endif
}
__device__ __forceinline__ Pack8 tr_frag8(const uint16_t *X, int ld, int rows4_lo, int rows4_hi, int col0, int lane) {
  const int i = lane & 15;
  const int c = col0 + ((lane & 31) >> 4) * 16 + (i & 3) * 4;
  const int j = i >> 2;
  s16x4 lo = ds_read_tr16(X + (rows4_lo + j) * ld + c);
  s16x4 hi = ds_read_tr16(X + (rows4_hi + j) * ld + c);
  Pack8 r;
  __builtin_memcpy(&r.w[0], &lo, 8);
  __builtin_memcpy(&r.w[2], &hi, 8);
  return r;
}

// The same read through an LDS-address-space pointer.  lane_base = tr_lane_base(X, ld, lane) is
// computed once per lane; every further offset is a compile-time constant that the
// instruction's 16-bit offset field absorbs, so a whole tile of transposed operands costs one
// address register (the generic-pointer form above needs one register per read).
typedef __attribute__((address_space(3))) const uint16_t lds_cu16;
__device__ __forceinline__ lds_cu16 *to_lds(const void *lds_generic_ptr) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (lds_cu16 *)(uint32_t)(uintptr_t)lds_generic_ptr;
#else
  (void)lds_generic_ptr;
  return nullptr;
#endif
}
__device__ __forceinline__ lds_cu16 *tr_lane_base(const uint16_t *X, int ld, int lane) {
  const int i = lane & 15;
  return to_lds(X) + (i >> 2) * ld + ((lane & 31) >> 4) * 16 + (i & 3) * 4;
}
// elem_off_lo / elem_off_hi: (rows4_xx * ld + col0) of tr_frag8, in elements
__device__ __forceinline__ Pack8 tr_frag8_at(lds_cu16 *lane_base, int elem_off_lo, int elem_off_hi) {
  Pack8 r;
#if defined(__HIP_DEVICE_COMPILE__)
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(lane_base + elem_off_lo));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(lane_base + elem_off_hi));
  __builtin_memcpy(&r.w[0], &lo, 8);
  __builtin_memcpy(&r.w[2], &hi, 8);
#else
  (void)lane_base, (void)elem_off_lo, (void)elem_off_hi;
  r = Pack8{{0, 0, 0, 0}};
#endif
  return r;
}

// ------------------------------------------------------------------------------------
// wave utilities
// ------------------------------------------------------------------------------------
__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

// Orders LDS traffic of ONE wave (writes by some lanes, reads by others).
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The same order for the compiler only.  The LDS executes the instructions of one wave in the order they were issued, so
// a read that follows a write of another lane of the same wave needs no wait; the fence above also makes the wave wait
// for every LDS read it has in flight, which a software-pipelined loop keeps issued well ahead of their use.
__device__ __forceinline__ void wave_lds_order() {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" ::: "memory");
  __builtin_amdgcn_wave_barrier();
  asm volatile("" ::: "memory");
#endif
}

// Cross-half / cross-row exchanges on the VALU (gfx950 v_permlane32_swap / v_permlane16_swap)
// instead of the LDS crossbar.  swap32(x): {x of lanes l%32, x of lanes 32 + l%32};
// swap16(x): {x of the even 16-lane row of this row pair, x of the odd row}.
struct UPair {
  uint32_t a, b;
};
__device__ __forceinline__ UPair swap32(uint32_t x) {
#if defined(__HIP_DEVICE_COMPILE__)
  auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
  return UPair{(uint32_t)r[0], (uint32_t)r[1]};
#else
  return UPair{x, x};
#endif
}
__device__ __forceinline__ UPair swap16(uint32_t x) {
#if defined(__HIP_DEVICE_COMPILE__)
  auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
  return UPair{(uint32_t)r[0], (uint32_t)r[1]};
#else
  return UPair{x, x};
#endif
}
// value of the partner lane (l ^ 32)
__device__ __forceinline__ float shfl_xor32_f(float v) {
  const UPair p = swap32(__float_as_uint(v));
  return __uint_as_float((threadIdx.x & 32) ? p.a : p.b);
}
__device__ __forceinline__ int shfl_xor32_i(int v) {
  const UPair p = swap32((uint32_t)v);
  return (int)((threadIdx.x & 32) ? p.a : p.b);
}
// Column sums of a 32 x 32 bit matrix held one row per lane (row = lane % 32; both halves of the wave may hold a copy):
// five block-swap steps transpose it (step S exchanges, between lanes l and l ^ S, the bits whose position differs
// from the lane in bit S), then lane j holds column j and counts its bits.  The exchange is ds_swizzle in its
// bit-mask mode, which permutes within groups of 32 lanes and touches no memory.
template <int S>
__device__ __forceinline__ uint32_t bit_transpose_step(uint32_t x, int lane) {
  constexpr uint32_t m = S == 16 ? 0x0000ffffu : S == 8 ? 0x00ff00ffu : S == 4 ? 0x0f0f0f0fu : S == 2 ? 0x33333333u : 0x55555555u;
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t y = (uint32_t)__builtin_amdgcn_ds_swizzle((int)x, (S << 10) | 0x1f);
#else
  const uint32_t y = x;
#endif
  return (lane & S) ? (((y >> S) & m) | (x & ~m)) : ((x & m) | ((y & m) << S));
}
__device__ __forceinline__ int bit_column_count32(uint32_t row_word, int lane) {
  uint32_t x = row_word;
  x = bit_transpose_step<16>(x, lane);
  x = bit_transpose_step<8>(x, lane);
  x = bit_transpose_step<4>(x, lane);
  x = bit_transpose_step<2>(x, lane);
  x = bit_transpose_step<1>(x, lane);
  return __popc(x);
}

// reductions over the two halves of a wave (lanes l and l ^ 32), result in both lanes
__device__ __forceinline__ int sum_xor32_i(int v) {
  const UPair p = swap32((uint32_t)v);
  return (int)(p.a + p.b);
}
__device__ __forceinline__ float max_xor32_f(float v) {
  const UPair p = swap32(__float_as_uint(v));
  return fmaxf(__uint_as_float(p.a), __uint_as_float(p.b));
}
__device__ __forceinline__ float min_xor32_f(float v) {
  const UPair p = swap32(__float_as_uint(v));
  return fminf(__uint_as_float(p.a), __uint_as_float(p.b));
}
__device__ __forceinline__ float sum_xor32_f(float v) {
  const UPair p = swap32(__float_as_uint(v));
  return __uint_as_float(p.a) + __uint_as_float(p.b);
}
// reductions over the four 16-lane rows of a wave (lanes l, l^16, l^32, l^48), result everywhere
__device__ __forceinline__ float max_rows4_f(float v) {
  const UPair p = swap16(__float_as_uint(v));
  return max_xor32_f(fmaxf(__uint_as_float(p.a), __uint_as_float(p.b)));
}
__device__ __forceinline__ float sum_rows4_f(float v) {
  const UPair p = swap16(__float_as_uint(v));
  return sum_xor32_f(__uint_as_float(p.a) + __uint_as_float(p.b));
}

// Monotone map float -> uint32 (larger float => larger key); every non-NaN value,
// including -inf, maps to a key >= 0x007fffff > 0.
__device__ __forceinline__ uint32_t float_order_key(float f) {
  uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float order_key_float(uint32_t k) {
  uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}

// first position of an ascending list whose entry is not below v
__device__ __forceinline__ int lower_bound_i32(const int32_t *p, int n, int v) {
  int lo = 0, hi = n;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (p[mid] < v)
      lo = mid + 1;
    else
      hi = mid;
  }
  return lo;
}

// The same search by a whole wave (every lane passes the same arguments and gets the same result): 64 probes per
// step, so a list of a few thousand entries takes two or three dependent loads instead of a dozen.
__device__ __forceinline__ int lower_bound_wave_i32(const int32_t *p, int n, int v) {
  const int lane = threadIdx.x & 63;
  int lo = 0, hi = n;
  while (lo < hi) {
    const int step = (hi - lo + 63) >> 6;
    const int q = lo + lane * step;
    const bool below = q < hi && p[q] < v;
    const int cnt = __popcll(__ballot(below));  // the probes are ascending: the first cnt of them are below v
    if (cnt == 0) break;
    const int q1 = lo + (cnt - 1) * step;       // last probe below v: the answer lies in (q1, q1 + step]
    lo = q1 + 1;
    hi = min(q1 + step, hi);
  }
  return lo;
}

// Order of the n partial results of one (row, head) for the 16-lane group of `lane`: ord[r] = slot of the partial
// whose key-block id (ids[slot * stride]) has rank r in ascending order, equal ids ordered by slot.  n may differ
// between the four groups of a wave, nmax is the largest of them (the shuffles need all lanes).  Brute force: every
// lane ranks its slots li, li + 16, ... against all ids, 16 at a time through shuffles; a row of 32 visits costs 64
// comparisons per lane.  Ends with the group's LDS writes visible to its lanes.
__device__ __forceinline__ void group_rank_order(const int *ids, int stride, int n, int nmax, int *ord, int lane) {
  const int li = lane & 15;
  for (int j0 = 0; j0 < nmax; j0 += 16) {
    const int j = j0 + li;
    const int cj = j < n ? ids[(int64_t)j * stride] : 0x7fffffff;
    int rank = 0;
    for (int i0 = 0; i0 < nmax; i0 += 16) {
      const int cmine = (j0 == i0) ? cj : (i0 + li < n ? ids[(int64_t)(i0 + li) * stride] : 0x7fffffff);
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        const int ci = __shfl(cmine, (lane & 48) | t, 64);
        rank += (ci < cj || (ci == cj && i0 + t < j)) ? 1 : 0;
      }
    }
    if (j < n) ord[rank] = j;
  }
  wave_lds_fence();
}
// entries of a group's order list for rows of up to `cap` visits
static inline int combine_order_entries(int cap) { return ((cap > 0 ? cap : 1) + 15) / 16 * 16; }

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}): a loop whose index is a
// compile-time constant inside the body (register arrays, template arguments)
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// ------------------------------------------------------------------------------------
// Work items of a 1-D grid of npairs * nper workgroups, nper items per (sequence, head) pair.
// Workgroup i runs on XCD i % 8.  With a multiple of 8 pairs, pair p gets XCD p % 8 for all its
// items, so what the items of a pair share (its K / V, or the Q / dO rows that its key blocks
// gather again and again) stays in one L2; otherwise the items of a pair are simply consecutive.
// one_pair_at_a_time asks for the consecutive order in any case: when the rows a pair's items gather
// are far more than the L2s hold (kOnePairBytes and up), eight pairs at once also overflow the
// 256 MB memory-side cache, and the whole chip on one pair keeps that pair's rows in it
// (262144 tokens: dK/dV 20.9 -> 20.1 ms, forward columns 10.8 -> 10.3; at 32768 tokens, where
// an L2 still holds a good part of a pair, the same order costs 13 %).
// ------------------------------------------------------------------------------------
constexpr long long kOnePairBytes = 64ll << 20;
struct PairItem {
  int pair, idx;
};
__device__ __forceinline__ PairItem xcd_pair_item(int id, int npairs, int nper, bool one_pair_at_a_time = false) {
  PairItem w;
  if (npairs % 8 == 0 && !one_pair_at_a_time) {
    const int s = id >> 3;
    const int pl = s / nper;
    w.pair = pl * 8 + (id & 7);
    w.idx = s - pl * nper;
  } else {
    w.pair = id / nper;
    w.idx = id - w.pair * nper;
  }
  return w;
}

__device__ __forceinline__ Pack8 ld_global16(const void *p) { return *reinterpret_cast<const Pack8 *>(p); }
// Partial results (one per visit of a row, written by the column passes and added up by the combine kernels) go
// through the caches once in each direction: non-temporal stores and loads keep them from pushing the rows that
// the column passes gather again and again out of the caches (262144 tokens: dK/dV 20.0 -> 18.4 ms, forward
// columns 10.1 -> 9.6; 32768 tokens: step 9.95 -> 9.55 ms).  The dS tiles of the dS form were tried the same
// way: no difference on the headline batch (3.35-3.41 against 3.37-3.40 ms).
// 16 bytes that are read once: a non-temporal load
__device__ __forceinline__ Pack8 ld_stream16(const void *p) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const u32x4 x = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
  Pack8 r;
  r.w[0] = x[0];
  r.w[1] = x[1];
  r.w[2] = x[2];
  r.w[3] = x[3];
  return r;
}
// 16 bytes that are written once and read once by a later kernel: a non-temporal store
__device__ __forceinline__ void st_stream16(void *p, const Pack8 &v) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  u32x4 x = {v.w[0], v.w[1], v.w[2], v.w[3]};
  __builtin_nontemporal_store(x, reinterpret_cast<u32x4 *>(p));
}
__device__ __forceinline__ Pack8 zero_pack8() {
  Pack8 r;
  r.w[0] = r.w[1] = r.w[2] = r.w[3] = 0u;
  return r;
}

// ------------------------------------------------------------------------------------
// gathered tiles that global loads write straight into LDS: rows of exactly HD elements (one load
// instruction writes 64 lanes x 16 bytes to consecutive addresses), swizzled instead of padded
// ------------------------------------------------------------------------------------
// piece c of tile row r is stored at piece c ^ tile_swz<HD>(r)
template <int HD>
__device__ __forceinline__ int tile_swz(int r) {
  if constexpr (HD > 64)
    return ((r & 3) << 2) | ((r >> 2) & 3);  // 16 pieces per row, one row per sweep of the banks
  else
    return (((r >> 1) & 1) << 2) | ((r >> 2) & 1);  // 8 pieces per row, two rows per sweep
}
template <int HD>
struct TileSwz {
  static constexpr int kRow8 = HD > 64 ? 2 : 0;  // tile_swz(r + 8) ^ tile_swz(r)
};

// (read as ONE vector: as a struct of four words the read is split and put together again by what the compiler knows
// of the address bits, and where it knows nothing -- an address that comes out of an assembly statement, or round a
// loop -- it comes out as two 8-byte reads of 4-byte alignment, which meet in half of the banks)
__device__ __forceinline__ Pack8 lds_read16(uint32_t byte_addr) {
#if defined(__HIP_DEVICE_COMPILE__)
  const u32x4_t v = *(__attribute__((address_space(3))) const u32x4_t *)byte_addr;
  return Pack8{{v[0], v[1], v[2], v[3]}};
#else
  (void)byte_addr;
  return Pack8{{0, 0, 0, 0}};
#endif
}
template <typename V>
__device__ __forceinline__ V lds_read_vec(uint32_t byte_addr) {
#if defined(__HIP_DEVICE_COMPILE__)
  return *(__attribute__((address_space(3))) const V *)byte_addr;
#else
  (void)byte_addr;
  return V{};
#endif
}
template <typename V>
__device__ __forceinline__ void lds_write_vec(uint32_t byte_addr, const V &v) {
#if defined(__HIP_DEVICE_COMPILE__)
  *(__attribute__((address_space(3))) V *)byte_addr = v;
#else
  (void)byte_addr, (void)v;
#endif
}
// 8 x 16-bit operand of a transposing read: two 8-byte reads
__device__ __forceinline__ Pack8 lds_tr8(uint32_t addr_lo, uint32_t addr_hi) {
  Pack8 r;
#if defined(__HIP_DEVICE_COMPILE__)
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)addr_lo);
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)addr_hi);
  __builtin_memcpy(&r.w[0], &lo, 8);
  __builtin_memcpy(&r.w[2], &hi, 8);
#else
  (void)addr_lo, (void)addr_hi;
  r = Pack8{{0, 0, 0, 0}};
#endif
  return r;
}
// 64 lanes x 16 bytes from each lane's own global address to LDS bytes [lds_base, lds_base + 1024), lane order;
// lds_base is the same for the whole wave.  Written as assembly because the compiler makes every later LDS read wait
// for a load that it knows to write LDS, and these are meant to stay in flight for a whole round: the kernel waits for
// them itself (wait_all_loads) before the barrier that hands the tiles over.  m0 is not in the clobber list: the compiler reserves it, warns that such a
// clobber may not be honoured, and sets it itself right before each of its own instructions that read it.
__device__ __forceinline__ void global_to_lds16(const void *g, uint32_t lds_base) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_base) : "memory");
#else
  (void)g, (void)lds_base;
#endif
}
// The same load with the address split into a wave-uniform 64-bit base and a 32-bit byte offset per lane (unsigned):
// a tile whose rows lie at a fixed stride costs no vector instruction per load.
__device__ __forceinline__ void global_to_lds16_sbase(uint32_t lane_byte_off, const void *uniform_base, uint32_t lds_base) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_byte_off), "s"(uniform_base), "s"(lds_base) : "memory");
#else
  (void)lane_byte_off, (void)uniform_base, (void)lds_base;
#endif
}
__device__ __forceinline__ void wait_all_loads() {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
}
// The dS workspace of the backward (16-bit): tiles of 32 consecutive positions of the row-index array; inside a tile
// the 16-byte pieces (8 keys) of one key group of all 32 entries are contiguous:
//   [position / 32][key of the column / 8][position % 32][8 keys].
// The dK/dV pass writes a gathered tile (32 consecutive positions) in runs of consecutive pieces, and the dQ pass
// brings a run of positions into LDS one contiguous kilobyte (two key groups of a tile) per load instruction.
// Returns the element offset of piece (position p, key group kg); kgs = key groups per entry (column width / 8).
__host__ __device__ __forceinline__ int64_t ds_piece_offset(int64_t p, int kg, int kgs) { return ((((p >> 5) * kgs + kg) << 5) + (p & 31)) << 3; }
static inline size_t ds_workspace_tiles(int64_t positions) { return (size_t)((positions > 0 ? positions : 0) + 31) / 32 + 1; }

// Row id of a gathered tile row as it is kept in LDS: r itself if the entry is present and the row exists, else
// negative with a row that exists in the low 31 bits (the entry's own if it exists: past the end of a list that is the
// list's last row, whose data the column meets anyway; else row 0).  The tile loads fetch that row unconditionally, the
// arithmetic treats every negative id as absent.
__device__ __forceinline__ int tile_row_code(int r, bool present, int rows) {
  const bool exists = (r >= 0) & (r < rows);
  const int src = exists ? r : 0;
  return (present & exists) ? src : (int)((uint32_t)src | 0x80000000u);
}


}  // namespace fmoba
