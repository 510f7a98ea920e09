// Device-side building blocks shared by the reduction kernels (gfx950): the
// 16-byte vector types, streaming loads and stores, and the storage traits
// that say how elements of each type are unpacked into accumulators and packed
// back.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fairring_hip.h"
#include "ksum_kernels.h"

// Launch shape, chosen by measurement on MI355X with K = 8 fp32 and 25 MiB
// slices: 128-thread blocks, two vectors per lane (a tile of 4 KiB per
// contribution), and a small persistent grid. A small grid keeps the window of
// addresses in flight narrow (a few MiB per contribution), which the HBM
// controllers reward with more row hits; what covers the latency is the 16
// independent 16-byte loads per lane, not the wave count. Non-temporal
// loads are worth ~7 %, non-temporal stores ~3 %.
#ifndef FRG_BLOCK
#define FRG_BLOCK 128
#endif
#ifndef FRG_UNROLL
#define FRG_UNROLL 2
#endif
#ifndef FRG_NONTEMPORAL
#define FRG_NONTEMPORAL 1
#endif
// Vectors per lane in a piece of the remainder round (1 = pieces of kBlock
// vectors, spread over the most blocks; FRG_UNROLL = whole tiles).
#ifndef FRG_REMAINDER_PIECE_UNROLL
#define FRG_REMAINDER_PIECE_UNROLL 1
#endif
// Loads in flight per CU that the grid is sized for: blocks per CU =
// FRG_LOADS_PER_CU / (loads per lane), so that fewer contributions per launch
// are made up for by more resident waves.
#ifndef FRG_LOADS_PER_CU
#define FRG_LOADS_PER_CU 32
#endif

namespace frg {
namespace {

constexpr int kBlock = FRG_BLOCK;
constexpr int kUnroll = FRG_UNROLL;
// Tiles start on a multiple of this many bytes of the first contribution (the
// default tile: 128 lanes x 2 vectors x 16 bytes).
constexpr uintptr_t kLaunchAlignBytes = 4096;
constexpr int kChunk = 8;  // contributions loaded together in the runtime-K path

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename V>
__device__ __forceinline__ V ldStream(const V* p) {
#if FRG_NONTEMPORAL
  return __builtin_nontemporal_load(p);
#else
  return *p;
#endif
}

template <typename V>
__device__ __forceinline__ void stStream(V v, V* p) {
#if FRG_NONTEMPORAL
  __builtin_nontemporal_store(v, p);
#else
  *p = v;
#endif
}

__device__ __forceinline__ float bitsToFloat(unsigned int u) {
  return __builtin_bit_cast(float, u);
}

// fp32 -> bf16 bits, round to nearest even, NaN -> 0x7FC0 (as ATen). gfx950
// converts in hardware (v_cvt_pk_bf16_f32, two values per instruction); the NaN
// pattern is fixed up afterwards.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ unsigned int f32PairToBf16Rne(float lo, float hi) {
  f32x2 v;
  v[0] = lo;
  v[1] = hi;
  unsigned int r = __builtin_bit_cast(unsigned int, __builtin_convertvector(v, bf16x2));
  if (lo != lo) r = (r & 0xFFFF0000u) | 0x7FC0u;
  if (hi != hi) r = (r & 0x0000FFFFu) | 0x7FC00000u;
  return r;
}

__device__ __forceinline__ unsigned int f32ToBf16Rne(float f) {
  const unsigned short r = __builtin_bit_cast(unsigned short, static_cast<__bf16>(f));
  return (f != f) ? 0x7FC0u : static_cast<unsigned int>(r);
}

// ---- storage traits: how a "vector" of elements is loaded and unpacked ------
//
// elem_t: storage element; vec_t: what one lane loads (16 bytes in the vector
// variants, one element in the scalar ones); acc_t: the type the fold runs in
// (fp32 for fp32/bf16/fp16 as ATen accumulates them, fp64 for fp64, the
// element's own width with wrap-around for integers).

struct F32Vec {
  using elem_t = float;
  using vec_t = f32x4;
  using acc_t = float;
  static constexpr int kLanes = 4;
  static constexpr bool kFloating = true;
  __device__ static void unpack(const vec_t& v, acc_t (&f)[kLanes]) {
    f[0] = v[0]; f[1] = v[1]; f[2] = v[2]; f[3] = v[3];
  }
  __device__ static vec_t pack(const acc_t (&f)[kLanes]) {
    vec_t v;
    v[0] = f[0]; v[1] = f[1]; v[2] = f[2]; v[3] = f[3];
    return v;
  }
  // an accumulator value rounded to the storage type and widened again
  __device__ static acc_t roundStorage(acc_t f) { return f; }
};

struct F32Scalar {
  using elem_t = float;
  using vec_t = float;
  using acc_t = float;
  static constexpr int kLanes = 1;
  static constexpr bool kFloating = true;
  __device__ static void unpack(const vec_t& v, acc_t (&f)[kLanes]) { f[0] = v; }
  __device__ static vec_t pack(const acc_t (&f)[kLanes]) { return f[0]; }
  __device__ static acc_t roundStorage(acc_t f) { return f; }
};

struct Bf16Vec {  // 8 bf16 in 16 bytes
  using elem_t = unsigned short;
  using vec_t = u32x4;
  using acc_t = float;
  static constexpr int kLanes = 8;
  static constexpr bool kFloating = true;
  __device__ static void unpack(const vec_t& v, acc_t (&f)[kLanes]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = bitsToFloat(v[j] << 16);
      f[2 * j + 1] = bitsToFloat(v[j] & 0xFFFF0000u);
    }
  }
  __device__ static vec_t pack(const acc_t (&f)[kLanes]) {
    vec_t v;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[j] = f32PairToBf16Rne(f[2 * j], f[2 * j + 1]);
    }
    return v;
  }
  __device__ static acc_t roundStorage(acc_t f) { return bitsToFloat(f32ToBf16Rne(f) << 16); }
};

struct Bf16Scalar {
  using elem_t = unsigned short;
  using vec_t = unsigned short;
  using acc_t = float;
  static constexpr int kLanes = 1;
  static constexpr bool kFloating = true;
  __device__ static void unpack(const vec_t& v, acc_t (&f)[kLanes]) {
    f[0] = bitsToFloat(static_cast<unsigned int>(v) << 16);
  }
  __device__ static vec_t pack(const acc_t (&f)[kLanes]) {
    return static_cast<unsigned short>(f32ToBf16Rne(f[0]));
  }
  __device__ static acc_t roundStorage(acc_t f) { return bitsToFloat(f32ToBf16Rne(f) << 16); }
};

// Conversions between fp16 storage and fp32 accumulators go through here. The
// value is made opaque on the fp32 side, which keeps the compiler from folding a
// neighbouring multiply into the conversion as a mixed-precision fma with a +0
// addend (v_fma_mix*): that instruction turns a product of -0 into +0, where
// ATen, and the multiply followed by the conversion, keep the sign.
template <typename A, typename E>
__device__ __forceinline__ A widenElem(E e) {
  A a = static_cast<A>(e);
  if constexpr (sizeof(E) == 2 && sizeof(A) == 4) asm("" : "+v"(a));
  return a;
}

template <typename E, typename A>
__device__ __forceinline__ E narrowElem(A a) {
  if constexpr (sizeof(E) == 2 && sizeof(A) == 4) asm("" : "+v"(a));
  return static_cast<E>(a);
}

// Element-wise traits for types whose vector is an ext_vector of the element:
// convert up on unpack, down (round to nearest even for fp16, wrap-around for
// integers) on pack.
template <typename E, typename A, int LANES, bool FLOATING>
struct PlainVec {
  using elem_t = E;
  typedef E vec_t __attribute__((ext_vector_type(LANES)));
  using acc_t = A;
  static constexpr int kLanes = LANES;
  static constexpr bool kFloating = FLOATING;
  __device__ static void unpack(const vec_t& v, acc_t (&f)[kLanes]) {
#pragma unroll
    for (int j = 0; j < LANES; ++j) f[j] = widenElem<A, E>(v[j]);
  }
  __device__ static vec_t pack(const acc_t (&f)[kLanes]) {
    vec_t v;
#pragma unroll
    for (int j = 0; j < LANES; ++j) v[j] = narrowElem<E, A>(f[j]);
    return v;
  }
  __device__ static acc_t roundStorage(acc_t f) { return widenElem<A, E>(narrowElem<E, A>(f)); }
};

template <typename E, typename A, bool FLOATING>
struct PlainScalar {
  using elem_t = E;
  using vec_t = E;
  using acc_t = A;
  static constexpr int kLanes = 1;
  static constexpr bool kFloating = FLOATING;
  __device__ static void unpack(const vec_t& v, acc_t (&f)[kLanes]) { f[0] = widenElem<A, E>(v); }
  __device__ static vec_t pack(const acc_t (&f)[kLanes]) { return narrowElem<E, A>(f[0]); }
  __device__ static acc_t roundStorage(acc_t f) { return widenElem<A, E>(narrowElem<E, A>(f)); }
};

using F16Vec = PlainVec<_Float16, float, 8, true>;
using F16Scalar = PlainScalar<_Float16, float, true>;
using F64Vec = PlainVec<double, double, 2, true>;
using F64Scalar = PlainScalar<double, double, true>;
// Integers fold in an unsigned type of the element's width or wider (sums wrap
// like two's complement); the maximum compares in the element's own signedness.
using I32Vec = PlainVec<int, int, 4, false>;
using I32Scalar = PlainScalar<int, int, false>;
using I64Vec = PlainVec<long long, long long, 2, false>;
using I64Scalar = PlainScalar<long long, long long, false>;
using U8Vec = PlainVec<unsigned char, unsigned int, 16, false>;
using U8Scalar = PlainScalar<unsigned char, unsigned int, false>;
using I8Vec = PlainVec<signed char, int, 16, false>;
using I8Scalar = PlainScalar<signed char, int, false>;

__device__ __forceinline__ int addWrap(int a, int b) {
  return static_cast<int>(static_cast<unsigned int>(a) + static_cast<unsigned int>(b));
}
__device__ __forceinline__ long long addWrap(long long a, long long b) {
  return static_cast<long long>(static_cast<unsigned long long>(a) +
                                static_cast<unsigned long long>(b));
}
__device__ __forceinline__ unsigned int addWrap(unsigned int a, unsigned int b) { return a + b; }
__device__ __forceinline__ float addWrap(float a, float b) { return a + b; }
__device__ __forceinline__ double addWrap(double a, double b) { return a + b; }

template <int OP, typename A>
__device__ __forceinline__ A combine(A a, A b) {
  if (OP == FRG_SUM) {
    return addWrap(a, b);
  } else {
    // maximum with NaN propagation, as at::amax (the NaN tests fold away for integers)
    return (a != a) ? a : ((b != b) ? b : (a > b ? a : b));
  }
}

// Pointer table passed by value in the kernel arguments: no dependent load
// sits between the launch and the first data load.
template <int KT>
struct Ptrs {
  const void* p[KT > 0 ? KT : kMaxContribsPerLaunch];
};

// fp32 values for a lane's elements of a 2-byte type (a raw fp32 bucket, or
// accumulators parked between two launches): 8 floats as two vectors, or one
// float in the element-wise variants.
template <int LANES>
struct Fp32Side;

template <>
struct Fp32Side<8> {
  struct regs_t {
    f32x4 a, b;
  };
  __device__ static regs_t load(const float* base, unsigned int lane) {
    const f32x4* p = reinterpret_cast<const f32x4*>(reinterpret_cast<const char*>(base) + lane * 32u);
    regs_t r;
    r.a = ldStream(p);
    r.b = ldStream(p + 1);
    return r;
  }
  __device__ static void unpack(const regs_t& r, float (&f)[8]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[j] = r.a[j];
      f[4 + j] = r.b[j];
    }
  }
  __device__ static void store(float* base, unsigned int lane, const float (&f)[8]) {
    f32x4* p = reinterpret_cast<f32x4*>(reinterpret_cast<char*>(base) + lane * 32u);
    f32x4 a, b;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      a[j] = f[j];
      b[j] = f[4 + j];
    }
    stStream(a, p);
    stStream(b, p + 1);
  }
};

template <>
struct Fp32Side<1> {
  struct regs_t {
    float a;
  };
  __device__ static regs_t load(const float* base, unsigned int lane) {
    regs_t r;
    r.a = ldStream(base + lane);
    return r;
  }
  __device__ static void unpack(const regs_t& r, float (&f)[1]) { f[0] = r.a; }
  __device__ static void store(float* base, unsigned int lane, const float (&f)[1]) {
    stStream(f[0], base + lane);
  }
};

}  // namespace
}  // namespace frg
