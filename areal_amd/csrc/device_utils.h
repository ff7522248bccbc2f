// Device helpers shared by the gfx950 kernels: 16-bit float packing, wave64 and
// workgroup reductions, and the (max, sum-exp, sum x*exp) softmax partials.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <float.h>

#include "../../include/areal_amd.h"

namespace aa {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// Finite stand-in for "no element seen yet": exp2((kNegBig - m) * c) is 0 for
// every finite m, and 0 * kNegBig stays finite (no NaN from inf * 0).
constexpr float kNegBig = -3.0e38f;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// ---- 16-bit element access: DT is an aa_dtype value -------------------------
template <int DT>
struct Elem;

template <>
struct Elem<AA_BF16> {
  typedef uint16_t storage;
  static constexpr int kBytes = 2;
  __device__ static __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
  __device__ static __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
  __device__ static __forceinline__ float load1(const void* p, int64_t i) {
    return __uint_as_float(((uint32_t)((const uint16_t*)p)[i]) << 16);
  }
  __device__ static __forceinline__ uint32_t pack(float a, float b) {
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  }
  __device__ static __forceinline__ void store1(void* p, int64_t i, float v) {
    ((uint16_t*)p)[i] = (uint16_t)(pack(v, 0.f) & 0xffffu);
  }
};

template <>
struct Elem<AA_F16> {
  typedef uint16_t storage;
  static constexpr int kBytes = 2;
  __device__ static __forceinline__ float lo(uint32_t w) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
  }
  __device__ static __forceinline__ float hi(uint32_t w) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
  }
  __device__ static __forceinline__ float load1(const void* p, int64_t i) {
    return (float)((const _Float16*)p)[i];
  }
  __device__ static __forceinline__ uint32_t pack(float a, float b) {
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
  }
  __device__ static __forceinline__ void store1(void* p, int64_t i, float v) {
    ((_Float16*)p)[i] = (_Float16)v;
  }
};

template <>
struct Elem<AA_F32> {
  typedef float storage;
  static constexpr int kBytes = 4;
  __device__ static __forceinline__ float load1(const void* p, int64_t i) { return ((const float*)p)[i]; }
  __device__ static __forceinline__ void store1(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
};

// Eight consecutive elements starting at element index i (i * kBytes must be
// 16-byte aligned relative to an aligned base).
template <int DT>
__device__ __forceinline__ void load8(const void* base, int64_t i, float (&x)[8]) {
  if constexpr (DT == AA_F32) {
    const float4* p = (const float4*)((const float*)base + i);
    float4 a = p[0], b = p[1];
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
  } else {
    uint4 q = *(const uint4*)((const uint16_t*)base + i);
    x[0] = Elem<DT>::lo(q.x); x[1] = Elem<DT>::hi(q.x);
    x[2] = Elem<DT>::lo(q.y); x[3] = Elem<DT>::hi(q.y);
    x[4] = Elem<DT>::lo(q.z); x[5] = Elem<DT>::hi(q.z);
    x[6] = Elem<DT>::lo(q.w); x[7] = Elem<DT>::hi(q.w);
  }
}

// The same with the `nt` cache policy: for data that is read once (a read-only pass over a large array sustains
// 7.1 TB/s with it against 6.3 TB/s without on this part).
template <int DT>
__device__ __forceinline__ void load8_stream(const void* base, int64_t i, float (&x)[8]) {
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  if constexpr (DT == AA_F32) {
    const u32x4_t* p = (const u32x4_t*)((const float*)base + i);
    const u32x4_t a = __builtin_nontemporal_load(p), b = __builtin_nontemporal_load(p + 1);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      x[q] = __uint_as_float(a[q]);
      x[4 + q] = __uint_as_float(b[q]);
    }
  } else {
    const u32x4_t q = __builtin_nontemporal_load((const u32x4_t*)((const uint16_t*)base + i));
    x[0] = Elem<DT>::lo(q[0]); x[1] = Elem<DT>::hi(q[0]);
    x[2] = Elem<DT>::lo(q[1]); x[3] = Elem<DT>::hi(q[1]);
    x[4] = Elem<DT>::lo(q[2]); x[5] = Elem<DT>::hi(q[2]);
    x[6] = Elem<DT>::lo(q[3]); x[7] = Elem<DT>::hi(q[3]);
  }
}

// four consecutive fp32 values at a 16-byte aligned address, `nt` policy
__device__ __forceinline__ void load4_stream(const float* p, float* x) {
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  const u32x4_t a = __builtin_nontemporal_load((const u32x4_t*)p);
#pragma unroll
  for (int q = 0; q < 4; ++q) x[q] = __uint_as_float(a[q]);
}

__device__ __forceinline__ void store4_stream(float* p, const float* x) {
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  const u32x4_t v = {__float_as_uint(x[0]), __float_as_uint(x[1]), __float_as_uint(x[2]), __float_as_uint(x[3])};
  __builtin_nontemporal_store(v, (u32x4_t*)p);
}

// eight 16-bit values to consecutive addresses, `nt` policy
template <int DT>
__device__ __forceinline__ void store8_stream16(void* base, int64_t i, const float (&x)[8]) {
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  const u32x4_t q = {Elem<DT>::pack(x[0], x[1]), Elem<DT>::pack(x[2], x[3]), Elem<DT>::pack(x[4], x[5]),
                     Elem<DT>::pack(x[6], x[7])};
  __builtin_nontemporal_store(q, (u32x4_t*)((uint16_t*)base + i));
}

template <int DT>
__device__ __forceinline__ void store8(void* base, int64_t i, const float (&x)[8]) {
  if constexpr (DT == AA_F32) {
    float4* p = (float4*)((float*)base + i);
    p[0] = make_float4(x[0], x[1], x[2], x[3]);
    p[1] = make_float4(x[4], x[5], x[6], x[7]);
  } else {
    uint4 q;
    q.x = Elem<DT>::pack(x[0], x[1]);
    q.y = Elem<DT>::pack(x[2], x[3]);
    q.z = Elem<DT>::pack(x[4], x[5]);
    q.w = Elem<DT>::pack(x[6], x[7]);
    *(uint4*)((uint16_t*)base + i) = q;
  }
}

// ---- extrema of a few values ------------------------------------------------
// IEEE 754-2019 maximum / minimum (a NaN input gives NaN, as torch.max does) on the three-input instructions of
// gfx950.  fmaxf / fminf would first pass every value that comes straight out of a load or a shift through a
// canonicalising v_max_f32 x, x: one more instruction per element in loops that are bound by their instructions.
__device__ __forceinline__ float max3(float a, float b, float c) {
  return __builtin_elementwise_maximum(__builtin_elementwise_maximum(a, b), c);
}
__device__ __forceinline__ float min3(float a, float b, float c) {
  return __builtin_elementwise_minimum(__builtin_elementwise_minimum(a, b), c);
}
template <int N>
__device__ __forceinline__ float max_of(const float* x) {
  static_assert(N == 4 || N == 8, "four or eight values");
  if constexpr (N == 4) return max3(max3(x[0], x[1], x[2]), x[3], x[3]);
  else return max3(max3(x[0], x[1], x[2]), max3(x[3], x[4], x[5]), __builtin_elementwise_maximum(x[6], x[7]));
}
template <int N>
__device__ __forceinline__ float min_of(const float* x) {
  static_assert(N == 4 || N == 8, "four or eight values");
  if constexpr (N == 4) return min3(min3(x[0], x[1], x[2]), x[3], x[3]);
  else return min3(min3(x[0], x[1], x[2]), min3(x[3], x[4], x[5]), __builtin_elementwise_minimum(x[6], x[7]));
}

// ---- wave64 reductions -------------------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, kWave));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ int wave_sum(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

inline int launch_status() { return hipGetLastError() == hipSuccess ? AA_OK : AA_ERR_LAUNCH; }

}  // namespace aa
