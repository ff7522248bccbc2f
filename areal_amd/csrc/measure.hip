// Measurement helpers.  For the HBM-bound kernels: plain streams (read only, write only, copy) with either cache
// policy, which give the rates that this memory system sustains in each direction.  For the matrix cores: a loop that
// issues nothing but MFMAs on operands that never leave the registers.  What it sustains is the ceiling that this chip, at its power limit, sets for any bf16 tile GEMM (no LDS,
// no memory traffic, no epilogue), in the same sense in which k_copy16 is the measured ceiling of the HBM-bound kernels.
// Not on any product path.
#include "device_utils.h"

namespace aa {
namespace measure {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t mix(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

// eight bf16 values: zeros, or random sign and mantissa with exponents of 1/4 .. 1 (roughly what activations look like)
__device__ __forceinline__ bf16x8_t operand(bool random, uint32_t seed) {
  u32x4_t w;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    uint32_t lo = 0, hi = 0;
    if (random) {
      const uint32_t h = mix(seed * 4 + q);
      lo = (h & 0x807f) | ((125 + ((h >> 8) % 3)) << 7);
      hi = ((h >> 16) & 0x807f) | ((125 + ((h >> 28) % 3)) << 7);
    }
    w[q] = lo | (hi << 16);
  }
  return __builtin_bit_cast(bf16x8_t, w);
}

// 4 waves per workgroup, one per SIMD; per iteration a wave issues the MFMAs of one 16-wide (32 x 32 x 16 form) or
// 32-wide (16 x 16 x 32 form) k step of a 128 x 128 block: 16 MFMAs of 32768 flops or 64 MFMAs of 16384 flops, i.e.
// 524288 or 1048576 flops per wave and iteration.
__global__ __launch_bounds__(256) void k_mfma_32x32x16(float* __restrict__ out, int iters, int random) {
  const uint32_t id = blockIdx.x * 256 + threadIdx.x;
  bf16x8_t a[4], b[4];
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    a[x] = operand(random != 0, id * 8 + x);
    b[x] = operand(random != 0, id * 8 + 4 + x);
  }
  f32x16_t acc[4][4];
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[m][n][i] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int n = 0; n < 4; ++n) acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[m], b[n], acc[m][n], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) s += acc[m][n][i];
  out[id] = s;
}

__global__ __launch_bounds__(256) void k_mfma_16x16x32(float* __restrict__ out, int iters, int random) {
  const uint32_t id = blockIdx.x * 256 + threadIdx.x;
  bf16x8_t a[8], b[8];
#pragma unroll
  for (int x = 0; x < 8; ++x) {
    a[x] = operand(random != 0, id * 16 + x);
    b[x] = operand(random != 0, id * 16 + 8 + x);
  }
  f32x4_t acc[8][8];
#pragma unroll
  for (int m = 0; m < 8; ++m)
#pragma unroll
    for (int n = 0; n < 8; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[m][n][i] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
      for (int n = 0; n < 8; ++n) acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[m], b[n], acc[m][n], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int m = 0; m < 8; ++m)
#pragma unroll
    for (int n = 0; n < 8; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i) s += acc[m][n][i];
  out[id] = s;
}

// ---- HBM streams: read only, write only, copy ------------------------------------------------------------------------
// Every workgroup moves spans of kSpan pieces of 256 threads x 8 vectors of 16 bytes (a span is 512 KB of consecutive
// addresses, 1 KB per wave instruction, eight instructions in flight per lane), dealt round-robin: the way the
// row-per-workgroup kernels of the logits path walk memory.  NT selects the `nt` cache policy.  The read kernel folds
// what it reads into a word that is never equal to the magic value, so nothing is written.
constexpr int kU = 8;
constexpr int kSpan = 16;
constexpr int64_t kPieceVecs = 256 * kU;

template <bool NT>
__global__ __launch_bounds__(256) void k_stream_read(const u32x4_t* __restrict__ src, int64_t n_vec, uint32_t* sink) {
  u32x4_t acc = {0u, 0u, 0u, 0u};
  for (int64_t sp = blockIdx.x; sp * (kSpan * kPieceVecs) < n_vec; sp += gridDim.x) {
    for (int j = 0; j < kSpan; ++j) {
      const int64_t at = (sp * kSpan + j) * kPieceVecs + threadIdx.x;
      if (at - threadIdx.x >= n_vec) break;
      u32x4_t v[kU];
#pragma unroll
      for (int i = 0; i < kU; ++i) {
        const u32x4_t* q = at + i * 256 < n_vec ? src + at + i * 256 : src;
        v[i] = NT ? __builtin_nontemporal_load(q) : *q;
      }
#pragma unroll
      for (int i = 0; i < kU; ++i) acc ^= v[i];
    }
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5a17c0deu && sink) sink[0] = acc[0];
}

template <bool NT>
__global__ __launch_bounds__(256) void k_stream_write(u32x4_t* __restrict__ dst, int64_t n_vec) {
  const u32x4_t v = {threadIdx.x, blockIdx.x, 2u, 3u};
  for (int64_t sp = blockIdx.x; sp * (kSpan * kPieceVecs) < n_vec; sp += gridDim.x) {
    for (int j = 0; j < kSpan; ++j) {
      const int64_t at = (sp * kSpan + j) * kPieceVecs + threadIdx.x;
      if (at - threadIdx.x >= n_vec) break;
#pragma unroll
      for (int i = 0; i < kU; ++i) {
        if (at + i * 256 < n_vec) {
          if (NT) __builtin_nontemporal_store(v, dst + at + i * 256);
          else dst[at + i * 256] = v;
        }
      }
    }
  }
}

template <bool NT>
__global__ __launch_bounds__(256) void k_stream_copy(const u32x4_t* __restrict__ src, u32x4_t* __restrict__ dst, int64_t n_vec) {
  for (int64_t sp = blockIdx.x; sp * (kSpan * kPieceVecs) < n_vec; sp += gridDim.x) {
    for (int j = 0; j < kSpan; ++j) {
      const int64_t at = (sp * kSpan + j) * kPieceVecs + threadIdx.x;
      if (at - threadIdx.x >= n_vec) break;
      u32x4_t v[kU];
#pragma unroll
      for (int i = 0; i < kU; ++i) {
        const u32x4_t* q = at + i * 256 < n_vec ? src + at + i * 256 : src;
        v[i] = NT ? __builtin_nontemporal_load(q) : *q;
      }
#pragma unroll
      for (int i = 0; i < kU; ++i) {
        if (at + i * 256 < n_vec) {
          if (NT) __builtin_nontemporal_store(v[i], dst + at + i * 256);
          else dst[at + i * 256] = v[i];
        }
      }
    }
  }
}

}  // namespace measure
}  // namespace aa

using namespace aa;

extern "C" int aa_hbm_stream_probe(int kind, int nt_policy, const void* src, void* dst, int64_t bytes, int workgroups,
                                   void* stream) {
  if (kind < 0 || kind > 2 || bytes <= 0 || bytes % 16 != 0 || workgroups <= 0 || workgroups > 65536) return AA_ERR_INVALID_ARGUMENT;
  if ((kind != 1 && (!src || ((uintptr_t)src & 15))) || (kind != 0 && (!dst || ((uintptr_t)dst & 15)))) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  const int64_t n_vec = bytes / 16;
  const dim3 grid((unsigned)workgroups), block(256);
  typedef measure::u32x4_t vec;
  if (kind == 0) {
    if (nt_policy) hipLaunchKernelGGL(measure::k_stream_read<true>, grid, block, 0, st, (const vec*)src, n_vec, (uint32_t*)dst);
    else hipLaunchKernelGGL(measure::k_stream_read<false>, grid, block, 0, st, (const vec*)src, n_vec, (uint32_t*)dst);
  } else if (kind == 1) {
    if (nt_policy) hipLaunchKernelGGL(measure::k_stream_write<true>, grid, block, 0, st, (vec*)dst, n_vec);
    else hipLaunchKernelGGL(measure::k_stream_write<false>, grid, block, 0, st, (vec*)dst, n_vec);
  } else {
    if (nt_policy) hipLaunchKernelGGL(measure::k_stream_copy<true>, grid, block, 0, st, (const vec*)src, (vec*)dst, n_vec);
    else hipLaunchKernelGGL(measure::k_stream_copy<false>, grid, block, 0, st, (const vec*)src, (vec*)dst, n_vec);
  }
  return launch_status();
}

extern "C" int aa_mfma_only_loop(int form, int random_operands, int workgroups, int iters, float* out, void* stream) {
  if (!out || workgroups <= 0 || workgroups > 65536 || iters <= 0 || (form != 0 && form != 1)) return AA_ERR_INVALID_ARGUMENT;
  if (form == 0)
    hipLaunchKernelGGL(measure::k_mfma_32x32x16, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream, out, iters,
                       random_operands);
  else
    hipLaunchKernelGGL(measure::k_mfma_16x16x32, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream, out, iters,
                       random_operands);
  return launch_status();
}
