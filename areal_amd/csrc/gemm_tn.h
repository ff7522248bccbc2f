// bf16 "TN" tile GEMM on gfx950 matrix cores:  D[m][n] = sum_k A[m][k] * B[n][k]
// with A [M, K] and B [N, K] both row-major (K contiguous), fp32 accumulation.
//
// One workgroup of 256 threads (4 waves, 2 x 2) computes a 256 x 256 tile of D
// with v_mfma_f32_32x32x16_bf16; each wave owns 128 x 128 = 4 x 4 MFMA tiles
// (256 accumulator registers).  Operands are staged through LDS in 64-wide K
// slices, double buffered, with the next slice's global loads in flight while
// the current one is multiplied.  What happens to the accumulators is decided
// by an epilogue functor, so the same main loop serves the lm_head forward
// statistics, the d(logits) recompute and the two gradient GEMMs.
//
// Register layout of one 32 x 32 x 16 MFMA (checked on the hardware):
//   A operand, lane l: A[m = l % 32][k = 8 (l / 32) + j], j = 0..7
//   B operand, lane l: B[n = l % 32][k = 8 (l / 32) + j]
//   D, lane l, register i: n = l % 32, m = 8 (i / 4) + 4 (l / 32) + i % 4
// i.e. a lane owns one column n of D and 16 of its rows m: row-wise (over m)
// reductions for a fixed n stay inside a lane.
#pragma once
#include "device_utils.h"

namespace aa {
namespace gemm {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kThreads = 256;
constexpr int kPitch = BK + 8;               // LDS row pitch in elements (144 B): conflict-free 16-byte reads
constexpr int kTileElems = 256 * kPitch;     // one operand, one stage
constexpr int kLdsBytes = 2 * 2 * kTileElems * 2;  // 2 stages x (A, B) x bf16 = 147456 B

// Accumulators of one wave: acc[mt][nt] is the 32 x 32 tile at rows mt * 32, columns nt * 32 of its 128 x 128 block.
struct Acc {
  f32x16_t v[4][4];
};

// row (m) and column (n) inside the wave's 128 x 128 block of accumulator element (mt, nt, i) of lane `lane`
__device__ __forceinline__ int acc_row(int mt, int i, int lane) { return mt * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3); }
__device__ __forceinline__ int acc_col(int nt, int lane) { return nt * 32 + (lane & 31); }

// Tile order: the hardware deals consecutive workgroup ids to the 8 XCDs in
// turn.  Ids are first regrouped so that each XCD gets a contiguous range, and
// that range then walks the tile grid in bands of `kGroupM` tile rows, so that
// tiles that run at the same time on one XCD share A and B slices in its L2.
constexpr int kGroupM = 8;
// The XCD regrouping above is a bijection only when the tile count is a multiple of 8; otherwise use the plain order.
__device__ __forceinline__ void tile_of(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  int q = pid;
  if ((total & 7) == 0) q = (pid & 7) * (total >> 3) + (pid >> 3);
  const int in_group = kGroupM * tiles_n;
  const int g = q / in_group;
  const int first_m = g * kGroupM;
  const int gsz = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
  tm = first_m + (q % in_group) % gsz;
  tn = (q % in_group) / gsz;
}

struct Operand {
  const uint16_t* ptr;  // bf16 bits
  int64_t ld;           // row stride in elements
  int rows;             // valid rows (rows beyond are clamped on load; the epilogue masks them)
};

// Main loop.  Leaves the result in `acc`; `lds` is kLdsBytes of dynamic shared memory.
__device__ __forceinline__ void mainloop(const Operand& A, const Operand& B, int K, int m0, int n0, Acc& acc,
                                         uint16_t* lds) {
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  uint16_t* As = lds;                    // [2][256][kPitch]
  uint16_t* Bs = lds + 2 * kTileElems;   // [2][256][kPitch]

  // global -> register staging: thread t covers rows t / 8 + 32 j (j = 0..7), 8 elements at column (t % 8) * 8
  const int ld_row = tid >> 3, ld_col = (tid & 7) * 8;
  const uint16_t* a_ptr[8];
  const uint16_t* b_ptr[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    int ra = m0 + ld_row + 32 * j; if (ra > A.rows - 1) ra = A.rows - 1;
    int rb = n0 + ld_row + 32 * j; if (rb > B.rows - 1) rb = B.rows - 1;
    a_ptr[j] = A.ptr + (int64_t)ra * A.ld + ld_col;
    b_ptr[j] = B.ptr + (int64_t)rb * B.ld + ld_col;
  }
  u32x4_t sa[8], sb[8];
  auto g_load = [&](int k0) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      sa[j] = *(const u32x4_t*)(a_ptr[j] + k0);
      sb[j] = *(const u32x4_t*)(b_ptr[j] + k0);
    }
  };
  auto s_store = [&](int stage) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int off = stage * kTileElems + (ld_row + 32 * j) * kPitch + ld_col;
      *(u32x4_t*)(As + off) = sa[j];
      *(u32x4_t*)(Bs + off) = sb[j];
    }
  };

#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc.v[mt][nt][i] = 0.f;

  // fragment addresses: row (lane % 32) of sub-tile, 8 elements at column 8 (lane / 32) of each 16-wide k step
  const int fa_off = (wm * 128 + (lane & 31)) * kPitch + 8 * (lane >> 5);
  const int fb_off = (wn * 128 + (lane & 31)) * kPitch + 8 * (lane >> 5);

  const int nk = K / BK;
  g_load(0);
  s_store(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) g_load((kt + 1) * BK);
    const uint16_t* as = As + cur * kTileElems + fa_off;
    const uint16_t* bs = Bs + cur * kTileElems + fb_off;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8_t fa[4], fb[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        fa[x] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(as + x * 32 * kPitch + kk * 16));
        fb[x] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(bs + x * 32 * kPitch + kk * 16));
      }
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
          acc.v[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[mt], fb[nt], acc.v[mt][nt], 0, 0, 0);
    }
    if (kt + 1 < nk) s_store(cur ^ 1);
    __syncthreads();
  }
}

}  // namespace gemm
}  // namespace aa
