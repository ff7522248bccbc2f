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
constexpr int kRowBytes = BK * 2;               // one row of a K slice in LDS: 128 B = 8 chunks of 16 B, no padding
constexpr int kTileBytes = 256 * kRowBytes;     // one operand, one stage: 32 KiB
constexpr int kLdsBytes = 2 * 2 * kTileBytes;   // 2 stages x (A, B) = 128 KiB

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
constexpr int kGroupM = 4;
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

constexpr int kBufferFlags = 0x00020000;  // raw buffer descriptor, 32-bit data format

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// Main loop.  Leaves the result in `acc`; `lds` is kLdsBytes of dynamic shared memory.
//
// K slices of 64 go from global memory straight into LDS (buffer_load ... lds: lane i of a wave deposits its 16
// bytes at the wave's LDS base + 16 i), so no staging registers and no LDS store instructions are spent on them.
// A slice of one operand is 256 rows x 128 B, held without padding as 32 blocks of 1 KiB (8 rows each); inside a
// row the eight 16-byte chunks are XOR-swizzled, chunk c of row r at slot c ^ ((r >> 1) & 7): with this key the
// 16-byte fragment reads of a wave (32 rows x 2 chunks) run at the full LDS rate (measured 125 B/clk per CU against
// 87 B/clk with the key r & 7).  The swizzle costs nothing: each lane simply
// fetches the global chunk that belongs at its slot.  Buffer descriptors cover exactly the valid rows of the tile
// (rows past the end of an operand read as zero).  LDS holds two slices; fragments are double buffered in
// registers, so that the 8 fragment loads of the next 16-wide k step are in flight during the 16 MFMAs of this one.
__device__ __forceinline__ void mainloop(const Operand& A, const Operand& B, int K, int m0, int n0, Acc& acc,
                                         uint16_t* lds) {
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  char* As = (char*)lds;                   // [2][256][128 B]
  char* Bs = (char*)lds + 2 * kTileBytes;  // [2][256][128 B]

  // Loading: block b = 4 j + wave (j = 0..7) holds rows 8 b .. 8 b + 7; lane l brings row r = 8 b + l / 8 and puts
  // global chunk (l % 8) ^ ((r >> 1) & 7) at slot l % 8; (r >> 1) & 7 = (4 (wave & 1) + l / 16) & 7 for every j.
  const int ld_row = 8 * wave + (lane >> 3);
  const int ld_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);  // ((row >> 1) & 7) of the row this lane brings
  const int rows_a = (A.rows - m0) < BM ? (A.rows - m0) : BM;
  const int rows_b = (B.rows - n0) < BN ? (B.rows - n0) : BN;
  const uint16_t* a_base = A.ptr + (int64_t)m0 * A.ld;
  const uint16_t* b_base = B.ptr + (int64_t)n0 * B.ld;
  const int a_voff = (int)(((int64_t)ld_row * A.ld + ld_chunk * 8) * 2);
  const int b_voff = (int)(((int64_t)ld_row * B.ld + ld_chunk * 8) * 2);
  const int a_jstep = (int)(32 * A.ld * 2), b_jstep = (int)(32 * B.ld * 2);
  const int a_bytes = (int)((int64_t)rows_a * A.ld * 2), b_bytes = (int)((int64_t)rows_b * B.ld * 2);

  auto g_load = [&](int stage, int k0) {
    // the descriptor starts at column k0, so row r is in range iff r < rows (the last row may end early, never late)
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)(a_base + k0), 0, a_bytes - k0 * 2, kBufferFlags);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)(b_base + k0), 0, b_bytes - k0 * 2, kBufferFlags);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int blk = stage * kTileBytes + (4 * j + wave) * 1024;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(As + blk), 16, a_voff, j * a_jstep, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(Bs + blk), 16, b_voff, j * b_jstep, 0, 0);
    }
  };

#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc.v[mt][nt][i] = 0.f;

  // Fragment of sub-tile x at k step kk: row r = w * 128 + 32 x + lane % 32, global chunk 2 kk + lane / 32, found at
  // slot (2 kk + lane / 32) ^ ((r >> 1) & 7); (r >> 1) & 7 = (lane >> 1) & 7 because the other terms are multiples of 16.
  const int fr_a = (wm * 128 + (lane & 31)) * kRowBytes;
  const int fr_b = (wn * 128 + (lane & 31)) * kRowBytes;
  const int half = lane >> 5, r7 = (lane >> 1) & 7;
  bf16x8_t fa[2][4], fb[2][4];
  auto f_load = [&](int buf, const char* as, const char* bs, int kk) {
    const int slot = (((2 * kk + half) ^ r7) << 4);
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      fa[buf][x] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(as + fr_a + x * 32 * kRowBytes + slot));
      fb[buf][x] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(bs + fr_b + x * 32 * kRowBytes + slot));
    }
  };

  const int nk = K / BK;
  g_load(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of the slice has landed
  __syncthreads();
  f_load(0, As, Bs, 0);
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < nk;
    if (more) g_load(cur ^ 1, (kt + 1) * BK);  // the other stage was released by the barrier that ended slice kt - 1
    const char* as = As + cur * kTileBytes;
    const char* bs = Bs + cur * kTileBytes;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      const int buf = kk & 1;
      if (kk + 1 < BK / 16) f_load(buf ^ 1, as, bs, kk + 1);
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
          acc.v[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][mt], fb[buf][nt], acc.v[mt][nt], 0, 0, 0);
      if (kk + 1 < BK / 16) {  // spread the fragment loads between the MFMAs
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
          __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // two MFMAs
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    __syncthreads();
    if (more) f_load(0, As + (cur ^ 1) * kTileBytes, Bs + (cur ^ 1) * kTileBytes, 0);
  }
}

}  // namespace gemm
}  // namespace aa
