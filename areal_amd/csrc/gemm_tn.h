// bf16 "TN" tile GEMM on gfx950 matrix cores:  D[m][n] = sum_k A[m][k] * B[n][k]
// with A [M, K] and B [N, K] both row-major (K contiguous), fp32 accumulation.
//
// One workgroup computes a 256 x 256 tile of D with v_mfma_f32_32x32x16_bf16.  Operands are staged through LDS in
// 32-wide K slices that go from global memory straight into LDS (buffer_load ... lds), in a ring of kStages slices:
// while slice k is multiplied, slices k + 1 .. k + kStages - 1 are landed or in flight, and the only wait for
// memory is a counted vmcnt that leaves the younger slices outstanding.  What happens to the accumulators is decided
// by the caller (an epilogue after mainloop()), so the same loop serves the lm_head statistics, the d(logits) tiles
// and the two gradient GEMMs.
//
// Register layout of one 32 x 32 x 16 MFMA (checked on the hardware):
//   A operand, lane l: A[m = l % 32][k = 8 (l / 32) + j], j = 0..7
//   B operand, lane l: B[n = l % 32][k = 8 (l / 32) + j]
//   D, lane l, register i: n = l % 32, m = 8 (i / 4) + 4 (l / 32) + i % 4
// i.e. a lane owns one column n of D and 16 of its rows m: reductions over m for a fixed n stay inside a lane
// (plus its partner lane l ^ 32).
#pragma once
#include "device_utils.h"

namespace aa {
namespace gemm {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256, BK = 32;
constexpr int kRowBytes = BK * 2;                    // one row of a K slice in LDS: 64 B = 4 chunks of 16 B
constexpr int kOperandStageBytes = 256 * kRowBytes;  // one operand, one stage: 16 KiB

// WAVES_M x WAVES_N waves share the tile; each owns (256 / WAVES_M) x (256 / WAVES_N) of it.
template <int WAVES_M, int WAVES_N, int STAGES>
struct Shape {
  static constexpr int kWavesM = WAVES_M, kWavesN = WAVES_N, kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = 64 * kWaves;
  static constexpr int kStages = STAGES;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int MT = WTM / 32, NT = WTN / 32;  // 32 x 32 accumulator tiles of a wave
  static constexpr int kBlocksPerWave = 16 / kWaves;  // 1 KiB blocks (16 rows) of one operand slice that a wave brings
  static constexpr int kLoadsPerSlice = 2 * kBlocksPerWave;
  static constexpr int kLdsBytes = 2 * STAGES * kOperandStageBytes;
  static_assert(16 % kWaves == 0 && STAGES >= 2 && STAGES <= 4, "unsupported shape");
};

// Accumulators of one wave: v[mt][nt] is the 32 x 32 tile at rows mt * 32, columns nt * 32 of its block.
template <class S>
struct Acc {
  f32x16_t v[S::MT][S::NT];
};

// row (m) and column (n) inside the wave's block of accumulator element (mt, nt, i) of lane `lane`
__device__ __forceinline__ int acc_row(int mt, int i, int lane) { return mt * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3); }
__device__ __forceinline__ int acc_col(int nt, int lane) { return nt * 32 + (lane & 31); }

// Tile order: the hardware deals consecutive workgroup ids to the 8 XCDs in turn.  Ids are first regrouped so that
// each XCD gets a contiguous range, and that range then walks the tile grid in bands of `kGroupM` tile rows, so that
// tiles that run at the same time on one XCD share A and B slices in its L2.
constexpr int kGroupM = 4;
// The XCD regrouping above is a bijection only when the tile count is a multiple of 8; otherwise use the plain order.
__device__ __forceinline__ void tile_of(int pid, int tiles_m, int tiles_n, int& tm, int& tn, int group_m = kGroupM) {
  const int total = tiles_m * tiles_n;
  int q = pid;
  if ((total & 7) == 0) q = (pid & 7) * (total >> 3) + (pid >> 3);
  const int in_group = group_m * tiles_n;
  const int g = q / in_group;
  const int first_m = g * group_m;
  const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  tm = first_m + (q % in_group) % gsz;
  tn = (q % in_group) / gsz;
}

struct Operand {
  const uint16_t* ptr;  // bf16 bits
  int64_t ld;           // row stride in elements (a multiple of 8; 256 rows of it must stay below 2^30 elements)
  int rows;             // valid rows (rows beyond read as zero)
};

constexpr int kBufferFlags = 0x00020000;  // raw buffer descriptor, 32-bit data format

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// s_waitcnt immediate of gfx9: vmcnt in bits [3:0] and [15:14], expcnt [6:4], lgkmcnt [11:8]
constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8); }

// Main loop.  Leaves the result in `acc`; `lds` is S::kLdsBytes of dynamic shared memory.  K % 8 == 0.
//
// A slice of one operand is 256 rows x 64 B, held without padding as 16 blocks of 1 KiB (16 rows each): one
// buffer_load ... lds of a wave fills one block, lane i depositing its 16 bytes at block + 16 i.  Inside a row the
// four 16-byte chunks are XOR-swizzled, chunk c of row r at slot c ^ ((r >> 2) & 3), so that the 16 lanes that LDS
// serves together in a fragment read (16 consecutive rows, one chunk) fall on 16 different bank groups.  The swizzle
// costs nothing: each lane simply fetches the global chunk that belongs at its slot.  Buffer descriptors cover exactly
// the valid rows of the tile; slices at or past K get an empty descriptor (no memory traffic, zeros in LDS) so that
// the count of loads per slice, and with it the vmcnt arithmetic, is the same from the first slice to the last.
//
// Per slice (two 16-wide k steps, fragments double buffered in registers):
//   fragment reads of step 1, global loads of slice k + kStages - 1, MFMAs of step 0
//   wait: own fragment reads done, own loads of slice k + 1 landed (younger ones stay in flight); barrier
//   fragment reads of step 0 of slice k + 1, MFMAs of step 1
// The barrier both publishes slice k + 1 and retires slice k, whose stage the next iteration's loads overwrite.
// ABL (probing only, results are then wrong): bit 0 no global loads, bit 1 no barriers, bit 2 no fragment reads,
// bit 3 global loads fetch whole 128-byte lines (8 rows x 128 B per instruction, same bytes in another order).
template <class S, int ABL = 0>
__device__ __forceinline__ void mainloop(const Operand& A, const Operand& B, int K, int m0, int n0, Acc<S>& acc,
                                         char* lds) {
  constexpr int MT = S::MT, NT = S::NT, NS = S::kStages, MN = MT * NT, NR = MT + NT, NL = S::kLoadsPerSlice;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: LDS block addresses stay in scalar registers
  const int wm = wave / S::kWavesN, wn = wave % S::kWavesN;
  char* As = lds;                            // [NS][256][64 B]
  char* Bs = lds + NS * kOperandStageBytes;  // [NS][256][64 B]

  // Loading: block b = kWaves j + wave holds rows 16 b .. 16 b + 15; lane l brings row r = 16 b + l / 4 and puts
  // global chunk (l % 4) ^ ((r >> 2) & 3) at slot l % 4; (r >> 2) & 3 = (l >> 4) & 3 for every b.
  const int ld_row = 16 * wave + (lane >> 2);
  const int ld_chunk = (lane & 3) ^ ((lane >> 4) & 3);
  const int rows_a = (A.rows - m0) < BM ? (A.rows - m0) : BM;
  const int rows_b = (B.rows - n0) < BN ? (B.rows - n0) : BN;
  const uint16_t* a_base = A.ptr + (int64_t)m0 * A.ld;
  const uint16_t* b_base = B.ptr + (int64_t)n0 * B.ld;
  const int a_voff = (int)(((int64_t)ld_row * A.ld + ld_chunk * 8) * 2);
  const int b_voff = (int)(((int64_t)ld_row * B.ld + ld_chunk * 8) * 2);
  const int a_jstep = (int)(16 * S::kWaves * A.ld * 2), b_jstep = (int)(16 * S::kWaves * B.ld * 2);
  const int a_bytes = (int)((int64_t)rows_a * A.ld * 2), b_bytes = (int)((int64_t)rows_b * B.ld * 2);

  // The loads of one slice: `desc` prepares the two descriptors, load q (0 .. NL - 1) then brings one block.
  __amdgpu_buffer_rsrc_t ra, rb;
  int past = 0;
  auto desc = [&](int slice) {
    const int k0 = slice * BK;
    const bool live = k0 < K;
    // the descriptor starts at column k0, so row r is in range iff r < rows (the last row may end early, never late)
    ra = __builtin_amdgcn_make_buffer_rsrc((void*)(a_base + (live ? k0 : 0)), 0, live ? a_bytes - k0 * 2 : 0, kBufferFlags);
    rb = __builtin_amdgcn_make_buffer_rsrc((void*)(b_base + (live ? k0 : 0)), 0, live ? b_bytes - k0 * 2 : 0, kBufferFlags);
    // a slice that straddles K (K % 32 != 0): chunks at or past K are pushed out of the descriptor's range
    past = (k0 + BK > K && k0 + ld_chunk * 8 >= K) ? (int)0x80000000 : 0;
    if (ABL & 8) {
      const int64_t kk0 = (slice >> 1) * 64, r0 = (slice & 1) * 128;
      ra = __builtin_amdgcn_make_buffer_rsrc((void*)(a_base + (live ? kk0 + r0 * A.ld : 0)), 0, live ? a_bytes - (int)(kk0 + r0 * A.ld) * 2 : 0, kBufferFlags);
      rb = __builtin_amdgcn_make_buffer_rsrc((void*)(b_base + (live ? kk0 + r0 * B.ld : 0)), 0, live ? b_bytes - (int)(kk0 + r0 * B.ld) * 2 : 0, kBufferFlags);
      past = 0;
    }
  };
  const int a_voff8 = (int)(((int64_t)(8 * wave + (lane >> 3)) * A.ld + (lane & 7) * 8) * 2);
  const int b_voff8 = (int)(((int64_t)(8 * wave + (lane >> 3)) * B.ld + (lane & 7) * 8) * 2);
  auto g_load1 = [&](int stage, int q) {
    if (ABL & 1) return;
    const int j = q >> 1;
    const int blk = stage * kOperandStageBytes + (S::kWaves * j + wave) * 1024;
    if (ABL & 8) {
      if ((q & 1) == 0)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(As + blk), 16, a_voff8 + j * (a_jstep / 2), 0, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(Bs + blk), 16, b_voff8 + j * (b_jstep / 2), 0, 0, 0);
      return;
    }
    if (ABL & 32) {  // one LDS address, no range fix-up: the fewest instructions a load can take
      if ((q & 1) == 0) __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)As, 16, a_voff + j * a_jstep, 0, 0, 0);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)As, 16, b_voff + j * b_jstep, 0, 0, 0);
      return;
    }
    if ((q & 1) == 0)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(As + blk), 16, (a_voff + j * a_jstep) | past, 0, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(Bs + blk), 16, (b_voff + j * b_jstep) | past, 0, 0, 0);
  };

#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc.v[mt][nt][i] = 0.f;

  // Fragment of sub-tile x at k step kk: row r = block row + 32 x + lane % 32, global chunk 2 kk + lane / 32, found at
  // slot (2 kk + lane / 32) ^ ((r >> 2) & 3); (r >> 2) & 3 = (lane >> 2) & 3 because the other terms are multiples of 32.
  const int half = lane >> 5, r3 = (lane >> 2) & 3;
  const int fr_a = (wm * S::WTM + (lane & 31)) * kRowBytes;
  const int fr_b = (wn * S::WTN + (lane & 31)) * kRowBytes;
  const int slot0 = ((half ^ r3) << 4), slot1 = (((2 + half) ^ r3) << 4);
  bf16x8_t fa[2][MT], fb[2][NT];
  if (ABL & 4) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
#pragma unroll
      for (int x = 0; x < MT; ++x) fa[b][x] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(As + fr_a + x * 2048 + b * 16));
#pragma unroll
      for (int x = 0; x < NT; ++x) fb[b][x] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(Bs + fr_b + x * 2048 + b * 16));
    }
  }
  // fragment r of a step: r < MT is A sub-tile r, otherwise B sub-tile r - MT
  auto f_load1 = [&](int buf, int stage, int kk, int r) {
    const int slot = kk ? slot1 : slot0;
    if (ABL & 4) return;
    if (r < MT)
      fa[buf][r] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(As + stage * kOperandStageBytes + fr_a + slot + r * 32 * kRowBytes));
    else
      fb[buf][r - MT] =
          __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(Bs + stage * kOperandStageBytes + fr_b + slot + (r - MT) * 32 * kRowBytes));
  };
  auto mfma1 = [&](int buf, int i) {
    const int mt = i / NT, nt = i % NT;
    acc.v[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][mt], fb[buf][nt], acc.v[mt][nt], 0, 0, 0);
  };

  // Slices are taken kStages at a time, so that stage numbers are compile-time constants; the slices past K that this
  // adds (at most kStages - 1, none for the shapes of the lm_head path) multiply the zeros their empty loads left.
  // The instruction order below is the issue order: every group ends in a scheduling barrier.  The global loads are
  // spread evenly over the MFMAs (the four SIMDs share one address unit, which takes 16 cycles per load: issued
  // back to back from every wave they stall the waves behind its queue).  Stage k % kStages is free from the barrier
  // in the middle of slice k on; the loads of slice k + kStages go there, the first half of them during the rest of
  // slice k, the second half during the first half of slice k + 1.
  constexpr int LP = NL / 2;       // loads per phase
  constexpr int kEvery = MN / LP;  // one load after every kEvery MFMAs
  static_assert(NL % 2 == 0 && MN % LP == 0 && NR <= MN, "schedule does not fit");
  const int nk = (K + BK - 1) / BK;
#pragma unroll
  for (int s = 0; s < NS - 1; ++s) {
    desc(s);
#pragma unroll
    for (int q = 0; q < NL; ++q) g_load1(s, q);
  }
  desc(NS - 1);
#pragma unroll
  for (int q = 0; q < LP; ++q) g_load1(NS - 1, q);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm((NS - 2) * NL + LP, 15));  // this wave's part of slice 0 has landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int r = 0; r < NR; ++r) f_load1(0, 0, 0, r);
  for (int kt = 0; kt < nk; kt += NS) {
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      desc(kt + s + NS - 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < MN; ++i) {
        mfma1(0, i);
        if (i < NR) f_load1(1, s, 1, i);
        if ((i + 1) % kEvery == 0) g_load1((s + NS - 1) % NS, LP + i / kEvery);
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_s_waitcnt(waitcnt_imm((ABL & 16) ? 63 : (NS - 2) * NL, 0));
      if (!(ABL & 2)) __builtin_amdgcn_s_barrier();
      desc(kt + s + NS);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < MN; ++i) {
        mfma1(1, i);
        if (i < NR) f_load1(0, (s + 1) % NS, 0, i);
        if ((i + 1) % kEvery == 0) g_load1(s, i / kEvery);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  // the empty loads of the last slices may still deposit zeros: let them finish before the caller reuses LDS
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  __builtin_amdgcn_s_barrier();
}

// The same loop for 4 waves and 4 stages with the global loads issued by one wave at a time.  The four SIMDs of a
// compute unit share one address unit; when every wave issues its load at the same point of the (barrier-aligned)
// instruction stream, three of the four wait in its queue and their next MFMA with them.  Here a half slice (the 16
// blocks of one operand) is brought by a single wave, one block per MFMA, and the waves take turns phase by phase,
// so the address unit sees one load every 32 cycles.  Half slice hs = 2 slice + operand is issued during phase
// p = hs - 7 (phase 2 k is the first half of slice k) by wave p % 4; every wave therefore issues 16 loads every
// fourth phase, and "at most 16 of my loads outstanding" before the barrier of slice k means that everything up to
// slice k + 1 has landed, whichever wave brought it.
template <int ABL = 0>
__device__ __forceinline__ void mainloop_rot(const Operand& A, const Operand& B, int K, int m0, int n0,
                                             Acc<Shape<2, 2, 4>>& acc, char* lds) {
  typedef Shape<2, 2, 4> S;
  constexpr int MT = 4, NT = 4, NS = 4, MN = 16, NR = 8;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  char* As = lds;
  char* Bs = lds + NS * kOperandStageBytes;
  const uint32_t lds32 = (uint32_t)(uintptr_t)(lds_ptr_t)lds;  // LDS byte address of the ring

  // block b holds rows 16 b .. 16 b + 15; lane l brings row 16 b + l / 4, global chunk (l % 4) ^ ((l >> 4) & 3)
  const int ld_chunk = (lane & 3) ^ ((lane >> 4) & 3);
  const int rows_a = (A.rows - m0) < BM ? (A.rows - m0) : BM;
  const int rows_b = (B.rows - n0) < BN ? (B.rows - n0) : BN;
  const uint16_t* a_base = A.ptr + (int64_t)m0 * A.ld;
  const uint16_t* b_base = B.ptr + (int64_t)n0 * B.ld;
  const int a_voff = (int)(((int64_t)(lane >> 2) * A.ld + ld_chunk * 8) * 2);
  const int b_voff = (int)(((int64_t)(lane >> 2) * B.ld + ld_chunk * 8) * 2);
  const int a_bstep = (int)(16 * A.ld * 2), b_bstep = (int)(16 * B.ld * 2);
  const int a_bytes = (int)((int64_t)rows_a * A.ld * 2), b_bytes = (int)((int64_t)rows_b * B.ld * 2);

  __amdgpu_buffer_rsrc_t rs;
  int past = 0;
  auto desc = [&](int slice, int operand) {
    const int k0 = slice * BK;
    const bool live = k0 < K;
    const uint16_t* base = operand ? b_base : a_base;
    const int bytes = operand ? b_bytes : a_bytes;
    rs = __builtin_amdgcn_make_buffer_rsrc((void*)(base + (live ? k0 : 0)), 0, live ? bytes - k0 * 2 : 0, kBufferFlags);
    past = (k0 + BK > K && k0 + ld_chunk * 8 >= K) ? (int)0x80000000 : 0;
  };
  auto g_load1 = [&](int stage, int operand, int b) {
    if (ABL & 1) return;
    const uint32_t dst = lds32 + ((operand ? NS : 0) + stage) * kOperandStageBytes + b * 1024;
    const int voff = operand ? b_voff + b * b_bstep : a_voff + b * a_bstep;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)(uintptr_t)dst, 16, voff | past, 0, 0, 0);
  };

#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc.v[mt][nt][i] = 0.f;

  const int half = lane >> 5, r3 = (lane >> 2) & 3;
  const int fr_a = (wm * S::WTM + (lane & 31)) * kRowBytes;
  const int fr_b = (wn * S::WTN + (lane & 31)) * kRowBytes;
  const int slot0 = ((half ^ r3) << 4), slot1 = (((2 + half) ^ r3) << 4);
  bf16x8_t fa[2][MT], fb[2][NT];
  auto f_load1 = [&](int buf, int stage, int kk, int r) {
    const int slot = kk ? slot1 : slot0;
    if (r < MT)
      fa[buf][r] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(As + stage * kOperandStageBytes + fr_a + slot + r * 32 * kRowBytes));
    else
      fb[buf][r - MT] =
          __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(Bs + stage * kOperandStageBytes + fr_b + slot + (r - MT) * 32 * kRowBytes));
  };
  auto mfma1 = [&](int buf, int i) {
    const int mt = i / NT, nt = i % NT;
    acc.v[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][mt], fb[buf][nt], acc.v[mt][nt], 0, 0, 0);
  };

  const int nk = (K + BK - 1) / BK;
  // half slices 0 .. 6 (slices 0 .. 2 and operand A of slice 3), each by the wave whose turn it would have been
#pragma unroll
  for (int hs = 0; hs < 2 * NS - 1; ++hs) {
    if (wave == ((hs + 1) & 3)) {
      desc(hs >> 1, hs & 1);
#pragma unroll
      for (int b = 0; b < 16; ++b) g_load1(hs >> 1, hs & 1, b);
    }
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(16, 15));
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int r = 0; r < NR; ++r) f_load1(0, 0, 0, r);
  for (int kt = 0; kt < nk; kt += NS) {
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      // first half of slice kt + s; operand B of slice kt + s + 3 goes to the stage that slice kt + s - 1 left
      {
        const bool mine = wave == ((2 * s) & 3);
        if (mine) desc(kt + s + NS - 1, 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < MN; ++i) {
          mfma1(0, i);
          if (i < NR) f_load1(1, s, 1, i);
          __builtin_amdgcn_sched_barrier(0);
          if (mine) g_load1((s + NS - 1) % NS, 1, i);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(16, 0));
      if (!(ABL & 2)) __builtin_amdgcn_s_barrier();
      // second half; operand A of slice kt + s + 4 goes to this slice's own stage, free from the barrier on
      {
        const bool mine = wave == ((2 * s + 1) & 3);
        if (mine) desc(kt + s + NS, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < MN; ++i) {
          mfma1(1, i);
          if (i < NR) f_load1(0, (s + 1) % NS, 0, i);
          __builtin_amdgcn_sched_barrier(0);
          if (mine) g_load1(s, 0, i);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  __builtin_amdgcn_s_barrier();
}

// ---- 64-wide slices, whole cache lines --------------------------------------------------------------------------
// The same tile GEMM with K slices of 64: every global load instruction fetches 8 rows x 128 B, i.e. whole cache
// lines.  Measured next to a full MFMA stream, a compute unit sustains about 58 B/clk of such loads but only about
// 30 B/clk of the 16 rows x 64 B loads that 32-wide slices need, and the tile consumes 32 B/clk at full MFMA rate.
// LDS (160 KiB) holds a ring of five 32 KiB units, a unit being the 256 x 64 slice of one operand; units follow each
// other as A0 B0 A1 B1 A2 ...  While slice k is multiplied, A(k+1) and B(k+1) are landed or landing and A(k+2) is in
// flight; the one barrier per slice (before its last 16-wide step) retires A(k), B(k), whose slots the next loads take.
namespace wide {

constexpr int BK = 64;
constexpr int kRowBytes = BK * 2;            // 128 B: 8 chunks of 16 B
constexpr int kUnitBytes = 256 * kRowBytes;  // 32 KiB
constexpr int kUnits = 5;
constexpr int kLdsBytes = kUnits * kUnitBytes;  // 160 KiB
constexpr int kThreads = 256;
typedef Shape<2, 2, 4> S;  // 4 waves, 128 x 128 each (the stage count of Shape is not used here)

// what a wave needs to bring its blocks of one unit
struct Cursor {
  __amdgpu_buffer_rsrc_t rs;
  int past, voff, jstep;
  uint32_t dst;
};

// ABL (probing only): bit 0 no global loads, bit 1 no barrier, bit 2 no fragment reads.
template <int ABL = 0>
__device__ __forceinline__ void mainloop(const Operand& A, const Operand& B, int K, int m0, int n0, Acc<S>& acc,
                                         char* lds) {
  constexpr int MT = 4, NT = 4, MN = 16, NR = 8;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const uint32_t lds32 = (uint32_t)(uintptr_t)(lds_ptr_t)lds;

  // Loading a unit: 32 blocks of 1 KiB (8 rows each); block b = 4 j + wave, j = 0..7; lane l brings row 8 b + l / 8
  // and puts global chunk (l % 8) ^ ((r >> 1) & 7) at slot l % 8; (r >> 1) & 7 = (4 (wave & 1) + l / 16) & 7.
  const int ld_row = 8 * wave + (lane >> 3);
  const int ld_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
  const int rows_a = (A.rows - m0) < BM ? (A.rows - m0) : BM;
  const int rows_b = (B.rows - n0) < BN ? (B.rows - n0) : BN;
  const uint16_t* a_base = A.ptr + (int64_t)m0 * A.ld;
  const uint16_t* b_base = B.ptr + (int64_t)n0 * B.ld;
  const int a_voff = (int)(((int64_t)ld_row * A.ld + ld_chunk * 8) * 2);
  const int b_voff = (int)(((int64_t)ld_row * B.ld + ld_chunk * 8) * 2);
  const int a_jstep = (int)(32 * A.ld * 2), b_jstep = (int)(32 * B.ld * 2);
  const int a_bytes = (int)((int64_t)rows_a * A.ld * 2), b_bytes = (int)((int64_t)rows_b * B.ld * 2);

  // unit u = 2 slice + operand lives in slot u % 5
  auto open_unit = [&](Cursor& c, int slice, int operand, int slot) {
    const int k0 = slice * BK;
    const bool live = k0 < K;
    const uint16_t* base = operand ? b_base : a_base;
    const int bytes = operand ? b_bytes : a_bytes;
    // the descriptor starts at column k0, so row r is in range iff r < rows (the last row may end early, never late)
    c.rs = __builtin_amdgcn_make_buffer_rsrc((void*)(base + (live ? k0 : 0)), 0, live ? bytes - k0 * 2 : 0, kBufferFlags);
    // a slice that straddles K: chunks at or past K are pushed out of the descriptor's range
    c.past = (k0 + BK > K && k0 + ld_chunk * 8 >= K) ? (int)0x80000000 : 0;
    c.voff = operand ? b_voff : a_voff;
    c.jstep = operand ? b_jstep : a_jstep;
    c.dst = lds32 + slot * kUnitBytes + wave * 1024;
  };
  auto g_load1 = [&](const Cursor& c, int j) {
    if (ABL & 1) return;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(c.rs, (lds_ptr_t)(uintptr_t)(c.dst + j * 4096), 16, (c.voff + j * c.jstep) | c.past,
                                             0, 0, 0);
  };

#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc.v[mt][nt][i] = 0.f;

  // Fragment of sub-tile x at k step kk: row r = block row + 32 x + lane % 32, global chunk 2 kk + lane / 32, found at
  // slot (2 kk + lane / 32) ^ ((r >> 1) & 7); (r >> 1) & 7 = (lane >> 1) & 7 because the other terms are multiples of 32.
  const int half = lane >> 5, r7 = (lane >> 1) & 7;
  const int fr_a = (wm * 128 + (lane & 31)) * kRowBytes;
  const int fr_b = (wn * 128 + (lane & 31)) * kRowBytes;
  int sl[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) sl[kk] = ((2 * kk + half) ^ r7) << 4;
  bf16x8_t fa[2][MT], fb[2][NT];
  if (ABL & 4) {
#pragma unroll
    for (int bq = 0; bq < 2; ++bq)
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        fa[bq][x] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(lds + fr_a + x * 4096 + bq * 16));
        fb[bq][x] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(lds + kUnitBytes + fr_b + x * 4096 + bq * 16));
      }
  }
  // fragment r of a step: r < MT is A sub-tile r, otherwise B sub-tile r - MT; slot_a / slot_b are the units' slots
  auto f_load1 = [&](int buf, int slot_a, int slot_b, int kk, int r) {
    if (ABL & 4) return;
    if (r < MT)
      fa[buf][r] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(lds + slot_a * kUnitBytes + fr_a + sl[kk] + r * 32 * kRowBytes));
    else
      fb[buf][r - MT] =
          __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(lds + slot_b * kUnitBytes + fr_b + sl[kk] + (r - MT) * 32 * kRowBytes));
  };
  auto mfma1 = [&](int buf, int i) {
    const int mt = i / NT, nt = i % NT;
    acc.v[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][mt], fb[buf][nt], acc.v[mt][nt], 0, 0, 0);
  };
  // one 16-wide k step: 16 MFMAs from fragment buffer `buf`; in their shadow the 8 fragment reads of the next step
  // (k step nkk of the units in slots na, nb) and 4 global loads (blocks j0 .. j0 + 3 of the unit behind `c`)
  auto step = [&](int buf, int na, int nb, int nkk, const Cursor& c, int j0) {
#pragma unroll
    for (int i = 0; i < MN; ++i) {
      mfma1(buf, i);
      if (i < NR) f_load1(buf ^ 1, na, nb, nkk, i);
      if ((i & 3) == 3) g_load1(c, j0 + (i >> 2));
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto next_slot = [](int s, int by) { s += by; return s >= kUnits ? s - kUnits : s; };

  const int nk = (K + BK - 1) / BK;
  Cursor cx, cy;  // cx: the unit whose first half was issued before the barrier; cy: the unit issued in steps 1 and 2
  // units 0, 1, 2 and the first half of unit 3
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    open_unit(cx, u >> 1, u & 1, u);
#pragma unroll
    for (int j = 0; j < (u < 3 ? 8 : 4); ++j) g_load1(cx, j);
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(12, 15));  // this wave's parts of units 0 and 1 have landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int r = 0; r < NR; ++r) f_load1(0, 0, 1, 0, r);
  int sa = 0;  // slot of A(k) = (2 k) % 5
  for (int k = 0; k < nk; ++k) {
    const int sb = next_slot(sa, 1), sa1 = next_slot(sa, 2), sb1 = next_slot(sa, 3), s4 = next_slot(sa, 4);
    // cx is unit 2 k + 3 = B(k + 1) in slot sb1, opened when its first half was issued
    __builtin_amdgcn_sched_barrier(0);
    step(0, sa, sb, 1, cx, 4);
    open_unit(cy, k + 2, 0, s4);  // unit 2 k + 4 = A(k + 2)
    __builtin_amdgcn_sched_barrier(0);
    step(1, sa, sb, 2, cy, 0);
    step(0, sa, sb, 3, cy, 4);
    // own reads of slice k done; own loads through unit 2 k + 3 landed (unit 2 k + 4 may be in flight)
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(8, 0));
    if (!(ABL & 2)) __builtin_amdgcn_s_barrier();
    open_unit(cx, k + 2, 1, sa);  // unit 2 k + 5 = B(k + 2) takes the slot of A(k)
    __builtin_amdgcn_sched_barrier(0);
    step(1, sa1, sb1, 0, cx, 0);
    sa = sa1;
  }
  // the empty loads of the last slices may still deposit zeros: let them finish before the caller reuses LDS
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  __builtin_amdgcn_s_barrier();
}

}  // namespace wide

}  // namespace gemm
}  // namespace aa
