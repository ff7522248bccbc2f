// bf16 tile GEMM on gfx950 matrix cores:  D[m][n] = sum_k A[m][k] * B[n][k], fp32 accumulation.
//
// One workgroup of 4 waves computes a 256 x 256 tile of D with v_mfma_f32_32x32x16_bf16, each wave a 128 x 128 block
// (256 accumulator registers).  Either operand may be stored K-contiguous (row x of the array holds A[x][0..K), the
// usual "row-major [M, K]") or K-major (row k of the array holds A[0..M)[k], i.e. the array is [K, M]): the second
// form lets a product contract over the rows of two row-major arrays without a transposed copy of either.
//
// Operands are staged through LDS in 64-wide K slices that go from global memory straight into LDS
// (buffer_load ... lds, 16 bytes per lane): every load instruction fetches whole 128-byte lines (8 rows x 128 B of a
// K-contiguous operand, 2 rows x 512 B of a K-major one).  Measured next to a full MFMA stream, a compute unit
// sustains about 58 B/clk of such loads but only about 30 B/clk of 64-byte row pieces, and the tile consumes 32 B/clk
// at full MFMA rate.  LDS (160 KiB) holds a ring of five 32 KiB units, a unit being the 256 x 64 slice of one operand;
// units follow each other as A0 B0 A1 B1 A2 ...  While slice k is multiplied, A(k+1) and B(k+1) are landed or landing
// and A(k+2) is in flight; the only wait for memory is a counted vmcnt that leaves the youngest unit outstanding, and
// the one barrier per slice (before its last 16-wide step) both publishes slice k + 1 and retires A(k), B(k), whose
// slots the next loads take.  What happens to the accumulators is decided by the caller (an epilogue after
// mainloop()).  mainloop16(), at the end of this file, is the same loop issued as v_mfma_f32_16x16x32_bf16 for two
// K-contiguous operands.
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
typedef short s16x4_t __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kUnitBytes = 256 * BK * 2;        // one operand, one slice: 32 KiB
constexpr int kUnits = 5;
constexpr int kLdsBytes = kUnits * kUnitBytes;  // 160 KiB
constexpr int kThreads = 256;

// Accumulators of one wave: v[mt][nt] is the 32 x 32 tile at rows mt * 32, columns nt * 32 of its 128 x 128 block.
struct Acc {
  f32x16_t v[4][4];
};

// row (m) and column (n) inside the wave's block of accumulator element (mt, nt, i) of lane `lane`
__device__ __forceinline__ int acc_row(int mt, int i, int lane) { return mt * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3); }
__device__ __forceinline__ int acc_col(int nt, int lane) { return nt * 32 + (lane & 31); }

// Tile order: the hardware deals consecutive workgroup ids to the 8 XCDs in turn.  Ids are first regrouped so that
// each XCD gets a contiguous range, and that range then walks the tile grid in bands of `kGroupM` tile rows, so that
// tiles that run at the same time on one XCD share A and B slices in its L2.
constexpr int kGroupM = 4;
// XCD x runs the ids x, x + 8, ...: ceil((total - x) / 8) of them, so its range starts after those of the XCDs before
// it, at x * (total / 8) + min(x, total % 8): a bijection for every count.
__device__ __forceinline__ int xcd_contiguous(int pid, int total) {
  const int x = pid & 7, rem = total & 7;
  return x * (total >> 3) + (x < rem ? x : rem) + (pid >> 3);
}

// tile number q of the band walk: bands of group_m tile rows, inside a band down the rows first
__device__ __forceinline__ void tile_at(int q, int tiles_m, int tiles_n, int& tm, int& tn, int group_m = kGroupM) {
  const int in_group = group_m * tiles_n;
  const int g = q / in_group;
  const int first_m = g * group_m;
  const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  tm = first_m + (q % in_group) % gsz;
  tn = (q % in_group) / gsz;
}

__device__ __forceinline__ void tile_of(int pid, int tiles_m, int tiles_n, int& tm, int& tn, int group_m = kGroupM) {
  tile_at(xcd_contiguous(pid, tiles_m * tiles_n), tiles_m, tiles_n, tm, tn, group_m);
}

// One operand.  K-contiguous: element (x, k) at ptr[x * ld + k], `rows` = number of valid x.  K-major: element (x, k)
// at ptr[k * ld + x], `rows` = number of valid x (the columns of the array).  ld and rows are multiples of 8 (16-byte
// pieces never straddle an edge); 256 array rows must stay below 2^30 elements (32-bit byte offsets inside a tile).
// Everything outside the valid range reads as zero.
struct Operand {
  const uint16_t* ptr;  // bf16 bits
  int64_t ld;
  int rows;
};

constexpr int kBufferFlags = 0x00020000;  // raw buffer descriptor, 32-bit data format

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// s_waitcnt immediate of gfx9: vmcnt in bits [3:0] and [15:14], expcnt [6:4], lgkmcnt [11:8]
constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8); }

// ds_read_b64_tr_b16 at addr + off, off one of the eight offsets a fragment read uses.  Written as inline assembly
// because the compiler makes its own intrinsic wait for every outstanding buffer_load ... lds (it cannot tell that
// they write other units); the caller therefore waits for the result itself (s_waitcnt lgkmcnt) before using it.
__device__ __forceinline__ s16x4_t lds_read_tr(uint32_t addr, int off) {
  s16x4_t v;
  switch (off) {
    case 0:     asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(addr)); break;
    case 2048:  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:2048" : "=v"(v) : "v"(addr)); break;
    case 8192:  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:8192" : "=v"(v) : "v"(addr)); break;
    case 10240: asm volatile("ds_read_b64_tr_b16 %0, %1 offset:10240" : "=v"(v) : "v"(addr)); break;
    case 16384: asm volatile("ds_read_b64_tr_b16 %0, %1 offset:16384" : "=v"(v) : "v"(addr)); break;
    case 18432: asm volatile("ds_read_b64_tr_b16 %0, %1 offset:18432" : "=v"(v) : "v"(addr)); break;
    case 24576: asm volatile("ds_read_b64_tr_b16 %0, %1 offset:24576" : "=v"(v) : "v"(addr)); break;
    default:    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:26624" : "=v"(v) : "v"(addr)); break;
  }
  return v;
}

// what a wave needs to bring its 8 blocks of one unit
struct Cursor {
  __amdgpu_buffer_rsrc_t rs;
  int voff;  // per lane, range fix-ups included
  uint32_t dst;
};

// Per-operand constants of a wave.
//
// K-contiguous unit: 256 rows x 128 B, 32 blocks of 1 KiB (8 rows each); block b = 4 j + wave, j = 0..7; lane l
// brings row 8 b + l / 8 and puts global chunk (l % 8) ^ ((r >> 1) & 7) at slot l % 8 of the row (XOR swizzle: the 16
// lanes that LDS serves together in a fragment read, 16 consecutive rows and one chunk, fall on 16 different bank
// groups).  (r >> 1) & 7 = (4 (wave & 1) + l / 16) & 7 for every j.  A fragment (sub-tile x, k step kk) of lane l is
// the 16 bytes of row 32 x + l % 32, chunk 2 kk + l / 32.
//
// K-major unit: 64 k-rows x 512 B, 32 blocks of 1 KiB (2 k-rows each); lane l of block b brings k-row 2 b + l / 32
// and puts global chunk (l % 32) ^ (4 (k & 3)) at slot l % 32, so that the four k-rows a transposing read touches
// together lie 64 bytes apart in the banks.  Fragments come through ds_read_b64_tr_b16: in each group of 16 lanes,
// lane s points at four consecutive elements E[s][0..3] and lane j receives E[4 q + j / 4][j % 4], q = 0..3.  With
// lane s pointing at (k = kb + s / 4, x = xb + 4 (s % 4)) lane j receives k = kb .. kb + 3 at x = xb + j: four
// consecutive k of one row of the operand, half of the eight an MFMA lane needs.
struct Side {
  const uint16_t* base;  // tile origin
  int64_t ld;
  int voff, jstep, bytes;  // load: per-lane byte offset inside a slice, step per block index j, valid bytes of the tile
  int chunk;               // K-contiguous: the global chunk (of 8) this lane brings; used for slices that straddle K
  int frag[4];             // fragment read: per-lane byte offsets inside a unit (K-contiguous: per kk; K-major: per x)
};

template <bool KMAJOR>
__device__ __forceinline__ Side make_side(const Operand& X, int x0, int wq, int wave, int lane) {
  Side s;
  s.ld = X.ld;
  const int valid = (X.rows - x0) < 256 ? (X.rows - x0) : 256;
  if constexpr (!KMAJOR) {
    const int ld_row = 8 * wave + (lane >> 3);
    s.chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
    s.base = X.ptr + (int64_t)x0 * X.ld;
    s.voff = (int)(((int64_t)ld_row * X.ld + s.chunk * 8) * 2);
    s.jstep = (int)(32 * X.ld * 2);
    s.bytes = (int)((int64_t)valid * X.ld * 2);
    const int half = lane >> 5, r7 = (lane >> 1) & 7;
    const int fr = (wq * 128 + (lane & 31)) * 128;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) s.frag[kk] = fr + (((2 * kk + half) ^ r7) << 4);
  } else {
    const int krow = 2 * wave + (lane >> 5);  // k-row inside block group j: 8 j + krow
    s.chunk = (lane & 31) ^ (4 * (krow & 3));
    s.base = X.ptr + x0;
    // chunks at or past the valid columns are pushed out of the descriptor's range
    s.voff = (int)(((int64_t)krow * X.ld + s.chunk * 8) * 2) | (s.chunk * 8 >= valid ? (int)0x80000000 : 0);
    s.jstep = (int)(8 * X.ld * 2);
    s.bytes = 0;  // per slice: the valid k-rows times ld
    const int sl = lane & 15, half = lane >> 5, mb = (lane >> 4) & 1;
    const int lanebase = (8 * half + (sl >> 2)) * 512 + 16 * (16 * wq + 2 * mb + ((sl >> 1) & 1)) + 8 * (sl & 1);
#pragma unroll
    for (int x = 0; x < 4; ++x) s.frag[x] = lanebase + 64 * (x ^ (sl >> 2));
  }
  return s;
}

// Main loop.  Leaves the result in `acc`; `lds` is kLdsBytes of dynamic shared memory.  K % 8 == 0.
// AKM / BKM: the operand is K-major.
//
// Per slice (four 16-wide k steps, fragments double buffered in registers; every step issues its 16 MFMAs with the 8
// fragment reads of the next step behind MFMAs 0-7 and 4 global loads behind MFMAs 8, 10, 12, 14 (a load blocks the
// wave's issue for about as long as one MFMA runs: next to a fragment read it costs idle cycles), in exactly the order
// written here):
//   steps 0, 1, 2; wait: own fragment reads done, own loads through B(k+1) landed (A(k+2) may be in flight); barrier;
//   step 3 (reads the first fragments of slice k + 1)
// Slices at or past K get an empty descriptor (no memory traffic, zeros in LDS) so that the count of loads per slice,
// and with it the vmcnt arithmetic, is the same from the first slice to the last.
template <bool AKM, bool BKM>
__device__ __forceinline__ void mainloop(const Operand& A, const Operand& B, int K, int m0, int n0, Acc& acc, char* lds) {
  constexpr int MN = 16, NR = 8;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: LDS block addresses stay in scalar registers
  const int wm = wave >> 1, wn = wave & 1;
  const uint32_t lds32 = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
  const Side sa_ = make_side<AKM>(A, m0, wm, wave, lane);
  const Side sb_ = make_side<BKM>(B, n0, wn, wave, lane);

  // unit u = 2 slice + operand lives in slot u % 5
  auto open_unit = [&](Cursor& c, const Side& s, bool kmajor, int slice, int slot) {
    const int k0 = slice * BK;
    const bool live = k0 < K;
    if (!kmajor) {
      // the descriptor starts at column k0, so row r is in range iff r < rows (the last row may end early, never late);
      // a slice that straddles K: chunks at or past K are pushed out of the descriptor's range
      c.rs = __builtin_amdgcn_make_buffer_rsrc((void*)(s.base + (live ? k0 : 0)), 0, live ? s.bytes - k0 * 2 : 0, kBufferFlags);
      c.voff = s.voff | ((k0 + BK > K && k0 + s.chunk * 8 >= K) ? (int)0x80000000 : 0);
    } else {
      // the descriptor starts at k-row k0 and covers the valid k-rows of the slice
      const int krows = live ? ((K - k0) < BK ? (K - k0) : BK) : 0;
      c.rs = __builtin_amdgcn_make_buffer_rsrc((void*)(s.base + (live ? (int64_t)k0 * s.ld : 0)), 0, (int)(krows * s.ld * 2),
                                               kBufferFlags);
      c.voff = s.voff;
    }
    c.dst = lds32 + slot * kUnitBytes + wave * 1024;
  };
  auto open_a = [&](Cursor& c, int slice, int slot) { open_unit(c, sa_, AKM, slice, slot); };
  auto open_b = [&](Cursor& c, int slice, int slot) { open_unit(c, sb_, BKM, slice, slot); };
  auto g_load1 = [&](const Cursor& c, int jstep, int j) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(c.rs, (lds_ptr_t)(uintptr_t)(c.dst + j * 4096), 16, c.voff + j * jstep, 0, 0, 0);
  };

#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc.v[mt][nt][i] = 0.f;

  bf16x8_t fa[2][4], fb[2][4];
  // fragment of sub-tile x at k step kk from the unit in `slot`
  auto frag = [&](const Side& s, bool kmajor, int slot, int kk, int x) -> bf16x8_t {
    if (!kmajor) return __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(lds + slot * kUnitBytes + s.frag[kk] + x * 4096));
    const uint32_t at = lds32 + slot * kUnitBytes + s.frag[x];
    const s16x4_t lo = lds_read_tr(at, kk * 8192);
    const s16x4_t hi = lds_read_tr(at, kk * 8192 + 2048);
    return __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  // fragment r of a step: r < 4 is A sub-tile r, otherwise B sub-tile r - 4; slot_a / slot_b are the units' slots
  auto f_load1 = [&](int buf, int slot_a, int slot_b, int kk, int r) {
    if (r < 4)
      fa[buf][r] = frag(sa_, AKM, slot_a, kk, r);
    else
      fb[buf][r - 4] = frag(sb_, BKM, slot_b, kk, r - 4);
  };
  auto mfma1 = [&](int buf, int i) {
    const int mt = i >> 2, nt = i & 3;
    acc.v[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][mt], fb[buf][nt], acc.v[mt][nt], 0, 0, 0);
  };
  // one 16-wide k step: 16 MFMAs from fragment buffer `buf`; in their shadow the 8 fragment reads of the next step
  // (k step nkk of the units in slots na, nb) and 4 global loads (blocks j0 .. j0 + 3 of the unit behind `c`)
  auto step = [&](int buf, int na, int nb, int nkk, const Cursor& c, int jstep, int j0) {
#pragma unroll
    for (int i = 0; i < MN; ++i) {
      mfma1(buf, i);
      if (i < NR) f_load1(buf ^ 1, na, nb, nkk, i);
      if (i >= 8 && !(i & 1)) g_load1(c, jstep, j0 + ((i - 8) >> 1));  // behind MFMAs 8, 10, 12, 14
      __builtin_amdgcn_sched_barrier(0);
    }
    // the transposing reads are invisible to the compiler's own wait insertion: they were issued in the first half
    // of the step, wait for them here, before the next step multiplies their results
    if (AKM || BKM) {
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto next_slot = [](int s, int by) { s += by; return s >= kUnits ? s - kUnits : s; };

  const int nk = (K + BK - 1) / BK;
  Cursor cx, cy;  // cx: the B unit whose first half was issued before the barrier; cy: the A unit issued in steps 1, 2
  // units 0, 1, 2 (A0, B0, A1) and the first half of unit 3 (B1)
  open_a(cy, 0, 0);
#pragma unroll
  for (int j = 0; j < 8; ++j) g_load1(cy, sa_.jstep, j);
  open_b(cx, 0, 1);
#pragma unroll
  for (int j = 0; j < 8; ++j) g_load1(cx, sb_.jstep, j);
  open_a(cy, 1, 2);
#pragma unroll
  for (int j = 0; j < 8; ++j) g_load1(cy, sa_.jstep, j);
  open_b(cx, 1, 3);
#pragma unroll
  for (int j = 0; j < 4; ++j) g_load1(cx, sb_.jstep, j);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(12, 15));  // this wave's parts of units 0 and 1 have landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int r = 0; r < NR; ++r) f_load1(0, 0, 1, 0, r);
  if (AKM || BKM) __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
  int sa = 0;  // slot of A(k) = (2 k) % 5
  for (int k = 0; k < nk; ++k) {
    const int sb = next_slot(sa, 1), sa1 = next_slot(sa, 2), sb1 = next_slot(sa, 3), s4 = next_slot(sa, 4);
    // cx is unit 2 k + 3 = B(k + 1) in slot sb1, opened when its first half was issued
    __builtin_amdgcn_sched_barrier(0);
    step(0, sa, sb, 1, cx, sb_.jstep, 4);
    open_a(cy, k + 2, s4);  // unit 2 k + 4 = A(k + 2)
    __builtin_amdgcn_sched_barrier(0);
    step(1, sa, sb, 2, cy, sa_.jstep, 0);
    step(0, sa, sb, 3, cy, sa_.jstep, 4);
    // own reads of slice k done; own loads through unit 2 k + 3 landed (unit 2 k + 4 may be in flight)
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(8, 0));
    __builtin_amdgcn_s_barrier();
    open_b(cx, k + 2, sa);  // unit 2 k + 5 = B(k + 2) takes the slot of A(k)
    __builtin_amdgcn_sched_barrier(0);
    step(1, sa1, sb1, 0, cx, sb_.jstep, 0);
    sa = sa1;
  }
  // the empty loads of the last slices may still deposit zeros: let them finish before the caller reuses LDS
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  __builtin_amdgcn_s_barrier();
}

// ---- the same loop on v_mfma_f32_16x16x32_bf16, for two K-contiguous operands ----------------------------------------
// The chip is power-limited on random operands, and the 16 x 16 x 32 form draws less power per flop (half the
// accumulator register traffic): an MFMA-only loop sustains 2.06 PFLOP/s at 2.06 GHz with it against 1.87 at 1.80 GHz
// with 32 x 32 x 16.  With twice as many MFMAs per slice every direct-to-LDS load falls behind a 16-cycle instead of a
// 32-cycle MFMA and costs more idle cycles (164 k cycles per 256 x 256 x 4096 tile instead of 151 k), but at
// 1.9 GHz instead of 1.66: 5 % faster as a bare loop on K-contiguous operands, 2-3 % in the kernels that use it.
// K-major operands (two transposing reads per fragment) gain nothing, so the products that contract K-major arrays
// stay on mainloop().
//
// Register layout of one 16 x 16 x 32 MFMA (checked on the hardware):
//   A operand, lane l: A[m = l % 16][k = 8 (l / 16) + j], j = 0..7
//   B operand, lane l: B[n = l % 16][k = 8 (l / 16) + j]
//   D, lane l, register i: n = l % 16, m = 4 (l / 16) + i
// i.e. a lane owns one column n of D and 4 consecutive rows m; the lanes l ^ 16, l ^ 32 own the other rows of that n.
typedef float f32x4acc_t __attribute__((ext_vector_type(4)));
constexpr int kAcc16Tiles = 8;  // per direction: a wave's 128 x 128 block is 8 x 8 tiles of 16 x 16
struct Acc16 {
  f32x4acc_t v[kAcc16Tiles][kAcc16Tiles];
};
__device__ __forceinline__ int acc16_row(int mt, int i, int lane) { return mt * 16 + 4 * (lane >> 4) + i; }
__device__ __forceinline__ int acc16_col(int nt, int lane) { return nt * 16 + (lane & 15); }

// Per-operand constants of a wave (K-contiguous unit as above: same loads, same swizzle).  A fragment (sub-tile x of 16
// rows, 32-wide k step kk) of lane l is the 16 bytes of row 16 x + l % 16, chunk 4 kk + l / 16.
struct Side16 {
  const uint16_t* base;  // tile origin
  int bytes;             // valid bytes of the tile
  int chunk;             // the global chunk (of 8) this lane brings
  int voffj[8];          // load j of a unit: per-lane byte offset inside the slice (range fix-ups included)
  int frag[2];           // fragment read: per-lane byte offset inside a unit, per k step
};

__device__ __forceinline__ Side16 make_side16(const Operand& X, int x0, int wq, int wave, int lane) {
  Side16 s;
  const int valid = (X.rows - x0) < 256 ? (X.rows - x0) : 256;
  const int ld_row = 8 * wave + (lane >> 3);
  s.chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
  s.base = X.ptr + (int64_t)x0 * X.ld;
#pragma unroll
  for (int j = 0; j < 8; ++j) s.voffj[j] = (int)((((int64_t)ld_row + 32 * j) * X.ld + s.chunk * 8) * 2);
  s.bytes = (int)((int64_t)valid * X.ld * 2);
  const int kgrp = lane >> 4, r7 = (lane >> 1) & 7;  // row 16 x + lane % 16: (row >> 1) & 7 = (lane >> 1) & 7
  const int fr = (wq * 128 + (lane & 15)) * 128;
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) s.frag[kk] = fr + (((4 * kk + kgrp) ^ r7) << 4);
  return s;
}

// A slice is two 32-wide k steps of 64 MFMAs (A sub-tile mt x B sub-tile nt, 8 x 8); the fragments of both steps live
// in registers (2 x 16 fragments).  A step is issued as two halves of 32 MFMAs: the first half multiplies A0-3 with
// B0-3, then with B4-7; the second half A4-7 with B0-7.  So a step can start once A0-3 and B0-3 are there, B4-7 are
// needed 16 MFMAs later and A4-7 a half later.  Every half carries 8 fragment reads (behind its first 8 MFMAs) and 4
// global loads (behind MFMAs 7, 15, 23, 31; other placements take 1.5 % fewer cycles at a clock that much lower), in
// exactly the order written here:
//   half 0 (step 0, first)    reads B4-7, A4-7 of step 0            loads the second half of B(k+1)
//   half 1 (step 0, second)   reads B0-3, A0-3 of step 1            loads the first half of A(k+2)
//   half 2 (step 1, first)    reads B4-7, A4-7 of step 1            loads the second half of A(k+2)
//   wait: own fragment reads done, own loads through B(k+1) landed (A(k+2) may be in flight); barrier
//   half 3 (step 1, second)   reads B0-3, A0-3 of slice k+1 step 0  loads the first half of B(k+2) into A(k)'s slot
// The ring of units, the counted waits and the empty descriptors past K are those of mainloop().
__device__ __forceinline__ void mainloop16(const Operand& A, const Operand& B, int K, int m0, int n0, Acc16& acc, char* lds) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const uint32_t lds32 = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
  Side16 sa_ = make_side16(A, m0, wm, wave, lane);
  Side16 sb_ = make_side16(B, n0, wn, wave, lane);
  struct Unit {
    __amdgpu_buffer_rsrc_t rs;
    uint32_t dst;
  };
  auto open_unit = [&](Unit& c, Side16& s, int slice, int slot) {
    const int k0 = slice * BK;
    const bool live = k0 < K;
    // the descriptor starts at column k0, so row r is in range iff r < rows (the last row may end early, never late)
    c.rs = __builtin_amdgcn_make_buffer_rsrc((void*)(s.base + (live ? k0 : 0)), 0, live ? s.bytes - k0 * 2 : 0, kBufferFlags);
    // the one slice that straddles K: chunks at or past K are pushed out of the descriptor's range, for good (the
    // slices after it are empty anyway)
    if (live && k0 + BK > K) {
      const int out = (k0 + s.chunk * 8 >= K) ? (int)0x80000000 : 0;
#pragma unroll
      for (int j = 0; j < 8; ++j) s.voffj[j] |= out;
    }
    c.dst = lds32 + slot * kUnitBytes + wave * 1024;
  };
  auto g_load1 = [&](const Unit& c, const Side16& s, int j) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(c.rs, (lds_ptr_t)(uintptr_t)(c.dst + j * 4096), 16, s.voffj[j], 0, 0, 0);
  };

#pragma unroll
  for (int mt = 0; mt < kAcc16Tiles; ++mt)
#pragma unroll
    for (int nt = 0; nt < kAcc16Tiles; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc.v[mt][nt][i] = 0.f;

  bf16x8_t fa[2][8], fb[2][8];
  // fragment read r (0..7) of a half: group = 0 reads B0-3 then A0-3, group = 1 reads B4-7 then A4-7, of k step kk of
  // the units in slot_a / slot_b, into fragment buffer buf
  auto f_load1 = [&](int buf, int slot_a, int slot_b, int kk, int group, int r) {
    const int x = 4 * group + (r & 3);
    if (r < 4)
      fb[buf][x] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(lds + slot_b * kUnitBytes + sb_.frag[kk] + x * 2048));
    else
      fa[buf][x] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(lds + slot_a * kUnitBytes + sa_.frag[kk] + x * 2048));
  };
  auto mfma1 = [&](int buf, int mt, int nt) {
    acc.v[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[buf][mt], fb[buf][nt], acc.v[mt][nt], 0, 0, 0);
  };
  // one half of a 32-wide k step: 32 MFMAs from fragment buffer `buf` (second = 0: A0-3 x B0-3, then A0-3 x B4-7;
  // second = 1: A4-7 x B0-7); in their shadow 8 fragment reads (group rgroup of k step rkk of the units in slots ra, rb,
  // into buffer rbuf) and 4 global loads (blocks j0 .. j0 + 3 of the unit `c` of operand side `cs`)
  auto half = [&](int buf, int second, int rbuf, int ra, int rb, int rkk, int rgroup, const Unit& c, const Side16& cs, int j0) {
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      if (second)
        mfma1(buf, 4 + (i >> 3), i & 7);
      else
        mfma1(buf, (i >> 2) & 3, (i & 3) + 4 * (i >> 4));
      if (i < 8) f_load1(rbuf, ra, rb, rkk, rgroup, i);
      if ((i & 7) == 7) g_load1(c, cs, j0 + (i >> 3));
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto next_slot = [](int s, int by) { s += by; return s >= kUnits ? s - kUnits : s; };

  const int nk = (K + BK - 1) / BK;
  Unit cx, cy;  // cx: the B unit whose first half was issued before the barrier; cy: the A unit issued in halves 1, 2
  // units 0, 1, 2 (A0, B0, A1) and the first half of unit 3 (B1)
  open_unit(cy, sa_, 0, 0);
#pragma unroll
  for (int j = 0; j < 8; ++j) g_load1(cy, sa_, j);
  open_unit(cx, sb_, 0, 1);
#pragma unroll
  for (int j = 0; j < 8; ++j) g_load1(cx, sb_, j);
  open_unit(cy, sa_, 1, 2);
#pragma unroll
  for (int j = 0; j < 8; ++j) g_load1(cy, sa_, j);
  open_unit(cx, sb_, 1, 3);
#pragma unroll
  for (int j = 0; j < 4; ++j) g_load1(cx, sb_, j);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(12, 15));  // this wave's parts of units 0 and 1 have landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int r = 0; r < 8; ++r) f_load1(0, 0, 1, 0, 0, r);
  int sa = 0;  // slot of A(k) = (2 k) % 5
  for (int k = 0; k < nk; ++k) {
    const int sb = next_slot(sa, 1), sa1 = next_slot(sa, 2), sb1 = next_slot(sa, 3), s4 = next_slot(sa, 4);
    // cx is unit 2 k + 3 = B(k + 1) in slot sb1, opened when its first half was issued
    __builtin_amdgcn_sched_barrier(0);
    half(0, 0, 0, sa, sb, 0, 1, cx, sb_, 4);
    open_unit(cy, sa_, k + 2, s4);  // unit 2 k + 4 = A(k + 2)
    __builtin_amdgcn_sched_barrier(0);
    half(0, 1, 1, sa, sb, 1, 0, cy, sa_, 0);
    half(1, 0, 1, sa, sb, 1, 1, cy, sa_, 4);
    // own reads of slice k done; own loads through unit 2 k + 3 landed (unit 2 k + 4 may be in flight)
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(8, 0));
    __builtin_amdgcn_s_barrier();
    open_unit(cx, sb_, k + 2, sa);  // unit 2 k + 5 = B(k + 2) takes the slot of A(k)
    __builtin_amdgcn_sched_barrier(0);
    half(1, 1, 0, sa1, sb1, 0, 0, cx, sb_, 0);
    sa = sa1;
  }
  // the empty loads of the last slices may still deposit zeros: let them finish before the caller reuses LDS
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  __builtin_amdgcn_s_barrier();
}

}  // namespace gemm
}  // namespace aa
