// lm_head path for gfx950: log-prob / entropy of softmax(hidden @ weight.T / T), their backward, and the whole
// lm_head + PPO-loss training step, on this library's own bf16 MFMA tile GEMM (gemm_tn.h), without ever writing the
// [T, V] logits to memory.  The reference has no such path: its equivalent is the lm_head matmul followed by
// gather_logprobs_entropy (areal/utils/functional/vocab_parallel.py:23-29), ppo_actor_loss_fn
// (areal/utils/functional/functional.py:429-559) and autograd.
//
// Forward (aa_lmhead_fwd, and the first half of the training step): 256 (vocabulary) x 256 (tokens) tiles of the
// logits are formed in accumulator registers; the epilogue reduces every 128-row block of a tile to the softmax
// partials (k, s, u) per token; the label's logit comes from a dot product per token (k_label_logit), and a small
// kernel merges the partials of all blocks into log-prob and entropy.  Nothing of size T x V is written.
//
// Backward needs d(logits) twice (for d_hidden and for d_weight), so a bf16 panel [tokens with gradient, V] of it is
// written once per token chunk and contracted by two plain tile GEMMs (which read the panel, the weight and the
// hidden states as they lie: no transposed copies).  Two ways to fill the panel:
//   recompute   the logits tiles are formed again and turned into d(logits) in registers (2 T_grad V H extra flops);
//               what aa_lmhead_bwd does, where the upstream gradients only exist after the forward has returned.
//   carry       (training step only) the forward tiles also write p_v / p_label = 2^((x_v - x_label) c), as bf16, for the
//               tokens that will have a gradient (the label logit is known before the tiles run).  Once the loss is
//               known, d(logits) of a row is that row times one factor per token, -(g / T) p_label (the label entry
//               is patched to 1 - 1 / p_label first), and the factor is applied inside the two GEMMs: no second logits
//               GEMM and no pass over the panel.  A chunk that holds a token whose label is too unlikely for that
//               range (log-prob below -80) is redone by the recompute tiles, decided on the device.
// Tokens whose loss mask is zero have a zero gradient row: they are left out of the panel and of both GEMMs.
#include "device_utils.h"
#include "gemm_tn.h"
#include "ppo_math.h"

namespace aa {
namespace lmhead {

using namespace gemm;

typedef float f32x4_t __attribute__((ext_vector_type(4)));

// token chunk of the panel.  Measured: with 32768 the forward tiles run 2.4 % slower at H = 4096 (the hidden rows of
// a chunk, 2 * chunk * H bytes, no longer fit the 256 MB memory-side cache that every band of tiles re-reads them from)
constexpr int kChunkTokens = 16384;
constexpr int kPanelPitch = BM + 8;        // pitch (elements) of the tile staged in LDS as [token][vocab]
constexpr int kStageBytes = 256 * kPanelPitch * 2;  // 135168 B, inside the 160 KiB the main loop uses
static_assert(kStageBytes + 256 * 4 <= kLdsBytes, "the staged tile and its 256 row numbers must fit the main loop's LDS");

__host__ __device__ __forceinline__ int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

enum { kModeStats = 0, kModeStatsCarry = 1, kModeRecompute = 2 };

// ---- the row count of a chunk, when only the device knows it -------------------------------------------------------
// k_compact_map leaves four words per chunk: how many tokens have a panel row, and what the kernels behind it derive
// from that number, worked out once instead of by every workgroup: the tiles of BN rows that cover them, the count
// rounded up to a whole K slice (at least one: the main loop always starts one), and the number of parts the d_hidden
// product over those rows is cut into (choose_splits).  Kernels that are given these words are queued for the
// largest count possible and stop at the rows in use.
enum { kRowsTotal = 0, kRowsLive = 1, kRowsSliced = 2, kRowsSplits = 3 };
enum { kBoundNone = 0, kBoundN = 1, kBoundK = 2 };

struct TileArgs {
  // statistics per (128-row vocabulary block, token): planes [blocks][pitch_t]
  float* pk;
  float* ps;
  float* pu;
  float* pn;              // nullable: smallest raw logit of the block (for vocab_min_logits), same layout
  float* xy;              // [tokens of the chunk] raw label logit (k_label_logit, before the tiles run)
  const int64_t* labels;  // labels of the chunk
  int64_t pitch_t;
  float c;                // log2(e) / temperature
  // panel [rows, panel_ld] bf16, panel_ld = V rounded up to 8 (the entries past V are written as zeros): row
  // out_rows[token] (or the token itself when out_rows is null); negative: no row
  uint16_t* panel;
  int64_t panel_ld;
  const int32_t* out_rows;
  // recompute: per token of the chunk; column n of the tile is token col_tokens[n] (or n when null; negative: none)
  const int32_t* col_tokens;
  const float* row_lse;    // natural-log logsumexp of the row
  const float* row_ez;     // sum_j p_j z_j (used with g_entropy)
  const float* g_logp;
  const float* g_entropy;  // nullable
  float inv_t;
  const int32_t* run_if;   // recompute tiles only: when given, the kernel does nothing unless *run_if != 0
  const int32_t* n_bound;  // recompute tiles only: when given, the row-count words of the chunk (kRowsLive is used):
                           // only the tiles over the token columns in use run
};

// Carry mode stores 2^(x c - kref) with kref = c * (label logit of the token): a reference that is known before the
// first tile runs and is the same in every vocabulary block, so that d(logits) of a panel row is the stored row times
// ONE factor per token (applied where the gradient GEMMs already touch the token: the d_hidden epilogue and the gather
// of the hidden rows for d_weight) and no pass over the panel is needed.  The stored value is p_v / p_label, finite
// in bf16 (which has the exponent range of fp32) as long as the label's log-prob is above about -87; the exponent is
// clamped so that nothing overflows, and a chunk with such a token (kCarryMinLogp, never seen in training: the label
// would have to be e^-80 unlikely) is redone by the recompute tiles, decided on the device.
constexpr float kCarryMaxShift = 126.f;
constexpr float kCarryMinLogp = -80.f;
// d_weight takes the row's factor f = -(g / T) p_label inside the hidden rows, rounded to bf16: |f| times a hidden
// entry has to stay a normal number (above 2^-126) for entries down to 2^-26 of magnitude, or the chunk is redone
constexpr float kCarryMinFactor = 0x1p-100f;

// Statistics (and, with CARRY, the staged probability ratios) of one wave's 128 x 128 block, accumulators in the
// 16 x 16 tile layout: a lane holds, for each of 8 tokens (nt), 8 runs (mt) of 4 consecutive vocabulary rows, and the
// lanes l ^ 16, l ^ 32 hold the other rows of the same tokens.  RAGGED: the block may reach past the vocabulary (last
// tile row only), rows at or past V are left out.
template <bool CARRY, bool RAGGED>
__device__ __forceinline__ void block_stats(const Acc16& acc, const TileArgs& a, int tm, int wm, int wn, int n0, int N,
                                            int V, int mbase, int lane, uint16_t* Z) {
  constexpr int PZ = kPanelPitch;
#pragma unroll
  for (int nt = 0; nt < kAcc16Tiles; ++nt) {
    const int nloc = wn * 128 + acc16_col(nt, lane);
    const int n = n0 + nloc;
    float mx = -FLT_MAX;
    if constexpr (!RAGGED) {
#pragma unroll
      for (int mt = 0; mt < kAcc16Tiles; ++mt)
#pragma unroll
        for (int i = 0; i < 4; i += 2) mx = fmaxf(fmaxf(mx, acc.v[mt][nt][i]), acc.v[mt][nt][i + 1]);  // one v_max3 per pair
    } else {
#pragma unroll
      for (int mt = 0; mt < kAcc16Tiles; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = (mbase + acc16_row(mt, i, lane) < V) ? fmaxf(mx, acc.v[mt][nt][i]) : mx;
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));  // four lanes hold the same token
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    if (a.pn) {  // uniform: the caller wants the smallest logit of every token as well
      float mn = FLT_MAX;
      if constexpr (!RAGGED) {
#pragma unroll
        for (int mt = 0; mt < kAcc16Tiles; ++mt)
#pragma unroll
          for (int i = 0; i < 4; i += 2) mn = fminf(fminf(mn, acc.v[mt][nt][i]), acc.v[mt][nt][i + 1]);
      } else {
#pragma unroll
        for (int mt = 0; mt < kAcc16Tiles; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) mn = (mbase + acc16_row(mt, i, lane) < V) ? fminf(mn, acc.v[mt][nt][i]) : mn;
      }
      mn = fminf(mn, __shfl_xor(mn, 16, kWave));
      mn = fminf(mn, __shfl_xor(mn, 32, kWave));
      if (lane < 16 && n < N) a.pn[(int64_t)(tm * 2 + wm) * a.pitch_t + n] = mn;  // FLT_MAX: no valid row in this block
    }
    const float k = fmaxf(mx * a.c, kNegBig);   // kNegBig: no valid row in this block
    float to_ref = 1.f;                         // 2^(k - kref): block-relative -> label-relative exponentials
    if constexpr (CARRY) {
      const float kref = n < N ? a.xy[n] * a.c : 0.f;
      // a label outside the vocabulary has no logit (NaN): keep the block-relative values, the row's factor is NaN or 0
      to_ref = fabsf(kref) < 1e30f ? fast_exp2(fminf(k - kref, kCarryMaxShift)) : 1.f;
    }
    float s = 0.f, u = 0.f;
#pragma unroll
    for (int mt = 0; mt < kAcc16Tiles; ++mt) {
      float e[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float t = fmaf(acc.v[mt][nt][q], a.c, -k);
        e[q] = fast_exp2(t);
        if constexpr (RAGGED) e[q] = (mbase + acc16_row(mt, q, lane) < V) ? e[q] : 0.f;
        s += e[q];
        u = fmaf(t, e[q], u);
      }
      if constexpr (CARRY) {
        uint2 pk;
        pk.x = Elem<AA_BF16>::pack(e[0] * to_ref, e[1] * to_ref);
        pk.y = Elem<AA_BF16>::pack(e[2] * to_ref, e[3] * to_ref);
        *(uint2*)(Z + nloc * PZ + wm * 128 + acc16_row(mt, 0, lane)) = pk;
      }
    }
    s += __shfl_xor(s, 16, kWave);
    s += __shfl_xor(s, 32, kWave);
    u += __shfl_xor(u, 16, kWave);
    u += __shfl_xor(u, 32, kWave);
    if (lane < 16 && n < N) {
      const int64_t at = (int64_t)(tm * 2 + wm) * a.pitch_t + n;
      a.pk[at] = k;
      a.ps[at] = s;
      a.pu[at] = u;
    }
  }
}

// One 256 x 256 tile: rows m = vocabulary (operand A = weight), columns n = tokens (operand B = hidden states), so
// that everything a token needs from the tile sits in one lane and its partner lanes ^ 16, ^ 32.  Both operands are
// K-contiguous: the 16 x 16 x 32 main loop.
template <int MODE>
__global__ __launch_bounds__(kThreads) void k_lmhead_tiles(Operand W, Operand Hd, int K, int tiles_m, int tiles_n,
                                                                 TileArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  if constexpr (MODE == kModeRecompute) {
    if (a.run_if && *a.run_if == 0) return;  // uniform over the grid
  }
  if constexpr (MODE == kModeRecompute) {
    // token columns in use, known to the device alone: the tiles that cover them are numbered as if the host had
    // launched exactly those (the same walk over the XCDs), the workgroups beyond them return
    if (a.n_bound) {
      const int live = a.n_bound[kRowsLive];
      tiles_n = live < tiles_n ? live : tiles_n;
      if ((int)blockIdx.x >= tiles_m * tiles_n) return;  // the same decision in every thread of the workgroup
    }
  }
  int tm, tn;
  tile_of(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  Acc16 acc;
  mainloop16(W, Hd, K, m0, n0, acc, lds);  // ends with a barrier: LDS is free

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int V = W.rows, N = Hd.rows;
  const int mbase = m0 + wm * 128;  // first vocabulary row of this wave's block
  uint16_t* Z = (uint16_t*)lds;     // [256 tokens][kPanelPitch] bf16
  constexpr int PZ = kPanelPitch;

  if constexpr (MODE != kModeRecompute) {
    if (m0 + BM > V)  // rows past the vocabulary: last tile row only
      block_stats<MODE == kModeStatsCarry, true>(acc, a, tm, wm, wn, n0, N, V, mbase, lane, Z);
    else
      block_stats<MODE == kModeStatsCarry, false>(acc, a, tm, wm, wn, n0, N, V, mbase, lane, Z);
  } else {
    const bool ragged_rows = m0 + BM > V;
#pragma unroll
    for (int nt = 0; nt < kAcc16Tiles; ++nt) {
      const int nloc = wn * 128 + acc16_col(nt, lane);
      const int n = n0 + nloc;
      float A = 0.f, B = 0.f, lab_add = 0.f, lse2 = 0.f;
      int64_t y = -1;
      const int t = n < N ? (a.col_tokens ? a.col_tokens[n] : n) : -1;
      if (t >= 0) {
        const float gl = a.g_logp[t];
        const float gh = a.g_entropy ? a.g_entropy[t] : 0.f;
        const float ez = a.g_entropy ? a.row_ez[t] : 0.f;
        lse2 = a.row_lse[t] * kLog2e;
        A = a.inv_t * (gh * ez - gl);
        B = -gh * a.inv_t * a.inv_t;
        lab_add = gl * a.inv_t;
        y = a.labels[t];
      }
      const int rel = (int)(y - mbase < -1 ? -1 : (y - mbase > 128 ? 128 : y - mbase));  // outside [0, 128): not here
#pragma unroll
      for (int mt = 0; mt < kAcc16Tiles; ++mt) {
        float o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float x = acc.v[mt][nt][q];
          o[q] = fast_exp2(fmaf(x, a.c, -lse2)) * fmaf(B, x, A);  // columns past the tokens: never written out
        }
        const int r0 = acc16_row(mt, 0, lane);  // row of o[0] inside the wave's block
        if (ragged_rows) {  // uniform; rows at or past V: the last piece of a panel row may reach them, they hold zeros
#pragma unroll
          for (int q = 0; q < 4; ++q) o[q] = (mbase + r0 + q < V) ? o[q] : 0.f;
        }
        if (rel >= r0 && rel < r0 + 4) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (rel - r0 == q) o[q] += lab_add;
        }
        uint2 pk;
        pk.x = Elem<AA_BF16>::pack(o[0], o[1]);
        pk.y = Elem<AA_BF16>::pack(o[2], o[3]);
        *(uint2*)(Z + nloc * PZ + wm * 128 + r0) = pk;
      }
    }
  }
  if constexpr (MODE != kModeStats) {
    // panel row of each of the tile's 256 tokens (-1: none), looked up once and shared through LDS behind the staged
    // tile, so that the store loop below has no dependent global load in it
    int32_t* rows_lds = (int32_t*)(lds + 256 * PZ * 2);
    {
      const int n = n0 + tid;
      rows_lds[tid] = n < N ? (a.out_rows ? a.out_rows[n] : n) : -1;
    }
    __syncthreads();
    // panel rows: 16-byte pieces along the vocabulary (the pitch is a multiple of 8: the piece that straddles V ends in
    // the row's own padding, whose entries were formed as zeros)
    const int mc = (tid & 31) * 8, m = m0 + mc;
    if (m < V) {
#pragma unroll 8
      for (int i = 0; i < 32; ++i) {
        const int nloc = (tid >> 5) + 8 * i;
        const int r = rows_lds[nloc];
        if (r >= 0) *(u32x4_t*)(a.panel + (int64_t)r * a.panel_ld + m) = *(const u32x4_t*)(Z + nloc * PZ + mc);
      }
    }
  }
}

// Raw label logit of every token: xy[t] = hidden[t] . weight[label[t]] in fp32 (NaN for a label outside [0, V)).  One
// wave per token.
__global__ __launch_bounds__(256) void k_label_logit(const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ weight,
                                                     const int64_t* __restrict__ labels, int n_tok, int H, int V,
                                                     float* __restrict__ xy, int32_t* __restrict__ clear_flag) {
  if (clear_flag && blockIdx.x == 0 && threadIdx.x == 0) *clear_flag = 0;  // the chunk's "redo by recompute" flag
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (t >= n_tok) return;
  const int64_t y = labels[t];
  if (y < 0 || y >= V) {
    if (lane == 0) xy[t] = __builtin_nanf("");
    return;
  }
  const uint16_t* h = hidden + (int64_t)t * H;
  const uint16_t* w = weight + y * H;
  float acc = 0.f;
  for (int j = lane * 8; j < H; j += 64 * 8) {
    float a[8], b[8];
    load8<AA_BF16>(h, j, a);
    load8<AA_BF16>(w, j, b);
#pragma unroll
    for (int q = 0; q < 8; ++q) acc = fmaf(a[q], b[q], acc);
  }
  acc = wave_sum(acc);
  if (lane == 0) xy[t] = acc;
}

// Merge of the block partials of 64 tokens by a workgroup of 1024 threads: lane = token, wave w folds blocks
// w, w + 16, ... in order, then the 16 wave results are folded in wave order by every wave alike.  Fixed order:
// deterministic.
struct Merged {
  float k, s, u;
  float n;  // smallest raw logit (FLT_MAX when the minimum plane was not asked for)
};
constexpr int kMergeWaves = 16;
constexpr int kMergeSmemFloats = 4 * kMergeWaves * 64;

__device__ __forceinline__ void merge_into(Merged& m, float bk, float bs, float bu) {
  const float nk = fmaxf(m.k, bk);
  const float da = m.k - nk, db = bk - nk;
  const float fa = fast_exp2(da), fb = fast_exp2(db);
  m.u = fa * fmaf(da, m.s, m.u) + fb * fmaf(db, bs, bu);
  m.s = m.s * fa + bs * fb;
  m.k = nk;
}

// t: the token of this lane (may be past the end: then the result is meaningless and the caller drops it)
__device__ __forceinline__ Merged merge_blocks(const float* __restrict__ pk, const float* __restrict__ ps,
                                               const float* __restrict__ pu, const float* __restrict__ pn, int blocks,
                                               int64_t pitch_t, int64_t t, bool live, float* smem /* [4][16][64] */) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  Merged m{kNegBig, 0.f, 0.f, FLT_MAX};
  if (live)
    for (int b = wave; b < blocks; b += kMergeWaves) {
      const int64_t at = (int64_t)b * pitch_t + t;
      merge_into(m, pk[at], ps[at], pu[at]);
      if (pn) m.n = fminf(m.n, pn[at]);
    }
  smem[(0 * kMergeWaves + wave) * 64 + lane] = m.k;
  smem[(1 * kMergeWaves + wave) * 64 + lane] = m.s;
  smem[(2 * kMergeWaves + wave) * 64 + lane] = m.u;
  smem[(3 * kMergeWaves + wave) * 64 + lane] = m.n;
  __syncthreads();
  Merged r{kNegBig, 0.f, 0.f, FLT_MAX};
#pragma unroll
  for (int w = 0; w < kMergeWaves; ++w) {
    merge_into(r, smem[(0 * kMergeWaves + w) * 64 + lane], smem[(1 * kMergeWaves + w) * 64 + lane],
               smem[(2 * kMergeWaves + w) * 64 + lane]);
    r.n = fminf(r.n, smem[(3 * kMergeWaves + w) * 64 + lane]);
  }
  return r;
}

// forward of the stand-alone op: 64 tokens per workgroup.  vmax / vmin (nullable, together): largest and smallest raw
// logit of the row (what FSDPEngine._get_vocab_min_max_logits takes from materialised logits,
// areal/engine/fsdp_engine.py:1893-1906); the largest is recovered from the merged exponent k = c * max, i.e. to one
// rounding, the smallest comes from its own plane.
__global__ __launch_bounds__(1024) void k_combine(const float* __restrict__ pk, const float* __restrict__ ps,
                                                  const float* __restrict__ pu, const float* __restrict__ pn,
                                                  const float* __restrict__ xy, int blocks, int64_t pitch_t, int n_tok,
                                                  float c, float* __restrict__ logp, float* __restrict__ entropy,
                                                  float* __restrict__ row_lse, float* __restrict__ row_ez,
                                                  float* __restrict__ vmax, float* __restrict__ vmin) {
  __shared__ float smem[kMergeSmemFloats];
  const int t = blockIdx.x * 64 + (threadIdx.x & 63);
  const Merged m = merge_blocks(pk, ps, pu, pn, blocks, pitch_t, t, t < n_tok, smem);
  if (t >= n_tok || threadIdx.x >= 64) return;
  const float log2s = fast_log2(m.s);
  const float mean_t = m.u / m.s;
  logp[t] = (fmaf(xy[t], c, -m.k) - log2s) * kLn2;  // xy is NaN for a label outside [0, V)
  if (entropy) entropy[t] = (log2s - mean_t) * kLn2;
  if (row_lse) row_lse[t] = (m.k + log2s) * kLn2;
  if (row_ez) row_ez[t] = (m.k + mean_t) * kLn2;
  if (vmax) vmax[t] = m.k / c;
  if (vmin) vmin[t] = m.n;
}

// What carry mode needs per panel row, written by k_token_loss
struct CarryOut {
  float* row_factor;   // [rows] d(logits) of the row = row_factor * stored row (with the label entry patched, below)
  uint16_t* panel;     // the label entry of each row is overwritten so that the product gives (g / T) (1 - p_label)
  int64_t panel_ld;
  int32_t* redo_flag;  // set to 1 when a token with a gradient has a label log-prob below kCarryMinLogp
};

struct TokenLossArgs {
  const float* prox_logp;
  const float* adv;
  const uint8_t* mask_eff;
  const float* behave_w;
  const int32_t* n_valid;
  const float* grad_scale;
  float* logp;
  float* entropy;
  float* stat_loss;
  float* ratio;
  uint8_t* flags;
  float* vmax;  // nullable (together with vmin): largest / smallest raw logit of the row
  float* vmin;
  aa_ppo_params P;
  int64_t act;  // tokens of the chunk that are inside T_active
};

// Training step, after the forward tiles of a chunk: log-prob, entropy, per-token loss outputs (as the fused logits
// kernel writes them, areal/utils/functional/functional.py:505-558) and g = d(scaled loss) / d(logp); then what the
// backward needs: g and the row's logsumexp per token (recompute), or the row coefficients per panel row (carry).
__global__ __launch_bounds__(1024) void k_token_loss(const float* __restrict__ pk, const float* __restrict__ ps,
                                                     const float* __restrict__ pu, const float* __restrict__ pn,
                                                     const float* __restrict__ xy, int blocks,
                                                     int64_t pitch_t, int n_tok, int V, float c, float inv_t,
                                                     const int64_t* __restrict__ labels, TokenLossArgs a,
                                                     const int32_t* __restrict__ out_rows, float* __restrict__ g_tok,
                                                     float* __restrict__ lse_tok, CarryOut carry) {
  __shared__ float smem[kMergeSmemFloats];
  const int t = blockIdx.x * 64 + (threadIdx.x & 63);
  const Merged m = merge_blocks(pk, ps, pu, pn, blocks, pitch_t, t, t < n_tok, smem);
  if (t >= n_tok || threadIdx.x >= 64) return;
  const float log2s = fast_log2(m.s);
  const float lp = (fmaf(xy[t], c, -m.k) - log2s) * kLn2;
  a.logp[t] = lp;
  if (a.entropy) a.entropy[t] = (log2s - m.u / m.s) * kLn2;
  if (a.vmax) a.vmax[t] = m.k / c;
  if (a.vmin) a.vmin[t] = m.n;
  float g = 0.f;
  if (t < a.act) {
    int n = *a.n_valid;
    float fn;
    if (a.P.loss_kind == AA_LOSS_NLL) {
      fn = (float)n + 1e-5f;  // the supervised loss divides by 1e-5 + count (areal/trainer/sft/lm_engine.py:96)
    } else {
      fn = (float)(n < 1 ? 1 : n);
    }
    const float gscale = a.grad_scale ? *a.grad_scale : 1.f;
    const bool on = a.mask_eff[t] != 0;
    if (a.P.loss_kind == AA_LOSS_NLL) {
      a.stat_loss[t] = on ? -lp : 0.f;
      a.ratio[t] = 0.f;
      a.flags[t] = 0;
      g = on ? (-1.f / fn) * gscale : 0.f;
    } else {
      // the clipped surrogate sees a ratio of zero at masked tokens; SAPO's ratio is not masked (functional.py:509, 600)
      const bool sapo = a.P.loss_kind == AA_LOSS_SAPO;
      const float r = (on || sapo) ? expf(lp - a.prox_logp[t]) : 0.f;
      const Surrogate sg = sapo ? sapo_surrogate(r, a.adv[t], a.P)
                                : surrogate(r, a.adv[t], a.P.has_behave_weight ? a.behave_w[t] : 1.f, a.P);
      a.stat_loss[t] = sg.loss;
      a.ratio[t] = r;
      a.flags[t] = (uint8_t)(((sg.clip && on) ? 1 : 0) | ((sg.dual && on) ? 2 : 0));
      g = on ? (sg.dloss_dr * r / fn) * gscale : 0.f;
    }
  }
  if (g_tok) g_tok[t] = g;
  if (lse_tok) lse_tok[t] = (m.k + log2s) * kLn2;
  if (carry.row_factor) {
    const int r = out_rows ? out_rows[t] : t;
    if (r >= 0) {
      // stored row: q_v = p_v / p_label.  d(logits)_v = (g / T) (onehot_v - p_v) = f q_v with f = -(g / T) p_label for
      // every v but the label, whose entry is replaced by 1 - 1 / p_label: f (1 - 1 / p_label) = (g / T) (1 - p_label)
      const float kref = xy[t] * c;                                   // as the tiles formed it
      const float p_label = fast_exp2(kref - (m.k + log2s));
      const float f = g == 0.f ? 0.f : -(g * inv_t) * p_label;  // g == 0: whatever the row holds counts for nothing
      carry.row_factor[r] = f;
      const int64_t y = labels[t];
      // a row without gradient keeps its label entry (1): 1 - 1 / p_label is not finite for a label more than 88 nats
      // unlikely, and d_weight multiplies every entry of the row, by a zero there
      if (g != 0.f && y >= 0 && y < V) {
        const float patched = -expm1f(-lp);
        carry.panel[(int64_t)r * carry.panel_ld + y] = (uint16_t)(Elem<AA_BF16>::pack(patched, 0.f) & 0xffffu);
      }
      // redo by recompute when the stored form cannot carry the row: the ratios would overflow (label too unlikely), or
      // the factor is so small that factor x hidden, which d_weight takes rounded to bf16, leaves the normal range
      if (g != 0.f && (lp < kCarryMinLogp || fabsf(f) < kCarryMinFactor)) *carry.redo_flag = 1;
    }
  }
}

// After the conditional recompute of a flagged chunk the panel holds d(logits) itself: every row factor becomes 1.
__global__ __launch_bounds__(256) void k_unit_factors(float* __restrict__ row_factor, int rows, const int32_t* __restrict__ flag) {
  if (*flag == 0) return;
  const int r = blockIdx.x * 256 + threadIdx.x;
  if (r < rows) row_factor[r] = 1.f;
}

// Backward of the stand-alone op in carry form: what k_token_loss does for the rows of the training step, for upstream
// gradients that only exist once the forward has returned.  Per token t of the chunk with a panel row r: the row's
// factor -(g / T) p_label from the saved log-prob, the label entry patched to 1 - 1 / p_label, and the chunk's redo
// flag when the stored form cannot carry the row.
__global__ __launch_bounds__(256) void k_carry_factors(const float* __restrict__ logp, const float* __restrict__ g_logp,
                                                       const int64_t* __restrict__ labels,
                                                       const int32_t* __restrict__ out_rows, int n_tok, int V, float inv_t,
                                                       CarryOut carry) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= n_tok) return;
  const int r = out_rows ? out_rows[t] : t;
  if (r < 0) return;
  const float lp = logp[t], g = g_logp[t];
  const float f = g == 0.f ? 0.f : -(g * inv_t) * fast_exp2(lp * kLog2e);
  carry.row_factor[r] = f;
  const int64_t y = labels[t];
  if (g != 0.f && y >= 0 && y < V)
    carry.panel[(int64_t)r * carry.panel_ld + y] = (uint16_t)(Elem<AA_BF16>::pack(-expm1f(-lp), 0.f) & 0xffffu);
  if (g != 0.f && (lp < kCarryMinLogp || fabsf(f) < kCarryMinFactor)) *carry.redo_flag = 1;
}

// ---- the d_hidden product cut along K: into how many parts ---------------------------------------------------------
// Into how many parts along K a product of `tiles` tiles and `slices` K slices is cut (1: not at all): the number of
// parts, up to kMaxSplits, that shortens the time in rounds of tiles, ceil(tiles * parts / units) / parts, the most,
// with 0.03 rounds charged per part for writing and adding its fp32 plane; at least 5 % have to be won, and a part
// keeps at least 64 slices.  In whole numbers (rounds x 1200) so that the host and the device (k_compact_map, from a
// row count that only the device holds) come to the same answer.
constexpr int kMaxSplits = 4;
constexpr int kRoundsUnit = 1200;  // divisible by every number of parts
static_assert(kRoundsUnit % 2 == 0 && kRoundsUnit % 3 == 0 && kRoundsUnit % 4 == 0 && kMaxSplits <= 4, "rounds in whole numbers");
__host__ __device__ inline int choose_splits(int64_t tiles, int64_t slices, int units) {
  if (units <= 0 || tiles <= 0) return 1;
  int best = 1;
  int64_t best_rounds = (tiles + units - 1) / units * (kRoundsUnit * 95 / 100);  // one part, less the 5 % to be won
  for (int parts = 2; parts <= kMaxSplits && slices / parts >= 64; ++parts) {
    const int64_t r = (tiles * parts + units - 1) / units * (kRoundsUnit / parts) + (kRoundsUnit * 3 / 100) * parts;
    if (r < best_rounds) {
      best = parts;
      best_rounds = r;
    }
  }
  return best;
}

// ---- plain product C = B . A^T on the same main loop ---------------------------------------------------------------
// C [N, M] row-major with leading dimension ldc: C[n][m] = sum_k B[n][k] A[m][k]; AKM / BKM: the operand is stored
// K-major (see gemm_tn.h).  The operand whose rows are the columns of C goes first, because a lane of the accumulator layout owns one n and runs of four consecutive m: four
// neighbouring outputs of a row of C.  bf16 C: the tile is staged in LDS as [n][m] and leaves in 16-byte pieces,
// 512 contiguous bytes per row; row n of the product is written to row c_rows[n] of C when a row list is given.
// fp32 C: 16-byte stores straight from the registers; ACCUM adds to what C holds.
// BOUND: `bounds` holds the row-count words of the chunk (the number of panel rows in use is known to the device alone
// and is at most the N or K the host launched with).  kBoundN: only the tiles over the rows of B in use run, numbered
// as a grid of just those tiles (the walk over the XCDs is the one a grid sized by the host has; the other workgroups
// return at once), and the whole grid returns when the product over those rows is one that k_gemm_splitk, queued
// beside it, cuts along K.  kBoundK: the contraction stops at the count rounded up to a whole K slice (the rows up to
// there are zero).  kBoundNone is the kernel without any of this.
template <bool AKM, bool BKM, typename OutT, bool ACCUM, int BOUND>
__global__ __launch_bounds__(kThreads) void k_gemm_store(Operand A, Operand B, int K, int tiles_m, int tiles_n,
                                                         OutT* __restrict__ C, int64_t ldc,
                                                         const int32_t* __restrict__ c_rows,
                                                         const float* __restrict__ n_scale,
                                                         const int32_t* __restrict__ bounds) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  if constexpr (BOUND == kBoundN) {
    const int live = bounds[kRowsLive];
    tiles_n = live < tiles_n ? live : tiles_n;
    // the same decision in every thread of the workgroup
    if (bounds[kRowsSplits] != 1 || (int)blockIdx.x >= tiles_m * tiles_n) return;
  }
  int tm, tn;
  tile_of(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  if constexpr (BOUND == kBoundK) {
    const int kb = bounds[kRowsSliced];
    K = kb < K ? kb : K;
  }
  Acc acc;
  mainloop<AKM, BKM>(A, B, K, m0, n0, acc, lds);  // ends with a barrier: LDS is free
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int M = A.rows, N = B.rows;
  if constexpr (sizeof(OutT) == 2) {
    uint16_t* Z = (uint16_t*)lds;  // [256 n][kPanelPitch] bf16
    constexpr int PZ = kPanelPitch;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int nloc = wn * 128 + acc_col(nt, lane);
      // optional factor per row of C (a lane owns one n): applied to the fp32 sums, before the one rounding to bf16.  A
      // factor of zero gives a zero row whatever the sums hold (a row without gradient may have summed to infinity)
      const float f = (n_scale && n0 + nloc < N) ? n_scale[n0 + nloc] : 1.f;
      const bool dead = f == 0.f;
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          uint2 pk;
          pk.x = dead ? 0u : Elem<AA_BF16>::pack(acc.v[mt][nt][g4 * 4] * f, acc.v[mt][nt][g4 * 4 + 1] * f);
          pk.y = dead ? 0u : Elem<AA_BF16>::pack(acc.v[mt][nt][g4 * 4 + 2] * f, acc.v[mt][nt][g4 * 4 + 3] * f);
          *(uint2*)(Z + nloc * PZ + wm * 128 + mt * 32 + 8 * g4 + 4 * (lane >> 5)) = pk;
        }
    }
    int32_t* rows_lds = (int32_t*)(lds + 256 * PZ * 2);  // row of C of each of the tile's 256 n (-1: past the end)
    {
      const int n = n0 + tid;
      rows_lds[tid] = n < N ? (c_rows ? c_rows[n] : n) : -1;
    }
    __syncthreads();
    const int mc = (tid & 31) * 8, m = m0 + mc;  // M % 8 == 0 (M is a hidden size): a piece never straddles the end
    if (m < M) {
#pragma unroll 8
      for (int i = 0; i < 32; ++i) {
        const int nloc = (tid >> 5) + 8 * i;
        const int r = rows_lds[nloc];
        if (r >= 0) *(u32x4_t*)(C + (int64_t)r * ldc + m) = *(const u32x4_t*)(Z + nloc * PZ + mc);
      }
    }
  } else {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int n = n0 + wn * 128 + acc_col(nt, lane);
      if (n >= N) continue;
      float* row = (float*)C + (c_rows ? c_rows[n] : n) * ldc;
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int m = m0 + wm * 128 + mt * 32 + 8 * g4 + 4 * (lane >> 5);  // M % 4 == 0
          if (m >= M) continue;
          f32x4_t v = {acc.v[mt][nt][g4 * 4], acc.v[mt][nt][g4 * 4 + 1], acc.v[mt][nt][g4 * 4 + 2], acc.v[mt][nt][g4 * 4 + 3]};
          if (ACCUM) v += *(const f32x4_t*)(row + m);
          *(f32x4_t*)(row + m) = v;
        }
    }
  }
}

// ---- the same product cut along K ------------------------------------------------------------------------------
// d_hidden has few tiles (16 x rows / 256 at H = 4096): when their number is a little above a multiple of the compute
// units, the last round of tiles runs on a mostly idle chip and costs almost a whole round all the same (measured:
// 576 tiles = 2.25 rounds take 9.7 ms where 512 tiles take 6.9 ms).  Cut along K into `splits` parts, the tiles are
// `splits` times as many and as much shorter, so the last round wastes that much less.  Part s of tile (tm, tn) sums
// the K slices [s * per, (s + 1) * per) into its own fp32 plane; k_splitk_rows adds the planes in order.  Workgroups
// are numbered so that an XCD runs a contiguous range of (part, tile): the tiles that share operand slices in its L2
// are those of one part.
// BOUNDED (the rows of B in use are known to the device alone; `bounds`: the row-count words of the chunk): the tiles
// over those rows are numbered as a grid of just those, cut into the number of parts that the host would have chosen
// with that count; the workgroups beyond tiles x parts return at once, all of them when the product is not cut.
template <bool AKM, bool BKM, bool BOUNDED>
__global__ __launch_bounds__(kThreads) void k_gemm_splitk(Operand A, Operand B, int K, int tiles_m, int tiles_n, int splits,
                                                          float* __restrict__ part, int64_t ldc, int64_t plane,
                                                          const int32_t* __restrict__ bounds) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  if constexpr (BOUNDED) {
    const int live = bounds[kRowsLive];
    tiles_n = live < tiles_n ? live : tiles_n;
    splits = bounds[kRowsSplits];
    if (splits == 1 || (int)blockIdx.x >= tiles_m * tiles_n * splits) return;  // the same in every thread
  }
  const int tiles = tiles_m * tiles_n;
  const int q = xcd_contiguous(blockIdx.x, tiles * splits);
  const int split = q / tiles;
  int tm, tn;
  tile_at(q - split * tiles, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int nk = (K + BK - 1) / BK, per = (nk + splits - 1) / splits;
  const int k_begin = split * per * BK;
  int k_len = K - k_begin;
  k_len = k_len < 0 ? 0 : (k_len > per * BK ? per * BK : k_len);  // 0: this part has nothing, its plane gets zeros
  const int64_t shift = k_len > 0 ? k_begin : 0;
  A.ptr += AKM ? shift * A.ld : shift;
  B.ptr += BKM ? shift * B.ld : shift;
  Acc acc;
  mainloop<AKM, BKM>(A, B, k_len, m0, n0, acc, lds);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int M = A.rows, N = B.rows;
  float* C = part + (int64_t)split * plane;
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    const int n = n0 + wn * 128 + acc_col(nt, lane);
    if (n >= N) continue;
    float* row = C + n * ldc;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int m = m0 + wm * 128 + mt * 32 + 8 * g4 + 4 * (lane >> 5);  // M % 4 == 0
        if (m >= M) continue;
        const f32x4_t v = {acc.v[mt][nt][g4 * 4], acc.v[mt][nt][g4 * 4 + 1], acc.v[mt][nt][g4 * 4 + 2], acc.v[mt][nt][g4 * 4 + 3]};
        *(f32x4_t*)(row + m) = v;
      }
  }
}

// out[c_rows[r], :] = bf16(n_scale[r] * (plane 0 + plane 1 + ...)[r, :]), the planes added in order; M % 8 == 0.
// c_rows == nullptr: row r itself (a negative entry: the row is dropped); n_scale == nullptr: 1.
// With `bounds` (the row-count words of the chunk, see k_gemm_splitk) only the rows in use are written, from the number
// of planes that kernel was cut into; none when it was not cut.
__global__ __launch_bounds__(256) void k_splitk_rows(const float* __restrict__ part, int splits, int64_t plane, int M,
                                                     const int32_t* __restrict__ c_rows, const float* __restrict__ n_scale,
                                                     uint16_t* __restrict__ out, int64_t ldo,
                                                     const int32_t* __restrict__ bounds) {
  const int64_t r = blockIdx.x;
  if (bounds) {
    splits = bounds[kRowsSplits];
    if (splits == 1 || r >= bounds[kRowsTotal]) return;
  }
  const int64_t dst = c_rows ? c_rows[r] : r;
  if (dst < 0) return;
  const float f = n_scale ? n_scale[r] : 1.f;
  for (int m = threadIdx.x * 8; m < M; m += 256 * 8) {
    float a[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = 0.f;
    for (int sp = 0; sp < splits; ++sp) {
      const float* src = part + (int64_t)sp * plane + r * M + m;
      const f32x4_t lo = *(const f32x4_t*)src, hi = *(const f32x4_t*)(src + 4);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[i] += lo[i];
        a[4 + i] += hi[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = f == 0.f ? 0.f : a[i] * f;  // a zero factor gives a zero row whatever the sums hold
    store8<AA_BF16>(out + dst * ldo, m, a);
  }
}

// ---- tokens without gradient are left out of the backward GEMMs -------------------------------------------------
// A token whose loss mask is zero has d(loss)/d(logits) == 0: its row adds nothing to d_weight and its d_hidden row
// is zero.  k_compact_map numbers the tokens of a chunk that do have a mask (in order): out_rows[t] = position of
// token t among them, or -1; act_rows[position] = t.  `limit` is the count the host sized the GEMMs with; tokens
// beyond it are dropped.  A host count larger than what the mask holds leaves positions without a token: they get
// act_rows = -1 (the gathers then produce zero rows and the scatters skip them) and a row factor of zero when factors
// are in use; the true count goes to total_out (the four row-count words of the chunk; dh_tiles_m, dh_slices and units
// describe the d_hidden product for choose_splits), and k_clear_surplus_rows, launched behind this kernel, clears their
// panel rows, which no tile writes, so that nothing stale (possibly not even finite) enters the d_weight product.
// One workgroup; mask has `act` entries (tokens at and after `act` have none).
__global__ __launch_bounds__(1024) void k_compact_map(const uint8_t* __restrict__ mask, int act, int n_tok, int limit,
                                                      int32_t* __restrict__ out_rows, int32_t* __restrict__ act_rows,
                                                      float* __restrict__ row_factor, int32_t* __restrict__ total_out,
                                                      int dh_tiles_m, int dh_slices, int units) {
  __shared__ int wave_sum[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per = (n_tok + 1023) / 1024;
  const int beg = tid * per, end = min(beg + per, n_tok);
  int cnt = 0;
  for (int t = beg; t < end; ++t) cnt += (t < act && mask[t] != 0) ? 1 : 0;
  int incl = cnt;  // inclusive scan over the wave, then over the 16 waves
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  if (lane == 63) wave_sum[wave] = incl;
  __syncthreads();
  int base = 0;
  for (int w = 0; w < wave; ++w) base += wave_sum[w];
  int pos = base + incl - cnt;
  for (int t = beg; t < end; ++t) {
    const bool on = (t < act && mask[t] != 0) && pos < limit;
    out_rows[t] = on ? pos : -1;
    if (on) act_rows[pos] = t;
    pos += (t < act && mask[t] != 0) ? 1 : 0;
  }
  int total = 0;
  for (int w = 0; w < 16; ++w) total += wave_sum[w];
  if (tid == 0) {
    const int rows = total < limit ? total : limit;
    const int live = (rows + BN - 1) / BN;
    total_out[kRowsTotal] = rows;
    total_out[kRowsLive] = live;
    total_out[kRowsSliced] = rows > 0 ? (rows + BK - 1) / BK * BK : BK;
    total_out[kRowsSplits] = choose_splits((int64_t)dh_tiles_m * live, dh_slices, units);
  }
  for (int p = total + tid; p < limit; p += 1024) {  // the usual case: none
    act_rows[p] = -1;
    if (row_factor) row_factor[p] = 0.f;
  }
}

// Panel rows [*total, limit) are rows without a token (see k_compact_map): cleared, one workgroup per row at a time.
// In the usual case (*total == limit) every workgroup returns at once.
// With `bounded` the kernels that read the panel stop at *total themselves (rounded up to a K slice of the d_weight
// product), and only the rows up to there are cleared.
__global__ __launch_bounds__(256) void k_clear_surplus_rows(const int32_t* __restrict__ total, int limit, int bounded,
                                                            u32x4_t* __restrict__ panel, int64_t panel_ld) {
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  const int64_t vec = panel_ld / 8;
  if (bounded) {
    const int up = total[kRowsSliced];
    limit = up < limit ? up : limit;
  }
  for (int64_t r = (int64_t)*total + blockIdx.x; r < limit; r += gridDim.x)
    for (int64_t i = threadIdx.x; i < vec; i += 256) panel[r * vec + i] = zero;
}

static int compute_units();

// numbering of the tokens with a panel row, and the rows without a token cleared (both kernels); H and V are those of
// the lm_head (they shape the d_hidden product that the row-count words describe)
static void launch_compact_map(hipStream_t st, const uint8_t* mask, int64_t act, int64_t n_tok, int64_t limit,
                               int32_t* out_rows, int32_t* act_rows, float* row_factor, int32_t* total_word,
                               uint16_t* panel, int64_t panel_ld, int64_t H, int64_t V, bool bounded = false) {
  hipLaunchKernelGGL(k_compact_map, dim3(1), dim3(1024), 0, st, mask, (int)act, (int)n_tok, (int)limit, out_rows, act_rows,
                     row_factor, total_word, (int)((H + BM - 1) / BM), (int)((V + BK - 1) / BK), compute_units());
  const int64_t blocks = bounded ? (limit < BK ? limit : BK) : (limit < 512 ? limit : 512);
  if (blocks > 0)
    hipLaunchKernelGGL(k_clear_surplus_rows, dim3((unsigned)blocks), dim3(256), 0, st, total_word, (int)limit,
                       bounded ? 1 : 0, (u32x4_t*)panel, panel_ld);
}

// dst[r, :] = scale[r] * src[rows[r], :] (H % 8 == 0); rows == nullptr: row r itself (a negative entry: a zero row);
// scale == nullptr: 1;
// run_if, when given: nothing happens unless *run_if != 0
__global__ __launch_bounds__(256) void k_gather_rows(const u32x4_t* __restrict__ src, const int32_t* __restrict__ rows,
                                                     u32x4_t* __restrict__ dst, int h_vec,
                                                     const float* __restrict__ scale, const int32_t* __restrict__ run_if) {
  if (run_if && *run_if == 0) return;
  const int64_t r = blockIdx.x;
  const int64_t t = rows ? rows[r] : r;
  if (t < 0) {  // a position without a token
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    for (int j = threadIdx.x; j < h_vec; j += 256) dst[r * h_vec + j] = zero;
    return;
  }
  if (!scale) {
    for (int j = threadIdx.x; j < h_vec; j += 256) dst[r * h_vec + j] = src[t * h_vec + j];
    return;
  }
  const float f = scale[r];
  for (int j = threadIdx.x; j < h_vec; j += 256) {
    float x[8];
    load8<AA_BF16>((const uint16_t*)(src + t * h_vec), (int64_t)j * 8, x);
#pragma unroll
    for (int q = 0; q < 8; ++q) x[q] *= f;
    store8<AA_BF16>((uint16_t*)(dst + r * h_vec), (int64_t)j * 8, x);
  }
}

__global__ __launch_bounds__(256) void k_zero16(u32x4_t* __restrict__ p, int64_t n_vec) {
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_vec; i += step) p[i] = zero;
}

static void launch_zero(hipStream_t st, void* p, int64_t bytes) {  // bytes % 16 == 0
  const int64_t n = bytes / 16;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (blocks > 0) hipLaunchKernelGGL(k_zero16, dim3((unsigned)blocks), dim3(256), 0, st, (u32x4_t*)p, n);
}

// fp32 -> bf16 (round to nearest even), 8 elements per thread; n % 8 == 0

__global__ __launch_bounds__(256) void k_f32_to_bf16(const f32x4_t* __restrict__ src, u32x4_t* __restrict__ dst,
                                                     int64_t n8) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  const f32x4_t a = __builtin_nontemporal_load(src + 2 * i), b = __builtin_nontemporal_load(src + 2 * i + 1);
  u32x4_t o;
  o[0] = Elem<AA_BF16>::pack(a[0], a[1]);
  o[1] = Elem<AA_BF16>::pack(a[2], a[3]);
  o[2] = Elem<AA_BF16>::pack(b[0], b[1]);
  o[3] = Elem<AA_BF16>::pack(b[2], b[3]);
  __builtin_nontemporal_store(o, dst + i);
}

// ---- workspace ---------------------------------------------------------------------------------------------------

struct Workspace {
  int64_t chunk, blocks;                // tokens per chunk, 128-row vocabulary blocks
  int64_t off_pk, off_ps, off_pu;       // block partials [blocks][chunk]
  int64_t panel_ld;                     // pitch of the panel: V rounded up to 8 elements
  int64_t off_xy, off_g, off_lse;       // per token of the chunk: label logit, g, logsumexp
  int64_t fwd_bytes;                    // what the forward alone needs
  int64_t off_pn;                       // smallest logit per block [blocks][chunk] (only when the extrema are asked for)
  int64_t fwd_stats_bytes;              // what the forward needs when it also returns the extrema of the logits
  int64_t off_rowf, off_flag;           // carry mode: factor per panel row; the chunk's redo flag
  int64_t off_total;                    // number of tokens the mask of the chunk really holds (k_compact_map)
  int64_t off_rows;                     // out_rows, act_rows (2 x chunk int32)
  int64_t off_panel;                    // d(logits) rows [chunk, V]
  int64_t off_hc;                       // the hidden rows of the tokens with gradient, closed up [chunk, H]
  int64_t off_dw;                       // fp32 accumulator of a bf16 d_weight when there is more than one chunk
  int64_t off_dhp;                      // fp32 planes of a d_hidden product cut along K [kMaxSplits][chunk, H]
  int64_t bytes;
};

// external_panel: the d(logits) rows live in an array of the caller's (the op that keeps them from its forward to its
// backward), not in the workspace
static Workspace plan(int64_t T, int64_t H, int64_t V, bool external_panel = false) {
  Workspace w{};
  auto up = [](int64_t x) { return (x + 255) / 256 * 256; };
  w.chunk = T < kChunkTokens ? round_up(T, 256) : kChunkTokens;
  w.blocks = 2 * ((V + BM - 1) / BM);
  int64_t off = 0;
  w.off_pk = off;  off += up(w.blocks * w.chunk * 4);
  w.off_ps = off;  off += up(w.blocks * w.chunk * 4);
  w.off_pu = off;  off += up(w.blocks * w.chunk * 4);
  w.off_xy = off;  off += up(w.chunk * 4);
  w.off_g = off;   off += up(w.chunk * 4);
  w.off_lse = off; off += up(w.chunk * 4);
  w.fwd_bytes = off;
  w.off_pn = off;  off += up(w.blocks * w.chunk * 4);
  w.fwd_stats_bytes = off;
  w.off_rowf = off;    off += up(w.chunk * 4);  // factor per panel row (carry mode)
  w.off_flag = off;    off += 256;              // the chunk's "redo by recompute" flag
  w.off_total = off;   off += 256;
  w.off_rows = off;    off += up(2 * w.chunk * 4);
  w.panel_ld = round_up(V, 8);
  w.off_panel = off;   off += external_panel ? 0 : up(w.chunk * w.panel_ld * 2);
  w.off_hc = off;      off += up(w.chunk * H * 2);
  w.off_dw = off;      off += T > w.chunk ? up(V * H * 4) : 0;
  w.off_dhp = off;     off += up(kMaxSplits * w.chunk * H * 4);
  w.bytes = off;
  return w;
}

static bool shapes_ok(int64_t T, int64_t H, int64_t V) {
  // 256 rows of any operand must stay below 2^30 elements (32-bit byte offsets inside a tile)
  return T > 0 && H > 0 && V > 0 && (H % 8) == 0 && T < (1 << 30) && V < (1 << 22) && H < (1 << 22);
}

// The tile kernels use all 160 KiB of LDS: allow it once per kernel and device.
template <typename Kern>
static bool allow_big_lds(Kern k) {
  return hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) == hipSuccess;
}

static bool prepare_kernels() {
  constexpr int kMaxDevices = 64;
  static bool done[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return false;
  if (done[dev]) return true;
  const bool ok = allow_big_lds(k_lmhead_tiles<kModeStats>) && allow_big_lds(k_lmhead_tiles<kModeStatsCarry>) &&
                  allow_big_lds(k_lmhead_tiles<kModeRecompute>) &&
                  allow_big_lds(k_gemm_store<true, false, uint16_t, false, kBoundNone>) &&
                  allow_big_lds(k_gemm_store<true, false, uint16_t, false, kBoundN>) &&
                  allow_big_lds(k_gemm_store<true, true, uint16_t, false, kBoundNone>) &&
                  allow_big_lds(k_gemm_store<true, true, uint16_t, false, kBoundK>) &&
                  allow_big_lds(k_gemm_store<true, true, float, false, kBoundNone>) &&
                  allow_big_lds(k_gemm_store<true, true, float, false, kBoundK>) &&
                  allow_big_lds(k_gemm_store<true, true, float, true, kBoundNone>) &&
                  allow_big_lds(k_gemm_store<true, true, float, true, kBoundK>) &&
                  allow_big_lds(k_gemm_splitk<true, false, false>) && allow_big_lds(k_gemm_splitk<true, false, true>);
  done[dev] = ok;
  return ok;
}

// compute units of the current device (0 if unknown), asked for once per device
static int compute_units() {
  constexpr int kMaxDevices = 64;
  static int units[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  if (units[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
    units[dev] = n > 0 ? n : -1;
  }
  return units[dev] > 0 ? units[dev] : 0;
}

template <int MODE>
static void launch_tiles(hipStream_t st, const void* weight, const uint16_t* hid, int64_t n_tok, int64_t H, int64_t V,
                         const TileArgs& a) {
  const int tiles_m = (int)((V + BM - 1) / BM), tiles_n = (int)((n_tok + BN - 1) / BN);
  Operand W{(const uint16_t*)weight, H, (int)V};
  Operand Hd{hid, H, (int)n_tok};
  hipLaunchKernelGGL(k_lmhead_tiles<MODE>, dim3((unsigned)(tiles_m * tiles_n)), dim3(kThreads), kLdsBytes, st,
                     W, Hd, (int)H, tiles_m, tiles_n, a);
}

// C [N, M] = B . A^T over K (rows of C through c_rows when given); lda / ldb: leading dimensions of the arrays as stored.
// BOUND / bounds: see k_gemm_store.
template <bool AKM, bool BKM, typename OutT, bool ACCUM, int BOUND = kBoundNone>
static void launch_gemm(hipStream_t st, const uint16_t* A, int64_t lda, int64_t M, const uint16_t* B, int64_t ldb, int64_t N,
                        int64_t K, OutT* C, int64_t ldc, const int32_t* c_rows = nullptr,
                        const float* n_scale = nullptr, const int32_t* bounds = nullptr) {
  const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
  Operand a{A, lda, (int)M}, b{B, ldb, (int)N};
  hipLaunchKernelGGL((k_gemm_store<AKM, BKM, OutT, ACCUM, BOUND>), dim3((unsigned)(tiles_m * tiles_n)), dim3(kThreads),
                     kLdsBytes, st, a, b, (int)K, tiles_m, tiles_n, C, ldc, c_rows, n_scale, bounds);
}

// d_weight (+)= ds^T . hidden rows in the dtype and mode asked for; with `bounds` the contraction stops at the rows in use
template <int BOUND>
static void launch_d_weight(hipStream_t st, const uint16_t* hid_rows, int64_t H, const uint16_t* ds, int64_t ldp, int64_t V,
                            int64_t n_rows, void* d_weight, bool dw_f32, bool first, const int32_t* bounds) {
  if (!dw_f32)
    launch_gemm<true, true, uint16_t, false, BOUND>(st, hid_rows, H, H, ds, ldp, V, n_rows, (uint16_t*)d_weight, H, nullptr,
                                                    nullptr, bounds);
  else if (first)
    launch_gemm<true, true, float, false, BOUND>(st, hid_rows, H, H, ds, ldp, V, n_rows, (float*)d_weight, H, nullptr,
                                                 nullptr, bounds);
  else
    launch_gemm<true, true, float, true, BOUND>(st, hid_rows, H, H, ds, ldp, V, n_rows, (float*)d_weight, H, nullptr, nullptr,
                                                bounds);
}

// The two GEMMs that contract the d(logits) rows ds [n_rows, V] of one token chunk, ds = row_factor[r] * panel[r, :]
// (row_factor == nullptr: the panel holds d(logits) itself):
//   d_hidden rows [n_rows, H] = ds . W                  contraction over V: panel K-contiguous, W [V, H] K-major;
//                                                       the factor multiplies the fp32 sums in the epilogue
//   d_weight [V, H] (+)= ds^T . hidden rows             contraction over the rows: both arrays K-major; the factor
//                                                       goes into the copy of the hidden rows
// No transposed copy of anything is made.  token_of_row, when given, lists the tokens of the chunk that the n_rows
// rows belong to (tokens without gradient were left out): their hidden rows are closed up first, and the d_hidden rows
// go to those tokens (the caller has cleared the others).
static void panel_gradients(hipStream_t st, const Workspace& w, char* ws, const uint16_t* ds, const void* weight,
                            const uint16_t* hid, const int32_t* token_of_row, const float* row_factor, int64_t n_rows,
                            int64_t H, int64_t V, uint16_t* d_hidden_chunk, void* d_weight, bool dw_f32, bool first,
                            const int32_t* rows_in_use = nullptr) {
  const uint16_t* hid_rows = hid;
  if (token_of_row || row_factor) {
    uint16_t* hc = (uint16_t*)(ws + w.off_hc);
    hipLaunchKernelGGL(k_gather_rows, dim3((unsigned)n_rows), dim3(256), 0, st, (const u32x4_t*)hid, token_of_row,
                       (u32x4_t*)hc, (int)(H / 8), row_factor, (const int32_t*)nullptr);
    hid_rows = hc;
  }
  const int64_t ldp = w.panel_ld;
  {
    const int tiles_m = (int)((H + BM - 1) / BM), tiles_n = (int)((n_rows + BN - 1) / BN);
    const int64_t slices = (V + BK - 1) / BK;
    const int units = compute_units();
    float* part = (float*)(ws + w.off_dhp);
    const int64_t plane = n_rows * H;
    Operand a{(const uint16_t*)weight, H, (int)H}, b{ds, ldp, (int)n_rows};
    if (rows_in_use) {
      // the row count is on the device alone (n_rows is its upper bound): both forms of the product are queued, the
      // row-count words say whether the product is cut along the vocabulary and into how many parts (what the host
      // would have chosen with that count), and the form that is not in turn returns at once
      int64_t cut_groups = 0, cut_rows = 0;  // the largest grid, and the most rows, the cut product can come with
      for (int tn = 1; tn <= tiles_n; ++tn) {
        const int parts = choose_splits((int64_t)tiles_m * tn, slices, units);
        if (parts == 1) continue;
        if ((int64_t)tiles_m * tn * parts > cut_groups) cut_groups = (int64_t)tiles_m * tn * parts;
        cut_rows = (int64_t)tn * BN < n_rows ? (int64_t)tn * BN : n_rows;
      }
      launch_gemm<true, false, uint16_t, false, kBoundN>(st, (const uint16_t*)weight, H, H, ds, ldp, n_rows, V,
                                                         d_hidden_chunk, H, token_of_row, row_factor, rows_in_use);
      if (cut_groups) {
        hipLaunchKernelGGL((k_gemm_splitk<true, false, true>), dim3((unsigned)cut_groups), dim3(kThreads), kLdsBytes, st, a,
                           b, (int)V, tiles_m, tiles_n, 0, part, H, plane, rows_in_use);
        hipLaunchKernelGGL(k_splitk_rows, dim3((unsigned)cut_rows), dim3(256), 0, st, part, 0, plane, (int)H, token_of_row,
                           row_factor, d_hidden_chunk, H, rows_in_use);
      }
    } else {
      const int splits = choose_splits((int64_t)tiles_m * tiles_n, slices, units);
      if (splits == 1) {
        launch_gemm<true, false, uint16_t, false>(st, (const uint16_t*)weight, H, H, ds, ldp, n_rows, V, d_hidden_chunk, H,
                                                  token_of_row, row_factor);
      } else {
        hipLaunchKernelGGL((k_gemm_splitk<true, false, false>), dim3((unsigned)(tiles_m * tiles_n * splits)), dim3(kThreads),
                           kLdsBytes, st, a, b, (int)V, tiles_m, tiles_n, splits, part, H, plane, (const int32_t*)nullptr);
        hipLaunchKernelGGL(k_splitk_rows, dim3((unsigned)n_rows), dim3(256), 0, st, part, splits, plane, (int)H,
                           token_of_row, row_factor, d_hidden_chunk, H, (const int32_t*)nullptr);
      }
    }
  }
  if (rows_in_use)
    launch_d_weight<kBoundK>(st, hid_rows, H, ds, ldp, V, n_rows, d_weight, dw_f32, first, rows_in_use);
  else
    launch_d_weight<kBoundNone>(st, hid_rows, H, ds, ldp, V, n_rows, d_weight, dw_f32, first, nullptr);
}

// Recompute: d(logits) of the panel rows from the logits tiles formed again.  With a row map only the hidden rows that
// have a panel row are multiplied (gathered first); `a` carries the per-token inputs of the chunk.  With run_if the
// kernels are enqueued but do nothing unless *run_if != 0 when they start.
static void recompute_panel(hipStream_t st, const Workspace& w, char* ws, uint16_t* panel, const void* weight,
                            const uint16_t* hid, int64_t n_tok, const int32_t* token_of_row, int64_t rows, int64_t H,
                            int64_t V, TileArgs a, const int32_t* run_if = nullptr, const int32_t* rows_in_use = nullptr) {
  a.panel = panel;
  a.panel_ld = w.panel_ld;
  a.out_rows = nullptr;
  a.run_if = run_if;
  a.n_bound = token_of_row ? rows_in_use : nullptr;
  if (!token_of_row) {
    a.col_tokens = nullptr;
    launch_tiles<kModeRecompute>(st, weight, hid, n_tok, H, V, a);
    return;
  }
  uint16_t* hc = (uint16_t*)(ws + w.off_hc);
  hipLaunchKernelGGL(k_gather_rows, dim3((unsigned)rows), dim3(256), 0, st, (const u32x4_t*)hid, token_of_row, (u32x4_t*)hc,
                     (int)(H / 8), (const float*)nullptr, run_if);
  a.col_tokens = token_of_row;
  launch_tiles<kModeRecompute>(st, weight, hc, rows, H, V, a);
}

// d_weight of dtype AA_F32 is accumulated in place.  A bf16 d_weight is written by the GEMM itself when there is one
// chunk, and otherwise accumulated in fp32 in the workspace and rounded once at the end.
struct WeightGrad {
  void* acc;    // what the GEMMs write
  bool acc_f32;
  bool convert; // acc is the workspace buffer: round it into the caller's bf16 array at the end
};

static WeightGrad weight_grad(const Workspace& w, char* ws, void* d_weight, int dtype, int64_t T) {
  if (dtype == AA_F32) return {d_weight, true, false};
  if (T <= w.chunk) return {d_weight, false, false};
  return {ws + w.off_dw, true, true};
}

static void finish_weight_grad(hipStream_t st, const WeightGrad& g, void* d_weight, int64_t V, int64_t H) {
  if (!g.convert) return;
  const int64_t n8 = V * H / 8;
  hipLaunchKernelGGL(k_f32_to_bf16, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, st, (const f32x4_t*)g.acc,
                     (u32x4_t*)d_weight, n8);
}

static TileArgs stats_args(const Workspace& w, char* ws, const int64_t* labels, float inv_t, bool want_min) {
  TileArgs a{};
  a.pk = (float*)(ws + w.off_pk);
  a.ps = (float*)(ws + w.off_ps);
  a.pu = (float*)(ws + w.off_pu);
  a.pn = want_min ? (float*)(ws + w.off_pn) : nullptr;
  a.xy = (float*)(ws + w.off_xy);
  a.labels = labels;
  a.pitch_t = w.chunk;
  a.c = kLog2e * inv_t;
  a.inv_t = inv_t;
  return a;
}

}  // namespace lmhead
}  // namespace aa

using namespace aa;
using namespace aa::lmhead;

extern "C" int64_t aa_lmhead_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  if (!shapes_ok(T, H, V)) return -1;
  return plan(T, H, V).bytes;
}

extern "C" int64_t aa_lmhead_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  if (!shapes_ok(T, H, V)) return -1;
  return plan(T, H, V).fwd_bytes;
}

extern "C" int64_t aa_lmhead_fwd_stats_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  if (!shapes_ok(T, H, V)) return -1;
  return plan(T, H, V).fwd_stats_bytes;
}

extern "C" int64_t aa_lmhead_chunk_tokens(void) { return kChunkTokens; }

extern "C" int aa_lmhead_prepare(void) { return prepare_kernels() ? AA_OK : AA_ERR_LAUNCH; }

extern "C" int aa_lmhead_fwd(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                             const int64_t* labels, float inv_temperature, float* logp, float* entropy,
                             float* row_lse, float* row_ez, float* vocab_max, float* vocab_min, void* workspace,
                             int64_t workspace_bytes, void* stream) {
  if (!hidden || !weight || !labels || !logp || !workspace || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  if ((vocab_max != nullptr) != (vocab_min != nullptr)) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V)) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace) & 15) != 0) return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V);
  if (workspace_bytes < (vocab_min ? w.fwd_stats_bytes : w.fwd_bytes)) return AA_ERR_INVALID_ARGUMENT;
  if (!prepare_kernels()) return AA_ERR_LAUNCH;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  auto at = [](float* p, int64_t t0) { return p ? p + t0 : nullptr; };
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    const TileArgs a = stats_args(w, ws, labels + t0, inv_temperature, vocab_min != nullptr);
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    hipLaunchKernelGGL(k_label_logit, dim3((unsigned)((n_tok + 3) / 4)), dim3(256), 0, st, hid, (const uint16_t*)weight,
                       labels + t0, (int)n_tok, (int)H, (int)V, a.xy, (int32_t*)nullptr);
    launch_tiles<kModeStats>(st, weight, hid, n_tok, H, V, a);
    hipLaunchKernelGGL(k_combine, dim3((unsigned)((n_tok + 63) / 64)), dim3(1024), 0, st, a.pk, a.ps, a.pu, a.pn, a.xy,
                       (int)w.blocks, a.pitch_t, (int)n_tok, a.c, logp + t0, at(entropy, t0), at(row_lse, t0),
                       at(row_ez, t0), at(vocab_max, t0), at(vocab_min, t0));
  }
  return launch_status();
}

// ---- forward for callers that cannot allocate ---------------------------------------------------------------------
// The softmax partials of aa_lmhead_fwd live in a device array of the library itself instead of a caller's workspace.
// Host code never uses the array by name (that is a host-side stand-in, not a device address): its address on a device
// is asked for once, with that device current, and kept.
constexpr int64_t kStaticScratchBytes = 32ll << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static char* static_scratch_on_current_device() {
  constexpr int kMaxDevices = 64;
  static char* ptr[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  if (!ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    ptr[dev] = (char*)p;
  }
  return ptr[dev];
}

// tokens per pass of aa_lmhead_fwd_static for a vocabulary of V: what fits the array (a multiple of 256), 0 if none do
static int64_t static_chunk_tokens(int64_t V) {
  const int64_t blocks = 2 * ((V + BM - 1) / BM);
  const int64_t per_token = (3 * blocks + 1) * 4;          // three planes of partials and the label logit
  int64_t c = (kStaticScratchBytes - 4 * 256) / per_token;  // four arrays, each starting on a 256-byte boundary
  c = c / 256 * 256;
  return c > kChunkTokens ? kChunkTokens : c;
}

extern "C" int64_t aa_lmhead_fwd_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int64_t aa_lmhead_fwd_static_max_vocab(void) {
  // largest V whose partials of 256 tokens fit: (3 * 2 * ceil(V / 256) + 1) * 4 * 256 + 1024 <= kStaticScratchBytes
  const int64_t blocks = ((kStaticScratchBytes - 1024) / (4 * 256) - 1) / 3;
  return blocks / 2 * BM;
}

extern "C" int aa_lmhead_fwd_static(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                                    const int64_t* labels, float inv_temperature, float* logp, float* entropy,
                                    float* row_lse, float* row_ez, void* stream) {
  if (!hidden || !weight || !labels || !logp || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V)) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight) & 15) != 0) return AA_ERR_INVALID_ARGUMENT;
  const int64_t chunk = static_chunk_tokens(V);
  if (chunk < 256) return AA_ERR_UNSUPPORTED;  // V > aa_lmhead_fwd_static_max_vocab(): not even 256 tokens fit
  if (!prepare_kernels()) return AA_ERR_LAUNCH;
  char* ws = static_scratch_on_current_device();
  if (!ws) return AA_ERR_LAUNCH;
  hipStream_t st = (hipStream_t)stream;
  auto up = [](int64_t x) { return (x + 255) / 256 * 256; };
  const int64_t blocks = 2 * ((V + BM - 1) / BM);
  TileArgs a{};
  a.pk = (float*)ws;
  a.ps = (float*)(ws + up(blocks * chunk * 4));
  a.pu = (float*)(ws + 2 * up(blocks * chunk * 4));
  a.xy = (float*)(ws + 3 * up(blocks * chunk * 4));
  a.pitch_t = chunk;
  a.c = kLog2e * inv_temperature;
  a.inv_t = inv_temperature;
  auto at = [](float* p, int64_t t0) { return p ? p + t0 : nullptr; };
  for (int64_t t0 = 0; t0 < T; t0 += chunk) {
    const int64_t n_tok = (T - t0) < chunk ? (T - t0) : chunk;
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    a.labels = labels + t0;
    hipLaunchKernelGGL(k_label_logit, dim3((unsigned)((n_tok + 3) / 4)), dim3(256), 0, st, hid, (const uint16_t*)weight,
                       labels + t0, (int)n_tok, (int)H, (int)V, a.xy, (int32_t*)nullptr);
    launch_tiles<kModeStats>(st, weight, hid, n_tok, H, V, a);
    hipLaunchKernelGGL(k_combine, dim3((unsigned)((n_tok + 63) / 64)), dim3(1024), 0, st, a.pk, a.ps, a.pu,
                       (const float*)nullptr, a.xy, (int)blocks, a.pitch_t, (int)n_tok, a.c, logp + t0, at(entropy, t0),
                       at(row_lse, t0), at(row_ez, t0), (float*)nullptr, (float*)nullptr);
  }
  return launch_status();
}

extern "C" int aa_lmhead_bwd(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                             const int64_t* labels, float inv_temperature, const float* row_lse, const float* row_ez,
                             const float* g_logp, const float* g_entropy, const uint8_t* row_has_gradient,
                             const int64_t* kept_per_chunk, void* d_hidden, void* d_weight, int d_weight_dtype,
                             void* workspace, int64_t workspace_bytes, void* stream) {
  if (!hidden || !weight || !labels || !row_lse || !g_logp || !d_hidden || !d_weight || !workspace)
    return AA_ERR_INVALID_ARGUMENT;
  if ((g_entropy && !row_ez) || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  if ((kept_per_chunk != nullptr) != (row_has_gradient != nullptr)) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V) || (d_weight_dtype != AA_F32 && d_weight_dtype != AA_BF16)) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace | (uintptr_t)d_hidden | (uintptr_t)d_weight) & 15))
    return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V);
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  if (!prepare_kernels()) return AA_ERR_LAUNCH;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  const WeightGrad dw = weight_grad(w, ws, d_weight, d_weight_dtype, T);
  int32_t* out_rows = (int32_t*)(ws + w.off_rows);
  int32_t* act_rows = out_rows + w.chunk;
  uint16_t* ws_panel = (uint16_t*)(ws + w.off_panel);
  bool first = true;  // no GEMM has written d_weight yet
  int64_t chunk_index = 0;
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk, ++chunk_index) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    uint16_t* dh = (uint16_t*)d_hidden + t0 * H;
    TileArgs a{};
    a.labels = labels + t0;
    a.c = kLog2e * inv_temperature;
    a.inv_t = inv_temperature;
    a.row_lse = row_lse + t0;
    a.row_ez = row_ez ? row_ez + t0 : nullptr;
    a.g_logp = g_logp + t0;
    a.g_entropy = g_entropy ? g_entropy + t0 : nullptr;
    if (!kept_per_chunk) {
      recompute_panel(st, w, ws, ws_panel, weight, hid, n_tok, nullptr, n_tok, H, V, a);
      panel_gradients(st, w, ws, ws_panel, weight, hid, nullptr, nullptr, n_tok, H, V, dh, dw.acc, dw.acc_f32, first);
      first = false;
      continue;
    }
    // rows whose upstream gradients are all zero are left out, as in aa_lmhead_ppo_fused
    int64_t kept = kept_per_chunk[chunk_index];
    const bool on_device = kept == AA_LMHEAD_COUNT_ON_DEVICE;  // the kernels stop at the count they find themselves
    kept = on_device ? n_tok : (kept < 0 ? 0 : (kept > n_tok ? n_tok : kept));
    if (kept == 0) {
      launch_zero(st, dh, n_tok * H * 2);
      continue;
    }
    int32_t* total_word = (int32_t*)(ws + w.off_total);
    const int32_t* rows_in_use = on_device ? total_word : nullptr;
    launch_compact_map(st, row_has_gradient + t0, n_tok, n_tok, kept, out_rows, act_rows, nullptr, total_word, ws_panel,
                       w.panel_ld, H, V, on_device);
    recompute_panel(st, w, ws, ws_panel, weight, hid, n_tok, act_rows, kept, H, V, a, nullptr, rows_in_use);
    launch_zero(st, dh, n_tok * H * 2);  // the rows of the other tokens
    panel_gradients(st, w, ws, ws_panel, weight, hid, act_rows, nullptr, kept, H, V, dh, dw.acc, dw.acc_f32, first,
                    rows_in_use);
    first = false;
  }
  if (first) launch_zero(st, dw.acc, V * H * (dw.acc_f32 ? 4 : 2));  // no row of the batch has a gradient
  finish_weight_grad(st, dw, d_weight, V, H);
  return launch_status();
}

extern "C" int64_t aa_lmhead_carry_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  if (!shapes_ok(T, H, V)) return -1;
  return plan(T, H, V, true).bytes;
}

extern "C" int64_t aa_lmhead_panel_pitch(int64_t V) { return round_up(V, 8); }

// rows of the panel that the chunks before chunk `upto` take: the tokens named by the host's counts, or all of them
static int64_t panel_rows_before(const int64_t* kept_per_chunk, int64_t chunk, int64_t T, int64_t upto) {
  int64_t rows = 0;
  for (int64_t c = 0; c < upto; ++c) {
    const int64_t n_tok = (T - c * chunk) < chunk ? (T - c * chunk) : chunk;
    int64_t k = kept_per_chunk ? kept_per_chunk[c] : n_tok;
    if (k == AA_LMHEAD_COUNT_ON_DEVICE) k = n_tok;  // the count is on the device alone: room for every token
    rows += k < 0 ? 0 : (k > n_tok ? n_tok : k);
  }
  return rows;
}

extern "C" int aa_lmhead_fwd_carry(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                                   const int64_t* labels, float inv_temperature, const uint8_t* row_has_gradient,
                                   const int64_t* kept_per_chunk, float* logp, float* entropy, float* row_lse,
                                   float* row_ez, float* vocab_max, float* vocab_min, void* panel, int64_t panel_rows,
                                   void* workspace, int64_t workspace_bytes, void* stream) {
  if (!hidden || !weight || !labels || !logp || !row_lse || !panel || !workspace || !(inv_temperature > 0.f))
    return AA_ERR_INVALID_ARGUMENT;
  if ((kept_per_chunk != nullptr) != (row_has_gradient != nullptr)) return AA_ERR_INVALID_ARGUMENT;
  if ((vocab_max != nullptr) != (vocab_min != nullptr)) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V)) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace | (uintptr_t)panel) & 15)) return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V, true);
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  const int64_t n_chunks = (T + w.chunk - 1) / w.chunk;
  if (panel_rows < panel_rows_before(kept_per_chunk, w.chunk, T, n_chunks)) return AA_ERR_INVALID_ARGUMENT;
  if (!prepare_kernels()) return AA_ERR_LAUNCH;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  int32_t* out_rows = (int32_t*)(ws + w.off_rows);
  int32_t* act_rows = out_rows + w.chunk;
  auto at = [](float* p, int64_t t0) { return p ? p + t0 : nullptr; };
  int64_t chunk_index = 0, row0 = 0;
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk, ++chunk_index) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    uint16_t* chunk_panel = (uint16_t*)panel + row0 * w.panel_ld;
    int64_t rows = n_tok;
    if (kept_per_chunk) {
      rows = kept_per_chunk[chunk_index];
      const bool on_device = rows == AA_LMHEAD_COUNT_ON_DEVICE;  // the chunk keeps room for every token
      rows = on_device ? n_tok : (rows < 0 ? 0 : (rows > n_tok ? n_tok : rows));
      launch_compact_map(st, row_has_gradient + t0, n_tok, n_tok, rows, out_rows, act_rows, nullptr,
                         (int32_t*)(ws + w.off_total), chunk_panel, w.panel_ld, H, V, on_device);
    }
    TileArgs a = stats_args(w, ws, labels + t0, inv_temperature, vocab_min != nullptr);
    a.panel = chunk_panel;
    a.panel_ld = w.panel_ld;
    a.out_rows = kept_per_chunk ? out_rows : nullptr;
    hipLaunchKernelGGL(k_label_logit, dim3((unsigned)((n_tok + 3) / 4)), dim3(256), 0, st, hid, (const uint16_t*)weight,
                       labels + t0, (int)n_tok, (int)H, (int)V, a.xy, (int32_t*)nullptr);
    if (rows > 0)
      launch_tiles<kModeStatsCarry>(st, weight, hid, n_tok, H, V, a);
    else
      launch_tiles<kModeStats>(st, weight, hid, n_tok, H, V, a);
    hipLaunchKernelGGL(k_combine, dim3((unsigned)((n_tok + 63) / 64)), dim3(1024), 0, st, a.pk, a.ps, a.pu, a.pn, a.xy,
                       (int)w.blocks, a.pitch_t, (int)n_tok, a.c, logp + t0, at(entropy, t0), row_lse + t0, at(row_ez, t0),
                       at(vocab_max, t0), at(vocab_min, t0));
    row0 += rows;
  }
  return launch_status();
}

extern "C" int aa_lmhead_bwd_carry(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                                   const int64_t* labels, float inv_temperature, const float* logp, const float* row_lse,
                                   const float* g_logp, const uint8_t* row_has_gradient, const int64_t* kept_per_chunk,
                                   void* panel, int64_t panel_rows, void* d_hidden, void* d_weight, int d_weight_dtype,
                                   void* workspace, int64_t workspace_bytes, void* stream) {
  if (!hidden || !weight || !labels || !logp || !row_lse || !g_logp || !panel || !d_hidden || !d_weight || !workspace)
    return AA_ERR_INVALID_ARGUMENT;
  if (!(inv_temperature > 0.f) || (kept_per_chunk != nullptr) != (row_has_gradient != nullptr)) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V) || (d_weight_dtype != AA_F32 && d_weight_dtype != AA_BF16)) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace | (uintptr_t)d_hidden | (uintptr_t)d_weight |
        (uintptr_t)panel) & 15))
    return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V, true);
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  const int64_t n_chunks = (T + w.chunk - 1) / w.chunk;
  if (panel_rows < panel_rows_before(kept_per_chunk, w.chunk, T, n_chunks)) return AA_ERR_INVALID_ARGUMENT;
  if (!prepare_kernels()) return AA_ERR_LAUNCH;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  const WeightGrad dw = weight_grad(w, ws, d_weight, d_weight_dtype, T);
  int32_t* out_rows = (int32_t*)(ws + w.off_rows);
  int32_t* act_rows = out_rows + w.chunk;
  float* row_factor = (float*)(ws + w.off_rowf);
  int32_t* redo_flag = (int32_t*)(ws + w.off_flag);
  bool first = true;  // no GEMM has written d_weight yet
  int64_t chunk_index = 0, row0 = 0;
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk, ++chunk_index) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    uint16_t* dh = (uint16_t*)d_hidden + t0 * H;
    uint16_t* chunk_panel = (uint16_t*)panel + row0 * w.panel_ld;
    int64_t rows = n_tok;
    const int32_t* row_of_token = nullptr;
    const int32_t* token_of_row = nullptr;
    const int32_t* rows_in_use = nullptr;  // the count of the chunk, when only the device has it
    if (kept_per_chunk) {
      rows = kept_per_chunk[chunk_index];
      const bool on_device = rows == AA_LMHEAD_COUNT_ON_DEVICE;
      rows = on_device ? n_tok : (rows < 0 ? 0 : (rows > n_tok ? n_tok : rows));
      if (rows == 0) {
        launch_zero(st, dh, n_tok * H * 2);
        continue;
      }
      // the same numbering as in the forward (the mask has not changed); surplus rows get a factor of zero
      int32_t* total_word = (int32_t*)(ws + w.off_total);
      launch_compact_map(st, row_has_gradient + t0, n_tok, n_tok, rows, out_rows, act_rows, row_factor, total_word,
                         chunk_panel, w.panel_ld, H, V, on_device);
      if (on_device) rows_in_use = total_word;
      row_of_token = out_rows;
      token_of_row = act_rows;
    }
    launch_zero(st, redo_flag, 256);
    hipLaunchKernelGGL(k_carry_factors, dim3((unsigned)((n_tok + 255) / 256)), dim3(256), 0, st, logp + t0, g_logp + t0,
                       labels + t0, row_of_token, (int)n_tok, (int)V, inv_temperature,
                       CarryOut{row_factor, chunk_panel, w.panel_ld, redo_flag});
    // a chunk whose rows do not fit the stored form is redone from the logits tiles, decided on the device
    TileArgs a{};
    a.labels = labels + t0;
    a.c = kLog2e * inv_temperature;
    a.inv_t = inv_temperature;
    a.row_lse = row_lse + t0;
    a.g_logp = g_logp + t0;
    a.panel_ld = w.panel_ld;
    recompute_panel(st, w, ws, chunk_panel, weight, hid, n_tok, token_of_row, rows, H, V, a, redo_flag, rows_in_use);
    hipLaunchKernelGGL(k_unit_factors, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, st, row_factor, (int)rows, redo_flag);
    if (token_of_row) launch_zero(st, dh, n_tok * H * 2);  // the rows of the tokens without a panel row
    panel_gradients(st, w, ws, chunk_panel, weight, hid, token_of_row, row_factor, rows, H, V, dh, dw.acc, dw.acc_f32, first,
                    rows_in_use);
    first = false;
    row0 += rows;
  }
  if (first) launch_zero(st, dw.acc, V * H * (dw.acc_f32 ? 4 : 2));  // no row of the batch has a gradient
  finish_weight_grad(st, dw, d_weight, V, H);
  return launch_status();
}

extern "C" int aa_lmhead_ppo_fused(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                                   const int64_t* labels, float inv_temperature, int64_t T_active,
                                   const float* prox_logp, const float* adv, const uint8_t* mask_eff,
                                   const float* behave_w, const aa_ppo_params* params, const int32_t* n_valid,
                                   const float* grad_scale, const int64_t* kept_per_chunk, int backward_mode,
                                   float* logp, float* entropy, float* stat_loss, float* ratio, uint8_t* flags,
                                   float* vocab_max, float* vocab_min, void* d_hidden, void* d_weight,
                                   int d_weight_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  if (!hidden || !weight || !labels || !d_hidden || !d_weight || !workspace) return AA_ERR_INVALID_ARGUMENT;
  if ((vocab_max != nullptr) != (vocab_min != nullptr)) return AA_ERR_INVALID_ARGUMENT;
  if (!params || !n_valid || !logp) return AA_ERR_INVALID_ARGUMENT;
  if (T_active < 0 || T_active > T || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  if (backward_mode != AA_LMHEAD_RECOMPUTE && backward_mode != AA_LMHEAD_CARRY) return AA_ERR_INVALID_ARGUMENT;
  if (params->loss_kind != AA_LOSS_PPO && params->loss_kind != AA_LOSS_NLL && params->loss_kind != AA_LOSS_SAPO)
    return AA_ERR_INVALID_ARGUMENT;
  if (params->loss_kind == AA_LOSS_SAPO &&
      (params->has_behave_weight || !(params->sapo_tau_pos > 0.f) || !(params->sapo_tau_neg > 0.f)))
    return AA_ERR_INVALID_ARGUMENT;
  const bool nll = params->loss_kind == AA_LOSS_NLL;  // prox_logp and adv are not used by that loss
  if (T_active > 0 && (!mask_eff || !stat_loss || !ratio || !flags)) return AA_ERR_INVALID_ARGUMENT;
  if (T_active > 0 && !nll && (!prox_logp || !adv)) return AA_ERR_INVALID_ARGUMENT;
  if (T_active > 0 && params->has_behave_weight && !behave_w) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V) || (d_weight_dtype != AA_F32 && d_weight_dtype != AA_BF16)) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace | (uintptr_t)d_hidden | (uintptr_t)d_weight) & 15))
    return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V);
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  if (!prepare_kernels()) return AA_ERR_LAUNCH;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  const bool carry = backward_mode == AA_LMHEAD_CARRY;
  const WeightGrad dw = weight_grad(w, ws, d_weight, d_weight_dtype, T);
  int32_t* out_rows = (int32_t*)(ws + w.off_rows);
  int32_t* act_rows = out_rows + w.chunk;
  float* g_tok = (float*)(ws + w.off_g);
  float* lse_tok = (float*)(ws + w.off_lse);
  float* row_factor = (float*)(ws + w.off_rowf);
  int32_t* redo_flag = (int32_t*)(ws + w.off_flag);
  uint16_t* panel = (uint16_t*)(ws + w.off_panel);
  bool first = true;  // no GEMM has written d_weight yet
  int64_t chunk_index = 0;
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk, ++chunk_index) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    int64_t act = T_active - t0;
    act = act < 0 ? 0 : (act > n_tok ? n_tok : act);
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    uint16_t* dh = (uint16_t*)d_hidden + t0 * H;
    auto at = [t0](auto* p) { return p ? p + t0 : nullptr; };
    // which tokens get a panel row: those with a mask when the host gave their count, every token otherwise
    int64_t rows = n_tok;
    const int32_t* row_of_token = nullptr;
    const int32_t* token_of_row = nullptr;
    const int32_t* rows_in_use = nullptr;
    if (kept_per_chunk) {
      rows = kept_per_chunk[chunk_index];
      // the count may be left to the device: every active token could have a row, the kernels stop at those in use
      const bool on_device = rows == AA_LMHEAD_COUNT_ON_DEVICE;
      rows = on_device ? act : (rows < 0 ? 0 : (rows > act ? act : rows));
      int32_t* total_word = (int32_t*)(ws + w.off_total);
      launch_compact_map(st, at(mask_eff), act, n_tok, rows, out_rows, act_rows, carry ? row_factor : nullptr, total_word,
                         panel, w.panel_ld, H, V, on_device);
      if (on_device) rows_in_use = total_word;
      row_of_token = out_rows;
      token_of_row = act_rows;
    }
    // forward tiles: block partials (and, in carry mode, the unnormalised probabilities of the panel rows)
    TileArgs a = stats_args(w, ws, labels + t0, inv_temperature, vocab_min != nullptr);
    a.panel = panel;
    a.panel_ld = w.panel_ld;
    a.out_rows = row_of_token;
    hipLaunchKernelGGL(k_label_logit, dim3((unsigned)((n_tok + 3) / 4)), dim3(256), 0, st, hid, (const uint16_t*)weight,
                       labels + t0, (int)n_tok, (int)H, (int)V, a.xy, redo_flag);
    if (carry && rows > 0)
      launch_tiles<kModeStatsCarry>(st, weight, hid, n_tok, H, V, a);
    else
      launch_tiles<kModeStats>(st, weight, hid, n_tok, H, V, a);
    // row statistics, per-token outputs, g
    TokenLossArgs la{at(prox_logp), at(adv), at(mask_eff), at(behave_w), n_valid, grad_scale, logp + t0, at(entropy),
                     at(stat_loss), at(ratio), at(flags), at(vocab_max), at(vocab_min), *params, act};
    hipLaunchKernelGGL(k_token_loss, dim3((unsigned)((n_tok + 63) / 64)), dim3(1024), 0, st, a.pk, a.ps, a.pu, a.pn, a.xy,
                       (int)w.blocks, a.pitch_t, (int)n_tok, (int)V, a.c, inv_temperature, labels + t0, la, row_of_token,
                       g_tok, lse_tok,
                       (carry && rows > 0) ? CarryOut{row_factor, panel, w.panel_ld, redo_flag}
                                           : CarryOut{nullptr, nullptr, 0, nullptr});
    if (rows == 0) {
      launch_zero(st, dh, n_tok * H * 2);
      continue;
    }
    // d(logits) rows by recompute: always in that mode; in carry mode only if the chunk was flagged (decided on the
    // device: the kernels start and return at once otherwise), and then the row factors become 1
    a.row_lse = lse_tok;
    a.g_logp = g_tok;
    recompute_panel(st, w, ws, panel, weight, hid, n_tok, token_of_row, rows, H, V, a, carry ? redo_flag : nullptr,
                    rows_in_use);
    if (carry)
      hipLaunchKernelGGL(k_unit_factors, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, st, row_factor, (int)rows, redo_flag);
    if (token_of_row) launch_zero(st, dh, n_tok * H * 2);  // the rows of the tokens without gradient
    panel_gradients(st, w, ws, panel, weight, hid, token_of_row, carry ? row_factor : nullptr, rows, H, V, dh, dw.acc,
                    dw.acc_f32, first, rows_in_use);
    first = false;
  }
  if (first) launch_zero(st, dw.acc, V * H * (dw.acc_f32 ? 4 : 2));  // no token of the batch has a gradient
  finish_weight_grad(st, dw, d_weight, V, H);
  return launch_status();
}
