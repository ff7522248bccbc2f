// lm_head path for gfx950: log-prob / entropy of softmax(hidden @ weight.T / T), their backward, and the whole
// lm_head + PPO-loss training step, without ever holding the [T, V] logits in memory.  The reference has no such
// path: its equivalent is the lm_head matmul followed by gather_logprobs_entropy
// (areal/utils/functional/vocab_parallel.py:23-29), ppo_actor_loss_fn and autograd.
//
// Stand-alone op, forward: a bf16 MFMA tile GEMM (gemm_tn.h) forms 256 (vocabulary) x 256 (tokens) tiles of the
// logits in accumulator registers; its epilogue reduces each tile to the softmax partials (k, s, u) per token and
// captures the label logit; a second small kernel merges the partials of all vocabulary tiles.
//
// Stand-alone op, backward: the logits tile is formed again, turned into d(logits) in registers (bf16) and written
// to a reusable panel [token chunk, V]; the two plain GEMMs that contract the panel with the weights (d_hidden)
// and with the hidden states (d_weight, fp32) go to hipBLASLt (lt_gemm.h), both in the form the library runs
// fastest (contraction index contiguous in both operands), fed by transposed copies made with k_transpose_bf16.
//
// Training step (aa_lmhead_ppo_fused): per token chunk, a library GEMM writes the bf16 logits panel, the fused
// row kernel of the logits path turns it in place into d(loss)/d(logits), and the same two library GEMMs follow.
#include "gemm_tn.h"
#include "lt_gemm.h"

namespace aa {
namespace lmhead {

using namespace gemm;

constexpr int kChunkTokens = 16384;  // token chunk of the backward panel
constexpr int kPanelPitch = BM + 8;   // pitch (elements) of the d(logits) tile staged in LDS as [token][vocab]
constexpr int kLdsBytesDs = 256 * kPanelPitch * 2 > kLdsBytes ? 256 * kPanelPitch * 2 : kLdsBytes;  // 135168 B

__host__ __device__ __forceinline__ int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// ---- forward epilogue: softmax partials of a tile --------------------------------------------------------------
// part[(tile_v * T + token)] = (k, s, u, 0);   xy[token] = raw label logit (written by the one tile that holds it)
__global__ __launch_bounds__(kThreads) void k_lmhead_stats(Operand W, Operand Hd, int K, int tiles_m, int tiles_n,
                                                           float c, const int64_t* __restrict__ labels,
                                                           float4* __restrict__ part, float* __restrict__ xy) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  int tm, tn;
  tile_of(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  Acc acc;
  mainloop(W, Hd, K, m0, n0, acc, lds);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int V = W.rows, T = Hd.rows;
  const int mbase = m0 + wm * 128;
  const bool ragged = m0 + BM > V;
  float* red = (float*)lds;  // [2 (wm)][256 tokens][3]

#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    const int token = n0 + wn * 128 + acc_col(nt, lane);
    float mx = -FLT_MAX;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const bool in = !ragged || (mbase + acc_row(mt, i, lane) < V);  // rows past the vocabulary: last tile only
        mx = in ? fmaxf(mx, acc.v[mt][nt][i]) : mx;
      }
    // both halves of the wave (lane, lane ^ 32) hold the same token: agree on the maximum first
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float k = fmaxf(mx * c, kNegBig);  // kNegBig: no valid row in this wave's block
    float s = 0.f, u = 0.f;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const bool in = !ragged || (mbase + acc_row(mt, i, lane) < V);
        const float t = in ? fmaf(acc.v[mt][nt][i], c, -k) : 0.f;
        const float e = in ? fast_exp2(t) : 0.f;
        s += e;
        u = fmaf(t, e, u);
      }
    s += __shfl_xor(s, 32, kWave);
    u += __shfl_xor(u, 32, kWave);
    if (lane < 32) {
      float* r = red + (wm * 256 + wn * 128 + nt * 32 + lane) * 3;
      r[0] = k; r[1] = s; r[2] = u;
    }
    // label logit, if the label falls into this wave's 128 vocabulary rows
    if (token < T) {
      const int64_t y = labels[token];
      const int64_t rel = y - mbase;
      if (rel >= 0 && rel < 128 && y < V && (int)((rel >> 2) & 1) == (lane >> 5)) {
        const int mt_y = (int)(rel >> 5), r5 = (int)(rel & 31);
        const int i_y = ((r5 >> 3) << 2) | (r5 & 3);
        float val = 0.f;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (mt == mt_y && i == i_y) val = acc.v[mt][nt][i];
        xy[token] = val;
      }
    }
  }
  __syncthreads();
  {  // merge the two vocabulary halves of the tile; thread = token
    const int token = n0 + tid;
    const float* a = red + tid * 3;
    const float* b = red + (256 + tid) * 3;
    const float k = fmaxf(a[0], b[0]);
    const float da = a[0] - k, db = b[0] - k;
    const float fa = fast_exp2(da), fb = fast_exp2(db);
    const float s = a[1] * fa + b[1] * fb;
    const float u = fa * fmaf(da, a[1], a[2]) + fb * fmaf(db, b[1], b[2]);
    if (token < T) part[(int64_t)tm * T + token] = make_float4(k, s, u, 0.f);
  }
}

__global__ __launch_bounds__(256) void k_fill_f32(float* p, int64_t n, float v) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = v;
}

// merge the partials of all vocabulary tiles, one thread per token (fixed order: deterministic)
__global__ __launch_bounds__(256) void k_lmhead_combine(const float4* __restrict__ part, const float* __restrict__ xy,
                                                        int tiles_m, int T, float c, float* __restrict__ logp,
                                                        float* __restrict__ entropy, float* __restrict__ row_lse,
                                                        float* __restrict__ row_ez) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= T) return;
  float k = kNegBig, s = 0.f, u = 0.f;
  for (int vt = 0; vt < tiles_m; ++vt) {
    const float4 p = part[(int64_t)vt * T + t];
    const float nk = fmaxf(k, p.x);
    const float da = k - nk, db = p.x - nk;
    const float fa = fast_exp2(da), fb = fast_exp2(db);
    u = fa * fmaf(da, s, u) + fb * fmaf(db, p.y, p.z);
    s = s * fa + p.y * fb;
    k = nk;
  }
  const float log2s = fast_log2(s);
  const float mean_t = u / s;
  logp[t] = (fmaf(xy[t], c, -k) - log2s) * kLn2;  // xy stays NaN for a label outside [0, V)
  if (entropy) entropy[t] = (log2s - mean_t) * kLn2;
  if (row_lse) row_lse[t] = (k + log2s) * kLn2;
  if (row_ez) row_ez[t] = (k + mean_t) * kLn2;
}

// ---- backward epilogue: d(logits) of a tile, written into the panel [tokens, V] -------------------------------------
struct DsArgs {
  const float* row_lse;   // [T] natural log
  const float* row_ez;    // [T] (nullable when g_entropy is null)
  const float* g_logp;    // [T]
  const float* g_entropy; // [T] nullable
  const int64_t* labels;  // [T]
  uint16_t* ds;           // [chunk tokens, V] bf16, ld = V
  int64_t t0;             // first token of the chunk (hidden operand is already offset)
  float inv_t;
};

__global__ __launch_bounds__(kThreads) void k_lmhead_ds(Operand W, Operand Hd, int K, int tiles_m, int tiles_n,
                                                        DsArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  int tm, tn;
  tile_of(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  Acc acc;
  mainloop(W, Hd, K, m0, n0, acc, lds);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int V = W.rows, N = Hd.rows;
  const int mbase = m0 + wm * 128;
  const float c = kLog2e * a.inv_t;
  constexpr int PZ = kPanelPitch;
  uint16_t* Z = lds;  // 256 x 264 bf16 = 135168 B, over the operand stages (the main loop is done with them)

#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    const int nloc = wn * 128 + acc_col(nt, lane);
    const int n = n0 + nloc;
    float A = 0.f, B = 0.f, lab_add = 0.f, lse2 = 0.f;
    int64_t y = -1;
    const bool live = n < N;
    if (live) {
      const int64_t t = a.t0 + n;
      const float gl = a.g_logp[t];
      const float gh = a.g_entropy ? a.g_entropy[t] : 0.f;
      const float ez = a.g_entropy ? a.row_ez[t] : 0.f;
      lse2 = a.row_lse[t] * kLog2e;
      A = a.inv_t * (gh * ez - gl);
      B = -gh * a.inv_t * a.inv_t;
      lab_add = gl * a.inv_t;
      y = a.labels[t];
    }
    const int64_t rel = y - mbase;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        float o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float x = acc.v[mt][nt][g4 * 4 + q];
          o[q] = live ? fast_exp2(fmaf(x, c, -lse2)) * fmaf(B, x, A) : 0.f;
        }
        const int r0 = mt * 32 + 8 * g4 + 4 * (lane >> 5);  // row of o[0] inside the wave block
        if (rel >= r0 && rel < r0 + 4) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (rel - r0 == q) o[q] += lab_add;
        }
        if (mbase + r0 + 3 >= V) {  // rows outside the vocabulary (last tile only)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (mbase + r0 + q >= V) o[q] = 0.f;
        }
        uint2 pk;
        pk.x = Elem<AA_BF16>::pack(o[0], o[1]);
        pk.y = Elem<AA_BF16>::pack(o[2], o[3]);
        *(uint2*)(Z + nloc * PZ + wm * 128 + r0) = pk;
      }
    }
  }
  __syncthreads();
  // panel [token][vocab]: 16-byte pieces along the vocabulary
  for (int p = tid; p < 256 * 32; p += kThreads) {
    const int nloc = p >> 5, mc = (p & 31) * 8;
    const int n = n0 + nloc, m = m0 + mc;
    if (n < N && m < V) {
      const u32x4_t v = *(const u32x4_t*)(Z + nloc * PZ + mc);
      *(u32x4_t*)(a.ds + (int64_t)n * V + m) = v;  // V % 8 == 0: a piece never straddles the end
    }
  }
}

// ---- bf16 transpose: dst[c, r] = src[r, c] ----------------------------------------------------------------------
// src is [R, C] with row pitch lds (elements), dst is [C, ldd] with ldd = R rounded up to 8; columns R .. ldd - 1 of dst
// are written as zeros.  One workgroup moves a 64 x 64 tile through LDS: each thread loads 8 elements of two
// adjacent rows (16 B each), pairs them into 32-bit words (two consecutive dst columns) and stores the words
// transposed; the second half reads 16 B per thread and writes 128 B contiguous per dst row.  The word index is
// XOR-ed with a key of the row so that both halves run without bank conflicts.  Requires C % 8 == 0, lds % 8 == 0.
// Tiles are numbered along r first, in bands of kTransposeBand tile rows, so that the workgroups in flight together
// write long contiguous pieces of the dst rows (measured: 5.2 TB/s against 3.9 with c first).
constexpr int kTransposeBand = 64;

__global__ __launch_bounds__(256) void k_transpose_bf16(const uint16_t* __restrict__ src, int R, int C, int64_t lds,
                                                        uint16_t* __restrict__ dst, int64_t ldd, int tiles_c,
                                                        int tiles_r) {
  __shared__ uint32_t tile[64 * 32];
  const int t = threadIdx.x;
  const int per_band = kTransposeBand * tiles_c;
  const int band = blockIdx.x / per_band, rem = blockIdx.x % per_band;
  const int rows_in_band = min(kTransposeBand, tiles_r - band * kTransposeBand);
  const int c0 = (rem / rows_in_band) * 64, r0 = (band * kTransposeBand + rem % rows_in_band) * 64;
  {
    const int rp = t >> 3, c8 = (t & 7) * 8;
    const int r = r0 + 2 * rp, c = c0 + c8;
    u32x4_t a = {0u, 0u, 0u, 0u}, b = {0u, 0u, 0u, 0u};
    if (c < C) {
      if (r < R) a = __builtin_nontemporal_load((const u32x4_t*)(src + (int64_t)r * lds + c));
      if (r + 1 < R) b = __builtin_nontemporal_load((const u32x4_t*)(src + (int64_t)(r + 1) * lds + c));
    }
    const int key = ((t & 7) & 3) << 3;  // = (((c8 + j) >> 3) & 3) << 3 for every j < 8
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t wa = a[j >> 1], wb = b[j >> 1];
      const uint32_t lo = (j & 1) ? (wa >> 16) : (wa & 0xffffu);
      const uint32_t hi = (j & 1) ? (wb & 0xffff0000u) : (wb << 16);
      tile[(c8 + j) * 32 + (rp ^ key)] = lo | hi;
    }
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int cl = (t >> 3) + 32 * p, g = t & 7;
    const int key = ((cl >> 3) & 3) << 3;
    const u32x4_t v = *(const u32x4_t*)(tile + cl * 32 + ((4 * g) ^ key));
    const int c = c0 + cl;
    const int64_t r = r0 + 8 * g;
    if (c < C && r < ldd) *(u32x4_t*)(dst + (int64_t)c * ldd + r) = v;
  }
}

static void launch_transpose(hipStream_t st, const uint16_t* src, int64_t R, int64_t C, int64_t lds, uint16_t* dst) {
  const int64_t ldd = round_up(R, 8);
  const int64_t tiles_c = (C + 63) / 64, tiles_r = (R + 63) / 64;
  hipLaunchKernelGGL(k_transpose_bf16, dim3((unsigned)(tiles_c * tiles_r)), dim3(256), 0, st, src, (int)R, (int)C, lds, dst,
                     ldd, (int)tiles_c, (int)tiles_r);
}

struct Workspace {
  int64_t off_part, off_xy;  // forward: per-tile partials, label logits
  int64_t off_ds, off_lt;    // backward / step: the [chunk, V] panel, scratch of the GEMM library
  int64_t off_dst, off_wt, off_ht;  // transposed copies: panel [V, chunk], weight [H, V], hidden chunk [H, chunk]
  int64_t chunk;
  int64_t bytes;
};

static Workspace plan(int64_t T, int64_t H, int64_t V) {
  Workspace w{};
  auto up = [](int64_t x) { return (x + 255) / 256 * 256; };
  const int64_t tiles_v = (V + BM - 1) / BM;
  int64_t off = 0;
  w.off_part = off; off += up(tiles_v * T * (int64_t)sizeof(float4));
  w.off_xy = off;   off += up(T * (int64_t)sizeof(float));
  const int64_t fwd_bytes = off;
  off = 0;
  w.chunk = T < kChunkTokens ? (T + 255) / 256 * 256 : kChunkTokens;
  w.off_ds = off;  off += up(w.chunk * V * 2);
  w.off_lt = off;  off += lt::kWorkspaceBytes;
  w.off_dst = off; off += up(w.chunk * V * 2);
  w.off_wt = off;  off += up(H * V * 2);
  w.off_ht = off;  off += up(w.chunk * H * 2);
  w.bytes = off > fwd_bytes ? off : fwd_bytes;
  return w;
}

// The two GEMMs that contract the d(logits) panel ds [n_tok, V] of one token chunk:
//   d_hidden[chunk] = ds . W          (bf16)          d_weight (+)= ds^T . hidden[chunk]   (fp32)
// Both run in the library's fastest form, with the contraction index contiguous in both operands ("TN"), which
// takes transposed copies of the panel and of the hidden chunk (made here) and of the weight (made once per call,
// by the caller, at ws + off_wt).  The copies pad the token count to a multiple of 8 with zeros.
static bool panel_gradients(hipStream_t st, const Workspace& w, char* ws, const uint16_t* hid, int64_t n_tok, int64_t H,
                            int64_t V, uint16_t* d_hidden_chunk, float* d_weight, bool first) {
  const uint16_t* ds = (const uint16_t*)(ws + w.off_ds);
  uint16_t* ds_t = (uint16_t*)(ws + w.off_dst);
  const uint16_t* w_t = (const uint16_t*)(ws + w.off_wt);
  uint16_t* hid_t = (uint16_t*)(ws + w.off_ht);
  void* lt_ws = ws + w.off_lt;
  const int64_t kp = round_up(n_tok, 8);
  // column-major [H, n_tok] = (W^T)'^T [H, V] . ds' [V, n_tok]
  if (!lt::gemm(st, true, false, H, n_tok, V, w_t, V, ds, V, d_hidden_chunk, H, false, 0.f, lt_ws, lt::kWorkspaceBytes))
    return false;
  launch_transpose(st, ds, n_tok, V, V, ds_t);
  launch_transpose(st, hid, n_tok, H, H, hid_t);
  // column-major [H, V] = (hidden^T)'^T [H, kp] . (ds^T)' [kp, V], fp32, accumulated over the chunks
  return lt::gemm(st, true, false, H, V, kp, hid_t, kp, ds_t, kp, d_weight, H, true, first ? 0.f : 1.f, lt_ws,
                  lt::kWorkspaceBytes);
}

static bool shapes_ok(int64_t T, int64_t H, int64_t V) {
  return T > 0 && H > 0 && V > 0 && (H % BK) == 0 && (V % BK) == 0 && T < (1 << 30) && V < (1 << 30) && H < (1 << 30) &&
         (V / 64 + 1) * ((H > kChunkTokens ? H : kChunkTokens) / 64 + 1) < (1LL << 31);  // transpose grids
}

template <typename Kern>
static bool allow_big_lds(Kern k, int bytes = kLdsBytes) {
  return hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess;
}

}  // namespace lmhead
}  // namespace aa

using namespace aa;
using namespace aa::lmhead;

extern "C" int64_t aa_lmhead_workspace_bytes(int64_t T, int64_t H, int64_t V) {
  if (!shapes_ok(T, H, V)) return -1;
  return plan(T, H, V).bytes;
}

extern "C" int aa_lmhead_fwd(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                             const int64_t* labels, float inv_temperature, float* logp, float* entropy,
                             float* row_lse, float* row_ez, void* workspace, int64_t workspace_bytes, void* stream) {
  if (!hidden || !weight || !labels || !logp || !workspace || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V)) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace) & 15) != 0) return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V);
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  static const bool ok = allow_big_lds(k_lmhead_stats);
  if (!ok) return AA_ERR_LAUNCH;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  float4* part = (float4*)(ws + w.off_part);
  float* xy = (float*)(ws + w.off_xy);
  const int tiles_m = (int)((V + BM - 1) / BM), tiles_n = (int)((T + BN - 1) / BN);
  hipLaunchKernelGGL(k_fill_f32, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, st, xy, T, __builtin_nanf(""));
  Operand W{(const uint16_t*)weight, H, (int)V};
  Operand Hd{(const uint16_t*)hidden, H, (int)T};
  const float c = kLog2e * inv_temperature;
  hipLaunchKernelGGL(k_lmhead_stats, dim3((unsigned)(tiles_m * tiles_n)), dim3(kThreads), kLdsBytes, st, W, Hd, (int)H,
                     tiles_m, tiles_n, c, labels, part, xy);
  hipLaunchKernelGGL(k_lmhead_combine, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, st, part, xy, tiles_m, (int)T,
                     c, logp, entropy, row_lse, row_ez);
  return launch_status();
}

extern "C" int aa_lmhead_bwd(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                             const int64_t* labels, float inv_temperature, const float* row_lse, const float* row_ez,
                             const float* g_logp, const float* g_entropy, void* d_hidden, float* d_weight,
                             void* workspace, int64_t workspace_bytes, void* stream) {
  if (!hidden || !weight || !labels || !row_lse || !g_logp || !d_hidden || !d_weight || !workspace)
    return AA_ERR_INVALID_ARGUMENT;
  if ((g_entropy && !row_ez) || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V) || (V % 8) != 0) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace | (uintptr_t)d_hidden | (uintptr_t)d_weight) & 15))
    return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V);
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  static const bool ok = allow_big_lds(k_lmhead_ds, kLdsBytesDs);
  if (!ok) return AA_ERR_LAUNCH;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  uint16_t* ds = (uint16_t*)(ws + w.off_ds);  // [chunk, V]
  launch_transpose(st, (const uint16_t*)weight, V, H, H, (uint16_t*)(ws + w.off_wt));
  const int tiles_v = (int)((V + BM - 1) / BM);
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    const int tiles_t = (int)((n_tok + BN - 1) / BN);
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    Operand W{(const uint16_t*)weight, H, (int)V};
    Operand Hd{hid, H, (int)n_tok};
    DsArgs a{row_lse, row_ez, g_logp, g_entropy, labels, ds, t0, inv_temperature};
    hipLaunchKernelGGL(k_lmhead_ds, dim3((unsigned)(tiles_v * tiles_t)), dim3(kThreads), kLdsBytesDs, st, W, Hd, (int)H,
                       tiles_v, tiles_t, a);
    if (!panel_gradients(st, w, ws, hid, n_tok, H, V, (uint16_t*)d_hidden + t0 * H, d_weight, t0 == 0))
      return AA_ERR_LAUNCH;
  }
  return launch_status();
}

extern "C" int aa_lmhead_ppo_fused(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                                   const int64_t* labels, float inv_temperature, int64_t T_active,
                                   const float* prox_logp, const float* adv, const uint8_t* mask_eff,
                                   const float* behave_w, const aa_ppo_params* params, const int32_t* n_valid,
                                   const float* grad_scale, float* logp, float* entropy, float* stat_loss, float* ratio,
                                   uint8_t* flags, void* d_hidden, float* d_weight, int32_t* work, void* workspace,
                                   int64_t workspace_bytes, void* stream) {
  if (!hidden || !weight || !labels || !d_hidden || !d_weight || !workspace) return AA_ERR_INVALID_ARGUMENT;
  if (!params || !n_valid || !logp) return AA_ERR_INVALID_ARGUMENT;
  if (T_active < 0 || T_active > T || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  if (T_active > 0 && (!prox_logp || !adv || !mask_eff || !stat_loss || !ratio || !flags)) return AA_ERR_INVALID_ARGUMENT;
  if (T_active > 0 && params->has_behave_weight && !behave_w) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V) || (V % 8) != 0) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace | (uintptr_t)d_hidden | (uintptr_t)d_weight) & 15))
    return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V);
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  uint16_t* ds = (uint16_t*)(ws + w.off_ds);  // [chunk, V]: logits of the chunk, then their gradient in place
  void* lt_ws = ws + w.off_lt;
  launch_transpose(st, (const uint16_t*)weight, V, H, H, (uint16_t*)(ws + w.off_wt));
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    int64_t act = T_active - t0;
    act = act < 0 ? 0 : (act > n_tok ? n_tok : act);
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    // logits[t0 : t0 + n_tok, :] = hidden . W^T, rounded to bf16 as the reference's lm_head output is.
    // Row-major [n_tok, V] is column-major [V, n_tok]: W'^T [V, H] . hidden' [H, n_tok].
    if (!lt::gemm(st, true, false, V, n_tok, H, weight, H, hid, H, ds, V, false, 0.f, lt_ws, lt::kWorkspaceBytes))
      return AA_ERR_LAUNCH;
    // log-prob, entropy, PPO loss and d(loss)/d(logits) in place: one streaming pass over the panel
    auto at = [t0](auto* p) { return p ? p + t0 : nullptr; };
    const int rc = aa_logits_ppo_fused(ds, AA_BF16, n_tok, V, V, labels + t0, inv_temperature, act, at(prox_logp), at(adv),
                                       at(mask_eff), at(behave_w), params, n_valid, grad_scale, logp + t0, at(entropy),
                                       nullptr, nullptr, at(stat_loss), at(ratio), at(flags), ds, work, stream);
    if (rc != AA_OK) return rc;
    if (!panel_gradients(st, w, ws, hid, n_tok, H, V, (uint16_t*)d_hidden + t0 * H, d_weight, t0 == 0))
      return AA_ERR_LAUNCH;
  }
  return launch_status();
}
