// lm_head path for gfx950: log-prob / entropy of softmax(hidden @ weight.T / T), their backward, and the whole
// lm_head + PPO-loss training step, holding at most one token chunk of logits in memory.  The reference has no such
// path: its equivalent is the lm_head matmul followed by gather_logprobs_entropy
// (areal/utils/functional/vocab_parallel.py:23-29), ppo_actor_loss_fn and autograd.
//
// Tokens go through in chunks of at most kChunkTokens.  Per chunk the plain GEMMs go to hipBLASLt (lt_gemm.h), always
// in the form the library runs fastest on this chip (contraction index contiguous in both operands), and everything
// else is one of this library's streaming kernels over the chunk's bf16 logits panel:
//   forward        panel = hidden_c . W^T (bf16, as the reference's lm_head output is)  ->  k_logits_fwd
//   backward       panel again  ->  k_logits_bwd in place  ->  d_hidden_c, d_weight
//   training step  panel  ->  the fused log-prob / entropy / PPO-loss / gradient kernel in place  ->  d_hidden_c, d_weight
// The gradient GEMMs take transposed copies of the panel, of the hidden chunk and of the weight (k_transpose_bf16).
#include "device_utils.h"
#include "lt_gemm.h"

namespace aa {
namespace lmhead {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kChunkTokens = 16384;  // token chunk of the logits panel

__host__ __device__ __forceinline__ int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

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

// fp32 -> bf16 (round to nearest even), 8 elements per thread; n % 8 == 0
typedef float f32x4_t __attribute__((ext_vector_type(4)));

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

struct Workspace {
  int64_t off_ds, off_lt;           // the [chunk, V] panel, scratch of the GEMM library
  int64_t off_dst, off_wt, off_ht;  // transposed copies: panel [V, chunk], weight [H, V], hidden chunk [H, chunk]
  int64_t off_dw;                   // fp32 accumulator of a bf16 d_weight when there is more than one chunk
  int64_t chunk;
  int64_t bytes;
};

static Workspace plan(int64_t T, int64_t H, int64_t V) {
  Workspace w{};
  auto up = [](int64_t x) { return (x + 255) / 256 * 256; };
  int64_t off = 0;
  w.chunk = T < kChunkTokens ? round_up(T, 256) : kChunkTokens;
  w.off_ds = off;  off += up(w.chunk * V * 2);
  w.off_lt = off;  off += lt::kWorkspaceBytes;
  w.off_dst = off; off += up(w.chunk * V * 2);
  w.off_wt = off;  off += up(H * V * 2);
  w.off_ht = off;  off += up(w.chunk * H * 2);
  w.off_dw = off;  off += T > w.chunk ? up(V * H * 4) : 0;
  w.bytes = off;
  return w;
}

// logits[t0 : t0 + n_tok, :] = hidden . W^T, rounded to bf16.  Row-major [n_tok, V] is column-major [V, n_tok]:
// W'^T [V, H] . hidden' [H, n_tok].
static bool panel_logits(hipStream_t st, const Workspace& w, char* ws, const uint16_t* hid, const void* weight,
                         int64_t n_tok, int64_t H, int64_t V) {
  return lt::gemm(st, true, false, V, n_tok, H, weight, H, hid, H, ws + w.off_ds, V, false, 0.f, ws + w.off_lt,
                  lt::kWorkspaceBytes);
}

// The two GEMMs that contract the d(logits) panel ds [n_tok, V] of one token chunk:
//   d_hidden[chunk] = ds . W          (bf16)          d_weight (+)= ds^T . hidden[chunk]   (fp32, or bf16 when first)
// with transposed copies of the panel and of the hidden chunk (made here) and of the weight (made once per call, by
// the caller, at ws + off_wt).  The copies pad the token count to a multiple of 8 with zeros.
static bool panel_gradients(hipStream_t st, const Workspace& w, char* ws, const uint16_t* hid, int64_t n_tok, int64_t H,
                            int64_t V, uint16_t* d_hidden_chunk, void* d_weight, bool dw_f32, bool first) {
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
  return lt::gemm(st, true, false, H, V, kp, hid_t, kp, ds_t, kp, d_weight, H, dw_f32, first ? 0.f : 1.f, lt_ws,
                  lt::kWorkspaceBytes);
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

static bool shapes_ok(int64_t T, int64_t H, int64_t V) {
  return T > 0 && H > 0 && V > 0 && (H % 8) == 0 && (V % 8) == 0 && T < (1 << 30) && V < (1 << 30) && H < (1 << 30) &&
         (V / 64 + 1) * ((H > kChunkTokens ? H : kChunkTokens) / 64 + 1) < (1LL << 31);  // transpose grids
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
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  auto at = [](float* p, int64_t t0) { return p ? p + t0 : nullptr; };
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    if (!panel_logits(st, w, ws, (const uint16_t*)hidden + t0 * H, weight, n_tok, H, V)) return AA_ERR_LAUNCH;
    const int rc = aa_logits_fwd(ws + w.off_ds, AA_BF16, n_tok, V, V, labels + t0, inv_temperature, logp + t0,
                                 at(entropy, t0), at(row_lse, t0), at(row_ez, t0), nullptr, nullptr, stream);
    if (rc != AA_OK) return rc;
  }
  return launch_status();
}

extern "C" int aa_lmhead_bwd(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                             const int64_t* labels, float inv_temperature, const float* row_lse, const float* row_ez,
                             const float* g_logp, const float* g_entropy, void* d_hidden, void* d_weight,
                             int d_weight_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  if (!hidden || !weight || !labels || !row_lse || !g_logp || !d_hidden || !d_weight || !workspace)
    return AA_ERR_INVALID_ARGUMENT;
  if ((g_entropy && !row_ez) || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V) || (d_weight_dtype != AA_F32 && d_weight_dtype != AA_BF16)) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace | (uintptr_t)d_hidden | (uintptr_t)d_weight) & 15))
    return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V);
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  void* ds = ws + w.off_ds;  // [chunk, V]: logits of the chunk, then their gradient in place
  launch_transpose(st, (const uint16_t*)weight, V, H, H, (uint16_t*)(ws + w.off_wt));
  const WeightGrad dw = weight_grad(w, ws, d_weight, d_weight_dtype, T);
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    if (!panel_logits(st, w, ws, hid, weight, n_tok, H, V)) return AA_ERR_LAUNCH;
    const int rc = aa_logits_bwd(ds, AA_BF16, n_tok, V, V, labels + t0, inv_temperature, row_lse + t0,
                                 row_ez ? row_ez + t0 : nullptr, g_logp + t0, g_entropy ? g_entropy + t0 : nullptr, n_tok,
                                 ds, stream);
    if (rc != AA_OK) return rc;
    if (!panel_gradients(st, w, ws, hid, n_tok, H, V, (uint16_t*)d_hidden + t0 * H, dw.acc, dw.acc_f32, t0 == 0))
      return AA_ERR_LAUNCH;
  }
  finish_weight_grad(st, dw, d_weight, V, H);
  return launch_status();
}

extern "C" int aa_lmhead_ppo_fused(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                                   const int64_t* labels, float inv_temperature, int64_t T_active,
                                   const float* prox_logp, const float* adv, const uint8_t* mask_eff,
                                   const float* behave_w, const aa_ppo_params* params, const int32_t* n_valid,
                                   const float* grad_scale, float* logp, float* entropy, float* stat_loss, float* ratio,
                                   uint8_t* flags, void* d_hidden, void* d_weight, int d_weight_dtype, int32_t* work,
                                   void* workspace, int64_t workspace_bytes, void* stream) {
  if (!hidden || !weight || !labels || !d_hidden || !d_weight || !workspace) return AA_ERR_INVALID_ARGUMENT;
  if (!params || !n_valid || !logp) return AA_ERR_INVALID_ARGUMENT;
  if (T_active < 0 || T_active > T || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  if (T_active > 0 && (!prox_logp || !adv || !mask_eff || !stat_loss || !ratio || !flags)) return AA_ERR_INVALID_ARGUMENT;
  if (T_active > 0 && params->has_behave_weight && !behave_w) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V) || (d_weight_dtype != AA_F32 && d_weight_dtype != AA_BF16)) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace | (uintptr_t)d_hidden | (uintptr_t)d_weight) & 15))
    return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V);
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  uint16_t* ds = (uint16_t*)(ws + w.off_ds);  // [chunk, V]: logits of the chunk, then their gradient in place
  launch_transpose(st, (const uint16_t*)weight, V, H, H, (uint16_t*)(ws + w.off_wt));
  const WeightGrad dw = weight_grad(w, ws, d_weight, d_weight_dtype, T);
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    int64_t act = T_active - t0;
    act = act < 0 ? 0 : (act > n_tok ? n_tok : act);
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    if (!panel_logits(st, w, ws, hid, weight, n_tok, H, V)) return AA_ERR_LAUNCH;
    // log-prob, entropy, PPO loss and d(loss)/d(logits) in place: one streaming pass over the panel
    auto at = [t0](auto* p) { return p ? p + t0 : nullptr; };
    const int rc = aa_logits_ppo_fused(ds, AA_BF16, n_tok, V, V, labels + t0, inv_temperature, act, at(prox_logp), at(adv),
                                       at(mask_eff), at(behave_w), params, n_valid, grad_scale, logp + t0, at(entropy),
                                       nullptr, nullptr, at(stat_loss), at(ratio), at(flags), ds, work, stream);
    if (rc != AA_OK) return rc;
    if (!panel_gradients(st, w, ws, hid, n_tok, H, V, (uint16_t*)d_hidden + t0 * H, dw.acc, dw.acc_f32, t0 == 0))
      return AA_ERR_LAUNCH;
  }
  finish_weight_grad(st, dw, d_weight, V, H);
  return launch_status();
}
