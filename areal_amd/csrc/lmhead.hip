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
#include "logits_path.h"
#include "lt_gemm.h"

namespace aa {
namespace lmhead {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kChunkTokens = 16384;  // token chunk of the logits panel

__host__ __device__ __forceinline__ int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// ---- bf16 transpose: dst[c, r] = src[r, c] ----------------------------------------------------------------------
// src is [R, C] with row pitch lds (elements), dst is [C, ldd] with ldd = R rounded up to 8; columns R .. ldd - 1 of dst
// are written as zeros; with src_rows, row r of the source is row src_rows[r] of the array.  One workgroup moves a 64 x 64 tile through LDS: each thread loads 8 elements of two
// adjacent rows (16 B each), pairs them into 32-bit words (two consecutive dst columns) and stores the words
// transposed; the second half reads 16 B per thread and writes 128 B contiguous per dst row.  The word index is
// XOR-ed with a key of the row so that both halves run without bank conflicts.  Requires C % 8 == 0, lds % 8 == 0.
// Tiles are numbered along r first, in bands of kTransposeBand tile rows, so that the workgroups in flight together
// write long contiguous pieces of the dst rows (measured: 5.2 TB/s against 3.9 with c first).
constexpr int kTransposeBand = 64;

__global__ __launch_bounds__(256) void k_transpose_bf16(const uint16_t* __restrict__ src, int R, int C, int64_t lds,
                                                        uint16_t* __restrict__ dst, int64_t ldd, int tiles_c,
                                                        int tiles_r, const int32_t* __restrict__ src_rows) {
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
    if (c < C) {  // logical row r of the source is row src_rows[r] of src when a row list is given
      if (r < R) a = __builtin_nontemporal_load((const u32x4_t*)(src + (int64_t)(src_rows ? src_rows[r] : r) * lds + c));
      if (r + 1 < R)
        b = __builtin_nontemporal_load((const u32x4_t*)(src + (int64_t)(src_rows ? src_rows[r + 1] : r + 1) * lds + c));
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

// dst gets ldd columns (ldd >= R, a multiple of 8): the transposed R rows of src, then zeros
static void launch_transpose(hipStream_t st, const uint16_t* src, int64_t R, int64_t C, int64_t lds, uint16_t* dst,
                             int64_t ldd, const int32_t* src_rows = nullptr) {
  const int64_t tiles_c = (C + 63) / 64, tiles_r = (ldd + 63) / 64;
  hipLaunchKernelGGL(k_transpose_bf16, dim3((unsigned)(tiles_c * tiles_r)), dim3(256), 0, st, src, (int)R, (int)C, lds, dst,
                     ldd, (int)tiles_c, (int)tiles_r, src_rows);
}

// ---- tokens without gradient are left out of the backward GEMMs -------------------------------------------------
// A token whose loss mask is zero has d(loss)/d(logits) == 0: its row adds nothing to d_weight and its d_hidden row
// is zero.  k_compact_map numbers the tokens of a chunk that do have a mask (in order): out_rows[t] = position of
// token t among them, or -1; act_rows[position] = t.  `limit` is the count the host sized the GEMMs with; tokens
// beyond it are dropped.  One workgroup; mask has `act` entries (tokens at and after `act` have no mask).
__global__ __launch_bounds__(1024) void k_compact_map(const uint8_t* __restrict__ mask, int act, int n_tok, int limit,
                                                      int32_t* __restrict__ out_rows, int32_t* __restrict__ act_rows) {
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
  // a host count larger than what the mask holds leaves positions without a token: point them at row 0, so that the
  // gathers that follow stay inside the chunk (their contribution is then meaningless, as the caller's count was)
  int total = 0;
  for (int w = 0; w < 16; ++w) total += wave_sum[w];
  for (int p = total + tid; p < limit; p += 1024) act_rows[p] = 0;
}

// dst[t, :] = out_rows[t] >= 0 ? src[out_rows[t], :] : 0 for the n_tok rows of a chunk (H % 8 == 0)
__global__ __launch_bounds__(256) void k_scatter_rows(const u32x4_t* __restrict__ src, const int32_t* __restrict__ out_rows,
                                                      u32x4_t* __restrict__ dst, int h_vec) {
  const int64_t t = blockIdx.x;
  const int r = out_rows[t];
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  for (int j = threadIdx.x; j < h_vec; j += 256) dst[t * h_vec + j] = r >= 0 ? src[(int64_t)r * h_vec + j] : zero;
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
  int64_t off_rows, off_dhc;        // row maps of k_compact_map (2 x chunk int32), d_hidden of the kept tokens
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
  w.off_rows = off; off += up(2 * w.chunk * 4);
  w.off_dhc = off;  off += up(w.chunk * H * 2);
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

// The two GEMMs that contract the d(logits) rows ds [n_rows, V] of one token chunk:
//   d_hidden rows = ds . W          (bf16)          d_weight (+)= ds^T . hidden rows   (fp32, or bf16 when first)
// with transposed copies of ds and of the hidden rows (made here) and of the weight (made once per call, by the
// caller, at ws + off_wt).  ds sits in one of the two panel buffers (byte offset ds_off), its transpose goes to the
// other (dst_off).  hid_rows, when given, lists the rows of the hidden chunk that the n_rows rows of ds belong to
// (tokens without gradient were left out).  The GEMMs run on n_gemm >= n_rows rows (the library is much faster on
// round sizes): the transposed copies carry zeros there.  d_hidden_rows receives n_dh rows (n_rows, or n_gemm when
// it is a scratch buffer with room for them).
static bool panel_gradients(hipStream_t st, const Workspace& w, char* ws, int64_t ds_off, int64_t dst_off,
                            const uint16_t* hid, const int32_t* hid_rows, int64_t n_rows, int64_t n_gemm, int64_t n_dh,
                            int64_t H, int64_t V, uint16_t* d_hidden_rows, void* d_weight, bool dw_f32, bool first) {
  const uint16_t* ds = (const uint16_t*)(ws + ds_off);
  uint16_t* ds_t = (uint16_t*)(ws + dst_off);
  const uint16_t* w_t = (const uint16_t*)(ws + w.off_wt);
  uint16_t* hid_t = (uint16_t*)(ws + w.off_ht);
  void* lt_ws = ws + w.off_lt;
  // column-major [H, n_dh] = (W^T)'^T [H, V] . ds' [V, n_dh]
  if (!lt::gemm(st, true, false, H, n_dh, V, w_t, V, ds, V, d_hidden_rows, H, false, 0.f, lt_ws, lt::kWorkspaceBytes))
    return false;
  launch_transpose(st, ds, n_rows, V, V, ds_t, n_gemm);
  launch_transpose(st, hid, n_rows, H, H, hid_t, n_gemm, hid_rows);
  // column-major [H, V] = (hidden^T)'^T [H, n_gemm] . (ds^T)' [n_gemm, V], fp32, accumulated over the chunks
  return lt::gemm(st, true, false, H, V, n_gemm, hid_t, n_gemm, ds_t, n_gemm, d_weight, H, dw_f32, first ? 0.f : 1.f,
                  lt_ws, lt::kWorkspaceBytes);
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

// Row count of the d_hidden GEMM for `kept` rows with a gradient (its output is a scratch buffer with room for a whole
// chunk, the extra rows are never read).  The library's kernels for a small output with a very long contraction
// split the contraction over the compute units, and at H = 4096 (16 tiles of 256 across) they run 20 % slower when
// the 256 x 256 output tiles do not come to a multiple of half the unit count (n = 11520: 720 tiles, 11.9 ms;
// n = 12288: 768 tiles, 9.9 ms).  Where H allows such a multiple within 2048 rows the count is rounded up to it;
// otherwise (H = 5376: 21 tiles across, no gain measured) to the tile size.  The d_weight GEMM, where the rows are
// the contraction, always takes the count rounded up to 256.
static int64_t d_hidden_gemm_rows(int64_t kept, int64_t chunk, int64_t H) {
  static const int64_t half_units = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 2)
      cus = 256;
    return (int64_t)cus / 2;
  }();
  const int64_t tiles_across = (H + 255) / 256;
  int64_t step = 256;
  if (half_units % tiles_across == 0 && half_units / tiles_across <= 8) step = 256 * (half_units / tiles_across);
  const int64_t n = round_up(kept, step);
  return n < chunk ? n : chunk;
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
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  launch_transpose(st, (const uint16_t*)weight, V, H, H, (uint16_t*)(ws + w.off_wt), V);
  const WeightGrad dw = weight_grad(w, ws, d_weight, d_weight_dtype, T);
  int32_t* out_rows = (int32_t*)(ws + w.off_rows);
  int32_t* act_rows = out_rows + w.chunk;
  bool first = true;  // no GEMM has written d_weight yet
  int64_t chunk_index = 0;
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk, ++chunk_index) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    uint16_t* dh = (uint16_t*)d_hidden + t0 * H;
    const float* ez = row_ez ? row_ez + t0 : nullptr;
    const float* gh = g_entropy ? g_entropy + t0 : nullptr;
    if (!kept_per_chunk) {
      void* ds = ws + w.off_ds;  // [chunk, V]: logits of the chunk, then their gradient in place
      if (!panel_logits(st, w, ws, hid, weight, n_tok, H, V)) return AA_ERR_LAUNCH;
      const int rc = aa_logits_bwd(ds, AA_BF16, n_tok, V, V, labels + t0, inv_temperature, row_lse + t0, ez, g_logp + t0,
                                   gh, n_tok, ds, stream);
      if (rc != AA_OK) return rc;
      if (!panel_gradients(st, w, ws, w.off_ds, w.off_dst, hid, nullptr, n_tok, round_up(n_tok, 8), n_tok, H, V, dh,
                           dw.acc, dw.acc_f32, first))
        return AA_ERR_LAUNCH;
      first = false;
      continue;
    }
    // rows whose upstream gradients are all zero are left out, as in aa_lmhead_ppo_fused
    int64_t kept = kept_per_chunk[chunk_index];
    kept = kept < 0 ? 0 : (kept > n_tok ? n_tok : kept);
    if (kept == 0) {
      launch_zero(st, dh, n_tok * H * 2);
      continue;
    }
    hipLaunchKernelGGL(k_compact_map, dim3(1), dim3(1024), 0, st, row_has_gradient + t0, (int)n_tok, (int)n_tok, (int)kept,
                       out_rows, act_rows);
    if (!panel_logits(st, w, ws, hid, weight, n_tok, H, V)) return AA_ERR_LAUNCH;
    const int rc = logits_bwd_rows(ws + w.off_ds, AA_BF16, n_tok, V, V, labels + t0, inv_temperature, row_lse + t0, ez,
                                   g_logp + t0, gh, n_tok, ws + w.off_dst, out_rows, stream);
    if (rc != AA_OK) return rc;
    uint16_t* dh_kept = (uint16_t*)(ws + w.off_dhc);
    if (!panel_gradients(st, w, ws, w.off_dst, w.off_ds, hid, act_rows, kept, round_up(kept, 256),
                         d_hidden_gemm_rows(kept, w.chunk, H), H, V, dh_kept, dw.acc,
                         dw.acc_f32, first))
      return AA_ERR_LAUNCH;
    first = false;
    hipLaunchKernelGGL(k_scatter_rows, dim3((unsigned)n_tok), dim3(256), 0, st, (const u32x4_t*)dh_kept, out_rows,
                       (u32x4_t*)dh, (int)(H / 8));
  }
  if (first) launch_zero(st, dw.acc, V * H * (dw.acc_f32 ? 4 : 2));  // no row of the batch has a gradient
  finish_weight_grad(st, dw, d_weight, V, H);
  return launch_status();
}

extern "C" int64_t aa_lmhead_chunk_tokens(void) { return kChunkTokens; }

extern "C" int aa_lmhead_ppo_fused(const void* hidden, const void* weight, int64_t T, int64_t H, int64_t V,
                                   const int64_t* labels, float inv_temperature, int64_t T_active,
                                   const float* prox_logp, const float* adv, const uint8_t* mask_eff,
                                   const float* behave_w, const aa_ppo_params* params, const int32_t* n_valid,
                                   const float* grad_scale, const int64_t* kept_per_chunk, float* logp, float* entropy,
                                   float* stat_loss, float* ratio, uint8_t* flags, void* d_hidden, void* d_weight,
                                   int d_weight_dtype, int32_t* work, void* workspace, int64_t workspace_bytes,
                                   void* stream) {
  if (!hidden || !weight || !labels || !d_hidden || !d_weight || !workspace) return AA_ERR_INVALID_ARGUMENT;
  if (!params || !n_valid || !logp) return AA_ERR_INVALID_ARGUMENT;
  if (T_active < 0 || T_active > T || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  const bool nll = params->loss_kind == AA_LOSS_NLL;  // prox_logp and adv are not used by that loss
  if (T_active > 0 && (!mask_eff || !stat_loss || !ratio || !flags)) return AA_ERR_INVALID_ARGUMENT;
  if (T_active > 0 && !nll && (!prox_logp || !adv)) return AA_ERR_INVALID_ARGUMENT;
  if (T_active > 0 && params->has_behave_weight && !behave_w) return AA_ERR_INVALID_ARGUMENT;
  if (!shapes_ok(T, H, V) || (d_weight_dtype != AA_F32 && d_weight_dtype != AA_BF16)) return AA_ERR_UNSUPPORTED;
  if ((((uintptr_t)hidden | (uintptr_t)weight | (uintptr_t)workspace | (uintptr_t)d_hidden | (uintptr_t)d_weight) & 15))
    return AA_ERR_INVALID_ARGUMENT;
  const Workspace w = plan(T, H, V);
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  launch_transpose(st, (const uint16_t*)weight, V, H, H, (uint16_t*)(ws + w.off_wt), V);
  const WeightGrad dw = weight_grad(w, ws, d_weight, d_weight_dtype, T);
  int32_t* out_rows = (int32_t*)(ws + w.off_rows);
  int32_t* act_rows = out_rows + w.chunk;
  bool first = true;  // no GEMM has written d_weight yet
  int64_t chunk_index = 0;
  for (int64_t t0 = 0; t0 < T; t0 += w.chunk, ++chunk_index) {
    const int64_t n_tok = (T - t0) < w.chunk ? (T - t0) : w.chunk;
    int64_t act = T_active - t0;
    act = act < 0 ? 0 : (act > n_tok ? n_tok : act);
    const uint16_t* hid = (const uint16_t*)hidden + t0 * H;
    uint16_t* dh = (uint16_t*)d_hidden + t0 * H;
    auto at = [t0](auto* p) { return p ? p + t0 : nullptr; };
    if (!panel_logits(st, w, ws, hid, weight, n_tok, H, V)) return AA_ERR_LAUNCH;
    if (!kept_per_chunk) {
      // log-prob, entropy, PPO loss and d(loss)/d(logits) in place: one streaming pass over the panel
      void* ds = ws + w.off_ds;
      const int rc = aa_logits_ppo_fused(ds, AA_BF16, n_tok, V, V, labels + t0, inv_temperature, act, at(prox_logp),
                                         at(adv), at(mask_eff), at(behave_w), params, n_valid, grad_scale, logp + t0,
                                         at(entropy), nullptr, nullptr, at(stat_loss), at(ratio), at(flags), ds, work,
                                         stream);
      if (rc != AA_OK) return rc;
      if (!panel_gradients(st, w, ws, w.off_ds, w.off_dst, hid, nullptr, n_tok, round_up(n_tok, 8), n_tok, H, V, dh,
                           dw.acc, dw.acc_f32, first))
        return AA_ERR_LAUNCH;
      first = false;
      continue;
    }
    // Tokens whose mask is zero have no gradient: the streaming pass writes the gradient rows of the other tokens,
    // closed up, into the second panel buffer, and the backward GEMMs run on those rows only.
    int64_t kept = kept_per_chunk[chunk_index];
    kept = kept < 0 ? 0 : (kept > act ? act : kept);
    hipLaunchKernelGGL(k_compact_map, dim3(1), dim3(1024), 0, st, at(mask_eff), (int)act, (int)n_tok, (int)kept, out_rows,
                       act_rows);
    const int rc = logits_ppo_fused_rows(ws + w.off_ds, AA_BF16, n_tok, V, V, labels + t0, inv_temperature, act,
                                         at(prox_logp), at(adv), at(mask_eff), at(behave_w), params, n_valid, grad_scale,
                                         logp + t0, at(entropy), nullptr, nullptr, at(stat_loss), at(ratio), at(flags),
                                         ws + w.off_dst, out_rows, work, stream);
    if (rc != AA_OK) return rc;
    if (kept == 0) {
      launch_zero(st, dh, n_tok * H * 2);
      continue;
    }
    uint16_t* dh_kept = (uint16_t*)(ws + w.off_dhc);
    if (!panel_gradients(st, w, ws, w.off_dst, w.off_ds, hid, act_rows, kept, round_up(kept, 256),
                         d_hidden_gemm_rows(kept, w.chunk, H), H, V, dh_kept, dw.acc,
                         dw.acc_f32, first))
      return AA_ERR_LAUNCH;
    first = false;
    hipLaunchKernelGGL(k_scatter_rows, dim3((unsigned)n_tok), dim3(256), 0, st, (const u32x4_t*)dh_kept, out_rows,
                       (u32x4_t*)dh, (int)(H / 8));
  }
  if (first) launch_zero(st, dw.acc, V * H * (dw.acc_f32 ? 4 : 2));  // no token of the batch has a gradient
  finish_weight_grad(st, dw, d_weight, V, H);
  return launch_status();
}
