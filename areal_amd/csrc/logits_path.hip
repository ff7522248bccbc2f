// Logits path for gfx950: per-token log-prob / entropy over the full vocabulary,
// its backward, and the fused forward + token-level PPO loss + backward.
//
// Replaces, for one GPU, the PyTorch sequence
//   log_softmax(logits.float() / T) -> gather -> (entropy) -> ppo_actor_loss_fn -> autograd
// (areal/utils/functional/vocab_parallel.py:15-29,
//  areal/utils/functional/functional.py:429-559).
//
// All kernels are HBM-streaming kernels: one workgroup owns one row of the
// [T, V] logits.  Exponentials are taken in base 2 with c = log2(e) / T folded
// into one fma per element; with t_j = x_j c - k row statistics are carried as
//   k = max_j x_j * c,   s = sum_j 2^t_j,   u = sum_j t_j 2^t_j
// so that  logp = ln2 (t_label - log2 s)  and  entropy = ln2 (log2 s - u / s)
// are differences of small numbers whatever the magnitude of the logits.
#include "device_utils.h"
#include "ppo_math.h"

namespace aa {

// -----------------------------------------------------------------------------
// Generic row traversal (any V, any row alignment): a scalar head up to the
// first 16-byte boundary, 8-element vectors, a scalar tail.
// -----------------------------------------------------------------------------
struct RowSplit {
  int head;   // scalar elements before the vector body
  int nvec;   // 8-element vectors
  int tail0;  // first element of the scalar tail
};

template <int DT>
__device__ __forceinline__ RowSplit split_row(const void* row, int V, bool vec_ok) {
  RowSplit r;
  if (!vec_ok) {
    r.head = V; r.nvec = 0; r.tail0 = V;
    return r;
  }
  const int mis = (int)((uintptr_t)row & 15);
  int head = mis ? (16 - mis) / Elem<DT>::kBytes : 0;
  if (head > V) head = V;
  r.head = head;
  r.nvec = (V - head) >> 3;
  r.tail0 = head + (r.nvec << 3);
  return r;
}

struct ThreadStats {
  float k, s, u, mx, mn;
};

// move the partial sums to a larger reference exponent k_new >= a.k
__device__ __forceinline__ void rebase(ThreadStats& a, float k_new) {
  const float d = a.k - k_new;
  const float f = fast_exp2(d);
  a.u = f * fmaf(d, a.s, a.u);
  a.s *= f;
  a.k = k_new;
}

__device__ __forceinline__ void stats_add1(ThreadStats& a, float x, float c) {
  const float xc = x * c;
  if (xc > a.k) rebase(a, xc);
  const float t = fmaf(x, c, -a.k);
  const float e = fast_exp2(t);
  a.s += e;
  a.u = fmaf(t, e, a.u);
  a.mx = __builtin_elementwise_maximum(a.mx, x);
  a.mn = __builtin_elementwise_minimum(a.mn, x);
}

__device__ __forceinline__ void stats_add8(ThreadStats& a, const float (&x)[8], float c) {
  const float m8 = max_of<8>(x), n8 = min_of<8>(x);
  const float kc = m8 * c;
  if (kc > a.k) rebase(a, kc);
  a.mx = __builtin_elementwise_maximum(a.mx, m8);
  a.mn = __builtin_elementwise_minimum(a.mn, n8);
  float s = 0.f, u = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float t = fmaf(x[i], c, -a.k);
    const float e = fast_exp2(t);
    s += e;
    u = fmaf(t, e, u);
  }
  a.s += s;
  a.u += u;
}

// The same with the parts left out that a caller has no use for: the entropy sum u (WANT_U) and the extrema
// (WANT_MM; the eight-way maximum is needed for the reference exponent either way).  A forward pass for log-probs
// alone is otherwise bound by these instructions on 16-bit rows, not by the memory.
template <bool WANT_U, bool WANT_MM>
__device__ __forceinline__ void stats_add8_sel(ThreadStats& a, const float (&x)[8], float c) {
  const float m8 = max_of<8>(x);
  const float kc = m8 * c;
  if (kc > a.k) rebase(a, kc);
  if constexpr (WANT_MM) {
    const float n8 = min_of<8>(x);
    a.mx = __builtin_elementwise_maximum(a.mx, m8);
    a.mn = __builtin_elementwise_minimum(a.mn, n8);
  }
  float s = 0.f, u = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float t = fmaf(x[i], c, -a.k);
    const float e = fast_exp2(t);
    s += e;
    if constexpr (WANT_U) u = fmaf(t, e, u);
  }
  a.s += s;
  if constexpr (WANT_U) a.u += u;
}

struct RowStats {
  float k, s, u, mx, mn;  // merged over the workgroup, same value in every thread
};

// Merge in a fixed order: lane butterflies inside each wave, then a butterfly
// over the per-wave entries (each lane reads entry lane % NWAVES, so every
// thread ends with the same value without a second barrier).
template <int NWAVES>
__device__ __forceinline__ RowStats block_stats(const ThreadStats& t, float* smem) {
  static_assert(NWAVES >= 1 && NWAVES <= 16 && (NWAVES & (NWAVES - 1)) == 0, "power-of-two wave count");
  const float wk = wave_max(t.k);
  const float dk = t.k - wk;
  const float f = fast_exp2(dk);
  const float ws = wave_sum(t.s * f);
  const float wu = wave_sum(f * fmaf(dk, t.s, t.u));
  const float wmx = wave_max(t.mx);
  const float wmn = wave_min(t.mn);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  __syncthreads();  // smem may still be read from a previous use
  if (lane == 0) {
    smem[wave * 5 + 0] = wk; smem[wave * 5 + 1] = ws; smem[wave * 5 + 2] = wu;
    smem[wave * 5 + 3] = wmx; smem[wave * 5 + 4] = wmn;
  }
  __syncthreads();
  const int e = lane & (NWAVES - 1);
  RowStats r{smem[e * 5 + 0], smem[e * 5 + 1], smem[e * 5 + 2], smem[e * 5 + 3], smem[e * 5 + 4]};
#pragma unroll
  for (int o = NWAVES / 2; o > 0; o >>= 1) {
    const float qk = __shfl_xor(r.k, o, kWave);
    const float qs = __shfl_xor(r.s, o, kWave);
    const float qu = __shfl_xor(r.u, o, kWave);
    const float nk = fmaxf(r.k, qk);
    const float da = r.k - nk, db = qk - nk;
    const float fa = fast_exp2(da), fb = fast_exp2(db);
    // symmetric in (r, q): both partners compute bit-identical sums
    r.u = fa * fmaf(da, r.s, r.u) + fb * fmaf(db, qs, qu);
    r.s = r.s * fa + qs * fb;
    r.k = nk;
    r.mx = fmaxf(r.mx, __shfl_xor(r.mx, o, kWave));
    r.mn = fminf(r.mn, __shfl_xor(r.mn, o, kWave));
  }
  return r;
}

template <int DT, int NT, bool STREAM = false, bool WANT_U = true, bool WANT_MM = true>
__device__ __forceinline__ RowStats row_stats_generic(const void* row, int V, bool vec_ok, float c, float* smem) {
  ThreadStats a{kNegBig, 0.f, 0.f, -FLT_MAX, FLT_MAX};
  const RowSplit sp = split_row<DT>(row, V, vec_ok);
  const int tid = threadIdx.x;
  for (int j = tid; j < sp.head; j += NT) stats_add1(a, Elem<DT>::load1(row, j), c);
  if constexpr (STREAM && DT == AA_F32) {
    // fp32, read once: a thread's eight values are two 16-byte pieces NT pieces apart, so that every load instruction
    // of a wave covers 1 KB of consecutive addresses (eight values side by side make two instructions touch every
    // 128-byte line: slower, and the nt policy then costs instead of gaining); statistics do not depend on the order
    const int n4 = sp.nvec * 2;  // 16-byte pieces of the vector body
    const float* body = (const float*)row + sp.head;
    int v = tid;
    for (; v + NT < n4; v += 2 * NT) {
      float x[8];
      load4_stream(body + ((int64_t)v << 2), x);
      load4_stream(body + ((int64_t)(v + NT) << 2), x + 4);
      stats_add8_sel<WANT_U, WANT_MM>(a, x, c);
    }
    if (v < n4) {
      float x[4];
      load4_stream(body + ((int64_t)v << 2), x);
#pragma unroll
      for (int i = 0; i < 4; ++i) stats_add1(a, x[i], c);
    }
  } else {
    for (int v = tid; v < sp.nvec; v += NT) {
      float x[8];
      if constexpr (STREAM) load8_stream<DT>(row, sp.head + ((int64_t)v << 3), x);  // the row is not read again
      else load8<DT>(row, sp.head + ((int64_t)v << 3), x);
      stats_add8_sel<WANT_U, WANT_MM>(a, x, c);
    }
  }
  for (int j = sp.tail0 + tid; j < V; j += NT) stats_add1(a, Elem<DT>::load1(row, j), c);
  return block_stats<NT / kWave>(a, smem);
}

// Row-level quantities derived from the merged statistics.
struct RowOut {
  float log2s;    // log2 s
  float lse2;     // log2 sum_j 2^(x_j c) = k + log2 s
  float lse;      // natural-log logsumexp of z = x / T
  float ez;       // sum_j p_j z_j
  float entropy;  // lse - ez, formed without cancellation
};

__device__ __forceinline__ RowOut finish_row(const RowStats& r) {
  RowOut o;
  const float mean_t = r.u / r.s;  // sum_j p_j t_j  (<= 0)
  o.log2s = fast_log2(r.s);
  o.lse2 = r.k + o.log2s;
  o.lse = o.lse2 * kLn2;
  o.ez = (r.k + mean_t) * kLn2;
  o.entropy = (o.log2s - mean_t) * kLn2;
  return o;
}

// log-prob of the label from its raw logit
__device__ __forceinline__ float label_logp(float xy, float c, const RowStats& r, const RowOut& o) {
  return (fmaf(xy, c, -r.k) - o.log2s) * kLn2;
}

// out_j = p_j * (A + B x_j), p_j = 2^(x_j c - lse2); the label gets + lab_add.
struct GradCoef {
  float c, lse2, A, B, lab_add;
  int label;  // -1 = none
};

// A + B x.  With B == 0 (no gradient flows through the entropy) the product is left out, so that a logit of -inf
// (a masked vocabulary entry) gets the gradient 0 that autograd gives it and not 0 * inf.  With B != 0 such a logit
// has a NaN gradient in the reference as well (the entropy itself is NaN there).
__device__ __forceinline__ float grad_weight(const GradCoef& g, float x) { return g.B == 0.f ? g.A : fmaf(g.B, x, g.A); }

// STREAM: the row and its gradient pass through once (`nt` policy on loads and stores); fp32 rows then go in 16-byte
// pieces, so that every load and store instruction of a wave covers 1 KB of consecutive addresses.
template <int DT, int NT, bool STREAM = false>
__device__ __forceinline__ void row_grad_generic(const void* row, void* out, int V, bool vec_ok, const GradCoef& g) {
  const RowSplit sp = split_row<DT>(row, V, vec_ok);
  const int tid = threadIdx.x;
  auto one = [&](int j) {
    const float x = Elem<DT>::load1(row, j);
    float o = fast_exp2(fmaf(x, g.c, -g.lse2)) * grad_weight(g, x);
    if (j == g.label) o += g.lab_add;
    Elem<DT>::store1(out, j, o);
  };
  for (int j = tid; j < sp.head; j += NT) one(j);
  if constexpr (STREAM && DT == AA_F32) {
    const int n4 = sp.nvec * 2;
    for (int v = tid; v < n4; v += NT) {
      const int e0 = sp.head + (v << 2);
      float x[4], o[4];
      load4_stream((const float*)row + e0, x);
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = fast_exp2(fmaf(x[i], g.c, -g.lse2)) * grad_weight(g, x[i]);
      if ((unsigned)(g.label - e0) < 4u) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (e0 + i == g.label) o[i] += g.lab_add;
      }
      store4_stream((float*)out + e0, o);
    }
    for (int j = sp.tail0 + tid; j < V; j += NT) one(j);
    return;
  }
  for (int v = tid; v < sp.nvec; v += NT) {
    const int e0 = sp.head + (v << 3);
    float x[8], o[8];
    if constexpr (STREAM) load8_stream<DT>(row, e0, x);
    else load8<DT>(row, e0, x);
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = fast_exp2(fmaf(x[i], g.c, -g.lse2)) * grad_weight(g, x[i]);
    if ((unsigned)(g.label - e0) < 8u) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (e0 + i == g.label) o[i] += g.lab_add;
    }
    if constexpr (STREAM && DT != AA_F32) store8_stream16<DT>(out, e0, o);
    else store8<DT>(out, e0, o);
  }
  for (int j = sp.tail0 + tid; j < V; j += NT) one(j);
}

template <int DT, int NT, bool STREAM = false>
__device__ __forceinline__ void row_zero_generic(const void* row_like, void* out, int V, bool vec_ok) {
  const RowSplit sp = split_row<DT>(row_like, V, vec_ok);
  const int tid = threadIdx.x;
  const float z[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int j = tid; j < sp.head; j += NT) Elem<DT>::store1(out, j, 0.f);
  if constexpr (STREAM && DT == AA_F32) {
    for (int v = tid; v < sp.nvec * 2; v += NT) store4_stream((float*)out + sp.head + (v << 2), z);
  } else if constexpr (STREAM) {
    for (int v = tid; v < sp.nvec; v += NT) store8_stream16<DT>(out, sp.head + (v << 3), z);
  } else {
    for (int v = tid; v < sp.nvec; v += NT) store8<DT>(out, sp.head + (v << 3), z);
  }
  for (int j = sp.tail0 + tid; j < V; j += NT) Elem<DT>::store1(out, j, 0.f);
}

__device__ __forceinline__ const void* row_ptr(const void* base, int64_t t, int64_t stride, int bytes) {
  return (const char*)base + t * stride * bytes;
}

// -----------------------------------------------------------------------------
// Forward: logp, entropy, row statistics.  grid = T rows, NT threads.
// -----------------------------------------------------------------------------
template <int DT, int NT, bool WANT_U, bool WANT_MM>
__global__ __launch_bounds__(NT) void k_logits_fwd(const void* __restrict__ logits, int V, int64_t stride,
                                                   const int64_t* __restrict__ labels, float inv_t, int vec_ok,
                                                   float* __restrict__ logp, float* __restrict__ entropy,
                                                   float* __restrict__ row_lse, float* __restrict__ row_ez,
                                                   float* __restrict__ vmax, float* __restrict__ vmin) {
  __shared__ float smem[(NT / kWave) * 5];
  const int64_t t = blockIdx.x;
  const void* row = row_ptr(logits, t, stride, Elem<DT>::kBytes);
  const float c = kLog2e * inv_t;
  const int64_t y = labels[t];
  const bool y_ok = (y >= 0) && (y < V);
  const float xy = y_ok ? Elem<DT>::load1(row, y) : 0.f;
  const RowStats rs = row_stats_generic<DT, NT, true, WANT_U, WANT_MM>(row, V, vec_ok != 0, c, smem);
  if (threadIdx.x == 0) {
    const RowOut ro = finish_row(rs);
    logp[t] = y_ok ? label_logp(xy, c, rs, ro) : __builtin_nanf("");
    if (entropy) entropy[t] = ro.entropy;
    if (row_lse) row_lse[t] = ro.lse;
    if (row_ez) row_ez[t] = ro.ez;
    if (vmax) vmax[t] = rs.mx;
    if (vmin) vmin[t] = rs.mn;
  }
}

// Pointer types of an input / output pair that may be ONE array (the gradient written over the logits, ALIAS): the
// restrict qualifier, which tells the compiler that the two never overlap, is there only when they are known to be
// distinct.  The kernels that take such a pair are instantiated both ways and the entry points choose.
template <bool ALIAS, typename T>
struct InPtr {
  typedef const T* __restrict__ type;
};
template <typename T>
struct InPtr<true, T> {
  typedef const T* type;
};
template <bool ALIAS, typename T>
struct OutPtr {
  typedef T* __restrict__ type;
};
template <typename T>
struct OutPtr<true, T> {
  typedef T* type;
};

// -----------------------------------------------------------------------------
// Backward: dlogits from g_logp / g_entropy and the saved row statistics.
// -----------------------------------------------------------------------------
// STREAM: `nt` loads and stores (the host asks for them when the rows start on 128-byte lines: with rows that do
// not, the pieces that two waves write into one line are no longer merged in the cache, and the pass is slower).
template <int DT, int NT, bool ALIAS, bool STREAM>
__global__ __launch_bounds__(NT) void k_logits_bwd(typename InPtr<ALIAS, void>::type logits, int V, int64_t stride,
                                                   const int64_t* __restrict__ labels, float inv_t, int vec_ok,
                                                   const float* __restrict__ row_lse,
                                                   const float* __restrict__ row_ez,
                                                   const float* __restrict__ g_logp,
                                                   const float* __restrict__ g_entropy, int64_t T_active,
                                                   typename OutPtr<ALIAS, void>::type dlogits) {
  const int64_t t = blockIdx.x;
  const void* row = row_ptr(logits, t, stride, Elem<DT>::kBytes);
  void* out = (void*)row_ptr(dlogits, t, stride, Elem<DT>::kBytes);
  const float gl = (t < T_active) ? g_logp[t] : 0.f;
  const float gh = (t < T_active && g_entropy) ? g_entropy[t] : 0.f;
  if (gl == 0.f && gh == 0.f) {
    row_zero_generic<DT, NT, STREAM>(row, out, V, vec_ok != 0);
    return;
  }
  const int64_t y = labels[t];
  GradCoef g;
  g.c = kLog2e * inv_t;
  g.lse2 = row_lse[t] * kLog2e;
  const float ez = (gh != 0.f) ? row_ez[t] : 0.f;
  g.A = inv_t * (gh * ez - gl);
  g.B = -gh * inv_t * inv_t;
  g.lab_add = gl * inv_t;
  g.label = (y >= 0 && y < V) ? (int)y : -1;
  row_grad_generic<DT, NT, STREAM>(row, out, V, vec_ok != 0, g);
}

// -----------------------------------------------------------------------------
// Per-token tail of the fused kernels: PPO surrogate from the row's log-prob,
// per-token outputs, and the coefficient of the gradient row.
// -----------------------------------------------------------------------------
struct FusedTokenArgs {
  const float* prox_logp;
  const float* adv;
  const uint8_t* mask_eff;
  const float* behave_w;
  const int32_t* n_valid;
  const float* grad_scale;
  float* logp;
  float* entropy;
  float* vmax;
  float* vmin;
  float* stat_loss;
  float* ratio;
  uint8_t* flags;
  aa_ppo_params P;
  int64_t T_active;
};

// Per-token inputs of the loss, fetched ahead of the row statistics so that
// their latency hides behind the streaming passes.  The loads are
// unconditional (index clamped into [0, T_active)) and nothing is converted
// here, so no wait is forced at the point of issue.  Needs T_active > 0.
struct TokenIn {
  float prox, adv, w;
  uint8_t mask_raw;
  bool active;
  __device__ __forceinline__ bool mask() const { return active && mask_raw != 0; }
};

__device__ __forceinline__ TokenIn load_token_in(const FusedTokenArgs& a, int64_t t) {
  TokenIn in;
  in.active = t < a.T_active;
  const int64_t tc = in.active ? t : a.T_active - 1;
  in.mask_raw = a.mask_eff[tc];
  in.prox = a.prox_logp[tc];
  in.adv = a.adv[tc];
  in.w = a.P.has_behave_weight ? a.behave_w[tc] : 1.f;
  return in;
}

// Same, for the persistent kernel: the arrays come in as separate read-only
// kernel arguments and every access is an aligned 32-bit load at a
// workgroup-uniform address, so that the values can travel through scalar
// loads into scalar registers instead of occupying vector registers for the
// length of a row.
// mask byte i of an array whose enclosing aligned words start at mask32 (the
// host passes the byte pointer rounded down to 4 bytes, and the remainder)
__device__ __forceinline__ uint32_t load_byte_uniform(const uint32_t* __restrict__ mask32, unsigned mis, int64_t i) {
  const int64_t j = i + mis;
  return (mask32[j >> 2] >> ((unsigned)(j & 3) * 8)) & 0xffu;
}

__device__ __forceinline__ TokenIn load_token_in_ro(const float* __restrict__ prox, const float* __restrict__ adv,
                                                    const uint32_t* __restrict__ mask32, unsigned mask_mis,
                                                    const float* __restrict__ bw, bool has_w, int64_t T_active,
                                                    int64_t t) {
  TokenIn in;
  in.active = t < T_active;
  const int64_t tc = in.active ? t : T_active - 1;
  in.mask_raw = (uint8_t)load_byte_uniform(mask32, mask_mis, tc);
  in.prox = prox[tc];
  in.adv = adv[tc];
  in.w = has_w ? bw[tc] : 1.f;
  return in;
}

// raw 16-bit pattern of element i of a row of 16-bit values (row 4-byte aligned)
__device__ __forceinline__ uint32_t load_u16_uniform(const void* __restrict__ row, int64_t i) {
  const uint32_t w = ((const uint32_t*)row)[i >> 1];
  return (i & 1) ? (w >> 16) : (w & 0xffffu);
}

// 1 / max(n_valid, 1) times the optional gradient scale: the factor between
// d(surrogate)/d(logp) and d(scaled loss)/d(logp).
__device__ __forceinline__ void load_loss_scale(const FusedTokenArgs& a, float& fn, float& gscale) {
  int n = *a.n_valid;
  if (a.P.loss_kind == AA_LOSS_NLL) {
    fn = (float)n + 1e-5f;  // the supervised loss divides by 1e-5 + count (areal/trainer/sft/lm_engine.py:96)
  } else {
    if (n < 1) n = 1;
    fn = (float)n;
  }
  gscale = a.grad_scale ? *a.grad_scale : 1.f;
}

// Returns g = d(scaled loss)/d(logp_t); writes the per-token outputs from one thread.
__device__ __forceinline__ float fused_token_tail(const FusedTokenArgs& a, int64_t t, const TokenIn& in, float fn,
                                                  float gscale, float lp, const RowStats& rs, const RowOut& ro,
                                                  bool writer) {
  if (writer) {
    a.logp[t] = lp;
    if (a.entropy) a.entropy[t] = ro.entropy;
    if (a.vmax) a.vmax[t] = rs.mx;
    if (a.vmin) a.vmin[t] = rs.mn;
  }
  if (!in.active) return 0.f;
  const bool m = in.mask();
  if (a.P.loss_kind == AA_LOSS_NLL) {  // loss = -logp of the label, d loss / d logp = -1 on the selected tokens
    if (writer) {
      a.stat_loss[t] = m ? -lp : 0.f;  // what the trainer logs per token: -where(mask, logp, 0)
      a.ratio[t] = 0.f;
      a.flags[t] = 0;
    }
    return m ? (-1.f / fn) * gscale : 0.f;
  }
  // the clipped surrogate sees a ratio of zero at masked tokens (functional.py:509); SAPO's ratio is not masked (:600)
  const bool sapo = a.P.loss_kind == AA_LOSS_SAPO;
  const float r = (m || sapo) ? expf(lp - in.prox) : 0.f;
  const Surrogate s = sapo ? sapo_surrogate(r, in.adv, a.P) : surrogate(r, in.adv, in.w, a.P);
  if (writer) {
    a.stat_loss[t] = s.loss;
    a.ratio[t] = r;
    a.flags[t] = (uint8_t)(((s.clip && m) ? 1 : 0) | ((s.dual && m) ? 2 : 0));
  }
  if (!m) return 0.f;
  return (s.dloss_dr * r / fn) * gscale;
}

constexpr int64_t kWalkRowBytes = 256 * 1024;  // rows at least this long are walked by kWalkGroups workgroups
constexpr int kWalkGroups = 512;               // two per compute unit

template <int DT, int NT, bool ALIAS>
__global__ __launch_bounds__(NT) void k_fused_generic(typename InPtr<ALIAS, void>::type logits, int64_t T_rows, int V,
                                                      int64_t stride, const int64_t* __restrict__ labels, float inv_t,
                                                      int vec_ok, FusedTokenArgs a,
                                                      typename OutPtr<ALIAS, void>::type dlogits) {
  __shared__ float smem[(NT / kWave) * 5];
  const float c = kLog2e * inv_t;
  float fn, gscale;
  load_loss_scale(a, fn, gscale);
  // one row per trip; with fewer workgroups than rows (T_rows > gridDim.x) a workgroup walks rows t, t + grid, ...
  for (int64_t t = blockIdx.x; t < T_rows; t += gridDim.x) {
    const void* row = row_ptr(logits, t, stride, Elem<DT>::kBytes);
    void* out = (void*)row_ptr(dlogits, t, stride, Elem<DT>::kBytes);
    const int64_t y = labels[t];
    const bool y_ok = (y >= 0) && (y < V);
    const float xy = y_ok ? Elem<DT>::load1(row, y) : 0.f;
    TokenIn tin{0.f, 0.f, 1.f, 0, false};
    if (a.T_active > 0) tin = load_token_in(a, t);
    const RowStats rs = row_stats_generic<DT, NT>(row, V, vec_ok != 0, c, smem);
    const RowOut ro = finish_row(rs);
    const float lp = y_ok ? label_logp(xy, c, rs, ro) : __builtin_nanf("");
    const float g = fused_token_tail(a, t, tin, fn, gscale, lp, rs, ro, threadIdx.x == 0);
    {
      if (g == 0.f) {
        row_zero_generic<DT, NT>(row, out, V, vec_ok != 0);
      } else {
        GradCoef gc;
        gc.c = c; gc.lse2 = ro.lse2; gc.A = -g * inv_t; gc.B = 0.f; gc.lab_add = g * inv_t;
        gc.label = y_ok ? (int)y : -1;
        row_grad_generic<DT, NT>(row, out, V, vec_ok != 0, gc);
      }
    }
    __syncthreads();  // the statistics scratch is reused by the next row
  }
}

// -----------------------------------------------------------------------------
// Fused kernel for fp32 logits, the row held on the chip between its one read and the one write of its gradient.
// One workgroup of 1024 threads per compute unit (its registers and the LDS belong to one row).  A row is cut into
// chunks of 8192 values, 8 per thread; the first chunks stay in registers, the next ones in LDS, and only what is
// left after those is read a second time for the gradient.  Two ways of holding a value:
//   exact (PACK = false, rows up to 114 688 values): 10 chunks in registers (80 VGPRs), 4 in LDS (128 KB);
//   24 bits (PACK = true, longer rows; a 608 KB row of V = 151 936 does not fit the 512 KB register file): the
//     statistics (log-prob, entropy, extrema) are taken from the fp32 values as they arrive, and what stays on the
//     chip is each value rounded to its upper 24 bits (sign, exponent, 15 bits of mantissa), four values in three
//     words: 13 chunks in registers (78 VGPRs), 6 in LDS (144 KB), 155 648 values.  The rounding moves x_j by at
//     most |x_j| 2^-16, so the probabilities behind the gradient row carry a relative error of at most
//     |x_j| / T * 2^-16 (2e-4 at |x_j| / T = 13): ten times finer than the bf16 rounding of a 16-bit gradient row,
//     cosine to the exact fp32 row 1 - 1e-9.
// A thread's eight values of a chunk are two pieces of four, 16 KB apart (values tid * 4 .. + 3 of each half of the
// chunk), so that every load and store instruction of a wave covers 1 KB of consecutive addresses (with the eight
// values side by side, every 128-byte line is touched by two instructions: 12 % slower).
// Loads run ahead of the arithmetic through buffer descriptors (no branch around a load; lanes past the end of the
// row read zeros and are left out of the statistics).  The chunks that go to LDS are taken first, while no register
// holds a chunk of the row yet: four chunks are in flight then, fewer as the registers fill, and at least the load
// of the next chunk is issued before the arithmetic of this one (twelve chunks in flight measured 7 % slower: the
// registers they need are spilled).  The first loads of the next row are issued right behind the stores of this
// one; loads and stores carry the `nt` policy.  Rows are handed out through the device counter (work) when there
// is one.  Needs V % 8 == 0, 16-byte aligned rows and rows below 2 GB.
// -----------------------------------------------------------------------------
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
constexpr int kBufferFlags = 0x00020000;  // raw buffer, 32-bit data format
constexpr int kAuxStream = 2;  // cache-policy bit 'nt': data is touched once, do not keep it in the caches
constexpr int kHoldChunk = 8 * 1024;  // values per chunk: 8 per thread
constexpr int kHoldChunkBytes = kHoldChunk * 4;
constexpr int kHoldStageRegs = 32;  // VGPRs for chunks in flight plus chunks held in registers, while that binds

template <bool PACK, int NREG, int NLDS>
struct HoldPlan {
  static constexpr int kReg = NREG;             // chunks in registers
  static constexpr int kLds = NLDS;             // chunks in LDS
  static constexpr int kWords = PACK ? 6 : 8;   // words per thread and chunk
  static constexpr int kChunks = kReg + kLds;
  static_assert(kReg * kWords <= 80 && kLds * kWords * 4096 <= 147456, "the row does not fit");
  // step i of a row handles this chunk
  __host__ __device__ static constexpr int chunk_of(int i) { return i < kLds ? kReg + i : i - kLds; }
  // number of chunks whose loads have been issued when step i begins
  __host__ __device__ static constexpr int issued_at(int i) {
    const int in_regs = i < kLds ? 0 : i - kLds;
    int room = (kHoldStageRegs - kWords * in_regs) / 8;
    if (room < 1) room = 1;
    const int n = i + room;
    return n < kChunks ? n : kChunks;
  }
};
constexpr int kHoldExactMaxV = 14 * kHoldChunk;  // 10 chunks in registers (80 VGPRs), 4 in LDS (128 KB)

// upper 24 bits of x, rounded half up in magnitude (bits 7..0 of the result are not part of the value)
__device__ __forceinline__ uint32_t round24(float x) { return __float_as_uint(x) + 0x80u; }

// Four values in kWords / 2 words.  PACK: words 0..2 keep values 0..2 in their upper three bytes; their low bytes
// hold bytes 1..3 of value 3.
template <bool PACK>
__device__ __forceinline__ void hold4(const float* x, uint32_t* w) {
  if constexpr (PACK) {
    const uint32_t r3 = round24(x[3]);
    w[0] = __builtin_amdgcn_perm(round24(x[0]), r3, 0x07060501u);
    w[1] = __builtin_amdgcn_perm(round24(x[1]), r3, 0x07060502u);
    w[2] = __builtin_amdgcn_perm(round24(x[2]), r3, 0x07060503u);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = __float_as_uint(x[i]);
  }
}

template <bool PACK>
__device__ __forceinline__ void held4(const uint32_t* w, float* x) {
  if constexpr (PACK) {
    x[0] = __uint_as_float(w[0] & 0xffffff00u);
    x[1] = __uint_as_float(w[1] & 0xffffff00u);
    x[2] = __uint_as_float(w[2] & 0xffffff00u);
    const uint32_t lo = __builtin_amdgcn_perm(w[1], w[0], 0x0c04000cu);    // [0, w0.b0, w1.b0, 0]
    x[3] = __uint_as_float(__builtin_amdgcn_perm(w[2], lo, 0x04020100u));  // [0, w0.b0, w1.b0, w2.b0]
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = __uint_as_float(w[i]);
  }
}

// statistics of N more values without a branch (the rescaling factor is 1 when the maximum stays)
template <int N>
__device__ __forceinline__ void stats_add_flat(ThreadStats& a, const float* x, float c) {
  const float m = max_of<N>(x), n = min_of<N>(x);
  const float k_new = fmaxf(a.k, m * c);
  const float d = a.k - k_new;
  const float f = fast_exp2(d);
  a.mx = __builtin_elementwise_maximum(a.mx, m);
  a.mn = __builtin_elementwise_minimum(a.mn, n);
  float s = 0.f, u = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float t = fmaf(x[i], c, -k_new);
    const float e = fast_exp2(t);
    s += e;
    u = fmaf(t, e, u);
  }
  a.u = fmaf(f, fmaf(d, a.s, a.u), u);
  a.s = fmaf(f, a.s, s);
  a.k = k_new;
}

struct Stage8 {
  u32x4_t lo, hi;
};

// SHIFTED: the 16 KB requests of a row (1024 threads x 16 bytes, two per chunk) are laid back by a shift of the
// row's own, as in k_fused_regs with SHIFT == 2 below: the descriptor of a row starts `sh` bytes before it, the first
// sh / 16 threads hold the last pieces of the row in their first slot of chunk 0, and a slot past the row's piece
// count is empty (the descriptor no longer drops its store: the thread skips it).
template <bool PACK, int NREG, int NLDS, bool SHIFTED = false>
__global__ __launch_bounds__(1024) void k_fused_f32_hold(const float* logits, int64_t T_rows, int V, int64_t stride,
                                                         const int64_t* __restrict__ labels, float inv_t,
                                                         FusedTokenArgs a, float* dlogits, int32_t* work) {
  typedef HoldPlan<PACK, NREG, NLDS> Plan;
  constexpr int kW = Plan::kWords, kH = kW / 2;
  constexpr int kHalf = kHoldChunk / 2;  // values per half chunk
  constexpr int kHalfBytes = kHoldChunkBytes / 2;
  __shared__ float smem[16 * 5];
  __shared__ uint2 held[(Plan::kLds > 0 ? Plan::kLds : 1) * kH * 1024];  // [chunk][word pair][thread]
  __shared__ int64_t next_row[2];  // written at the top of a row, read behind its barriers: two slots, no reuse race
  int slot = 0;
  const int tid = threadIdx.x;
  const int voff = tid * 16;
  const int tid4 = tid * 4;
  const float c = kLog2e * inv_t;
  float fn, gscale;
  load_loss_scale(a, fn, gscale);
  Stage8 sg[Plan::kChunks];
  int sh = 0;  // SHIFTED: the shift of the row in hand, in bytes (uniform)
  auto issue = [&](const __amdgpu_buffer_rsrc_t rsrc, int i) {
    const int off = Plan::chunk_of(i) * kHoldChunkBytes;
    if (SHIFTED && Plan::chunk_of(i) == 0)
      sg[i].lo = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff + (voff < sh ? V * 4 : 0), 0, kAuxStream);
    else
      sg[i].lo = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, off, kAuxStream);
    sg[i].hi = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, off + kHalfBytes, kAuxStream);
  };
  // The smallest shift that puts the requests of a row on a 1 KB boundary other than a 4 KB one, from the row's
  // place in the array as if the array started on a 4 KB boundary (results do not depend on where an array lies).
  auto row_shift = [&](int64_t row_index) -> int {
    if constexpr (!SHIFTED) return 0;
    else {
      const int off = (int)(((uint32_t)row_index * (uint32_t)((stride * 4) & 4095)) & 4095);
      const int a = off & 1023;
      return __builtin_amdgcn_readfirstlane((off >> 10) == 0 ? a + 1024 : a);
    }
  };
  auto row_rsrc = [&](const float* row, int shift) {
    return __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)row - shift), 0, V * 4 + shift, kBufferFlags);
  };

  int64_t t = blockIdx.x;  // the host launches at most T_rows workgroups
  sh = row_shift(t);
  __amdgpu_buffer_rsrc_t rsrc = row_rsrc(logits + t * stride, sh);
#pragma unroll
  for (int j = 0; j < Plan::issued_at(0); ++j) issue(rsrc, j);
  for (;;) {
    // claim the row after this one (through the device counter when there is one, so that compute units that get
    // through their rows faster take more of them); the answer is picked up behind the barriers of block_stats
    if (tid == 0) next_row[slot] = work ? (int64_t)atomicAdd(&work[0], 1) + gridDim.x : t + gridDim.x;
    const float* row = logits + t * stride;
    float* out = dlogits + t * stride;
    const int64_t y = labels[t];
    const bool y_ok = (y >= 0) && (y < V);
    const float xy = y_ok ? row[y] : 0.f;
    TokenIn tin{0.f, 0.f, 1.f, 0, false};
    if (a.T_active > 0) tin = load_token_in(a, t);

    // pass 1: statistics of the whole row from the fp32 values as they arrive; the row stays on the chip
    ThreadStats st{kNegBig, 0.f, 0.f, -FLT_MAX, FLT_MAX};
    uint32_t pr[Plan::kReg][kW];
#pragma unroll
    for (int i = 0; i < Plan::kChunks; ++i) {
#pragma unroll
      for (int j = Plan::issued_at(i); j < Plan::issued_at(i + 1); ++j) issue(rsrc, j);
      __builtin_amdgcn_sched_barrier(0);  // the loads stay where they are issued: no more of them in flight than planned
      float x[8];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        x[q] = __uint_as_float(sg[i].lo[q]);
        x[4 + q] = __uint_as_float(sg[i].hi[q]);
      }
      if (PACK && i >= Plan::kLds) {  // in the 24-bit form the register chunks lie inside every row that comes here
        stats_add_flat<8>(st, x, c);
      } else {  // the row may end in this chunk or before it: what lies past it read as zeros and is never stored
        const int left = V - Plan::chunk_of(i) * kHoldChunk;  // values of the row from this chunk on (same in all threads)
        if (tid4 < left) stats_add_flat<4>(st, x, c);
        if (tid4 < left - kHalf) stats_add_flat<4>(st, x + 4, c);
      }
      if (i < Plan::kLds) {
        uint32_t w[kW];
        hold4<PACK>(x, w);
        hold4<PACK>(x + 4, w + kH);
        // The LDS addresses are formed here, chunk by chunk, from a copy of the thread index that the compiler
        // cannot follow: computed once for all rows they end up spilled, and a reload from scratch in the middle
        // of a row waits for every load (here) or store (in pass 2) that is in flight.
        int ti = tid;
        asm volatile("" : "+v"(ti));
#pragma unroll
        for (int q = 0; q < kH; ++q) held[(i * kH + q) * 1024 + ti] = make_uint2(w[2 * q], w[2 * q + 1]);
      } else {
        uint32_t* w = pr[i - Plan::kLds];
        hold4<PACK>(x, w);
        hold4<PACK>(x + 4, w + kH);
        // the words are formed here (no instruction is emitted): left to the compiler, the rounding and packing move
        // down to the gradient pass and the registers hold the eight fp32 values until then
#pragma unroll
        for (int q = 0; q < kW; ++q) asm volatile("" : "+v"(w[q]));
      }
    }
    // what the chip does not hold (SHIFTED: the slots end sh bytes earlier in the row, and its last sh bytes are held)
    const int rest0 = Plan::kChunks * kHoldChunk - (sh >> 2), rest1 = V - (sh >> 2);
    for (int e0 = rest0 + tid * 8; e0 < rest1; e0 += kHoldChunk) {
      float x[8];
      load8<AA_F32>(row, e0, x);
      stats_add8(st, x, c);
    }
    const RowStats rs = block_stats<16>(st, smem);
    const int64_t tn = next_row[slot];
    slot ^= 1;
    const RowOut ro = finish_row(rs);
    const float lp = y_ok ? label_logp(xy, c, rs, ro) : __builtin_nanf("");
    const float g = fused_token_tail(a, t, tin, fn, gscale, lp, rs, ro, tid == 0);

    // pass 2: the gradient row (every thread reads back only what it stored itself: no barrier needed)
    const __amdgpu_buffer_rsrc_t wsrc = row_rsrc(out, sh);
    // the offsets of the stores are formed here, row by row: computed once for all rows they would occupy 38 registers
    int so = voff;
    asm volatile("" : "+v"(so));
    if (g == 0.f) {
      const u32x4_t z = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int k = 0; k < 2 * Plan::kChunks; ++k) {  // pieces past the row are dropped by the descriptor
        if constexpr (SHIFTED) {
          if (k == 0) __builtin_amdgcn_raw_buffer_store_b128(z, wsrc, so + (so < sh ? V * 4 : 0), 0, kAuxStream);
          else if (k * kHalf + tid4 < V) __builtin_amdgcn_raw_buffer_store_b128(z, wsrc, so + k * kHalfBytes, 0, kAuxStream);
        } else {
          __builtin_amdgcn_raw_buffer_store_b128(z, wsrc, so + k * kHalfBytes, 0, kAuxStream);
        }
      }
      const float z8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      for (int e0 = rest0 + tid * 8; e0 < rest1; e0 += kHoldChunk) store8<AA_F32>(out, e0, z8);
    } else {
      const float A = -g * inv_t, lab_add = g * inv_t, lse2 = ro.lse2;
      const int label = y_ok ? (int)y : -1;
      // SHIFTED: the label's place on the grid of slots
      int label_slot = label;
      if constexpr (SHIFTED) {
        if (label >= 0) {
          label_slot = label + (sh >> 2);
          if (label_slot >= V) label_slot -= V;
        }
      }
      // the thread's four values of the piece that starts at element `base` of the row and byte `off` of its storage
      // (the label's place is found from one per-thread value and numbers that are the same in all threads)
      auto emit4 = [&](int base, int off, const float* x) {
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = fast_exp2(fmaf(x[i], c, -lse2)) * A;
        const int d = (label_slot - base) - tid4;
        if ((unsigned)d < 4u) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (d == i) o[i] += lab_add;
        }
        const u32x4_t v = {__float_as_uint(o[0]), __float_as_uint(o[1]), __float_as_uint(o[2]), __float_as_uint(o[3])};
        if constexpr (SHIFTED) {
          if (base == 0) __builtin_amdgcn_raw_buffer_store_b128(v, wsrc, so + (so < sh ? V * 4 : 0), 0, kAuxStream);
          else if (base + tid4 < V) __builtin_amdgcn_raw_buffer_store_b128(v, wsrc, so + off, 0, kAuxStream);
        } else {
          __builtin_amdgcn_raw_buffer_store_b128(v, wsrc, so + off, 0, kAuxStream);
        }
      };
      auto emit = [&](int k, const uint32_t* w) {
        float x[8];
        held4<PACK>(w, x);
        held4<PACK>(w + kH, x + 4);
        emit4(k * kHoldChunk, k * kHoldChunkBytes, x);
        emit4(k * kHoldChunk + kHalf, k * kHoldChunkBytes + kHalfBytes, x + 4);
      };
#pragma unroll
      for (int k = 0; k < Plan::kReg; ++k) emit(k, pr[k]);
#pragma unroll
      for (int k = 0; k < Plan::kLds; ++k) {  // pieces past the row: the descriptor drops the store
        uint32_t w[kW];
        int ti = tid;
        asm volatile("" : "+v"(ti));
#pragma unroll
        for (int q = 0; q < kH; ++q) {
          const uint2 v = held[(k * kH + q) * 1024 + ti];
          w[2 * q] = v.x;
          w[2 * q + 1] = v.y;
        }
        emit(Plan::kReg + k, w);
      }
      for (int e0 = rest0 + tid * 8; e0 < rest1; e0 += kHoldChunk) {
        float x[8], o[8];
        load8<AA_F32>(row, e0, x);
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = fast_exp2(fmaf(x[i], c, -lse2)) * A;
        if ((unsigned)(label - e0) < 8u) {
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (e0 + i == label) o[i] += lab_add;
        }
        store8<AA_F32>(out, e0, o);
      }
    }
    t = tn;
    if (t >= T_rows) break;
    sh = row_shift(t);
    rsrc = row_rsrc(logits + t * stride, sh);
#pragma unroll
    for (int j = 0; j < Plan::issued_at(0); ++j) issue(rsrc, j);
  }
  if (work && tid == 0) {  // the last workgroup to finish leaves both words at zero for the next launch
    __threadfence();
    if (atomicAdd(&work[1], 1) == (int)gridDim.x - 1) {
      work[0] = 0;
      work[1] = 0;
      __threadfence();
    }
  }
}

// -----------------------------------------------------------------------------
// Fused kernel, register-resident row: 1024 threads hold one row of 16-bit
// logits as NCH 16-byte chunks per thread, so HBM sees exactly one read of the
// row and one write of its gradient.  Requires V % 8 == 0, 16-byte aligned
// rows and 8192 * (NCH - 1) < V <= 8192 * NCH, so that only the last chunk can
// be partly out of range (longer rows: the EXT variant below, which adds chunks
// held in LDS and chunks that are read twice).  Rows are addressed through buffer descriptors: one
// VGPR offset per thread, and the hardware drops out-of-range lanes (loads
// return 0, stores are ignored).  Loads take the chunk offset in the scalar
// offset operand.  Stores must NOT: with a register in the scalar-offset operand
// the compiler leaves out the wait states between a 16-byte buffer store and
// the next write of its data registers, and on gfx950 the store then picks up
// the overwritten value in some lanes.  The chunk offset of a store is added to
// the VGPR offset instead.
// -----------------------------------------------------------------------------
typedef short s16x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));

// Marks the packed row as modified (no instruction is emitted) so that the
// unpacked floats of one pass are not kept alive for the next: the row stays
// at 4 registers per chunk instead of 12.
template <int NCH>
__device__ __forceinline__ void keep_packed(u32x4_t (&d)[NCH]) {
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    uint32_t a = d[i][0], b = d[i][1], c = d[i][2], e = d[i][3];
    asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(e));
    d[i][0] = a; d[i][1] = b; d[i][2] = c; d[i][3] = e;
  }
}

// Gradient of one register-resident row, chunk by chunk:
//   out_j = -(g / T) p_j  (+ g / T at the label),  p_j = 2^(x_j c - lse2).
// The factor g / T is folded into the exponent, 2^(x_j c - lse2 + log2|g / T|),
// and its sign is applied in the conversion to 16 bits, so an element costs
// one fma and one exponential.
// Rows of whole chunks at a stride of whole chunks run 2-4 % below what they can when every 16 KB request of a
// workgroup starts on a 4 KB boundary; asked for 1, 2 or 3 KB off that grid they do not (measured on V = 90 112 ...
// 262 144 with the plain grid and the base of both arrays moved in steps of 128 bytes: multiples of 4 KB read
// 75.4-76.4 % of the HBM peak, the other multiples of 1 KB 77.6-77.7 %, anything else 75-76.3 %; worst at strides of
// whole 32 KB, where some layouts of the arrays lose 4 % more).  SHIFT instantiations therefore lay the chunk grid of a row
// kShiftPieces 16-byte pieces back: slot (chunk c, thread) holds piece c * 1024 + thread - kShiftPieces, and the first
// kShiftPieces threads of chunk 0, whose piece would lie before the row, hold its last kShiftPieces pieces instead
// (rows of whole chunks only, so every slot holds a piece).  Only chunk 0, which is always in registers, needs an
// offset of its own per thread (voff_first); a label's slot moves with the grid (shifted_piece).
constexpr int kShiftPieces = 64;
constexpr int kShiftBytes = kShiftPieces * 16;
__device__ __forceinline__ int shifted_piece(int piece, int row_pieces) {
  if (piece < 0) return -1;
  const int q = piece + kShiftPieces;
  return q < row_pieces ? q : q - row_pieces;
}

// SHIFT == 2 (rows that are not whole chunks, or not a whole number of chunks apart): the same idea with a shift of
// the row's own, `sh` bytes (a multiple of 16, below 16 KB), chosen so that the 16 KB requests of the row start
// kShiftTargetBytes past a 16 KB boundary of the address space.  The buffer descriptor of the row starts `sh` bytes
// before the row, so slot (chunk c, thread) is asked for at c * 16 KB + thread * 16 as in the plain grid and holds
// piece c * 1024 + thread - sh / 16; the threads of chunk 0 below sh / 16, whose piece would lie before the row, hold
// its last pieces, which the plain grid's slots at and past the row's piece count would have held: those slots stay
// empty (the same test as in the plain grid), but the descriptor no longer drops what they would store, so the last
// chunk's store is skipped by the threads without a piece (longer rows: the store of every chunk in LDS or in the
// tail is).
constexpr int kShiftTargetBytes = 1024;
__device__ __forceinline__ int shifted_piece_by(int piece, int shift_pieces, int row_pieces) {
  if (piece < 0) return -1;
  const int q = piece + shift_pieces;
  return q < row_pieces ? q : q - row_pieces;
}

// SHIFT == 3 (rows that start at any even address: V or the stride not a multiple of 8 values, or arrays that do not
// start on a 16-byte boundary): the grid of SHIFT == 2 laid over the 16-byte pieces of memory that hold the row.  The
// first of them may hold values of the row before (`head` values), the last one values of the row after; both are
// pieces of chunk 0 (the grid is always laid back by at least one piece: the last piece goes to the thread before the
// one that holds the first).  What does not belong to the row is replaced by a value of the row when the piece
// arrives (the extrema keep, the sums are corrected by the thread), and these two threads store their values of the
// gradient one by one.
struct RowEdge {
  int lo, hi;  // this thread's piece of chunk 0 holds values lo .. hi - 1 of the row's (0, 8 for every thread but two)
};
__device__ __forceinline__ uint32_t patch_edge(u32x4_t& v, RowEdge e) {
  const uint32_t fill = e.lo > 0 ? (v[3] >> 16) : (v[0] & 0xffffu);
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    uint32_t w = v[q];
    if (2 * q < e.lo || 2 * q >= e.hi) w = (w & 0xffff0000u) | fill;
    if (2 * q + 1 < e.lo || 2 * q + 1 >= e.hi) w = (w & 0xffffu) | (fill << 16);
    v[q] = w;
  }
  return fill;
}
__device__ __forceinline__ void store_edge(u32x4_t r, __amdgpu_buffer_rsrc_t wsrc, int off, RowEdge e) {
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const uint32_t w = r[q >> 1];
    if (q >= e.lo && q < e.hi)
      __builtin_amdgcn_raw_buffer_store_b16((short)((q & 1) ? (w >> 16) : (w & 0xffffu)), wsrc, off + 2 * q, 0, kAuxStream);
  }
}

template <int DT, int NCH, bool G_POSITIVE, int SHIFT = 0>
__device__ __forceinline__ void grad_pass(const u32x4_t (&d)[NCH], float g, float inv_t, float c, float lse2,
                                          int64_t y, int tid, int voff, __amdgpu_buffer_rsrc_t wsrc, int voff_first = 0,
                                          int row_pieces = 0, int sh = 0, bool last_ok = true, int head = 0,
                                          RowEdge edge = RowEdge{0, 8}) {
  constexpr int NT = 1024;
  constexpr int kChunkBytes = NT * 16;
  const float lab_add = g * inv_t;
  const float kk = fast_log2(fabsf(lab_add)) - lse2;
  int yv = y >= 0 ? (int)((y + head) >> 3) : -1;
  if constexpr (SHIFT == 1) yv = shifted_piece(yv, row_pieces);
  if constexpr (SHIFT == 2 || SHIFT == 3) yv = shifted_piece_by(yv, sh >> 4, row_pieces);
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float o[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float e0 = fast_exp2(fmaf(Elem<DT>::lo(d[i][q]), c, kk));
      const float e1 = fast_exp2(fmaf(Elem<DT>::hi(d[i][q]), c, kk));
      o[2 * q] = G_POSITIVE ? -e0 : e0;
      o[2 * q + 1] = G_POSITIVE ? -e1 : e1;
    }
    if (yv - i * NT == tid) {  // uniform left side: no per-chunk index registers
      const int e = (int)((y + head) & 7);
#pragma unroll
      for (int q = 0; q < 8; ++q)
        if (q == e) o[q] += lab_add;
    }
    u32x4_t r;
    r[0] = Elem<DT>::pack(o[0], o[1]);
    r[1] = Elem<DT>::pack(o[2], o[3]);
    r[2] = Elem<DT>::pack(o[4], o[5]);
    r[3] = Elem<DT>::pack(o[6], o[7]);
    if constexpr (SHIFT == 2 || SHIFT == 3) {
      if (i == 0) {
        const int off = voff + (voff < sh ? row_pieces * 16 : 0);
        if (SHIFT == 3 && edge.hi - edge.lo != 8) store_edge(r, wsrc, off, edge);
        else __builtin_amdgcn_raw_buffer_store_b128(r, wsrc, off, 0, kAuxStream);
      } else if (i < NCH - 1 || last_ok)
        __builtin_amdgcn_raw_buffer_store_b128(r, wsrc, voff + i * kChunkBytes, 0, kAuxStream);
    } else if (SHIFT == 1 && i == 0) {
      __builtin_amdgcn_raw_buffer_store_b128(r, wsrc, voff_first, 0, kAuxStream);
    } else {
      __builtin_amdgcn_raw_buffer_store_b128(r, wsrc, voff + i * kChunkBytes - (SHIFT == 1 ? kShiftBytes : 0), 0, kAuxStream);
    }
  }
}

// ---- rows longer than the register file --------------------------------------
// The extended variant of k_fused_regs (EXT) keeps kExtRegChunks chunks of the row in registers, up to
// kExtLdsChunks more in LDS (brought in by direct-to-LDS loads, each thread reads back only the 16 bytes its own
// lane deposited) and reads up to kExtTailChunks last chunks twice: for the statistics (both passes use the one
// fetch, left in the cache) and for the gradient.  These helpers are the
// per-chunk bodies of the three passes for a chunk that is not in registers.
typedef __attribute__((address_space(3))) void* lds_ptr_t;
constexpr int kExtRegChunks = 21;
constexpr int kExtLdsChunks = 9;
constexpr int kExtTailChunks = 2;

struct MinMax16 {
  s16x2_t smax, smin;
  u16x2_t umax, umin;
};

__device__ __forceinline__ void minmax_chunk(MinMax16& m, const u32x4_t v) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const uint32_t w = v[q];
    const s16x2_t ws = __builtin_bit_cast(s16x2_t, w);
    const u16x2_t wu = __builtin_bit_cast(u16x2_t, w);
    m.smax = __builtin_elementwise_max(m.smax, ws);
    m.smin = __builtin_elementwise_min(m.smin, ws);
    m.umax = __builtin_elementwise_max(m.umax, wu);
    m.umin = __builtin_elementwise_min(m.umin, wu);
  }
}

template <int DT>
__device__ __forceinline__ void sum_chunk(const u32x4_t v, float c, float k, float& s, float& u) {
  float cs = 0.f, cu = 0.f;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float lo = Elem<DT>::lo(v[q]), hi = Elem<DT>::hi(v[q]);
    const float t0 = fmaf(lo, c, -k), t1 = fmaf(hi, c, -k);
    const float e0 = fast_exp2(t0), e1 = fast_exp2(t1);
    cs += e0 + e1;
    cu = fmaf(t0, e0, cu);
    cu = fmaf(t1, e1, cu);
  }
  s += cs;
  u += cu;
}

// gradient of chunk `ci` (any chunk index), as grad_pass does it for the register chunks
template <int DT>
__device__ __forceinline__ u32x4_t grad_chunk(const u32x4_t v, float c, float kk, float lab_add, bool g_positive,
                                              int yv, int y_elem, int ci, int tid) {
  float o[8];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float e0 = fast_exp2(fmaf(Elem<DT>::lo(v[q]), c, kk));
    const float e1 = fast_exp2(fmaf(Elem<DT>::hi(v[q]), c, kk));
    o[2 * q] = g_positive ? -e0 : e0;
    o[2 * q + 1] = g_positive ? -e1 : e1;
  }
  if (yv - ci * 1024 == tid) {
#pragma unroll
    for (int q = 0; q < 8; ++q)
      if (q == y_elem) o[q] += lab_add;
  }
  u32x4_t r;
  r[0] = Elem<DT>::pack(o[0], o[1]);
  r[1] = Elem<DT>::pack(o[2], o[3]);
  r[2] = Elem<DT>::pack(o[4], o[5]);
  r[3] = Elem<DT>::pack(o[6], o[7]);
  return r;
}

// Rows of up to two chunks go to the two-pass kernel instead: 256 threads per row and eight rows per compute unit
// hide the per-row latency better than one or two 1024-thread workgroups, and the second read of a 32 KB row comes
// from the cache (V = 8192: 3.8 against 2.6 TB/s, V = 16 384: 4.7 against 4.2; from three chunks on this kernel wins).
constexpr int64_t kTwoPassMaxV = 16 * 1024;
constexpr int kTwoPerUnitChunks = 7;  // rows this short run two workgroups per compute unit

// Rows are handed out through a device counter (work[0]) so that compute
// units that get through their rows faster take more of them; work[1] counts
// finished workgroups, and the last one puts both words back to zero, which is
// the state the next launch expects.  With work == nullptr the rows are dealt
// round-robin (t, t + gridDim.x, ...).
// With EXT the row continues past the NCH register chunks: n_lds chunks in dynamic LDS, then the tail chunks.
// Up to kTwoPerUnitChunks chunks the kernel is compiled for 8 waves per SIMD, so that two workgroups fit on a
// compute unit: without that request the scalar registers alone (106 per wave: 7 waves) keep the second one out.
// SHIFT (see grad_pass): 1: the chunk grid of a row laid 1 KB back, for rows of whole chunks a whole number of chunks
// apart; 2: laid back by an amount of the row's own; 3: the same over the 16-byte pieces of memory that hold a row which
// starts at any even address (stride_vec is then the stride in values, and NCH counts the chunks of those pieces).
template <int DT, int NCH, bool EXT, bool ALIAS, int SHIFT = 0>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu((!EXT && NCH <= kTwoPerUnitChunks) ? 8 : 1)))
void k_fused_regs(typename InPtr<ALIAS, uint4>::type logits, int V, int64_t stride_vec,
                                                     const int64_t* __restrict__ labels, float inv_t,
                                                     const float* __restrict__ in_prox,
                                                     const float* __restrict__ in_adv,
                                                     const uint32_t* __restrict__ in_mask32, unsigned mask_mis,
                                                     const float* __restrict__ in_bw, FusedTokenArgs a,
                                                     typename OutPtr<ALIAS, uint4>::type dlogits, int64_t T, int32_t* work,
                                                     int n_lds) {
  constexpr int NT = 1024;
  constexpr int kChunkBytes = NT * 16;
  const bool has_w = a.P.has_behave_weight != 0;
  extern __shared__ __align__(16) unsigned char ext_lds[];  // EXT: n_lds chunks of 16 KiB
  __shared__ float smem[(NT / kWave) * 5];
  __shared__ int64_t next_row[2];  // written at the top of a row, read behind its barriers: two slots, no reuse race
  int slot = 0;
  constexpr bool kRowShift = SHIFT == 2 || SHIFT == 3;
  int nvec = V >> 3;  // 16-byte pieces of a row (SHIFT == 3: of the memory that holds it, set row by row)
  const int tid = threadIdx.x;
  const float c = kLog2e * inv_t;
  const int voff = tid * 16;
  constexpr int kSh = SHIFT == 1 ? kShiftBytes : 0;  // chunks 1, 2, ... are asked for this many bytes before their place
  // SHIFT: this thread's byte offset in chunk 0 (the last pieces of the row for the first kShiftPieces threads)
  const int voff_first = tid < kShiftPieces ? voff + (nvec - kShiftPieces) * 16 : voff - kShiftBytes;
  // EXT: every register chunk is full; SHIFT: the row is whole chunks (the comparison stays, so that the passes over
  // the row keep the schedule of the other instantiations)
  bool last_ok = EXT || (NCH - 1) * NT + (SHIFT == 1 ? (tid & 1) : tid) < nvec;
  // SHIFT == 2: the shift of a row in bytes (uniform), and the descriptor of a row that starts that far before it
  // It is taken from where the row starts inside the array (row index x stride), as if the array started on a 4 KB
  // boundary, which large allocations do: results then do not depend on where an array lies.  The smallest shift that
  // puts the requests on a 1 KB boundary other than a 4 KB one.
  auto row_shift = [&](int64_t row_index) -> int {
    if constexpr (SHIFT != 2) return 0;
    else {
      const int off = (int)(((uint32_t)row_index * (uint32_t)((stride_vec * 16) & 4095)) & 4095);
      const int a = off & 1023;
      return __builtin_amdgcn_readfirstlane((off >> 10) == 0 ? a + 1024 : a);
    }
  };
  // SHIFT == 3: stride_vec is the stride in values; a row starts `head` values into its first piece.  The place of a
  // row is taken from its index and from where the arrays start inside a 16-byte piece (both arrays the same).
  int head = 0;
  RowEdge edge{0, 8};
  const uint32_t base_mis = SHIFT == 3 ? (uint32_t)((uintptr_t)logits & 15) : 0u;
  auto set_row = [&](int64_t row_index) -> int {  // returns the shift in bytes (a multiple of 16); sets head, nvec, ...
    if constexpr (SHIFT != 3) return row_shift(row_index);
    else {
      const uint32_t off = ((uint32_t)row_index * (uint32_t)((stride_vec * 2) & 4095) + base_mis) & 4095u;
      const int h = (int)(off & 15u), off16 = (int)(off & ~15u);
      const int a = off16 & 1023, k = off16 >> 10;
      int s16 = k == 0 ? a + 1024 : a;
      if (s16 == 0) s16 = k == 1 ? 2048 : 1024;
      s16 = __builtin_amdgcn_readfirstlane(s16);
      head = __builtin_amdgcn_readfirstlane(h >> 1);
      nvec = __builtin_amdgcn_readfirstlane((h + V * 2 + 15) >> 4);
      last_ok = EXT || (NCH - 1) * NT + tid < nvec;
      const int p0 = s16 >> 4;
      edge.lo = tid == p0 ? head : 0;
      edge.hi = tid == p0 - 1 ? ((h + V * 2 - (nvec - 1) * 16) >> 1) : 8;
      return s16;
    }
  };
  auto row_in = [&](int64_t row_index) -> const char* {
    return (const char*)logits + row_index * stride_vec * (SHIFT == 3 ? 2 : 16);
  };
  auto row_out = [&](int64_t row_index) -> const char* {
    return (const char*)dlogits + row_index * stride_vec * (SHIFT == 3 ? 2 : 16);
  };
  // the descriptor of a row on a grid laid back by sh bytes (SHIFT == 3: and by the row's place in its first piece; it
  // ends with the last piece that holds values of the row)
  auto row_rsrc = [&](const void* row, int sh) {
    if constexpr (SHIFT == 3)
      return __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)row - sh - head * 2), 0, sh + nvec * 16, kBufferFlags);
    else
      return __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)row - sh), 0, V * 2 + sh, kBufferFlags);
  };
  auto label_bits = [&](const void* row, int64_t i) -> uint32_t {
    if constexpr (SHIFT == 3) return ((const uint16_t*)row)[i];
    else return load_u16_uniform(row, i);
  };
  float fn, gscale;
  load_loss_scale(a, fn, gscale);
  // EXT: chunk NCH + j goes to LDS for j < n_lds; each wave deposits its 1 KiB piece, lane by lane
  const u32x4_t* my_lds = (const u32x4_t*)ext_lds + tid;
  const int lds_wave_off = (tid >> 6) * 1024;
  const int tail0 = NCH + n_lds;  // first chunk that is neither in registers nor in LDS
  auto load_lds_chunks = [&](const __amdgpu_buffer_rsrc_t rsrc) {
    for (int j = 0; j < n_lds; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)(ext_lds + j * kChunkBytes + lds_wave_off), 16, voff,
                                               (NCH + j) * kChunkBytes - kSh, 0, kAuxStream);
  };
  // load of register chunk i (a compile-time slot)
  auto load_reg = [&](const __amdgpu_buffer_rsrc_t rsrc, int i, int sh) {
    if (kRowShift && i == 0)
      return __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff + (voff < sh ? nvec * 16 : 0), 0, kAuxStream);
    if (SHIFT == 1 && i == 0) return __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff_first, 0, kAuxStream);
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, i * kChunkBytes - kSh, kAuxStream);
  };

  int64_t t = blockIdx.x;  // the host launches at most T workgroups
  const char* src = row_in(t);
  u32x4_t d[NCH];
  int sh = set_row(t);
  {
    const __amdgpu_buffer_rsrc_t rsrc = row_rsrc(src, sh);
#pragma unroll
    for (int i = 0; i < NCH; ++i) d[i] = load_reg(rsrc, i, sh);
    if constexpr (EXT) load_lds_chunks(rsrc);
  }
  int64_t y = labels[t];
  bool y_ok = (y >= 0) && (y < V);
  uint32_t xy_raw = label_bits(src, y_ok ? y : 0);
  TokenIn tin = load_token_in_ro(in_prox, in_adv, in_mask32, mask_mis, in_bw, has_w, a.T_active, t);

  for (;;) {
    // claim the row after this one; the answer is picked up behind the barriers of block_stats
    if (tid == 0) next_row[slot] = work ? (int64_t)atomicAdd(&work[0], 1) + gridDim.x : t + gridDim.x;

    // pass 1 over registers: thread maximum / minimum, taken on the raw 16-bit
    // patterns with packed integer min/max (two elements per instruction, no
    // unpacking).  For sign-magnitude floats: if any value is non-negative the
    // largest signed pattern is the maximum, otherwise the smallest signed
    // pattern is; if any value is negative the largest unsigned pattern is the
    // minimum, otherwise the smallest unsigned pattern is.
    s16x2_t smax = {-32768, -32768}, smin = {32767, 32767};
    u16x2_t umax = {0, 0}, umin = {65535, 65535};
    // SHIFT == 3: what the first and the last piece hold of other rows is replaced by a value of this row
    uint32_t edge_fill = 0;
    if constexpr (SHIFT == 3) {
      if (edge.hi - edge.lo != 8) edge_fill = patch_edge(d[0], edge);
    }
    // EXT: the tail chunks of this row, fetched here for the statistics and once more for the gradient (lanes past
    // the row read zeros)
    __amdgpu_buffer_rsrc_t rsrc_t;
    u32x4_t tv[kExtTailChunks];
    bool tail_ok[kExtTailChunks];
    if constexpr (EXT) {
      rsrc_t = row_rsrc((const void*)row_in(t), sh);
#pragma unroll
      for (int q = 0; q < kExtTailChunks; ++q) {
        tv[q] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_t, voff, (tail0 + q) * kChunkBytes - kSh, 0);  // stays cached for the second read
        tail_ok[q] = (tail0 + q) * NT + tid < nvec;
      }
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (i < NCH - 1 || last_ok) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t w = d[i][q];  // a scalar copy: bit_cast of a vector element expression reads element 0
          const s16x2_t ws = __builtin_bit_cast(s16x2_t, w);
          const u16x2_t wu = __builtin_bit_cast(u16x2_t, w);
          smax = __builtin_elementwise_max(smax, ws);
          smin = __builtin_elementwise_min(smin, ws);
          umax = __builtin_elementwise_max(umax, wu);
          umin = __builtin_elementwise_min(umin, wu);
        }
      }
    }
    if constexpr (EXT) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the direct-to-LDS loads of this row have landed
      MinMax16 m{smax, smin, umax, umin};
      for (int j = 0; j < n_lds; ++j)
        if ((NCH + j) * NT + tid < nvec) minmax_chunk(m, my_lds[j * NT]);
#pragma unroll
      for (int q = 0; q < kExtTailChunks; ++q)
        if (tail_ok[q]) minmax_chunk(m, tv[q]);
      smax = m.smax; smin = m.smin; umax = m.umax; umin = m.umin;
    }
    const int hi_s = smax[0] > smax[1] ? smax[0] : smax[1];
    const int lo_s = smin[0] < smin[1] ? smin[0] : smin[1];
    const unsigned hi_u = umax[0] > umax[1] ? umax[0] : umax[1];
    const unsigned lo_u = umin[0] < umin[1] ? umin[0] : umin[1];
    const float mx = Elem<DT>::lo((uint32_t)((hi_s >= 0 ? hi_s : lo_s) & 0xffff));
    const float mn = Elem<DT>::lo(lo_s < 0 ? hi_u : lo_u);
    keep_packed(d);
    // one maximum per wave keeps the second pass free of rescaling
    ThreadStats ts;
    ts.k = fmaxf(wave_max(mx) * c, kNegBig);
    ts.mx = mx; ts.mn = mn;
    float s = 0.f, u = 0.f;
    if constexpr (EXT) {  // the tail chunks first: they are still in the registers pass 1 read them into
#pragma unroll
      for (int q = 0; q < kExtTailChunks; ++q)
        if (tail_ok[q]) sum_chunk<DT>(tv[q], c, ts.k, s, u);
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      float cs = 0.f, cu = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float lo = Elem<DT>::lo(d[i][q]), hi = Elem<DT>::hi(d[i][q]);
        const float t0 = fmaf(lo, c, -ts.k), t1 = fmaf(hi, c, -ts.k);
        const float e0 = fast_exp2(t0), e1 = fast_exp2(t1);
        cs += e0 + e1;
        cu = fmaf(t0, e0, cu);
        cu = fmaf(t1, e1, cu);
      }
      if (i == NCH - 1 && !last_ok) { cs = 0.f; cu = 0.f; }
      s += cs;
      u += cu;
    }
    if constexpr (EXT) {
      for (int j = 0; j < n_lds; ++j)
        if ((NCH + j) * NT + tid < nvec) sum_chunk<DT>(my_lds[j * NT], c, ts.k, s, u);
    }
    if constexpr (SHIFT == 3) {  // the values that stand in for other rows' leave the sums again
      if (edge.hi - edge.lo != 8) {
        const float m = (float)(8 - (edge.hi - edge.lo));
        const float t0 = fmaf(Elem<DT>::lo(edge_fill), c, -ts.k);
        const float e0 = fast_exp2(t0);
        s = fmaf(-m, e0, s);
        u = fmaf(-m, t0 * e0, u);
      }
    }
    ts.s = s; ts.u = u;
    keep_packed(d);
    const RowStats rs = block_stats<NT / kWave>(ts, smem);
    const int64_t tn = next_row[slot];
    slot ^= 1;
    const RowOut ro = finish_row(rs);
    const float xy = Elem<DT>::lo(xy_raw);
    const float lp = y_ok ? label_logp(xy, c, rs, ro) : __builtin_nanf("");
    const float g = fused_token_tail(a, t, tin, fn, gscale, lp, rs, ro, tid == 0);

    // scalars of the next row, fetched ahead of the gradient pass
    const bool more = tn < T;
    const char* src_n = row_in(more ? tn : t);
    const int64_t y_n = more ? labels[tn] : -1;
    const bool y_ok_n = (y_n >= 0) && (y_n < V);
    const uint32_t xy_raw_n = label_bits(src_n, y_ok_n ? y_n : 0);
    const TokenIn tin_n = load_token_in_ro(in_prox, in_adv, in_mask32, mask_mis, in_bw, has_w, a.T_active, more ? tn : t);

    const __amdgpu_buffer_rsrc_t wsrc = row_rsrc((const void*)row_out(t), sh);
    if constexpr (EXT) {
      if (g != 0.f) {
#pragma unroll
        for (int q = 0; q < kExtTailChunks; ++q)
          tv[q] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_t, voff, (tail0 + q) * kChunkBytes - kSh, kAuxStream);
      }
    }
    if (g == 0.f) {
      const u32x4_t z = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        if constexpr (kRowShift) {
          if (i == 0) {
            const int off = voff + (voff < sh ? nvec * 16 : 0);
            if (SHIFT == 3 && edge.hi - edge.lo != 8) store_edge(z, wsrc, off, edge);
            else __builtin_amdgcn_raw_buffer_store_b128(z, wsrc, off, 0, kAuxStream);
          } else if (i < NCH - 1 || last_ok)
            __builtin_amdgcn_raw_buffer_store_b128(z, wsrc, voff + i * kChunkBytes, 0, kAuxStream);
        } else {
          __builtin_amdgcn_raw_buffer_store_b128(z, wsrc, (SHIFT == 1 && i == 0) ? voff_first : voff + i * kChunkBytes - kSh,
                                                 0, kAuxStream);
        }
      }
      if constexpr (EXT) {
        // chunks past the row are dropped by the descriptor (SHIFT == 1: the first of them would reach back into the
        // row; a shift per row: the descriptor ends behind the pieces that chunk 0 holds, so threads without a piece skip)
        for (int j = 0; j < n_lds + kExtTailChunks && !(SHIFT == 1 && (NCH + j) * NT >= nvec); ++j)
          if (!kRowShift || (NCH + j) * NT + tid < nvec)
            __builtin_amdgcn_raw_buffer_store_b128(z, wsrc, voff + (NCH + j) * kChunkBytes - kSh, 0, kAuxStream);
      }
    } else if (g > 0.f) {
      grad_pass<DT, NCH, true, SHIFT>(d, g, inv_t, c, ro.lse2, y_ok ? y : -1, tid, voff, wsrc, voff_first, nvec, sh, last_ok, head, edge);
    } else {
      grad_pass<DT, NCH, false, SHIFT>(d, g, inv_t, c, ro.lse2, y_ok ? y : -1, tid, voff, wsrc, voff_first, nvec, sh, last_ok, head, edge);
    }
    if constexpr (EXT) {
      if (g != 0.f) {
        const float lab_add = g * inv_t;
        const float kk = fast_log2(fabsf(lab_add)) - ro.lse2;
        const int yv_row = y_ok ? (int)((y + head) >> 3) : -1;
        const int yv = SHIFT == 1 ? shifted_piece(yv_row, nvec) : kRowShift ? shifted_piece_by(yv_row, sh >> 4, nvec) : yv_row;
        const int y_elem = (int)((y + head) & 7);
        for (int j = 0; j < n_lds; ++j) {
          const u32x4_t r = grad_chunk<DT>(my_lds[j * NT], c, kk, lab_add, g > 0.f, yv, y_elem, NCH + j, tid);
          if (!kRowShift || (NCH + j) * NT + tid < nvec)
            __builtin_amdgcn_raw_buffer_store_b128(r, wsrc, voff + (NCH + j) * kChunkBytes - kSh, 0, kAuxStream);
        }
#pragma unroll
        for (int q = 0; q < kExtTailChunks; ++q) {
          // SHIFT: a chunk past the row would reach back into it (the descriptor drops it otherwise)
          if (SHIFT == 1 && (tail0 + q) * NT >= nvec) continue;
          const u32x4_t r = grad_chunk<DT>(tv[q], c, kk, lab_add, g > 0.f, yv, y_elem, tail0 + q, tid);
          if (!kRowShift || tail_ok[q])
            __builtin_amdgcn_raw_buffer_store_b128(r, wsrc, voff + (tail0 + q) * kChunkBytes - kSh, 0, kAuxStream);
        }
      }
    }
    if (!more) break;
    // All stores of this row are issued before the loads of the next one:
    // alternating them chunk by chunk costs bandwidth on this memory system.
    {
      sh = set_row(more ? tn : t);
      const __amdgpu_buffer_rsrc_t rsrc_n = row_rsrc(src_n, sh);
#pragma unroll
      for (int i = 0; i < NCH; ++i) d[i] = load_reg(rsrc_n, i, sh);
      if constexpr (EXT) {
        asm volatile("" ::: "memory");  // the LDS reads of the gradient pass stay ahead of the next row's deposits
        load_lds_chunks(rsrc_n);
      }
    }
    t = tn; y = y_n; y_ok = y_ok_n; xy_raw = xy_raw_n; tin = tin_n;
  }
  if (work && tid == 0) {
    __threadfence();
    if (atomicAdd(&work[1], 1) == (int)gridDim.x - 1) {
      work[0] = 0;
      work[1] = 0;
      __threadfence();
    }
  }
}

// -----------------------------------------------------------------------------
// One GPU's share of the vocabulary-parallel log-prob op (areal/utils/functional/vocab_parallel.py:84-372): every
// shard runs the streaming forward pass on its [T, V / tp] slice and ends with three numbers per row: its own
// logsumexp, its own sum_j softmax_j z_j, and the label's log-prob where the label lies in the shard (NaN where
// not).  This kernel is the reduction the ranks would do with one exchange of those numbers: the global
// logsumexp, sum p z, log-prob and entropy.  Fixed order over the shards.
// -----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_vocab_partials_combine(const float* __restrict__ lse,
                                                                const float* __restrict__ ez,
                                                                const float* __restrict__ logp_local, int S,
                                                                int64_t T, float* __restrict__ logp,
                                                                float* __restrict__ entropy,
                                                                float* __restrict__ lse_out,
                                                                float* __restrict__ ez_out) {
  for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < T; t += (int64_t)gridDim.x * 256) {
    float m = -__builtin_inff();
    for (int i = 0; i < S; ++i) m = fmaxf(m, lse[i * T + t]);
    float sum = 0.f;
    for (int i = 0; i < S; ++i) sum += expf(lse[i * T + t] - m);
    const float L = m + logf(sum);
    float e = 0.f, lp = __builtin_nanf("");
    for (int i = 0; i < S; ++i) {
      const float li = lse[i * T + t];
      e = fmaf(expf(li - L), ez[i * T + t], e);
      const float q = logp_local[i * T + t];
      if (q == q) lp = q + li - L;  // the shard that holds the label: z_label = logp_local + lse_i
    }
    logp[t] = lp;
    if (entropy) entropy[t] = L - e;
    if (lse_out) lse_out[t] = L;
    if (ez_out) ez_out[t] = e;
  }
}

// -----------------------------------------------------------------------------
// Plain copy (calibration of the HBM counters) and in-place scaling.
// -----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_copy16(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n) {
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) dst[i] = src[i];
}

template <int DT>
__global__ __launch_bounds__(256) void k_scale(void* __restrict__ data, int64_t n, const float* __restrict__ factor) {
  const float f = *factor;
  if (f == 1.0f) return;
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step)
    Elem<DT>::store1(data, i, Elem<DT>::load1(data, i) * f);
}

// rows of V elements that start `stride` elements apart: the elements between the rows are left alone
template <int DT>
__global__ __launch_bounds__(256) void k_scale_rows(void* __restrict__ data, int64_t T, int64_t V, int64_t stride,
                                                    const float* __restrict__ factor) {
  const float f = *factor;
  if (f == 1.0f) return;
  const int64_t n = T * V, step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const int64_t at = (i / V) * stride + i % V;
    Elem<DT>::store1(data, at, Elem<DT>::load1(data, at) * f);
  }
}

// -----------------------------------------------------------------------------
// Host-side dispatch
// -----------------------------------------------------------------------------
static bool common_args_ok(const void* logits, int dtype, int64_t T, int64_t V, int64_t stride,
                           const int64_t* labels) {
  if (!logits || !labels) return false;
  if (dtype != AA_BF16 && dtype != AA_F16 && dtype != AA_F32) return false;
  if (T <= 0 || V <= 0 || V > 0x7fffffff || stride < V) return false;
  if (T > 0x7fffffff) return false;  // one workgroup per row, grid.x limit
  return true;
}

static bool rows_vec_ok(const void* a, const void* b, int dtype) {
  // element alignment is guaranteed by the element type; vector access needs
  // both buffers to reach a 16-byte boundary after the same number of elements
  const int eb = dtype == AA_F32 ? 4 : 2;
  if (((uintptr_t)a % eb) != 0) return false;
  if (b && ((((uintptr_t)a) ^ ((uintptr_t)b)) & 15)) return false;
  return true;
}

// Largest row (in 16 KiB chunks) that still fits the register file without spills.
constexpr int kMaxRegChunks = 21;

// One 1024-thread workgroup per compute unit (its row fills the register file).
static int persistent_workgroups() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    n = cus;
  }
  return n;
}

template <int DT, int NCH, int SHIFT = 0>
static void launch_regs(const void* logits, int64_t T, int V, int64_t stride, const int64_t* labels, float inv_t,
                        const FusedTokenArgs& a, void* dlogits, int32_t* work, hipStream_t st) {
  // Short rows (up to 6 chunks: at most 64 VGPRs per thread) leave room for a second workgroup on every compute
  // unit; with two rows in flight per unit the fixed cost per row (three passes, two reductions) overlaps.
  const int64_t resident = (int64_t)persistent_workgroups() * (NCH <= kTwoPerUnitChunks ? 2 : 1);
  const int64_t wgs = T < resident ? T : resident;
  const uintptr_t mask_addr = (uintptr_t)a.mask_eff;
  if (dlogits == logits)
    hipLaunchKernelGGL((k_fused_regs<DT, NCH, false, true, SHIFT>), dim3((unsigned)wgs), dim3(1024), 0, st, (const uint4*)logits, V,
                       SHIFT == 3 ? stride : stride >> 3, labels, inv_t, a.prox_logp, a.adv, (const uint32_t*)(mask_addr & ~(uintptr_t)3),
                       (unsigned)(mask_addr & 3), a.behave_w, a, (uint4*)dlogits, T, work, 0);
  else
    hipLaunchKernelGGL((k_fused_regs<DT, NCH, false, false, SHIFT>), dim3((unsigned)wgs), dim3(1024), 0, st, (const uint4*)logits, V,
                       SHIFT == 3 ? stride : stride >> 3, labels, inv_t, a.prox_logp, a.adv, (const uint32_t*)(mask_addr & ~(uintptr_t)3),
                       (unsigned)(mask_addr & 3), a.behave_w, a, (uint4*)dlogits, T, work, 0);
}

// Rows of more than kMaxRegChunks chunks: registers + LDS + streamed tail (see k_fused_regs, EXT).
constexpr int kMaxExtChunks = kExtRegChunks + kExtLdsChunks + kExtTailChunks;

template <int DT, int SHIFT>
static bool launch_regs_ext(int nch, const void* logits, int64_t T, int V, int64_t stride, const int64_t* labels,
                            float inv_t, const FusedTokenArgs& a, void* dlogits, int32_t* work, hipStream_t st) {
  static const bool ok =
      hipFuncSetAttribute((const void*)k_fused_regs<DT, kExtRegChunks, true, false, SHIFT>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, kExtLdsChunks * 16384) == hipSuccess &&
      hipFuncSetAttribute((const void*)k_fused_regs<DT, kExtRegChunks, true, true, SHIFT>,
                          hipFuncAttributeMaxDynamicSharedMemorySize, kExtLdsChunks * 16384) == hipSuccess;
  if (!ok || nch <= kExtRegChunks || nch > kMaxExtChunks) return false;
  const int n_lds = nch - kExtRegChunks < kExtLdsChunks ? nch - kExtRegChunks : kExtLdsChunks;
  const int64_t wgs = T < persistent_workgroups() ? T : persistent_workgroups();
  const uintptr_t mask_addr = (uintptr_t)a.mask_eff;
  if (dlogits == logits)
    hipLaunchKernelGGL((k_fused_regs<DT, kExtRegChunks, true, true, SHIFT>), dim3((unsigned)wgs), dim3(1024), n_lds * 16384, st,
                       (const uint4*)logits, V, SHIFT == 3 ? stride : stride >> 3, labels, inv_t, a.prox_logp, a.adv,
                       (const uint32_t*)(mask_addr & ~(uintptr_t)3), (unsigned)(mask_addr & 3), a.behave_w, a,
                       (uint4*)dlogits, T, work, n_lds);
  else
    hipLaunchKernelGGL((k_fused_regs<DT, kExtRegChunks, true, false, SHIFT>), dim3((unsigned)wgs), dim3(1024), n_lds * 16384, st,
                       (const uint4*)logits, V, SHIFT == 3 ? stride : stride >> 3, labels, inv_t, a.prox_logp, a.adv,
                       (const uint32_t*)(mask_addr & ~(uintptr_t)3), (unsigned)(mask_addr & 3), a.behave_w, a,
                       (uint4*)dlogits, T, work, n_lds);
  return true;
}

// Rows of whole chunks at a stride of whole chunks, from kShiftMinChunks chunks on, take the shifted chunk grid (see
// grad_pass): their requests would all start on 16 KB boundaries.  (Below 10 chunks the shift does nothing or costs.)
constexpr int kShiftMinChunks = 10;
static bool wants_shift(int nch, int V, int64_t stride) {
  return nch >= kShiftMinChunks && V % 8192 == 0 && stride % 8192 == 0;
}

// A shift of the row's own (SHIFT == 2) for rows that are not a whole number of KB apart (from kShiftMinChunks chunks
// on: +1 point at V = 151 936, nothing or a loss when the rows already start on 1 KB boundaries), and for any rows
// that are not a whole number of 128-byte lines apart (+3.5 to +10 points: V = 50 272, 50 280, 65 544, 163 848).
// Rows longer than the registers hold gain the same way (V = 200 064: +0.6, 229 376 at a stride of 229 440: +1.2,
// 180 232: +8.9, 256 000 at a stride of 256 008: +7.8).
static bool wants_row_shift(int nch, int64_t stride) {
  const int64_t step = stride * 2;
  return (nch >= kShiftMinChunks && step % 1024 != 0) || step % 128 != 0;
}

// Rows that do not start on 16-byte boundaries (V or the stride not a multiple of 8 values, arrays that start inside a
// 16-byte piece, both at the same place in it): SHIFT == 3.  The chunks are counted over the 16-byte pieces of memory
// that hold a row: one more than the row has when it starts and ends inside a piece.
static int any_alignment_chunks(int64_t V) { return (int)((((14 + V * 2 + 15) >> 4) + 1023) / 1024); }
static bool wants_any_alignment(const void* logits, const void* dlogits, int64_t V, int64_t stride) {
  const uintptr_t a = (uintptr_t)logits, b = (uintptr_t)dlogits;
  if (V % 8 == 0 && stride % 8 == 0 && ((a | b) & 15) == 0) return false;
  return ((a | b) & 1) == 0 && ((a ^ b) & 15) == 0;
}

template <int DT>
static bool dispatch_regs(int mode, int nch, const void* logits, int64_t T, int V, int64_t stride, const int64_t* labels,
                          float inv_t, const FusedTokenArgs& a, void* dlogits, int32_t* work, hipStream_t st) {
  if (mode == 3) {
    switch (nch) {
#define AA_CASE(N) \
  case N: launch_regs<DT, N, 3>(logits, T, V, stride, labels, inv_t, a, dlogits, work, st); return true;
      AA_CASE(3) AA_CASE(4) AA_CASE(5) AA_CASE(6) AA_CASE(7) AA_CASE(8) AA_CASE(9) AA_CASE(10) AA_CASE(11) AA_CASE(12) AA_CASE(13) AA_CASE(14) AA_CASE(15)
      AA_CASE(16) AA_CASE(17) AA_CASE(18) AA_CASE(19) AA_CASE(20) AA_CASE(21)
#undef AA_CASE
      default: return false;
    }
  }
  if (mode == 1) {
    switch (nch) {
#define AA_CASE(N) \
  case N: launch_regs<DT, N, 1>(logits, T, V, stride, labels, inv_t, a, dlogits, work, st); return true;
      AA_CASE(10) AA_CASE(11) AA_CASE(12) AA_CASE(13) AA_CASE(14) AA_CASE(15)
      AA_CASE(16) AA_CASE(17) AA_CASE(18) AA_CASE(19) AA_CASE(20) AA_CASE(21)
#undef AA_CASE
      default: break;
    }
  } else if (mode == 2) {
    switch (nch) {
#define AA_CASE(N) \
  case N: launch_regs<DT, N, 2>(logits, T, V, stride, labels, inv_t, a, dlogits, work, st); return true;
      AA_CASE(3) AA_CASE(4) AA_CASE(5) AA_CASE(6) AA_CASE(7) AA_CASE(8) AA_CASE(9) AA_CASE(10) AA_CASE(11) AA_CASE(12) AA_CASE(13) AA_CASE(14) AA_CASE(15)
      AA_CASE(16) AA_CASE(17) AA_CASE(18) AA_CASE(19) AA_CASE(20) AA_CASE(21)
#undef AA_CASE
      default: break;
    }
  }
  switch (nch) {
#define AA_CASE(N) \
  case N: launch_regs<DT, N>(logits, T, V, stride, labels, inv_t, a, dlogits, work, st); return true;
    AA_CASE(1) AA_CASE(2) AA_CASE(3) AA_CASE(4) AA_CASE(5) AA_CASE(6) AA_CASE(7) AA_CASE(8)
    AA_CASE(9) AA_CASE(10) AA_CASE(11) AA_CASE(12) AA_CASE(13) AA_CASE(14) AA_CASE(15) AA_CASE(16)
    AA_CASE(17) AA_CASE(18) AA_CASE(19) AA_CASE(20) AA_CASE(21)
#undef AA_CASE
    default: return false;
  }
}

}  // namespace aa

using namespace aa;

extern "C" int aa_logits_fwd(const void* logits, int dtype, int64_t T, int64_t V, int64_t row_stride,
                             const int64_t* labels, float inv_temperature, float* logp, float* entropy,
                             float* row_lse, float* row_ez, float* vmax, float* vmin, void* stream) {
  if (!common_args_ok(logits, dtype, T, V, row_stride, labels) || !logp) return AA_ERR_INVALID_ARGUMENT;
  if (!(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  const int vec_ok = rows_vec_ok(logits, nullptr, dtype) ? 1 : 0;
  constexpr int NT = 256;
  // the entropy sum and the extrema are left out of the pass when no output asks for them
  const bool want_u = entropy || row_ez, want_mm = vmax || vmin;
#define AA_LAUNCH_AS(DT, U, MM)                                                                                      \
  hipLaunchKernelGGL((k_logits_fwd<DT, NT, U, MM>), dim3((unsigned)T), dim3(NT), 0, st, logits, (int)V, row_stride, \
                     labels, inv_temperature, vec_ok, logp, entropy, row_lse, row_ez, vmax, vmin)
#define AA_LAUNCH(DT)                                        \
  do {                                                       \
    if (want_u && want_mm) AA_LAUNCH_AS(DT, true, true);     \
    else if (want_u) AA_LAUNCH_AS(DT, true, false);          \
    else if (want_mm) AA_LAUNCH_AS(DT, false, true);         \
    else AA_LAUNCH_AS(DT, false, false);                     \
  } while (0)
  if (dtype == AA_BF16) AA_LAUNCH(AA_BF16);
  else if (dtype == AA_F16) AA_LAUNCH(AA_F16);
  else AA_LAUNCH(AA_F32);
#undef AA_LAUNCH
#undef AA_LAUNCH_AS
  return launch_status();
}

extern "C" int aa_logits_bwd(const void* logits, int dtype, int64_t T, int64_t V, int64_t row_stride,
                             const int64_t* labels, float inv_temperature, const float* row_lse,
                             const float* row_ez, const float* g_logp, const float* g_entropy, int64_t T_active,
                             void* dlogits, void* stream) {
  if (!common_args_ok(logits, dtype, T, V, row_stride, labels)) return AA_ERR_INVALID_ARGUMENT;
  if (!row_lse || !g_logp || !dlogits || (g_entropy && !row_ez)) return AA_ERR_INVALID_ARGUMENT;
  if (T_active < 0 || T_active > T || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  const int vec_ok = rows_vec_ok(logits, dlogits, dtype) ? 1 : 0;
  constexpr int NT = 256;
  // rows on 128-byte lines take the streaming cache policy
  const int64_t row_bytes = row_stride * (dtype == AA_F32 ? 4 : 2);
  const bool streaming = vec_ok && row_bytes % 128 == 0 && ((((uintptr_t)logits | (uintptr_t)dlogits) & 127) == 0);
#define AA_LAUNCH_AS(DT, ALIAS, STREAM)                                                                               \
  hipLaunchKernelGGL((k_logits_bwd<DT, NT, ALIAS, STREAM>), dim3((unsigned)T), dim3(NT), 0, st, logits, (int)V,      \
                     row_stride, labels, inv_temperature, vec_ok, row_lse, row_ez, g_logp, g_entropy, T_active, dlogits)
#define AA_LAUNCH(DT)                                                \
  do {                                                               \
    if (dlogits == logits) {                                         \
      if (streaming) AA_LAUNCH_AS(DT, true, true);                    \
      else AA_LAUNCH_AS(DT, true, false);                            \
    } else {                                                         \
      if (streaming) AA_LAUNCH_AS(DT, false, true);                    \
      else AA_LAUNCH_AS(DT, false, false);                           \
    }                                                                \
  } while (0)
  if (dtype == AA_BF16) AA_LAUNCH(AA_BF16);
  else if (dtype == AA_F16) AA_LAUNCH(AA_F16);
  else AA_LAUNCH(AA_F32);
#undef AA_LAUNCH
#undef AA_LAUNCH_AS
  return launch_status();
}

// dlogits may be the logits array itself.  What makes that work in each kernel below: a row belongs to one workgroup;
// the label's logit and the row statistics are read before the first store of the row; and an element that is read a
// second time for the gradient (two-pass rows, the tail of a row that does not fit on the chip) is read and then
// written by the same thread, the store depending on the load.  The two pointers are restrict-qualified (the
// register kernel measures 0.7 % slower without that) only in the instantiations that run on two distinct arrays; the
// in-place call runs the instantiation without the qualifier.  Tests compare the in-place result bit for bit on every
// kernel.
extern "C" int aa_logits_ppo_fused(const void* logits, int dtype, int64_t T, int64_t V, int64_t row_stride,
                                   const int64_t* labels, float inv_temperature, int64_t T_active,
                                   const float* prox_logp, const float* adv, const uint8_t* mask_eff,
                                   const float* behave_w, const aa_ppo_params* params, const int32_t* n_valid,
                                   const float* grad_scale, float* logp, float* entropy, float* vmax, float* vmin,
                                   float* stat_loss, float* ratio, uint8_t* flags, void* dlogits, int32_t* work,
                                   void* stream) {
  if (!common_args_ok(logits, dtype, T, V, row_stride, labels)) return AA_ERR_INVALID_ARGUMENT;
  if (!params || !n_valid || !logp || !dlogits) return AA_ERR_INVALID_ARGUMENT;
  if (T_active < 0 || T_active > T || !(inv_temperature > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  // the per-token arrays have T_active entries: with no active token they may be absent
  if (params->loss_kind != AA_LOSS_PPO && params->loss_kind != AA_LOSS_NLL && params->loss_kind != AA_LOSS_SAPO)
    return AA_ERR_INVALID_ARGUMENT;
  if (params->loss_kind == AA_LOSS_SAPO &&
      (params->has_behave_weight || !(params->sapo_tau_pos > 0.f) || !(params->sapo_tau_neg > 0.f)))
    return AA_ERR_INVALID_ARGUMENT;
  if (T_active > 0 && (!mask_eff || !stat_loss || !ratio || !flags)) return AA_ERR_INVALID_ARGUMENT;
  if (params->loss_kind == AA_LOSS_NLL) {
    if (params->has_behave_weight) return AA_ERR_INVALID_ARGUMENT;
    // The kernels fetch these arrays ahead of the row pass whatever the loss; in this mode the values are never
    // used, so any readable array of T_active floats serves.
    if (!prox_logp) prox_logp = stat_loss;
    if (!adv) adv = stat_loss;
  }
  if (T_active > 0 && (!prox_logp || !adv)) return AA_ERR_INVALID_ARGUMENT;
  if (T_active > 0 && params->has_behave_weight && !behave_w) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  FusedTokenArgs a;
  a.prox_logp = prox_logp; a.adv = adv; a.mask_eff = mask_eff; a.behave_w = behave_w;
  a.n_valid = n_valid; a.grad_scale = grad_scale;
  a.logp = logp; a.entropy = entropy; a.vmax = vmax; a.vmin = vmin;
  a.stat_loss = stat_loss; a.ratio = ratio; a.flags = flags;
  a.P = *params; a.T_active = T_active;

  const bool any_alignment = wants_any_alignment(logits, dlogits, V, row_stride);
  const bool fast = (dtype != AA_F32) && (V > kTwoPassMaxV) && (T_active > 0) &&
                    (any_alignment ? any_alignment_chunks(V) <= kMaxExtChunks
                                   : (V % 8 == 0) && (row_stride % 8 == 0) && (((uintptr_t)logits & 15) == 0) &&
                                         (((uintptr_t)dlogits & 15) == 0) && (V <= kMaxExtChunks * 8192));
  if (fast) {
    const int nch = any_alignment ? any_alignment_chunks(V) : (int)((V / 8 + 1023) / 1024);
    const int mode = any_alignment ? 3 : wants_shift(nch, (int)V, row_stride) ? 1 : wants_row_shift(nch, row_stride) ? 2 : 0;
    bool ok;
    if (nch <= kMaxRegChunks) {
      ok = (dtype == AA_BF16) ? dispatch_regs<AA_BF16>(mode, nch, logits, T, (int)V, row_stride, labels, inv_temperature, a,
                                                       dlogits, work, st)
                              : dispatch_regs<AA_F16>(mode, nch, logits, T, (int)V, row_stride, labels, inv_temperature, a,
                                                      dlogits, work, st);
    } else {
#define AA_EXT(DT, S) launch_regs_ext<DT, S>(nch, logits, T, (int)V, row_stride, labels, inv_temperature, a, dlogits, work, st)
#define AA_EXT_MODES(DT) (mode == 3 ? AA_EXT(DT, 3) : mode == 2 ? AA_EXT(DT, 2) : mode == 1 ? AA_EXT(DT, 1) : AA_EXT(DT, 0))
      ok = (dtype == AA_BF16) ? AA_EXT_MODES(AA_BF16) : AA_EXT_MODES(AA_F16);
#undef AA_EXT_MODES
#undef AA_EXT
    }
    if (ok) return launch_status();
  }
  if (dtype == AA_F32 && (V % 8 == 0) && (row_stride % 4 == 0) && V >= kHoldChunk && V <= ((int64_t)1 << 28) &&
      ((((uintptr_t)logits | (uintptr_t)dlogits) & 15) == 0)) {
    const int cus = persistent_workgroups();
    const unsigned grid = (unsigned)(T < cus ? T : cus);
    // rows that the exact form would read twice in part are held in 24 bits per value; the pointers are not
    // restrict-qualified: the same code serves dlogits == logits
    // Rows that are not a whole number of 128-byte lines apart take the grid shifted per row (V = 151 944 at a stride
    // of 151 948: 64.1 -> 71.0 % of the HBM peak).  Rows on the lines do not: measured on rows of 65 536 to 200 000
    // values, whole chunks apart or not, the shifted grid reads 0.5 to 1.8 points less there (one case +0.9).
    const bool shifted = (row_stride * 4) % 128 != 0;
#define AA_LAUNCH_HOLD_AS(PACK, NREG, NLDS, SHIFTED)                                                                   \
  hipLaunchKernelGGL((k_fused_f32_hold<PACK, NREG, NLDS, SHIFTED>), dim3(grid), dim3(1024), 0, st, (const float*)logits, \
                     T, (int)V, row_stride, labels, inv_temperature, a, (float*)dlogits, work)
#define AA_LAUNCH_HOLD(PACK, NREG, NLDS)                 \
  do {                                                   \
    if (shifted) AA_LAUNCH_HOLD_AS(PACK, NREG, NLDS, true); \
    else AA_LAUNCH_HOLD_AS(PACK, NREG, NLDS, false);     \
  } while (0)
    if (V > kHoldExactMaxV) AA_LAUNCH_HOLD(true, 13, 6);
    else if (V > 8 * kHoldChunk) AA_LAUNCH_HOLD(false, 10, 4);
    else if (V > 4 * kHoldChunk) AA_LAUNCH_HOLD(false, 8, 0);  // shorter rows: no arithmetic on chunks that no row has
    else AA_LAUNCH_HOLD(false, 4, 0);
#undef AA_LAUNCH_HOLD
#undef AA_LAUNCH_HOLD_AS
    return launch_status();
  }
  const int vec_ok = rows_vec_ok(logits, dlogits, dtype) ? 1 : 0;
  // A row is read twice (statistics, then gradient).  Long rows: few, large workgroups that walk the rows, so that
  // the rows in flight (one per workgroup) stay small enough for the second read to come from the caches.
  const int64_t row_bytes = V * (dtype == AA_F32 ? 4 : 2);
  const bool walk = row_bytes >= kWalkRowBytes && T > kWalkGroups;
#define AA_LAUNCH_AS(DT, ALIAS)                                                                                          \
  do {                                                                                                                   \
    if (walk)                                                                                                            \
      hipLaunchKernelGGL((k_fused_generic<DT, 1024, ALIAS>), dim3((unsigned)kWalkGroups), dim3(1024), 0, st, logits, T,  \
                         (int)V, row_stride, labels, inv_temperature, vec_ok, a, dlogits);                               \
    else                                                                                                                 \
      hipLaunchKernelGGL((k_fused_generic<DT, 256, ALIAS>), dim3((unsigned)T), dim3(256), 0, st, logits, T, (int)V,      \
                         row_stride, labels, inv_temperature, vec_ok, a, dlogits);                                       \
  } while (0)
#define AA_LAUNCH(DT)                                  \
  do {                                                 \
    if (dlogits == logits) AA_LAUNCH_AS(DT, true);     \
    else AA_LAUNCH_AS(DT, false);                      \
  } while (0)
  if (dtype == AA_BF16) AA_LAUNCH(AA_BF16);
  else if (dtype == AA_F16) AA_LAUNCH(AA_F16);
  else AA_LAUNCH(AA_F32);
#undef AA_LAUNCH
#undef AA_LAUNCH_AS
  return launch_status();
}

// -----------------------------------------------------------------------------
// (row, label) pairs that are not "the next token of the same row": the transitions of a packed prefix tree
// (areal/models/tree_attn/functional.py:160-203), where the row that predicts and the token it predicts sit at
// unrelated positions and one row may predict several tokens.
// -----------------------------------------------------------------------------
namespace aa {
template <int DT>
__global__ __launch_bounds__(256) void k_pairs_fwd(const void* __restrict__ logits, int64_t T, int V, int64_t stride,
                                                   const int64_t* __restrict__ rows, const int64_t* __restrict__ labels,
                                                   int64_t K, float inv_t, const float* __restrict__ row_lse,
                                                   const float* __restrict__ row_entropy, float* __restrict__ logp,
                                                   float* __restrict__ entropy) {
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x; k < K; k += step) {
    const int64_t r = rows[k], y = labels[k];
    const bool ok = r >= 0 && r < T && y >= 0 && y < V;
    float lp = __builtin_nanf("");
    if (ok) lp = Elem<DT>::load1(row_ptr(logits, r, stride, Elem<DT>::kBytes), y) * inv_t - row_lse[r];
    logp[k] = lp;
    if (entropy) entropy[k] = (r >= 0 && r < T) ? row_entropy[r] : __builtin_nanf("");
  }
}

// dlogits[rows[k], labels[k]] += g[k] * inv_t; pairs must be distinct (read-modify-write without atomics)
template <int DT>
__global__ __launch_bounds__(256) void k_pairs_scatter(void* __restrict__ dlogits, int64_t T, int V, int64_t stride,
                                                       const int64_t* __restrict__ rows,
                                                       const int64_t* __restrict__ labels, int64_t K,
                                                       const float* __restrict__ g, float inv_t) {
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x; k < K; k += step) {
    const int64_t r = rows[k], y = labels[k];
    if (r < 0 || r >= T || y < 0 || y >= V) continue;
    void* row = (void*)row_ptr(dlogits, r, stride, Elem<DT>::kBytes);
    Elem<DT>::store1(row, y, Elem<DT>::load1(row, y) + g[k] * inv_t);
  }
}
}  // namespace aa

extern "C" int aa_logits_pairs_fwd(const void* logits, int dtype, int64_t T, int64_t V, int64_t row_stride,
                                   const int64_t* rows, const int64_t* labels, int64_t K, float inv_temperature,
                                   const float* row_lse, const float* row_entropy, float* logp, float* entropy,
                                   void* stream) {
  if (K < 0 || T < 0 || V < 1 || V > 0x7fffffff || row_stride < V || !(inv_temperature > 0.f))
    return AA_ERR_INVALID_ARGUMENT;
  if (K == 0) return AA_OK;
  if (!logits || !rows || !labels || !row_lse || !logp || (entropy && !row_entropy)) return AA_ERR_INVALID_ARGUMENT;
  int64_t blocks = (K + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  hipStream_t st = (hipStream_t)stream;
#define AA_LAUNCH(DT)                                                                                              \
  hipLaunchKernelGGL((k_pairs_fwd<DT>), dim3((unsigned)blocks), dim3(256), 0, st, logits, T, (int)V, row_stride, rows, \
                     labels, K, inv_temperature, row_lse, row_entropy, logp, entropy)
  if (dtype == AA_BF16) AA_LAUNCH(AA_BF16);
  else if (dtype == AA_F16) AA_LAUNCH(AA_F16);
  else if (dtype == AA_F32) AA_LAUNCH(AA_F32);
  else return AA_ERR_INVALID_ARGUMENT;
#undef AA_LAUNCH
  return launch_status();
}

extern "C" int aa_logits_pairs_scatter(void* dlogits, int dtype, int64_t T, int64_t V, int64_t row_stride,
                                       const int64_t* rows, const int64_t* labels, int64_t K, const float* g,
                                       float inv_temperature, void* stream) {
  if (K < 0 || T < 0 || V < 1 || V > 0x7fffffff || row_stride < V) return AA_ERR_INVALID_ARGUMENT;
  if (K == 0) return AA_OK;
  if (!dlogits || !rows || !labels || !g) return AA_ERR_INVALID_ARGUMENT;
  int64_t blocks = (K + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  hipStream_t st = (hipStream_t)stream;
#define AA_LAUNCH(DT)                                                                                                \
  hipLaunchKernelGGL((k_pairs_scatter<DT>), dim3((unsigned)blocks), dim3(256), 0, st, dlogits, T, (int)V, row_stride, \
                     rows, labels, K, g, inv_temperature)
  if (dtype == AA_BF16) AA_LAUNCH(AA_BF16);
  else if (dtype == AA_F16) AA_LAUNCH(AA_F16);
  else if (dtype == AA_F32) AA_LAUNCH(AA_F32);
  else return AA_ERR_INVALID_ARGUMENT;
#undef AA_LAUNCH
  return launch_status();
}

extern "C" int aa_copy_bytes(const void* src, void* dst, int64_t nbytes, void* stream) {
  if (!src || !dst || nbytes < 0 || (nbytes & 15) || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15))
    return AA_ERR_INVALID_ARGUMENT;
  if (nbytes == 0) return AA_OK;
  const int64_t n = nbytes >> 4;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  hipLaunchKernelGGL(k_copy16, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint4*)src,
                     (uint4*)dst, n);
  return launch_status();
}

extern "C" int aa_scale_inplace(void* data, int dtype, int64_t n, const float* factor, void* stream) {
  if (!data || !factor || n < 0) return AA_ERR_INVALID_ARGUMENT;
  if (n == 0) return AA_OK;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == AA_BF16) hipLaunchKernelGGL(k_scale<AA_BF16>, dim3((unsigned)blocks), dim3(256), 0, st, data, n, factor);
  else if (dtype == AA_F16) hipLaunchKernelGGL(k_scale<AA_F16>, dim3((unsigned)blocks), dim3(256), 0, st, data, n, factor);
  else if (dtype == AA_F32) hipLaunchKernelGGL(k_scale<AA_F32>, dim3((unsigned)blocks), dim3(256), 0, st, data, n, factor);
  else return AA_ERR_INVALID_ARGUMENT;
  return launch_status();
}

extern "C" int aa_scale_rows_inplace(void* data, int dtype, int64_t T, int64_t V, int64_t row_stride, const float* factor,
                                     void* stream) {
  if (!data || !factor || T < 0 || V < 0 || row_stride < V) return AA_ERR_INVALID_ARGUMENT;
  if (row_stride == V) return aa_scale_inplace(data, dtype, T * V, factor, stream);
  if (T == 0 || V == 0) return AA_OK;
  int64_t blocks = (T * V + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == AA_BF16) hipLaunchKernelGGL(k_scale_rows<AA_BF16>, dim3((unsigned)blocks), dim3(256), 0, st, data, T, V, row_stride, factor);
  else if (dtype == AA_F16) hipLaunchKernelGGL(k_scale_rows<AA_F16>, dim3((unsigned)blocks), dim3(256), 0, st, data, T, V, row_stride, factor);
  else if (dtype == AA_F32) hipLaunchKernelGGL(k_scale_rows<AA_F32>, dim3((unsigned)blocks), dim3(256), 0, st, data, T, V, row_stride, factor);
  else return AA_ERR_INVALID_ARGUMENT;
  return launch_status();
}

extern "C" int aa_vocab_partials_combine(const float* shard_lse, const float* shard_ez, const float* shard_logp,
                                         int n_shards, int64_t T, float* logp, float* entropy, float* row_lse,
                                         float* row_ez, void* stream) {
  if (n_shards < 1 || T < 0 || !logp) return AA_ERR_INVALID_ARGUMENT;
  if (T == 0) return AA_OK;
  if (!shard_lse || !shard_ez || !shard_logp) return AA_ERR_INVALID_ARGUMENT;
  int64_t blocks = (T + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(k_vocab_partials_combine, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, shard_lse,
                     shard_ez, shard_logp, n_shards, T, logp, entropy, row_lse, row_ez);
  return launch_status();
}
