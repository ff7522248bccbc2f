// Per-token kernels of the PPO actor loss on packed sequences: rejection
// sampling (importance-weight cap), the clipped surrogate with its closed-form
// derivative at token and sequence level, and the deterministic masked sum.
//
// Follows areal/utils/functional/functional.py:56-149 (sequence-level ratio),
// :185-426 (apply_rejection_sampling), :429-559 (ppo_actor_loss_fn) and
// areal/utils/data.py:1620-1656 (KL estimators k1/k2/k3).
//
// All of this is O(T) work on a few floats per token; the kernels are written
// for determinism (fixed reduction order, integer atomics only) rather than
// bandwidth.
#include "device_utils.h"
#include "ppo_math.h"

namespace aa {

constexpr int kSegThreads = 256;

struct Segments {
  const int32_t* cu;  // [B+1] or nullptr
  int64_t B;
  int64_t n;
  // [begin, end) of segment b; b == B is the uncovered tail after cu[B]
  __device__ __forceinline__ void range(int64_t b, int64_t& beg, int64_t& end) const {
    if (cu) {
      if (b < B) { beg = cu[b]; end = cu[b + 1]; }
      else { beg = cu[B]; end = n; }
      if (beg < 0) beg = 0;
      if (end > n) end = n;
    } else {
      const int64_t S = n / B;
      if (b < B) { beg = b * S; end = beg + S; }
      else { beg = B * S; end = n; }
    }
  }
};

template <typename T>
__device__ __forceinline__ T block_sum(T v, T* smem) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  T r = smem[0];
  for (int w = 1; w < (int)(blockDim.x / kWave); ++w) r += smem[w];
  return r;
}

__device__ __forceinline__ float block_max(float v, float* smem) {
  v = wave_max(v);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float r = smem[0];
  for (int w = 1; w < (int)(blockDim.x / kWave); ++w) r = fmaxf(r, smem[w]);
  return r;
}

// ---- rejection sampling ------------------------------------------------------
struct RsCfg {
  int level, action, metric, agg, has_lower;
  float upper, lower;
};

__device__ __forceinline__ float rs_log_ratio(float prox, float old) {
  const float lr = prox - old;
  return isfinite(lr) ? lr : 0.f;  // functional.py:231-233
}

// metric value per token; the KL estimators see the raw difference
// (data.py:1620-1656 with apply_clamp=False)
__device__ __forceinline__ float rs_metric(int metric, float prox, float old, float lr) {
  switch (metric) {
    case AA_RS_RATIO: return expf(lr);
    case AA_RS_KL_K1: return prox - old;
    case AA_RS_KL_K2: { const float d = prox - old; return d * d / 2.0f; }
    default: { const float d = -(prox - old); return expf(d) - 1.f - d; }
  }
}

__device__ __forceinline__ bool rs_in_bounds(float v, const RsCfg& c) {
  return c.has_lower ? ((v >= c.lower) && (v <= c.upper)) : (v <= c.upper);
}

__device__ __forceinline__ float rs_clamp(float w, const RsCfg& c) {
  const float lo = c.has_lower ? c.lower : 0.f;
  return nan_min(nan_max(w, lo), c.upper);
}

__global__ void k_zero_i32(int32_t* p, int n) {
  if ((int)threadIdx.x < n) p[threadIdx.x] = 0;
}

__global__ __launch_bounds__(256) void k_rs_token(const float* __restrict__ prox, const float* __restrict__ old,
                                                  const uint8_t* __restrict__ mask, int64_t n, RsCfg c,
                                                  uint8_t* __restrict__ mask_out, float* __restrict__ w_out,
                                                  int32_t* __restrict__ counts) {
  __shared__ int smem[256 / kWave];
  int total = 0, hit = 0;
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const bool m = mask[i] != 0;
    const float p = prox[i], o = old[i];
    const float lr = rs_log_ratio(p, o);
    float w = expf(lr);
    bool keep = m;
    if (c.action == AA_RS_ACTION_MASK) {
      const bool inb = rs_in_bounds(rs_metric(c.metric, p, o, lr), c);
      keep = m && inb;
      hit += (m && !inb) ? 1 : 0;
    } else {
      const float wc = rs_clamp(w, c);
      hit += (m && (wc != w)) ? 1 : 0;
      w = wc;
    }
    total += m ? 1 : 0;
    mask_out[i] = keep ? 1 : 0;
    w_out[i] = keep ? w : 0.f;
  }
  total = block_sum<int>(total, smem);
  hit = block_sum<int>(hit, smem);
  if (threadIdx.x == 0) {
    if (total) atomicAdd(&counts[0], total);
    if (hit) atomicAdd(&counts[1], hit);
  }
}

__global__ __launch_bounds__(kSegThreads) void k_rs_sequence(const float* __restrict__ prox,
                                                             const float* __restrict__ old,
                                                             const uint8_t* __restrict__ mask, Segments seg, RsCfg c,
                                                             uint8_t* __restrict__ mask_out,
                                                             float* __restrict__ w_out,
                                                             int32_t* __restrict__ counts) {
  __shared__ double smem_d[kSegThreads / kWave];
  __shared__ float smem_f[kSegThreads / kWave];
  __shared__ int smem_i[kSegThreads / kWave];
  const int64_t b = blockIdx.x;
  int64_t beg, end;
  seg.range(b, beg, end);
  if (b == seg.B) {  // tokens no sequence covers
    for (int64_t i = beg + threadIdx.x; i < end; i += kSegThreads) { mask_out[i] = 0; w_out[i] = 0.f; }
    return;
  }
  const bool log_agg = c.metric == AA_RS_RATIO;
  double sum = 0.0;
  float mx = -INFINITY;
  int cnt = 0;
  for (int64_t i = beg + threadIdx.x; i < end; i += kSegThreads) {
    if (mask[i] != 0) {
      const float p = prox[i], o = old[i];
      const float lr = rs_log_ratio(p, o);
      const float v = log_agg ? lr : rs_metric(c.metric, p, o, lr);
      sum += (double)v;
      mx = nan_max(mx, v);
      cnt += 1;
    }
  }
  const float fsum = (float)block_sum<double>(sum, smem_d);
  mx = block_max(mx, smem_f);
  const int raw = block_sum<int>(cnt, smem_i);
  const float fcnt = (float)(raw < 1 ? 1 : raw);
  const float w_seq = log_agg ? expf(fsum / fcnt) : 0.f;  // geometric mean as uniform weight
  float agg;
  if (c.agg == AA_RS_AGG_SUM) agg = fsum;
  else if (c.agg == AA_RS_AGG_MEAN) agg = fsum / fcnt;
  else agg = (raw == 0) ? 0.f : mx;
  const float seq_metric = log_agg ? expf(agg) : agg;
  const bool inb = rs_in_bounds(seq_metric, c);
  int hit = 0;
  for (int64_t i = beg + threadIdx.x; i < end; i += kSegThreads) {
    const bool m = mask[i] != 0;
    float w = log_agg ? w_seq : expf(rs_log_ratio(prox[i], old[i]));
    bool keep = m;
    if (c.action == AA_RS_ACTION_MASK) {
      keep = m && inb;
      hit += (m && !inb) ? 1 : 0;
    } else {
      const float wc = inb ? w : rs_clamp(w, c);
      hit += (m && (wc != w)) ? 1 : 0;
      w = wc;
    }
    mask_out[i] = keep ? 1 : 0;
    w_out[i] = keep ? w : 0.f;
  }
  hit = block_sum<int>(hit, smem_i);
  if (threadIdx.x == 0) {
    if (raw) atomicAdd(&counts[0], raw);
    if (hit) atomicAdd(&counts[1], hit);
  }
}

__global__ __launch_bounds__(1024) void k_count_nonzero(const uint8_t* __restrict__ mask, int64_t n,
                                                        int32_t* __restrict__ count) {
  __shared__ int smem[1024 / kWave];
  int c = 0;
  const int64_t n4 = ((((uintptr_t)mask) & 3) == 0) ? (n >> 2) : 0;  // four mask bytes per load
  for (int64_t q = threadIdx.x; q < n4; q += 1024) {
    const uint32_t m = ((const uint32_t*)mask)[q];
    c += ((m & 0x000000ffu) ? 1 : 0) + ((m & 0x0000ff00u) ? 1 : 0) + ((m & 0x00ff0000u) ? 1 : 0) +
         ((m & 0xff000000u) ? 1 : 0);
  }
  for (int64_t i = (n4 << 2) + threadIdx.x; i < n; i += 1024) c += mask[i] != 0 ? 1 : 0;
  c = block_sum<int>(c, smem);
  if (threadIdx.x == 0) count[0] = c;
}

// ---- clipped surrogate, token level -------------------------------------------
__global__ __launch_bounds__(256) void k_ppo_token(const float* __restrict__ logp, const float* __restrict__ prox,
                                                   const float* __restrict__ adv, const uint8_t* __restrict__ mask,
                                                   const float* __restrict__ bw, int64_t n, aa_ppo_params P,
                                                   const int32_t* __restrict__ n_valid,
                                                   float* __restrict__ stat_loss, float* __restrict__ ratio,
                                                   uint8_t* __restrict__ flags, float* __restrict__ g_logp) {
  int nv = *n_valid;
  if (nv < 1) nv = 1;
  const float fn = (float)nv;
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const bool m = mask[i] != 0;
    const float r = m ? expf(logp[i] - prox[i]) : 0.f;
    const Surrogate s = surrogate(r, adv[i], P.has_behave_weight ? bw[i] : 1.f, P);
    stat_loss[i] = s.loss;
    ratio[i] = r;
    flags[i] = (uint8_t)(((s.clip && m) ? 1 : 0) | ((s.dual && m) ? 2 : 0));
    g_logp[i] = m ? s.dloss_dr * r / fn : 0.f;
  }
}

// ---- clipped surrogate, sequence level (GSPO) -----------------------------------
__global__ __launch_bounds__(kSegThreads) void k_ppo_sequence(const float* __restrict__ logp,
                                                              const float* __restrict__ prox,
                                                              const float* __restrict__ adv,
                                                              const uint8_t* __restrict__ mask,
                                                              const float* __restrict__ bw, Segments seg,
                                                              aa_ppo_params P, const int32_t* __restrict__ n_valid,
                                                              float* __restrict__ stat_loss,
                                                              float* __restrict__ ratio, uint8_t* __restrict__ flags,
                                                              float* __restrict__ g_logp) {
  __shared__ double smem_d[kSegThreads / kWave];
  __shared__ int smem_i[kSegThreads / kWave];
  const int64_t b = blockIdx.x;
  int64_t beg, end;
  seg.range(b, beg, end);
  if (b == seg.B) {
    for (int64_t i = beg + threadIdx.x; i < end; i += kSegThreads) {
      stat_loss[i] = 0.f; ratio[i] = 0.f; flags[i] = 0; g_logp[i] = 0.f;
    }
    return;
  }
  double slr = 0.0, sadv = 0.0;
  int cnt = 0;
  for (int64_t i = beg + threadIdx.x; i < end; i += kSegThreads) {
    if (mask[i] != 0) {
      slr += (double)(logp[i] - prox[i]);
      sadv += (double)adv[i];
      cnt += 1;
    }
  }
  const float f_slr = (float)block_sum<double>(slr, smem_d);
  const float f_sadv = (float)block_sum<double>(sadv, smem_d);
  const int raw = block_sum<int>(cnt, smem_i);
  const float fcnt = (float)(raw < 1 ? 1 : raw);
  const float r_seq = expf(f_slr / fcnt);
  const float a_seq = f_sadv / fcnt;
  double gsum = 0.0;
  for (int64_t i = beg + threadIdx.x; i < end; i += kSegThreads) {
    const bool m = mask[i] != 0;
    const float r = m ? r_seq : 0.f;
    const float a = m ? a_seq : 0.f;
    const Surrogate s = surrogate(r, a, P.has_behave_weight ? bw[i] : 1.f, P);
    stat_loss[i] = s.loss;
    ratio[i] = r;
    flags[i] = (uint8_t)(((s.clip && m) ? 1 : 0) | ((s.dual && m) ? 2 : 0));
    if (m) gsum += (double)s.dloss_dr;
  }
  const float G = (float)block_sum<double>(gsum, smem_d);
  int nv = *n_valid;
  if (nv < 1) nv = 1;
  const float gk = G * r_seq / fcnt / (float)nv;
  for (int64_t i = beg + threadIdx.x; i < end; i += kSegThreads) g_logp[i] = (mask[i] != 0) ? gk : 0.f;
}

// ---- deterministic masked sum ---------------------------------------------------
__global__ __launch_bounds__(1024) void k_masked_sum(const float* __restrict__ values,
                                                     const uint8_t* __restrict__ mask, int64_t n,
                                                     const int32_t* __restrict__ n_valid,
                                                     const float* __restrict__ scale, float* __restrict__ out) {
  __shared__ double smem[1024 / kWave];
  double acc = 0.0;
  // four elements per thread and trip (16-byte value loads when the base allows), always in the same order
  const bool vec = (((uintptr_t)values) & 15) == 0 && (!mask || (((uintptr_t)mask) & 3) == 0);
  const int64_t n4 = vec ? (n >> 2) : 0;
  auto part_of = [](const float4 v, const uint32_t m) {
    double part = 0.0;
    if (m & 0x000000ffu) part += (double)v.x;
    if (m & 0x0000ff00u) part += (double)v.y;
    if (m & 0x00ff0000u) part += (double)v.z;
    if (m & 0xff000000u) part += (double)v.w;
    return part;
  };
  // four trips at a time, their loads issued together (one workgroup: the loop is bound by memory latency); the
  // order of the additions is the one of the plain loop
  int64_t q = threadIdx.x;
  for (; q + 3 * 1024 < n4; q += 4 * 1024) {
    float4 v[4];
    uint32_t m[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[j] = ((const float4*)values)[q + j * 1024];
      m[j] = mask ? ((const uint32_t*)mask)[q + j * 1024] : 0x01010101u;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) acc += part_of(v[j], m[j]);
  }
  for (; q < n4; q += 1024) acc += part_of(((const float4*)values)[q], mask ? ((const uint32_t*)mask)[q] : 0x01010101u);
  for (int64_t i = (n4 << 2) + threadIdx.x; i < n; i += 1024)
    if (!mask || mask[i] != 0) acc += (double)values[i];
  acc = block_sum<double>(acc, smem);
  if (threadIdx.x == 0) {
    int nv = n_valid ? *n_valid : 1;
    if (nv < 1) nv = 1;
    float r = (float)acc / (float)nv;
    if (scale) r *= *scale;
    out[0] = r;
  }
}

// ---- the derived entries of the stat dict (functional.py:505-558), one launch instead of one per entry ------------
__global__ __launch_bounds__(256) void k_ppo_stat_outputs(const float* __restrict__ logp, const float* __restrict__ prox,
                                                          const float* __restrict__ old, const uint8_t* __restrict__ flags,
                                                          const float* __restrict__ behave_w,
                                                          const uint8_t* __restrict__ mask_eff, int64_t n,
                                                          float* __restrict__ approx_kl, uint8_t* __restrict__ clip,
                                                          uint8_t* __restrict__ dual, uint8_t* __restrict__ behave_mask,
                                                          float* __restrict__ behave_kl) {
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const float p = prox[i];
    approx_kl[i] = logp[i] - p;
    const uint8_t f = flags[i];
    clip[i] = f & 1;
    dual[i] = (f >> 1) & 1;
    if (behave_mask) {
      const bool on = behave_w[i] > 0.f && mask_eff[i] != 0;
      behave_mask[i] = on ? 1 : 0;
      behave_kl[i] = on ? p - old[i] : 0.f;
    }
  }
}

// ---- SAPO: soft sigmoid gates instead of clipping (functional.py:562-638) ---------------------------------------
struct SapoTerm {
  float loss, dloss_dr, soft, gate_pos, gate_neg;
};

__device__ __forceinline__ float sigmoidf(float z) { return 1.f / (1.f + expf(-z)); }

__device__ __forceinline__ SapoTerm sapo_term(float r, float adv, float tau_pos, float tau_neg) {
  const float gp = sigmoidf(tau_pos * (r - 1.f)), gn = sigmoidf(tau_neg * (r - 1.f));
  SapoTerm o;
  o.gate_pos = gp * (4.f / tau_pos);
  o.gate_neg = gn * (4.f / tau_neg);
  const bool pos = adv > 0.f;
  o.soft = pos ? o.gate_pos : o.gate_neg;
  o.loss = -o.soft * adv;
  const float g = pos ? gp : gn;
  o.dloss_dr = -4.f * adv * g * (1.f - g);  // (4 / tau) * sigmoid'(tau (r - 1)) * tau
  return o;
}

__global__ __launch_bounds__(256) void k_sapo_token(const float* __restrict__ logp, const float* __restrict__ old,
                                                    const float* __restrict__ adv, const uint8_t* __restrict__ mask,
                                                    int64_t n, float tau_pos, float tau_neg,
                                                    const int32_t* __restrict__ n_valid, float* __restrict__ stat_loss,
                                                    float* __restrict__ ratio, float* __restrict__ gates,
                                                    float* __restrict__ g_logp) {
  int nv = *n_valid;
  if (nv < 1) nv = 1;
  const float fn = (float)nv;
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const float r = expf(logp[i] - old[i]);  // not masked: functional.py:600
    const SapoTerm t = sapo_term(r, adv[i], tau_pos, tau_neg);
    stat_loss[i] = t.loss;
    ratio[i] = r;
    gates[i] = t.soft;
    gates[n + i] = t.gate_pos;
    gates[2 * n + i] = t.gate_neg;
    g_logp[i] = mask[i] != 0 ? t.dloss_dr * r / fn : 0.f;
  }
}

__global__ __launch_bounds__(kSegThreads) void k_sapo_sequence(const float* __restrict__ logp,
                                                               const float* __restrict__ old,
                                                               const float* __restrict__ adv,
                                                               const uint8_t* __restrict__ mask, Segments seg,
                                                               float tau_pos, float tau_neg,
                                                               const int32_t* __restrict__ n_valid,
                                                               float* __restrict__ stat_loss,
                                                               float* __restrict__ ratio, float* __restrict__ gates,
                                                               float* __restrict__ g_logp) {
  __shared__ double smem_d[kSegThreads / kWave];
  __shared__ int smem_i[kSegThreads / kWave];
  const int64_t b = blockIdx.x, n = seg.n;
  int64_t beg, end;
  seg.range(b, beg, end);
  double slr = 0.0, sadv = 0.0;
  int cnt = 0;
  const bool tail = b == seg.B;  // tokens no sequence covers: ratio 0, advantage 0
  if (!tail) {
    for (int64_t i = beg + threadIdx.x; i < end; i += kSegThreads) {
      if (mask[i] != 0) {
        slr += (double)(logp[i] - old[i]);
        sadv += (double)adv[i];
        cnt += 1;
      }
    }
  }
  const float f_slr = (float)block_sum<double>(slr, smem_d);
  const float f_sadv = (float)block_sum<double>(sadv, smem_d);
  const int raw = block_sum<int>(cnt, smem_i);
  const float fcnt = (float)(raw < 1 ? 1 : raw);
  const float r_seq = expf(f_slr / fcnt);
  const float a_seq = f_sadv / fcnt;
  double gsum = 0.0;
  for (int64_t i = beg + threadIdx.x; i < end; i += kSegThreads) {
    const bool m = !tail && mask[i] != 0;
    const SapoTerm t = sapo_term(m ? r_seq : 0.f, m ? a_seq : 0.f, tau_pos, tau_neg);
    stat_loss[i] = t.loss;
    ratio[i] = m ? r_seq : 0.f;
    gates[i] = t.soft;
    gates[n + i] = t.gate_pos;
    gates[2 * n + i] = t.gate_neg;
    if (m) gsum += (double)t.dloss_dr;
  }
  const float G = (float)block_sum<double>(gsum, smem_d);
  int nv = *n_valid;
  if (nv < 1) nv = 1;
  const float gk = G * r_seq / fcnt / (float)nv;
  for (int64_t i = beg + threadIdx.x; i < end; i += kSegThreads) g_logp[i] = (!tail && mask[i] != 0) ? gk : 0.f;
}

// ---- clipped value loss of the critic (functional.py:704-778) ---------------------------------------------------
__device__ __forceinline__ void value_loss_term(int huber, float x, float y, float& loss, float& dx) {
  const float e = x - y;
  if (!huber) {
    loss = 0.5f * e * e;
    dx = e;
    return;
  }
  const float delta = 10.f, diff = fabsf(e);
  if (diff < delta) {
    loss = 0.5f * diff * diff;
    dx = e;
  } else {
    loss = delta * (diff - 0.5f * delta);
    dx = e > 0.f ? delta : -delta;
  }
}

__global__ __launch_bounds__(256) void k_critic_loss(const float* __restrict__ value, const float* __restrict__ old,
                                                     const float* __restrict__ target,
                                                     const uint8_t* __restrict__ mask, int64_t n, float eps,
                                                     int huber, const int32_t* __restrict__ n_valid,
                                                     float* __restrict__ stat_loss, uint8_t* __restrict__ clip,
                                                     float* __restrict__ g_value) {
  // the reference divides by count_nonzero (or by n without a mask) with no floor: an empty mask gives 0 / 0
  const float fn = (float)(*n_valid);
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const float v = value[i], o = old[i], y = target[i];
    const float d = v - o;
    const float dc = nan_min(nan_max(d, -eps), eps);
    const bool in_range = (d >= -eps) && (d <= eps);
    float l1, g1, l2, g2;
    value_loss_term(huber, v, y, l1, g1);
    value_loss_term(huber, o + dc, y, l2, g2);
    const bool m = mask ? mask[i] != 0 : true;
    const float w1 = (l1 == l2) ? 0.5f : ((l1 > l2) ? 1.f : 0.f);
    stat_loss[i] = nan_max(l1, l2);
    clip[i] = (uint8_t)((l2 > l1 && m) ? 1 : 0);
    g_value[i] = m ? (w1 * g1 + (in_range ? (1.f - w1) * g2 : 0.f)) / fn : 0.f;
  }
}

// ---- proximal log-prob approximations from per-token policy versions (actor.py:604-684) --------------------------
__global__ __launch_bounds__(256) void k_prox_approx(const float* __restrict__ old, const float* __restrict__ logp,
                                                     const int32_t* __restrict__ versions, int64_t n,
                                                     int current_version, int method, float* __restrict__ out) {
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step)
    out[i] = prox_approx_value(old[i], logp[i], versions[i], current_version, method);
}

// ---- joint-distillation terms of the actor loss (actor.py:482-511) ------------------------------------------------
// pure (rl_loss_weight == 0):  term = exp(logp - old) * (teacher - logp) * mask,  d term / d logp = term
//                              (the reward teacher - logp is detached; the importance weight carries the gradient)
// joint:                       term = (logp - teacher) * mask,                     d term / d logp = mask
__global__ __launch_bounds__(256) void k_kd_terms(const float* __restrict__ logp, const float* __restrict__ old,
                                                  const float* __restrict__ teacher, const uint8_t* __restrict__ mask,
                                                  int64_t n, int pure, float* __restrict__ term,
                                                  float* __restrict__ dterm) {
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const float m = mask[i] ? 1.f : 0.f;
    const float lp = logp[i], tl = teacher[i];
    float t, d;
    if (pure) {
      t = expf(lp - old[i]) * (tl - lp) * m;  // (x * y) * mask as the reference orders it: NaN/inf propagate alike
      d = t;
    } else {
      t = (lp - tl) * m;
      d = m;
    }
    term[i] = t;
    dterm[i] = d;
  }
}

static unsigned grid_for(int64_t n) {
  int64_t b = (n + 255) / 256;
  if (b > 2048) b = 2048;
  if (b < 1) b = 1;
  return (unsigned)b;
}

}  // namespace aa

using namespace aa;

extern "C" int aa_rejection_sampling(const float* prox_logp, const float* old_logp, const uint8_t* mask_in, int64_t n,
                                     const int32_t* cu_seqlens, int64_t B, int level, int action, int metric, int agg,
                                     float upper, float lower, int has_lower, uint8_t* mask_out, float* behave_w,
                                     int32_t* counts, void* stream) {
  if (!counts || n < 0) return AA_ERR_INVALID_ARGUMENT;
  // an empty batch may come with null data pointers: only the counters are written
  if (n > 0 && (!prox_logp || !old_logp || !mask_in || !mask_out || !behave_w)) return AA_ERR_INVALID_ARGUMENT;
  if (level < 0 || level > 1 || action < 0 || action > 1 || metric < 0 || metric > 3 || agg < 0 || agg > 2)
    return AA_ERR_INVALID_ARGUMENT;
  if (action == AA_RS_ACTION_CLAMP && metric != AA_RS_RATIO) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  RsCfg c{level, action, metric, agg, has_lower, upper, lower};
  hipLaunchKernelGGL(k_zero_i32, dim3(1), dim3(64), 0, st, counts, 3);
  if (n == 0) return launch_status();
  if (level == AA_RS_LEVEL_TOKEN) {
    hipLaunchKernelGGL(k_rs_token, dim3(grid_for(n)), dim3(256), 0, st, prox_logp, old_logp, mask_in, n, c, mask_out,
                       behave_w, counts);
  } else {
    if (B <= 0 || B > 0x7ffffffe) return AA_ERR_INVALID_ARGUMENT;
    if (!cu_seqlens && (n % B) != 0) return AA_ERR_INVALID_ARGUMENT;
    Segments seg{cu_seqlens, B, n};
    hipLaunchKernelGGL(k_rs_sequence, dim3((unsigned)(B + 1)), dim3(kSegThreads), 0, st, prox_logp, old_logp, mask_in,
                       seg, c, mask_out, behave_w, counts);
  }
  return launch_status();
}

extern "C" int aa_count_nonzero_u8(const uint8_t* mask, int64_t n, int32_t* count, void* stream) {
  if ((!mask && n > 0) || !count || n < 0) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_count_nonzero, dim3(1), dim3(1024), 0, (hipStream_t)stream, mask, n, count);
  return launch_status();
}

extern "C" int aa_ppo_loss(const float* logp, const float* prox_logp, const float* adv, const uint8_t* mask_eff,
                           const float* behave_w, int64_t n, const int32_t* cu_seqlens, int64_t B, int sequence_level,
                           const aa_ppo_params* params, const int32_t* n_valid, float* stat_loss, float* ratio,
                           uint8_t* flags, float* g_logp, void* stream) {
  if (!params || !n_valid || n < 0) return AA_ERR_INVALID_ARGUMENT;
  if (n == 0) return AA_OK;
  if (!logp || !prox_logp || !adv || !mask_eff || !stat_loss || !ratio || !flags || !g_logp)
    return AA_ERR_INVALID_ARGUMENT;
  if (params->has_behave_weight && !behave_w) return AA_ERR_INVALID_ARGUMENT;
  if (params->loss_kind != AA_LOSS_PPO) return AA_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  if (!sequence_level) {
    hipLaunchKernelGGL(k_ppo_token, dim3(grid_for(n)), dim3(256), 0, st, logp, prox_logp, adv, mask_eff, behave_w, n,
                       *params, n_valid, stat_loss, ratio, flags, g_logp);
  } else {
    if (B <= 0 || B > 0x7ffffffe) return AA_ERR_INVALID_ARGUMENT;
    if (!cu_seqlens && (n % B) != 0) return AA_ERR_INVALID_ARGUMENT;
    Segments seg{cu_seqlens, B, n};
    hipLaunchKernelGGL(k_ppo_sequence, dim3((unsigned)(B + 1)), dim3(kSegThreads), 0, st, logp, prox_logp, adv,
                       mask_eff, behave_w, seg, *params, n_valid, stat_loss, ratio, flags, g_logp);
  }
  return launch_status();
}

extern "C" int aa_masked_sum(const float* values, const uint8_t* mask, int64_t n, const int32_t* n_valid,
                             const float* scale, float* out, void* stream) {
  if (!out || n < 0 || (n > 0 && !values)) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_masked_sum, dim3(1), dim3(1024), 0, (hipStream_t)stream, values, mask, n, n_valid, scale, out);
  return launch_status();
}

extern "C" int aa_ppo_stat_outputs(const float* logp, const float* prox_logp, const float* old_logp, const uint8_t* flags,
                                   const float* behave_w, const uint8_t* mask_eff, int64_t n, float* approx_kl,
                                   uint8_t* clip_mask, uint8_t* dual_clip_mask, uint8_t* behave_mask,
                                   float* behave_approx_kl, void* stream) {
  if (n < 0) return AA_ERR_INVALID_ARGUMENT;
  if (n == 0) return AA_OK;
  if (!logp || !prox_logp || !flags || !approx_kl || !clip_mask || !dual_clip_mask) return AA_ERR_INVALID_ARGUMENT;
  if ((behave_mask != nullptr) != (behave_approx_kl != nullptr)) return AA_ERR_INVALID_ARGUMENT;
  if (behave_mask && (!old_logp || !behave_w || !mask_eff)) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_ppo_stat_outputs, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream, logp, prox_logp, old_logp,
                     flags, behave_w, mask_eff, n, approx_kl, clip_mask, dual_clip_mask, behave_mask, behave_approx_kl);
  return launch_status();
}

extern "C" int aa_sapo_loss(const float* logp, const float* old_logp, const float* adv, const uint8_t* mask, int64_t n,
                            const int32_t* cu_seqlens, int64_t B, int sequence_level, float tau_pos, float tau_neg,
                            const int32_t* n_valid, float* stat_loss, float* ratio, float* gates, float* g_logp,
                            void* stream) {
  if (!n_valid || n < 0 || !(tau_pos > 0.f) || !(tau_neg > 0.f)) return AA_ERR_INVALID_ARGUMENT;
  if (n == 0) return AA_OK;
  if (!logp || !old_logp || !adv || !mask || !stat_loss || !ratio || !gates || !g_logp) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  if (!sequence_level) {
    hipLaunchKernelGGL(k_sapo_token, dim3(grid_for(n)), dim3(256), 0, st, logp, old_logp, adv, mask, n, tau_pos,
                       tau_neg, n_valid, stat_loss, ratio, gates, g_logp);
  } else {
    if (B <= 0 || B > 0x7ffffffe) return AA_ERR_INVALID_ARGUMENT;
    if (!cu_seqlens && (n % B) != 0) return AA_ERR_INVALID_ARGUMENT;
    Segments seg{cu_seqlens, B, n};
    hipLaunchKernelGGL(k_sapo_sequence, dim3((unsigned)(B + 1)), dim3(kSegThreads), 0, st, logp, old_logp, adv, mask,
                       seg, tau_pos, tau_neg, n_valid, stat_loss, ratio, gates, g_logp);
  }
  return launch_status();
}

extern "C" int aa_critic_loss(const float* value, const float* old_value, const float* target_value,
                              const uint8_t* mask, int64_t n, float value_eps_clip, int loss_type,
                              const int32_t* n_valid, float* stat_loss, uint8_t* clip_mask, float* g_value,
                              void* stream) {
  if (!n_valid || n < 0 || loss_type < 0 || loss_type > 1) return AA_ERR_INVALID_ARGUMENT;
  if (n == 0) return AA_OK;
  if (!value || !old_value || !target_value || !stat_loss || !clip_mask || !g_value) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_critic_loss, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream, value, old_value,
                     target_value, mask, n, value_eps_clip, loss_type, n_valid, stat_loss, clip_mask, g_value);
  return launch_status();
}

extern "C" int aa_prox_logp_approx(const float* old_logp, const float* logp, const int32_t* versions, int64_t n,
                                   int current_version, int method, float* out, void* stream) {
  if (n < 0 || method < 0 || method > 2) return AA_ERR_INVALID_ARGUMENT;
  if (n == 0) return AA_OK;
  if (!old_logp || !logp || !versions || !out) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_prox_approx, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream, old_logp, logp, versions, n,
                     current_version, method, out);
  return launch_status();
}

extern "C" int aa_kd_terms(const float* logp, const float* old_logp, const float* teacher_logp, const uint8_t* mask,
                           int64_t n, int pure_distillation, float* term, float* dterm, void* stream) {
  if (n < 0) return AA_ERR_INVALID_ARGUMENT;
  if (n == 0) return AA_OK;
  if (!logp || !teacher_logp || !mask || !term || !dterm || (pure_distillation && !old_logp))
    return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_kd_terms, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream, logp, old_logp, teacher_logp, mask,
                     n, pure_distillation ? 1 : 0, term, dterm);
  return launch_status();
}
