// Advantage pipeline of the PPO actor on gfx950: the GAE reverse scan, reward / advantage normalisation, and the
// masked moments the statistics logger asks for.  Reference: areal/trainer/ppo/actor.py:209-236 (GAE, a Python
// loop over max_seqlen), areal/utils/data.py:1378-1596 (Normalization), areal/utils/stats_tracker.py:227-285.
#include "device_utils.h"

namespace aa {
namespace adv {

constexpr int kThreads = 1024;

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

// ------------------------------------------------------------------------------------------------------------------
// GAE.  Going backwards over t = L-2 .. 0 the reference carries (nv, lg) = (next value, last advantage):
//     delta = r_t + gamma * nv - v_t;  new = delta + gamma * lambda * lg
//     nv <- nv (1 - m_t) + v_t m_t;    lg <- lg (1 - m_t) + new m_t;    adv_t = lg
// which is the affine map  nv' = a nv + e,  lg' = c nv + d lg + f  with
//     a = 1 - m, e = m v, c = m gamma, d = 1 - m + m gamma lambda, f = m (r - v).
// Affine maps compose, so a row can be cut into chunks whose composite maps are scanned in parallel.
// ------------------------------------------------------------------------------------------------------------------
struct Affine {
  float a, c, d, e, f;
};

// `first` is applied before `second`
__device__ __forceinline__ Affine compose(const Affine& first, const Affine& second) {
  Affine r;
  r.a = second.a * first.a;
  r.c = fmaf(second.c, first.a, second.d * first.c);
  r.d = second.d * first.d;
  r.e = fmaf(second.a, first.e, second.e);
  r.f = fmaf(second.c, first.e, fmaf(second.d, first.f, second.f));
  return r;
}

__device__ __forceinline__ Affine shfl_up(const Affine& x, int delta) {
  Affine r;
  r.a = __shfl_up(x.a, delta, kWave);
  r.c = __shfl_up(x.c, delta, kWave);
  r.d = __shfl_up(x.d, delta, kWave);
  r.e = __shfl_up(x.e, delta, kWave);
  r.f = __shfl_up(x.f, delta, kWave);
  return r;
}

// One workgroup per row, walking the row from its end in super-blocks of 256 x 16 positions.  A super-block is
// copied into LDS with coalesced loads; thread k then owns the k-th chunk of 16 consecutive positions counted from
// the end of the super-block (thread order = processing order), composes the maps of its chunk, an exclusive scan
// over the 256 threads (wave scan + wave totals through LDS) gives the state entering the chunk, the thread walks
// its chunk with the recurrence as written, and the results leave through LDS with coalesced stores.  Chunks are
// padded by one word in LDS so that the 64 lanes of a wave, 16 positions apart, hit different banks.
constexpr int kGaeThreads = 256;
constexpr int kGaeChunk = 16;
constexpr int kGaeBlock = kGaeThreads * kGaeChunk;                 // positions per super-block
constexpr int kGaeLds = kGaeBlock + kGaeThreads;                   // + one pad word per chunk

__device__ __forceinline__ int gae_slot(int i) { return i + i / kGaeChunk; }

__global__ __launch_bounds__(kGaeThreads) void k_gae(const float* __restrict__ rewards, const float* __restrict__ values,
                                                     const float* __restrict__ mask, const uint8_t* __restrict__ no_eos,
                                                     int64_t bs, int64_t L, float gamma, float lam,
                                                     float* __restrict__ adv, float* __restrict__ returns) {
  __shared__ float sr[kGaeLds], sv[kGaeLds], sm[kGaeLds];
  __shared__ Affine wave_tot[kGaeThreads / kWave];
  __shared__ float carry[2];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int64_t row = blockIdx.x;
  const float* r = rewards + row * L;
  const float* v = values ? values + row * L : nullptr;
  const float* m = mask + row * L;
  float* out_a = adv + row * L;
  float* out_r = returns ? returns + row * L : nullptr;
  const float v_last = v ? v[L - 1] : 0.f;
  if (tid == 0) {
    out_a[L - 1] = 0.f;
    if (out_r) out_r[L - 1] = v_last;
    carry[0] = (no_eos && no_eos[row]) ? v_last : 0.f;   // nextvalues = values[:, L-1] * seq_no_eos_mask
    carry[1] = 0.f;                                       // lastgaelam
  }
  const float gl = gamma * lam;
  const Affine ident{1.f, 0.f, 1.f, 0.f, 0.f};
  // positions 0 .. L-2, super-blocks aligned to the end: [base, base + cnt)
  for (int64_t end = L - 1; end > 0; end -= kGaeBlock) {
    const int64_t base = end > kGaeBlock ? end - kGaeBlock : 0;
    const int cnt = (int)(end - base);
    __syncthreads();  // the previous super-block has been written out; carry is visible
    for (int i = tid; i < cnt; i += kGaeThreads) {
      const int sl = gae_slot(i);
      sr[sl] = r[base + i];
      sv[sl] = v ? v[base + i] : 0.f;
      sm[sl] = m[base + i];
    }
    __syncthreads();
    // local index i = position - base; thread k owns [hi - 15, hi] with hi = cnt - 1 - 16 k (clipped at 0)
    const int hi = cnt - 1 - tid * kGaeChunk;
    const int lo = hi - kGaeChunk + 1 > 0 ? hi - kGaeChunk + 1 : 0;
    Affine x = ident;
    for (int i = hi; i >= lo; --i) {
      const int sl = gae_slot(i);
      const float mt = sm[sl], vt = sv[sl], rt = sr[sl];
      Affine e;
      e.a = 1.f - mt;
      e.e = mt * vt;
      e.c = mt * gamma;
      e.d = (1.f - mt) + mt * gl;
      e.f = mt * (rt - vt);
      x = compose(x, e);
    }
    Affine inc = x;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const Affine prev = shfl_up(inc, o);
      if (lane >= o) inc = compose(prev, inc);
    }
    if (lane == kWave - 1) wave_tot[wave] = inc;
    const float nv0 = carry[0], lg0 = carry[1];
    __syncthreads();
    Affine before = ident;  // everything processed in this super-block before this thread's chunk
    for (int w = 0; w < wave; ++w) before = compose(before, wave_tot[w]);
    Affine excl = shfl_up(inc, 1);
    if (lane == 0) excl = ident;
    before = compose(before, excl);
    float nv = fmaf(before.a, nv0, before.e);
    float lg = fmaf(before.c, nv0, fmaf(before.d, lg0, before.f));
    for (int i = hi; i >= lo; --i) {
      const int sl = gae_slot(i);
      const float mt = sm[sl], vt = sv[sl], rt = sr[sl];
      const float delta = rt + gamma * nv - vt;
      const float newlg = delta + gl * lg;
      nv = nv * (1.f - mt) + vt * mt;
      lg = lg * (1.f - mt) + newlg * mt;
      sr[sl] = lg;        // advantages
      sv[sl] = lg + vt;   // returns
    }
    if (tid == kGaeThreads - 1) {  // the last thread ends at the front of the super-block: its state carries on
      carry[0] = nv;
      carry[1] = lg;
    }
    __syncthreads();
    for (int i = tid; i < cnt; i += kGaeThreads) {
      const int sl = gae_slot(i);
      out_a[base + i] = sr[sl];
      if (out_r) out_r[base + i] = sv[sl];
    }
  }
}

// ------------------------------------------------------------------------------------------------------------------
// Normalization.  Segment 0 is the whole batch, segment 1 + g is group g (group_size rows of `inner` elements);
// rows past the last full group belong to no group (the reference leaves their mean and std at zero).
// stats[seg] = {sum(x m), sum(m), sum((x m - mean m)^2), -}
// ------------------------------------------------------------------------------------------------------------------
struct NormArgs {
  const float* x;
  const float* mask;  // nullable
  int64_t n;          // bs * inner
  int64_t seg_elems;  // group_size * inner
  int64_t n_groups;   // bs / group_size
  int64_t group_size;
  int mean_level, mean_leave1out, std_level, std_unbiased;  // levels: 0 none, 1 batch, 2 group
  float eps;
};

__device__ __forceinline__ void seg_range(const NormArgs& a, int seg, int64_t& beg, int64_t& end) {
  if (seg == 0) {
    beg = 0;
    end = a.n;
  } else {
    beg = (int64_t)(seg - 1) * a.seg_elems;
    end = beg + a.seg_elems;
  }
}

// mean of Normalization._compute_mean for one element, from the (sum, count) of its segment
__device__ __forceinline__ double level_mean(double S, double F, bool loo, bool has_mask, double xi, double mi) {
  if (loo) {
    if (F <= 1.0) return 0.0;
    if (!has_mask) return (S - xi) / (F - 1.0);
    if (mi > 0.0) {
      double den = F - mi;
      if (den < 1.0) den = 1.0;
      return (S - xi * mi) / den;
    }
    return S / F;
  }
  return F == 0.0 ? 0.0 : S / F;
}

// The mean the reference subtracts from element i.  `as_float`: the reference keeps group-level (and absent) means
// in a tensor of the dtype of x, batch-level means in float64.
__device__ __forceinline__ double mean_at(const NormArgs& a, const double4* stats, int64_t i, float xi, float mi,
                                          bool& as_float) {
  as_float = true;
  if (a.mean_level == 0) return 0.0;
  const bool has_mask = a.mask != nullptr;
  if (a.mean_level == 1) {
    as_float = false;
    return level_mean(stats[0].x, stats[0].y, a.mean_leave1out != 0, has_mask, xi, mi);
  }
  const int64_t g = i / a.seg_elems;
  if (g >= a.n_groups) return 0.0;
  if (a.group_size == 1 && a.mean_leave1out) return 0.0;
  const double4 s = stats[1 + g];
  return (double)(float)level_mean(s.x, s.y, a.mean_leave1out != 0, has_mask, xi, mi);
}

// Pass 0 accumulates (sum x m, sum m), pass 1 sum (x m - mean m)^2.  A segment is cut into `parts` equal slices, one
// workgroup each, so that the batch-wide segment fills the chip; k_norm_finish adds the slices in index order.
template <int PASS>
__global__ __launch_bounds__(kThreads) void k_norm_partial(NormArgs a, const double4* __restrict__ stats, int parts,
                                                           double2* __restrict__ partial) {
  __shared__ double smem[kThreads / kWave];
  const int seg = blockIdx.x / parts, part = blockIdx.x % parts;
  int64_t beg, end;
  seg_range(a, seg, beg, end);
  const int64_t per = (end - beg + parts - 1) / parts;
  const int64_t pb = beg + part * per;
  const int64_t pe = pb + per < end ? pb + per : end;
  double s = 0.0, f = 0.0;
  for (int64_t i = pb + threadIdx.x; i < pe; i += kThreads) {
    const float xi = a.x[i];
    const float mi = a.mask ? a.mask[i] : 1.f;
    if (PASS == 0) {
      s += (double)xi * (double)mi;
      f += (double)mi;
    } else {
      bool as_float;
      const double mean = mean_at(a, stats, i, xi, mi, as_float);
      const double d = (double)xi * (double)mi - mean * (double)mi;  // x_masked - mean * mask
      s += d * d;
    }
  }
  s = block_sum<double>(s, smem);
  if (PASS == 0) f = block_sum<double>(f, smem);
  if (threadIdx.x == 0) partial[blockIdx.x] = make_double2(s, f);
}

// one wave per segment: lane l adds slices l, l + 64, ... in order, then a fixed butterfly adds the lanes
template <int PASS>
__global__ __launch_bounds__(kWave) void k_norm_finish(const double2* __restrict__ partial, int parts, int segs,
                                                       double4* __restrict__ stats) {
  const int seg = blockIdx.x;
  double s = 0.0, f = 0.0;
  for (int p = threadIdx.x; p < parts; p += kWave) {
    const double2 v = partial[seg * parts + p];
    s += v.x;
    f += v.y;
  }
  s = wave_sum(s);
  f = wave_sum(f);
  if (threadIdx.x == 0) {
    if (PASS == 0) stats[seg] = make_double4(s, f, 0.0, 0.0);
    else stats[seg].z = s;
  }
}

__device__ __forceinline__ double level_std(double Q, double F, bool unbiased) {
  if (unbiased) return F <= 1.0 ? 1.0 : sqrt(Q / (F - 1.0));
  return F == 0.0 ? 1.0 : sqrt(Q / F);
}

__global__ __launch_bounds__(256) void k_norm_apply(NormArgs a, const double4* __restrict__ stats,
                                                    float* __restrict__ out) {
  const bool has_mask = a.mask != nullptr;
  const bool passthrough = has_mask && stats[0].y == 0.0;  // nothing active: the input comes back unchanged
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n; i += (int64_t)gridDim.x * blockDim.x) {
    const float xi = a.x[i];
    if (passthrough) {
      out[i] = xi;
      continue;
    }
    const float mi = has_mask ? a.mask[i] : 1.f;
    bool mean_f;
    const double mean = mean_at(a, stats, i, xi, mi, mean_f);
    // x - mean, then * mask, in the precision the reference's tensors have at that point
    double cen;
    if (mean_f) {
      float c = xi - (float)mean;
      if (has_mask) c *= mi;
      cen = (double)c;
    } else {
      cen = (double)xi - mean;
      if (has_mask) cen *= (double)mi;
    }
    double sd;
    bool std_f = true;
    float eps = a.eps;
    if (a.std_level == 0) {
      sd = 1.0;
      eps = 0.f;
    } else if (a.std_level == 1) {
      sd = level_std(stats[0].z, stats[0].y, a.std_unbiased != 0);
      std_f = false;
    } else {
      const int64_t g = i / a.seg_elems;
      if (g >= a.n_groups) sd = 0.0;
      else if (a.group_size == 1 && a.std_unbiased) sd = 1.0;
      else sd = (double)(float)level_std(stats[1 + g].z, stats[1 + g].y, a.std_unbiased != 0);
    }
    float r;
    if (std_f && mean_f) {
      r = (float)cen / ((float)sd + eps);
    } else if (std_f) {
      r = (float)(cen / (double)((float)sd + eps));
    } else {
      r = (float)(cen / (sd + (double)eps));
    }
    out[i] = r;
  }
}

// ------------------------------------------------------------------------------------------------------------------
// KL-regularised token rewards (actor.py:182-207): kl_rewards = -kl_ctl * KL(old_logp * m, ref_logp * m) with the
// k1 / k2 / k3 estimators clamped to [-10, 10] (data.py:1620-1656), then per sequence the reward at position
// seqlen - 1 is cleared and the sequence's scalar reward is added at position max(seqlen - 2, 0).
// ------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_kl_rewards(const float* __restrict__ old_logp, const float* __restrict__ ref_logp,
                                                    const float* __restrict__ mask, const int64_t* __restrict__ seqlens,
                                                    const float* __restrict__ score, int64_t bs, int64_t L,
                                                    float kl_ctl, int estimator, int mask_no_eos_with_zero,
                                                    float* __restrict__ rewards, float* __restrict__ kl_rewards) {
  const int64_t n = bs * L;
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const int64_t b = i / L, t = i - b * L;
    const float m = mask[i];
    const float lo = old_logp[i] * m, lr = (ref_logp ? ref_logp[i] : 0.f) * m;
    float d = lo - lr;
    if (estimator == 1) d = d * d / 2.0f;
    else if (estimator == 2) { d = -d; d = expf(d) - 1.f - d; }
    d = (d != d) ? d : fminf(fmaxf(d, -10.f), 10.f);  // torch.clamp keeps NaN
    const float kr = -kl_ctl * d;
    kl_rewards[i] = kr;
    const int64_t sl = seqlens[b];
    int64_t last = sl - 1;
    if (last < 0) last += L;  // Python's negative index, as the reference's fancy indexing does
    int64_t put = sl - 2;
    if (put < 0) put = 0;
    float r = (t == last) ? 0.f : kr;
    if (t == put) {
      const bool no_eos = sl == L;
      r += (mask_no_eos_with_zero && no_eos) ? 0.f : score[b];
    }
    rewards[i] = r;
  }
}

// ------------------------------------------------------------------------------------------------------------------
// Length penalty on the sequence rewards (reward_overlong_penalty, areal/utils/functional/functional.py:782-803):
// with len_b = long(sum of the row's loss mask), rewards[b] += min(-(len_b - (max_len - overlong)) / overlong * factor, 0),
// the quotient and the product in float32 as the reference's tensor arithmetic.  One workgroup per sequence.
// ------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_overlong_penalty(float* __restrict__ rewards, const float* __restrict__ mask,
                                                          int64_t L, int overlong_tokens, float factor,
                                                          int64_t max_response_length) {
  __shared__ float part[4];
  const int64_t b = blockIdx.x;
  float s = 0.f;
  for (int64_t t = threadIdx.x; t < L; t += 256) s += mask[b * L + t];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, kWave);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    const int64_t len = (int64_t)((part[0] + part[1]) + (part[2] + part[3]));
    const int64_t exceed = len - (max_response_length - overlong_tokens);
    const float pen = ((float)(-exceed) / (float)overlong_tokens) * factor;
    if (pen < 0.f) rewards[b] += pen;
  }
}

// ------------------------------------------------------------------------------------------------------------------
// Masked moments of up to kMaxTensors per-token tensors under one mask: out[k] = {sum, min, max, count}
// (min = +inf, max = -inf when nothing is selected).  One workgroup per tensor, fixed summation order.
// ------------------------------------------------------------------------------------------------------------------
constexpr int kMaxTensors = 16;
struct MomentArgs {
  const float* v[kMaxTensors];
};

__global__ __launch_bounds__(kThreads) void k_masked_moments(MomentArgs a, const uint8_t* __restrict__ mask, int64_t n,
                                                             float* __restrict__ out) {
  __shared__ double smem_d[kThreads / kWave];
  __shared__ float smem_lo[kThreads / kWave], smem_hi[kThreads / kWave];
  const float* v = a.v[blockIdx.x];
  double s = 0.0, c = 0.0;
  float lo = __builtin_inff(), hi = -__builtin_inff();
  for (int64_t i = threadIdx.x; i < n; i += kThreads) {
    if (mask[i] != 0) {
      const float x = v[i];
      s += (double)x;
      c += 1.0;
      lo = fminf(lo, x);
      hi = fmaxf(hi, x);
    }
  }
  s = block_sum<double>(s, smem_d);
  c = block_sum<double>(c, smem_d);
  lo = wave_min(lo);
  hi = wave_max(hi);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) {
    smem_lo[wave] = lo;
    smem_hi[wave] = hi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kThreads / kWave; ++w) {
      lo = fminf(lo, smem_lo[w]);
      hi = fmaxf(hi, smem_hi[w]);
    }
    float* o = out + 4 * blockIdx.x;
    o[0] = (float)s;
    o[1] = lo;
    o[2] = hi;
    o[3] = (float)c;
  }
}

// ------------------------------------------------------------------------------------------------------------------
// masked_normalization (areal/utils/functional/functional.py:16-53): every row of an [R, C] view is whitened by
// the mean and the E[x^2] - E[x]^2 variance of its masked values.  A row is cut into `parts` slices, one workgroup
// each; the second launch adds the slices of its row in a fixed order and writes the result.
// ------------------------------------------------------------------------------------------------------------------
struct MnPartial {
  double s, q, f;
};

__host__ __device__ inline int mn_parts(int64_t R, int64_t C) {
  int64_t parts = (C + 8191) / 8192;                     // at least 8192 values per workgroup
  const int64_t want = (1024 + R - 1) / (R > 0 ? R : 1); // about 1024 workgroups in all
  if (parts > want) parts = want;
  if (parts > 256) parts = 256;
  return parts < 1 ? 1 : (int)parts;
}

__device__ __forceinline__ void mn_slice(int64_t C, int parts, int part, int64_t& b, int64_t& e) {
  const int64_t per = (C + parts - 1) / parts;
  b = (int64_t)part * per;
  e = b + per < C ? b + per : C;
  if (b > e) b = e;
}

__global__ __launch_bounds__(kThreads) void k_mn_partial(const float* __restrict__ x, const float* __restrict__ mask,
                                                         int64_t C, int parts, MnPartial* __restrict__ partial) {
  __shared__ double smem[kThreads / kWave];
  const int64_t row = blockIdx.x / parts;
  int64_t b, e;
  mn_slice(C, parts, blockIdx.x % parts, b, e);
  const float* xr = x + row * C;
  const float* mr = mask ? mask + row * C : nullptr;
  double s = 0.0, q = 0.0, f = 0.0;
  for (int64_t i = b + threadIdx.x; i < e; i += kThreads) {
    const double m = mr ? (double)mr[i] : 1.0;
    const double v = (double)xr[i] * m;
    s += v;
    q += v * v;
    f += m;
  }
  s = block_sum<double>(s, smem);
  q = block_sum<double>(q, smem);
  f = block_sum<double>(f, smem);
  if (threadIdx.x == 0) partial[blockIdx.x] = MnPartial{s, q, f};
}

__global__ __launch_bounds__(kThreads) void k_mn_apply(const float* __restrict__ x, const float* __restrict__ mask,
                                                       int64_t C, int parts, const MnPartial* __restrict__ partial,
                                                       int unbiased, double eps, float* __restrict__ out) {
  __shared__ double stat[2];
  const int64_t row = blockIdx.x / parts;
  if (threadIdx.x < kWave) {  // parts <= 256: lane l adds slices l, l + 64, ... in order, then a fixed butterfly
    double s = 0.0, q = 0.0, f = 0.0;
    for (int p = threadIdx.x; p < parts; p += kWave) {
      const MnPartial v = partial[row * parts + p];
      s += v.s;
      q += v.q;
      f += v.f;
    }
    s = wave_sum(s);
    q = wave_sum(q);
    f = wave_sum(f);
    if (threadIdx.x == 0) {
      const double mean = s / f;
      double var = q / f - mean * mean;
      if (unbiased) var *= f / (f - 1.0);
      stat[0] = mean;
      stat[1] = sqrt(var) + eps;
    }
  }
  __syncthreads();
  const double mean = stat[0], den = stat[1];
  int64_t b, e;
  mn_slice(C, parts, blockIdx.x % parts, b, e);
  const float* xr = x + row * C;
  const float* mr = mask ? mask + row * C : nullptr;
  float* o = out + row * C;
  for (int64_t i = b + threadIdx.x; i < e; i += kThreads) {
    const double v = (double)xr[i] * (mr ? (double)mr[i] : 1.0);
    o[i] = (float)((v - mean) / den);
  }
}

// KLEstimator (areal/utils/data.py:1598-1656) per element: k1 = d, k2 = d^2 / 2, k3 = exp(-d) - 1 + d with
// d = logp - logp_base, optionally clamped to [-10, 10].
__global__ __launch_bounds__(256) void k_kl_estimate(const float* __restrict__ logp, const float* __restrict__ base,
                                                     int64_t n, int estimator, int clamp, float* __restrict__ out) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    float d = logp[i] - base[i];
    if (estimator == 1) d = d * d / 2.0f;
    else if (estimator == 2) { d = -d; d = expf(d) - 1.f - d; }
    if (clamp) d = (d != d) ? d : fminf(fmaxf(d, -10.f), 10.f);
    out[i] = d;
  }
}

}  // namespace adv
}  // namespace aa

using namespace aa;
using namespace aa::adv;

extern "C" int aa_gae(const float* rewards, const float* values, const float* loss_mask, const uint8_t* seq_no_eos,
                      int64_t bs, int64_t L, float discount, float gae_lambda, float* advantages, float* returns,
                      void* stream) {
  if (bs < 0 || L < 1) return AA_ERR_INVALID_ARGUMENT;
  if (bs == 0) return AA_OK;
  if (!rewards || !loss_mask || !advantages) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_gae, dim3((unsigned)bs), dim3(kGaeThreads), 0, (hipStream_t)stream, rewards, values, loss_mask,
                     seq_no_eos, bs, L, discount, gae_lambda, advantages, returns);
  return launch_status();
}

static int norm_parts(int64_t n) {
  int64_t p = (n + 8191) / 8192;
  return (int)(p < 1 ? 1 : (p > 256 ? 256 : p));
}

extern "C" int64_t aa_normalize_scratch_bytes(int64_t bs, int64_t inner, int64_t group_size) {
  if (bs < 0 || inner < 1 || group_size < 1) return -1;
  const int64_t segs = 1 + bs / group_size;
  return segs * (int64_t)sizeof(double4) + segs * norm_parts(bs * inner) * (int64_t)sizeof(double2);
}

extern "C" int aa_normalize(const float* x, const float* loss_mask, int64_t bs, int64_t inner,
                            const aa_norm_params* params, float* out, void* scratch, int64_t scratch_bytes,
                            void* stream) {
  if (!x || !out || !params || !scratch || bs < 0 || inner < 1) return AA_ERR_INVALID_ARGUMENT;
  const aa_norm_params& p = *params;
  if (p.mean_level < 0 || p.mean_level > 2 || p.std_level < 0 || p.std_level > 2) return AA_ERR_INVALID_ARGUMENT;
  const bool grouped = p.mean_level == 2 || p.std_level == 2;
  if (grouped && p.group_size < 1) return AA_ERR_INVALID_ARGUMENT;
  if (bs == 0) return AA_OK;
  const int64_t gs = grouped ? p.group_size : bs;
  const int64_t n_groups = grouped ? bs / gs : 0;
  const int64_t segs = 1 + n_groups;
  const int parts = norm_parts(bs * inner);
  if (segs * parts > (int64_t)0x7fffffff) return AA_ERR_UNSUPPORTED;
  const int64_t need = segs * (int64_t)sizeof(double4) + segs * parts * (int64_t)sizeof(double2);
  if (scratch_bytes < need || (((uintptr_t)scratch) & 31)) return AA_ERR_INVALID_ARGUMENT;
  NormArgs a{x, loss_mask, bs * inner, gs * inner, n_groups, gs, p.mean_level, p.mean_leave1out, p.std_level,
             p.std_unbiased, p.eps};
  hipStream_t st = (hipStream_t)stream;
  double4* stats = (double4*)scratch;
  double2* partial = (double2*)(stats + segs);
  const unsigned fin = (unsigned)segs;
  hipLaunchKernelGGL(k_norm_partial<0>, dim3((unsigned)(segs * parts)), dim3(kThreads), 0, st, a, stats, parts, partial);
  hipLaunchKernelGGL(k_norm_finish<0>, dim3(fin), dim3(kWave), 0, st, partial, parts, (int)segs, stats);
  if (p.std_level != 0) {
    hipLaunchKernelGGL(k_norm_partial<1>, dim3((unsigned)(segs * parts)), dim3(kThreads), 0, st, a, stats, parts,
                       partial);
    hipLaunchKernelGGL(k_norm_finish<1>, dim3(fin), dim3(kWave), 0, st, partial, parts, (int)segs, stats);
  }
  int64_t blocks = (a.n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(k_norm_apply, dim3((unsigned)blocks), dim3(256), 0, st, a, stats, out);
  return launch_status();
}

extern "C" int aa_masked_moments(const float* const* values, int n_tensors, const uint8_t* mask, int64_t n,
                                 float* out, void* stream) {
  if (!values || !out || n_tensors < 0 || n_tensors > kMaxTensors || n < 0 || (n > 0 && !mask))
    return AA_ERR_INVALID_ARGUMENT;
  if (n_tensors == 0) return AA_OK;
  MomentArgs a{};
  for (int k = 0; k < n_tensors; ++k) {
    if (!values[k] && n > 0) return AA_ERR_INVALID_ARGUMENT;
    a.v[k] = values[k];
  }
  hipLaunchKernelGGL(k_masked_moments, dim3((unsigned)n_tensors), dim3(kThreads), 0, (hipStream_t)stream, a, mask, n,
                     out);
  return launch_status();
}

extern "C" int aa_kl_rewards(const float* old_logp, const float* ref_logp, const float* loss_mask,
                             const int64_t* seqlens, const float* reward_score, int64_t bs, int64_t L, float kl_ctl,
                             int estimator, int mask_no_eos_with_zero, float* rewards, float* kl_rewards,
                             void* stream) {
  if (bs < 0 || L < 1 || estimator < 0 || estimator > 2) return AA_ERR_INVALID_ARGUMENT;
  if (bs == 0) return AA_OK;
  if (!old_logp || !loss_mask || !seqlens || !reward_score || !rewards || !kl_rewards) return AA_ERR_INVALID_ARGUMENT;
  int64_t blocks = (bs * L + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(k_kl_rewards, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, old_logp, ref_logp,
                     loss_mask, seqlens, reward_score, bs, L, kl_ctl, estimator, mask_no_eos_with_zero, rewards,
                     kl_rewards);
  return launch_status();
}

extern "C" int aa_overlong_penalty(float* rewards, const float* loss_mask, int64_t bs, int64_t L, int overlong_tokens,
                                   float overlong_penalty_factor, int64_t max_response_length, void* stream) {
  if (bs < 0 || L < 1 || overlong_tokens == 0) return AA_ERR_INVALID_ARGUMENT;
  if (bs == 0) return AA_OK;
  if (!rewards || !loss_mask) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_overlong_penalty, dim3((unsigned)bs), dim3(256), 0, (hipStream_t)stream, rewards, loss_mask, L,
                     overlong_tokens, overlong_penalty_factor, max_response_length);
  return launch_status();
}

extern "C" int64_t aa_masked_normalization_scratch_bytes(int64_t rows, int64_t cols) {
  if (rows < 0 || cols < 0) return -1;
  return rows * mn_parts(rows, cols) * (int64_t)sizeof(MnPartial);
}

extern "C" int aa_masked_normalization(const float* x, const float* mask, int64_t rows, int64_t cols, int unbiased,
                                       double eps, float* out, void* scratch, int64_t scratch_bytes, void* stream) {
  if (rows < 0 || cols < 0) return AA_ERR_INVALID_ARGUMENT;
  if (rows == 0 || cols == 0) return AA_OK;
  const int parts = mn_parts(rows, cols);
  if (!x || !out || !scratch || scratch_bytes < rows * parts * (int64_t)sizeof(MnPartial) ||
      rows * parts > 0x7fffffff)
    return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  MnPartial* partial = (MnPartial*)scratch;
  const unsigned grid = (unsigned)(rows * parts);
  hipLaunchKernelGGL(k_mn_partial, dim3(grid), dim3(kThreads), 0, st, x, mask, cols, parts, partial);
  hipLaunchKernelGGL(k_mn_apply, dim3(grid), dim3(kThreads), 0, st, x, mask, cols, parts, partial, unbiased, eps, out);
  return launch_status();
}

extern "C" int aa_kl_estimate(const float* logp, const float* logp_base, int64_t n, int estimator, int apply_clamp,
                              float* out, void* stream) {
  if (n < 0 || estimator < 0 || estimator > 2) return AA_ERR_INVALID_ARGUMENT;
  if (n == 0) return AA_OK;
  if (!logp || !logp_base || !out) return AA_ERR_INVALID_ARGUMENT;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(k_kl_estimate, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, logp, logp_base, n,
                     estimator, apply_clamp ? 1 : 0, out);
  return launch_status();
}
