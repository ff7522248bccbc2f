// Direct preference optimisation on a packed batch of interleaved (chosen, rejected) sequences on gfx950:
// per-sequence fp64 sums of the response log-probabilities under the mask shifted to next-token alignment, the
// per-pair preference loss, and the gradient back to the per-token log-probabilities.
// Reference: areal/utils/functional/functional.py:641-703 (dpo_pair_logratios, dpo_preference_loss) and
// areal/trainer/dpo/dpo_engine.py:22-28, 147-213 (_dpo_valid_pairs, compute_dpo_loss).
#include "device_utils.h"

namespace aa {
namespace dpo {

constexpr int kThreads = 256;       // per-pair kernels
constexpr int kSeqThreads = 1024;   // per-sequence kernels: one workgroup walks one sequence
constexpr int kMaxWaves = kSeqThreads / kWave;

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// Sum over the workgroup in a fixed order: xor tree inside each wave, wave totals added in wave order.
__device__ __forceinline__ double block_sum_f64(double v, double* smem) {
  v = wave_sum_f64(v);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  double r = smem[0];
  for (int w = 1; w < (int)(blockDim.x / kWave); ++w) r += smem[w];
  return r;
}

// Sequence s covers tokens [b, e) of the packed batch.  Position t predicts token t + 1, so it counts when
// loss_mask[t + 1] is set, and the last position of a sequence never counts (functional.py:663-667).
__device__ __forceinline__ void seq_range(const int32_t* cu, int64_t s, int64_t T, int64_t& b, int64_t& e) {
  b = cu[s];
  e = cu[s + 1];
  if (b < 0) b = 0;
  if (e > T) e = T;
}

// One workgroup per sequence.  The product logp * mask is formed in fp32 as the reference forms it (exact for a
// finite logp, NaN for a non-finite one under a cleared mask, as there), then widened and summed in fp64.
__global__ __launch_bounds__(kSeqThreads) void k_seq_sums(const float* __restrict__ logp, const float* __restrict__ ref,
                                                       const uint8_t* __restrict__ mask,
                                                       const int32_t* __restrict__ cu, int64_t T,
                                                       double* __restrict__ policy_sums, double* __restrict__ ref_sums,
                                                       double* __restrict__ lens) {
  __shared__ double smem[3][kMaxWaves];
  const int64_t s = blockIdx.x;
  int64_t b, e;
  seq_range(cu, s, T, b, e);
  double ap = 0.0, ar = 0.0, an = 0.0;
#pragma unroll 4
  for (int64_t t = b + threadIdx.x; t < e; t += kSeqThreads) {
    const float m = (t + 1 < e && mask[t + 1]) ? 1.f : 0.f;
    ap += (double)(logp[t] * m);
    ar += (double)(ref[t] * m);
    an += (double)m;
  }
  // the three sums share one pass through LDS: wave totals first, then thread k adds up column k in wave order
  ap = wave_sum_f64(ap);
  ar = wave_sum_f64(ar);
  an = wave_sum_f64(an);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) {
    smem[0][wave] = ap;
    smem[1][wave] = ar;
    smem[2][wave] = an;
  }
  __syncthreads();
  if (threadIdx.x < 3) {
    double r = smem[threadIdx.x][0];
    for (int w = 1; w < kMaxWaves; ++w) r += smem[threadIdx.x][w];
    (threadIdx.x == 0 ? policy_sums : threadIdx.x == 1 ? ref_sums : lens)[s] = r;
  }
}

// d logp[t] = (float)(g[s(t)] * scale) * shifted_mask[t].  Workgroup n_seqs clears the tokens no sequence covers.
__global__ __launch_bounds__(kSeqThreads) void k_seq_sums_bwd(const double* __restrict__ g, const float* __restrict__ scale,
                                                           const uint8_t* __restrict__ mask,
                                                           const int32_t* __restrict__ cu, int64_t n_seqs, int64_t T,
                                                           float* __restrict__ dlogp) {
  const int64_t s = blockIdx.x;
  if (s == n_seqs) {
    int64_t first = cu[0], last = cu[n_seqs];
    if (first > T) first = T;
    if (last < 0) last = 0;
    for (int64_t t = threadIdx.x; t < first; t += kSeqThreads) dlogp[t] = 0.f;
    for (int64_t t = last + threadIdx.x; t < T; t += kSeqThreads) dlogp[t] = 0.f;
    return;
  }
  int64_t b, e;
  seq_range(cu, s, T, b, e);
  const float gs = (float)(scale ? g[s] * (double)scale[0] : g[s]);
#pragma unroll 4
  for (int64_t t = b + threadIdx.x; t < e; t += kSeqThreads) {
    const float m = (t + 1 < e && mask[t + 1]) ? 1.f : 0.f;
    dlogp[t] = gs * m;
  }
}

// -logsigmoid(z) = -min(z, 0) + log1p(exp(-|z|)) and its derivative -sigmoid(-z), both in fp32.
__device__ __forceinline__ void neg_logsigmoid(float z, float& loss, float& dz) {
  const float en = expf(-fabsf(z));
  loss = -fminf(z, 0.f) + log1pf(en);
  // sigmoid(-z) = 1 / (1 + exp(z)): en / (1 + en) for z >= 0, 1 / (1 + en) for z < 0
  dz = -((z >= 0.f) ? en / (1.f + en) : 1.f / (1.f + en));
}

// loss_type 0: -logsigmoid(beta * x); 1: (x - 1 / (2 beta))^2.  dloss = d loss / d x.
__device__ __forceinline__ void preference(float x, double beta, int loss_type, float& loss, float& dloss) {
  if (loss_type == 0) {
    const float bf = (float)beta;
    float dz;
    neg_logsigmoid(bf * x, loss, dz);
    dloss = bf * dz;
  } else {
    const float c = (float)(1.0 / (2.0 * beta));
    const float d = x - c;
    loss = d * d;
    dloss = 2.f * d;
  }
}

__global__ __launch_bounds__(kThreads) void k_preference_loss(const float* __restrict__ x, int64_t n, double beta,
                                                              int loss_type, float* __restrict__ loss,
                                                              float* __restrict__ dloss) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n) return;
  float l, d;
  preference(x[i], beta, loss_type, l, d);
  loss[i] = l;
  if (dloss) dloss[i] = d;
}

// The tail of compute_dpo_loss in one workgroup: per pair the validity test (both sequences non-empty), the logit
// in fp64 from the per-sequence sums, the loss in fp32, the implicit rewards, and d mean_loss / d policy_sums.
__global__ __launch_bounds__(kThreads) void k_pair_loss(const double* __restrict__ policy_sums,
                                                        const double* __restrict__ ref_sums,
                                                        const double* __restrict__ lens,
                                                        const int32_t* __restrict__ cu, int64_t n_pairs, double beta,
                                                        int loss_type, float* __restrict__ loss_mean,
                                                        int32_t* __restrict__ n_valid, float* __restrict__ pair_loss,
                                                        float* __restrict__ chosen_reward,
                                                        float* __restrict__ rejected_reward,
                                                        uint8_t* __restrict__ valid, double* __restrict__ g_seq) {
  __shared__ double smem[kThreads / kWave];
  double acc = 0.0, cnt = 0.0;
  for (int64_t p = threadIdx.x; p < n_pairs; p += kThreads) {
    const int64_t c = 2 * p, r = 2 * p + 1;
    const bool ok = cu[c + 1] != cu[c] && cu[r + 1] != cu[r];
    float l = 0.f, cr = 0.f, rr = 0.f;
    double gc = 0.0, gr = 0.0;
    if (ok) {
      const double dc = policy_sums[c] - ref_sums[c], dr = policy_sums[r] - ref_sums[r];
      double x, wc = 1.0, wr = 1.0;
      if (loss_type == 1) {
        wc = 1.0 / fmax(lens[c], 1.0);
        wr = 1.0 / fmax(lens[r], 1.0);
        x = dc / fmax(lens[c], 1.0) - dr / fmax(lens[r], 1.0);
      } else {
        x = (policy_sums[c] - policy_sums[r]) - (ref_sums[c] - ref_sums[r]);
      }
      float dl;
      preference((float)x, beta, loss_type, l, dl);
      gc = (double)dl * wc;
      gr = -(double)dl * wr;
      cr = (float)(beta * dc);
      rr = (float)(beta * dr);
      acc += (double)l;
      cnt += 1.0;
    }
    pair_loss[p] = l;
    chosen_reward[p] = cr;
    rejected_reward[p] = rr;
    valid[p] = ok ? 1 : 0;
    g_seq[c] = gc;
    g_seq[r] = gr;
  }
  acc = block_sum_f64(acc, smem);
  cnt = block_sum_f64(cnt, smem);
  const double inv = cnt > 0.0 ? 1.0 / cnt : 0.0;
  // every thread rescales the entries it wrote itself
  for (int64_t p = threadIdx.x; p < n_pairs; p += kThreads) {
    g_seq[2 * p] *= inv;
    g_seq[2 * p + 1] *= inv;
  }
  if (threadIdx.x == 0) {
    loss_mean[0] = (float)(acc * inv);
    n_valid[0] = (int32_t)cnt;
  }
}

// both sequences of pair p are non-empty (rw_engine.py:20-22) and their last tokens lie inside the score array
__device__ __forceinline__ bool rw_pair_ok(const int32_t* cu, int64_t p, int64_t T) {
  const int64_t b = cu[2 * p], ec = cu[2 * p + 1], er = cu[2 * p + 2];
  return ec != b && er != ec && ec >= 1 && er >= 1 && ec <= T && er <= T;
}

// Reward-model loss (areal/trainer/rw/rw_engine.py:115-146): the score of a sequence is the one at its last token;
// per valid pair -logsigmoid(score_chosen - score_rejected), mean over the valid pairs.  One workgroup: it first
// clears the gradient of every token, then writes the two entries of each valid pair.
__global__ __launch_bounds__(kSeqThreads) void k_rw_pair_loss(const float* __restrict__ scores, int64_t T,
                                                              const int32_t* __restrict__ cu, int64_t n_pairs,
                                                              float* __restrict__ loss_mean,
                                                              int32_t* __restrict__ n_valid,
                                                              float* __restrict__ pair_loss,
                                                              float* __restrict__ pos_score,
                                                              float* __restrict__ neg_score,
                                                              uint8_t* __restrict__ valid,
                                                              float* __restrict__ g_scores) {
  __shared__ double smem[kMaxWaves];
  if (g_scores) {
    for (int64_t t = threadIdx.x; t < T; t += kSeqThreads) g_scores[t] = 0.f;
    __syncthreads();
  }
  // pass 1: the number of valid pairs (the gradient of a pair is 1 / that number times its own derivative)
  double cnt = 0.0;
  for (int64_t p = threadIdx.x; p < n_pairs; p += kSeqThreads) cnt += rw_pair_ok(cu, p, T) ? 1.0 : 0.0;
  cnt = block_sum_f64(cnt, smem);
  const float inv = cnt > 0.0 ? (float)(1.0 / cnt) : 0.f;
  double acc = 0.0;
  for (int64_t p = threadIdx.x; p < n_pairs; p += kSeqThreads) {
    const int64_t ec = cu[2 * p + 1], er = cu[2 * p + 2];
    const bool ok = rw_pair_ok(cu, p, T);
    float l = 0.f, sc = 0.f, sr = 0.f;
    if (ok) {
      sc = scores[ec - 1];
      sr = scores[er - 1];
      float dl;
      neg_logsigmoid(sc - sr, l, dl);
      acc += (double)l;
      if (g_scores) {
        g_scores[ec - 1] = dl * inv;
        g_scores[er - 1] = -dl * inv;
      }
    }
    pair_loss[p] = l;
    pos_score[p] = sc;
    neg_score[p] = sr;
    valid[p] = ok ? 1 : 0;
  }
  acc = block_sum_f64(acc, smem);
  if (threadIdx.x == 0) {
    loss_mean[0] = (float)(acc * (double)inv);
    n_valid[0] = (int32_t)cnt;
  }
}

}  // namespace dpo
}  // namespace aa

using namespace aa::dpo;

extern "C" int aa_dpo_seq_sums(const float* logp, const float* ref_logp, const uint8_t* loss_mask,
                               const int32_t* cu_seqlens, int64_t n_seqs, int64_t T, double* policy_sums,
                               double* ref_sums, double* completion_lens, void* stream) {
  if (n_seqs < 0 || T < 0 || n_seqs > 0x7fffffff) return AA_ERR_INVALID_ARGUMENT;
  if (n_seqs == 0) return AA_OK;
  if (!cu_seqlens || !policy_sums || !ref_sums || !completion_lens) return AA_ERR_INVALID_ARGUMENT;
  if (T > 0 && (!logp || !ref_logp || !loss_mask)) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_seq_sums, dim3((unsigned)n_seqs), dim3(kSeqThreads), 0, (hipStream_t)stream, logp, ref_logp,
                     loss_mask, cu_seqlens, T, policy_sums, ref_sums, completion_lens);
  return hipGetLastError() == hipSuccess ? AA_OK : AA_ERR_LAUNCH;
}

extern "C" int aa_dpo_seq_sums_bwd(const double* g_policy_sums, const float* scale, const uint8_t* loss_mask,
                                   const int32_t* cu_seqlens, int64_t n_seqs, int64_t T, float* d_logp,
                                   void* stream) {
  if (n_seqs < 0 || T < 0 || n_seqs >= 0x7fffffff) return AA_ERR_INVALID_ARGUMENT;
  if (T == 0) return AA_OK;
  if (!loss_mask || !cu_seqlens || !d_logp || (n_seqs > 0 && !g_policy_sums)) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_seq_sums_bwd, dim3((unsigned)n_seqs + 1), dim3(kSeqThreads), 0, (hipStream_t)stream,
                     g_policy_sums, scale, loss_mask, cu_seqlens, n_seqs, T, d_logp);
  return hipGetLastError() == hipSuccess ? AA_OK : AA_ERR_LAUNCH;
}

extern "C" int aa_dpo_preference_loss(const float* logits, int64_t n, double beta, int loss_type, float* loss,
                                      float* dloss, void* stream) {
  if (n < 0 || (loss_type != 0 && loss_type != 1)) return AA_ERR_INVALID_ARGUMENT;
  if (n == 0) return AA_OK;
  if (!logits || !loss) return AA_ERR_INVALID_ARGUMENT;
  const int64_t grid = (n + kThreads - 1) / kThreads;
  if (grid > 0x7fffffff) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_preference_loss, dim3((unsigned)grid), dim3(kThreads), 0, (hipStream_t)stream, logits, n, beta,
                     loss_type, loss, dloss);
  return hipGetLastError() == hipSuccess ? AA_OK : AA_ERR_LAUNCH;
}

extern "C" int aa_dpo_pair_loss(const double* policy_sums, const double* ref_sums, const double* completion_lens,
                                const int32_t* cu_seqlens, int64_t n_pairs, double beta, int loss_type,
                                float* loss_mean, int32_t* n_valid, float* pair_loss, float* chosen_reward,
                                float* rejected_reward, uint8_t* valid, double* g_policy_sums, void* stream) {
  if (n_pairs < 0 || (loss_type != 0 && loss_type != 1)) return AA_ERR_INVALID_ARGUMENT;
  if (!loss_mean || !n_valid) return AA_ERR_INVALID_ARGUMENT;
  if (n_pairs > 0 && (!policy_sums || !ref_sums || !completion_lens || !cu_seqlens || !pair_loss || !chosen_reward ||
                      !rejected_reward || !valid || !g_policy_sums))
    return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_pair_loss, dim3(1), dim3(kThreads), 0, (hipStream_t)stream, policy_sums, ref_sums,
                     completion_lens, cu_seqlens, n_pairs, beta, loss_type, loss_mean, n_valid, pair_loss,
                     chosen_reward, rejected_reward, valid, g_policy_sums);
  return hipGetLastError() == hipSuccess ? AA_OK : AA_ERR_LAUNCH;
}

extern "C" int aa_rw_pair_loss(const float* scores, int64_t T, const int32_t* cu_seqlens, int64_t n_pairs,
                               float* loss_mean, int32_t* n_valid, float* pair_loss, float* pos_score,
                               float* neg_score, uint8_t* valid, float* g_scores, void* stream) {
  if (T < 0 || n_pairs < 0 || !loss_mean || !n_valid) return AA_ERR_INVALID_ARGUMENT;
  if (n_pairs > 0 && (!cu_seqlens || !pair_loss || !pos_score || !neg_score || !valid)) return AA_ERR_INVALID_ARGUMENT;
  if (T > 0 && !scores) return AA_ERR_INVALID_ARGUMENT;
  hipLaunchKernelGGL(k_rw_pair_loss, dim3(1), dim3(kSeqThreads), 0, (hipStream_t)stream, scores, T, cu_seqlens, n_pairs,
                     loss_mean, n_valid, pair_loss, pos_score, neg_score, valid, g_scores);
  return hipGetLastError() == hipSuccess ? AA_OK : AA_ERR_LAUNCH;
}
