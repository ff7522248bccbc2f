// Supervised fine-tuning loss over a packed batch on gfx950: the masked mean negative log-likelihood with its
// gradient, and the per-sequence mean log-prob / perplexity the trainer logs, without a host loop over sequences.
// Reference: compute_packed_sft_loss, areal/trainer/sft/lm_engine.py:81-131.
#include "device_utils.h"

namespace aa {
namespace sft {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / kWave;

// Workgroup b < n_seqs covers sequence b = [cu[b], cu[b+1]); workgroup n_seqs covers the tokens no sequence covers
// (before cu[0] and after cu[n_seqs]; all of them when there is no cu_seqlens).  Each writes the fp64 sum of the
// selected log-probs and their number for its range, and the per-token outputs of its range.
__global__ __launch_bounds__(kThreads) void k_seq(const float* __restrict__ logp, const uint8_t* __restrict__ mask,
                                                  int64_t T, const int32_t* __restrict__ cu, int64_t n_seqs,
                                                  const int32_t* __restrict__ n_valid, const float* __restrict__ scale,
                                                  float* __restrict__ g_logp, float* __restrict__ stat_loss,
                                                  double* __restrict__ seq_sum, int32_t* __restrict__ seq_count) {
  __shared__ double sh_sum[kWaves];
  __shared__ int sh_cnt[kWaves];
  const int64_t b = blockIdx.x;
  const float g = -(scale ? scale[0] : 1.f) / ((float)n_valid[0] + 1e-5f);   // lm_engine.py:96
  double acc = 0.0;
  int cnt = 0;
  // up to two ranges: [b0, e0) and, for the last workgroup, also [b1, e1)
  int64_t b0, e0, b1 = 0, e1 = 0;
  if (b < n_seqs) {
    b0 = cu[b];
    e0 = cu[b + 1];
  } else if (cu && n_seqs > 0) {
    b0 = 0;
    e0 = cu[0];
    b1 = cu[n_seqs];
    e1 = T;
  } else {
    b0 = 0;
    e0 = T;
  }
  if (b0 < 0) b0 = 0;
  if (e0 > T) e0 = T;
  if (b1 < 0) b1 = 0;
  for (int r = 0; r < 2; ++r) {
    const int64_t lo = r ? b1 : b0, hi = r ? e1 : e0;
    for (int64_t t = lo + threadIdx.x; t < hi; t += kThreads) {
      const bool m = mask[t] != 0;
      const float lp = m ? logp[t] : 0.f;     // torch.where(loss_mask, logprobs, 0), lm_engine.py:93
      acc += (double)lp;
      cnt += m ? 1 : 0;
      if (g_logp) g_logp[t] = m ? g : 0.f;
      if (stat_loss) stat_loss[t] = -lp;
    }
  }
  acc = wave_sum(acc);
  cnt = wave_sum(cnt);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) {
    sh_sum[wave] = acc;
    sh_cnt[wave] = cnt;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double s = sh_sum[0];
    int c = sh_cnt[0];
    for (int w = 1; w < kWaves; ++w) {
      s += sh_sum[w];
      c += sh_cnt[w];
    }
    seq_sum[b] = s;
    seq_count[b] = c;
  }
}

// One workgroup: the total in a fixed order (thread k adds ranges k, k + 1024, ...; xor tree per wave; wave totals
// in wave order), then per sequence the mean log-prob over its selected tokens and exp(-mean).
__global__ __launch_bounds__(kThreads) void k_finish(int64_t n_seqs, const int32_t* __restrict__ n_valid,
                                                     const float* __restrict__ scale, double* __restrict__ seq_logp,
                                                     const int32_t* __restrict__ seq_count, float* __restrict__ seq_ppl,
                                                     float* __restrict__ loss) {
  __shared__ double sh_sum[kWaves];
  double acc = 0.0;
  for (int64_t b = threadIdx.x; b <= n_seqs; b += kThreads) acc += seq_logp[b];
  acc = wave_sum(acc);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) sh_sum[wave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double s = sh_sum[0];
    for (int w = 1; w < kWaves; ++w) s += sh_sum[w];
    loss[0] = -(scale ? scale[0] : 1.f) * ((float)s / ((float)n_valid[0] + 1e-5f));
  }
  for (int64_t b = threadIdx.x; b < n_seqs; b += kThreads) {
    const int c = seq_count[b];
    // a sequence without a selected token is skipped by the reference: its mean stays 0 (lm_engine.py:104-112)
    const double mean = c > 0 ? seq_logp[b] / (double)c : 0.0;
    seq_logp[b] = mean;
    if (seq_ppl) seq_ppl[b] = (float)exp(-mean);
  }
}

}  // namespace sft
}  // namespace aa

using namespace aa;
using namespace aa::sft;

extern "C" int aa_sft_loss(const float* logp, const uint8_t* mask, int64_t T, const int32_t* cu_seqlens,
                           int64_t n_seqs, const int32_t* n_valid, const float* scale, float* loss, float* g_logp,
                           float* stat_loss, double* seq_logp, int32_t* seq_count, float* seq_ppl, void* stream) {
  if (T < 0 || n_seqs < 0 || n_seqs >= 0x7fffffff || !n_valid || !loss || !seq_logp || !seq_count)
    return AA_ERR_INVALID_ARGUMENT;
  if (T > 0 && (!logp || !mask)) return AA_ERR_INVALID_ARGUMENT;
  if (n_seqs > 0 && !cu_seqlens) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(k_seq, dim3((unsigned)n_seqs + 1), dim3(kThreads), 0, st, logp, mask, T, cu_seqlens, n_seqs,
                     n_valid, scale, g_logp, stat_loss, seq_logp, seq_count);
  hipLaunchKernelGGL(k_finish, dim3(1), dim3(kThreads), 0, st, n_seqs, n_valid, scale, seq_logp, seq_count, seq_ppl,
                     loss);
  return launch_status();
}
