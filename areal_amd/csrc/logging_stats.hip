// What the actor's loss function logs about the proximal-policy approximations, the drift between the training and
// the inference policy and the staleness of the samples, reduced under the mask in one pass instead of one
// per-token tensor and one reduction per logged quantity.
// Reference: areal/trainer/ppo/actor.py:852-1110 (_log_proximal_approximation_stats, _log_version_staleness_stats
// and their helpers), reduced as areal/utils/stats_tracker.py:227-285 reduces a tensor under a denominator mask.
#include "ppo_math.h"

namespace aa {
namespace logstats {

constexpr int kThreads = 256;      // ten fp64 sums with extrema and counts per thread: needs the large register budget
constexpr int kWaves = kThreads / kWave;
constexpr int kGroups = 4;        // group 0: ground truth, KL estimators, staleness; groups 1-3: one method each
constexpr int kPerGroup = 10;     // quantities per group
constexpr int kSlots = AA_LOGSTAT_SLOTS;
constexpr float kEps = 1e-8f;     // _EPSILON, actor.py:856
static_assert(kSlots == 4 + 3 * kPerGroup + 2, "slot layout");

struct Partial {
  double sum, cnt;
  float lo, hi;
  float pad[2];
};

struct Acc {
  double sum = 0.0;
  int cnt = 0;
  float lo = __builtin_inff(), hi = -__builtin_inff();
  __device__ __forceinline__ void add(float x) {
    sum += (double)x;
    cnt += 1;
    lo = nan_min(lo, x);
    hi = nan_max(hi, x);
  }
};

// slot of quantity j of group g in the output table; -1 = unused
__device__ __forceinline__ int slot_of(int g, int j) {
  if (g == 0) return j < 4 ? j : (j < 6 ? 4 + 3 * kPerGroup + (j - 4) : -1);
  return 4 + (g - 1) * kPerGroup + j;
}

__device__ __forceinline__ void errors(float gt, float approx, float& abs_e, float& rel_e, float& sq_e) {
  const float d = gt - approx;
  abs_e = fabsf(d);
  rel_e = fabsf(d / (fabsf(gt) + kEps));
  sq_e = d * d;
}

// grid = kGroups * parts; workgroup (g, part) reduces its slice of the tokens for the quantities of group g
__global__ __launch_bounds__(kThreads) void k_partial(const float* __restrict__ old, const float* __restrict__ logp,
                                                      const float* __restrict__ gt, const int32_t* __restrict__ versions,
                                                      const uint8_t* __restrict__ mask, int64_t n, int current_version,
                                                      int methods, int with_errors, int parts,
                                                      Partial* __restrict__ partial) {
  __shared__ double sh_sum[kWaves], sh_cnt[kWaves];
  __shared__ float sh_lo[kWaves], sh_hi[kWaves];
  const int g = blockIdx.x / parts, part = blockIdx.x % parts;
  const int64_t per = (n + parts - 1) / parts;
  const int64_t b = (int64_t)part * per, e = b + per < n ? b + per : n;
  Acc acc[kPerGroup];
  const bool active = g == 0 || ((methods >> (g - 1)) & 1);
  if (active) {
    for (int64_t i = b + threadIdx.x; i < e; i += kThreads) {
      if (mask[i] == 0) continue;
      const float lo = old[i], ln = logp[i];
      if (g == 0) {
        if (gt) acc[0].add(gt[i]);
        if (versions) {
          const float lr = ln - lo;                       // actor.py:1049
          acc[1].add(-lr);
          acc[2].add(lr * lr / 2.0f);
          acc[3].add(expf(lr) - 1.f - lr);
          const int ver = versions[i];
          if (ver >= 0) {                                 // actor.py:1087-1094
            acc[4].add((float)(current_version - 1) - (float)ver);
            acc[5].add((float)current_version - (float)ver);
          }
        }
      } else {
        const float ap = prox_approx_value(lo, ln, versions[i], current_version, g - 1);
        const float bw = expf(ap - lo), iw = expf(ln - ap);     // actor.py:924-925
        acc[0].add(ap);
        acc[1].add(bw);
        acc[2].add(iw);
        if (with_errors) {                                      // actor.py:934-968
          const float p = gt[i];
          float a, r, s;
          errors(p, ap, a, r, s);
          acc[3].add(a);
          acc[4].add(r);
          acc[5].add(s);
          errors(expf(p - lo), bw, a, r, s);
          acc[6].add(a);
          acc[7].add(r);
          errors(expf(ln - p), iw, a, r, s);
          acc[8].add(a);
          acc[9].add(r);
        }
      }
    }
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
  for (int j = 0; j < kPerGroup; ++j) {
    const double s = wave_sum(acc[j].sum), c = (double)wave_sum(acc[j].cnt);
    float lo = acc[j].lo, hi = acc[j].hi;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      lo = nan_min(lo, __shfl_xor(lo, o, kWave));
      hi = nan_max(hi, __shfl_xor(hi, o, kWave));
    }
    __syncthreads();
    if (lane == 0) {
      sh_sum[wave] = s;
      sh_cnt[wave] = c;
      sh_lo[wave] = lo;
      sh_hi[wave] = hi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      Partial r{sh_sum[0], sh_cnt[0], sh_lo[0], sh_hi[0], {0.f, 0.f}};
      for (int w = 1; w < kWaves; ++w) {
        r.sum += sh_sum[w];
        r.cnt += sh_cnt[w];
        r.lo = nan_min(r.lo, sh_lo[w]);
        r.hi = nan_max(r.hi, sh_hi[w]);
      }
      partial[((int64_t)g * parts + part) * kPerGroup + j] = r;
    }
  }
}

// one wave per (group, quantity): lane l folds slices l, l + 64, ... in index order, then a fixed butterfly folds
// the lanes; out[slot] = {sum, min, max, count}
__global__ __launch_bounds__(kWave) void k_finish(const Partial* __restrict__ partial, int parts,
                                                  float* __restrict__ out) {
  const int g = blockIdx.x / kPerGroup, j = blockIdx.x % kPerGroup;
  const int slot = slot_of(g, j);
  if (slot < 0) return;
  double sum = 0.0, cnt = 0.0;
  float lo = __builtin_inff(), hi = -__builtin_inff();
  for (int p = threadIdx.x; p < parts; p += kWave) {
    const Partial v = partial[((int64_t)g * parts + p) * kPerGroup + j];
    sum += v.sum;
    cnt += v.cnt;
    lo = nan_min(lo, v.lo);
    hi = nan_max(hi, v.hi);
  }
  sum = wave_sum(sum);
  cnt = wave_sum(cnt);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    lo = nan_min(lo, __shfl_xor(lo, o, kWave));
    hi = nan_max(hi, __shfl_xor(hi, o, kWave));
  }
  if (threadIdx.x == 0) {
    float* o = out + 4 * slot;
    o[0] = (float)sum;
    o[1] = lo;
    o[2] = hi;
    o[3] = (float)cnt;
  }
}

inline int parts_for(int64_t n) {
  int64_t parts = (n + 2047) / 2048;   // at least 8 tokens per thread
  if (parts > 256) parts = 256;
  return parts < 1 ? 1 : (int)parts;
}

}  // namespace logstats
}  // namespace aa

using namespace aa;
using namespace aa::logstats;

extern "C" int64_t aa_logging_stats_scratch_bytes(int64_t n) {
  if (n < 0) return -1;
  return (int64_t)kGroups * parts_for(n) * kPerGroup * (int64_t)sizeof(Partial);
}

extern "C" int aa_logging_stats(const float* old_logp, const float* logp, const float* prox_logp_gt,
                                const int32_t* versions, const uint8_t* mask, int64_t n, int current_version,
                                int methods, int with_errors, float* out, void* scratch, int64_t scratch_bytes,
                                void* stream) {
  if (n < 0 || !out || !scratch || methods < 0 || methods > 7) return AA_ERR_INVALID_ARGUMENT;
  if (n > 0 && (!old_logp || !logp || !mask)) return AA_ERR_INVALID_ARGUMENT;
  // an empty batch may come with null data pointers: nothing is dereferenced, every row comes out empty
  if (n > 0 && methods != 0 && !versions) return AA_ERR_INVALID_ARGUMENT;
  if (n > 0 && with_errors && !prox_logp_gt) return AA_ERR_INVALID_ARGUMENT;
  const int parts = parts_for(n);
  if (scratch_bytes < (int64_t)kGroups * parts * kPerGroup * (int64_t)sizeof(Partial)) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  Partial* partial = (Partial*)scratch;
  hipLaunchKernelGGL(k_partial, dim3((unsigned)(kGroups * parts)), dim3(kThreads), 0, st, old_logp, logp, prox_logp_gt,
                     versions, mask, n, current_version, methods, with_errors ? 1 : 0, parts, partial);
  hipLaunchKernelGGL(k_finish, dim3(kGroups * kPerGroup), dim3(kWave), 0, st, partial, parts, out);
  return launch_status();
}
