// M2PO masking (areal/trainer/ppo/actor.py:769-850): among the valid tokens, drop those with the largest second
// momentum (old_logp - prox_logp)^2 until the mean of what is left falls below the threshold.
//
// The reference sorts the selected values in descending order, forms suffix means and masks everything before
// the first suffix whose mean is below the threshold.  Here: one radix sort of (value, index) pairs over all n
// tokens with unselected tokens keyed below every real value, one single-workgroup pass that finds the cut from
// float64 suffix sums, and a scatter of the kept ranks.  Equal values keep index order (the sort is stable).
#include "device_utils.h"

#include <hipcub/hipcub.hpp>

namespace aa {
namespace m2po {

constexpr int kThreads = 1024;

struct Layout {
  int64_t off_keys_in, off_keys_out, off_idx_in, off_idx_out, off_info, off_sort;
  size_t sort_bytes;
  int64_t bytes;
};

static bool plan(int64_t n, Layout& w) {
  auto up = [](int64_t x) { return (x + 255) / 256 * 256; };
  size_t sort_bytes = 0;
  if (hipcub::DeviceRadixSort::SortPairsDescending(nullptr, sort_bytes, (const float*)nullptr, (float*)nullptr,
                                                   (const uint32_t*)nullptr, (uint32_t*)nullptr, (int)n) != hipSuccess)
    return false;
  int64_t off = 0;
  w.off_keys_in = off;  off += up(n * 4);
  w.off_keys_out = off; off += up(n * 4);
  w.off_idx_in = off;   off += up(n * 4);
  w.off_idx_out = off;  off += up(n * 4);
  w.off_info = off;     off += 256;
  w.off_sort = off;     off += up((int64_t)sort_bytes);
  w.sort_bytes = sort_bytes;
  w.bytes = off;
  return true;
}

__global__ __launch_bounds__(256) void k_keys(const float* __restrict__ old, const float* __restrict__ prox,
                                              const uint8_t* __restrict__ mask, int64_t n, float* __restrict__ keys,
                                              uint32_t* __restrict__ idx, uint8_t* __restrict__ mask_out) {
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const float d = old[i] - prox[i];
    keys[i] = mask[i] != 0 ? d * d : -1.f;  // squares are >= 0: unselected tokens sort behind all selected ones
    idx[i] = (uint32_t)i;
    mask_out[i] = 0;
  }
}

// info[0] = number of selected tokens, info[1] = number of leading (largest) tokens to mask
__global__ __launch_bounds__(kThreads) void k_cut(const float* __restrict__ sorted, int64_t n, float threshold,
                                                  int32_t* __restrict__ info) {
  __shared__ double part[kThreads];
  __shared__ int64_t cnt_s[kThreads];
  __shared__ int64_t first_s[kThreads / kWave];
  const int tid = threadIdx.x;
  const int64_t per = (n + kThreads - 1) / kThreads;
  const int64_t beg = tid * per, end = (beg + per < n) ? beg + per : n;
  double s = 0.0;
  int64_t c = 0;
  for (int64_t i = beg; i < end; ++i) {
    const float v = sorted[i];
    if (v >= 0.f) {
      s += (double)v;
      c += 1;
    }
  }
  part[tid] = s;
  cnt_s[tid] = c;
  __syncthreads();
  // suffix sum of the slices after this thread's, and the number of selected tokens (fixed order)
  double after = 0.0;
  int64_t n_sel = 0;
  for (int t = kThreads - 1; t > tid; --t) after += part[t];
  for (int t = 0; t < kThreads; ++t) n_sel += cnt_s[t];
  // first index whose suffix mean is below the threshold: walk the slice from its end
  int64_t first = INT64_MAX;
  double suffix = after;
  for (int64_t i = end - 1; i >= beg; --i) {
    const float v = sorted[i];
    if (v < 0.f) continue;  // past the selected range
    suffix += (double)v;
    const float avg = (float)suffix / (float)(n_sel - i);
    if (avg < threshold) first = i;  // walking towards the front: the last hit is the smallest index of the slice
  }
  // suffix means never shrink towards the front, so the qualifying indices form a tail [k, n_sel): take the minimum
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const int64_t other = __shfl_xor(first, o, kWave);
    first = other < first ? other : first;
  }
  if ((tid & (kWave - 1)) == 0) first_s[tid / kWave] = first;
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < kThreads / kWave; ++w) first = first_s[w] < first ? first_s[w] : first;
    int64_t k = first == INT64_MAX ? (n_sel > 0 ? n_sel - 1 : 0) : first;  // nothing qualifies: keep one token
    info[0] = (int32_t)n_sel;
    info[1] = (int32_t)k;
  }
}

__global__ __launch_bounds__(256) void k_scatter(const uint32_t* __restrict__ sorted_idx, int64_t n,
                                                 const int32_t* __restrict__ info, uint8_t* __restrict__ mask_out) {
  const int64_t n_sel = info[0], k = info[1];
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x; j < n_sel; j += step)
    if (j >= k) mask_out[sorted_idx[j]] = 1;
}

}  // namespace m2po
}  // namespace aa

using namespace aa;
using namespace aa::m2po;

extern "C" int64_t aa_m2po_workspace_bytes(int64_t n) {
  if (n < 0 || n > 0x7fffffff) return -1;
  Layout w;
  if (!plan(n > 0 ? n : 1, w)) return -1;
  return w.bytes;
}

extern "C" int aa_m2po_mask(const float* old_logp, const float* prox_logp, const uint8_t* mask_in, int64_t n,
                            float m2_threshold, uint8_t* mask_out, int32_t* info, void* workspace,
                            int64_t workspace_bytes, void* stream) {
  if (n < 0 || n > 0x7fffffff || !info) return AA_ERR_INVALID_ARGUMENT;
  if (n == 0) return AA_OK;
  if (!old_logp || !prox_logp || !mask_in || !mask_out || !workspace || (((uintptr_t)workspace) & 255))
    return AA_ERR_INVALID_ARGUMENT;
  Layout w;
  if (!plan(n, w)) return AA_ERR_LAUNCH;
  if (workspace_bytes < w.bytes) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  float* keys_in = (float*)(ws + w.off_keys_in);
  float* keys_out = (float*)(ws + w.off_keys_out);
  uint32_t* idx_in = (uint32_t*)(ws + w.off_idx_in);
  uint32_t* idx_out = (uint32_t*)(ws + w.off_idx_out);
  int64_t blocks = (n + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  hipLaunchKernelGGL(k_keys, dim3((unsigned)blocks), dim3(256), 0, st, old_logp, prox_logp, mask_in, n, keys_in,
                     idx_in, mask_out);
  size_t sort_bytes = w.sort_bytes;
  if (hipcub::DeviceRadixSort::SortPairsDescending(ws + w.off_sort, sort_bytes, keys_in, keys_out, idx_in, idx_out,
                                                   (int)n, 0, 32, st) != hipSuccess)
    return AA_ERR_LAUNCH;
  hipLaunchKernelGGL(k_cut, dim3(1), dim3(kThreads), 0, st, keys_out, n, m2_threshold, info);
  hipLaunchKernelGGL(k_scatter, dim3((unsigned)blocks), dim3(256), 0, st, idx_out, n, info, mask_out);
  return launch_status();
}
