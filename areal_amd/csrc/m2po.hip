// M2PO masking (areal/trainer/ppo/actor.py:769-850): among the valid tokens, drop those with the largest second
// momentum (old_logp - prox_logp)^2 until the mean of what is left falls below the threshold.
//
// The reference sorts the selected values in descending order, forms suffix means and masks everything before
// the first suffix whose mean is below the threshold.  Here: one radix sort of (value, index) pairs over all n
// tokens with unselected tokens keyed below every real value, a two-level pass that finds the cut from float64
// suffix sums, and a scatter of the kept ranks.  Equal values keep index order (the sort is stable).
#include "device_utils.h"

#include <hipcub/hipcub.hpp>

namespace aa {
namespace m2po {

constexpr int kThreads = 1024;

struct Layout {
  int64_t off_keys_in, off_keys_out, off_idx_in, off_idx_out, off_info, off_sort, off_tile_sums, off_tile_cnts;
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
  const int64_t tiles = (n + 4095) / 4096;
  w.off_tile_sums = off; off += up(tiles * 8);
  w.off_tile_cnts = off; off += up(tiles * 4);
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

// ---- the cut ----------------------------------------------------------------------------------------------------
// sorted[] holds the selected values in descending order, then -1 for every unselected token.  With n_sel selected
// values, suffix(i) = sum of sorted[i .. n_sel) and the cut k is the smallest i whose suffix mean
// (float)suffix(i) / (float)(n_sel - i) is below the threshold (suffix means never shrink towards the front, so the
// qualifying indices form a tail); if none qualifies one token is kept, k = n_sel - 1.
// Two kernels, every load coalesced: k_tile_sums reduces tiles of kTile values to (float64 sum, count) in parallel;
// k_cut (one workgroup) forms the suffix sums at the tile starts, finds the first tile start that qualifies, and
// looks for the cut inside the one tile before it.  All sums have a fixed order: repeated calls agree bit for bit.
constexpr int kTile = 4096;

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

__global__ __launch_bounds__(256) void k_tile_sums(const float* __restrict__ sorted, int64_t n,
                                                   double* __restrict__ sums, int32_t* __restrict__ cnts) {
  __shared__ double ps[4];
  __shared__ int pc[4];
  const int64_t base = (int64_t)blockIdx.x * kTile;
  double s = 0.0;
  int c = 0;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int64_t i0 = base + (int64_t)(k * 256 + threadIdx.x) * 4;
    if (i0 < n) {  // the buffer is padded to 256 bytes: the vector load stays inside it
      const float4 v = *(const float4*)(sorted + i0);
      const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (i0 + q < n && e[q] >= 0.f) {
          s += (double)e[q];
          c += 1;
        }
    }
  }
  s = wave_sum_f64(s);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, kWave);
  if ((threadIdx.x & 63) == 0) {
    ps[threadIdx.x >> 6] = s;
    pc[threadIdx.x >> 6] = c;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    sums[blockIdx.x] = (ps[0] + ps[1]) + (ps[2] + ps[3]);
    cnts[blockIdx.x] = pc[0] + pc[1] + pc[2] + pc[3];
  }
}

// sum over the threads after this one (exclusive suffix) of a per-thread value: suffix scan inside the wave by
// shuffles, then the totals of the later waves from LDS; fixed order
__device__ __forceinline__ double after_me(double* part, double mine, int tid) {
  const int lane = tid & (kWave - 1), wave = tid / kWave;
  double incl = mine;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const double down = __shfl_down(incl, o, kWave);
    if (lane + o < kWave) incl += down;
  }
  __syncthreads();  // part may still be read by a previous call
  if (lane == 0) part[wave] = incl;
  __syncthreads();
  double after = incl - mine;
  for (int w = kThreads / kWave - 1; w > wave; --w) after += part[w];
  return after;
}

__device__ __forceinline__ int64_t block_min(int64_t* slot, int64_t v, int tid) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const int64_t other = __shfl_xor(v, o, kWave);
    v = other < v ? other : v;
  }
  __syncthreads();
  if ((tid & (kWave - 1)) == 0) slot[tid / kWave] = v;
  __syncthreads();
  int64_t r = slot[0];
  for (int w = 1; w < kThreads / kWave; ++w) r = slot[w] < r ? slot[w] : r;
  return r;
}

// info[0] = number of selected tokens, info[1] = number of leading (largest) tokens to mask
__global__ __launch_bounds__(kThreads) void k_cut(const float* __restrict__ sorted, int64_t n, float threshold,
                                                  const double* __restrict__ sums, const int32_t* __restrict__ cnts,
                                                  int m, int32_t* __restrict__ info) {
  __shared__ double part[kThreads];
  __shared__ int64_t slot[kThreads / kWave];
  __shared__ int64_t n_sel_s;
  const int tid = threadIdx.x;
  const int per = (m + kThreads - 1) / kThreads;
  const int beg = tid * per < m ? tid * per : m, end = beg + per < m ? beg + per : m;
  // number of selected values
  int64_t c = 0;
  for (int j = beg; j < end; ++j) c += cnts[j];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, kWave);
  if ((tid & (kWave - 1)) == 0) slot[tid / kWave] = c;
  __syncthreads();
  if (tid == 0) {
    int64_t t = 0;
    for (int w = 0; w < kThreads / kWave; ++w) t += slot[w];
    n_sel_s = t;
  }
  __syncthreads();
  const int64_t n_sel = n_sel_s;
  if (n_sel == 0) {
    if (tid == 0) {
      info[0] = 0;
      info[1] = 0;
    }
    return;
  }
  // suffix sums at the tile starts: first tile whose start qualifies
  double mine = 0.0;
  for (int j = beg; j < end; ++j) mine += sums[j];
  double suffix = after_me(part, mine, tid);
  int64_t first_tile = INT64_MAX;
  for (int j = end - 1; j >= beg; --j) {
    suffix += sums[j];
    const int64_t start = (int64_t)j * kTile;
    if (start < n_sel && (float)suffix / (float)(n_sel - start) < threshold) first_tile = j;
  }
  const int64_t jstar = block_min(slot, first_tile, tid);
  int64_t k;
  if (jstar == 0) {
    k = 0;
  } else {
    // the cut, if any lies before the start of tile jstar, is inside tile d
    const int64_t d = jstar != INT64_MAX ? jstar - 1 : (n_sel - 1) / kTile;
    double later = 0.0;  // sum of the tiles after d
    for (int j = beg; j < end; ++j)
      if (j > d) later += sums[j];
    const double from_me_on = after_me(part, later, tid) + later;  // thread 0 holds the whole sum: broadcast it
    __syncthreads();
    if (tid == 0) part[0] = from_me_on;
    __syncthreads();
    const double tail = part[0];
    const int64_t i0 = d * kTile + (int64_t)tid * 4;
    float e[4] = {0.f, 0.f, 0.f, 0.f};
    if (i0 < n) {
      const float4 v = *(const float4*)(sorted + i0);
      e[0] = v.x; e[1] = v.y; e[2] = v.z; e[3] = v.w;
    }
    double own = 0.0;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (i0 + q < n_sel) own += (double)e[q];
    double sfx = tail + after_me(part, own, tid);
    int64_t first = INT64_MAX;
#pragma unroll
    for (int q = 3; q >= 0; --q) {
      const int64_t i = i0 + q;
      if (i < n_sel) {
        sfx += (double)e[q];
        if ((float)sfx / (float)(n_sel - i) < threshold) first = i;
      }
    }
    const int64_t found = block_min(slot, first, tid);
    const int64_t at_start = jstar != INT64_MAX ? jstar * kTile : INT64_MAX;
    k = found < at_start ? found : at_start;
    if (k == INT64_MAX) k = n_sel - 1;  // nothing qualifies: keep one token
  }
  if (tid == 0) {
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
  const int tiles = (int)((n + kTile - 1) / kTile);
  double* tile_sums = (double*)(ws + w.off_tile_sums);
  int32_t* tile_cnts = (int32_t*)(ws + w.off_tile_cnts);
  hipLaunchKernelGGL(k_tile_sums, dim3((unsigned)tiles), dim3(256), 0, st, keys_out, n, tile_sums, tile_cnts);
  hipLaunchKernelGGL(k_cut, dim3(1), dim3(kThreads), 0, st, keys_out, n, m2_threshold, tile_sums, tile_cnts, tiles, info);
  hipLaunchKernelGGL(k_scatter, dim3((unsigned)blocks), dim3(256), 0, st, idx_out, n, info, mask_out);
  return launch_status();
}
