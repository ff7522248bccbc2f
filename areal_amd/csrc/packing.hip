// Segmented row copy for packed sequences on gfx950: the data movement behind pack_tensor_dict,
// pad_packed_tensor_dict and unpad_logits (areal/utils/data.py:492-541, 818-978, 1046-1074), which the reference
// performs as one slice assignment per sequence from a Python loop (with a device-to-host sync per bound).
//
// Rows (tokens) are enumerated 0 .. total_rows-1 in segment order; seg_cu[i] is the number of rows in segments
// before i.  Row r of segment i, offset o = r - seg_cu[i], goes from src row src_starts[i] + o to dst row
// dst_starts[i] + o.  Pure HBM-to-HBM byte movement: 16-byte accesses where row size and alignment allow.
#include "device_utils.h"

namespace aa {
namespace packing {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// largest i with seg_cu[i] <= r, 0 <= i < B (seg_cu has B + 1 entries, seg_cu[0] = 0)
__device__ __forceinline__ int64_t find_segment(const int32_t* __restrict__ seg_cu, int64_t B, int64_t r) {
  int64_t lo = 0, hi = B;  // invariant: seg_cu[lo] <= r < seg_cu[hi]
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)seg_cu[mid] <= r) lo = mid;
    else hi = mid;
  }
  return lo;
}

// rows of W bytes, one thread per row
template <typename W>
__global__ __launch_bounds__(256) void k_copy_small(const W* __restrict__ src, W* __restrict__ dst,
                                                    const int64_t* __restrict__ src_starts,
                                                    const int64_t* __restrict__ dst_starts,
                                                    const int32_t* __restrict__ seg_cu, int64_t B, int64_t total) {
  const int64_t step = (int64_t)gridDim.x * 256;
  for (int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x; r < total; r += step) {
    const int64_t s = find_segment(seg_cu, B, r);
    const int64_t o = r - seg_cu[s];
    dst[dst_starts[s] + o] = src[src_starts[s] + o];
  }
}

// Rows of n_words words of type W, cut into pieces of kPieceWords words (eight per thread): one workgroup per piece,
// grid-stride, pieces numbered along the rows.  The workgroups in flight together then cover one contiguous stretch of
// source and destination (a few dozen rows) instead of thousands of separate row streams, which the memory system
// serves markedly faster.
constexpr int kPieceWords = 2048;

template <typename W>
__global__ __launch_bounds__(256) void k_copy_rows(const W* __restrict__ src, W* __restrict__ dst, int64_t n_words,
                                                   const int64_t* __restrict__ src_starts,
                                                   const int64_t* __restrict__ dst_starts,
                                                   const int32_t* __restrict__ seg_cu, int64_t B, int64_t total,
                                                   int64_t pieces_per_row) {
  const int64_t n_pieces = total * pieces_per_row;
  for (int64_t id = blockIdx.x; id < n_pieces; id += gridDim.x) {
    const int64_t r = id / pieces_per_row;
    const int64_t s = find_segment(seg_cu, B, r);
    const int64_t o = r - seg_cu[s];
    const W* p = src + (src_starts[s] + o) * n_words;
    W* q = dst + (dst_starts[s] + o) * n_words;
    const int64_t i = (id - r * pieces_per_row) * kPieceWords + threadIdx.x;
    if (i + 7 * 256 < n_words) {  // eight independent loads in flight per thread before the first store
      W v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = __builtin_nontemporal_load(p + i + k * 256);
#pragma unroll
      for (int k = 0; k < 8; ++k) __builtin_nontemporal_store(v[k], q + i + k * 256);
    } else {
      for (int64_t j = i; j < n_words && j < i + kPieceWords; j += 256)
        __builtin_nontemporal_store(__builtin_nontemporal_load(p + j), q + j);
    }
  }
}

template <typename W>
static void launch(const void* src, void* dst, int64_t row_bytes, const int64_t* ss, const int64_t* ds,
                   const int32_t* cu, int64_t B, int64_t total, hipStream_t st) {
  const int64_t n_words = row_bytes / (int64_t)sizeof(W);
  if (n_words == 1) {
    int64_t blocks = (total + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(k_copy_small<W>, dim3((unsigned)blocks), dim3(256), 0, st, (const W*)src, (W*)dst, ss, ds, cu, B,
                       total);
  } else {
    const int64_t pieces_per_row = (n_words + kPieceWords - 1) / kPieceWords;
    const int64_t n_pieces = total * pieces_per_row;
    const int64_t blocks = n_pieces < (1 << 20) ? n_pieces : (1 << 20);
    hipLaunchKernelGGL(k_copy_rows<W>, dim3((unsigned)blocks), dim3(256), 0, st, (const W*)src, (W*)dst, n_words, ss,
                       ds, cu, B, total, pieces_per_row);
  }
}

}  // namespace packing
}  // namespace aa

using namespace aa;
using namespace aa::packing;

extern "C" int aa_segment_copy(const void* src, void* dst, int64_t row_bytes, const int64_t* src_starts,
                               const int64_t* dst_starts, const int32_t* seg_cu, int64_t B, int64_t total_rows,
                               void* stream) {
  if (row_bytes < 1 || B < 0 || total_rows < 0) return AA_ERR_INVALID_ARGUMENT;
  if (total_rows == 0 || B == 0) return AA_OK;
  if (!src || !dst || !src_starts || !dst_starts || !seg_cu) return AA_ERR_INVALID_ARGUMENT;
  hipStream_t st = (hipStream_t)stream;
  const uintptr_t a = (uintptr_t)src | (uintptr_t)dst | (uintptr_t)row_bytes;
  if ((a & 15) == 0) launch<u32x4_t>(src, dst, row_bytes, src_starts, dst_starts, seg_cu, B, total_rows, st);
  else if ((a & 7) == 0) launch<uint64_t>(src, dst, row_bytes, src_starts, dst_starts, seg_cu, B, total_rows, st);
  else if ((a & 3) == 0) launch<uint32_t>(src, dst, row_bytes, src_starts, dst_starts, seg_cu, B, total_rows, st);
  else if ((a & 1) == 0) launch<uint16_t>(src, dst, row_bytes, src_starts, dst_starts, seg_cu, B, total_rows, st);
  else launch<uint8_t>(src, dst, row_bytes, src_starts, dst_starts, seg_cu, B, total_rows, st);
  return launch_status();
}
