// Masked-position compaction and row gather/scatter for gfx950.
//
// Device counterpart of `_compact_valid_loss_rows`
// (dllm_parallel/core/models/backbones/nemotron/model.py:4234-4253):
//   row_idx = nonzero(labels != ignore_index)   (ascending int64)
//   hidden_c = hidden.index_select(0, row_idx), labels_c = labels.index_select(0, row_idx)
// and of the same step on a boolean mask (`nonzero(supervised_mask)`,
// dllm_parallel/core/models/backbones/dflash/model.py:870-871, dflash2.py:577-578).
// Two passes over the flags: a ballot/popcount per 1024-flag block, then each
// block writes its indices at wave-ballot prefix positions behind the blocks
// before it.  Up to 256 blocks a block adds up the earlier counts itself; for
// longer inputs one workgroup turns the counts into exclusive offsets between
// the two passes.  No spin-waits between blocks: the passes are separate
// launches.
#include "tlce_common.h"

namespace tlce {

constexpr int kCompactThreads = 256;
constexpr int kCompactItems = 4;
constexpr int kCompactBlock = kCompactThreads * kCompactItems;  // flags per block
constexpr int kScanThreads = 1024;

// What marks a position as kept: a label different from the ignore value, or a
// non-zero mask byte.
struct LabelFlags {
  const int64_t* labels;
  int64_t ignore;
  __device__ __forceinline__ bool operator()(int64_t i) const { return labels[i] != ignore; }
};
struct MaskFlags {
  const uint8_t* mask;
  __device__ __forceinline__ bool operator()(int64_t i) const { return mask[i] != 0; }
};

template <class Flags>
__global__ __launch_bounds__(kCompactThreads) void compact_count_kernel(
    Flags flags, int64_t n, int* __restrict__ block_counts) {
  __shared__ int wave_counts[kCompactThreads / 64];
  const int64_t base = (int64_t)blockIdx.x * kCompactBlock;
  int count = 0;
#pragma unroll
  for (int q = 0; q < kCompactItems; ++q) {
    const int64_t i = base + q * kCompactThreads + threadIdx.x;
    const bool keep = (i < n) && flags(i);
    count += __popcll(__ballot(keep));  // wave-uniform
  }
  if ((threadIdx.x & 63) == 0) wave_counts[threadIdx.x >> 6] = count;
  __syncthreads();
  if (threadIdx.x == 0) {
    int total = 0;
#pragma unroll
    for (int w = 0; w < kCompactThreads / 64; ++w) total += wave_counts[w];
    block_counts[blockIdx.x] = total;
  }
}

// One workgroup: block_offsets[b] = sum of block_counts[0 .. b), 1024 blocks per
// round with the running total carried from round to round.
__global__ __launch_bounds__(kScanThreads) void compact_scan_kernel(
    const int* __restrict__ block_counts, int blocks, int64_t* __restrict__ block_offsets) {
  constexpr int kWaves = kScanThreads / 64;
  __shared__ int64_t wave_totals[kWaves];
  __shared__ int64_t carry;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int first = 0; first < blocks; first += kScanThreads) {
    const int b = first + threadIdx.x;
    const int64_t mine = b < blocks ? block_counts[b] : 0;
    int64_t incl = mine;   // inclusive prefix within the wave
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int64_t up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    if (lane == 63) wave_totals[wave] = incl;
    __syncthreads();
    int64_t before = carry;
    for (int w = 0; w < wave; ++w) before += wave_totals[w];
    if (b < blocks) block_offsets[b] = before + incl - mine;
    __syncthreads();
    if (threadIdx.x == kScanThreads - 1) carry = before + incl;
    __syncthreads();
  }
}

// block_offsets == null: the block sums the counts before it itself (few blocks).
template <class Flags>
__global__ __launch_bounds__(kCompactThreads) void compact_write_kernel(
    Flags flags, int64_t n, const int* __restrict__ block_counts,
    const int64_t* __restrict__ block_offsets, int64_t* __restrict__ row_idx,
    int64_t* __restrict__ count_out) {
  constexpr int kWaves = kCompactThreads / 64;
  __shared__ int64_t wave_partial[kWaves];
  __shared__ int slot_counts[kCompactItems * kWaves];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;

  if (block_offsets == nullptr) {
    // exclusive prefix of the block counts before this block
    int64_t before = 0;
    for (int b = threadIdx.x; b < (int)blockIdx.x; b += kCompactThreads) before += block_counts[b];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) before += __shfl_xor(before, o, 64);
    if (lane == 0) wave_partial[wave] = before;
  }

  const int64_t base = (int64_t)blockIdx.x * kCompactBlock;
  bool keep[kCompactItems];
  int rank[kCompactItems];
#pragma unroll
  for (int q = 0; q < kCompactItems; ++q) {
    const int64_t i = base + q * kCompactThreads + threadIdx.x;
    keep[q] = (i < n) && flags(i);
    const unsigned long long mask = __ballot(keep[q]);
    rank[q] = __popcll(mask & ((1ull << lane) - 1ull));
    if (lane == 0) slot_counts[q * kWaves + wave] = __popcll(mask);
  }
  __syncthreads();

  int64_t block_offset = 0;
  if (block_offsets == nullptr) {
#pragma unroll
    for (int w = 0; w < kWaves; ++w) block_offset += wave_partial[w];
  } else {
    block_offset = block_offsets[blockIdx.x];
  }

  int running = 0;
#pragma unroll
  for (int q = 0; q < kCompactItems; ++q) {
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      if (w == wave && keep[q]) {
        const int64_t i = base + q * kCompactThreads + threadIdx.x;
        row_idx[block_offset + running + rank[q]] = i;
      }
      running += slot_counts[q * kWaves + w];
    }
  }
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) count_out[0] = block_offset + running;
}

template <typename V>
__global__ __launch_bounds__(256) void gather_rows_kernel(const V* __restrict__ src,
                                                          const int64_t* __restrict__ row_idx,
                                                          int64_t total, int vecs_per_row,
                                                          V* __restrict__ dst) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const int64_t r = e / vecs_per_row;
    const int c = (int)(e - r * vecs_per_row);
    dst[e] = src[row_idx[r] * vecs_per_row + c];
  }
}

template <typename V>
__global__ __launch_bounds__(256) void scatter_rows_kernel(const V* __restrict__ src,
                                                           const int64_t* __restrict__ row_idx,
                                                           int64_t total, int vecs_per_row,
                                                           V* __restrict__ dst) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const int64_t r = e / vecs_per_row;
    const int c = (int)(e - r * vecs_per_row);
    dst[row_idx[r] * vecs_per_row + c] = src[e];
  }
}

// Gather of everything the masked-token loss needs from its loss-bearing rows in
// one launch, with the row count read on the device: for r < *row_count the
// hidden row, label and loss weight of position row_idx[r]; the rows from
// *row_count up to the next multiple of 64 (inside the destination's
// padded_rows) become zero rows with the ignore label and weight 0, so that a
// contraction over whole 64-row slabs of the gathered rows never meets
// uninitialised memory.  One workgroup per destination row.
template <typename V>
__global__ __launch_bounds__(256) void gather_loss_rows_kernel(
    const V* __restrict__ hidden_src, const int64_t* __restrict__ labels_src,
    const float* __restrict__ weights_src, const int64_t* __restrict__ row_idx,
    const int64_t* __restrict__ row_count, int64_t capacity, int64_t padded_rows,
    int vecs_per_row, int64_t ignore, V* __restrict__ hidden_dst,
    int64_t* __restrict__ labels_dst, float* __restrict__ weights_dst) {
  // row_idx holds `capacity` entries: a count outside [0, capacity] is clamped, as
  // every consumer of the count clamps it
  const int64_t count = min(max(*row_count, (int64_t)0), capacity);
  const int64_t fill_end = min(padded_rows, (count + 63) / 64 * 64);
  for (int64_t r = blockIdx.x; r < fill_end; r += gridDim.x) {
    V* dst = hidden_dst + r * vecs_per_row;
    if (r < count) {
      const int64_t s = row_idx[r];
      const V* src = hidden_src + s * vecs_per_row;
      for (int c = threadIdx.x; c < vecs_per_row; c += 256) dst[c] = src[c];
      if (threadIdx.x == 0) {
        labels_dst[r] = labels_src[s];
        if (weights_dst != nullptr) weights_dst[r] = weights_src[s];
      }
    } else {
      V z;
      memset(&z, 0, sizeof(V));
      for (int c = threadIdx.x; c < vecs_per_row; c += 256) dst[c] = z;
      if (threadIdx.x == 0) {
        labels_dst[r] = ignore;
        if (weights_dst != nullptr) weights_dst[r] = 0.0f;
      }
    }
  }
}

static int pick_vector_bytes(const void* a, const void* b, int64_t row_bytes) {
  const uintptr_t bits = (uintptr_t)a | (uintptr_t)b | (uintptr_t)row_bytes;
  if ((bits & 15) == 0) return 16;
  if ((bits & 7) == 0) return 8;
  if ((bits & 3) == 0) return 4;
  if ((bits & 1) == 0) return 2;
  return 1;
}

static int move_grid(int64_t total) {
  return (int)std::min<int64_t>(ceil_div(total, 256), 256 * 32);
}

template <bool kGather>
static int move_rows(const void* src, const int64_t* row_idx, int64_t m, int64_t row_bytes,
                     void* dst, hipStream_t stream) {
  TLCE_REQUIRE(m >= 0 && row_bytes >= 0, "row move: negative size");
  if (m == 0 || row_bytes == 0) return 0;
  TLCE_REQUIRE(src && dst && row_idx, "row move: null pointer");
  const int vb = pick_vector_bytes(src, dst, row_bytes);
  const int64_t vpr = row_bytes / vb;
  TLCE_REQUIRE(vpr <= INT32_MAX, "row move: row too long");
  const int64_t total = m * vpr;
  const int grid = move_grid(total);
#define TLCE_MOVE(V)                                                                        \
  do {                                                                                      \
    if (kGather)                                                                            \
      gather_rows_kernel<V><<<grid, 256, 0, stream>>>((const V*)src, row_idx, total,        \
                                                      (int)vpr, (V*)dst);                   \
    else                                                                                    \
      scatter_rows_kernel<V><<<grid, 256, 0, stream>>>((const V*)src, row_idx, total,       \
                                                       (int)vpr, (V*)dst);                  \
  } while (0)
  switch (vb) {
    case 16: TLCE_MOVE(uint4); break;
    case 8: TLCE_MOVE(uint2); break;
    case 4: TLCE_MOVE(uint32_t); break;
    case 2: TLCE_MOVE(uint16_t); break;
    default: TLCE_MOVE(uint8_t); break;
  }
#undef TLCE_MOVE
  TLCE_LAUNCH_CHECK();
  return 0;
}

}  // namespace tlce

using namespace tlce;

// workspace: int block_counts[blocks], then int64 block_offsets[blocks]
static int64_t compact_counts_bytes(int64_t n) {
  return align256(ceil_div(std::max<int64_t>(n, 1), kCompactBlock) * (int64_t)sizeof(int));
}

extern "C" int64_t tlce_compact_workspace_bytes(int64_t n) {
  if (n < 0) return -1;
  const int64_t blocks = ceil_div(std::max<int64_t>(n, 1), kCompactBlock);
  return compact_counts_bytes(n) + align256(blocks * (int64_t)sizeof(int64_t));
}

template <class Flags>
static int compact_flags(Flags flags, int64_t n, int64_t* row_idx_out, int64_t* count_out,
                         void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  TLCE_REQUIRE(workspace_bytes >= tlce_compact_workspace_bytes(n),
               "compact: workspace too small (%lld < %lld)", (long long)workspace_bytes,
               (long long)tlce_compact_workspace_bytes(n));
  const int blocks = (int)ceil_div(n, kCompactBlock);
  int* block_counts = static_cast<int*>(workspace);
  int64_t* block_offsets = nullptr;
  compact_count_kernel<Flags><<<blocks, kCompactThreads, 0, stream>>>(flags, n, block_counts);
  TLCE_LAUNCH_CHECK();
  if (blocks > kCompactThreads) {
    block_offsets = reinterpret_cast<int64_t*>(static_cast<char*>(workspace) +
                                               compact_counts_bytes(n));
    compact_scan_kernel<<<1, kScanThreads, 0, stream>>>(block_counts, blocks, block_offsets);
    TLCE_LAUNCH_CHECK();
  }
  compact_write_kernel<Flags><<<blocks, kCompactThreads, 0, stream>>>(
      flags, n, block_counts, block_offsets, row_idx_out, count_out);
  TLCE_LAUNCH_CHECK();
  return 0;
}

extern "C" int tlce_compact_rows(const int64_t* labels, int64_t n, int64_t ignore_index,
                                 int64_t* row_idx_out, int64_t* count_out, void* workspace,
                                 int64_t workspace_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  TLCE_REQUIRE(n >= 0 && n < (int64_t)INT32_MAX, "compact: n=%lld out of range", (long long)n);
  TLCE_REQUIRE(count_out != nullptr, "compact: count_out is null");
  if (n == 0) {
    // count = 0 through the fill kernel so the call stays capturable
    return tlce_fill_zero(count_out, sizeof(int64_t), stream_);
  }
  TLCE_REQUIRE(labels && row_idx_out && workspace, "compact: null pointer");
  return compact_flags(LabelFlags{labels, ignore_index}, n, row_idx_out, count_out, workspace,
                       workspace_bytes, stream);
}

extern "C" int tlce_compact_mask(const uint8_t* mask, int64_t n, int64_t* row_idx_out,
                                 int64_t* count_out, void* workspace, int64_t workspace_bytes,
                                 void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  TLCE_REQUIRE(n >= 0 && n < (int64_t)INT32_MAX, "compact_mask: n=%lld out of range",
               (long long)n);
  TLCE_REQUIRE(count_out != nullptr, "compact_mask: count_out is null");
  if (n == 0) return tlce_fill_zero(count_out, sizeof(int64_t), stream_);
  TLCE_REQUIRE(mask && row_idx_out && workspace, "compact_mask: null pointer");
  return compact_flags(MaskFlags{mask}, n, row_idx_out, count_out, workspace, workspace_bytes,
                       stream);
}

extern "C" int tlce_gather_rows(const void* src, const int64_t* row_idx, int64_t m,
                                int64_t row_bytes, void* dst, void* stream) {
  return move_rows<true>(src, row_idx, m, row_bytes, dst, static_cast<hipStream_t>(stream));
}

extern "C" int tlce_scatter_rows(const void* src, const int64_t* row_idx, int64_t m,
                                 int64_t row_bytes, void* dst, void* stream) {
  return move_rows<false>(src, row_idx, m, row_bytes, dst, static_cast<hipStream_t>(stream));
}

extern "C" int tlce_gather_loss_rows(const void* hidden_src, const int64_t* labels_src,
                                     const float* weights_src, const int64_t* row_idx,
                                     const int64_t* row_count, int64_t capacity,
                                     int64_t padded_rows, int64_t row_bytes,
                                     int64_t ignore_index, void* hidden_dst,
                                     int64_t* labels_dst, float* weights_dst, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  TLCE_REQUIRE(capacity >= 0 && padded_rows >= capacity && row_bytes > 0,
               "gather_loss_rows: bad sizes");
  if (capacity == 0) return 0;
  TLCE_REQUIRE(hidden_src && labels_src && row_idx && row_count && hidden_dst && labels_dst,
               "gather_loss_rows: null pointer");
  TLCE_REQUIRE((weights_src == nullptr) == (weights_dst == nullptr),
               "gather_loss_rows: weights source and destination go together");
  const int vb = pick_vector_bytes(hidden_src, hidden_dst, row_bytes);
  const int64_t vpr = row_bytes / vb;
  TLCE_REQUIRE(vpr <= INT32_MAX, "gather_loss_rows: row too long");
  const int grid = (int)std::min<int64_t>(padded_rows, 256 * 32);
#define TLCE_GATHER(V)                                                                      \
  gather_loss_rows_kernel<V><<<grid, 256, 0, stream>>>(                                     \
      static_cast<const V*>(hidden_src), labels_src, weights_src, row_idx, row_count,       \
      capacity, padded_rows, (int)vpr, ignore_index, static_cast<V*>(hidden_dst), labels_dst,         \
      weights_dst)
  switch (vb) {
    case 16: TLCE_GATHER(uint4); break;
    case 8: TLCE_GATHER(uint2); break;
    case 4: TLCE_GATHER(uint32_t); break;
    case 2: TLCE_GATHER(uint16_t); break;
    default: TLCE_GATHER(uint8_t); break;
  }
#undef TLCE_GATHER
  TLCE_LAUNCH_CHECK();
  return 0;
}
