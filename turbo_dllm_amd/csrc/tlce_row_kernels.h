// Kernels of the fused linear cross-entropy that do not depend on a tile engine or
// an element type: per-row scales, the KL finish, the top-k scan and the zero fill.
// Compiled once, in the translation unit that holds the C ABI; the engine
// translation units reach them through the launch_* / fill_zero host functions.
#pragma once

#include "tlce_kernels.h"

namespace tlce {

__global__ __launch_bounds__(256) void lce_token_scale_kernel(ScaleArgs p) {
  const int r = blockIdx.x * 256 + threadIdx.x;
  if (r >= p.mp) return;
  p.m = effective_rows(p.m, p.m_dev);
  float s = 0.0f;
  if (p.labels == nullptr) {
    // no labels: every real row gets grad_output[r] (per-row objectives) or the constant
    s = (r < p.m) ? (p.grad_output != nullptr ? p.grad_output[r] : p.constant) : 0.0f;
  } else if (r < p.m && p.labels[r] != p.ignore) {
    if (p.reduction == TLCE_REDUCTION_NONE) {
      s = p.grad_output[(p.row_idx != nullptr) ? p.row_idx[r] : (int64_t)r];
    } else if (p.reduction == TLCE_REDUCTION_SUM) {
      s = p.grad_output[0];
    } else {
      s = p.grad_output[0] / p.valid_count[0];
    }
  }
  if (p.token_weights != nullptr && r < p.m) s *= p.token_weights[r];
  p.scale[r] = s * p.multiplier;
}

// out[0] = sum of x[0..n) in a fixed order (one workgroup, pairwise tree): the
// weighted loss sum of the masked-token loss, reproducible run to run.
__global__ __launch_bounds__(1024) void lce_sum_kernel(const float* __restrict__ x, int n,
                                                       float* __restrict__ out) {
  __shared__ float part[1024];
  float s = 0.0f;
  for (int i = threadIdx.x; i < n; i += 1024) s += x[i];
  part[threadIdx.x] = s;
  __syncthreads();
  for (int o = 512; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) part[threadIdx.x] += part[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[0] = part[0];
}

// Per-sample numerators of the DFlash loss (numerators.scatter_add_(0, sample_indices,
// token_loss * position_weights), dflash/model.py:925-937) without atomics: the
// compacted rows are in ascending position order, so the rows of sample s (positions
// [s * segment_length, (s + 1) * segment_length)) are one contiguous run of row_idx,
// found by two binary searches; one workgroup per sample adds the run in a fixed
// order (strided partial sums, then a pairwise tree): reproducible run to run.
__global__ __launch_bounds__(256) void lce_segment_weighted_sum_kernel(
    const float* __restrict__ values, const float* __restrict__ weights,
    const int64_t* __restrict__ row_idx, const int64_t* __restrict__ row_count, int64_t m,
    int64_t segment_length, float* __restrict__ out) {
  __shared__ float part[256];
  if (row_count != nullptr) {
    const int64_t c = *row_count;
    m = c < 0 ? 0 : (c < m ? c : m);
  }
  auto lower_bound = [&](int64_t position) -> int64_t {   // first r with row_idx[r] >= position
    int64_t lo = 0, hi = m;
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if (row_idx[mid] < position) lo = mid + 1;
      else hi = mid;
    }
    return lo;
  };
  const int64_t first = lower_bound((int64_t)blockIdx.x * segment_length);
  const int64_t last = lower_bound(((int64_t)blockIdx.x + 1) * segment_length);
  float s = 0.0f;
  for (int64_t r = first + threadIdx.x; r < last; r += 256)
    s += weights != nullptr ? values[r] * weights[r] : values[r];
  part[threadIdx.x] = s;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) part[threadIdx.x] += part[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[blockIdx.x] = part[0];
}

// losses[r] = sum_t loss_part[t][r] + (sum_t tsum_part[t][r]) * lse_draft[r] + 1 over the
// vocabulary tiles t (see lce_kl_panel_kernel), in a fixed order: 64 rows per workgroup of
// 16 waves, the rows across the lanes; wave w adds the tiles w, w + 16, ... in ascending
// order and the 16 sums are merged in wave order.
constexpr int kKlFinishWaves = 16;

__global__ __launch_bounds__(64 * kKlFinishWaves) void lce_kl_finish_kernel(
    float* losses, const float* loss_part, const float* tsum_part, int n_tiles, int64_t part_ld,
    const float* lse, int m) {
  __shared__ float sh_loss[kKlFinishWaves][64];
  __shared__ float sh_mass[kKlFinishWaves][64];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = blockIdx.x * 64 + lane;
  float loss = 0.0f, mass = 0.0f;
  if (r < m) {
    for (int t = wave; t < n_tiles; t += kKlFinishWaves) {
      loss += loss_part[(int64_t)t * part_ld + r];
      mass += tsum_part[(int64_t)t * part_ld + r];
    }
  }
  sh_loss[wave][lane] = loss;
  sh_mass[wave][lane] = mass;
  __syncthreads();
  if (wave != 0 || r >= m) return;
  loss = 0.0f;
  mass = 0.0f;
#pragma unroll
  for (int w = 0; w < kKlFinishWaves; ++w) {
    loss += sh_loss[w][lane];
    mass += sh_mass[w][lane];
  }
  losses[r] = loss + mass * lse[r] + 1.0f;
}

// Ordering of (value, id) pairs: larger value first, then smaller id.
__device__ __forceinline__ bool topk_before(float va, int64_t ia, float vb, int64_t ib) {
  return va > vb || (va == vb && ia < ib);
}

// The best (value, id) pair over the workgroup's 256 threads, returned to all
// of them; ends on a barrier-free read of red_*, so callers synchronise before
// the next call.
__device__ __forceinline__ void topk_workgroup_best(float& best_val, int64_t& best_id,
                                                    float* red_val, int64_t* red_id) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best_val, o, 64);
    const int64_t oi = __shfl_xor(best_id, o, 64);
    if (topk_before(ov, oi, best_val, best_id)) {
      best_val = ov;
      best_id = oi;
    }
  }
  if (lane == 0) {
    red_val[wave] = best_val;
    red_id[wave] = best_id;
  }
  __syncthreads();
  best_val = red_val[0];
  best_id = red_id[0];
#pragma unroll
  for (int w = 1; w < 4; ++w) {
    if (topk_before(red_val[w], red_id[w], best_val, best_id)) {
      best_val = red_val[w];
      best_id = red_id[w];
    }
  }
}

__global__ __launch_bounds__(256) void lce_topk_scan_kernel(TopkScanArgs p) {
  constexpr int kPerThread = 64;
  constexpr int kChunk = kPerThread * 256;
  constexpr int kSlots = 3;                       // gathered pairs per thread
  constexpr int kCapacity = kSlots * 256;
  __shared__ float list_val[256];
  __shared__ int64_t list_id[256];
  __shared__ float cand_val[kCapacity];
  __shared__ int64_t cand_id[kCapacity];
  __shared__ float red_val[4];
  __shared__ int64_t red_id[4];
  __shared__ float red_f[4];
  __shared__ int wave_total[4];
  __shared__ float tmax[256];
  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const int row = blockIdx.x;
  const float* src = p.panel + (int64_t)row * p.ld;
  float run_max = p.first ? -INFINITY : p.run_max[row];
  float run_sum = p.first ? 0.0f : p.run_sum[row];
  if (t < p.k) {
    // placeholders get distinct negative ids so that they stay distinguishable
    list_val[t] = p.first ? -INFINITY : p.top_values[(int64_t)row * p.k + t];
    list_id[t] = p.first ? (int64_t)(-1 - t) : p.top_ids[(int64_t)row * p.k + t];
  }
  __syncthreads();

  for (int c0 = 0; c0 < p.width; c0 += kChunk) {
    float vals[kPerThread];
    float local_max = -INFINITY;
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int idx = c0 + t + 256 * i;
      vals[i] = idx < p.width ? src[idx] : -INFINITY;
      local_max = fmaxf(local_max, vals[i]);
    }
    // running softmax statistics
    const float m = wave_max(local_max);
    if (lane == 0) red_f[wave] = m;
    __syncthreads();
    const float new_max =
        fmaxf(run_max, fmaxf(fmaxf(red_f[0], red_f[1]), fmaxf(red_f[2], red_f[3])));
    __syncthreads();
    float local_sum = 0.0f;
    if (new_max > -INFINITY) {
#pragma unroll
      for (int i = 0; i < kPerThread; ++i) local_sum += __expf(vals[i] - new_max);
    }
    local_sum = wave_sum(local_sum);
    if (lane == 0) red_f[wave] = local_sum;
    __syncthreads();
    run_sum = (run_max > -INFINITY ? run_sum * __expf(run_max - new_max) : 0.0f) +
              (red_f[0] + red_f[1] + red_f[2] + red_f[3]);
    run_max = new_max;

    // the list entry this thread carries into the selection
    const float own_val = t < p.k ? list_val[t] : -INFINITY;
    const int64_t own_id = t < p.k ? list_id[t] : INT64_MAX;
    float kth = list_val[p.k - 1];
    bool inclusive = false;
    if (kth == -INFINITY && p.k <= 256) {
      // nothing to compare with yet (a row's first logits): the k-th largest
      // of the 256 per-thread maxima is a value at least k logits reach
      __syncthreads();
      tmax[t] = local_max;
      __syncthreads();
      int before = 0;
      for (int j = 0; j < 256; ++j) {
        const float other = tmax[j];
        before += (other > local_max || (other == local_max && j < t)) ? 1 : 0;
      }
      if (before == p.k - 1) red_f[0] = local_max;
      __syncthreads();
      kth = red_f[0];
      inclusive = true;
      __syncthreads();
    }
    auto beats = [&](float v) { return inclusive ? v >= kth : v > kth; };
    auto chunk_id = [&](int i) -> int64_t {
      return (c0 + t + 256 * i < p.width) ? p.v0 + c0 + t + 256 * i : INT64_MAX;
    };
    // gather the logits that beat the current k-th value: count per thread,
    // exclusive prefix over the workgroup (no atomics), then write
    int mine = 0;
#pragma unroll
    for (int i = 0; i < kPerThread; ++i)
      mine += (beats(vals[i]) && c0 + t + 256 * i < p.width) ? 1 : 0;
    int scan = mine;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(scan, o, 64);
      if (lane >= o) scan += up;
    }
    if (lane == 63) wave_total[wave] = scan;
    __syncthreads();
    int offset = scan - mine;
    for (int w = 0; w < wave; ++w) offset += wave_total[w];
    const int n_cand = wave_total[0] + wave_total[1] + wave_total[2] + wave_total[3];
    if (n_cand <= kCapacity && mine > 0) {
#pragma unroll
      for (int i = 0; i < kPerThread; ++i) {
        if (beats(vals[i]) && c0 + t + 256 * i < p.width) {
          cand_val[offset] = vals[i];
          cand_id[offset] = chunk_id(i);
          ++offset;
        }
      }
    }
    __syncthreads();
    if (n_cand > kCapacity) {
      // too many to gather (rare): selection rounds over the whole chunk, eight
      // logits per thread at a time, read again from memory
      float prev_val = INFINITY;
      int64_t prev_id = INT64_MIN;
      for (int r = 0; r < p.k; ++r) {
        float best_val = -INFINITY;
        int64_t best_id = INT64_MAX;
        if (t < p.k && topk_before(prev_val, prev_id, own_val, own_id)) {
          best_val = own_val;
          best_id = own_id;
        }
        for (int i = 0; i < kPerThread; ++i) {
          const int idx = c0 + t + 256 * i;
          if (idx >= p.width) break;
          const float v = src[idx];
          const int64_t d = p.v0 + idx;
          if (topk_before(prev_val, prev_id, v, d) && topk_before(v, d, best_val, best_id)) {
            best_val = v;
            best_id = d;
          }
        }
        topk_workgroup_best(best_val, best_id, red_val, red_id);
        if (t == 0) {
          list_val[r] = best_val;
          list_id[r] = best_id;
        }
        prev_val = best_val;
        prev_id = best_id;
        __syncthreads();
      }
    } else if (n_cand > 0) {
      // merge by rank: the place of a pair in the new list is the number of
      // pairs, old and gathered, that come before it (ids are unique)
      int own_rank = t;
      if (t < p.k) {
        for (int c = 0; c < n_cand; ++c)
          own_rank += topk_before(cand_val[c], cand_id[c], own_val, own_id) ? 1 : 0;
      }
      int rank[kSlots];
      float gv[kSlots];
      int64_t gi[kSlots];
#pragma unroll
      for (int q = 0; q < kSlots; ++q) {
        const int pos = t + 256 * q;
        rank[q] = p.k;
        if (pos < n_cand) {
          gv[q] = cand_val[pos];
          gi[q] = cand_id[pos];
          int before = 0;
          for (int j = 0; j < p.k; ++j)
            before += topk_before(list_val[j], list_id[j], gv[q], gi[q]) ? 1 : 0;
          for (int c = 0; c < n_cand; ++c)
            before += topk_before(cand_val[c], cand_id[c], gv[q], gi[q]) ? 1 : 0;
          rank[q] = before;
        }
      }
      __syncthreads();
      if (t < p.k && own_rank < p.k) {
        list_val[own_rank] = own_val;
        list_id[own_rank] = own_id;
      }
#pragma unroll
      for (int q = 0; q < kSlots; ++q) {
        if (rank[q] < p.k) {
          list_val[rank[q]] = gv[q];
          list_id[rank[q]] = gi[q];
        }
      }
    }
    __syncthreads();
  }
  if (t < p.k) {
    p.top_values[(int64_t)row * p.k + t] = list_val[t];
    p.top_ids[(int64_t)row * p.k + t] = list_id[t];
  }
  if (t == 0) {
    p.run_max[row] = run_max;
    p.run_sum[row] = run_sum;
  }
}

__global__ __launch_bounds__(256) void lce_fill_zero_kernel(uint4* __restrict__ dst16,
                                                            int64_t n16, unsigned char* tail,
                                                            int ntail) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  const uint4 z = make_uint4(0u, 0u, 0u, 0u);
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) dst16[i] = z;
  if (blockIdx.x == 0 && (int)threadIdx.x < ntail) tail[threadIdx.x] = 0;
}

}  // namespace tlce
