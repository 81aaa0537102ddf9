// Row kernels of the forward that leaves the gradients (tlce_fused.h): the
// label-logit pass before the blocks, the per-block statistics / row-factor pass,
// the K-split reduction of grad_hidden and the final scale-and-cast.  Engine
// independent; compiled beside the C ABI.
#pragma once

#include "tlce_fused.h"

namespace tlce {

// One wave per row, 16 rows per workgroup (one atomic per workgroup for the count
// of rows with a loss).
template <typename T>
__global__ __launch_bounds__(256) void lce_label_logit_kernel(LabelLogitArgs p) {
  __shared__ int block_valid;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) block_valid = 0;
  __syncthreads();
  p.m = effective_rows(p.m, p.m_dev);
  int wave_valid = 0;
  for (int i = 0; i < 4; ++i) {
    const int r = blockIdx.x * 16 + wave * 4 + i;
    if (r >= p.m) continue;
    const int64_t label = p.labels[r];
    const bool valid = label != p.ignore;
    const bool here = valid && label >= 0 && label < p.v;
    float z = 0.0f;
    if (here) {
      const T* hrow = static_cast<const T*>(p.hidden) + (int64_t)r * p.h;
      const T* wrow = static_cast<const T*>(p.weight) + label * (int64_t)p.h;
      z = wave_dot<T>(hrow, wrow, p.h, lane) * p.logit_scale;
      if (p.softcap > 0.0f) z = p.softcap * tanhf(z / p.softcap);
    }
    if (lane == 0) {
      // a label on the excluded column or outside the vocabulary has no logit in the
      // loss (ce_forward_kernel, fused_linear_ce_cuda.cu:199-219); as a reference any
      // real column's logit serves
      p.target[r] = (here && label != p.exclude) ? z : 0.0f;
      p.ref[r] = valid ? z : INFINITY;
    }
    wave_valid += valid ? 1 : 0;
  }
  if (lane == 0 && wave_valid != 0) atomicAdd(&block_valid, wave_valid);
  __syncthreads();
  if (threadIdx.x == 0 && block_valid != 0) atomicAdd(p.valid_count, (float)block_valid);
}

// 64 rows per workgroup.  First the per-tile partials of the 64 rows are added up
// with the rows across the lanes (coalesced: partials are stored [tile][row]), each
// quarter of the workgroup taking every fourth vocabulary tile in order and the
// four quarter sums merged in a fixed order; then each wave finishes 16 rows (rows
// past m only get their zero row of scaled_hidden and a zero row factor).
constexpr int kFusedRowsPerBlock = 64;

template <typename T>
__global__ __launch_bounds__(256) void lce_fused_rows_kernel(FusedRowsArgs p) {
  if (p.run_flag != nullptr && *p.run_flag == 0) return;
  if (p.m_dev != nullptr) {
    p.m = effective_block_rows(p.m, p.m_dev, p.row0);
    p.m_pad = min(p.m_pad, (p.m + 255) / 256 * 256);   // the token tiles the producer wrote
  }
  __shared__ float sh_sum[4][kFusedRowsPerBlock];
  __shared__ float sh_max[4][kFusedRowsPerBlock];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int row0 = blockIdx.x * kFusedRowsPerBlock;
  {
    const int r = row0 + lane;
    float sum = 0.0f, mx2 = -INFINITY;
    if (r < p.m) {
      for (int t = wave; t < p.n_vtiles; t += 4) {
        sum += p.part_sum[(int64_t)t * p.part_ld + r];
        mx2 = fmaxf(mx2, p.part_max[(int64_t)t * p.part_ld + r]);
      }
    }
    sh_sum[wave][lane] = sum;
    sh_max[wave][lane] = mx2;
  }
  __syncthreads();
  T* scaled = static_cast<T*>(p.scaled_hidden);
  for (int i = 0; i < kFusedRowsPerBlock / 4; ++i) {
    const int rr = wave * (kFusedRowsPerBlock / 4) + i;
    const int r = row0 + rr;
    if (r >= p.m_pad) return;
    float factor = 0.0f;
    if (r < p.m) {
      const float c = p.ref[r];
      const bool live = c < INFINITY;   // rows without loss carry +inf
      const float sum = ((sh_sum[0][rr] + sh_sum[1][rr]) + sh_sum[2][rr]) + sh_sum[3][rr];
      const float mx = fmaxf(fmaxf(sh_max[0][rr], sh_max[1][rr]),
                             fmaxf(sh_max[2][rr], sh_max[3][rr])) * TLCE_LN2;
      const bool in_window = (mx - c <= p.window) && (mx - c >= -1.0f) && (sum > 0.0f) &&
                             (sum < 3.0e38f);
      const float lse = live ? c + logf(sum) : 0.0f;
      const float target = p.target[r];
      const float w = (p.token_weights != nullptr) ? p.token_weights[r] : 1.0f;
      const int64_t label = p.labels[r];
      if (live) factor = w * p.logit_scale / sum;
      if (lane == 0) {
        p.lse[r] = lse;
        if (p.losses != nullptr) {
          const int64_t o = (p.row_idx != nullptr) ? p.row_idx[r] : p.loss_row0 + r;
          p.losses[o] = live ? lse - target : 0.0f;
        }
        p.ref_next[r] = (live && !in_window) ? mx : c;
        if (live && !in_window) atomicOr(p.redo, 1);
        // the label's entry: s * entry = (softmax - 1) * cap'
        if (live && label >= 0 && label < p.v && label != p.exclude) {
          float dcap = 1.0f;
          if (p.softcap > 0.0f) {
            const float t = target / p.softcap;
            dcap = 1.0f - t * t;
          }
          const float entry = (expf(target - c) - sum) * dcap;
          static_cast<T*>(p.panel)[(int64_t)r * p.ld + label] = from_float<T>(entry);
        }
        p.row_scale[r] = factor;
      }
    } else if (lane == 0) {
      p.row_scale[r] = 0.0f;
    }
    if (scaled != nullptr) {
      const T* hrow = static_cast<const T*>(p.hidden) + (int64_t)min(r, p.m - 1) * p.h;
      T* out = scaled + (int64_t)r * p.h;
      if ((p.h % 8) == 0) {
        typedef T v8_t __attribute__((ext_vector_type(8)));
        for (int k = lane * 8; k < p.h; k += 64 * 8) {
          const v8_t x = *reinterpret_cast<const v8_t*>(hrow + k);
          v8_t y;
#pragma unroll
          for (int e = 0; e < 8; ++e) y[e] = from_float<T>(to_float<T>(x[e]) * factor);
          *reinterpret_cast<v8_t*>(out + k) = y;
        }
      } else {
        for (int k = lane; k < p.h; k += 64) out[k] = from_float<T>(to_float<T>(hrow[k]) * factor);
      }
    }
  }
}

// One wave per row, 16 rows per workgroup.
template <typename T>
__global__ __launch_bounds__(256) void lce_scale_rows_kernel(ScaleRowsArgs p) {
  float g = 0.0f;
  if (p.reduction != TLCE_REDUCTION_NONE) g = p.grad_output[0];
  if (p.reduction == TLCE_REDUCTION_MEAN) {
    const float count = p.valid_count[0];
    g = count > 0.0f ? g / count : 0.0f;
  }
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int m = effective_rows(p.m, p.m_dev);
  for (int i = 0; i < 4; ++i) {
    const int r = blockIdx.x * 16 + wave * 4 + i;
    if (r >= p.m_pad) return;
    if (p.reduction == TLCE_REDUCTION_NONE && r < m)
      g = p.grad_output[p.row_idx != nullptr ? p.row_idx[r] : (int64_t)r];
    const float factor = (r < m) ? g * p.row_scale[r] : 0.0f;
    const T* hrow = static_cast<const T*>(p.hidden) + (int64_t)min(r, max(m - 1, 0)) * p.h;
    T* out = static_cast<T*>(p.out) + (int64_t)r * p.h;
    typedef T v8_t __attribute__((ext_vector_type(8)));
    for (int k = lane * 8; k < p.h; k += 64 * 8) {
      v8_t y;
      if (r < m) {
        const v8_t x = *reinterpret_cast<const v8_t*>(hrow + k);
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = from_float<T>(to_float<T>(x[e]) * factor);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = from_float<T>(0.0f);
      }
      *reinterpret_cast<v8_t*>(out + k) = y;
    }
  }
}

__global__ __launch_bounds__(256) void lce_reduce_scaled_slabs_kernel(ReduceSlabsArgs p) {
  const int r = blockIdx.x;
  if (p.m_dev != nullptr) {
    const int rows = effective_block_rows(p.m, p.m_dev, p.row0);
    if (r >= rows) return;
    p.n_splits = dynamic_k_splits((rows + p.tile - 1) / p.tile, p.n_htiles, p.tile, p.h,
                                  p.launched_splits, p.slab_budget, p.k_steps, &p.split_stride);
  }
  const float s = p.row_scale[r];
  const float* src = p.slabs + (int64_t)r * p.h;
  for (int k = threadIdx.x * 4; k < p.h; k += 256 * 4) {
    f32x4_t sum = *reinterpret_cast<const f32x4_t*>(src + k);
    for (int q = 1; q < p.n_splits; ++q)
      sum += *reinterpret_cast<const f32x4_t*>(src + (int64_t)q * p.split_stride + k);
    sum = sum * s;
    if (p.out_t != nullptr) {
      store4<__bf16>(static_cast<__bf16*>(p.out_t) + (int64_t)r * p.h + k, sum[0], sum[1], sum[2],
                     sum[3]);
    } else {
      *reinterpret_cast<f32x4_t*>(p.out + (int64_t)r * p.h + k) = sum;
    }
  }
}

// blockIdx.x = row, blockIdx.y = a group of 8 vocabulary tiles: 32 threads per tile, 8
// columns each.  The logit gradient of the frozen-head KL from the two panels the
// forward left (rows from m on get zeros).
__global__ __launch_bounds__(256) void lce_kl_grad_from_exp_kernel(KlGradFromExpArgs p,
                                                                   int n_vtiles) {
  const int r = blockIdx.x;
  const int tile = blockIdx.y * 8 + (threadIdx.x >> 5);
  if (tile >= n_vtiles) return;
  const int64_t c = (int64_t)tile * 256 + (threadIdx.x & 31) * 8;
  __bf16* e = static_cast<__bf16*>(p.exp_panel) + (int64_t)r * p.ld + c;
  typedef __bf16 v8_t __attribute__((ext_vector_type(8)));
  v8_t out;
  if (r < p.m && p.teacher == nullptr) {
    // only normalise: softmax (times what the caller folded into draft_lse)
    const float f = exp2f(p.part_max[(int64_t)tile * p.part_ld + r] -
                          p.draft_lse[r] * TLCE_LOG2E);
    const v8_t ev = *reinterpret_cast<const v8_t*>(e);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = from_float<__bf16>(to_float<__bf16>(ev[i]) * f);
  } else if (r < p.m) {
    const float tile_max2 = p.part_max[(int64_t)tile * p.part_ld + r];
    const float f = exp2f(tile_max2 - p.draft_lse[r] * TLCE_LOG2E);
    const float ft = p.t_part_max != nullptr
                         ? exp2f(p.t_part_max[(int64_t)tile * p.part_ld + r] -
                                 p.t_lse[r] * TLCE_LOG2E)
                         : 1.0f;
    const float inv_cap = p.softcap > 0.0f ? TLCE_LN2 / p.softcap : 0.0f;
    const v8_t ev = *reinterpret_cast<const v8_t*>(e);
    const v8_t tv = *reinterpret_cast<const v8_t*>(static_cast<const __bf16*>(p.teacher) +
                                                   (int64_t)r * p.ld + c);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float ei = to_float<__bf16>(ev[i]);
      float g = ei * f - to_float<__bf16>(tv[i]) * ft;
      if (p.softcap > 0.0f) {
        // (an entry of 0 is a column past the vocabulary: its gradient is 0 anyway)
        const float t = ei > 0.0f ? (log2f(ei) + tile_max2) * inv_cap : 0.0f;
        g *= fmaxf(1.0f - t * t, 0.0f);   // (|z| <= cap: a rounded entry can say otherwise)
      }
      out[i] = from_float<__bf16>(g);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = from_float<__bf16>(0.0f);
  }
  *reinterpret_cast<v8_t*>(e) = out;
}

// One row and 2048 columns per workgroup, 8 columns per thread.
__global__ __launch_bounds__(256) void lce_exp_from_logits_kernel(ExpFromLogitsArgs p) {
  const int r = blockIdx.x;
  const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (c >= p.width) return;
  __bf16* dst = static_cast<__bf16*>(p.out) + (int64_t)r * p.ld_out + p.col0 + c;
  if (r >= p.m) {
    store4<__bf16>(dst, 0.0f, 0.0f, 0.0f, 0.0f);
    store4<__bf16>(dst + 4, 0.0f, 0.0f, 0.0f, 0.0f);
    return;
  }
  const float ref = p.run_max[r];
  if (c == 0) p.ref_used[r] = ref;
  const float* src = p.logits + (int64_t)r * p.ld + c;
  const f32x4_t z0 = *reinterpret_cast<const f32x4_t*>(src);
  const f32x4_t z1 = *reinterpret_cast<const f32x4_t*>(src + 4);
  float e[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float z = i < 4 ? z0[i] : z1[i - 4];
    float x = __expf(z - ref);            // -inf (past the vocabulary) gives 0
    if (p.softcap > 0.0f) {
      const float t = z / p.softcap;
      x = (z > -INFINITY) ? x * (1.0f - t * t) : 0.0f;
    }
    e[i] = x;
  }
  store4<__bf16>(dst, e[0], e[1], e[2], e[3]);
  store4<__bf16>(dst + 4, e[4], e[5], e[6], e[7]);
}

// blockIdx.y = logits panel (all but the last, which was written with the final
// maxima): rows whose maximum grew after the panel was written are brought to the
// final reference.
__global__ __launch_bounds__(256) void lce_rescale_exp_rows_kernel(RescaleExpArgs p) {
  const int r = blockIdx.x;
  const int j = blockIdx.y;
  const float used = p.ref_used[(int64_t)j * p.m_pad + r];
  const float fin = p.run_max[r];
  if (used == fin) return;
  const float f = __expf(used - fin);
  const int64_t c0 = (int64_t)j * p.panel_width;
  const int64_t c1 = min(c0 + p.panel_width, p.total_width);
  __bf16* row = static_cast<__bf16*>(p.panel) + (int64_t)r * p.ld;
  typedef __bf16 v8_t __attribute__((ext_vector_type(8)));
  for (int64_t c = c0 + threadIdx.x * 8; c < c1; c += 256 * 8) {
    v8_t x = *reinterpret_cast<v8_t*>(row + c);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = from_float<__bf16>(to_float<__bf16>(x[i]) * f);
    *reinterpret_cast<v8_t*>(row + c) = x;
  }
}

__global__ __launch_bounds__(256) void lce_topk_row_scale_kernel(TopkRowScaleArgs p) {
  const int r = blockIdx.x * 256 + threadIdx.x;
  if (r >= p.m_pad) return;
  p.row_scale[r] = (r < p.m) ? p.multiplier / p.run_sum[r] : 0.0f;
}

// One workgroup per row: grad_hidden[r, :] = ce_scale[r] * unit[r, :]
//   - ce_scale[r] * d'(label) * W[label] + sum_j grad_top_values[r, j] * d'(id_j) * W[id_j]
// (dflash_linear_topk.py:196-225) with d'(v) = multiplier * (1 - tanh^2(multiplier *
// h.W[v] / cap)) (multiplier alone without a cap), rounded once.  The coefficients
// of the single-row terms are formed first (under a soft cap one dot product each, a
// wave per entry), then every column is summed in float32.
constexpr int kTopkApplyMaxEntries = 257;   // top_k <= 256, plus the label

template <typename T>
__global__ __launch_bounds__(256) void lce_topk_apply_kernel(TopkApplyArgs p) {
  __shared__ float coef[kTopkApplyMaxEntries];
  __shared__ int64_t ids[kTopkApplyMaxEntries];
  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const int r = blockIdx.x;
  const T* hrow = static_cast<const T*>(p.hidden) + (int64_t)r * p.h;
  const float scale = p.ce_scale[r];
  const int n_entries = (p.grad_top_values != nullptr ? p.k : 0) + 1;
  // one wave per entry, the waves taking every fourth: the raw logit is needed only for
  // the soft cap's derivative
  for (int e = wave; e < n_entries; e += 4) {
    const bool is_label = e == n_entries - 1;
    const int64_t id = is_label ? p.labels[r] : p.top_ids[(int64_t)r * p.k + e];
    const float weight_in = is_label ? -scale : p.grad_top_values[(int64_t)r * p.k + e];
    float deriv = p.logit_scale;
    if (p.softcap > 0.0f && weight_in != 0.0f) {   // wave-uniform
      const T* wrow = static_cast<const T*>(p.weight) + id * (int64_t)p.h;
      const float raw = wave_dot<T>(hrow, wrow, p.h, lane) * p.logit_scale;
      const float th = tanhf(raw / p.softcap);
      deriv *= 1.0f - th * th;
    }
    if (lane == 0) {
      coef[e] = weight_in * deriv;
      ids[e] = id;
    }
  }
  __syncthreads();
  // eight consecutive columns per thread and step (h is a multiple of 64 on this path):
  // 16-byte reads of the weight rows, 16-byte store
  const float* unit = p.unit + (int64_t)r * p.h;
  T* out = static_cast<T*>(p.grad_hidden) + (int64_t)r * p.h;
  typedef T v8_t __attribute__((ext_vector_type(8)));
  for (int k = t * 8; k < p.h; k += 256 * 8) {
    const f32x4_t u0 = *reinterpret_cast<const f32x4_t*>(unit + k);
    const f32x4_t u1 = *reinterpret_cast<const f32x4_t*>(unit + k + 4);
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = scale * (i < 4 ? u0[i] : u1[i - 4]);
    for (int e = 0; e < n_entries; ++e) {
      const float c = coef[e];
      if (c == 0.0f) continue;   // workgroup-uniform
      const v8_t w = *reinterpret_cast<const v8_t*>(static_cast<const T*>(p.weight) +
                                                    ids[e] * (int64_t)p.h + k);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(c, to_float<T>(w[i]), acc[i]);
    }
    v8_t o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = from_float<T>(acc[i]);
    *reinterpret_cast<v8_t*>(out + k) = o;
  }
}

// 64 rows per workgroup of 16 waves, the rows across the lanes (the partials are
// stored [tile][row]: a wave reads 256 consecutive bytes per tile); wave w adds the
// tiles w, w + 16, ... in order and the 16 sums are merged in a fixed order.
constexpr int kSoftRowsWaves = 16;

__global__ __launch_bounds__(64 * kSoftRowsWaves) void lce_soft_rows_kernel(SoftRowsArgs p) {
  __shared__ float sh[kSoftRowsWaves][64];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = blockIdx.x * 64 + lane;
  float sum = 0.0f;
  if (r < p.m) {
    for (int t = wave; t < p.n_vtiles; t += kSoftRowsWaves)
      sum += p.part_sum[(int64_t)t * p.part_ld + r];
  }
  sh[wave][lane] = sum;
  __syncthreads();
  if (wave != 0 || r >= p.m_pad) return;
  sum = 0.0f;
#pragma unroll
  for (int w = 0; w < kSoftRowsWaves; ++w) sum += sh[w][lane];
  p.row_scale[r] = (r < p.m && sum > 0.0f) ? p.scale / sum : 0.0f;
}

// The tiles' (maximum, sum) pairs of an emitting pass merged into lse - log(scale), the
// same way: 64 rows per workgroup of 16 waves, wave w merging the tiles w, w + 16, ...
// in ascending order, the 16 partial pairs merged in wave order.
__global__ __launch_bounds__(64 * kSoftRowsWaves) void lce_emit_rows_kernel(EmitRowsArgs p) {
  __shared__ float sh_max[kSoftRowsWaves][64];
  __shared__ float sh_sum[kSoftRowsWaves][64];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = blockIdx.x * 64 + lane;
  float mx = -INFINITY, sum = 0.0f;
  if (r < p.m) {
    for (int t = wave; t < p.n_vtiles; t += kSoftRowsWaves) {
      const float pm = p.part_max[(int64_t)t * p.part_ld + r];
      const float ps = p.part_sum[(int64_t)t * p.part_ld + r];
      if (pm > -INFINITY) {
        const float nm = fmaxf(mx, pm);
        sum = sum * exp2f(mx - nm) + ps * exp2f(pm - nm);   // (exp2f(-inf) = 0 the first time)
        mx = nm;
      }
    }
  }
  sh_max[wave][lane] = mx;
  sh_sum[wave][lane] = sum;
  __syncthreads();
  if (wave != 0 || r >= p.m_pad) return;
  if (r >= p.m) {
    p.lse[r] = 0.0f;
    p.row_scale[r] = 0.0f;
    return;
  }
  mx = -INFINITY;
#pragma unroll
  for (int w = 0; w < kSoftRowsWaves; ++w) mx = fmaxf(mx, sh_max[w][lane]);
  sum = 0.0f;
#pragma unroll
  for (int w = 0; w < kSoftRowsWaves; ++w)
    if (sh_max[w][lane] > -INFINITY) sum += sh_sum[w][lane] * exp2f(sh_max[w][lane] - mx);
  p.lse[r] = (mx + log2f(sum)) * TLCE_LN2 - logf(p.scale);
  p.row_scale[r] = 1.0f;
}

template <typename T>
__global__ __launch_bounds__(256) void lce_scale_cast_rows_kernel(ScaleCastArgs p) {
  const int64_t r = blockIdx.x;
  if (p.m_dev != nullptr && r >= *p.m_dev) return;
  const int64_t o = (p.row_idx != nullptr) ? p.row_idx[r] : r;
  float g = p.grad_output[p.reduction == TLCE_REDUCTION_NONE ? o : 0];
  if (p.reduction == TLCE_REDUCTION_MEAN) {
    // no row with a loss: every gradient entry is zero and stays zero
    const float count = p.valid_count[0];
    g = count > 0.0f ? g / count : 0.0f;
  }
  const float* src = p.in + r * p.h;
  T* dst = static_cast<T*>(p.out) + o * p.h;
  for (int k = threadIdx.x * 4; k < p.h; k += 256 * 4) {
    const f32x4_t x = *reinterpret_cast<const f32x4_t*>(src + k);
    store4<T>(dst + k, x[0] * g, x[1] * g, x[2] * g, x[3] * g);
  }
}

}  // namespace tlce
