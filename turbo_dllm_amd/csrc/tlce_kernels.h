// Device kernels of the fused linear cross-entropy, templated on a tile engine
// (MfmaEngine for bf16/f16, SimtEngine for the generic float32-FMA path).
//
// Orientation used by every logits tile: the engine's "A rows" are vocabulary
// rows of the LM head and its "B rows" are token rows of hidden, i.e. a tile is
// logits^T[vocab, token].  A thread then owns a few token columns and holds many
// vocabulary entries of each in registers, so the softmax reductions over the
// vocabulary are in-lane and need no cross-lane traffic inside the tile loop.
#pragma once

#include "tlce_common.h"

namespace tlce {

typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------ forward --
// Per (token tile, vocabulary split): stream the split's vocabulary tiles,
// keeping a running (max, sum-exp) per token in registers (base-2 domain), and
// write one partial per token.  Math follows ce_forward_kernel
// (fused_linear_ce_cuda.cu:156-224): bias add, tanh soft cap, excluded column
// skipped, but as an online single pass instead of two passes over stored
// logits.
struct ForwardArgs {
  const void* hidden;   // [m, h]
  const void* weight;   // [v, h], or [h, v] for the kernels instantiated with kWDimFirst
  const float* bias;    // [v] or null
  int m, h, v;
  int64_t exclude;
  float softcap;
  float logit_scale = 1.0f;   // logits = cap(logit_scale * hidden . weight^T + bias); > 0
  int n_ttiles, n_vtiles, nsplit;
  float* part_max;      // [nsplit, part_ld]  base-2 running max
  float* part_sum;      // [nsplit, part_ld]
  int part_ld;
  // Row count known only to the device (null: m is exact).  m is then the
  // capacity; token tiles, vocabulary splits and part_ld follow the real count
  // exactly as the host plan would have set them for it.
  const int64_t* m_dev = nullptr;
};

// kWDimFirst (engines with K-major operands only): the head is stored [h, v]
// (fused_linear_ce.cpp:104 `weight_dim_first`) and read in place as a K-major
// operand, K = the hidden axis; v is then a multiple of 8.
template <class E, bool kSoftcap, bool kBias, bool kWDimFirst = false>
__global__ __launch_bounds__(E::kThreads) void lce_forward_stats_kernel(ForwardArgs p) {
  extern __shared__ __align__(16) char smem[];
  using T = typename E::T;
  if (p.m_dev != nullptr) {
    p.m = effective_rows(p.m, p.m_dev);
    p.n_ttiles = (p.m + E::kTile - 1) / E::kTile;
    p.nsplit = forward_vocab_splits(p.n_ttiles, p.n_vtiles);
    p.part_ld = p.n_ttiles * E::kTile;
  }
  const int logical = xcd_logical_block_of(blockIdx.x, p.n_ttiles * p.nsplit);
  if (logical < 0) return;
  int tt, vs;
  grouped_tile(logical, p.n_ttiles, p.nsplit, 4, &tt, &vs);
  const int vt0 = (int)((int64_t)vs * p.n_vtiles / p.nsplit);
  const int vt1 = (int)((int64_t)(vs + 1) * p.n_vtiles / p.nsplit);

  E eng;
  const T* hidden = static_cast<const T*>(p.hidden);
  const T* weight = static_cast<const T*>(p.weight);
  // the logit multiplier is applied where the raw dot product is first touched:
  // with the bias, else inside the soft cap's argument, else inside the
  // exponent's scale
  const float raw_scale = kBias ? 1.0f : p.logit_scale;
  const float inv_cap = kSoftcap ? raw_scale / p.softcap : 0.0f;
  const float log2e_scaled = kSoftcap ? TLCE_LOG2E : TLCE_LOG2E * raw_scale;

  float run_max[E::kCols], run_sum[E::kCols];
#pragma unroll
  for (int j = 0; j < E::kCols; ++j) {
    run_max[j] = -INFINITY;
    run_sum[j] = 0.0f;
  }

  for (int vt = vt0; vt < vt1; ++vt) {
    // Everything derived from the lane index is recomputed per tile: kept live as
    // loop invariants, those addresses get spilled across the epilogue below and
    // reloaded from scratch at the top of every tile (3 % of this kernel).
    eng.forget_lane_invariants();
    typename E::Acc acc;
    if constexpr (kWDimFirst) {
      const Operand<T> a = {weight, p.v, vt * E::kTile, p.v};
      const Operand<T> b = {hidden, p.h, tt * E::kTile, p.m};
      eng.template mainloop_ex<true, false, true>(a, b, 0, p.h, acc, smem);
    } else {
      eng.mainloop_set(weight, p.h, vt * E::kTile, p.v, hidden, p.h, tt * E::kTile, p.m, 0, p.h,
                       acc, smem);
    }
    const int vbase = vt * E::kTile;
    if (kBias) {
#pragma unroll
      for (int i = 0; i < E::kRows; ++i) {
        const float b = p.bias[min(vbase + eng.row(i), p.v - 1)];
#pragma unroll
        for (int j = 0; j < E::kCols; ++j)
          E::set(acc, j, i, fmaf(E::get(acc, j, i), p.logit_scale, b));
      }
    }
    // Only the last vocabulary tile (rows past v) and the tile that holds the
    // excluded column need per-element masking: a workgroup-uniform branch.
    const bool edge = (vbase + E::kTile > p.v) ||
                      (p.exclude >= vbase && p.exclude < vbase + E::kTile);
    if (kSoftcap || edge) {
      asm volatile("" ::: "memory");   // keep this a real branch, not per-element selects
      const int excluded = (int)p.exclude;
#pragma unroll
      for (int i = 0; i < E::kRows; ++i) {
        const int v = vbase + eng.row(i);
        const bool ok = (v < p.v) && (v != excluded);
#pragma unroll
        for (int j = 0; j < E::kCols; ++j) {
          float z = E::get(acc, j, i);
          if (kSoftcap) z = p.softcap * tanh_of<E::kPrecise>(z * inv_cap);
          E::set(acc, j, i, ok ? z : -INFINITY);
        }
      }
    }
    // online (max, sum-exp) in the base-2 domain: exp(z - m) = exp2(z*log2e - m2)
#pragma unroll
    for (int j = 0; j < E::kCols; ++j) {
      float tile_max = -INFINITY;
#pragma unroll
      for (int i = 0; i < E::kRows; ++i) tile_max = fmaxf(tile_max, E::get(acc, j, i));
      const float new_max = fmaxf(run_max[j], tile_max * log2e_scaled);
      if (new_max > -INFINITY) {
        float s = run_sum[j] * exp2_of<E::kPrecise>(run_max[j] - new_max);
#pragma unroll
        for (int i = 0; i < E::kRows; ++i)
          s += exp2_of<E::kPrecise>(fmaf(E::get(acc, j, i), log2e_scaled, -new_max));
        run_sum[j] = s;
        run_max[j] = new_max;
      }
    }
  }

  // merge the kShare threads that hold the same token column
  float* sh_max = reinterpret_cast<float*>(smem);
  float* sh_sum = sh_max + E::kShare * E::kTile;
  const int slot = eng.share_slot();
#pragma unroll
  for (int j = 0; j < E::kCols; ++j) {
    sh_max[slot * E::kTile + eng.col(j)] = run_max[j];
    sh_sum[slot * E::kTile + eng.col(j)] = run_sum[j];
  }
  __syncthreads();
  for (int c = threadIdx.x; c < E::kTile; c += E::kThreads) {
    float mx = -INFINITY;
#pragma unroll
    for (int s = 0; s < E::kShare; ++s) mx = fmaxf(mx, sh_max[s * E::kTile + c]);
    float sum = 0.0f;
    if (mx > -INFINITY) {
#pragma unroll
      for (int s = 0; s < E::kShare; ++s)
        sum += sh_sum[s * E::kTile + c] * exp2_of<E::kPrecise>(sh_max[s * E::kTile + c] - mx);
    }
    const int64_t o = (int64_t)vs * p.part_ld + tt * E::kTile + c;
    p.part_max[o] = mx;
    p.part_sum[o] = sum;
  }
}

// One wave per row: merge the vocabulary-split partials into lse, compute the
// target logit as a direct dot product hidden[r] . weight[label] (+bias, soft
// cap), and write loss = lse - target (0 for ignored rows; a label outside
// [0, v) or equal to the excluded column contributes target 0, as in
// ce_forward_kernel, fused_linear_ce_cuda.cu:199-219).
struct CombineArgs {
  const void* hidden;
  const void* weight;
  const float* bias;
  const int64_t* labels;
  const int64_t* row_idx;
  int m, h, v;
  int64_t ignore, exclude;
  float softcap;
  const float* part_max;
  const float* part_sum;
  int part_ld, nsplit;
  float* losses;
  float* lse;
  float* valid_count;
  // vocabulary-shard mode (local_max != null): labels and exclude are global
  // ids, the weight holds rows [label_offset, label_offset + v); the kernel
  // writes the shard's softmax statistics instead of lse and loss
  // (vocab_parallel_ce_stats_kernel, fused_linear_ce_cuda.cu:292-365)
  int64_t label_offset;
  float* local_max;
  float* local_sum;
  float* target_logits;
  // masked-token loss extras: the logit multiplier of the forward kernel, an
  // optional per-row weight [m] and, when weighted != null, the row's weighted
  // loss written compactly (weighted[r] = weight[r] * loss[r], 0 for ignored
  // rows and rows past the device row count) for a deterministic sum afterwards
  float logit_scale = 1.0f;
  const float* token_weights = nullptr;
  float* weighted = nullptr;
  int weighted_rows = 0;             // entries of `weighted` to define (rows past m get 0)
  int n_vtiles = 0, tile = 0;        // for the device-side plan when m_dev != null
  const int64_t* m_dev = nullptr;
  bool weight_dim_first = false;     // weight is [h, v]: the label's column is read with stride v
};

// Dot product of two rows of length h by one wave (every lane gets the sum):
// 16 bytes per lane and load for 2-byte types when the rows allow it.
template <typename T>
__device__ __forceinline__ float wave_dot(const T* a_row, const T* b_row, int h, int lane) {
  float dot = 0.0f;
  if (sizeof(T) == 2 && (h % 8) == 0 &&
      ((reinterpret_cast<uintptr_t>(a_row) | reinterpret_cast<uintptr_t>(b_row)) & 15) == 0) {
    typedef T v8_t __attribute__((ext_vector_type(8)));
    for (int k = lane * 8; k < h; k += 64 * 8) {
      const v8_t a = *reinterpret_cast<const v8_t*>(a_row + k);
      const v8_t b = *reinterpret_cast<const v8_t*>(b_row + k);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot = fmaf(to_float<T>(a[e]), to_float<T>(b[e]), dot);
    }
  } else {
    for (int k = lane; k < h; k += 64) dot = fmaf(to_float<T>(a_row[k]), to_float<T>(b_row[k]), dot);
  }
  return wave_sum(dot);
}

// Rows per workgroup of lce_combine_loss_kernel: 4 waves x 4 rows, so that the
// count of valid rows costs one global atomic per 16 rows (one per row
// serialises 32768 atomics on a single address: two thirds of this kernel).
constexpr int kCombineRowsPerBlock = 16;

template <typename T>
__global__ __launch_bounds__(256) void lce_combine_loss_kernel(CombineArgs p) {
  __shared__ int block_valid;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) block_valid = 0;
  __syncthreads();
  if (p.m_dev != nullptr) {
    p.m = effective_rows(p.m, p.m_dev);
    const int n_ttiles = (p.m + p.tile - 1) / p.tile;
    p.nsplit = forward_vocab_splits(n_ttiles, p.n_vtiles);
    p.part_ld = n_ttiles * p.tile;
  }
  int wave_valid = 0;
  for (int i = 0; i < kCombineRowsPerBlock / 4; ++i) {
    const int r = blockIdx.x * kCombineRowsPerBlock + wave * (kCombineRowsPerBlock / 4) + i;
    if (r >= p.m) {
      if (p.weighted != nullptr && r < p.weighted_rows && lane == 0) p.weighted[r] = 0.0f;
      continue;
    }
    float mx = -INFINITY;
    for (int s = lane; s < p.nsplit; s += 64)
      mx = fmaxf(mx, p.part_max[(int64_t)s * p.part_ld + r]);
    mx = wave_max(mx);
    float sum = 0.0f;
    for (int s = lane; s < p.nsplit; s += 64) {
      const float pm = p.part_max[(int64_t)s * p.part_ld + r];
      if (pm > -INFINITY) sum += p.part_sum[(int64_t)s * p.part_ld + r] * exp2_of<sizeof(T) == 4>(pm - mx);
    }
    sum = wave_sum(sum);
    const float lse = (mx + log2f(sum)) * TLCE_LN2;

    if (p.labels == nullptr) {   // statistics only (soft embedding): no targets, no loss
      if (lane == 0) p.lse[r] = lse;
      continue;
    }
    const int64_t label = p.labels[r];
    const bool valid = (label != p.ignore);
    const int64_t y = label - p.label_offset;   // row of the label in this weight
    const bool here = valid && y >= 0 && y < p.v;
    const bool has_target = here && label != p.exclude;
    float target = 0.0f;
    if (has_target) {
      const T* hrow = static_cast<const T*>(p.hidden) + (int64_t)r * p.h;
      float dot;
      if (p.weight_dim_first) {
        const T* wcol = static_cast<const T*>(p.weight) + y;
        float part = 0.0f;
        for (int k = lane; k < p.h; k += 64)
          part = fmaf(to_float<T>(hrow[k]), to_float<T>(wcol[(int64_t)k * p.v]), part);
        dot = wave_sum(part) * p.logit_scale;
      } else {
        const T* wrow = static_cast<const T*>(p.weight) + y * (int64_t)p.h;
        dot = wave_dot<T>(hrow, wrow, p.h, lane) * p.logit_scale;
      }
      if (p.bias != nullptr) dot += p.bias[y];
      if (p.softcap > 0.0f) dot = p.softcap * tanhf(dot / p.softcap);
      target = dot;
    }
    if (lane == 0) {
      if (p.local_max != nullptr) {
        // the partials are in base-2 units: max2 = max * log2(e), sum = sum exp(z - max)
        p.local_max[r] = mx * TLCE_LN2;
        p.local_sum[r] = (mx > -INFINITY) ? sum : 0.0f;
        p.target_logits[r] = (here && label == p.exclude) ? -INFINITY : target;
      } else {
        p.lse[r] = lse;
        const float loss = valid ? (lse - target) : 0.0f;
        if (p.losses != nullptr) {
          const int64_t o = (p.row_idx != nullptr) ? p.row_idx[r] : (int64_t)r;
          p.losses[o] = loss;
        }
        if (p.weighted != nullptr)
          p.weighted[r] = (p.token_weights != nullptr) ? loss * p.token_weights[r] : loss;
      }
    }
    wave_valid += valid ? 1 : 0;
  }
  if (p.valid_count == nullptr) return;   // uniform: statistics-only callers
  if (lane == 0 && wave_valid != 0) atomicAdd(&block_valid, wave_valid);
  __syncthreads();
  if (threadIdx.x == 0 && block_valid != 0) atomicAdd(p.valid_count, (float)block_valid);
}

// ----------------------------------------------------------------- backward --
// scale[r] = d loss / d token_loss[r]  (token_scale_value,
// fused_linear_ce_cuda.cu:226-238), 0 for ignored and padding rows.
struct ScaleArgs {
  const int64_t* labels;
  const int64_t* row_idx;
  const float* grad_output;
  const float* valid_count;
  int m, mp;
  int reduction;
  int64_t ignore;
  float constant;   // labels == null: every real row gets this scale
  float multiplier; // applied to every scale
  const float* token_weights = nullptr;   // optional per-row factor [m] (loss weights)
  const int64_t* m_dev = nullptr;   // device row count (null: m is exact); rows past it get 0
  float* scale;
};

// Recompute one logits^T tile of a vocabulary panel and turn it, in registers,
// into the logit gradient of ce_grad_logits_kernel
// (fused_linear_ce_cuda.cu:240-290):
//   g = (exp(cap(z) - lse) - [v == label]) * scale * (1 - tanh^2(z / cap)),
// 0 for ignored rows, the excluded column and padding.  g is rounded to the
// input dtype and written to the panel in both orientations: G[token, v] feeds
// the grad-hidden contraction, GT[v, token] the grad-weight contraction.
struct GradLogitsArgs {
  const void* hidden;
  const void* weight;
  const float* bias;
  const int64_t* labels;
  const float* lse;
  const float* scale;
  int m, h, v;
  int64_t ignore, exclude;
  float softcap;
  int64_t label_offset;  // global id of weight row 0 (vocabulary shards), else 0
  int probabilities;     // 1: g = softmax * scale (labels may be null; no onehot)
  int cap_grad;          // 1: g carries the soft cap's derivative 1 - tanh^2 (a gradient
                         // with respect to the raw logits), 0: it does not (probabilities)
  float logit_scale;     // logits = cap(logit_scale * hidden . weight^T + bias).  The caller
                         // folds it into `scale` for gradients.
  const int64_t* m_dev = nullptr;   // device row count (null: m is exact): m is then the
                         // capacity and only the token tiles below the real count are produced
  int v0;             // first vocabulary row of the panel
  int n_ttiles, n_ptiles;
  void* g;            // [mp, ldg]
  int64_t ldg;
  void* gt;           // [panel columns, ldgt] or null
  int64_t ldgt;
  float* grad_bias;   // [v] or null
};

template <typename T>
__device__ __forceinline__ void store4(T* dst, float a, float b, float c, float d) {
  if constexpr (sizeof(T) == 2) {
    typedef T v4_t __attribute__((ext_vector_type(4)));
    v4_t x;
    x[0] = from_float<T>(a);
    x[1] = from_float<T>(b);
    x[2] = from_float<T>(c);
    x[3] = from_float<T>(d);
    *reinterpret_cast<v4_t*>(dst) = x;
  } else {
    *reinterpret_cast<float4*>(dst) = make_float4(a, b, c, d);
  }
}

// Streaming store for the logit-gradient panels, which are far larger than L2
// and are read back only by later kernels: the non-temporal hint keeps them
// from evicting the operand tiles the workgroups of an XCD share through L2
// (3 % off the producing kernel; the same hint on the GEMM outputs and on the
// float32 grad_hidden slabs measured slower and is not used there).
__device__ __forceinline__ void stream_store16(void* dst, uint4 v) {
  typedef unsigned u4_t __attribute__((ext_vector_type(4)));
  u4_t x;
  x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
  __builtin_nontemporal_store(x, reinterpret_cast<u4_t*>(dst));
}

template <class E, bool kSoftcap, bool kBias, bool kWDimFirst = false>
__global__ __launch_bounds__(E::kThreads) void lce_grad_logits_panel_kernel(GradLogitsArgs p) {
  extern __shared__ __align__(16) char smem[];
  using T = typename E::T;
  if (p.m_dev != nullptr) {
    p.m = effective_rows(p.m, p.m_dev);
    p.n_ttiles = (p.m + E::kTile - 1) / E::kTile;
  }
  const int logical = xcd_logical_block_of(blockIdx.x, p.n_ttiles * p.n_ptiles);
  if (logical < 0) return;
  int tt, pv;
  grouped_tile(logical, p.n_ttiles, p.n_ptiles, 4, &tt, &pv);

  E eng;
  const T* hidden = static_cast<const T*>(p.hidden);
  const T* weight = static_cast<const T*>(p.weight);
  typename E::Acc acc;
  const int vbase = p.v0 + pv * E::kTile;
  // per owned token column: row of its label inside this tile (-1: none here),
  // lse in base-2 units, and the loss scale (0 for ignored and padding rows,
  // which zeroes their whole column of g without a per-element test).  Loaded
  // before the contraction so that their latency passes under it instead of
  // standing between the last MFMA and the gradient math.
  int label_row[E::kCols];
  float lse2[E::kCols], scale[E::kCols];
  bool label_here = false;
#pragma unroll
  for (int j = 0; j < E::kCols; ++j) {
    const int r = tt * E::kTile + eng.col(j);
    const int rc = min(r, p.m - 1);
    const int64_t y = p.probabilities ? p.label_offset - 1 : p.labels[rc];   // never in a tile
    const bool live = (r < p.m) && (p.probabilities || y != p.ignore);
    const int64_t rel = y - p.label_offset - vbase;
    const bool here = live && rel >= 0 && rel < E::kTile;
    label_row[j] = here ? (int)rel : -1;
    label_here |= here;
    lse2[j] = p.lse[rc] * TLCE_LOG2E;
    scale[j] = live ? p.scale[rc] : 0.0f;
  }
  if constexpr (kWDimFirst) {   // the head as stored, [h, v]: a K-major operand
    const Operand<T> a = {weight, p.v, vbase, p.v};
    const Operand<T> b = {hidden, p.h, tt * E::kTile, p.m};
    eng.template mainloop_ex<true, false, true>(a, b, 0, p.h, acc, smem);
  } else {
    eng.mainloop_set(weight, p.h, vbase, p.v, hidden, p.h, tt * E::kTile, p.m, 0, p.h, acc, smem);
  }

  // the bias add applies the logit multiplier itself (z = multiplier * dot + bias)
  const float raw_scale = kBias ? 1.0f : p.logit_scale;
  const float inv_cap = kSoftcap ? raw_scale / p.softcap : 0.0f;
  const float log2e_scaled = TLCE_LOG2E * raw_scale;
  const float inv_logit_scale = kBias ? 1.0f / p.logit_scale : 1.0f;
  if (kBias) {
#pragma unroll
    for (int i = 0; i < E::kRows; ++i) {
      const float b = p.bias[min(vbase + eng.row(i), p.v - 1)];
#pragma unroll
      for (int j = 0; j < E::kCols; ++j)
        E::set(acc, j, i, fmaf(E::get(acc, j, i), p.logit_scale, b));
    }
  }
  // Both selectors of the epilogue variant are workgroup-uniform (the variants
  // contain workgroup barriers, so every wave must take the same one): rows past
  // v or the excluded column in this tile; some lane of the workgroup owns a
  // label of this tile (rare).
  const bool edge = (vbase + E::kTile > p.v) ||
                    (p.exclude >= vbase && p.exclude < vbase + E::kTile);
  const bool onehot = __syncthreads_or(label_here ? 1 : 0) != 0;

  const int excluded = (int)p.exclude;
  // one logit -> its entry of g (kEdge: the tile holds rows past v or the
  // excluded column; kOnehot: some lane of the workgroup owns a label of the tile)
  auto grad_of = [&](float z, int j, int row, bool vok, auto edge_tag, auto onehot_tag) -> float {
    constexpr bool kEdge = decltype(edge_tag)::value;
    constexpr bool kOnehot = decltype(onehot_tag)::value;
    float dcap = 1.0f;
    float g;
    if (kSoftcap) {
      const float t = tanh_of<E::kPrecise>(z * inv_cap);   // inv_cap includes logit_scale
      z = p.softcap * t;
      dcap = 1.0f - t * t;
      g = exp2_of<E::kPrecise>(fmaf(z, TLCE_LOG2E, -lse2[j]));
    } else {
      g = exp2_of<E::kPrecise>(fmaf(z, log2e_scaled, -lse2[j]));
    }
    if (kOnehot && row == label_row[j]) g -= 1.0f;
    g *= scale[j];
    if (kSoftcap && p.cap_grad) g *= dcap;
    if (kEdge) g = vok ? g : 0.0f;
    return g;
  };
  auto add_grad_bias = [&](int row, float row_sum) {
    const int v = vbase + row;
    row_sum = eng.reduce_over_cols(row_sum);
    // g carries the logit multiplier (folded into scale); the bias sits outside it
    if (eng.col_leader() && v < p.v && row_sum != 0.0f)
      atomicAdd(p.grad_bias + v, row_sum * inv_logit_scale);
  };

  T* g_out = static_cast<T*>(p.g);
  T* gt_out = static_cast<T*>(p.gt);
  const int prow = pv * E::kTile;  // first panel column of this tile
  if constexpr (E::kHasKMajor && sizeof(T) == 2) {
    // The MFMA engine's LDS is free after the main loop: the tile is staged there
    // as [token][vocab] (512-byte rows, 16-byte chunk c of token t in slot
    // c ^ (t & 31)) and G is written in whole 512-byte rows.  The work goes by
    // owned column index j: the tokens with index j (a quarter of the tile) are
    // transformed, staged and stored while the next quarter is being transformed,
    // so that only the last quarter's stores are still in flight when the
    // workgroup ends and frees its CU.
    auto emit = [&](auto edge_tag, auto onehot_tag) {
      constexpr bool kEdge = decltype(edge_tag)::value;
      asm volatile("" ::: "memory");   // one real branch per variant, no merged selects
      float row_sum[kBias ? E::kRows : 1];
      if (kBias) {
#pragma unroll
        for (int i = 0; i < E::kRows; ++i) row_sum[i] = 0.0f;
      }
#pragma unroll
      for (int j = 0; j < E::kCols; ++j) {
        const int tok = eng.col(j);
#pragma unroll
        for (int i = 0; i < E::kRows; i += 4) {
          float g4[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int row = eng.row(i + q);
            const bool vok = !kEdge || ((vbase + row < p.v) && (vbase + row != excluded));
            g4[q] = grad_of(E::get(acc, j, i + q), j, row, vok, edge_tag, onehot_tag);
            if (kBias) row_sum[i + q] += g4[q];
          }
          const int vq = eng.row(i) >> 2;
          T* dst = reinterpret_cast<T*>(smem + tok * 512 + (((vq >> 1) ^ (tok & 31)) * 16) +
                                        (vq & 1) * 8);
          store4<T>(dst, g4[0], g4[1], g4[2], g4[3]);
        }
        __syncthreads();
        constexpr int kPieces = E::kTokensPerIndex * 32;   // 16-byte pieces of this quarter
#pragma unroll
        for (int it = 0; it < kPieces / E::kThreads; ++it) {
          const int c = it * E::kThreads + threadIdx.x;
          const int t = E::token_of_index(j, c >> 5);
          const int ch = c & 31;
          const uint4 val =
              *reinterpret_cast<const uint4*>(smem + t * 512 + ((ch ^ (t & 31)) * 16));
          stream_store16(g_out + ((int64_t)tt * E::kTile + t) * p.ldg + prow + ch * 8, val);
        }
      }
      if (kBias) {
#pragma unroll
        for (int i = 0; i < E::kRows; ++i) add_grad_bias(eng.row(i), row_sum[i]);
      }
    };
    if (edge) {
      emit(std::true_type{}, std::true_type{});
    } else if (onehot) {
      emit(std::false_type{}, std::true_type{});
    } else {
      emit(std::false_type{}, std::false_type{});
    }
    if (gt_out != nullptr) {
      // transposed copy for the contractions that cannot read G K-major (vocabulary
      // not a multiple of 64): the whole tile is still staged; thread = token
      const int tok = threadIdx.x % E::kTile;
      for (int vrow = threadIdx.x / E::kTile; vrow < E::kTile; vrow += E::kThreads / E::kTile) {
        const T val = *reinterpret_cast<const T*>(smem + tok * 512 +
                                                  (((vrow >> 3) ^ (tok & 31)) * 16) +
                                                  (vrow & 7) * 2);
        gt_out[(int64_t)(prow + vrow) * p.ldgt + (int64_t)tt * E::kTile + tok] = val;
      }
    }
  } else {
    auto transform = [&](auto edge_tag, auto onehot_tag) {
      constexpr bool kEdge = decltype(edge_tag)::value;
      asm volatile("" ::: "memory");
#pragma unroll
      for (int i = 0; i < E::kRows; ++i) {
        const int row = eng.row(i);
        const bool vok = !kEdge || ((vbase + row < p.v) && (vbase + row != excluded));
        float row_sum = 0.0f;
#pragma unroll
        for (int j = 0; j < E::kCols; ++j) {
          const float g = grad_of(E::get(acc, j, i), j, row, vok, edge_tag, onehot_tag);
          E::set(acc, j, i, g);
          row_sum += g;
        }
        if (kBias) add_grad_bias(row, row_sum);
      }
    };
    if (edge) {
      transform(std::true_type{}, std::true_type{});
    } else if (onehot) {
      transform(std::false_type{}, std::true_type{});
    } else {
      transform(std::false_type{}, std::false_type{});
    }
#pragma unroll
    for (int j = 0; j < E::kCols; ++j) {
      const int64_t r = (int64_t)tt * E::kTile + eng.col(j);
#pragma unroll
      for (int i = 0; i < E::kRows; i += 4) {
        store4<T>(g_out + r * p.ldg + prow + eng.row(i), E::get(acc, j, i),
                  E::get(acc, j, i + 1), E::get(acc, j, i + 2), E::get(acc, j, i + 3));
      }
    }
    if (gt_out != nullptr) {
#pragma unroll
      for (int j = 0; j < E::kCols; ++j) {
        const int64_t r = (int64_t)tt * E::kTile + eng.col(j);
#pragma unroll
        for (int i = 0; i < E::kRows; ++i)
          gt_out[(int64_t)(prow + eng.row(i)) * p.ldgt + r] = from_float<T>(E::get(acc, j, i));
      }
    }
  }
}

// Forward KL(teacher || draft) of two frozen heads, one vocabulary panel at a
// time (dflash_kl_forward_kernel / dflash_kl_grad_logits_kernel,
// fused_linear_ce_cuda.cu:367-480).  The panel holds the teacher probabilities
// t = softmax(cap(z_teacher)) rounded to the input dtype (written by
// lce_grad_logits_panel_kernel in its probabilities mode).  This kernel
// recomputes the draft logits tile and, with lp = cap(z_draft) - lse_draft:
//   mode kKlLoss: per vocabulary tile and token, sum_v ( t * (log t - cap(z_draft)) - t )
//                 and sum_v t go to loss_part / tsum_part (one slot per tile, no
//                 atomics: the caller adds the tiles in a fixed order, so the loss
//                 is reproducible run to run), and the tile's (max, sum exp) of the
//                 draft logits go to the forward partial arrays, so that no
//                 separate statistics pass over the draft head is needed.  The
//                 caller finishes with loss = losses + tsum * lse_draft + 1: the
//                 generalised KL sum_v t log(t/q) - t + q, which equals
//                 sum_v p_t (log p_t - log p_d) to first order in the rounding
//                 of t (the plain sum would be off by sum_v dt).  lse is not read.
//   mode kKlGrad: panel[token, v] = (exp(lp) - t) * scale[token] * cap'(z_draft)
//                 in place, rounded to the input dtype: the logit gradient that
//                 feeds the grad-hidden contraction.
//   kEmit (with kKlLoss): additionally panel[token, v] = exp2(z2 - tile maximum of
//                 the token) rounded to the input dtype, the teacher tile being
//                 read from panel_in.  The tile maximum (part_max) is the exact
//                 maximum over the tile's 256 vocabulary rows, found through LDS
//                 before the exponentials, so every entry is <= 1; once the draft
//                 lse is known, softmax = entry * exp2(part_max - lse2) per
//                 (token, tile): the logit gradient can be formed from the two
//                 panels without contracting the draft head again.
//   kNoTeacher (with kEmit): no teacher tile is read (t = 0, the loss outputs are
//                 meaningless): the pass only emits and leaves the softmax partials.
//                 Run on the teacher head, it replaces the teacher's statistics pass
//                 and its probabilities pass by one contraction; the draft pass then
//                 takes t = entry * exp2(t_part_max - t_lse2) per (token, tile).
enum { kKlLoss = 0, kKlGrad = 1 };

struct KlPanelArgs {
  const void* hidden;   // draft hidden [m, h]
  const void* weight;   // draft head [v, h]
  const float* lse;     // draft lse [m]
  const float* scale;   // kKlGrad: grad_output per row, 0 on padding rows [mp]
  int m, h, v;
  float softcap;
  int v0;               // first vocabulary row of the panel
  int n_ttiles, n_ptiles;
  void* panel;          // [mp, ld] teacher probabilities in, logit gradients out
  int64_t ld;
  const void* panel_in = nullptr;   // non-null: the teacher probabilities are read here
  int64_t ld_in = 0;                // ([mp, ld_in]) and `panel` only receives the gradients
  // non-null: the teacher panel holds exp2(z2 - tile maximum) of the teacher head, these
  // are its tile maxima [n vocabulary tiles, part_ld] and its lse [m] (natural units)
  const float* t_part_max = nullptr;
  const float* t_lse = nullptr;
  float* loss_part;     // kKlLoss: [n vocabulary tiles, part_ld] loss terms of the tile
  float* tsum_part;     // kKlLoss: [n vocabulary tiles, part_ld] teacher mass of the tile
  float* part_max;      // kKlLoss: [n vocabulary tiles, part_ld] base-2 tile maxima
  float* part_sum;      //          and sums of exp2(z2 - max2), as the forward writes them
  int part_ld;
  int mode;
};

template <class E, bool kSoftcap, bool kGrad, bool kEmit = false, bool kNoTeacher = false>
__global__ __launch_bounds__(E::kThreads) void lce_kl_panel_kernel(KlPanelArgs p) {
  static_assert(!(kGrad && kEmit), "kEmit belongs to the loss mode");
  static_assert(kEmit || !kNoTeacher, "kNoTeacher belongs to the emitting pass");
  extern __shared__ __align__(16) char smem[];
  using T = typename E::T;
  const int logical = xcd_logical_block(blockIdx.x, gridDim.x);
  if (logical >= p.n_ttiles * p.n_ptiles) return;
  int tt, pv;
  grouped_tile(logical, p.n_ttiles, p.n_ptiles, 4, &tt, &pv);

  E eng;
  typename E::Acc acc;
  const int vbase = p.v0 + pv * E::kTile;
  constexpr bool grad = kGrad;   // p.mode, fixed at compile time: no mode test per group of 4
  float lse2[E::kCols], scale[E::kCols], partial[E::kCols], tsum[E::kCols];
  float tile_max[E::kCols], tile_sum[E::kCols];
  float tscale[E::kCols];   // teacher entry -> teacher probability
  bool live[E::kCols];
  // the per-row operands are loaded before the contraction: their latency passes under it
#pragma unroll
  for (int j = 0; j < E::kCols; ++j) {
    const int r = tt * E::kTile + eng.col(j);
    const int rc = min(r, p.m - 1);
    live[j] = r < p.m;
    lse2[j] = grad ? p.lse[rc] * TLCE_LOG2E : 0.0f;
    scale[j] = (grad && live[j]) ? p.scale[rc] : 0.0f;
    partial[j] = 0.0f;
    tsum[j] = 0.0f;
    tile_max[j] = -INFINITY;
    tile_sum[j] = 0.0f;
    tscale[j] = 1.0f;
    if (kEmit && !kNoTeacher && p.t_part_max != nullptr) {
      const float pm = p.t_part_max[(int64_t)(vbase / E::kTile) * p.part_ld + rc];
      tscale[j] = exp2_of<E::kPrecise>(pm - p.t_lse[rc] * TLCE_LOG2E);
    }
  }
  eng.mainloop_set(static_cast<const T*>(p.weight), p.h, vbase, p.v,
                   static_cast<const T*>(p.hidden), p.h, tt * E::kTile, p.m, 0, p.h, acc, smem);

  const float inv_cap = kSoftcap ? 1.0f / p.softcap : 0.0f;
  if (!grad) {
    // maxima of the capped draft logits per owned column (base-2 units) for the
    // tile's softmax partial; the capped values replace the raw accumulators
#pragma unroll
    for (int i = 0; i < E::kRows; ++i) {
      const bool vok = vbase + eng.row(i) < p.v;
#pragma unroll
      for (int j = 0; j < E::kCols; ++j) {
        float z = E::get(acc, j, i);
        if (kSoftcap) z = p.softcap * tanh_of<E::kPrecise>(z * inv_cap);
        z = vok ? z * TLCE_LOG2E : -INFINITY;
        E::set(acc, j, i, z);
        tile_max[j] = fmaxf(tile_max[j], z);
      }
    }
    if constexpr (kEmit) {
      // the maximum over all of the tile's vocabulary rows per token, through the LDS
      // beyond the engine's stages (the launch allocates it), before any exponential
      float* all_max = reinterpret_cast<float*>(smem + E::kSmemBytes);
      const int slot = eng.share_slot();
#pragma unroll
      for (int j = 0; j < E::kCols; ++j) all_max[slot * E::kTile + eng.col(j)] = tile_max[j];
      __syncthreads();
#pragma unroll
      for (int j = 0; j < E::kCols; ++j) {
        float mx = all_max[eng.col(j)];
#pragma unroll
        for (int sl = 1; sl < E::kShare; ++sl) mx = fmaxf(mx, all_max[sl * E::kTile + eng.col(j)]);
        tile_max[j] = mx;
      }
    }
  }
  T* panel = static_cast<T*>(p.panel);
  const T* panel_in = p.panel_in != nullptr ? static_cast<const T*>(p.panel_in) : panel;
  const int64_t ld_in = p.panel_in != nullptr ? p.ld_in : p.ld;
  const int prow = pv * E::kTile;   // first panel column of this tile
  constexpr bool kCanStage = E::kHasKMajor && sizeof(T) == 2;

  // one group of 4 consecutive vocabulary rows of owned column j: t[] in,
  // gradient out (kKlGrad) or the loss partial updated (kKlLoss)
  auto process = [&](int j, int i4, const float (&t)[4], float (&g)[4]) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int row = eng.row(i4 + u);
      const bool vok = vbase + row < p.v;
      float z = E::get(acc, j, i4 + u);
      if (grad) {
        float dcap = 1.0f;
        if (kSoftcap) {
          const float th = tanh_of<E::kPrecise>(z * inv_cap);
          z = p.softcap * th;
          dcap = 1.0f - th * th;
        }
        const float lp2 = fmaf(z, TLCE_LOG2E, -lse2[j]);   // log2 of the draft probability
        const float v = (exp2_of<E::kPrecise>(lp2) - t[u]) * scale[j] * dcap;
        g[u] = vok ? v : 0.0f;
      } else {
        // z already is the capped draft logit in base-2 units (-inf past the vocabulary)
        // selects, not branches: the lanes of a wave disagree on tv > 0
        const float tv = kNoTeacher ? 0.0f : t[u] * tscale[j];
        const float e = exp2_of<E::kPrecise>(z - tile_max[j]);
        tile_sum[j] += vok ? e : 0.0f;
        if (kEmit) g[u] = (vok && tile_max[j] > -INFINITY) ? e : 0.0f;
        // (a product of an entry and a tile scale can be a denormal, whose fast log2 is
        // -inf: probabilities below the smallest normal number carry no loss)
        const bool use = vok && tv >= 1.17549435e-38f;
        const float term = tv * ((log2_of<E::kPrecise>(tv) - z) * TLCE_LN2) - tv;
        partial[j] += use ? term : 0.0f;
        tsum[j] += use ? tv : 0.0f;
      }
    }
  };

  if constexpr (kCanStage) {
    // the tile of the panel goes through LDS in whole 512-byte token rows
    // (16-byte chunk c of token t in slot c ^ (t & 31)), both ways
    if constexpr (!kNoTeacher) {
#pragma unroll 4
      for (int it = 0; it < (E::kTile * 32) / E::kThreads; ++it) {
        const int c = it * E::kThreads + threadIdx.x;
        const int tok = c >> 5;
        const int ch = c & 31;
        *reinterpret_cast<uint4*>(smem + tok * 512 + ((ch ^ (tok & 31)) * 16)) =
            *reinterpret_cast<const uint4*>(panel_in + ((int64_t)tt * E::kTile + tok) * ld_in +
                                            prow + ch * 8);
      }
      __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < E::kCols; ++j) {
      const int tok = eng.col(j);
#pragma unroll
      for (int i4 = 0; i4 < E::kRows; i4 += 4) {
        const int vq = eng.row(i4) >> 2;
        T* cell = reinterpret_cast<T*>(smem + tok * 512 + (((vq >> 1) ^ (tok & 31)) * 16) +
                                       (vq & 1) * 8);
        typedef T v4_t __attribute__((ext_vector_type(4)));
        v4_t tv = {};
        if constexpr (!kNoTeacher) tv = *reinterpret_cast<const v4_t*>(cell);
        const float t[4] = {to_float<T>(tv[0]), to_float<T>(tv[1]), to_float<T>(tv[2]),
                            to_float<T>(tv[3])};
        float g[4];
        process(j, i4, t, g);
        if (grad || kEmit) store4<T>(cell, g[0], g[1], g[2], g[3]);
      }
      if (grad || kEmit) {
        // the tokens with owned index j are complete: their rows go out while
        // the next quarter of the tile is being processed
        __syncthreads();
        constexpr int kPieces = E::kTokensPerIndex * 32;
        constexpr int kMine = kPieces / E::kThreads;
        uint4 val[kMine];   // LDS reads first, then the stores: one wait per quarter
#pragma unroll
        for (int it = 0; it < kMine; ++it) {
          const int c = it * E::kThreads + threadIdx.x;
          const int tok = E::token_of_index(j, c >> 5);
          const int ch = c & 31;
          val[it] = *reinterpret_cast<const uint4*>(smem + tok * 512 + ((ch ^ (tok & 31)) * 16));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int it = 0; it < kMine; ++it) {
          const int c = it * E::kThreads + threadIdx.x;
          const int tok = E::token_of_index(j, c >> 5);
          const int ch = c & 31;
          stream_store16(panel + ((int64_t)tt * E::kTile + tok) * p.ld + prow + ch * 8, val[it]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < E::kCols; ++j) {
      T* cell0 = panel + ((int64_t)tt * E::kTile + eng.col(j)) * p.ld + prow;
      const T* in0 = panel_in + ((int64_t)tt * E::kTile + eng.col(j)) * ld_in + prow;
#pragma unroll
      for (int i4 = 0; i4 < E::kRows; i4 += 4) {
        T* cell = cell0 + eng.row(i4);
        const T* in = in0 + eng.row(i4);
        const float t[4] = {to_float<T>(in[0]), to_float<T>(in[1]), to_float<T>(in[2]),
                            to_float<T>(in[3])};
        float g[4];
        process(j, i4, t, g);
        if (grad || kEmit) store4<T>(cell, g[0], g[1], g[2], g[3]);
      }
    }
  }
  if (!grad) {
    // merge the kShare threads that hold the same token column, in a fixed order,
    // and publish the tile's partials, as the forward kernel does per vocabulary split
    __syncthreads();
    float* sh_max = reinterpret_cast<float*>(smem);
    float* sh_sum = sh_max + E::kShare * E::kTile;
    float* sh_loss = sh_sum + E::kShare * E::kTile;
    float* sh_tsum = sh_loss + E::kShare * E::kTile;
    const int slot = eng.share_slot();
#pragma unroll
    for (int j = 0; j < E::kCols; ++j) {
      sh_max[slot * E::kTile + eng.col(j)] = tile_max[j];
      sh_sum[slot * E::kTile + eng.col(j)] = tile_sum[j];
      sh_loss[slot * E::kTile + eng.col(j)] = partial[j];
      sh_tsum[slot * E::kTile + eng.col(j)] = tsum[j];
    }
    __syncthreads();
    const int tile_index = vbase / E::kTile;
    for (int c = threadIdx.x; c < E::kTile; c += E::kThreads) {
      float mx = -INFINITY;
#pragma unroll
      for (int sl = 0; sl < E::kShare; ++sl) mx = fmaxf(mx, sh_max[sl * E::kTile + c]);
      float sum = 0.0f, loss = 0.0f, mass = 0.0f;
#pragma unroll
      for (int sl = 0; sl < E::kShare; ++sl) {
        if (mx > -INFINITY)
          sum += sh_sum[sl * E::kTile + c] *
                 exp2_of<E::kPrecise>(sh_max[sl * E::kTile + c] - mx);
        loss += sh_loss[sl * E::kTile + c];
        mass += sh_tsum[sl * E::kTile + c];
      }
      const int64_t o = (int64_t)tile_index * p.part_ld + tt * E::kTile + c;
      p.part_max[o] = mx;
      p.part_sum[o] = sum;
      if (p.loss_part != nullptr) {   // (null: a pass that only emits)
        p.loss_part[o] = loss;
        p.tsum_part[o] = mass;
      }
    }
  }
}

// ------------------------------------------------- cross entropy + exact top-k --
// Frozen-head cross entropy that also returns the k largest logits of every row
// (dflash_ce_topk_forward / _backward, fused_linear_ce_cuda.cu:482-599,1511-1773;
// torch form in dllm_parallel/core/kernels/dflash_linear_topk.py:100-225).
// The logits z = cap(multiplier * hidden . weight^T) cross memory once, in
// float32, in bounded vocabulary panels: lce_logits_panel_kernel writes a
// panel, lce_topk_scan_kernel folds it into the row's running (max, sum exp)
// and its running list of the k largest (value, id) pairs.
struct LogitsPanelArgs {
  const void* hidden;
  const void* weight;
  int m, h, v;
  float softcap, logit_scale;
  int v0;               // first vocabulary row of the panel
  int n_ttiles, n_ptiles;
  float* panel;         // [mp, ld] float32; columns past the vocabulary get -inf
  int64_t ld;
};

template <class E, bool kSoftcap>
__global__ __launch_bounds__(E::kThreads) void lce_logits_panel_kernel(LogitsPanelArgs p) {
  extern __shared__ __align__(16) char smem[];
  using T = typename E::T;
  const int logical = xcd_logical_block(blockIdx.x, gridDim.x);
  if (logical >= p.n_ttiles * p.n_ptiles) return;
  int tt, pv;
  grouped_tile(logical, p.n_ttiles, p.n_ptiles, 4, &tt, &pv);
  E eng;
  typename E::Acc acc;
  const int vbase = p.v0 + pv * E::kTile;
  eng.mainloop_set(static_cast<const T*>(p.weight), p.h, vbase, p.v,
                   static_cast<const T*>(p.hidden), p.h, tt * E::kTile, p.m, 0, p.h, acc, smem);
  const float inv_cap = kSoftcap ? p.logit_scale / p.softcap : 0.0f;
  const int prow = pv * E::kTile;
  auto logits4 = [&](int j, int i4) -> float4 {
    float z[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float raw = E::get(acc, j, i4 + u);
      const float val = kSoftcap ? p.softcap * tanh_of<E::kPrecise>(raw * inv_cap) : raw * p.logit_scale;
      z[u] = (vbase + eng.row(i4 + u) < p.v) ? val : -INFINITY;
    }
    return make_float4(z[0], z[1], z[2], z[3]);
  };
  if constexpr (E::kHasKMajor && E::kCols == 4) {
    // The float32 tile is twice the engine's LDS: it is staged and written in two
    // halves (the tokens of two owned column indices = 128 rows of 1 KiB, 16-byte
    // chunk c of staged row s in slot c ^ (s & 63)), so that G leaves in whole
    // 1 KiB rows instead of 16-byte pieces a row apart.
    constexpr int kPerIndex = E::kTokensPerIndex;     // 64 tokens per owned index
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      if (half) __syncthreads();                      // the first half has been read out
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const int j = 2 * half + jj;
        // position of this lane's token among those with index j, as token_of_index counts
        const int t = (eng.col(j) / (E::kTile / 2)) * 32 + (eng.col(j) & 31);
        const int s_row = jj * kPerIndex + t;
#pragma unroll
        for (int i4 = 0; i4 < E::kRows; i4 += 4) {
          const int c = eng.row(i4) >> 2;
          *reinterpret_cast<float4*>(smem + s_row * 1024 + ((c ^ (s_row & 63)) * 16)) =
              logits4(j, i4);
        }
      }
      __syncthreads();
#pragma unroll 4
      for (int it = 0; it < (2 * kPerIndex * 64) / E::kThreads; ++it) {
        const int idx = it * E::kThreads + threadIdx.x;
        const int s_row = idx >> 6;
        const int ch = idx & 63;
        const int tok = E::token_of_index(2 * half + s_row / kPerIndex, s_row % kPerIndex);
        const uint4 val =
            *reinterpret_cast<const uint4*>(smem + s_row * 1024 + ((ch ^ (s_row & 63)) * 16));
        stream_store16(p.panel + ((int64_t)tt * E::kTile + tok) * p.ld + prow + ch * 4, val);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < E::kCols; ++j) {
      float* out = p.panel + ((int64_t)tt * E::kTile + eng.col(j)) * p.ld + prow;
#pragma unroll
      for (int i4 = 0; i4 < E::kRows; i4 += 4)
        *reinterpret_cast<float4*>(out + eng.row(i4)) = logits4(j, i4);
    }
  }
}

// One workgroup per row: folds `width` float32 logits of the row (vocabulary ids
// v0 .. v0 + width) into run_max / run_sum (natural-log units) and into the
// row's sorted list of the k largest pairs, 16384 logits at a time (64 per
// thread, in registers).  Logits above the list's current k-th value (for a
// row's first logits: at least the k-th largest per-thread maximum) are
// gathered in LDS and merged with the list by rank; when there are too many
// of them, k rounds of "the best pair after the previous pick" run over the
// whole chunk instead.  Ties go to the smaller id.  k <= 256.
struct TopkScanArgs {
  const float* panel;
  int64_t ld;
  int m;
  int64_t v0;
  int width;
  int k;
  int first;            // 1: the lists and statistics are empty
  float* run_max;
  float* run_sum;
  float* top_values;    // [m, k]
  int64_t* top_ids;     // [m, k]
};

// One wave per row: lse, the label's logit as a direct dot product, loss and
// the label's probability exp(-loss).
struct TopkFinishArgs {
  const void* hidden;
  const void* weight;
  const int64_t* labels;
  int m, h;
  float softcap, logit_scale;
  const float* run_max;
  const float* run_sum;
  float* lse;
  float* losses;
  float* probabilities;
};

template <typename T>
__global__ __launch_bounds__(256) void lce_topk_finish_kernel(TopkFinishArgs p) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= p.m) return;
  const T* hrow = static_cast<const T*>(p.hidden) + (int64_t)r * p.h;
  const T* wrow = static_cast<const T*>(p.weight) + p.labels[r] * (int64_t)p.h;
  float dot = wave_dot<T>(hrow, wrow, p.h, lane) * p.logit_scale;
  if (p.softcap > 0.0f) dot = p.softcap * tanhf(dot / p.softcap);
  if (lane == 0) {
    const float lse = p.run_max[r] + logf(p.run_sum[r]);
    const float loss = lse - dot;
    p.lse[r] = lse;
    p.losses[r] = loss;
    p.probabilities[r] = expf(-loss);
  }
}

// grad_hidden terms that touch single weight rows, added to the float32
// accumulator before the final cast (dflash_linear_topk.py:196-225):
//   - ce_scale[r] * d'(label) * W[label]  +  sum_j grad_top_values[r, j] * d'(id_j) * W[id_j]
// with d'(v) = multiplier * (1 - tanh^2(multiplier * h.W[v] / cap)) (multiplier without cap).
struct TopkAdjustArgs {
  const void* hidden;
  const void* weight;
  const int64_t* labels;
  const int64_t* top_ids;          // [m, k]
  const float* ce_scale;           // [m]
  const float* grad_top_values;    // [m, k] or null
  int m, h, k;
  float softcap, logit_scale;
  float* acc32;                    // [mp, h]
};

template <typename T>
__global__ __launch_bounds__(256) void lce_topk_adjust_kernel(TopkAdjustArgs p) {
  __shared__ float red[4];
  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const int r = blockIdx.x;
  const T* hrow = static_cast<const T*>(p.hidden) + (int64_t)r * p.h;
  float* out = p.acc32 + (int64_t)r * p.h;
  const int n_entries = (p.grad_top_values != nullptr ? p.k : 0) + 1;
  for (int e = 0; e < n_entries; ++e) {
    const bool is_label = e == n_entries - 1;
    const int64_t id = is_label ? p.labels[r] : p.top_ids[(int64_t)r * p.k + e];
    const float weight_in = is_label ? -p.ce_scale[r] : p.grad_top_values[(int64_t)r * p.k + e];
    if (weight_in == 0.0f) continue;   // workgroup-uniform
    const T* wrow = static_cast<const T*>(p.weight) + id * (int64_t)p.h;
    float dot = 0.0f;
    for (int c = t; c < p.h; c += 256) dot = fmaf(to_float<T>(hrow[c]), to_float<T>(wrow[c]), dot);
    dot = wave_sum(dot);
    if (lane == 0) red[wave] = dot;
    __syncthreads();
    const float raw = (red[0] + red[1] + red[2] + red[3]) * p.logit_scale;
    __syncthreads();
    float deriv = p.logit_scale;
    if (p.softcap > 0.0f) {
      const float th = tanhf(raw / p.softcap);
      deriv *= 1.0f - th * th;
    }
    const float coef = weight_in * deriv;
    for (int c = t; c < p.h; c += 256) out[c] += coef * to_float<T>(wrow[c]);
  }
}

// C[j][i] (op)= sum_k A[i][k] * B[j][k]  - the two gradient contractions, with
// the "A rows" on the output's contiguous axis (the hidden dimension):
//   grad_hidden: A = weight^T [h, Kv], B = G panel [mp, Kv]   -> C float32 [mp, h]
//   grad_weight: A = hidden^T [h, Km], B = GT panel [pv, Km]  -> C dtype   [pv, h]
// An engine with K-major operand support reads the "transposed" operands
// straight from their stored form (kAKMajor / kBKMajor: the operand is given
// as X[k][row], `rows` = its valid columns): weight [v, h] for grad_hidden,
// hidden [m, h] and the G panel [mp, Kv] for grad_weight.
// (project_grad_hidden / accumulate_grad_weight, fused_linear_ce_cuda.cu:676-791,
// with float32 accumulation).  A thread holds runs of 4 consecutive A rows per
// owned B row, so it reads and writes the output 16 (float32) or 8 (dtype)
// bytes at a time.  blockIdx.y selects a K split.
enum { kStoreF32 = 0, kAddF32 = 1, kStoreT = 3 };

struct GemmArgs {
  const void* a;
  int64_t lda;
  int a_rows;
  const void* b;
  int64_t ldb;
  int b_rows;
  int k;            // padded K, multiple of the engine's BK
  int k_per_split;  // multiple of BK
  int ni, nj;       // tiles along A rows / B rows
  void* c;          // [c_rows, ldc]: row = B row, column = A row
  int64_t ldc;
  int64_t c_split_stride;  // elements between the outputs of consecutive K splits
  int c_rows, c_cols;
  int mode;
  // Token count known only to the device (null: the sizes above are exact).
  // m_role kRowsFollow: the B rows / output rows are tokens (grad_hidden): tiles
  // along j and c_rows shrink to the real count.  kKFollows: K is the token axis
  // (grad_weight): k shrinks to the real count rounded up to m_round.
  const int64_t* m_dev = nullptr;
  int m_role = 0, m_round = 1;
  int64_t m_dev_offset = 0;  // the operand's first token row is row m_dev_offset of the counted rows
  int64_t slab_budget = 0;   // kRowsFollow: float32 elements all K-split slabs may take
  int k_steps_plan = 0;      // kRowsFollow: K steps of a full panel, what the split rule plans on
};

// K splits and slab stride the grad_hidden contraction uses for a device-side
// row count: the host plan's rule applied to the real number of token tiles,
// limited to the splits launched and to the slab memory the plan allocated.
__device__ __forceinline__ int dynamic_k_splits(int n_ttiles, int n_htiles, int tile, int h,
                                                int launched, int64_t slab_budget, int k_steps,
                                                int64_t* stride) {
  const int64_t slab = (int64_t)n_ttiles * tile * h;
  int ks = grad_hidden_k_splits((int64_t)n_ttiles * n_htiles, launched, k_steps, slab);
  while (ks > 1 && ks * slab > slab_budget) --ks;
  *stride = slab;
  return ks;
}
enum { kRowsFollow = 1, kKFollows = 2 };
// Output tiles per K split below which lce_gemm_nt_kernel orders its workgroups
// split-major over the XCDs (measured: 20 tiles x 12 splits 150 -> 85 us; 112 tiles x
// 2 splits 1.78 -> 1.84 ms, hence not there).
constexpr int kSplitMajorBelowTiles = 64;

// Output stage of the contraction kernels for the direct engine: the accumulator
// tile leaves through LDS (free after the main loop) in whole output rows, so that
// one wave instruction touches 1 KiB (float32) or 512 B (2-byte types) of one row
// instead of 64 pieces 16 or 8 bytes long in 64 different rows.
//
// float32 output (the grad_hidden slabs): the tile is 256 KiB, twice the LDS, and
// goes in two halves, the rows of two owned column indices each (128 rows of
// 1 KiB, 16-byte chunk c of staged row s in slot c ^ (s & 63)).  kAdd: the slab's
// old values of a half are requested before its rows are staged, so their
// latency passes under the staging.

template <class E, bool kAdd>
__device__ __forceinline__ void store_tile_f32_by_rows(const E& eng, const typename E::Acc& acc,
                                                       char* smem, float* c, int64_t ldc,
                                                       int row0, int col0, int c_rows,
                                                       int c_cols) {
  constexpr int kPerIndex = E::kTokensPerIndex;                 // rows per owned index
  constexpr int kMine = (2 * kPerIndex * 64) / E::kThreads;     // 16-byte pieces per thread
  constexpr int kBatch = 8;
  constexpr int kBatches = kMine / kBatch;
  constexpr int kAhead = 2;                                     // batches of old values in flight
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    if (half) __syncthreads();                                  // the first half has been read out
    // piece `it` of this thread: output row / column and whether it exists
    auto place = [&](int it, int* s_row, int* ch, int* out_row, int* out_col) -> bool {
      const int idx = it * E::kThreads + threadIdx.x;
      *s_row = idx >> 6;
      *ch = idx & 63;
      *out_row = row0 + E::token_of_index(2 * half + *s_row / kPerIndex, *s_row % kPerIndex);
      *out_col = col0 + *ch * 4;
      return *out_row < c_rows && *out_col < c_cols;
    };
    f32x4_t old[kAdd ? kBatches : 1][kAdd ? kBatch : 1];
    auto request_old = [&](int batch) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        int s_row, ch, out_row, out_col;
        const bool ok = place(batch * kBatch + u, &s_row, &ch, &out_row, &out_col);
        const f32x4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
        old[batch][u] =
            ok ? *reinterpret_cast<const f32x4_t*>(c + (int64_t)out_row * ldc + out_col) : zero;
      }
    };
    if (kAdd) {
#pragma unroll
      for (int b = 0; b < kAhead; ++b) request_old(b);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const int j = 2 * half + jj;
      const int t = (eng.col(j) / (E::kTile / 2)) * 32 + (eng.col(j) & 31);
      const int s_row = jj * kPerIndex + t;
#pragma unroll
      for (int i4 = 0; i4 < E::kRows; i4 += 4) {
        const int chunk = eng.row(i4) >> 2;
        const f32x4_t quad = {E::get(acc, j, i4), E::get(acc, j, i4 + 1), E::get(acc, j, i4 + 2),
                              E::get(acc, j, i4 + 3)};
        *reinterpret_cast<f32x4_t*>(smem + s_row * 1024 + ((chunk ^ (s_row & 63)) * 16)) = quad;
      }
    }
    __syncthreads();
#pragma unroll
    for (int b = 0; b < kBatches; ++b) {
      if (kAdd && b + kAhead < kBatches) request_old(b + kAhead);
      f32x4_t val[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int idx = (b * kBatch + u) * E::kThreads + threadIdx.x;
        const int s_row = idx >> 6, ch = idx & 63;
        val[u] = *reinterpret_cast<const f32x4_t*>(smem + s_row * 1024 +
                                                   ((ch ^ (s_row & 63)) * 16));
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        int s_row, ch, out_row, out_col;
        const bool ok = place(b * kBatch + u, &s_row, &ch, &out_row, &out_col);
        f32x4_t v = val[u];
        if (kAdd) v += old[b][u];
        if (ok) *reinterpret_cast<f32x4_t*>(c + (int64_t)out_row * ldc + out_col) = v;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// 2-byte output (the rows of grad_weight): the whole 128 KiB tile is staged as
// [row][column] (512-byte rows, 16-byte chunk c of row r in slot c ^ (r & 31)).
template <class E>
__device__ __forceinline__ void store_tile_t_by_rows(const E& eng, const typename E::Acc& acc,
                                                     char* smem, typename E::T* c, int64_t ldc,
                                                     int row0, int col0, int c_rows, int c_cols) {
  using T = typename E::T;
#pragma unroll
  for (int j = 0; j < E::kCols; ++j) {
    const int r = eng.col(j);
#pragma unroll
    for (int i4 = 0; i4 < E::kRows; i4 += 4) {
      const int vq = eng.row(i4) >> 2;
      T* dst = reinterpret_cast<T*>(smem + r * 512 + (((vq >> 1) ^ (r & 31)) * 16) + (vq & 1) * 8);
      store4<T>(dst, E::get(acc, j, i4), E::get(acc, j, i4 + 1), E::get(acc, j, i4 + 2),
                E::get(acc, j, i4 + 3));
    }
  }
  __syncthreads();
  constexpr int kMine = (E::kTile * 32) / E::kThreads;   // 16-byte pieces per thread
  constexpr int kBatch = 8;
#pragma unroll
  for (int b0 = 0; b0 < kMine; b0 += kBatch) {
    u32x4_t val[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int idx = (b0 + u) * E::kThreads + threadIdx.x;
      const int r = idx >> 5, ch = idx & 31;
      val[u] = *reinterpret_cast<const u32x4_t*>(smem + r * 512 + ((ch ^ (r & 31)) * 16));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int idx = (b0 + u) * E::kThreads + threadIdx.x;
      const int r = idx >> 5, ch = idx & 31;
      const int out_row = row0 + r, out_col = col0 + ch * 8;
      if (out_row < c_rows && out_col < c_cols)
        *reinterpret_cast<u32x4_t*>(c + (int64_t)out_row * ldc + out_col) = val[u];
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <class E, bool kAKMajor, bool kBKMajor>
__global__ __launch_bounds__(E::kThreads) void lce_gemm_nt_kernel(GemmArgs p) {
  extern __shared__ __align__(16) char smem[];
  using T = typename E::T;
  int n_splits = gridDim.y;
  if (p.m_dev != nullptr) {
    if (p.m_role == kRowsFollow) {
      p.c_rows = effective_block_rows(p.c_rows, p.m_dev, p.m_dev_offset);
      p.nj = (p.c_rows + E::kTile - 1) / E::kTile;
      n_splits = dynamic_k_splits(p.nj, p.ni, E::kTile, (int)p.ldc, (int)gridDim.y,
                                  p.slab_budget, p.k_steps_plan, &p.c_split_stride);
      p.k_per_split = (p.k / E::kBK + n_splits - 1) / n_splits * E::kBK;
    } else if (p.m_role == kKFollows) {
      const int rows = effective_block_rows(p.k, p.m_dev, p.m_dev_offset);
      p.k = (rows + p.m_round - 1) / p.m_round * p.m_round;
      // nothing to add to an accumulator that already holds earlier blocks of rows
      if (p.k == 0 && p.mode == kAddF32) return;
    }
  }
  int logical, split;
  const int tiles = p.ni * p.nj;
  if (gridDim.y == 1 || tiles >= kSplitMajorBelowTiles) {
    // every split deals its tiles to the 8 XCDs in contiguous runs of tiles / 8
    split = blockIdx.y;
    if (split >= n_splits) return;
    logical = xcd_logical_block_of(blockIdx.x, tiles);
    if (logical < 0) return;
  } else {
    // Few output tiles under many K splits (a small head, the last rows of a call
    // whose row count is on the device): a run of tiles / 8 would be 2 or 3 tiles, and
    // all 8 XCDs would fetch every K range of both operands.  The (split, tile) pairs
    // in split-major order are dealt to the XCDs in 8 contiguous, equally long runs
    // instead, so the tiles that stream one K range sit on one XCD (or two) and share
    // it through that L2.
    const int total = n_splits * tiles;
    const int flat = blockIdx.y * gridDim.x + blockIdx.x;   // gridDim.x is a multiple of 8
    const int xcd = flat % kXcds, slot = flat / kXcds;
    const int first = (int)((int64_t)xcd * total / kXcds);
    const int last = (int)((int64_t)(xcd + 1) * total / kXcds);
    if (slot >= last - first) return;
    split = (first + slot) / tiles;
    logical = (first + slot) - split * tiles;
  }
  int ti, tj;
  grouped_tile(logical, p.ni, p.nj, 4, &ti, &tj);
  // each K split owns its own output slab: no atomics, reproducible sums; a
  // split whose K range is empty still writes its (zero) tile
  const int k_begin = split * p.k_per_split;
  const int k_end = min(p.k, k_begin + p.k_per_split);
  p.c = static_cast<char*>(p.c) +
        (int64_t)split * p.c_split_stride * (p.mode == kStoreT ? sizeof(T) : sizeof(float));

  E eng;
  typename E::Acc acc;
  if (k_begin >= k_end) {
    E::zero(acc);   // nothing to accumulate
  } else if constexpr (E::kHasKMajor) {
    const Operand<T> a = {static_cast<const T*>(p.a), p.lda, ti * E::kTile, p.a_rows};
    const Operand<T> b = {static_cast<const T*>(p.b), p.ldb, tj * E::kTile, p.b_rows};
    eng.template mainloop_ex<kAKMajor, kBKMajor, true>(a, b, k_begin, k_end, acc, smem);
  } else {
    eng.mainloop_set(static_cast<const T*>(p.a), p.lda, ti * E::kTile, p.a_rows,
                     static_cast<const T*>(p.b), p.ldb, tj * E::kTile, p.b_rows, k_begin, k_end,
                     acc, smem);
  }

  if constexpr (E::kHasKMajor && sizeof(T) == 2 && E::kCols == 4) {
    // The direct engine is only planned for hidden sizes that are multiples of 64
    // and its outputs (workspace slabs, rows of grad_weight) are 16-byte aligned:
    // whole output rows leave through LDS (the main loop has ended on a barrier).
    const int row0 = tj * E::kTile, col0 = ti * E::kTile;
    if (p.mode == kStoreT) {
      store_tile_t_by_rows<E>(eng, acc, smem, static_cast<T*>(p.c), p.ldc, row0, col0, p.c_rows,
                              p.c_cols);
    } else if (p.mode == kStoreF32) {
      store_tile_f32_by_rows<E, false>(eng, acc, smem, static_cast<float*>(p.c), p.ldc, row0,
                                       col0, p.c_rows, p.c_cols);
    } else {
      store_tile_f32_by_rows<E, true>(eng, acc, smem, static_cast<float*>(p.c), p.ldc, row0,
                                      col0, p.c_rows, p.c_cols);
    }
  } else {
    // runs of 4 can be moved as one vector when every row start keeps them aligned
    const bool vec_ok = (p.ldc % 4 == 0) && (p.c_cols % 4 == 0) &&
                        (reinterpret_cast<uintptr_t>(p.c) % 16 == 0);
#pragma unroll
    for (int j = 0; j < E::kCols; ++j) {
      const int out_row = tj * E::kTile + eng.col(j);
      if (out_row >= p.c_rows) continue;
#pragma unroll
      for (int i = 0; i < E::kRows; i += 4) {
        const int out_col = ti * E::kTile + eng.row(i);
        if (out_col >= p.c_cols) continue;
        const int64_t o = (int64_t)out_row * p.ldc + out_col;
        const float v0 = E::get(acc, j, i), v1 = E::get(acc, j, i + 1);
        const float v2 = E::get(acc, j, i + 2), v3 = E::get(acc, j, i + 3);
        if (vec_ok) {
          if (p.mode == kStoreT) {
            store4<T>(static_cast<T*>(p.c) + o, v0, v1, v2, v3);
          } else if (p.mode == kStoreF32) {
            *reinterpret_cast<float4*>(static_cast<float*>(p.c) + o) =
                make_float4(v0, v1, v2, v3);
          } else {
            float4* dst = reinterpret_cast<float4*>(static_cast<float*>(p.c) + o);
            float4 old = *dst;
            *dst = make_float4(old.x + v0, old.y + v1, old.z + v2, old.w + v3);
          }
        } else {
          const float vals[4] = {v0, v1, v2, v3};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (out_col + e >= p.c_cols) continue;
            if (p.mode == kStoreT) {
              static_cast<T*>(p.c)[o + e] = from_float<T>(vals[e]);
            } else if (p.mode == kStoreF32) {
              static_cast<float*>(p.c)[o + e] = vals[e];
            } else {
              static_cast<float*>(p.c)[o + e] += vals[e];
            }
          }
        }
      }
    }
  }
}

// out[c][r] = in[r][c] for r < rows, zero for rows <= r < out_cols: the
// K-contiguous copies (weight^T, hidden^T) the gradient contractions read.
// The zero padding keeps 0 * garbage out of the padded K range.
template <typename T>
__global__ __launch_bounds__(256) void lce_transpose_pad_kernel(const T* __restrict__ in,
                                                                int64_t ld_in, int rows, int cols,
                                                                T* __restrict__ out,
                                                                int64_t ld_out, int out_cols,
                                                                const int64_t* rows_dev) {
  __shared__ T tile[64][66];
  rows = effective_rows(rows, rows_dev);   // rows past a device-side count read as zero
  const int tx = threadIdx.x & 63;
  const int ty = threadIdx.x >> 6;
  const int c0 = blockIdx.x * 64;
  const int r0 = blockIdx.y * 64;
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    const int rr = ty + 4 * q;
    const int r = r0 + rr;
    const int c = c0 + tx;
    tile[rr][tx] = (r < rows && c < cols) ? in[(int64_t)r * ld_in + c] : from_float<T>(0.0f);
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    const int cc = ty + 4 * q;
    const int c = c0 + cc;
    const int r = r0 + tx;
    if (c < cols && r < out_cols) out[(int64_t)c * ld_out + r] = tile[tx][cc];
  }
}

// grad_hidden[row_idx[r], :] = dtype(sum over K splits of acc32[s][r, :])
// (cast_float_to_scalar_kernel, fused_linear_ce_cuda.cu:144-154, fused with the
// K-split reduction and the un-compaction scatter).
template <typename T>
__global__ __launch_bounds__(256) void lce_finalize_grad_hidden_kernel(
    const float* __restrict__ acc32, int n_splits, int64_t split_stride,
    const int64_t* __restrict__ row_idx, int m, int h, T* __restrict__ out,
    const int64_t* __restrict__ m_dev, int n_htiles, int tile, int launched_splits,
    int k_steps_plan) {
  const int r = blockIdx.x;
  if (m_dev != nullptr) {
    // the splits and slab stride the contraction derived from the real row count
    m = effective_rows(m, m_dev);
    n_splits = dynamic_k_splits((m + tile - 1) / tile, n_htiles, tile, h, launched_splits,
                                (int64_t)n_splits * split_stride, k_steps_plan, &split_stride);
  }
  if (r >= m) return;
  const int64_t o = (row_idx != nullptr) ? row_idx[r] : (int64_t)r;
  const float* src = acc32 + (int64_t)r * h;
  T* dst = out + o * h;
  if ((h % 4) == 0 && (split_stride % 4) == 0 &&
      ((reinterpret_cast<uintptr_t>(acc32) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
    // four hidden entries per thread: 16-byte loads of every slab, one vector store
    for (int k = threadIdx.x * 4; k < h; k += 256 * 4) {
      f32x4_t sum = *reinterpret_cast<const f32x4_t*>(src + k);
      for (int s = 1; s < n_splits; ++s)
        sum += *reinterpret_cast<const f32x4_t*>(src + (int64_t)s * split_stride + k);
      store4<T>(dst + k, sum[0], sum[1], sum[2], sum[3]);
    }
    return;
  }
  for (int k = threadIdx.x; k < h; k += 256) {
    float sum = src[k];
    for (int s = 1; s < n_splits; ++s) sum += src[(int64_t)s * split_stride + k];
    dst[k] = from_float<T>(sum);
  }
}

}  // namespace tlce
