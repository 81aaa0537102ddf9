// Forward that also leaves the gradients: three contractions instead of four.
//
// The plain forward keeps no logits, so the backward has to recompute them
// (ce_grad_logits_kernel works on stored logits, fused_linear_ce_cuda.cu:240-290;
// the reference's blocks hold float32 logits between its forward and backward
// halves, :618-791).  When the loss is reduced to a scalar ("mean" / "sum") the
// upstream gradient is one number, and the gradients of the loss SUM can be
// formed while the logits of a block of rows exist, then scaled by that number
// afterwards.  Rows are taken in blocks of as many rows as a bounded panel holds
// over the WHOLE vocabulary; per block:
//
//   1. lce_exp_logits_panel_kernel: one contraction; the panel receives
//      e[r, v] = exp(z[r, v] - c[r]) * cap'(z) rounded to bf16, where
//      c[r] is a per-row reference logit known beforehand (the label's logit, a
//      one-row dot product).  Any c within ~80 of the row maximum keeps e inside
//      bf16's exponent range (float32's) with full relative precision.  The
//      tile sums of exp(z - c) and the tile maxima go out as per-tile partials.
//   2. lce_fused_rows_kernel: lse[r] = c[r] + log(sum), loss, the row factor
//      s[r] = weight[r] / sum (softmax = s * e), the label's panel entry replaced
//      by (e_label - sum) * cap' so that s * entry = (p_label - 1) * cap', and
//      hidden rows scaled by s for the grad_weight contraction.  A row whose
//      maximum lies outside [c - 40, c + 40] marks the block; steps 1-2 are
//      launched a second time and run only for marked blocks, with c = the exact
//      row maximum found by the first try (cannot fail again).
//   3. grad_hidden[r, :] = s[r] * (panel . weight)[r, :]   (K = the vocabulary,
//      complete for the block: no read-modify-write of a slab across panels)
//   4. grad_weight += panel^T . (s * hidden)   (float32 accumulator [v, h], one
//      read-modify-write per block of rows)
//
// Both gradients stay float32 until the upstream gradient arrives
// (lce_scale_cast_rows_kernel), so each is rounded once.
#pragma once

#include "tlce_host.h"

namespace tlce {

// The row offset beyond which the first try is redone with the exact maximum
// (natural-log units).  exp(40) ~ 2e17 and its reciprocal are far inside the
// bf16 / float32 exponent range, also after a multiplication by a hidden entry
// or a loss weight.  f16 (largest number 65504) has no such room: the label's
// panel entry alone is of the size of sum_v exp(z - c) = 1 / softmax(label), so
// the sequence is built for bf16 only and f16 inputs keep the recomputing backward.
// Default bound of the panel of exponentiated logits: 32 token tiles over a
// 152 K vocabulary in 16-bit.  Per block of rows the grad_weight accumulator
// [v, h] float32 is read and written once, so fewer, larger blocks cost less
// (measured at 32768 x 4096 x 151936: 1 GiB 106.7 ms per step, 1.2 GiB 101.5,
// 2.4 GiB 96.9).
constexpr int64_t kDefaultFusedPanelBytes = 5ll << 29;
constexpr float kRefWindow = 40.0f;

struct ExpPanelArgs {
  const void* hidden;   // [m, h] the rows of this block
  const void* weight;   // [v, h]
  const float* ref;     // [m] reference logit per row (natural units); +inf: row without loss
  float ref_const = 0.0f;   // ref == null: the reference of every row
  int m, h, v;
  int64_t exclude;
  float softcap;
  float logit_scale;    // logits = cap(logit_scale * hidden . weight^T)
  int n_ttiles, n_vtiles;
  void* panel;          // [n_ttiles * tile, ld]
  int64_t ld;
  float* part_sum;      // [n_vtiles, part_ld] sum over the tile of exp(z - ref)
  float* part_max;      // [n_vtiles, part_ld] tile maximum of z in base-2 units
  int part_ld;
  const int* run_flag;  // non-null: the launch does nothing unless *run_flag != 0
  // Row count known only to the device (null: m is exact): m is then the block's
  // capacity, and the block holds rows [row0, row0 + m) of the counted rows.
  const int64_t* m_dev = nullptr;
  int64_t row0 = 0;
};

// kPlain: the panel receives exp(z - c) itself, without the soft cap's derivative
// (a forward value, the unnormalised softmax, not a logit gradient).
template <class E, bool kSoftcap, bool kPlain = false>
__global__ __launch_bounds__(E::kThreads) void lce_exp_logits_panel_kernel(ExpPanelArgs p) {
  extern __shared__ __align__(16) char smem[];
  using T = typename E::T;
  static_assert(E::kHasKMajor && sizeof(T) == 2 && E::kCols == 4,
                "written for the four-wave direct-to-LDS engine");
  if (p.run_flag != nullptr && *p.run_flag == 0) return;
  if (p.m_dev != nullptr) {
    p.m = effective_block_rows(p.m, p.m_dev, p.row0);
    p.n_ttiles = (p.m + E::kTile - 1) / E::kTile;
  }
  const int logical = xcd_logical_block_of(blockIdx.x, p.n_ttiles * p.n_vtiles);
  if (logical < 0) return;
  int tt, vt;
  balanced_grouped_tile(logical, p.n_ttiles, p.n_vtiles, 4, &tt, &vt);

  E eng;
  typename E::Acc acc;
  const int vbase = vt * E::kTile;
  // Reference logit of every token column of the tile in base-2 units; +inf for
  // rows past the block and rows without loss, whose whole column of e becomes 0.
  // Fetched before the contraction so that the latency passes under it, and parked
  // in the LDS beyond the engine's stages: during the main loop every register
  // of the wave is taken.
  float* ref_stash = reinterpret_cast<float*>(smem + E::kSmemBytes);
  for (int c = threadIdx.x; c < E::kTile; c += E::kThreads) {
    const int r = tt * E::kTile + c;
    ref_stash[c] = (r < p.m) ? (p.ref != nullptr ? p.ref[r] : p.ref_const) * TLCE_LOG2E
                             : INFINITY;
  }
  eng.mainloop_set(static_cast<const T*>(p.weight), p.h, vbase, p.v,
                   static_cast<const T*>(p.hidden), p.h, tt * E::kTile, p.m, 0, p.h, acc, smem);
  // (the main loop's barriers have made the stash visible to every wave)
  float ref2[E::kCols];
#pragma unroll
  for (int j = 0; j < E::kCols; ++j) ref2[j] = ref_stash[eng.col(j)];

  const float inv_cap = kSoftcap ? p.logit_scale / p.softcap : 0.0f;
  const float to_base2 = kSoftcap ? p.softcap * TLCE_LOG2E : p.logit_scale * TLCE_LOG2E;
  const bool edge = (vbase + E::kTile > p.v) ||
                    (p.exclude >= vbase && p.exclude < vbase + E::kTile);
  const int excluded = (int)p.exclude;
  float col_sum[E::kCols], col_max[E::kCols];
  T* panel = static_cast<T*>(p.panel);
  const int pcol = vt * E::kTile;   // first panel column of this tile

  // The tile is staged in LDS (free after the main loop) as [token][vocab]:
  // 512-byte rows, 16-byte chunk c of token t in slot c ^ (t & 31), and leaves in
  // whole rows, a quarter of the tokens (one owned column index) at a time.
  auto emit = [&](auto edge_tag) {
    constexpr bool kEdge = decltype(edge_tag)::value;
    asm volatile("" ::: "memory");   // one real branch per variant
#pragma unroll
    for (int j = 0; j < E::kCols; ++j) {
      const int tok = eng.col(j);
      float s = 0.0f, mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < E::kRows; i += 4) {
        float e4[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int row = eng.row(i + q);
          float z2, dcap = 1.0f;
          if (kSoftcap) {
            const float t = tanh_of<E::kPrecise>(E::get(acc, j, i + q) * inv_cap);
            z2 = t * to_base2;
            dcap = 1.0f - t * t;
          } else {
            z2 = E::get(acc, j, i + q) * to_base2;
          }
          float e = exp2_of<E::kPrecise>(z2 - ref2[j]);
          if (kEdge) {
            const bool ok = (vbase + row < p.v) && (vbase + row != excluded);
            e = ok ? e : 0.0f;
            z2 = ok ? z2 : -INFINITY;
          }
          mx = fmaxf(mx, z2);
          s += e;
          e4[q] = (kSoftcap && !kPlain) ? e * dcap : e;
        }
        const int vq = eng.row(i) >> 2;
        T* dst = reinterpret_cast<T*>(smem + tok * 512 + (((vq >> 1) ^ (tok & 31)) * 16) +
                                      (vq & 1) * 8);
        store4<T>(dst, e4[0], e4[1], e4[2], e4[3]);
      }
      col_sum[j] = s;
      col_max[j] = mx;
      __syncthreads();
      constexpr int kPieces = E::kTokensPerIndex * 32;   // 16-byte pieces of this quarter
#pragma unroll
      for (int it = 0; it < kPieces / E::kThreads; ++it) {
        const int c = it * E::kThreads + threadIdx.x;
        const int t = E::token_of_index(j, c >> 5);
        const int ch = c & 31;
        const uint4 val = *reinterpret_cast<const uint4*>(smem + t * 512 + ((ch ^ (t & 31)) * 16));
        stream_store16(panel + ((int64_t)tt * E::kTile + t) * p.ld + pcol + ch * 8, val);
      }
    }
  };
  if (edge) {
    emit(std::true_type{});
  } else {
    emit(std::false_type{});
  }

  // merge the kShare threads that hold the same token column, in a fixed order
  __syncthreads();   // the last quarter has been read out of the stage
  float* sh_sum = reinterpret_cast<float*>(smem);
  float* sh_max = sh_sum + E::kShare * E::kTile;
  const int slot = eng.share_slot();
#pragma unroll
  for (int j = 0; j < E::kCols; ++j) {
    sh_sum[slot * E::kTile + eng.col(j)] = col_sum[j];
    sh_max[slot * E::kTile + eng.col(j)] = col_max[j];
  }
  __syncthreads();
  for (int c = threadIdx.x; c < E::kTile; c += E::kThreads) {
    float sum = 0.0f, mx = -INFINITY;
#pragma unroll
    for (int sl = 0; sl < E::kShare; ++sl) {
      sum += sh_sum[sl * E::kTile + c];
      mx = fmaxf(mx, sh_max[sl * E::kTile + c]);
    }
    const int64_t o = (int64_t)vt * p.part_ld + tt * E::kTile + c;
    p.part_sum[o] = sum;
    p.part_max[o] = mx;
  }
}

template <class E, bool kSoftcap, bool kPlain = false>
int launch_exp_panel_variant(const ExpPanelArgs& a, hipStream_t stream) {
  static LdsOptIn lds;
  constexpr int kLdsBytes = E::kSmemBytes + E::kTile * (int)sizeof(float);   // stages + stash
  if (int rc = enable_large_lds(lce_exp_logits_panel_kernel<E, kSoftcap, kPlain>, kLdsBytes, lds))
    return rc;
  const int grid = xcd_grid((int64_t)a.n_ttiles * a.n_vtiles);
  ScopedTimer timer(kClassExpPanel, stream);
  lce_exp_logits_panel_kernel<E, kSoftcap, kPlain><<<grid, E::kThreads, kLdsBytes, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------- row kernels --
// (engine-independent; compiled beside the C ABI, reached through launch_*)

// Before the blocks: the label's logit of every row by a one-row dot product,
// which is both the loss's target term and the reference logit of the row.
struct LabelLogitArgs {
  const void* hidden;   // [m, h]
  const void* weight;   // [v, h]
  const int64_t* labels;
  int m, h, v;
  int64_t ignore, exclude;
  float softcap, logit_scale;
  float* target;        // [m] cap(scale * h . w[label]); 0 when the label has no logit
  float* ref;           // [m] reference logit; +inf for rows without loss
  float* valid_count;   // [1] += rows with a label other than `ignore`
  const int64_t* m_dev = nullptr;   // device row count (null: m is exact)
};

struct FusedRowsArgs {
  const void* hidden;          // [m, h] rows of the block
  const int64_t* labels;       // [m]
  const float* ref;            // [m] the reference the panel was produced with
  const float* target;         // [m]
  const float* token_weights;  // [m] or null
  const int64_t* row_idx;      // [m] or null: where the row's loss goes
  int64_t loss_row0;           // row_idx == null: index of the block's first row in `losses`
  const float* part_sum;
  const float* part_max;
  int part_ld, n_vtiles;
  int m, m_pad;                // rows of the block; rows of `scaled_hidden` to define (zeros past m)
  int h, v;
  int64_t ignore, exclude;
  float softcap, logit_scale, window;
  void* panel;                 // [.., ld]
  int64_t ld;
  float* lse;                  // [m]
  float* losses;               // scattered, or null
  float* row_scale;            // [m_pad]
  void* scaled_hidden;         // [m_pad, h] or null (no grad_weight)
  float* ref_next;             // [m] reference of the second try
  int* redo;                   // [1] set when some row needs the second try
  const int* run_flag;         // non-null: run only when *run_flag != 0
  const int64_t* m_dev = nullptr;   // device row count (null: m is exact); the block's
  int64_t row0 = 0;                 // first row among the counted rows
};

// grad_hidden32[r, :] = row_scale[r] * sum over K splits of slab[s][r, :]
struct ReduceSlabsArgs {
  const float* slabs;
  int n_splits;
  int64_t split_stride;
  const float* row_scale;
  int m, h;
  float* out;   // [m, h]
  void* out_t = nullptr;            // non-null: the result goes here in bf16 instead
  const int64_t* m_dev = nullptr;   // device row count (null: m is exact); the block's
  int64_t row0 = 0;                 // first row among the counted rows
  // with a device row count the contraction derives its K splits and slab stride from
  // the real rows of the block (dynamic_k_splits); the same inputs reproduce them here
  int n_htiles = 0, tile = 0, launched_splits = 0, k_steps = 0;
  int64_t slab_budget = 0;
};

// out[row_idx[r], :] = dtype(g * in[r, :]) with g = grad_output[0] (/ valid_count[0]
// for the mean): the upstream gradient applied to the float32 gradients the
// forward left, rounding each entry once.
struct ScaleCastArgs {
  const float* in;          // [rows, h]
  const int64_t* row_idx;   // or null
  const float* grad_output; // [1]; reduction none: one per output row, read at row_idx[r]
  const float* valid_count; // [1], read for the mean reduction only
  int reduction;
  int64_t rows;
  int h;
  void* out;
  const int64_t* m_dev = nullptr;   // device row count: rows past it are not written
};

// scaled[r, :] = dtype(g * row_scale[r] * hidden[r, :]) with g as in ScaleCastArgs, zero
// rows from the row count up to m_pad: the K-major operand of a grad_weight
// contraction that was postponed until the upstream gradient is known.
struct ScaleRowsArgs {
  const void* hidden;       // [m, h]
  const float* row_scale;   // [m]
  const float* grad_output; // [1]; reduction none: one per output row, read at row_idx[r]
  const float* valid_count; // [1], read for the mean reduction only
  int reduction;
  int m, m_pad, h;
  void* out;                // [m_pad, h]
  const int64_t* m_dev = nullptr;   // device row count (null: m is exact)
  const int64_t* row_idx = nullptr; // output row of row r (null: r)
};

// row_scale[r] = scale / sum over the vocabulary tiles of part_sum[tile][r] (0 for rows
// from m up to m_pad): the normaliser of rows whose panel holds exp(z - c).
struct SoftRowsArgs {
  const float* part_sum;
  int part_ld, n_vtiles;
  int m, m_pad;
  float scale;
  float* row_scale;
};

int launch_soft_rows(const SoftRowsArgs& a, hipStream_t stream);
int launch_label_logit(const LabelLogitArgs& a, hipStream_t stream);
int launch_scale_rows(const ScaleRowsArgs& a, hipStream_t stream);
int launch_fused_rows(const FusedRowsArgs& a, hipStream_t stream);
int launch_reduce_slabs(const ReduceSlabsArgs& a, hipStream_t stream);
int launch_scale_cast(const ScaleCastArgs& a, hipStream_t stream);

// ------------------------------------------------------------------- plan ----
struct FusedPlan {
  int64_t vp;           // panel columns: the vocabulary rounded up to whole tiles
  int n_vtiles, n_htiles;
  int64_t block_rows;   // rows per block, a multiple of the tile
  int n_blocks;
  int dh_ksplit;        // K splits of the grad_hidden contraction of a full block
};

inline bool fused_gradients_supported(int64_t h, int64_t v, int dtype) {
  return dtype == TLCE_DTYPE_BF16 && engine_class(h, dtype) == 2 && (v % 64) == 0;
}

inline FusedPlan make_fused_plan(int64_t m, int64_t h, int64_t v, int dtype, int64_t panel_bytes) {
  FusedPlan p;
  const int64_t tile = 256;
  p.vp = round_up(v, tile);
  p.n_vtiles = (int)(p.vp / tile);
  p.n_htiles = (int)ceil_div(h, tile);
  if (panel_bytes <= 0) panel_bytes = kDefaultFusedPanelBytes;
  const int64_t total = ceil_div(std::max<int64_t>(m, 1), tile);   // token tiles
  const int64_t budget =
      std::max<int64_t>(1, panel_bytes / (p.vp * dtype_bytes(dtype) * tile));
  p.n_blocks = (int)ceil_div(total, budget);
  int64_t per = ceil_div(total, p.n_blocks);   // balanced blocks
  // several blocks: 16 token tiles x 16 hidden tiles make whole rounds of 256
  // workgroups in the grad_hidden contraction
  if (p.n_blocks > 1 && round_up(per, 16) <= budget) per = round_up(per, 16);
  p.block_rows = per * tile;
  p.n_blocks = (int)ceil_div(total, per);
  const int64_t k_steps = p.vp / 64;
  const int max_split = (int)std::max<int64_t>(1, std::min<int64_t>(16, k_steps / 8));
  p.dh_ksplit = grad_hidden_k_splits((p.block_rows / tile) * p.n_htiles, max_split, k_steps,
                                     p.block_rows * h);
  return p;
}

struct FusedLayout {
  int64_t panel, part_sum, part_max, target, ref, ref_next, row_scale, scaled_hidden, slabs,
      redo, total;
};

inline FusedLayout fused_layout(const FusedPlan& p, int64_t m, int64_t h, int dtype,
                                bool weight_grad) {
  FusedLayout l;
  const int64_t es = dtype_bytes(dtype);
  const int64_t mp = round_up(std::max<int64_t>(m, 1), 256);
  int64_t off = 0;
  l.panel = off;      off += align256(p.block_rows * p.vp * es);
  l.part_sum = off;   off += align256((int64_t)p.n_vtiles * p.block_rows * 4);
  l.part_max = off;   off += align256((int64_t)p.n_vtiles * p.block_rows * 4);
  l.target = off;     off += align256(mp * 4);
  l.ref = off;        off += align256(mp * 4);
  l.ref_next = off;   off += align256(p.block_rows * 4);
  l.row_scale = off;  off += align256(p.block_rows * 4);
  l.scaled_hidden = off;
  if (weight_grad) off += align256(p.block_rows * h * es);
  l.slabs = off;      off += align256((int64_t)p.dh_ksplit * p.block_rows * h * 4);
  l.redo = off;       off += align256((int64_t)p.n_blocks * 4);
  l.total = off;
  return l;
}

// Options of the fused sequence beyond the operator's own arguments.
struct FusedOptions {
  float logit_scale = 1.0f;
  const float* token_weights = nullptr;   // [m] per-row loss weights or null
  const int64_t* row_count = nullptr;     // device int64: the real number of rows (m: capacity)
};

template <class E>
int fused_gradients_impl(const FusedPlan& p, const void* hidden, const void* weight,
                         const int64_t* labels, const int64_t* row_idx, int64_t m, int64_t h,
                         int64_t v, int dtype, int64_t ignore, int64_t exclude, float softcap,
                         float* losses, float* lse, float* valid_count, float* grad_hidden32,
                         float* grad_weight32, char* ws, hipStream_t stream,
                         const FusedOptions& opt) {
  // opt.row_count != null: m is the capacity every launch is sized for; the kernels
  // take the real count from the device and the workgroups past it exit at once
  const int64_t* m_dev = opt.row_count;
  using T = typename E::T;
  const bool weight_grad = grad_weight32 != nullptr;
  const FusedLayout l = fused_layout(p, m, h, dtype, weight_grad);
  T* panel = reinterpret_cast<T*>(ws + l.panel);
  float* part_sum = reinterpret_cast<float*>(ws + l.part_sum);
  float* part_max = reinterpret_cast<float*>(ws + l.part_max);
  float* target = reinterpret_cast<float*>(ws + l.target);
  float* ref = reinterpret_cast<float*>(ws + l.ref);
  float* ref_next = reinterpret_cast<float*>(ws + l.ref_next);
  float* row_scale = reinterpret_cast<float*>(ws + l.row_scale);
  T* scaled_hidden = weight_grad ? reinterpret_cast<T*>(ws + l.scaled_hidden) : nullptr;
  float* slabs = reinterpret_cast<float*>(ws + l.slabs);
  int* redo = reinterpret_cast<int*>(ws + l.redo);
  const T* hidden_t = static_cast<const T*>(hidden);

  if (int rc = fill_zero(redo, (int64_t)p.n_blocks * 4, stream)) return rc;
  LabelLogitArgs la;
  la.hidden = hidden; la.weight = weight; la.labels = labels;
  la.m = (int)m; la.h = (int)h; la.v = (int)v;
  la.ignore = ignore; la.exclude = exclude; la.softcap = softcap; la.logit_scale = opt.logit_scale;
  la.target = target; la.ref = ref; la.valid_count = valid_count; la.m_dev = m_dev;
  if (int rc = launch_label_logit(la, stream)) return rc;

  for (int block = 0; block < p.n_blocks; ++block) {
    const int64_t r0 = (int64_t)block * p.block_rows;
    const int64_t rows = std::min<int64_t>(p.block_rows, m - r0);
    if (rows <= 0) break;
    const int n_ttiles = (int)ceil_div(rows, E::kTile);
    const int64_t rows_p = (int64_t)n_ttiles * E::kTile;
    const int64_t rows64 = round_up(rows, 64);

    ExpPanelArgs ea;
    ea.hidden = hidden_t + r0 * h; ea.weight = weight;
    ea.m = (int)rows; ea.h = (int)h; ea.v = (int)v;
    ea.exclude = exclude; ea.softcap = softcap; ea.logit_scale = opt.logit_scale;
    ea.n_ttiles = n_ttiles; ea.n_vtiles = p.n_vtiles;
    ea.panel = panel; ea.ld = p.vp;
    ea.part_sum = part_sum; ea.part_max = part_max; ea.part_ld = (int)p.block_rows;
    ea.m_dev = m_dev; ea.row0 = r0;

    FusedRowsArgs ra;
    ra.hidden = hidden_t + r0 * h; ra.labels = labels + r0;
    ra.target = target + r0;
    ra.token_weights = opt.token_weights ? opt.token_weights + r0 : nullptr;
    ra.row_idx = row_idx ? row_idx + r0 : nullptr; ra.loss_row0 = r0;
    ra.part_sum = part_sum; ra.part_max = part_max;
    ra.part_ld = (int)p.block_rows; ra.n_vtiles = p.n_vtiles;
    ra.m = (int)rows; ra.m_pad = (int)rows_p; ra.h = (int)h; ra.v = (int)v;
    ra.ignore = ignore; ra.exclude = exclude; ra.softcap = softcap;
    ra.logit_scale = opt.logit_scale;
    ra.window = kRefWindow;
    ra.panel = panel; ra.ld = p.vp;
    ra.lse = lse + r0; ra.losses = losses;
    ra.row_scale = row_scale; ra.scaled_hidden = scaled_hidden;
    ra.ref_next = ref_next; ra.redo = redo + block;
    ra.m_dev = m_dev; ra.row0 = r0;

    for (int attempt = 0; attempt < 2; ++attempt) {
      ea.ref = attempt ? ref_next : ref + r0;
      ea.run_flag = attempt ? redo + block : nullptr;
      if (softcap > 0.0f) {
        if (int rc = launch_exp_panel_variant<E, true>(ea, stream)) return rc;
      } else {
        if (int rc = launch_exp_panel_variant<E, false>(ea, stream)) return rc;
      }
      ra.ref = ea.ref;
      ra.run_flag = ea.run_flag;
      // the second try must not mark the block again: it reads the flag the first set
      if (int rc = launch_fused_rows(ra, stream)) return rc;
    }

    // grad_hidden of the block: A = weight as stored (K-major, K = vocabulary), B = panel
    GemmArgs dh;
    dh.a = weight; dh.lda = h; dh.a_rows = (int)h;
    dh.b = panel; dh.ldb = p.vp; dh.b_rows = (int)rows_p;
    dh.k = (int)round_up(v, 64);
    dh.k_per_split = 0;
    dh.ni = p.n_htiles; dh.nj = n_ttiles;
    dh.c = slabs; dh.ldc = h; dh.c_rows = (int)rows_p; dh.c_cols = (int)h;
    dh.c_split_stride = p.block_rows * h;
    dh.mode = kStoreF32;
    int ksplit = (rows_p == p.block_rows)
                     ? p.dh_ksplit
                     : std::min(p.dh_ksplit,
                                grad_hidden_k_splits((int64_t)n_ttiles * p.n_htiles, p.dh_ksplit,
                                                     p.vp / 64, rows_p * h));
    ReduceSlabsArgs rs;
    if (m_dev != nullptr) {
      // The block may hold far fewer rows than it was sized for (down to none): up to 16
      // splits are launched and the kernel takes as many as the real rows call for,
      // within the slab memory the plan allocated; the others exit at once.
      dh.m_dev = m_dev; dh.m_role = kRowsFollow; dh.m_dev_offset = r0;
      dh.slab_budget = (int64_t)p.dh_ksplit * p.block_rows * h;
      dh.k_steps_plan = (int)(p.vp / 64);
      ksplit = (int)std::max<int64_t>(p.dh_ksplit, std::min<int64_t>(16, p.vp / 64 / 8));
      rs.n_htiles = p.n_htiles; rs.tile = E::kTile; rs.launched_splits = ksplit;
      rs.k_steps = dh.k_steps_plan; rs.slab_budget = dh.slab_budget;
    }
    if (int rc = launch_gemm<E, true, false>(dh, ksplit, kClassGradHidden, stream)) return rc;
    rs.slabs = slabs; rs.n_splits = ksplit; rs.split_stride = p.block_rows * h;
    rs.row_scale = row_scale; rs.m = (int)rows; rs.h = (int)h;
    rs.out = grad_hidden32 + r0 * h;
    rs.m_dev = m_dev; rs.row0 = r0;
    if (int rc = launch_reduce_slabs(rs, stream)) return rc;

    if (weight_grad) {
      // grad_weight += panel^T . (s * hidden): both operands K-major, K = the block's rows
      GemmArgs dw;
      dw.a = scaled_hidden; dw.lda = h; dw.a_rows = (int)h;
      dw.b = panel; dw.ldb = p.vp; dw.b_rows = (int)p.vp;
      dw.k = (int)rows64;
      dw.k_per_split = 0;
      dw.ni = p.n_htiles; dw.nj = p.n_vtiles;
      dw.c = grad_weight32; dw.ldc = h; dw.c_rows = (int)v; dw.c_cols = (int)h;
      dw.c_split_stride = 0;
      dw.mode = block == 0 ? kStoreF32 : kAddF32;
      dw.m_dev = m_dev; dw.m_role = kKFollows; dw.m_round = 64; dw.m_dev_offset = r0;
      if (int rc = launch_gemm<E, true, true>(dw, 1, kClassGradWeight, stream)) return rc;
    }
  }
  return 0;
}

// The grad_weight contraction of a single-block forward, postponed to the backward:
// when all rows fit one block the panel still holds every exp(z - c) after the forward,
// so grad_weight = panel^T . (g * s * hidden) can be formed once the upstream gradient
// g is known and stored directly in the input dtype: no float32 [v, h] accumulator
// and no pass that scales and rounds it.  `ws` is the forward's workspace, untouched
// since (the forward was called without a grad_weight buffer, as for a frozen head,
// on a workspace sized for one).
template <class E>
int deferred_grad_weight_impl(const FusedPlan& p, const void* hidden, int64_t m, int64_t h,
                              int64_t v, int dtype, const float* grad_output,
                              const float* valid_count, int reduction, const int64_t* m_dev,
                              const int64_t* row_idx, void* grad_weight, char* ws,
                              hipStream_t stream) {
  using T = typename E::T;
  const FusedLayout l = fused_layout(p, m, h, dtype, true);
  const int64_t rows_p = round_up(m, E::kTile);
  ScaleRowsArgs sa;
  sa.hidden = hidden; sa.row_scale = reinterpret_cast<const float*>(ws + l.row_scale);
  sa.grad_output = grad_output; sa.valid_count = valid_count; sa.reduction = reduction;
  sa.m = (int)m; sa.m_pad = (int)rows_p; sa.h = (int)h;
  sa.out = ws + l.scaled_hidden; sa.m_dev = m_dev; sa.row_idx = row_idx;
  if (int rc = launch_scale_rows(sa, stream)) return rc;
  GemmArgs dw;
  dw.a = ws + l.scaled_hidden; dw.lda = h; dw.a_rows = (int)h;
  dw.b = ws + l.panel; dw.ldb = p.vp; dw.b_rows = (int)p.vp;
  dw.k = (int)round_up(m, 64);
  dw.k_per_split = 0;
  dw.ni = p.n_htiles; dw.nj = p.n_vtiles;
  dw.c = static_cast<T*>(grad_weight); dw.ldc = h; dw.c_rows = (int)v; dw.c_cols = (int)h;
  dw.c_split_stride = 0;
  dw.mode = kStoreT;
  dw.m_dev = m_dev; dw.m_role = kKFollows; dw.m_round = 64;
  return launch_gemm<E, true, true>(dw, 1, kClassGradWeight, stream);
}

// Soft embedding under a soft cap in two contractions instead of three
// (streaming_soft_embedding.py:60-148 computes softmax(cap(h W^T)) W with running
// maxima over vocabulary chunks): capped logits lie in [-cap, cap], so exp(z - cap)
// lies in [exp(-2 cap), 1] and needs no row maximum.  Per block of rows over the whole
// vocabulary: the panel receives exp(z - cap) in bf16 and the per-tile sums go out as
// partials, then out[r, :] = (scale / sum_r) * (panel . weight)[r, :] in float32,
// rounded once.  cap <= kSoftEmbeddingMaxCap keeps exp(-2 cap) a normal bf16 number.
constexpr float kSoftEmbeddingMaxCap = 40.0f;

template <class E>
int soft_embedding_fused_impl(const FusedPlan& p, const void* hidden, const void* weight,
                              int64_t m, int64_t h, int64_t v, int dtype, float softcap,
                              float scale, void* out, char* ws, hipStream_t stream) {
  using T = typename E::T;
  const FusedLayout l = fused_layout(p, m, h, dtype, false);
  T* panel = reinterpret_cast<T*>(ws + l.panel);
  float* part_sum = reinterpret_cast<float*>(ws + l.part_sum);
  float* part_max = reinterpret_cast<float*>(ws + l.part_max);
  float* row_scale = reinterpret_cast<float*>(ws + l.row_scale);
  float* slabs = reinterpret_cast<float*>(ws + l.slabs);
  const T* hidden_t = static_cast<const T*>(hidden);
  for (int block = 0; block < p.n_blocks; ++block) {
    const int64_t r0 = (int64_t)block * p.block_rows;
    const int64_t rows = std::min<int64_t>(p.block_rows, m - r0);
    if (rows <= 0) break;
    const int n_ttiles = (int)ceil_div(rows, E::kTile);
    const int64_t rows_p = (int64_t)n_ttiles * E::kTile;

    ExpPanelArgs ea;
    ea.hidden = hidden_t + r0 * h; ea.weight = weight;
    ea.ref = nullptr; ea.ref_const = softcap;
    ea.m = (int)rows; ea.h = (int)h; ea.v = (int)v;
    ea.exclude = -1; ea.softcap = softcap; ea.logit_scale = 1.0f;
    ea.n_ttiles = n_ttiles; ea.n_vtiles = p.n_vtiles;
    ea.panel = panel; ea.ld = p.vp;
    ea.part_sum = part_sum; ea.part_max = part_max; ea.part_ld = (int)p.block_rows;
    ea.run_flag = nullptr;
    if (int rc = launch_exp_panel_variant<E, true, true>(ea, stream)) return rc;

    SoftRowsArgs sr;
    sr.part_sum = part_sum; sr.part_ld = (int)p.block_rows; sr.n_vtiles = p.n_vtiles;
    sr.m = (int)rows; sr.m_pad = (int)rows_p; sr.scale = scale; sr.row_scale = row_scale;
    if (int rc = launch_soft_rows(sr, stream)) return rc;

    // the contraction of grad_hidden in the forward that leaves the gradients: K = the
    // vocabulary, K splits into slabs for few rows
    GemmArgs g;
    g.a = weight; g.lda = h; g.a_rows = (int)h;
    g.b = panel; g.ldb = p.vp; g.b_rows = (int)rows_p;
    g.k = (int)round_up(v, 64); g.k_per_split = 0;
    g.ni = p.n_htiles; g.nj = n_ttiles;
    g.c = slabs; g.ldc = h; g.c_rows = (int)rows_p; g.c_cols = (int)h;
    g.c_split_stride = p.block_rows * h;
    g.mode = kStoreF32;
    const int ksplit = (rows_p == p.block_rows)
                           ? p.dh_ksplit
                           : std::min(p.dh_ksplit,
                                      grad_hidden_k_splits((int64_t)n_ttiles * p.n_htiles,
                                                           p.dh_ksplit, p.vp / 64, rows_p * h));
    if (int rc = launch_gemm<E, true, false>(g, ksplit, kClassGradHidden, stream)) return rc;
    ReduceSlabsArgs rs;
    rs.slabs = slabs; rs.n_splits = ksplit; rs.split_stride = p.block_rows * h;
    rs.row_scale = row_scale; rs.m = (int)rows; rs.h = (int)h;
    rs.out = nullptr; rs.out_t = static_cast<T*>(out) + r0 * h;
    if (int rc = launch_reduce_slabs(rs, stream)) return rc;
  }
  return 0;
}

// ---- frozen-head cross entropy with top-k: the gradient formed in the forward ----
// The backward of tlce_ce_topk_* recomputes the logits to form the softmax panel
// (3 contractions per step).  Here the forward, which stages float32 logits panels
// anyway, also writes e = exp(z - reference) * cap' of every panel in bf16 into a
// panel over the whole vocabulary and contracts it with the weight rows once:
//   unit[r, :] = (multiplier / sum_r) * (e . weight)[r, :] = d lse_r / d hidden[r, :]
// (2 contractions).  The reference of a panel is the row's largest logit so far (known
// after the panel's scan), so e <= 1; panels written before a row's maximum grew are
// multiplied by exp(old - final) afterwards (lce_rescale_exp_rows_kernel).  The
// backward is then one pass over rows: ce_scale[r] * unit[r, :] plus the single-row
// terms of the label and the top-k ids, rounded once.
struct RescaleExpArgs {
  void* panel;             // bf16 [m_pad, ld]
  int64_t ld;
  int m, m_pad;
  const float* ref_used;   // [n_panels, m_pad]
  const float* run_max;    // [m] the final row maxima
  int64_t panel_width;     // columns per logits panel
  int64_t total_width;     // columns of the whole panel
};

struct TopkRowScaleArgs {
  const float* run_sum;    // [m] sum of exp(z - max)
  float multiplier;
  int m, m_pad;
  float* row_scale;        // [m_pad] multiplier / sum; 0 from m on
};

struct TopkApplyArgs {
  const float* unit;       // [m, h] d lse / d hidden
  const void* hidden;
  const void* weight;
  const int64_t* labels;
  const int64_t* top_ids;          // [m, k]
  const float* ce_scale;           // [m]
  const float* grad_top_values;    // [m, k] or null
  int m, h, k;
  float softcap, logit_scale;
  void* grad_hidden;               // bf16 [m, h]
};

int launch_rescale_exp_rows(const RescaleExpArgs& a, int n_panels, hipStream_t stream);
int launch_topk_row_scale(const TopkRowScaleArgs& a, hipStream_t stream);
int launch_topk_apply(const TopkApplyArgs& a, hipStream_t stream);

struct TopkFusedLayout {
  int64_t forward, panel, ref_used, row_scale, slabs, total;
};

// Rows are taken in blocks of the panel budget of the forward that leaves the gradients
// (its default; panel_bytes bounds the float32 logits panels here): rows are independent,
// so a block is a call of its own on a part of every per-row buffer.
inline bool topk_gradient_in_forward_supported(int64_t m, int64_t h, int64_t v, int dtype) {
  (void)m;
  return fused_gradients_supported(h, v, dtype);
}

// Rows per block of the objectives that take whole blocks of rows one after the other.
inline int64_t fused_row_block(int64_t m, int64_t h, int64_t v, int dtype) {
  return make_fused_plan(m, h, v, dtype, 0).block_rows;
}

inline TopkFusedLayout topk_fused_layout(const TopkPlan& t, const FusedPlan& p, int64_t h) {
  TopkFusedLayout l;
  int64_t off = 0;
  l.forward = off;    off += align256(t.forward_total);
  l.panel = off;      off += align256(p.block_rows * p.vp * 2);
  l.ref_used = off;   off += align256((int64_t)t.n_fpanels * p.block_rows * 4);
  l.row_scale = off;  off += align256(p.block_rows * 4);
  l.slabs = off;      off += align256((int64_t)p.dh_ksplit * p.block_rows * h * 4);
  l.total = off;
  return l;
}

template <class E>
int topk_forward_with_gradient_impl(const TopkPlan& t, const FusedPlan& p, const void* hidden,
                                    const void* weight, const int64_t* labels, int64_t m,
                                    int64_t h, int64_t v, int top_k, float multiplier,
                                    float softcap, float* losses, float* probabilities,
                                    float* top_values, int64_t* top_ids, float* lse,
                                    float* unit_grad, char* ws, hipStream_t stream) {
  using T = typename E::T;
  const TopkFusedLayout l = topk_fused_layout(t, p, h);
  char* fws = ws + l.forward;
  T* panel = reinterpret_cast<T*>(ws + l.panel);
  float* ref_used = reinterpret_cast<float*>(ws + l.ref_used);
  float* row_scale = reinterpret_cast<float*>(ws + l.row_scale);
  float* slabs = reinterpret_cast<float*>(ws + l.slabs);
  const int m_pad = (int)p.block_rows;
  TopkExpHook hook;
  hook.panel = panel; hook.ld = p.vp; hook.m_pad = m_pad; hook.ref_used = ref_used;
  if (int rc = topk_forward_impl<E>(t, hidden, weight, labels, m, h, v, top_k, multiplier,
                                    softcap, losses, probabilities, top_values, top_ids, lse,
                                    fws, stream, &hook))
    return rc;
  const float* run_max = reinterpret_cast<const float*>(fws + t.run_max);
  const float* run_sum = reinterpret_cast<const float*>(fws + t.run_sum);
  if (t.n_fpanels > 1) {
    RescaleExpArgs ra;
    ra.panel = panel; ra.ld = p.vp; ra.m = (int)m; ra.m_pad = m_pad;
    ra.ref_used = ref_used; ra.run_max = run_max;
    ra.panel_width = t.vcf; ra.total_width = p.vp;
    if (int rc = launch_rescale_exp_rows(ra, t.n_fpanels - 1, stream)) return rc;
  }
  TopkRowScaleArgs sa;
  sa.run_sum = run_sum; sa.multiplier = multiplier; sa.m = (int)m; sa.m_pad = m_pad;
  sa.row_scale = row_scale;
  if (int rc = launch_topk_row_scale(sa, stream)) return rc;

  GemmArgs g;
  g.a = weight; g.lda = h; g.a_rows = (int)h;
  g.b = panel; g.ldb = p.vp; g.b_rows = m_pad;
  g.k = (int)round_up(v, 64); g.k_per_split = 0;
  g.ni = p.n_htiles; g.nj = m_pad / E::kTile;
  g.c = slabs; g.ldc = h; g.c_rows = m_pad; g.c_cols = (int)h;
  g.c_split_stride = p.block_rows * h;
  g.mode = kStoreF32;
  if (int rc = launch_gemm<E, true, false>(g, p.dh_ksplit, kClassGradHidden, stream)) return rc;
  ReduceSlabsArgs rs;
  rs.slabs = slabs; rs.n_splits = p.dh_ksplit; rs.split_stride = p.block_rows * h;
  rs.row_scale = row_scale; rs.m = (int)m; rs.h = (int)h;
  rs.out = unit_grad;
  return launch_reduce_slabs(rs, stream);
}

// ---- frozen-head KL: the gradient formed in the forward (3 contractions, not 6) ----
// A pass over a head holds every logit of a tile in registers.  The emitting variant of
// the KL panel kernel (lce_kl_panel_kernel<.., kEmit>) finds the exact maximum of each
// token over the tile's 256 vocabulary rows and writes e = exp2(z2 - tile maximum) <= 1
// in bf16 into a panel over the whole vocabulary, beside the tile's softmax partials:
// softmax = e * exp2(tile maximum - lse2) per (token, tile) once the lse is known, and
// nothing has to be known beforehand.  One such pass over the teacher head (no teacher
// tile to read: kNoTeacher) replaces its statistics pass and its probabilities pass;
// the draft pass reads the teacher's entries, scales them to probabilities per (token,
// tile), accumulates the loss terms and emits its own entries.  One elementwise pass
// then turns the two panels into the logit gradient
//   g[r, v] = e_d * exp2(max_d[tile, r] - lse2_d[r]) - e_t * exp2(max_t[tile, r] - lse2_t[r])
// (lce_kl_grad_from_exp_kernel), and one contraction with the draft head leaves
//   unit[r, :] = d loss[r] / d draft_hidden[r, :]       float32 [m, h].
// The backward multiplies row r by its upstream gradient and rounds once.  Under a soft
// cap the gradient also carries cap'(z) = 1 - (z / cap)^2, with z re-derived from the
// entry (z2 = log2(entry) + tile maximum; the rounding of the entry moves z by less than
// 0.003); a cap of at most kSoftEmbeddingMaxCap keeps every entry a normal bf16 number.
struct KlGradFromExpArgs {
  void* exp_panel;           // bf16 [mp, ld]: e in, logit gradient out
  const void* teacher;       // bf16 [mp, ld] teacher probabilities
  int64_t ld;
  int m, mp;
  const float* part_max;     // [n_vtiles, part_ld] base-2 tile maxima of the draft
  int part_ld;
  const float* draft_lse;    // [m] natural units
  float softcap = 0.0f;      // > 0: the gradient is multiplied by cap'(z)
  const float* t_part_max = nullptr;   // non-null: `teacher` holds entries of the same kind,
  const float* t_lse = nullptr;        // these are the teacher's tile maxima and lse
  // teacher == null: the entries are only normalised (softmax of the rows, times
  // exp(-draft_lse offset) if the caller folded a factor into draft_lse)
};

// lse[r] - log(scale) from the per-tile (maximum, sum) partials of an emitting pass
// (so that exp2(tile maximum - lse2) carries the factor `scale`), and row_scale = 1
// (0 from m on) for the slab reduction that follows.
struct EmitRowsArgs {
  const float* part_max;   // [n_vtiles, part_ld] base-2 tile maxima
  const float* part_sum;   // [n_vtiles, part_ld] sums of exp2(z2 - tile maximum)
  int part_ld, n_vtiles;
  int m, m_pad;
  float scale;             // > 0
  float* lse;              // [m_pad]
  float* row_scale;        // [m_pad]
};
int launch_emit_rows(const EmitRowsArgs& a, hipStream_t stream);
int launch_kl_grad_from_exp(const KlGradFromExpArgs& a, int n_vtiles, hipStream_t stream);

constexpr float kKlMinCap = 10.0f;

struct KlFusedLayout {
  int64_t kl, teacher_parts, teacher, exp_panel, slabs, total;
};

template <class E, bool kSoftcap, bool kNoTeacher>
int launch_kl_panel_emit_variant(const KlPanelArgs& a, hipStream_t stream) {
  static LdsOptIn lds;
  constexpr int kLdsBytes = E::kSmemBytes + E::kShare * E::kTile * (int)sizeof(float);
  if (int rc = enable_large_lds(lce_kl_panel_kernel<E, kSoftcap, false, true, kNoTeacher>,
                                kLdsBytes, lds))
    return rc;
  const int grid = xcd_grid((int64_t)a.n_ttiles * a.n_ptiles);
  ScopedTimer timer(kClassGradLogits, stream);
  lce_kl_panel_kernel<E, kSoftcap, false, true, kNoTeacher>
      <<<grid, E::kThreads, kLdsBytes, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

// panel_in == null: the pass over a head on its own (no teacher tile is read)
template <class E>
int launch_kl_panel_emit(const KlPanelArgs& a, hipStream_t stream) {
  if (a.panel_in == nullptr) {
    return a.softcap > 0.0f ? launch_kl_panel_emit_variant<E, true, true>(a, stream)
                            : launch_kl_panel_emit_variant<E, false, true>(a, stream);
  }
  return a.softcap > 0.0f ? launch_kl_panel_emit_variant<E, true, false>(a, stream)
                          : launch_kl_panel_emit_variant<E, false, false>(a, stream);
}

inline bool kl_gradient_in_forward_supported(int64_t m, int64_t hd, int64_t ht, int64_t v,
                                             int dtype, float softcap) {
  (void)m;   // rows beyond one block of the panel budget are taken block by block
  // cap'(z) is re-derived from entries rounded to bf16, which moves z by up to 0.003 and
  // cap' = 1 - (z / cap)^2 by up to 0.006 / cap: negligible beside the entries whose cap'
  // is of order one, but under a small cap with every logit deep in it nothing else is
  // left (measured: 2 % of the gradient's largest entry at cap 3): caps below 10 keep the
  // sequence that evaluates cap' on the float32 logit
  const bool cap_ok = softcap <= 0.0f || (softcap >= kKlMinCap && softcap <= kSoftEmbeddingMaxCap);
  return cap_ok && fused_gradients_supported(hd, v, dtype) && engine_class(ht, dtype) == 2;
}

inline KlFusedLayout kl_fused_layout(const KlLayout& kl, const Plan& pd, const FusedPlan& p,
                                     int64_t hd) {
  KlFusedLayout l;
  int64_t off = 0;
  l.kl = off;         off += align256(kl.total);
  l.teacher_parts = off;  off += 2 * kl.tile_part;
  l.teacher = off;    off += align256(pd.mp * pd.vp * 2);
  l.exp_panel = off;  off += align256(pd.mp * pd.vp * 2);
  l.slabs = off;      off += align256((int64_t)p.dh_ksplit * pd.mp * hd * 4);
  l.total = off;
  return l;
}

template <class E>
int kl_forward_with_gradient_impl(const Plan& pd, const Plan& pt, const KlLayout& kl,
                                  const FusedPlan& fp, const void* draft_hidden,
                                  const void* draft_weight, const void* teacher_hidden,
                                  const void* teacher_weight, int64_t m, int64_t hd, int64_t ht,
                                  int64_t v, int dtype, float softcap, float* losses,
                                  float* draft_lse, float* teacher_lse, float* unit_grad,
                                  char* ws, hipStream_t stream) {
  using T = typename E::T;
  const KlFusedLayout l = kl_fused_layout(kl, pd, fp, hd);
  char* kws = ws + l.kl;
  T* teacher = reinterpret_cast<T*>(ws + l.teacher);
  T* exp_panel = reinterpret_cast<T*>(ws + l.exp_panel);
  float* slabs = reinterpret_cast<float*>(ws + l.slabs);
  float* part_max = reinterpret_cast<float*>(kws + kl.stats);
  float* part_sum = reinterpret_cast<float*>(kws + kl.stats + kl.tile_part);
  float* loss_part = reinterpret_cast<float*>(kws + kl.stats + 2 * kl.tile_part);
  float* tsum_part = reinterpret_cast<float*>(kws + kl.stats + 3 * kl.tile_part);
  float* t_part_max = reinterpret_cast<float*>(ws + l.teacher_parts);
  float* t_part_sum = reinterpret_cast<float*>(ws + l.teacher_parts + kl.tile_part);
  float* ones = reinterpret_cast<float*>(kws + kl.ones);
  (void)pt;
  ScaleArgs sa;
  sa.labels = nullptr; sa.row_idx = nullptr; sa.grad_output = nullptr; sa.valid_count = nullptr;
  sa.m = (int)m; sa.mp = (int)pd.mp; sa.reduction = TLCE_REDUCTION_SUM; sa.ignore = 0;
  sa.scale = ones; sa.constant = 1.0f; sa.multiplier = 1.0f;
  if (int rc = launch_token_scale(sa, stream)) return rc;

  auto lse_from_partials = [&](const void* hidden, const void* weight, int64_t h,
                               const float* pmax, const float* psum, float* lse) -> int {
    CombineArgs ca;
    ca.hidden = hidden; ca.weight = weight; ca.bias = nullptr; ca.labels = nullptr;
    ca.row_idx = nullptr;
    ca.m = (int)m; ca.h = (int)h; ca.v = (int)v;
    ca.ignore = 0; ca.exclude = -1; ca.softcap = softcap;
    ca.part_max = pmax; ca.part_sum = psum;
    ca.part_ld = (int)pd.mp; ca.nsplit = pd.n_vtiles;
    ca.losses = nullptr; ca.lse = lse; ca.valid_count = nullptr;
    ca.label_offset = 0; ca.local_max = nullptr; ca.local_sum = nullptr;
    ca.target_logits = nullptr;
    ScopedTimer timer(kClassCombine, stream);
    lce_combine_loss_kernel<T><<<(int)ceil_div(m, kCombineRowsPerBlock), 256, 0, stream>>>(ca);
    TLCE_LAUNCH_CHECK();
    return 0;
  };

  KlPanelArgs ka;
  ka.lse = nullptr; ka.scale = nullptr;
  ka.m = (int)m; ka.v = (int)v; ka.softcap = softcap;
  ka.v0 = 0; ka.n_ttiles = pd.n_ttiles; ka.n_ptiles = pd.n_vtiles;
  ka.ld = pd.vp; ka.part_ld = (int)pd.mp; ka.mode = kKlLoss;
  ka.loss_part = loss_part; ka.tsum_part = tsum_part;
  // the teacher head on its own: entries and softmax partials in one contraction
  ka.hidden = teacher_hidden; ka.weight = teacher_weight; ka.h = (int)ht;
  ka.panel = teacher; ka.panel_in = nullptr;
  ka.part_max = t_part_max; ka.part_sum = t_part_sum;
  if (int rc = launch_kl_panel_emit<E>(ka, stream)) return rc;
  if (int rc = lse_from_partials(teacher_hidden, teacher_weight, ht, t_part_max, t_part_sum,
                                 teacher_lse))
    return rc;
  // the draft head against it: loss terms, softmax partials and its own entries
  ka.hidden = draft_hidden; ka.weight = draft_weight; ka.h = (int)hd;
  ka.panel = exp_panel; ka.panel_in = teacher; ka.ld_in = pd.vp;
  ka.t_part_max = t_part_max; ka.t_lse = teacher_lse;
  ka.part_max = part_max; ka.part_sum = part_sum;
  if (int rc = launch_kl_panel_emit<E>(ka, stream)) return rc;
  if (int rc = lse_from_partials(draft_hidden, draft_weight, hd, part_max, part_sum, draft_lse))
    return rc;
  {
    ScopedTimer timer(kClassCombine, stream);
    if (int rc = launch_kl_finish(losses, loss_part, tsum_part, pd.n_vtiles, pd.mp, draft_lse, m,
                                  stream))
      return rc;
  }
  KlGradFromExpArgs ga;
  ga.exp_panel = exp_panel; ga.teacher = teacher; ga.ld = pd.vp;
  ga.m = (int)m; ga.mp = (int)pd.mp;
  ga.part_max = part_max; ga.part_ld = (int)pd.mp; ga.draft_lse = draft_lse;
  ga.softcap = softcap;
  ga.t_part_max = t_part_max; ga.t_lse = teacher_lse;
  if (int rc = launch_kl_grad_from_exp(ga, pd.n_vtiles, stream)) return rc;

  GemmArgs g;
  g.a = draft_weight; g.lda = hd; g.a_rows = (int)hd;
  g.b = exp_panel; g.ldb = pd.vp; g.b_rows = (int)pd.mp;
  g.k = (int)round_up(v, 64); g.k_per_split = 0;
  g.ni = fp.n_htiles; g.nj = (int)(pd.mp / E::kTile);
  g.c = slabs; g.ldc = hd; g.c_rows = (int)pd.mp; g.c_cols = (int)hd;
  g.c_split_stride = pd.mp * hd;
  g.mode = kStoreF32;
  if (int rc = launch_gemm<E, true, false>(g, fp.dh_ksplit, kClassGradHidden, stream)) return rc;
  ReduceSlabsArgs rs;
  rs.slabs = slabs; rs.n_splits = fp.dh_ksplit; rs.split_stride = pd.mp * hd;
  rs.row_scale = ones; rs.m = (int)m; rs.h = (int)hd;
  rs.out = unit_grad;
  return launch_reduce_slabs(rs, stream);
}

// Soft embedding without a usable soft cap (none, or one above kSoftEmbeddingMaxCap), in
// two contractions as well: one emitting pass over the head (entries relative to exact
// tile maxima, softmax partials), the lse merged from the partials with the embedding
// scale folded in, one elementwise pass that normalises the entries per (token, tile),
// and the contraction with the weight rows.
template <class E>
int soft_embedding_emit_impl(const FusedPlan& p, const void* hidden, const void* weight,
                             int64_t m, int64_t h, int64_t v, int dtype, float softcap,
                             float scale, void* out, char* ws, hipStream_t stream) {
  using T = typename E::T;
  const FusedLayout l = fused_layout(p, m, h, dtype, false);
  T* panel = reinterpret_cast<T*>(ws + l.panel);
  float* part_sum = reinterpret_cast<float*>(ws + l.part_sum);
  float* part_max = reinterpret_cast<float*>(ws + l.part_max);
  float* lse = reinterpret_cast<float*>(ws + l.ref_next);
  float* row_scale = reinterpret_cast<float*>(ws + l.row_scale);
  float* slabs = reinterpret_cast<float*>(ws + l.slabs);
  const T* hidden_t = static_cast<const T*>(hidden);
  for (int block = 0; block < p.n_blocks; ++block) {
    const int64_t r0 = (int64_t)block * p.block_rows;
    const int64_t rows = std::min<int64_t>(p.block_rows, m - r0);
    if (rows <= 0) break;
    const int n_ttiles = (int)ceil_div(rows, E::kTile);
    const int64_t rows_p = (int64_t)n_ttiles * E::kTile;

    KlPanelArgs ka;
    ka.hidden = hidden_t + r0 * h; ka.weight = weight; ka.lse = nullptr; ka.scale = nullptr;
    ka.m = (int)rows; ka.h = (int)h; ka.v = (int)v; ka.softcap = softcap;
    ka.v0 = 0; ka.n_ttiles = n_ttiles; ka.n_ptiles = p.n_vtiles;
    ka.panel = panel; ka.ld = p.vp; ka.panel_in = nullptr;
    ka.loss_part = nullptr; ka.tsum_part = nullptr;
    ka.part_max = part_max; ka.part_sum = part_sum; ka.part_ld = (int)p.block_rows;
    ka.mode = kKlLoss;
    if (int rc = launch_kl_panel_emit<E>(ka, stream)) return rc;

    EmitRowsArgs er;
    er.part_max = part_max; er.part_sum = part_sum; er.part_ld = (int)p.block_rows;
    er.n_vtiles = p.n_vtiles; er.m = (int)rows; er.m_pad = (int)rows_p; er.scale = scale;
    er.lse = lse; er.row_scale = row_scale;
    if (int rc = launch_emit_rows(er, stream)) return rc;

    KlGradFromExpArgs ga;
    ga.exp_panel = panel; ga.teacher = nullptr; ga.ld = p.vp;
    ga.m = (int)rows; ga.mp = (int)rows_p;
    ga.part_max = part_max; ga.part_ld = (int)p.block_rows; ga.draft_lse = lse;
    ga.softcap = 0.0f;     // a forward value: no cap'
    if (int rc = launch_kl_grad_from_exp(ga, p.n_vtiles, stream)) return rc;

    GemmArgs g;
    g.a = weight; g.lda = h; g.a_rows = (int)h;
    g.b = panel; g.ldb = p.vp; g.b_rows = (int)rows_p;
    g.k = (int)round_up(v, 64); g.k_per_split = 0;
    g.ni = p.n_htiles; g.nj = n_ttiles;
    g.c = slabs; g.ldc = h; g.c_rows = (int)rows_p; g.c_cols = (int)h;
    g.c_split_stride = p.block_rows * h;
    g.mode = kStoreF32;
    const int ksplit = (rows_p == p.block_rows)
                           ? p.dh_ksplit
                           : std::min(p.dh_ksplit,
                                      grad_hidden_k_splits((int64_t)n_ttiles * p.n_htiles,
                                                           p.dh_ksplit, p.vp / 64, rows_p * h));
    if (int rc = launch_gemm<E, true, false>(g, ksplit, kClassGradHidden, stream)) return rc;
    ReduceSlabsArgs rs;
    rs.slabs = slabs; rs.n_splits = ksplit; rs.split_stride = p.block_rows * h;
    rs.row_scale = row_scale; rs.m = (int)rows; rs.h = (int)h;
    rs.out = nullptr; rs.out_t = static_cast<T*>(out) + r0 * h;
    if (int rc = launch_reduce_slabs(rs, stream)) return rc;
  }
  return 0;
}

#define TLCE_LAUNCHERS_EXP_PANEL(X, E)                                                  \
  X int launch_kl_panel_emit<E>(const KlPanelArgs&, hipStream_t);                       \
  X int launch_exp_panel_variant<E, false, false>(const ExpPanelArgs&, hipStream_t);    \
  X int launch_exp_panel_variant<E, true, false>(const ExpPanelArgs&, hipStream_t);     \
  X int launch_exp_panel_variant<E, true, true>(const ExpPanelArgs&, hipStream_t);
#define TLCE_FUSED_ENTRY_POINTS(X, E)                                                            \
  X int fused_gradients_impl<E>(const FusedPlan&, const void*, const void*, const int64_t*,      \
                                const int64_t*, int64_t, int64_t, int64_t, int, int64_t,         \
                                int64_t, float, float*, float*, float*, float*, float*, char*,   \
                                hipStream_t, const FusedOptions&);                               \
  X int soft_embedding_fused_impl<E>(const FusedPlan&, const void*, const void*, int64_t,        \
                                     int64_t, int64_t, int, float, float, void*, char*,          \
                                     hipStream_t);                                               \
  X int soft_embedding_emit_impl<E>(const FusedPlan&, const void*, const void*, int64_t,         \
                                    int64_t, int64_t, int, float, float, void*, char*,           \
                                    hipStream_t);                                                \
  X int topk_forward_with_gradient_impl<E>(const TopkPlan&, const FusedPlan&, const void*,       \
                                           const void*, const int64_t*, int64_t, int64_t,        \
                                           int64_t, int, float, float, float*, float*, float*,   \
                                           int64_t*, float*, float*, char*, hipStream_t);        \
  X int kl_forward_with_gradient_impl<E>(const Plan&, const Plan&, const KlLayout&,              \
                                         const FusedPlan&, const void*, const void*,             \
                                         const void*, const void*, int64_t, int64_t, int64_t,    \
                                         int64_t, int, float, float*, float*, float*, float*,    \
                                         char*, hipStream_t);                                    \
  X int deferred_grad_weight_impl<E>(const FusedPlan&, const void*, int64_t, int64_t, int64_t,   \
                                     int, const float*, const float*, int, const int64_t*,       \
                                     const int64_t*, void*, char*, hipStream_t);

}  // namespace tlce
