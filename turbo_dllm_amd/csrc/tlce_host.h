// Host scheduler of the fused linear cross-entropy for gfx950: tile plans,
// workspace layouts, kernel launches and the per-objective launch sequences,
// templated on a tile engine.
//
// Replaces fused_linear_ce_forward_cuda / fused_linear_ce_backward_cuda
// (dllm_parallel/core/csrc/fused_linear_ce/fused_linear_ce_cuda.cu:898-989,
// :991-1172).  Where the reference loops over ~1K-row blocks and round-trips
// float32 logits through memory three times per block, this scheduler
//   forward : one launch of the online-softmax tile kernel (+ a per-row merge);
//   backward: loops over vocabulary panels; per panel one launch recomputes the
//             logits tiles and writes the dtype-rounded logit gradients of the
//             panel, one contraction accumulates grad_hidden in float32 and
//             one writes the panel's rows of grad_weight, complete, in dtype.
// Nothing here allocates or synchronises.
//
// The launch sequences are instantiated once per engine, each in a translation
// unit of its own (tlce_engine_*.hip), so that the library builds in parallel;
// the C ABI (tlce_linear_ce.hip) sees them as extern templates.
#pragma once

#include <stdlib.h>

#include <algorithm>
#include <atomic>
#include <functional>
#include <vector>

#include "tlce_common.h"
#include "tlce_engine_mfma.h"
#include "tlce_engine_simt.h"
#include "tlce_kernels.h"

namespace tlce {

// ------------------------------------------------------------- profiling ----
// Optional per-kernel-class timing with HIP events on the caller's stream
// (tlce_profile_begin / tlce_profile_end).  Off by default; when off a launch
// costs one thread-local pointer test.  One profiling session per thread.
enum KernelClass {
  kClassForwardStats = 0,
  kClassCombine = 1,
  kClassGradLogits = 2,
  kClassGradHidden = 3,
  kClassGradWeight = 4,
  kClassTranspose = 5,
  kClassOther = 6,
  kClassExpPanel = 7,
  kNumClasses = 8
};

struct Profiler {
  struct Record { int cls; hipEvent_t start, stop; };
  std::vector<Record> records;
};
extern thread_local Profiler* g_profiler;   // defined beside the C ABI

struct ScopedTimer {
  Profiler* prof;
  hipStream_t stream;
  hipEvent_t start = nullptr, stop = nullptr;
  int cls;
  ScopedTimer(int cls_, hipStream_t s) : prof(g_profiler), stream(s), cls(cls_) {
    if (!prof) return;
    if (hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess) {
      prof = nullptr;
      return;
    }
    (void)hipEventRecord(start, stream);
  }
  ~ScopedTimer() {
    if (!prof) return;
    (void)hipEventRecord(stop, stream);
    prof->records.push_back({cls, start, stop});
  }
};

constexpr int64_t kDefaultPanelBytes = 1ll << 30;

struct Plan {
  int engine;   // 2 = direct-to-LDS MFMA, 1 = register-staged MFMA, 0 = generic
  bool kmajor;  // gradient contractions read K-major operands in place
  int tile;
  int bk;
  int64_t mp, vp;
  int n_ttiles, n_vtiles, n_htiles;
  int nsplit;         // forward vocabulary splits
  int64_t vc;         // panel columns
  int n_panels;
  int dh_ksplit;
  int dh_max_ksplit;  // upper bound of the rule that chose dh_ksplit
};

inline int engine_class(int64_t h, int dtype) {
  if (dtype == TLCE_DTYPE_F32 || (h % 8) != 0) return 0;
  return (h % 64) == 0 ? 2 : 1;
}

inline Plan make_plan(int64_t m, int64_t h, int64_t v, int dtype, bool weight_grad,
               int64_t panel_bytes, int max_engine = 2) {
  Plan p;
  // 2: four-wave direct-to-LDS MFMA (h % 64 == 0), 1: register-staged MFMA
  // (h % 8 == 0), 0: generic float32-FMA tiles
  p.engine = std::min(engine_class(h, dtype), max_engine);
  // The direct engine reads weight, hidden and the logit-gradient panel in
  // their stored form for the gradient contractions (no transposed copies) as
  // long as every 64-row K slab of weight exists.
  p.kmajor = (p.engine == 2) && (v % 64) == 0;
  p.tile = p.engine ? 256 : 64;
  p.bk = p.engine ? 64 : 16;
  const int64_t mm = std::max<int64_t>(m, 1);
  p.mp = round_up(mm, p.tile);
  p.vp = round_up(v, p.tile);
  p.n_ttiles = (int)(p.mp / p.tile);
  p.n_vtiles = (int)(p.vp / p.tile);
  p.n_htiles = (int)ceil_div(h, p.tile);
  // forward: token tiles x vocabulary splits workgroups, at most (and close to)
  // four whole waves of 256 workgroups
  p.nsplit = forward_vocab_splits(p.n_ttiles, p.n_vtiles);
  if (panel_bytes <= 0) panel_bytes = kDefaultPanelBytes;
  const int64_t col_bytes = p.mp * dtype_bytes(dtype) * ((weight_grad && !p.kmajor) ? 2 : 1);
  int64_t tiles_per_panel = std::max<int64_t>(1, panel_bytes / col_bytes / p.tile);
  tiles_per_panel = std::min<int64_t>(tiles_per_panel, p.n_vtiles);
  // A panel of 16*k vocabulary tiles gives the grad_weight launch (tiles x
  // n_htiles workgroups) and the logit-gradient launch (tiles x n_ttiles) whole
  // waves of 256 workgroups at the usual head sizes; the last panel takes the
  // remainder.  Small problems fall back to equal panels.
  if (tiles_per_panel >= 16 && tiles_per_panel < p.n_vtiles) {
    tiles_per_panel = tiles_per_panel / 16 * 16;
    p.vc = tiles_per_panel * p.tile;
  } else {
    p.n_panels = (int)ceil_div(p.n_vtiles, tiles_per_panel);
    p.vc = ceil_div(p.n_vtiles, p.n_panels) * p.tile;  // balanced panels
  }
  p.n_panels = (int)ceil_div(p.vp, p.vc);
  // grad_hidden: n_ttiles x n_htiles tiles per panel.  When that is not close
  // to whole waves of 256 workgroups, split K (each split accumulates into its
  // own float32 slab, summed by the final cast) by the factor with the least
  // estimated time (grad_hidden_k_splits).
  p.dh_ksplit = 1;
  p.dh_max_ksplit = 1;
  if (p.engine) {
    p.dh_max_ksplit = (int)std::max<int64_t>(1, std::min<int64_t>(16, p.vc / p.bk / 8));
    p.dh_ksplit = grad_hidden_k_splits((int64_t)p.n_ttiles * p.n_htiles, p.dh_max_ksplit,
                                       p.vc / p.bk, p.mp * h);
  }
  return p;
}

// What the masked-token loss adds to the plain operator
// (distributed_block_diffusion_loss, nemotron/model.py:2084-2151): the output
// multiplier applied to the logits instead of to a copy of the hidden states,
// per-row loss weights, the weighted loss sum, and a row count that stays on
// the device (row_count != null: m is the capacity every launch is sized for).
struct RowOptions {
  float logit_scale = 1.0f;
  const float* token_weights = nullptr;   // [m] float32, compacted order
  const int64_t* row_count = nullptr;     // device int64
  float* weighted_sum = nullptr;          // forward: [1] float32 out
  // the head and its gradient are stored [h, v] (weight_dim_first of the reference's
  // extension, fused_linear_ce.cpp:104,121) and are read / written in place
  bool weight_dim_first = false;
};

// A [h, v] head is taken in place by the engine with K-major operand loaders, for
// vocabularies made of whole 64-row K slabs.
inline bool dim_first_in_place(int64_t h, int64_t v, int dtype) {
  return engine_class(h, dtype) == 2 && (v % 64) == 0;
}

struct ForwardLayout {
  int64_t part_max, part_sum, weighted, total;
};
// dynamic_rows: the partials must fit whatever plan the kernels derive from a
// device-side row count <= m (at most kTargetWorkgroups tiles, or one split of
// all token tiles); weighted: room for the per-row weighted losses.
inline ForwardLayout forward_layout(const Plan& p, bool dynamic_rows = false,
                                    bool weighted = false) {
  ForwardLayout l;
  int64_t floats = (int64_t)p.nsplit * p.mp;
  if (dynamic_rows) floats = std::max<int64_t>((int64_t)kTargetWorkgroups * p.tile, p.mp);
  const int64_t part = align256(floats * 4);
  l.part_max = 0;
  l.part_sum = part;
  l.weighted = 2 * part;
  l.total = 2 * part + (weighted ? align256(p.mp * 4) : 0);
  return l;
}

struct BackwardLayout {
  int64_t scale, acc32, wt, ht, g, gt, total;
};
// wt / gt exist only on the transposed-copy path; ht is hidden^T there and, on
// the K-major path, a copy of hidden padded to a multiple of 64 rows (only when
// m is not one already).
inline BackwardLayout backward_layout(const Plan& p, int64_t m, int64_t h, int dtype, bool weight_grad) {
  BackwardLayout l;
  const int64_t es = dtype_bytes(dtype);
  int64_t off = 0;
  l.scale = off; off += align256(p.mp * 4);
  l.acc32 = off; off += align256(p.mp * h * 4 * p.dh_ksplit);   // one slab per K split
  l.wt = off;    off += p.kmajor ? 0 : align256(h * p.vp * es);
  l.ht = off;
  if (weight_grad) {
    if (!p.kmajor) off += align256(h * p.mp * es);
    else if (m % 64 != 0) off += align256(round_up(m, 64) * h * es);
  }
  l.g = off;     off += align256(p.mp * p.vc * es);
  l.gt = off;    off += (weight_grad && !p.kmajor) ? align256(p.vc * p.mp * es) : 0;
  l.total = off;
  return l;
}

// Kernels with more than 64 KiB of dynamic LDS need the limit raised once per
// kernel and device; `done` is the calling site's per-device record.
constexpr int kMaxDevices = 64;
struct LdsOptIn {
  std::atomic<bool> done[kMaxDevices] = {};
};

template <typename K>
int enable_large_lds(K kernel, int bytes, LdsOptIn& state) {
  if (bytes <= 64 * 1024) return 0;
  int device = 0;
  TLCE_HIP(hipGetDevice(&device));
  const bool tracked = device >= 0 && device < kMaxDevices;
  if (tracked && state.done[device].load(std::memory_order_acquire)) return 0;
  TLCE_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
  if (tracked) state.done[device].store(true, std::memory_order_release);
  return 0;
}

inline int validate_common(const void* hidden, const void* weight, int64_t m, int64_t h, int64_t v,
                    int dtype) {
  TLCE_REQUIRE(dtype == TLCE_DTYPE_F32 || dtype == TLCE_DTYPE_F16 || dtype == TLCE_DTYPE_BF16,
               "unsupported dtype code %d", dtype);
  TLCE_REQUIRE(m >= 0 && h > 0 && v > 0, "bad shape m=%lld h=%lld v=%lld", (long long)m,
               (long long)h, (long long)v);
  TLCE_REQUIRE(m < (1ll << 30) && h < (1ll << 30) && v < (1ll << 30),
               "shape exceeds 32-bit tile indexing");
  TLCE_REQUIRE(weight != nullptr && (hidden != nullptr || m == 0), "null input pointer");
  TLCE_REQUIRE(((uintptr_t)hidden & 15) == 0 && ((uintptr_t)weight & 15) == 0,
               "hidden and weight must be 16-byte aligned");
  return 0;
}

// ---------------------------------------------------------------- launches --
template <class E, bool kSoftcap, bool kBias, bool kWDimFirst = false>
int launch_forward_variant(const Plan& p, const ForwardArgs& a, hipStream_t stream) {
  static LdsOptIn lds;
  if (int rc = enable_large_lds(lce_forward_stats_kernel<E, kSoftcap, kBias, kWDimFirst>,
                                E::kSmemBytes, lds))
    return rc;
  // with a device-side row count: the most tiles any row count <= m can plan
  const int64_t tiles =
      a.m_dev == nullptr
          ? (int64_t)p.n_ttiles * p.nsplit
          : std::min<int64_t>((int64_t)p.n_ttiles * p.n_vtiles,
                              std::max<int64_t>(kTargetWorkgroups, p.n_ttiles));
  const int grid = xcd_grid(tiles);
  ScopedTimer timer(kClassForwardStats, stream);
  lce_forward_stats_kernel<E, kSoftcap, kBias, kWDimFirst>
      <<<grid, E::kThreads, E::kSmemBytes, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

template <class E>
int launch_forward(const Plan& p, const ForwardArgs& a, hipStream_t stream) {
  const bool softcap = a.softcap > 0.0f, bias = a.bias != nullptr;
  if (softcap && bias) return launch_forward_variant<E, true, true>(p, a, stream);
  if (softcap) return launch_forward_variant<E, true, false>(p, a, stream);
  if (bias) return launch_forward_variant<E, false, true>(p, a, stream);
  return launch_forward_variant<E, false, false>(p, a, stream);
}

// The same over a head stored [h, v] (engines with K-major operand loaders).
template <class E>
int launch_forward_dim_first(const Plan& p, const ForwardArgs& a, hipStream_t stream) {
  if constexpr (E::kHasKMajor) {
    const bool softcap = a.softcap > 0.0f, bias = a.bias != nullptr;
    if (softcap && bias) return launch_forward_variant<E, true, true, true>(p, a, stream);
    if (softcap) return launch_forward_variant<E, true, false, true>(p, a, stream);
    if (bias) return launch_forward_variant<E, false, true, true>(p, a, stream);
    return launch_forward_variant<E, false, false, true>(p, a, stream);
  } else {
    return fail("this engine cannot read a [h, v] head in place");
  }
}

template <class E, bool kSoftcap, bool kBias, bool kWDimFirst = false>
int launch_grad_logits_variant(const GradLogitsArgs& a, hipStream_t stream) {
  static LdsOptIn lds;
  if (int rc = enable_large_lds(lce_grad_logits_panel_kernel<E, kSoftcap, kBias, kWDimFirst>,
                                E::kSmemBytes, lds))
    return rc;
  const int grid = xcd_grid((int64_t)a.n_ttiles * a.n_ptiles);
  ScopedTimer timer(kClassGradLogits, stream);
  lce_grad_logits_panel_kernel<E, kSoftcap, kBias, kWDimFirst>
      <<<grid, E::kThreads, E::kSmemBytes, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

// The logit-gradient panel over a head stored [h, v] (engines with K-major loaders).
template <class E>
int launch_grad_logits_dim_first(const GradLogitsArgs& a, hipStream_t stream) {
  if constexpr (E::kHasKMajor) {
    const bool softcap = a.softcap > 0.0f, bias = a.bias != nullptr;
    if (softcap && bias) return launch_grad_logits_variant<E, true, true, true>(a, stream);
    if (softcap) return launch_grad_logits_variant<E, true, false, true>(a, stream);
    if (bias) return launch_grad_logits_variant<E, false, true, true>(a, stream);
    return launch_grad_logits_variant<E, false, false, true>(a, stream);
  } else {
    return fail("this engine cannot read a [h, v] head in place");
  }
}

template <class E>
int launch_grad_logits(const GradLogitsArgs& a, hipStream_t stream) {
  const bool softcap = a.softcap > 0.0f, bias = a.bias != nullptr;
  if (softcap && bias) return launch_grad_logits_variant<E, true, true>(a, stream);
  if (softcap) return launch_grad_logits_variant<E, true, false>(a, stream);
  if (bias) return launch_grad_logits_variant<E, false, true>(a, stream);
  return launch_grad_logits_variant<E, false, false>(a, stream);
}

template <class E, bool kAKMajor, bool kBKMajor>
int launch_gemm(GemmArgs a, int ksplit, int cls, hipStream_t stream) {
  static LdsOptIn lds;
  if (int rc = enable_large_lds(lce_gemm_nt_kernel<E, kAKMajor, kBKMajor>, E::kSmemBytes, lds))
    return rc;
  const int ksteps = a.k / E::kBK;
  a.k_per_split = (int)ceil_div(ksteps, ksplit) * E::kBK;
  // ksplit is the number of splits launched; with a device-side row count the
  // kernel may use fewer of them (a.slab_budget then bounds splits x slab)
  dim3 grid(xcd_grid((int64_t)a.ni * a.nj), ksplit, 1);
  ScopedTimer timer(cls, stream);
  lce_gemm_nt_kernel<E, kAKMajor, kBKMajor><<<grid, E::kThreads, E::kSmemBytes, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_transpose(const T* in, int64_t ld_in, int64_t rows, int64_t cols, T* out,
                     int64_t ld_out, int64_t out_cols, hipStream_t stream,
                     const int64_t* rows_dev = nullptr) {
  dim3 grid((unsigned)ceil_div(cols, 64), (unsigned)ceil_div(out_cols, 64), 1);
  TLCE_REQUIRE(grid.y <= 65535, "transpose: too many row tiles");
  ScopedTimer timer(kClassTranspose, stream);
  lce_transpose_pad_kernel<T><<<grid, 256, 0, stream>>>(in, ld_in, (int)rows, (int)cols, out,
                                                        ld_out, (int)out_cols, rows_dev);
  TLCE_LAUNCH_CHECK();
  return 0;
}

// Launchers of the engine-independent kernels (tlce_row_kernels.h), defined
// beside the C ABI.
int fill_zero(void* dst, int64_t bytes, hipStream_t stream);
int launch_token_scale(const ScaleArgs& sa, hipStream_t stream);
int launch_kl_finish(float* losses, const float* loss_part, const float* tsum_part, int n_tiles,
                     int64_t part_ld, const float* lse, int64_t m, hipStream_t stream);
int launch_topk_scan(const TopkScanArgs& sa, hipStream_t stream);
int launch_sum(const float* x, int64_t n, float* out, hipStream_t stream);

// ----------------------------------------------------------------- forward --
// Outputs of the vocabulary-shard forward (all null for the full-vocabulary one).
struct ShardStats {
  int64_t vocab_start = 0;
  float* local_max = nullptr;
  float* local_sum = nullptr;
  float* target_logits = nullptr;
};

template <class E>
int forward_impl(const Plan& p, const void* hidden, const void* weight, const float* bias,
                 const int64_t* labels, const int64_t* row_idx, int64_t m, int64_t h, int64_t v,
                 int64_t ignore, int64_t exclude, float softcap, float* losses, float* lse,
                 float* valid_count, const ShardStats& shard, char* ws, hipStream_t stream,
                 const RowOptions& opt) {
  using T = typename E::T;
  const bool dynamic = opt.row_count != nullptr;
  const ForwardLayout l = forward_layout(p, dynamic, opt.weighted_sum != nullptr);
  ForwardArgs fa;
  fa.hidden = hidden; fa.weight = weight; fa.bias = bias;
  fa.m = (int)m; fa.h = (int)h; fa.v = (int)v;
  fa.exclude = exclude - shard.vocab_start; fa.softcap = softcap;
  fa.logit_scale = opt.logit_scale; fa.m_dev = opt.row_count;
  fa.n_ttiles = p.n_ttiles; fa.n_vtiles = p.n_vtiles; fa.nsplit = p.nsplit;
  fa.part_max = reinterpret_cast<float*>(ws + l.part_max);
  fa.part_sum = reinterpret_cast<float*>(ws + l.part_sum);
  fa.part_ld = (int)p.mp;
  if (opt.weight_dim_first) {
    if (int rc = launch_forward_dim_first<E>(p, fa, stream)) return rc;
  } else {
    if (int rc = launch_forward<E>(p, fa, stream)) return rc;
  }

  CombineArgs ca;
  ca.hidden = hidden; ca.weight = weight; ca.bias = bias; ca.labels = labels;
  ca.row_idx = row_idx;
  ca.m = (int)m; ca.h = (int)h; ca.v = (int)v;
  ca.ignore = ignore; ca.exclude = exclude; ca.softcap = softcap;
  ca.part_max = fa.part_max; ca.part_sum = fa.part_sum;
  ca.part_ld = fa.part_ld; ca.nsplit = p.nsplit;
  ca.losses = losses; ca.lse = lse; ca.valid_count = valid_count;
  ca.label_offset = shard.vocab_start;
  ca.local_max = shard.local_max; ca.local_sum = shard.local_sum;
  ca.target_logits = shard.target_logits;
  ca.logit_scale = opt.logit_scale; ca.token_weights = opt.token_weights;
  ca.n_vtiles = p.n_vtiles; ca.tile = p.tile; ca.m_dev = opt.row_count;
  ca.weight_dim_first = opt.weight_dim_first;
  float* weighted = reinterpret_cast<float*>(ws + l.weighted);
  if (opt.weighted_sum != nullptr) {
    ca.weighted = weighted;
    ca.weighted_rows = (int)m;
  }
  {
    ScopedTimer timer(kClassCombine, stream);
    lce_combine_loss_kernel<T><<<(int)ceil_div(m, kCombineRowsPerBlock), 256, 0, stream>>>(ca);
  }
  TLCE_LAUNCH_CHECK();
  if (opt.weighted_sum != nullptr) return launch_sum(weighted, m, opt.weighted_sum, stream);
  return 0;
}

// ---------------------------------------------------------------- backward --
// The panel loop shared by every objective whose gradient is G . weight (and
// G^T . hidden): `produce(v0, width, g, gt)` fills the panel of rounded logit
// gradients for the vocabulary rows [v0, v0 + width); the loop contracts it
// into the float32 grad_hidden slabs and, when grad_weight != null, into the
// panel's rows of grad_weight, then casts / un-compacts grad_hidden.
template <class E, class Producer>
int panel_contractions(const Plan& p, const BackwardLayout& l, const void* hidden,
                       const void* weight, const int64_t* row_idx, int64_t m, int64_t n_out,
                       int64_t h, int64_t v, int dtype, void* grad_hidden, void* grad_weight,
                       char* ws, hipStream_t stream, Producer&& produce,
                       const std::function<int(float*)>& before_cast = nullptr,
                       const int64_t* m_dev = nullptr, bool dim_first = false) {
  using T = typename E::T;
  const bool weight_grad = grad_weight != nullptr;
  float* acc32 = reinterpret_cast<float*>(ws + l.acc32);
  T* wt = reinterpret_cast<T*>(ws + l.wt);
  T* ht = reinterpret_cast<T*>(ws + l.ht);
  T* g = reinterpret_cast<T*>(ws + l.g);
  T* gt = (weight_grad && !p.kmajor) ? reinterpret_cast<T*>(ws + l.gt) : nullptr;

  const T* hidden_t = static_cast<const T*>(hidden);
  const T* weight_t = static_cast<const T*>(weight);
  const T* hidden_k = hidden_t;          // K-major operand of grad_weight
  const int64_t m64 = round_up(m, 64);
  if (!p.kmajor) {
    // K-contiguous copies for engines that cannot read K-major operands
    if (int rc = launch_transpose<T>(weight_t, h, v, h, wt, p.vp, p.vp, stream)) return rc;
    if (weight_grad) {
      if (int rc = launch_transpose<T>(hidden_t, h, m, h, ht, p.mp, p.mp, stream, m_dev))
        return rc;
    }
  } else if (weight_grad && m64 != m && m_dev == nullptr) {
    // whole 64-row K slabs must exist: pad hidden with zero rows
    TLCE_HIP(hipMemcpyAsync(ht, hidden_t, (size_t)(m * h * sizeof(T)), hipMemcpyDeviceToDevice,
                            stream));
    if (int rc = fill_zero(ht + m * h, (m64 - m) * h * (int64_t)sizeof(T), stream)) return rc;
    hidden_k = ht;
  }

  for (int panel = 0; panel < p.n_panels; ++panel) {
    const int64_t v0 = (int64_t)panel * p.vc;
    const int64_t width = std::min<int64_t>(p.vc, p.vp - v0);   // multiple of tile
    const int64_t rows_valid = std::min<int64_t>(p.vc, v - v0);  // real vocabulary rows
    if (int rc = produce(v0, width, g, gt)) return rc;

    GemmArgs dh;
    dh.b = g; dh.ldb = p.vc; dh.b_rows = (int)p.mp;
    dh.k_per_split = 0;
    dh.ni = p.n_htiles; dh.nj = p.n_ttiles;
    dh.c = acc32; dh.ldc = h; dh.c_rows = (int)p.mp; dh.c_cols = (int)h;
    dh.c_split_stride = p.mp * h;
    dh.mode = (panel == 0) ? kStoreF32 : kAddF32;
    dh.m_dev = m_dev; dh.m_role = kRowsFollow;
    // device-side row count: up to four K splits are launched and the kernel picks
    // how many to use for the real count, within the slabs the plan allocated
    const int dh_launch_ksplit =
        m_dev == nullptr ? p.dh_ksplit : std::max(p.dh_ksplit, std::min(4, p.dh_max_ksplit));
    dh.slab_budget = (int64_t)p.dh_ksplit * p.mp * h;
    dh.k_steps_plan = (int)(p.vc / p.bk);
    GemmArgs dw;
    dw.m_dev = m_dev; dw.m_role = kKFollows; dw.m_round = p.bk;
    dw.k_per_split = 0;
    dw.ni = p.n_htiles; dw.nj = (int)(width / p.tile);
    dw.c = weight_grad ? static_cast<T*>(grad_weight) + v0 * h : nullptr; dw.ldc = h;
    dw.c_rows = (int)rows_valid; dw.c_cols = (int)h;
    dw.c_split_stride = 0;
    dw.mode = kStoreT;
    if constexpr (E::kHasKMajor) {
      if (p.kmajor && dim_first) {
        // The head is stored [h, v].  grad_hidden: A = its columns [v0, v0+K), which
        // are K-contiguous rows of the stored matrix; B = G.
        dh.a = weight_t + v0; dh.lda = v; dh.a_rows = (int)h;
        dh.k = (int)round_up(rows_valid, 64);
        if (int rc = launch_gemm<E, false, false>(dh, dh_launch_ksplit, kClassGradHidden, stream))
          return rc;
        if (weight_grad) {
          // grad_weight [h, v]: the roles of the operands swap so that the hidden axis
          // becomes the output's rows: A = G (its panel columns), B = hidden, both K-major
          GemmArgs dwt = dw;
          dwt.a = g; dwt.lda = p.vc; dwt.a_rows = (int)width;
          dwt.b = hidden_k; dwt.ldb = h; dwt.b_rows = (int)h;
          dwt.k = (int)m64;
          dwt.ni = (int)(width / p.tile); dwt.nj = p.n_htiles;
          dwt.c = static_cast<T*>(grad_weight) + v0; dwt.ldc = v;
          dwt.c_rows = (int)h; dwt.c_cols = (int)rows_valid;
          if (int rc = launch_gemm<E, true, true>(dwt, 1, kClassGradWeight, stream)) return rc;
        }
        continue;
      }
      if (p.kmajor) {
        // grad_hidden: A = weight rows [v0, v0+K) as stored (K-major), B = G
        dh.a = weight_t + v0 * h; dh.lda = h; dh.a_rows = (int)h;
        dh.k = (int)round_up(rows_valid, 64);
        if (int rc = launch_gemm<E, true, false>(dh, dh_launch_ksplit, kClassGradHidden, stream))
          return rc;
        if (weight_grad) {
          // grad_weight: A = hidden as stored, B = G as stored, both K-major (K = token)
          dw.a = hidden_k; dw.lda = h; dw.a_rows = (int)h;
          dw.b = g; dw.ldb = p.vc; dw.b_rows = (int)width;
          dw.k = (int)m64;
          if (int rc = launch_gemm<E, true, true>(dw, 1, kClassGradWeight, stream)) return rc;
        }
        continue;
      }
    }
    dh.a = wt + v0; dh.lda = p.vp; dh.a_rows = (int)h;
    dh.k = (int)width;
    if (int rc = launch_gemm<E, false, false>(dh, dh_launch_ksplit, kClassGradHidden, stream))
      return rc;
    if (weight_grad) {
      dw.a = ht; dw.lda = p.mp; dw.a_rows = (int)h;
      dw.b = gt; dw.ldb = p.mp; dw.b_rows = (int)width;
      dw.k = (int)p.mp;
      if (int rc = launch_gemm<E, false, false>(dw, 1, kClassGradWeight, stream)) return rc;
    }
  }

  if (before_cast) {
    if (int rc = before_cast(acc32)) return rc;   // extra float32 terms of grad_hidden
  }
  if (row_idx != nullptr || m_dev != nullptr) {
    if (int rc = fill_zero(grad_hidden, n_out * h * dtype_bytes(dtype), stream)) return rc;
  }
  {
    ScopedTimer timer(kClassOther, stream);
    lce_finalize_grad_hidden_kernel<T><<<(int)m, 256, 0, stream>>>(
        acc32, p.dh_ksplit, p.mp * h, row_idx, (int)m, (int)h, static_cast<T*>(grad_hidden),
        m_dev, p.n_htiles, p.tile, std::max(p.dh_ksplit, std::min(4, p.dh_max_ksplit)),
        (int)(p.vc / p.bk));
  }
  TLCE_LAUNCH_CHECK();
  return 0;
}

// vocab_start: global id of weight row 0 (labels and exclude are global ids).
// labels == null: the "gradient" panel holds softmax * probabilities_scale, so
// grad_hidden becomes the probability-weighted sum of weight rows.
template <class E>
int backward_impl(const Plan& p, const void* hidden, const void* weight, const float* bias,
                  const int64_t* labels, const int64_t* row_idx, const float* lse,
                  const float* valid_count, const float* grad_output, int64_t m, int64_t n_out,
                  int64_t h, int64_t v, int dtype, int reduction, int64_t ignore, int64_t exclude,
                  float softcap, int64_t vocab_start, void* grad_hidden, void* grad_weight,
                  float* grad_bias, char* ws, hipStream_t stream,
                  float probabilities_scale, const RowOptions& opt) {
  const BackwardLayout l = backward_layout(p, m, h, dtype, grad_weight != nullptr);
  float* scale = reinterpret_cast<float*>(ws + l.scale);
  ScaleArgs sa;
  sa.labels = labels; sa.row_idx = row_idx; sa.grad_output = grad_output;
  sa.valid_count = valid_count; sa.m = (int)m; sa.mp = (int)p.mp; sa.reduction = reduction;
  sa.ignore = ignore; sa.scale = scale; sa.constant = probabilities_scale;
  // the gradient with respect to the raw dot products carries the logit multiplier
  sa.multiplier = opt.logit_scale;
  sa.token_weights = opt.token_weights; sa.m_dev = opt.row_count;
  if (int rc = launch_token_scale(sa, stream)) return rc;
  if (grad_bias != nullptr) {
    if (int rc = fill_zero(grad_bias, v * 4, stream)) return rc;
  }
  auto produce = [&](int64_t v0, int64_t width, void* g, void* gt) -> int {
    GradLogitsArgs ga;
    ga.hidden = hidden; ga.weight = weight; ga.bias = bias; ga.labels = labels;
    ga.lse = lse; ga.scale = scale;
    ga.m = (int)m; ga.h = (int)h; ga.v = (int)v;
    ga.ignore = ignore; ga.exclude = exclude - vocab_start; ga.softcap = softcap;
    ga.label_offset = vocab_start;
    ga.probabilities = (labels == nullptr) ? 1 : 0;
    ga.cap_grad = (labels == nullptr) ? 0 : 1;
    ga.logit_scale = opt.logit_scale; ga.m_dev = opt.row_count;
    ga.v0 = (int)v0;
    ga.n_ttiles = p.n_ttiles; ga.n_ptiles = (int)(width / p.tile);
    ga.g = g; ga.ldg = p.vc; ga.gt = gt; ga.ldgt = p.mp;
    ga.grad_bias = (bias != nullptr) ? grad_bias : nullptr;
    if (opt.weight_dim_first) return launch_grad_logits_dim_first<E>(ga, stream);
    return launch_grad_logits<E>(ga, stream);
  };
  return panel_contractions<E>(p, l, hidden, weight, row_idx, m, n_out, h, v, dtype, grad_hidden,
                               grad_weight, ws, stream, produce, nullptr, opt.row_count,
                               opt.weight_dim_first);
}

// -------------------------------------------------------------- frozen KL ----
// KL(teacher || draft) of two frozen heads over one vocabulary
// (fused_dflash_kl_forward_cuda / _backward_cuda, fused_linear_ce_cuda.cu:1270-1509).
// Both heads run on one engine class (the less demanding of the two hidden sizes).
struct KlLayout {
  // stats: the teacher's forward partials, then the draft's per-tile partials
  // (part_max, part_sum, loss terms, teacher mass: n_vtiles x mp float32 each);
  // backward: BackwardLayout of the draft head
  int64_t stats, tile_part, ones, backward, total;
};

inline KlLayout kl_layout(const Plan& pd, const Plan& pt, int64_t m, int64_t hd, int dtype) {
  KlLayout l;
  l.stats = 0;
  l.tile_part = align256((int64_t)pd.n_vtiles * pd.mp * 4);
  int64_t off = std::max(4 * l.tile_part, forward_layout(pt).total);
  l.ones = off;      off += align256(pd.mp * 4);
  l.backward = off;  off += backward_layout(pd, m, hd, dtype, false).total;
  l.total = off;
  return l;
}

template <class E, bool kSoftcap, bool kGrad>
int launch_kl_panel_variant(const KlPanelArgs& a, hipStream_t stream) {
  static LdsOptIn lds;
  if (int rc = enable_large_lds(lce_kl_panel_kernel<E, kSoftcap, kGrad>, E::kSmemBytes, lds))
    return rc;
  const int grid = xcd_grid((int64_t)a.n_ttiles * a.n_ptiles);
  ScopedTimer timer(kClassGradLogits, stream);
  lce_kl_panel_kernel<E, kSoftcap, kGrad><<<grid, E::kThreads, E::kSmemBytes, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

template <class E>
int launch_kl_panel(const KlPanelArgs& a, hipStream_t stream) {
  const bool grad = a.mode == kKlGrad;
  if (a.softcap > 0.0f) {
    return grad ? launch_kl_panel_variant<E, true, true>(a, stream)
                : launch_kl_panel_variant<E, true, false>(a, stream);
  }
  return grad ? launch_kl_panel_variant<E, false, true>(a, stream)
              : launch_kl_panel_variant<E, false, false>(a, stream);
}

// Teacher probabilities of the panel [v0, v0 + width), then the draft pass over it.
template <class E>
int kl_panel(const Plan& pd, const void* draft_hidden, const void* draft_weight,
             const void* teacher_hidden, const void* teacher_weight, const float* draft_lse,
             const float* teacher_lse, const float* ones, const float* scale, int64_t m,
             int64_t hd, int64_t ht, int64_t v, float softcap, int64_t v0, int64_t width,
             void* g, float* loss_part, float* tsum_part, float* part_max, float* part_sum,
             int mode, hipStream_t stream, void* kept = nullptr, int64_t kept_ld = 0,
             bool kept_is_written = false) {
  // kept: a buffer over the whole vocabulary [mp, kept_ld] that holds the teacher
  // probabilities between forward and backward.  The forward produces each panel into
  // it (and reads it there); the backward (kept_is_written) skips the producer and
  // reads the panel from it, writing the logit gradients to g.
  void* teacher_panel = kept != nullptr ? static_cast<char*>(kept) + v0 * (int64_t)sizeof(typename E::T) : g;
  const int64_t teacher_ld = kept != nullptr ? kept_ld : pd.vc;
  KlPanelArgs ka;
  ka.hidden = draft_hidden; ka.weight = draft_weight; ka.lse = draft_lse; ka.scale = scale;
  ka.m = (int)m; ka.h = (int)hd; ka.v = (int)v; ka.softcap = softcap;
  ka.v0 = (int)v0; ka.n_ttiles = pd.n_ttiles; ka.n_ptiles = (int)(width / pd.tile);
  ka.loss_part = loss_part; ka.tsum_part = tsum_part;
  ka.part_max = part_max; ka.part_sum = part_sum; ka.part_ld = (int)pd.mp; ka.mode = mode;
  if (kept != nullptr && kept_is_written) {
    ka.panel = g; ka.ld = pd.vc; ka.panel_in = teacher_panel; ka.ld_in = teacher_ld;
    return launch_kl_panel<E>(ka, stream);
  }
  GradLogitsArgs ga;
  ga.hidden = teacher_hidden; ga.weight = teacher_weight; ga.bias = nullptr;
  ga.labels = nullptr; ga.lse = teacher_lse; ga.scale = ones;
  ga.m = (int)m; ga.h = (int)ht; ga.v = (int)v;
  ga.ignore = 0; ga.exclude = -1; ga.softcap = softcap;
  ga.label_offset = 0; ga.probabilities = 1; ga.cap_grad = 0; ga.logit_scale = 1.0f;
  ga.v0 = (int)v0;
  ga.n_ttiles = pd.n_ttiles; ga.n_ptiles = (int)(width / pd.tile);
  ga.g = teacher_panel; ga.ldg = teacher_ld; ga.gt = nullptr; ga.ldgt = 0;
  ga.grad_bias = nullptr;
  if (int rc = launch_grad_logits<E>(ga, stream)) return rc;
  ka.panel = teacher_panel; ka.ld = teacher_ld;
  return launch_kl_panel<E>(ka, stream);
}

template <class E>
int kl_forward_impl(const Plan& pd, const Plan& pt, const KlLayout& l, const void* draft_hidden,
                    const void* draft_weight, const void* teacher_hidden,
                    const void* teacher_weight, int64_t m, int64_t hd, int64_t ht, int64_t v,
                    int dtype, float softcap, float* losses, float* draft_lse, float* teacher_lse,
                    char* ws, hipStream_t stream, void* kept_teacher = nullptr) {
  using T = typename E::T;
  // teacher statistics first: its probabilities need the teacher lse
  if (int rc = forward_impl<E>(pt, teacher_hidden, teacher_weight, nullptr, nullptr, nullptr, m,
                               ht, v, 0, -1, softcap, nullptr, teacher_lse, nullptr, ShardStats{},
                               ws + l.stats, stream, RowOptions{}))
    return rc;
  float* ones = reinterpret_cast<float*>(ws + l.ones);
  float* part_max = reinterpret_cast<float*>(ws + l.stats);
  float* part_sum = reinterpret_cast<float*>(ws + l.stats + l.tile_part);
  float* loss_part = reinterpret_cast<float*>(ws + l.stats + 2 * l.tile_part);
  float* tsum_part = reinterpret_cast<float*>(ws + l.stats + 3 * l.tile_part);
  ScaleArgs sa;
  sa.labels = nullptr; sa.row_idx = nullptr; sa.grad_output = nullptr; sa.valid_count = nullptr;
  sa.m = (int)m; sa.mp = (int)pd.mp; sa.reduction = TLCE_REDUCTION_SUM; sa.ignore = 0;
  sa.scale = ones; sa.constant = 1.0f; sa.multiplier = 1.0f;
  if (int rc = launch_token_scale(sa, stream)) return rc;
  // one pass over the draft head per panel: loss terms and the draft's per-tile
  // softmax partials (the teacher partials above are dead by now)
  const BackwardLayout bl = backward_layout(pd, m, hd, dtype, false);
  void* g = ws + l.backward + bl.g;
  // teacher probabilities that go to a buffer over the whole vocabulary need no bounded
  // panel: one launch of each kernel covers all of it (fewer partly filled last rounds)
  const int n_panels = kept_teacher != nullptr ? 1 : pd.n_panels;
  const int64_t panel_width = kept_teacher != nullptr ? pd.vp : pd.vc;
  for (int panel = 0; panel < n_panels; ++panel) {
    const int64_t v0 = (int64_t)panel * panel_width;
    const int64_t width = std::min<int64_t>(panel_width, pd.vp - v0);
    if (int rc = kl_panel<E>(pd, draft_hidden, draft_weight, teacher_hidden, teacher_weight,
                             nullptr, teacher_lse, ones, nullptr, m, hd, ht, v, softcap, v0,
                             width, g, loss_part, tsum_part, part_max, part_sum, kKlLoss,
                             stream, kept_teacher, pd.vp, false))
      return rc;
  }
  CombineArgs ca;
  ca.hidden = draft_hidden; ca.weight = draft_weight; ca.bias = nullptr; ca.labels = nullptr;
  ca.row_idx = nullptr;
  ca.m = (int)m; ca.h = (int)hd; ca.v = (int)v;
  ca.ignore = 0; ca.exclude = -1; ca.softcap = softcap;
  ca.part_max = part_max; ca.part_sum = part_sum;
  ca.part_ld = (int)pd.mp; ca.nsplit = pd.n_vtiles;
  ca.losses = nullptr; ca.lse = draft_lse; ca.valid_count = nullptr;
  ca.label_offset = 0; ca.local_max = nullptr; ca.local_sum = nullptr; ca.target_logits = nullptr;
  {
    ScopedTimer timer(kClassCombine, stream);
    lce_combine_loss_kernel<T><<<(int)ceil_div(m, kCombineRowsPerBlock), 256, 0, stream>>>(ca);
    TLCE_LAUNCH_CHECK();
    if (int rc = launch_kl_finish(losses, loss_part, tsum_part, pd.n_vtiles, pd.mp, draft_lse, m,
                                  stream))
      return rc;
  }
  return 0;
}

template <class E>
int kl_backward_impl(const Plan& pd, const KlLayout& l, const void* draft_hidden,
                     const void* draft_weight, const void* teacher_hidden,
                     const void* teacher_weight, const float* draft_lse, const float* teacher_lse,
                     const float* grad_output, int64_t m, int64_t hd, int64_t ht, int64_t v,
                     int dtype, float softcap, void* grad_hidden, char* ws, hipStream_t stream,
                     const void* kept_teacher = nullptr) {
  float* ones = reinterpret_cast<float*>(ws + l.ones);
  char* bws = ws + l.backward;
  const BackwardLayout bl = backward_layout(pd, m, hd, dtype, false);
  float* scale = reinterpret_cast<float*>(bws + bl.scale);
  ScaleArgs sa;
  sa.labels = nullptr; sa.row_idx = nullptr; sa.grad_output = nullptr; sa.valid_count = nullptr;
  sa.m = (int)m; sa.mp = (int)pd.mp; sa.reduction = TLCE_REDUCTION_NONE; sa.ignore = 0;
  sa.scale = ones; sa.constant = 1.0f; sa.multiplier = 1.0f;
  if (int rc = launch_token_scale(sa, stream)) return rc;
  sa.grad_output = grad_output; sa.scale = scale;   // scale[r] = grad_output[r]
  if (int rc = launch_token_scale(sa, stream)) return rc;
  auto produce = [&](int64_t v0, int64_t width, void* g, void*) -> int {
    return kl_panel<E>(pd, draft_hidden, draft_weight, teacher_hidden, teacher_weight, draft_lse,
                       teacher_lse, ones, scale, m, hd, ht, v, softcap, v0, width, g, nullptr,
                       nullptr, nullptr, nullptr, kKlGrad, stream,
                       const_cast<void*>(kept_teacher), pd.vp, kept_teacher != nullptr);
  };
  return panel_contractions<E>(pd, bl, draft_hidden, draft_weight, nullptr, m, m, hd, v, dtype,
                               grad_hidden, nullptr, bws, stream, produce);
}

// ------------------------------------------------ cross entropy + top-k ----
struct TopkPlan {
  Plan plan;            // engine, tiles and the backward's panels (input dtype)
  int64_t vcf;          // columns of a float32 logits panel
  int n_fpanels;
  int64_t run_max, run_sum, fpanel, forward_total;
  int64_t ce_scale, backward, backward_total;
};

inline TopkPlan topk_plan(int64_t m, int64_t h, int64_t v, int dtype, int64_t panel_bytes) {
  TopkPlan t;
  t.plan = make_plan(m, h, v, dtype, false, panel_bytes);
  const Plan& p = t.plan;
  if (panel_bytes <= 0) panel_bytes = kDefaultPanelBytes;
  int64_t tiles = std::max<int64_t>(1, panel_bytes / (p.mp * 4) / p.tile);
  tiles = std::min<int64_t>(tiles, p.n_vtiles);
  if (tiles >= 16 && tiles < p.n_vtiles) tiles = tiles / 16 * 16;
  t.vcf = tiles * p.tile;
  t.n_fpanels = (int)ceil_div(p.vp, t.vcf);
  int64_t off = 0;
  t.run_max = off;  off += align256(m * 4);
  t.run_sum = off;  off += align256(m * 4);
  t.fpanel = off;   off += align256(p.mp * t.vcf * 4);
  t.forward_total = off;
  off = 0;
  t.ce_scale = off; off += align256(p.mp * 4);
  t.backward = off; off += backward_layout(p, m, h, dtype, false).total;
  t.backward_total = off;
  return t;
}

template <class E, bool kSoftcap>
int launch_logits_panel_variant(const LogitsPanelArgs& a, hipStream_t stream) {
  static LdsOptIn lds;
  if (int rc = enable_large_lds(lce_logits_panel_kernel<E, kSoftcap>, E::kSmemBytes, lds))
    return rc;
  const int grid = xcd_grid((int64_t)a.n_ttiles * a.n_ptiles);
  ScopedTimer timer(kClassGradLogits, stream);
  lce_logits_panel_kernel<E, kSoftcap><<<grid, E::kThreads, E::kSmemBytes, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

// After the scan of a float32 logits panel: exp(logit - the row's largest logit so
// far) * cap' of that panel, rounded to bf16, into a panel over the whole vocabulary
// (the operand of the gradient contraction formed in the forward).
struct ExpFromLogitsArgs {
  const float* logits;   // [m, ld] float32 (columns past the vocabulary hold -inf)
  int64_t ld;
  int m, m_pad;          // rows with logits; rows of `out` to define (zeros from m on)
  int width;             // columns of this logits panel, a multiple of 8
  float softcap;
  const float* run_max;  // [m] the reference: the row's largest logit so far
  float* ref_used;       // [m] out: the reference this panel was written with
  void* out;             // bf16 [m_pad, ld_out]; this panel goes to columns col0 ...
  int64_t ld_out, col0;
};
int launch_exp_from_logits(const ExpFromLogitsArgs& a, hipStream_t stream);

struct TopkExpHook {
  void* panel;           // bf16 [m_pad, ld]
  int64_t ld;
  int m_pad;
  float* ref_used;       // [n_fpanels, m_pad]
};

template <class E>
int topk_forward_impl(const TopkPlan& t, const void* hidden, const void* weight,
                      const int64_t* labels, int64_t m, int64_t h, int64_t v, int top_k,
                      float multiplier, float softcap, float* losses, float* probabilities,
                      float* top_values, int64_t* top_ids, float* lse, char* ws,
                      hipStream_t stream, const TopkExpHook* hook = nullptr) {
  using T = typename E::T;
  const Plan& p = t.plan;
  float* run_max = reinterpret_cast<float*>(ws + t.run_max);
  float* run_sum = reinterpret_cast<float*>(ws + t.run_sum);
  float* panel = reinterpret_cast<float*>(ws + t.fpanel);
  for (int pi = 0; pi < t.n_fpanels; ++pi) {
    const int64_t v0 = (int64_t)pi * t.vcf;
    const int64_t width = std::min<int64_t>(t.vcf, p.vp - v0);
    const int64_t valid = std::min<int64_t>(t.vcf, v - v0);
    LogitsPanelArgs la;
    la.hidden = hidden; la.weight = weight;
    la.m = (int)m; la.h = (int)h; la.v = (int)v;
    la.softcap = softcap; la.logit_scale = multiplier;
    la.v0 = (int)v0; la.n_ttiles = p.n_ttiles; la.n_ptiles = (int)(width / p.tile);
    la.panel = panel; la.ld = t.vcf;
    if (softcap > 0.0f) {
      if (int rc = launch_logits_panel_variant<E, true>(la, stream)) return rc;
    } else {
      if (int rc = launch_logits_panel_variant<E, false>(la, stream)) return rc;
    }
    TopkScanArgs sa;
    sa.panel = panel; sa.ld = t.vcf; sa.m = (int)m; sa.v0 = v0; sa.width = (int)valid;
    sa.k = top_k; sa.first = pi == 0;
    sa.run_max = run_max; sa.run_sum = run_sum; sa.top_values = top_values; sa.top_ids = top_ids;
    if (int rc = launch_topk_scan(sa, stream)) return rc;
    if (hook != nullptr) {
      ExpFromLogitsArgs xa;
      xa.logits = panel; xa.ld = t.vcf; xa.m = (int)m; xa.m_pad = hook->m_pad;
      xa.width = (int)width; xa.softcap = softcap;
      xa.run_max = run_max; xa.ref_used = hook->ref_used + (int64_t)pi * hook->m_pad;
      xa.out = hook->panel; xa.ld_out = hook->ld; xa.col0 = v0;
      if (int rc = launch_exp_from_logits(xa, stream)) return rc;
    }
  }
  TopkFinishArgs fa;
  fa.hidden = hidden; fa.weight = weight; fa.labels = labels; fa.m = (int)m; fa.h = (int)h;
  fa.softcap = softcap; fa.logit_scale = multiplier;
  fa.run_max = run_max; fa.run_sum = run_sum;
  fa.lse = lse; fa.losses = losses; fa.probabilities = probabilities;
  {
    ScopedTimer timer(kClassCombine, stream);
    lce_topk_finish_kernel<T><<<(int)ceil_div(m, 4), 256, 0, stream>>>(fa);
  }
  TLCE_LAUNCH_CHECK();
  return 0;
}

template <class E>
int topk_backward_impl(const TopkPlan& t, const void* hidden, const void* weight,
                       const int64_t* labels, const float* lse, const int64_t* top_ids,
                       const float* ce_scale, const float* grad_top_values, int64_t m, int64_t h,
                       int64_t v, int dtype, int top_k, float multiplier, float softcap,
                       void* grad_hidden, char* ws, hipStream_t stream) {
  using T = typename E::T;
  const Plan& p = t.plan;
  char* bws = ws + t.backward;
  const BackwardLayout bl = backward_layout(p, m, h, dtype, false);
  float* scale = reinterpret_cast<float*>(bws + bl.scale);
  // scale[r] = ce_scale[r] * multiplier: d loss / d raw logit carries the multiplier
  ScaleArgs sa;
  sa.labels = nullptr; sa.row_idx = nullptr; sa.grad_output = ce_scale; sa.valid_count = nullptr;
  sa.m = (int)m; sa.mp = (int)p.mp; sa.reduction = TLCE_REDUCTION_NONE; sa.ignore = 0;
  sa.scale = scale; sa.constant = 0.0f; sa.multiplier = multiplier;
  if (int rc = launch_token_scale(sa, stream)) return rc;
  auto produce = [&](int64_t v0, int64_t width, void* g, void* gt) -> int {
    GradLogitsArgs ga;
    ga.hidden = hidden; ga.weight = weight; ga.bias = nullptr; ga.labels = nullptr;
    ga.lse = lse; ga.scale = scale;
    ga.m = (int)m; ga.h = (int)h; ga.v = (int)v;
    ga.ignore = 0; ga.exclude = -1; ga.softcap = softcap;
    ga.label_offset = 0; ga.probabilities = 1; ga.cap_grad = 1; ga.logit_scale = multiplier;
    ga.v0 = (int)v0;
    ga.n_ttiles = p.n_ttiles; ga.n_ptiles = (int)(width / p.tile);
    ga.g = g; ga.ldg = p.vc; ga.gt = gt; ga.ldgt = p.mp;
    ga.grad_bias = nullptr;
    return launch_grad_logits<E>(ga, stream);
  };
  auto single_rows = [&](float* acc32) -> int {
    // with a K split the label / top-k terms go to the first slab only
    TopkAdjustArgs aa;
    aa.hidden = hidden; aa.weight = weight; aa.labels = labels; aa.top_ids = top_ids;
    aa.ce_scale = ce_scale; aa.grad_top_values = grad_top_values;
    aa.m = (int)m; aa.h = (int)h; aa.k = top_k;
    aa.softcap = softcap; aa.logit_scale = multiplier; aa.acc32 = acc32;
    ScopedTimer timer(kClassOther, stream);
    lce_topk_adjust_kernel<T><<<(int)m, 256, 0, stream>>>(aa);
    TLCE_LAUNCH_CHECK();
    return 0;
  };
  return panel_contractions<E>(p, bl, hidden, weight, nullptr, m, m, h, v, dtype, grad_hidden,
                               nullptr, bws, stream, produce, single_rows);
}



struct SoftEmbeddingLayout {
  int64_t forward_ws, lse, backward_ws, total;
};

inline SoftEmbeddingLayout soft_embedding_layout(const Plan& fp, const Plan& bp, int64_t m, int64_t h,
                                          int dtype) {
  SoftEmbeddingLayout l;
  l.forward_ws = 0;
  l.lse = round_up(forward_layout(fp).total, 256);
  l.backward_ws = l.lse + round_up(m * 4, 256);
  l.total = l.backward_ws + backward_layout(bp, m, h, dtype, false).total;
  return l;
}

template <class E>
int soft_embedding_impl(const Plan& fp, const Plan& bp, const SoftEmbeddingLayout& l,
                        const void* hidden, const void* weight, int64_t m, int64_t h, int64_t v,
                        int dtype, float softcap, float scale, void* out, char* ws,
                        hipStream_t stream) {
  float* lse = reinterpret_cast<float*>(ws + l.lse);
  if (int rc = forward_impl<E>(fp, hidden, weight, nullptr, nullptr, nullptr, m, h, v, 0, -1,
                               softcap, nullptr, lse, nullptr, ShardStats{}, ws + l.forward_ws,
                               stream, RowOptions{}))
    return rc;
  return backward_impl<E>(bp, hidden, weight, nullptr, nullptr, nullptr, lse, nullptr, nullptr, m,
                          m, h, v, dtype, TLCE_REDUCTION_SUM, 0, -1, softcap, 0, out, nullptr,
                          nullptr, ws + l.backward_ws, stream, scale, RowOptions{});
}


// The kernel launchers of one engine, by kernel family.  An engine whose
// kernels compile slowly is built as several translation units, one family
// each; X is `template` in the unit that owns the family and `extern template`
// in the others.
#define TLCE_LAUNCHERS_FORWARD(X, E) \
  X int launch_forward<E>(const Plan&, const ForwardArgs&, hipStream_t);
#define TLCE_LAUNCHERS_GRAD_LOGITS(X, E, kSoftcap, kBias) \
  X int launch_grad_logits_variant<E, kSoftcap, kBias>(const GradLogitsArgs&, hipStream_t);
#define TLCE_LAUNCHERS_FORWARD_DIM_FIRST(X, E) \
  X int launch_forward_dim_first<E>(const Plan&, const ForwardArgs&, hipStream_t);
#define TLCE_LAUNCHERS_GRAD_LOGITS_DIM_FIRST(X, E) \
  X int launch_grad_logits_dim_first<E>(const GradLogitsArgs&, hipStream_t);
#define TLCE_LAUNCHERS_GEMM(X, E)                                         \
  X int launch_gemm<E, false, false>(GemmArgs, int, int, hipStream_t);    \
  X int launch_gemm<E, true, false>(GemmArgs, int, int, hipStream_t);     \
  X int launch_gemm<E, true, true>(GemmArgs, int, int, hipStream_t);
#define TLCE_LAUNCHERS_KL(X, E) \
  X int launch_kl_panel<E>(const KlPanelArgs&, hipStream_t);
#define TLCE_LAUNCHERS_LOGITS(X, E)                                                     \
  X int launch_logits_panel_variant<E, true>(const LogitsPanelArgs&, hipStream_t);      \
  X int launch_logits_panel_variant<E, false>(const LogitsPanelArgs&, hipStream_t);

// The per-engine launch sequences the C ABI dispatches to.  X is `extern
// template` where they are used and `template` in the translation unit that
// instantiates engine E.
#define TLCE_ENGINE_ENTRY_POINTS(X, E)                                                          \
  X int forward_impl<E>(const Plan&, const void*, const void*, const float*, const int64_t*,    \
                        const int64_t*, int64_t, int64_t, int64_t, int64_t, int64_t, float,     \
                        float*, float*, float*, const ShardStats&, char*, hipStream_t,          \
                        const RowOptions&);                                                     \
  X int backward_impl<E>(const Plan&, const void*, const void*, const float*, const int64_t*,   \
                         const int64_t*, const float*, const float*, const float*, int64_t,     \
                         int64_t, int64_t, int64_t, int, int, int64_t, int64_t, float, int64_t, \
                         void*, void*, float*, char*, hipStream_t, float, const RowOptions&);   \
  X int soft_embedding_impl<E>(const Plan&, const Plan&, const SoftEmbeddingLayout&,            \
                               const void*, const void*, int64_t, int64_t, int64_t, int, float, \
                               float, void*, char*, hipStream_t);                               \
  X int kl_forward_impl<E>(const Plan&, const Plan&, const KlLayout&, const void*, const void*, \
                           const void*, const void*, int64_t, int64_t, int64_t, int64_t, int,   \
                           float, float*, float*, float*, char*, hipStream_t, void*);           \
  X int kl_backward_impl<E>(const Plan&, const KlLayout&, const void*, const void*,             \
                            const void*, const void*, const float*, const float*, const float*, \
                            int64_t, int64_t, int64_t, int64_t, int, float, void*, char*,       \
                            hipStream_t, const void*);                                          \
  X int topk_forward_impl<E>(const TopkPlan&, const void*, const void*, const int64_t*,         \
                             int64_t, int64_t, int64_t, int, float, float, float*, float*,      \
                             float*, int64_t*, float*, char*, hipStream_t,                      \
                             const TopkExpHook*);                                               \
  X int topk_backward_impl<E>(const TopkPlan&, const void*, const void*, const int64_t*,        \
                              const float*, const int64_t*, const float*, const float*,         \
                              int64_t, int64_t, int64_t, int, int, float, float, void*, char*,  \
                              hipStream_t);

}  // namespace tlce
