// Host scheduler and C ABI of the fused linear cross-entropy for gfx950.
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

char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return 1;
}

namespace {

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
  kNumClasses = 7
};

struct Profiler {
  struct Record { int cls; hipEvent_t start, stop; };
  std::vector<Record> records;
};
thread_local Profiler* g_profiler = nullptr;

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
constexpr int kTargetWorkgroups = 1024;  // 4 per CU on a 256-CU MI355X

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
};

int engine_class(int64_t h, int dtype) {
  if (dtype == TLCE_DTYPE_F32 || (h % 8) != 0) return 0;
  return (h % 64) == 0 ? 2 : 1;
}

Plan make_plan(int64_t m, int64_t h, int64_t v, int dtype, bool weight_grad,
               int64_t panel_bytes, int max_engine = 2) {
  Plan p;
  // 2: four-wave direct-to-LDS MFMA (h % 64 == 0), 1: register-staged MFMA
  // (h % 8 == 0), 0: generic float32-FMA tiles
  p.engine = std::min(engine_class(h, dtype), max_engine);
  if (const char* forced = getenv("TLCE_FORCE_ENGINE")) {
    const int e = atoi(forced);           // debugging aid: only to a less demanding engine
    if (e >= 0 && e < p.engine) p.engine = e;
  }
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
  p.nsplit = (int)std::min<int64_t>(
      p.n_vtiles, std::max<int64_t>(1, kTargetWorkgroups / p.n_ttiles));
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
  // own float32 slab, summed by the final cast) by the smallest factor that
  // fills at least 90 % of the last wave.
  p.dh_ksplit = 1;
  if (p.engine) {
    const int64_t tiles = (int64_t)p.n_ttiles * p.n_htiles;
    const int64_t max_split = std::max<int64_t>(1, std::min<int64_t>(16, p.vc / p.bk / 8));
    for (int64_t ks = 1; ks <= max_split; ++ks) {
      const double waves = (double)(tiles * ks) / 256.0;
      const double fill = waves / (double)ceil_div(tiles * ks, 256);
      p.dh_ksplit = (int)ks;
      if (fill >= 0.9 && (waves >= 2.0 || ks == max_split)) break;
    }
  }
  return p;
}

struct ForwardLayout {
  int64_t part_max, part_sum, total;
};
ForwardLayout forward_layout(const Plan& p) {
  ForwardLayout l;
  const int64_t part = align256((int64_t)p.nsplit * p.mp * 4);
  l.part_max = 0;
  l.part_sum = part;
  l.total = 2 * part;
  return l;
}

struct BackwardLayout {
  int64_t scale, acc32, wt, ht, g, gt, total;
};
// wt / gt exist only on the transposed-copy path; ht is hidden^T there and, on
// the K-major path, a copy of hidden padded to a multiple of 64 rows (only when
// m is not one already).
BackwardLayout backward_layout(const Plan& p, int64_t m, int64_t h, int dtype, bool weight_grad) {
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

int validate_common(const void* hidden, const void* weight, int64_t m, int64_t h, int64_t v,
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
template <class E, bool kSoftcap, bool kBias>
int launch_forward_variant(const Plan& p, const ForwardArgs& a, hipStream_t stream) {
  static LdsOptIn lds;
  if (int rc = enable_large_lds(lce_forward_stats_kernel<E, kSoftcap, kBias>, E::kSmemBytes, lds))
    return rc;
  const int grid = xcd_grid((int64_t)p.n_ttiles * p.nsplit);
  ScopedTimer timer(kClassForwardStats, stream);
  lce_forward_stats_kernel<E, kSoftcap, kBias><<<grid, E::kThreads, E::kSmemBytes, stream>>>(a);
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

template <class E, bool kSoftcap, bool kBias>
int launch_grad_logits_variant(const GradLogitsArgs& a, hipStream_t stream) {
  static LdsOptIn lds;
  if (int rc = enable_large_lds(lce_grad_logits_panel_kernel<E, kSoftcap, kBias>, E::kSmemBytes,
                                lds))
    return rc;
  const int grid = xcd_grid((int64_t)a.n_ttiles * a.n_ptiles);
  ScopedTimer timer(kClassGradLogits, stream);
  lce_grad_logits_panel_kernel<E, kSoftcap, kBias>
      <<<grid, E::kThreads, E::kSmemBytes, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
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
  dim3 grid(xcd_grid((int64_t)a.ni * a.nj), ksplit, 1);
  ScopedTimer timer(cls, stream);
  lce_gemm_nt_kernel<E, kAKMajor, kBKMajor><<<grid, E::kThreads, E::kSmemBytes, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

template <typename T>
int launch_transpose(const T* in, int64_t ld_in, int64_t rows, int64_t cols, T* out,
                     int64_t ld_out, int64_t out_cols, hipStream_t stream) {
  dim3 grid((unsigned)ceil_div(cols, 64), (unsigned)ceil_div(out_cols, 64), 1);
  TLCE_REQUIRE(grid.y <= 65535, "transpose: too many row tiles");
  ScopedTimer timer(kClassTranspose, stream);
  lce_transpose_pad_kernel<T><<<grid, 256, 0, stream>>>(in, ld_in, (int)rows, (int)cols, out,
                                                        ld_out, (int)out_cols);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int fill_zero(void* dst, int64_t bytes, hipStream_t stream) {
  if (bytes <= 0) return 0;
  TLCE_REQUIRE(((uintptr_t)dst & 15) == 0 || bytes < 16, "fill_zero: dst must be 16-byte aligned");
  const int64_t n16 = (((uintptr_t)dst & 15) == 0) ? bytes / 16 : 0;
  const int ntail = (int)(bytes - n16 * 16);
  const int grid = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(n16, 256), 256 * 16));
  ScopedTimer timer(kClassOther, stream);
  lce_fill_zero_kernel<<<grid, 256, 0, stream>>>(static_cast<uint4*>(dst), n16,
                                                 static_cast<unsigned char*>(dst) + n16 * 16, ntail);
  TLCE_LAUNCH_CHECK();
  return 0;
}

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
                 float* valid_count, const ShardStats& shard, char* ws, hipStream_t stream) {
  using T = typename E::T;
  const ForwardLayout l = forward_layout(p);
  ForwardArgs fa;
  fa.hidden = hidden; fa.weight = weight; fa.bias = bias;
  fa.m = (int)m; fa.h = (int)h; fa.v = (int)v;
  fa.exclude = exclude - shard.vocab_start; fa.softcap = softcap;
  fa.n_ttiles = p.n_ttiles; fa.n_vtiles = p.n_vtiles; fa.nsplit = p.nsplit;
  fa.part_max = reinterpret_cast<float*>(ws + l.part_max);
  fa.part_sum = reinterpret_cast<float*>(ws + l.part_sum);
  fa.part_ld = (int)p.mp;
  if (int rc = launch_forward<E>(p, fa, stream)) return rc;

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
  {
    ScopedTimer timer(kClassCombine, stream);
    lce_combine_loss_kernel<T><<<(int)ceil_div(m, kCombineRowsPerBlock), 256, 0, stream>>>(ca);
  }
  TLCE_LAUNCH_CHECK();
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
                       const std::function<int(float*)>& before_cast = nullptr) {
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
      if (int rc = launch_transpose<T>(hidden_t, h, m, h, ht, p.mp, p.mp, stream)) return rc;
    }
  } else if (weight_grad && m64 != m) {
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
    GemmArgs dw;
    dw.k_per_split = 0;
    dw.ni = p.n_htiles; dw.nj = (int)(width / p.tile);
    dw.c = weight_grad ? static_cast<T*>(grad_weight) + v0 * h : nullptr; dw.ldc = h;
    dw.c_rows = (int)rows_valid; dw.c_cols = (int)h;
    dw.c_split_stride = 0;
    dw.mode = kStoreT;
    if constexpr (E::kHasKMajor) {
      if (p.kmajor) {
        // grad_hidden: A = weight rows [v0, v0+K) as stored (K-major), B = G
        dh.a = weight_t + v0 * h; dh.lda = h; dh.a_rows = (int)h;
        dh.k = (int)round_up(rows_valid, 64);
        if (int rc = launch_gemm<E, true, false>(dh, p.dh_ksplit, kClassGradHidden, stream))
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
    if (int rc = launch_gemm<E, false, false>(dh, p.dh_ksplit, kClassGradHidden, stream))
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
  if (row_idx != nullptr) {
    if (int rc = fill_zero(grad_hidden, n_out * h * dtype_bytes(dtype), stream)) return rc;
  }
  {
    ScopedTimer timer(kClassOther, stream);
    lce_finalize_grad_hidden_kernel<T><<<(int)m, 256, 0, stream>>>(
        acc32, p.dh_ksplit, p.mp * h, row_idx, (int)m, (int)h, static_cast<T*>(grad_hidden));
  }
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_token_scale(const ScaleArgs& sa, hipStream_t stream) {
  ScopedTimer timer(kClassOther, stream);
  lce_token_scale_kernel<<<(int)ceil_div(sa.mp, 256), 256, 0, stream>>>(sa);
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
                  float probabilities_scale = 0.0f) {
  const BackwardLayout l = backward_layout(p, m, h, dtype, grad_weight != nullptr);
  float* scale = reinterpret_cast<float*>(ws + l.scale);
  ScaleArgs sa;
  sa.labels = labels; sa.row_idx = row_idx; sa.grad_output = grad_output;
  sa.valid_count = valid_count; sa.m = (int)m; sa.mp = (int)p.mp; sa.reduction = reduction;
  sa.ignore = ignore; sa.scale = scale; sa.constant = probabilities_scale; sa.multiplier = 1.0f;
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
    ga.logit_scale = 1.0f;
    ga.v0 = (int)v0;
    ga.n_ttiles = p.n_ttiles; ga.n_ptiles = (int)(width / p.tile);
    ga.g = g; ga.ldg = p.vc; ga.gt = gt; ga.ldgt = p.mp;
    ga.grad_bias = (bias != nullptr) ? grad_bias : nullptr;
    return launch_grad_logits<E>(ga, stream);
  };
  return panel_contractions<E>(p, l, hidden, weight, row_idx, m, n_out, h, v, dtype, grad_hidden,
                               grad_weight, ws, stream, produce);
}

// -------------------------------------------------------------- frozen KL ----
// KL(teacher || draft) of two frozen heads over one vocabulary
// (fused_dflash_kl_forward_cuda / _backward_cuda, fused_linear_ce_cuda.cu:1270-1509).
// Both heads run on one engine class (the less demanding of the two hidden sizes).
struct KlLayout {
  // stats: the teacher's forward partials, then the draft's per-tile partials
  // (part_max, part_sum: n_vtiles x mp float32 each); backward: BackwardLayout
  // of the draft head
  int64_t stats, tile_part, ones, tsum, backward, total;
};

KlLayout kl_layout(const Plan& pd, const Plan& pt, int64_t m, int64_t hd, int dtype) {
  KlLayout l;
  l.stats = 0;
  l.tile_part = align256((int64_t)pd.n_vtiles * pd.mp * 4);
  int64_t off = std::max(2 * l.tile_part, forward_layout(pt).total);
  l.ones = off;      off += align256(pd.mp * 4);
  l.tsum = off;      off += align256(pd.mp * 4);
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
             void* g, float* losses, float* tsum, float* part_max, float* part_sum, int mode,
             hipStream_t stream) {
  GradLogitsArgs ga;
  ga.hidden = teacher_hidden; ga.weight = teacher_weight; ga.bias = nullptr;
  ga.labels = nullptr; ga.lse = teacher_lse; ga.scale = ones;
  ga.m = (int)m; ga.h = (int)ht; ga.v = (int)v;
  ga.ignore = 0; ga.exclude = -1; ga.softcap = softcap;
  ga.label_offset = 0; ga.probabilities = 1; ga.cap_grad = 0; ga.logit_scale = 1.0f;
  ga.v0 = (int)v0;
  ga.n_ttiles = pd.n_ttiles; ga.n_ptiles = (int)(width / pd.tile);
  ga.g = g; ga.ldg = pd.vc; ga.gt = nullptr; ga.ldgt = 0;
  ga.grad_bias = nullptr;
  if (int rc = launch_grad_logits<E>(ga, stream)) return rc;
  KlPanelArgs ka;
  ka.hidden = draft_hidden; ka.weight = draft_weight; ka.lse = draft_lse; ka.scale = scale;
  ka.m = (int)m; ka.h = (int)hd; ka.v = (int)v; ka.softcap = softcap;
  ka.v0 = (int)v0; ka.n_ttiles = pd.n_ttiles; ka.n_ptiles = (int)(width / pd.tile);
  ka.panel = g; ka.ld = pd.vc; ka.losses = losses; ka.tsum = tsum;
  ka.part_max = part_max; ka.part_sum = part_sum; ka.part_ld = (int)pd.mp; ka.mode = mode;
  return launch_kl_panel<E>(ka, stream);
}

template <class E>
int kl_forward_impl(const Plan& pd, const Plan& pt, const KlLayout& l, const void* draft_hidden,
                    const void* draft_weight, const void* teacher_hidden,
                    const void* teacher_weight, int64_t m, int64_t hd, int64_t ht, int64_t v,
                    int dtype, float softcap, float* losses, float* draft_lse, float* teacher_lse,
                    char* ws, hipStream_t stream) {
  using T = typename E::T;
  // teacher statistics first: its probabilities need the teacher lse
  if (int rc = forward_impl<E>(pt, teacher_hidden, teacher_weight, nullptr, nullptr, nullptr, m,
                               ht, v, 0, -1, softcap, nullptr, teacher_lse, nullptr, ShardStats{},
                               ws + l.stats, stream))
    return rc;
  float* ones = reinterpret_cast<float*>(ws + l.ones);
  float* tsum = reinterpret_cast<float*>(ws + l.tsum);
  float* part_max = reinterpret_cast<float*>(ws + l.stats);
  float* part_sum = reinterpret_cast<float*>(ws + l.stats + l.tile_part);
  ScaleArgs sa;
  sa.labels = nullptr; sa.row_idx = nullptr; sa.grad_output = nullptr; sa.valid_count = nullptr;
  sa.m = (int)m; sa.mp = (int)pd.mp; sa.reduction = TLCE_REDUCTION_SUM; sa.ignore = 0;
  sa.scale = ones; sa.constant = 1.0f; sa.multiplier = 1.0f;
  if (int rc = launch_token_scale(sa, stream)) return rc;
  if (int rc = fill_zero(tsum, pd.mp * 4, stream)) return rc;
  if (int rc = fill_zero(losses, m * 4, stream)) return rc;
  // one pass over the draft head per panel: loss terms and the draft's per-tile
  // softmax partials (the teacher partials above are dead by now)
  const BackwardLayout bl = backward_layout(pd, m, hd, dtype, false);
  void* g = ws + l.backward + bl.g;
  for (int panel = 0; panel < pd.n_panels; ++panel) {
    const int64_t v0 = (int64_t)panel * pd.vc;
    const int64_t width = std::min<int64_t>(pd.vc, pd.vp - v0);
    if (int rc = kl_panel<E>(pd, draft_hidden, draft_weight, teacher_hidden, teacher_weight,
                             nullptr, teacher_lse, ones, nullptr, m, hd, ht, v, softcap, v0,
                             width, g, losses, tsum, part_max, part_sum, kKlLoss, stream))
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
    lce_kl_finish_kernel<<<(int)ceil_div(m, 256), 256, 0, stream>>>(losses, tsum, draft_lse,
                                                                    (int)m);
  }
  TLCE_LAUNCH_CHECK();
  return 0;
}

template <class E>
int kl_backward_impl(const Plan& pd, const KlLayout& l, const void* draft_hidden,
                     const void* draft_weight, const void* teacher_hidden,
                     const void* teacher_weight, const float* draft_lse, const float* teacher_lse,
                     const float* grad_output, int64_t m, int64_t hd, int64_t ht, int64_t v,
                     int dtype, float softcap, void* grad_hidden, char* ws, hipStream_t stream) {
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
                       nullptr, nullptr, nullptr, kKlGrad, stream);
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

TopkPlan topk_plan(int64_t m, int64_t h, int64_t v, int dtype, int64_t panel_bytes) {
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

template <class E>
int topk_forward_impl(const TopkPlan& t, const void* hidden, const void* weight,
                      const int64_t* labels, int64_t m, int64_t h, int64_t v, int top_k,
                      float multiplier, float softcap, float* losses, float* probabilities,
                      float* top_values, int64_t* top_ids, float* lse, char* ws,
                      hipStream_t stream) {
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
    {
      ScopedTimer timer(kClassOther, stream);
      lce_topk_scan_kernel<<<(int)m, 256, 0, stream>>>(sa);
    }
    TLCE_LAUNCH_CHECK();
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

}  // namespace
}  // namespace tlce

using namespace tlce;

#define TLCE_DISPATCH(plan, dtype, CALL)                                                   \
  do {                                                                                     \
    if ((plan).engine == 2) {                                                              \
      if ((dtype) == TLCE_DTYPE_BF16) { using E = MfmaDirect4Engine<__bf16>; return CALL; } \
      { using E = MfmaDirect4Engine<_Float16>; return CALL; }                              \
    }                                                                                      \
    if ((plan).engine == 1) {                                                              \
      if ((dtype) == TLCE_DTYPE_BF16) { using E = MfmaEngine<__bf16>; return CALL; }       \
      { using E = MfmaEngine<_Float16>; return CALL; }                                     \
    }                                                                                      \
    if ((dtype) == TLCE_DTYPE_F32) { using E = SimtEngine<float>; return CALL; }           \
    if ((dtype) == TLCE_DTYPE_BF16) { using E = SimtEngine<__bf16>; return CALL; }         \
    { using E = SimtEngine<_Float16>; return CALL; }                                       \
  } while (0)

extern "C" int tlce_version(void) { return TLCE_VERSION; }

extern "C" const char* tlce_last_error(void) { return error_buffer(); }

extern "C" int tlce_check_device(int device) {
  hipDeviceProp_t prop;
  TLCE_HIP(hipGetDeviceProperties(&prop, device));
  TLCE_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0,
               "device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
  return 0;
}

extern "C" int tlce_fill_zero(void* dst, int64_t bytes, void* stream) {
  TLCE_REQUIRE(bytes >= 0 && (dst != nullptr || bytes == 0), "fill_zero: bad arguments");
  return fill_zero(dst, bytes, static_cast<hipStream_t>(stream));
}

extern "C" int tlce_query_plan(int64_t m, int64_t h, int64_t v, int dtype, int compute_weight_grad,
                               int64_t panel_bytes, int* engine, int64_t* tile,
                               int64_t* forward_vocab_splits, int64_t* panel_columns,
                               int64_t* n_panels, int64_t* grad_hidden_k_splits) {
  TLCE_REQUIRE(m >= 0 && h > 0 && v > 0, "query_plan: bad shape");
  const Plan p = make_plan(m, h, v, dtype, compute_weight_grad != 0, panel_bytes);
  if (engine) *engine = p.engine;
  if (tile) *tile = p.tile;
  if (forward_vocab_splits) *forward_vocab_splits = p.nsplit;
  if (panel_columns) *panel_columns = p.vc;
  if (n_panels) *n_panels = p.n_panels;
  if (grad_hidden_k_splits) *grad_hidden_k_splits = p.dh_ksplit;
  return 0;
}

extern "C" int64_t tlce_forward_workspace_bytes(int64_t m, int64_t h, int64_t v, int dtype) {
  if (m < 0 || h <= 0 || v <= 0) return -1;
  return forward_layout(make_plan(m, h, v, dtype, false, 0)).total;
}

namespace {

int forward_entry(const void* hidden, const void* weight, const float* bias,
                  const int64_t* labels, const int64_t* row_idx, int64_t m, int64_t n_out,
                  int64_t h, int64_t v, int dtype, int64_t ignore_index, int64_t exclude_index,
                  float logit_softcap, float* losses, float* lse, float* valid_count,
                  const ShardStats& shard, void* workspace, int64_t workspace_bytes,
                  hipStream_t stream) {
  const bool local = shard.local_max != nullptr;
  if (int rc = validate_common(hidden, weight, m, h, v, dtype)) return rc;
  TLCE_REQUIRE(valid_count != nullptr, "forward: valid_count is null");
  TLCE_REQUIRE(n_out >= m, "forward: n_out=%lld < m=%lld", (long long)n_out, (long long)m);
  TLCE_REQUIRE(row_idx != nullptr || n_out == m || m == 0,
               "forward: n_out != m without row_idx");
  if (int rc = fill_zero(valid_count, 4, stream)) return rc;
  if (!local && (row_idx != nullptr || m == 0)) {
    TLCE_REQUIRE(losses != nullptr || n_out == 0, "forward: losses is null");
    if (int rc = fill_zero(losses, n_out * 4, stream)) return rc;
  }
  if (m == 0) return 0;
  TLCE_REQUIRE(labels && workspace && (local || (losses && lse)), "forward: null pointer");
  const Plan p = make_plan(m, h, v, dtype, false, 0);
  TLCE_REQUIRE(workspace_bytes >= forward_layout(p).total,
               "forward: workspace too small (%lld < %lld)", (long long)workspace_bytes,
               (long long)forward_layout(p).total);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0, "forward: workspace must be 256-byte aligned");
  TLCE_DISPATCH(p, dtype,
                forward_impl<E>(p, hidden, weight, bias, labels, row_idx, m, h, v, ignore_index,
                                exclude_index, logit_softcap, losses, lse, valid_count, shard,
                                static_cast<char*>(workspace), stream));
}

}  // namespace

extern "C" int tlce_forward(const void* hidden, const void* weight, const float* bias,
                            const int64_t* labels, const int64_t* row_idx, int64_t m,
                            int64_t n_out, int64_t h, int64_t v, int dtype, int64_t ignore_index,
                            int64_t exclude_index, float logit_softcap, float* losses, float* lse,
                            float* valid_count, void* workspace, int64_t workspace_bytes,
                            void* stream) {
  return forward_entry(hidden, weight, bias, labels, row_idx, m, n_out, h, v, dtype, ignore_index,
                       exclude_index, logit_softcap, losses, lse, valid_count, ShardStats{},
                       workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int tlce_forward_local(const void* hidden, const void* weight, const float* bias,
                                  const int64_t* labels, int64_t m, int64_t h, int64_t v_local,
                                  int dtype, int64_t vocab_start, int64_t ignore_index,
                                  int64_t exclude_index, float logit_softcap, float* local_max,
                                  float* local_sum, float* target_logits, float* valid_count,
                                  void* workspace, int64_t workspace_bytes, void* stream) {
  TLCE_REQUIRE(m == 0 || (local_max && local_sum && target_logits),
               "forward_local: null output pointer");
  if (m == 0) {
    TLCE_REQUIRE(valid_count != nullptr, "forward_local: valid_count is null");
    return fill_zero(valid_count, 4, static_cast<hipStream_t>(stream));
  }
  ShardStats shard;
  shard.vocab_start = vocab_start;
  shard.local_max = local_max;
  shard.local_sum = local_sum;
  shard.target_logits = target_logits;
  return forward_entry(hidden, weight, bias, labels, nullptr, m, m, h, v_local, dtype,
                       ignore_index, exclude_index, logit_softcap, nullptr, nullptr, valid_count,
                       shard, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int64_t tlce_backward_workspace_bytes(int64_t m, int64_t h, int64_t v, int dtype,
                                                 int compute_weight_grad, int has_bias,
                                                 int64_t panel_bytes) {
  (void)has_bias;
  if (m < 0 || h <= 0 || v <= 0) return -1;
  const Plan p = make_plan(m, h, v, dtype, compute_weight_grad != 0, panel_bytes);
  return backward_layout(p, m, h, dtype, compute_weight_grad != 0).total;
}

namespace {

int backward_entry(const void* hidden, const void* weight, const float* bias,
                   const int64_t* labels, const int64_t* row_idx, const float* lse,
                   const float* valid_count, const float* grad_output, int64_t m, int64_t n_out,
                   int64_t h, int64_t v, int dtype, int reduction_code, int64_t vocab_start,
                   int64_t ignore_index, int64_t exclude_index, float logit_softcap,
                   void* grad_hidden, void* grad_weight, float* grad_bias, int64_t panel_bytes,
                   void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  if (int rc = validate_common(hidden, weight, m, h, v, dtype)) return rc;
  TLCE_REQUIRE(reduction_code >= TLCE_REDUCTION_NONE && reduction_code <= TLCE_REDUCTION_MEAN,
               "backward: bad reduction code %d", reduction_code);
  TLCE_REQUIRE(n_out >= m, "backward: n_out=%lld < m=%lld", (long long)n_out, (long long)m);
  TLCE_REQUIRE(row_idx != nullptr || n_out == m || m == 0,
               "backward: n_out != m without row_idx");
  TLCE_REQUIRE(grad_hidden != nullptr || n_out == 0, "backward: grad_hidden is null");
  TLCE_REQUIRE((bias == nullptr) || (grad_bias != nullptr), "backward: bias without grad_bias");
  const int64_t es = dtype_bytes(dtype);
  if (m == 0) {
    if (int rc = fill_zero(grad_hidden, n_out * h * es, stream)) return rc;
    if (grad_weight != nullptr) {
      if (int rc = fill_zero(grad_weight, v * h * es, stream)) return rc;
    }
    if (bias != nullptr) return fill_zero(grad_bias, v * 4, stream);
    return 0;
  }
  TLCE_REQUIRE(labels && lse && valid_count && grad_output && workspace, "backward: null pointer");
  TLCE_REQUIRE(((uintptr_t)grad_hidden & 15) == 0 && ((uintptr_t)grad_weight & 15) == 0,
               "backward: gradients must be 16-byte aligned");
  const Plan p = make_plan(m, h, v, dtype, grad_weight != nullptr, panel_bytes);
  const int64_t need = backward_layout(p, m, h, dtype, grad_weight != nullptr).total;
  TLCE_REQUIRE(workspace_bytes >= need, "backward: workspace too small (%lld < %lld)",
               (long long)workspace_bytes, (long long)need);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0, "backward: workspace must be 256-byte aligned");
  TLCE_DISPATCH(p, dtype,
                backward_impl<E>(p, hidden, weight, bias, labels, row_idx, lse, valid_count,
                                 grad_output, m, n_out, h, v, dtype, reduction_code, ignore_index,
                                 exclude_index, logit_softcap, vocab_start, grad_hidden,
                                 grad_weight, (bias != nullptr) ? grad_bias : nullptr,
                                 static_cast<char*>(workspace), stream));
}

}  // namespace

extern "C" int tlce_backward(const void* hidden, const void* weight, const float* bias,
                             const int64_t* labels, const int64_t* row_idx, const float* lse,
                             const float* valid_count, const float* grad_output, int64_t m,
                             int64_t n_out, int64_t h, int64_t v, int dtype, int reduction_code,
                             int64_t ignore_index, int64_t exclude_index, float logit_softcap,
                             void* grad_hidden, void* grad_weight, float* grad_bias,
                             int64_t panel_bytes, void* workspace, int64_t workspace_bytes,
                             void* stream) {
  return backward_entry(hidden, weight, bias, labels, row_idx, lse, valid_count, grad_output, m,
                        n_out, h, v, dtype, reduction_code, 0, ignore_index, exclude_index,
                        logit_softcap, grad_hidden, grad_weight, grad_bias, panel_bytes, workspace,
                        workspace_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int tlce_backward_local(const void* hidden, const void* weight, const float* bias,
                                   const int64_t* labels, const float* global_lse,
                                   const float* valid_count, const float* grad_output, int64_t m,
                                   int64_t h, int64_t v_local, int dtype, int reduction_code,
                                   int64_t vocab_start, int64_t ignore_index,
                                   int64_t exclude_index, float logit_softcap, void* grad_hidden,
                                   void* grad_weight, float* grad_bias, int64_t panel_bytes,
                                   void* workspace, int64_t workspace_bytes, void* stream) {
  return backward_entry(hidden, weight, bias, labels, nullptr, global_lse, valid_count,
                        grad_output, m, m, h, v_local, dtype, reduction_code, vocab_start,
                        ignore_index, exclude_index, logit_softcap, grad_hidden, grad_weight,
                        grad_bias, panel_bytes, workspace, workspace_bytes,
                        static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------- soft embedding --
namespace {

struct SoftEmbeddingLayout {
  int64_t forward_ws, lse, backward_ws, total;
};

SoftEmbeddingLayout soft_embedding_layout(const Plan& fp, const Plan& bp, int64_t m, int64_t h,
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
                               stream))
    return rc;
  return backward_impl<E>(bp, hidden, weight, nullptr, nullptr, nullptr, lse, nullptr, nullptr, m,
                          m, h, v, dtype, TLCE_REDUCTION_SUM, 0, -1, softcap, 0, out, nullptr,
                          nullptr, ws + l.backward_ws, stream, scale);
}

}  // namespace

extern "C" int64_t tlce_soft_embedding_workspace_bytes(int64_t m, int64_t h, int64_t v, int dtype,
                                                       int64_t panel_bytes) {
  if (m < 0 || h <= 0 || v <= 0) return -1;
  const Plan fp = make_plan(m, h, v, dtype, false, 0);
  const Plan bp = make_plan(m, h, v, dtype, false, panel_bytes);
  return soft_embedding_layout(fp, bp, m, h, dtype).total;
}

extern "C" int tlce_soft_embedding(const void* hidden, const void* weight, int64_t m, int64_t h,
                                   int64_t v, int dtype, float logit_softcap,
                                   float embedding_scale, void* out, int64_t panel_bytes,
                                   void* workspace, int64_t workspace_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = validate_common(hidden, weight, m, h, v, dtype)) return rc;
  if (m == 0) return 0;
  TLCE_REQUIRE(out != nullptr && workspace != nullptr, "soft_embedding: null pointer");
  TLCE_REQUIRE(((uintptr_t)out & 15) == 0, "soft_embedding: out must be 16-byte aligned");
  const Plan fp = make_plan(m, h, v, dtype, false, 0);
  const Plan bp = make_plan(m, h, v, dtype, false, panel_bytes);
  const SoftEmbeddingLayout l = soft_embedding_layout(fp, bp, m, h, dtype);
  TLCE_REQUIRE(workspace_bytes >= l.total, "soft_embedding: workspace too small (%lld < %lld)",
               (long long)workspace_bytes, (long long)l.total);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0,
               "soft_embedding: workspace must be 256-byte aligned");
  TLCE_DISPATCH(fp, dtype,
                soft_embedding_impl<E>(fp, bp, l, hidden, weight, m, h, v, dtype, logit_softcap,
                                       embedding_scale, out, static_cast<char*>(workspace),
                                       stream));
}

// ---------------------------------------------------------------- frozen KL --
namespace {

struct KlPlans {
  Plan draft, teacher;
  KlLayout layout;
};

KlPlans kl_plans(int64_t m, int64_t hd, int64_t ht, int64_t v, int dtype, int64_t panel_bytes) {
  KlPlans k;
  const int engine = std::min(engine_class(hd, dtype), engine_class(ht, dtype));
  k.draft = make_plan(m, hd, v, dtype, false, panel_bytes, engine);
  k.teacher = make_plan(m, ht, v, dtype, false, panel_bytes, engine);
  // one engine class for both heads (TLCE_FORCE_ENGINE may have lowered either)
  const int common = std::min(k.draft.engine, k.teacher.engine);
  if (k.draft.engine != common) k.draft = make_plan(m, hd, v, dtype, false, panel_bytes, common);
  if (k.teacher.engine != common) k.teacher = make_plan(m, ht, v, dtype, false, panel_bytes, common);
  k.layout = kl_layout(k.draft, k.teacher, m, hd, dtype);
  return k;
}

int kl_validate(const void* draft_hidden, const void* draft_weight, const void* teacher_hidden,
                const void* teacher_weight, int64_t m, int64_t hd, int64_t ht, int64_t v,
                int dtype) {
  if (int rc = validate_common(draft_hidden, draft_weight, m, hd, v, dtype)) return rc;
  return validate_common(teacher_hidden, teacher_weight, m, ht, v, dtype);
}

}  // namespace

extern "C" int64_t tlce_kl_workspace_bytes(int64_t m, int64_t h_draft, int64_t h_teacher,
                                           int64_t v, int dtype, int64_t panel_bytes) {
  if (m < 0 || h_draft <= 0 || h_teacher <= 0 || v <= 0) return -1;
  return kl_plans(m, h_draft, h_teacher, v, dtype, panel_bytes).layout.total;
}

extern "C" int tlce_kl_forward(const void* draft_hidden, const void* draft_weight,
                               const void* teacher_hidden, const void* teacher_weight, int64_t m,
                               int64_t h_draft, int64_t h_teacher, int64_t v, int dtype,
                               float logit_softcap, float* losses, float* draft_lse,
                               float* teacher_lse, int64_t panel_bytes, void* workspace,
                               int64_t workspace_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = kl_validate(draft_hidden, draft_weight, teacher_hidden, teacher_weight, m,
                           h_draft, h_teacher, v, dtype))
    return rc;
  if (m == 0) return 0;
  TLCE_REQUIRE(losses && draft_lse && teacher_lse && workspace, "kl_forward: null pointer");
  const KlPlans k = kl_plans(m, h_draft, h_teacher, v, dtype, panel_bytes);
  TLCE_REQUIRE(workspace_bytes >= k.layout.total, "kl_forward: workspace too small (%lld < %lld)",
               (long long)workspace_bytes, (long long)k.layout.total);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0, "kl_forward: workspace must be 256-byte aligned");
  TLCE_DISPATCH(k.draft, dtype,
                kl_forward_impl<E>(k.draft, k.teacher, k.layout, draft_hidden, draft_weight,
                                   teacher_hidden, teacher_weight, m, h_draft, h_teacher, v, dtype,
                                   logit_softcap, losses, draft_lse, teacher_lse,
                                   static_cast<char*>(workspace), stream));
}

extern "C" int tlce_kl_backward(const void* draft_hidden, const void* draft_weight,
                                const void* teacher_hidden, const void* teacher_weight,
                                const float* draft_lse, const float* teacher_lse,
                                const float* grad_output, int64_t m, int64_t h_draft,
                                int64_t h_teacher, int64_t v, int dtype, float logit_softcap,
                                void* grad_hidden, int64_t panel_bytes, void* workspace,
                                int64_t workspace_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = kl_validate(draft_hidden, draft_weight, teacher_hidden, teacher_weight, m,
                           h_draft, h_teacher, v, dtype))
    return rc;
  if (m == 0) return 0;
  TLCE_REQUIRE(draft_lse && teacher_lse && grad_output && grad_hidden && workspace,
               "kl_backward: null pointer");
  TLCE_REQUIRE(((uintptr_t)grad_hidden & 15) == 0, "kl_backward: grad_hidden must be 16-byte aligned");
  const KlPlans k = kl_plans(m, h_draft, h_teacher, v, dtype, panel_bytes);
  TLCE_REQUIRE(workspace_bytes >= k.layout.total, "kl_backward: workspace too small (%lld < %lld)",
               (long long)workspace_bytes, (long long)k.layout.total);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0, "kl_backward: workspace must be 256-byte aligned");
  TLCE_DISPATCH(k.draft, dtype,
                kl_backward_impl<E>(k.draft, k.layout, draft_hidden, draft_weight, teacher_hidden,
                                    teacher_weight, draft_lse, teacher_lse, grad_output, m,
                                    h_draft, h_teacher, v, dtype, logit_softcap, grad_hidden,
                                    static_cast<char*>(workspace), stream));
}

// ---------------------------------------------------- cross entropy + top-k --
namespace {

int topk_validate(const void* hidden, const void* weight, const int64_t* labels, int64_t m,
                  int64_t h, int64_t v, int dtype, int top_k) {
  if (int rc = validate_common(hidden, weight, m, h, v, dtype)) return rc;
  TLCE_REQUIRE(top_k >= 1 && top_k <= 256 && top_k <= v,
               "ce_topk: top_k=%d must be in [1, min(256, v)]", top_k);
  TLCE_REQUIRE(labels != nullptr || m == 0, "ce_topk: labels is null");
  return 0;
}

}  // namespace

extern "C" int64_t tlce_ce_topk_forward_workspace_bytes(int64_t m, int64_t h, int64_t v,
                                                        int dtype, int64_t panel_bytes) {
  if (m < 0 || h <= 0 || v <= 0) return -1;
  return topk_plan(m, h, v, dtype, panel_bytes).forward_total;
}

extern "C" int64_t tlce_ce_topk_backward_workspace_bytes(int64_t m, int64_t h, int64_t v,
                                                         int dtype, int64_t panel_bytes) {
  if (m < 0 || h <= 0 || v <= 0) return -1;
  return topk_plan(m, h, v, dtype, panel_bytes).backward_total;
}

extern "C" int tlce_ce_topk_forward(const void* hidden, const void* weight, const int64_t* labels,
                                    int64_t m, int64_t h, int64_t v, int dtype, int top_k,
                                    float output_multiplier, float logit_softcap, float* losses,
                                    float* probabilities, float* top_values, int64_t* top_ids,
                                    float* lse, int64_t panel_bytes, void* workspace,
                                    int64_t workspace_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = topk_validate(hidden, weight, labels, m, h, v, dtype, top_k)) return rc;
  if (m == 0) return 0;
  TLCE_REQUIRE(losses && probabilities && top_values && top_ids && lse && workspace,
               "ce_topk_forward: null pointer");
  const TopkPlan t = topk_plan(m, h, v, dtype, panel_bytes);
  TLCE_REQUIRE(workspace_bytes >= t.forward_total,
               "ce_topk_forward: workspace too small (%lld < %lld)", (long long)workspace_bytes,
               (long long)t.forward_total);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0,
               "ce_topk_forward: workspace must be 256-byte aligned");
  TLCE_DISPATCH(t.plan, dtype,
                topk_forward_impl<E>(t, hidden, weight, labels, m, h, v, top_k, output_multiplier,
                                     logit_softcap, losses, probabilities, top_values, top_ids,
                                     lse, static_cast<char*>(workspace), stream));
}

extern "C" int tlce_ce_topk_backward(const void* hidden, const void* weight,
                                     const int64_t* labels, const float* lse,
                                     const int64_t* top_ids, const float* ce_scale,
                                     const float* grad_top_values, int64_t m, int64_t h, int64_t v,
                                     int dtype, int top_k, float output_multiplier,
                                     float logit_softcap, void* grad_hidden, int64_t panel_bytes,
                                     void* workspace, int64_t workspace_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = topk_validate(hidden, weight, labels, m, h, v, dtype, top_k)) return rc;
  if (m == 0) return 0;
  TLCE_REQUIRE(lse && top_ids && ce_scale && grad_hidden && workspace,
               "ce_topk_backward: null pointer");
  TLCE_REQUIRE(((uintptr_t)grad_hidden & 15) == 0,
               "ce_topk_backward: grad_hidden must be 16-byte aligned");
  const TopkPlan t = topk_plan(m, h, v, dtype, panel_bytes);
  TLCE_REQUIRE(workspace_bytes >= t.backward_total,
               "ce_topk_backward: workspace too small (%lld < %lld)", (long long)workspace_bytes,
               (long long)t.backward_total);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0,
               "ce_topk_backward: workspace must be 256-byte aligned");
  TLCE_DISPATCH(t.plan, dtype,
                topk_backward_impl<E>(t, hidden, weight, labels, lse, top_ids, ce_scale,
                                      grad_top_values, m, h, v, dtype, top_k, output_multiplier,
                                      logit_softcap, grad_hidden, static_cast<char*>(workspace),
                                      stream));
}

extern "C" int tlce_profile_begin(void) {
  TLCE_REQUIRE(g_profiler == nullptr, "profile_begin: a session is already open on this thread");
  g_profiler = new Profiler();
  return 0;
}

extern "C" int tlce_profile_end(double* class_ms, int64_t* class_launches, int n_classes) {
  TLCE_REQUIRE(g_profiler != nullptr, "profile_end: no session is open on this thread");
  Profiler* prof = g_profiler;
  g_profiler = nullptr;
  for (int c = 0; c < n_classes; ++c) {
    if (class_ms) class_ms[c] = 0.0;
    if (class_launches) class_launches[c] = 0;
  }
  int rc = 0;
  for (auto& r : prof->records) {
    float ms = 0.0f;
    if (rc == 0 && hipEventSynchronize(r.stop) != hipSuccess) rc = fail("profile_end: event sync failed");
    if (rc == 0 && hipEventElapsedTime(&ms, r.start, r.stop) != hipSuccess)
      rc = fail("profile_end: elapsed time failed");
    if (rc == 0 && r.cls < n_classes) {
      if (class_ms) class_ms[r.cls] += ms;
      if (class_launches) class_launches[r.cls] += 1;
    }
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  delete prof;
  return rc;
}
