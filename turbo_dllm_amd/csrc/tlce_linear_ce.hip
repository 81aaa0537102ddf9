// C ABI of the fused linear cross-entropy for gfx950 (declarations:
// include/tlce.h).  Validates arguments, builds the tile plan and dispatches
// to the launch sequences of tlce_host.h, which are instantiated per engine in
// the tlce_engine_*.hip translation units.  Also holds the launchers of the
// kernels that do not depend on an engine (tlce_row_kernels.h).
#include "tlce_host.h"
#include "tlce_row_kernels.h"
#include "tlce_fused_rows.h"

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

thread_local Profiler* g_profiler = nullptr;

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

int launch_token_scale(const ScaleArgs& sa, hipStream_t stream) {
  ScopedTimer timer(kClassOther, stream);
  lce_token_scale_kernel<<<(int)ceil_div(sa.mp, 256), 256, 0, stream>>>(sa);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_kl_finish(float* losses, const float* loss_part, const float* tsum_part, int n_tiles,
                     int64_t part_ld, const float* lse, int64_t m, hipStream_t stream) {
  lce_kl_finish_kernel<<<(int)ceil_div(m, 64), 64 * kKlFinishWaves, 0, stream>>>(
      losses, loss_part, tsum_part, n_tiles, part_ld, lse, (int)m);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_topk_scan(const TopkScanArgs& sa, hipStream_t stream) {
  ScopedTimer timer(kClassOther, stream);
  lce_topk_scan_kernel<<<sa.m, 256, 0, stream>>>(sa);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_sum(const float* x, int64_t n, float* out, hipStream_t stream) {
  ScopedTimer timer(kClassOther, stream);
  lce_sum_kernel<<<1, 1024, 0, stream>>>(x, (int)n, out);
  TLCE_LAUNCH_CHECK();
  return 0;
}

// ---- row kernels of the forward that leaves the gradients (tlce_fused_rows.h) ----
int launch_label_logit(const LabelLogitArgs& a, hipStream_t stream) {
  ScopedTimer timer(kClassCombine, stream);
  lce_label_logit_kernel<__bf16><<<(int)ceil_div(a.m, 16), 256, 0, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_fused_rows(const FusedRowsArgs& a, hipStream_t stream) {
  ScopedTimer timer(kClassCombine, stream);
  lce_fused_rows_kernel<__bf16>
      <<<(int)ceil_div(a.m_pad, kFusedRowsPerBlock), 256, 0, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_scale_rows(const ScaleRowsArgs& a, hipStream_t stream) {
  ScopedTimer timer(kClassOther, stream);
  lce_scale_rows_kernel<__bf16><<<(int)ceil_div(a.m_pad, 16), 256, 0, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_kl_grad_from_exp(const KlGradFromExpArgs& a, int n_vtiles, hipStream_t stream) {
  ScopedTimer timer(kClassOther, stream);
  lce_kl_grad_from_exp_kernel<<<dim3((unsigned)a.mp, (unsigned)ceil_div(n_vtiles, 8)), 256, 0,
                                stream>>>(a, n_vtiles);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_exp_from_logits(const ExpFromLogitsArgs& a, hipStream_t stream) {
  ScopedTimer timer(kClassOther, stream);
  lce_exp_from_logits_kernel<<<dim3((unsigned)a.m_pad, (unsigned)ceil_div(a.width, 2048)), 256, 0,
                               stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_rescale_exp_rows(const RescaleExpArgs& a, int n_panels, hipStream_t stream) {
  if (n_panels <= 0 || a.m <= 0) return 0;
  ScopedTimer timer(kClassOther, stream);
  lce_rescale_exp_rows_kernel<<<dim3((unsigned)a.m, (unsigned)n_panels), 256, 0, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_topk_row_scale(const TopkRowScaleArgs& a, hipStream_t stream) {
  ScopedTimer timer(kClassOther, stream);
  lce_topk_row_scale_kernel<<<(int)ceil_div(a.m_pad, 256), 256, 0, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_topk_apply(const TopkApplyArgs& a, hipStream_t stream) {
  ScopedTimer timer(kClassOther, stream);
  lce_topk_apply_kernel<__bf16><<<a.m, 256, 0, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_emit_rows(const EmitRowsArgs& a, hipStream_t stream) {
  ScopedTimer timer(kClassCombine, stream);
  lce_emit_rows_kernel<<<(int)ceil_div(a.m_pad, 64), 64 * kSoftRowsWaves, 0, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_soft_rows(const SoftRowsArgs& a, hipStream_t stream) {
  ScopedTimer timer(kClassCombine, stream);
  lce_soft_rows_kernel<<<(int)ceil_div(a.m_pad, 64), 64 * kSoftRowsWaves, 0, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_reduce_slabs(const ReduceSlabsArgs& a, hipStream_t stream) {
  ScopedTimer timer(kClassOther, stream);
  lce_reduce_scaled_slabs_kernel<<<a.m, 256, 0, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

int launch_scale_cast(const ScaleCastArgs& a, hipStream_t stream) {
  if (a.rows <= 0) return 0;
  ScopedTimer timer(kClassOther, stream);
  lce_scale_cast_rows_kernel<__bf16><<<(unsigned)a.rows, 256, 0, stream>>>(a);
  TLCE_LAUNCH_CHECK();
  return 0;
}

TLCE_FUSED_ENTRY_POINTS(extern template, MfmaDirect4Engine<__bf16>)
TLCE_ENGINE_ENTRY_POINTS(extern template, MfmaDirect4Engine<__bf16>)
TLCE_ENGINE_ENTRY_POINTS(extern template, MfmaDirect4Engine<_Float16>)
TLCE_ENGINE_ENTRY_POINTS(extern template, MfmaEngine<__bf16>)
TLCE_ENGINE_ENTRY_POINTS(extern template, MfmaEngine<_Float16>)
TLCE_ENGINE_ENTRY_POINTS(extern template, SimtEngine<float>)
TLCE_ENGINE_ENTRY_POINTS(extern template, SimtEngine<__bf16>)
TLCE_ENGINE_ENTRY_POINTS(extern template, SimtEngine<_Float16>)

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
                  hipStream_t stream, const RowOptions& opt = RowOptions{}) {
  const bool local = shard.local_max != nullptr;
  const bool fused = opt.weighted_sum != nullptr;   // the masked-token loss entry point
  if (int rc = validate_common(hidden, weight, m, h, v, dtype)) return rc;
  TLCE_REQUIRE(!opt.weight_dim_first || dim_first_in_place(h, v, dtype),
               "forward: a [h, v] head is read in place only for 16-bit inputs with h and v "
               "multiples of 64 (h=%lld v=%lld dtype=%d); re-lay it to [v, h] for the other "
               "entry points", (long long)h, (long long)v, dtype);
  TLCE_REQUIRE(valid_count != nullptr, "forward: valid_count is null");
  TLCE_REQUIRE(opt.logit_scale > 0.0f, "forward: the logit multiplier must be positive");
  TLCE_REQUIRE(n_out >= m, "forward: n_out=%lld < m=%lld", (long long)n_out, (long long)m);
  TLCE_REQUIRE(row_idx != nullptr || n_out == m || m == 0,
               "forward: n_out != m without row_idx");
  if (int rc = fill_zero(valid_count, 4, stream)) return rc;
  TLCE_REQUIRE(local || fused || losses != nullptr || n_out == 0, "forward: losses is null");
  if (!local && losses != nullptr && (row_idx != nullptr || m == 0 || opt.row_count != nullptr)) {
    if (int rc = fill_zero(losses, n_out * 4, stream)) return rc;
  }
  if (fused && m == 0) {
    if (int rc = fill_zero(opt.weighted_sum, 4, stream)) return rc;
  }
  if (m == 0) return 0;
  TLCE_REQUIRE(labels && workspace && (local || ((losses || fused) && lse)),
               "forward: null pointer");
  const Plan p = make_plan(m, h, v, dtype, false, 0);
  const int64_t need = forward_layout(p, opt.row_count != nullptr, fused).total;
  TLCE_REQUIRE(workspace_bytes >= need, "forward: workspace too small (%lld < %lld)",
               (long long)workspace_bytes, (long long)need);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0, "forward: workspace must be 256-byte aligned");
  TLCE_DISPATCH(p, dtype,
                forward_impl<E>(p, hidden, weight, bias, labels, row_idx, m, h, v, ignore_index,
                                exclude_index, logit_softcap, losses, lse, valid_count, shard,
                                static_cast<char*>(workspace), stream, opt));
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

// ------------------------------------------------ head stored [h, v] ----
extern "C" int tlce_dim_first_supported(int64_t h, int64_t v, int dtype) {
  return (h > 0 && v > 0 && dim_first_in_place(h, v, dtype)) ? 1 : 0;
}

extern "C" int tlce_forward_dim_first(const void* hidden, const void* weight, const float* bias,
                                      const int64_t* labels, const int64_t* row_idx, int64_t m,
                                      int64_t n_out, int64_t h, int64_t v, int dtype,
                                      int64_t ignore_index, int64_t exclude_index,
                                      float logit_softcap, float* losses, float* lse,
                                      float* valid_count, void* workspace,
                                      int64_t workspace_bytes, void* stream) {
  RowOptions opt;
  opt.weight_dim_first = true;
  return forward_entry(hidden, weight, bias, labels, row_idx, m, n_out, h, v, dtype, ignore_index,
                       exclude_index, logit_softcap, losses, lse, valid_count, ShardStats{},
                       workspace, workspace_bytes, static_cast<hipStream_t>(stream), opt);
}

// ------------------------------------------- forward without a workspace ----
// The forward's only scratch memory (the per-split softmax partials) in a
// file-scope device array, for callers that may not allocate.  Each GPU holds
// its own copy of the array at its own address: the address is looked up once
// per device, with that device current, and only that pointer (never the
// array's name, which on the host is a stand-in and not a device address) is
// handed to kernels.
static __device__ __align__(256) unsigned char scratch[TLCE_FORWARD_NOALLOC_SCRATCH_BYTES];

namespace {

std::atomic<void*> g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device.
int scratch_pointer(void** out) {
  int device = 0;
  TLCE_HIP(hipGetDevice(&device));
  TLCE_REQUIRE(device >= 0 && device < kMaxDevices, "device index %d out of range", device);
  void* ptr = g_scratch_ptr[device].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    TLCE_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    TLCE_REQUIRE(ptr != nullptr, "hipGetSymbolAddress returned a null scratch address");
    g_scratch_ptr[device].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return 0;
}

}  // namespace

extern "C" int tlce_forward_noalloc(const void* hidden, const void* weight, const float* bias,
                                    const int64_t* labels, const int64_t* row_idx, int64_t m,
                                    int64_t n_out, int64_t h, int64_t v, int dtype,
                                    int64_t ignore_index, int64_t exclude_index,
                                    float logit_softcap, float* losses, float* lse,
                                    float* valid_count, void* stream) {
  TLCE_REQUIRE(m >= 0 && h > 0 && v > 0, "forward_noalloc: bad shape m=%lld h=%lld v=%lld",
               (long long)m, (long long)h, (long long)v);
  const int64_t need = forward_layout(make_plan(m, h, v, dtype, false, 0)).total;
  TLCE_REQUIRE(need <= (int64_t)TLCE_FORWARD_NOALLOC_SCRATCH_BYTES,
               "forward_noalloc: m=%lld needs %lld bytes of softmax partials, the static scratch "
               "array holds %lld (at most %lld rows); use tlce_forward with a workspace",
               (long long)m, (long long)need, (long long)TLCE_FORWARD_NOALLOC_SCRATCH_BYTES,
               (long long)TLCE_FORWARD_NOALLOC_MAX_ROWS);
  void* ptr = nullptr;
  if (int rc = scratch_pointer(&ptr)) return rc;
  return forward_entry(hidden, weight, bias, labels, row_idx, m, n_out, h, v, dtype, ignore_index,
                       exclude_index, logit_softcap, losses, lse, valid_count, ShardStats{}, ptr,
                       (int64_t)TLCE_FORWARD_NOALLOC_SCRATCH_BYTES,
                       static_cast<hipStream_t>(stream));
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
                   void* workspace, int64_t workspace_bytes, hipStream_t stream,
                   const RowOptions& opt = RowOptions{}) {
  if (int rc = validate_common(hidden, weight, m, h, v, dtype)) return rc;
  TLCE_REQUIRE(!opt.weight_dim_first || dim_first_in_place(h, v, dtype),
               "backward: a [h, v] head is read in place only for 16-bit inputs with h and v "
               "multiples of 64 (h=%lld v=%lld dtype=%d); re-lay it to [v, h] for the other "
               "entry points", (long long)h, (long long)v, dtype);
  TLCE_REQUIRE(opt.logit_scale > 0.0f, "backward: the logit multiplier must be positive");
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
  TLCE_REQUIRE(labels && lse && grad_output && workspace, "backward: null pointer");
  TLCE_REQUIRE(valid_count != nullptr || reduction_code != TLCE_REDUCTION_MEAN,
               "backward: the mean reduction needs valid_count");
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
                                 static_cast<char*>(workspace), stream, 0.0f, opt));
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

extern "C" int tlce_backward_dim_first(const void* hidden, const void* weight, const float* bias,
                                       const int64_t* labels, const int64_t* row_idx,
                                       const float* lse, const float* valid_count,
                                       const float* grad_output, int64_t m, int64_t n_out,
                                       int64_t h, int64_t v, int dtype, int reduction_code,
                                       int64_t ignore_index, int64_t exclude_index,
                                       float logit_softcap, void* grad_hidden, void* grad_weight,
                                       float* grad_bias, int64_t panel_bytes, void* workspace,
                                       int64_t workspace_bytes, void* stream) {
  RowOptions opt;
  opt.weight_dim_first = true;
  return backward_entry(hidden, weight, bias, labels, row_idx, lse, valid_count, grad_output, m,
                        n_out, h, v, dtype, reduction_code, 0, ignore_index, exclude_index,
                        logit_softcap, grad_hidden, grad_weight, grad_bias, panel_bytes, workspace,
                        workspace_bytes, static_cast<hipStream_t>(stream), opt);
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

// --------------------------------------------------------- masked-token loss --
extern "C" int64_t tlce_masked_loss_forward_workspace_bytes(int64_t m, int64_t h, int64_t v,
                                                            int dtype, int dynamic_rows) {
  if (m < 0 || h <= 0 || v <= 0) return -1;
  return forward_layout(make_plan(m, h, v, dtype, false, 0), dynamic_rows != 0, true).total;
}

extern "C" int tlce_masked_loss_forward(const void* hidden, const void* weight, const float* bias,
                                        const int64_t* labels, const float* token_weights,
                                        const int64_t* row_idx, const int64_t* row_count,
                                        int64_t m, int64_t n_out, int64_t h, int64_t v, int dtype,
                                        int64_t ignore_index, int64_t exclude_index,
                                        float logit_softcap, float logit_multiplier,
                                        float* losses, float* lse, float* valid_count,
                                        float* weighted_sum, void* workspace,
                                        int64_t workspace_bytes, void* stream) {
  TLCE_REQUIRE(weighted_sum != nullptr || losses != nullptr || n_out == 0,
               "masked_loss_forward: neither weighted_sum nor losses given");
  RowOptions opt;
  opt.logit_scale = logit_multiplier;
  opt.token_weights = token_weights;
  opt.row_count = row_count;
  opt.weighted_sum = weighted_sum;
  return forward_entry(hidden, weight, bias, labels, row_idx, m, n_out, h, v, dtype, ignore_index,
                       exclude_index, logit_softcap, losses, lse, valid_count, ShardStats{},
                       workspace, workspace_bytes, static_cast<hipStream_t>(stream), opt);
}

extern "C" int tlce_masked_loss_backward(const void* hidden, const void* weight, const float* bias,
                                         const int64_t* labels, const float* token_weights,
                                         const int64_t* row_idx, const int64_t* row_count,
                                         const float* lse, const float* valid_count,
                                         const float* grad_output, int64_t m, int64_t n_out,
                                         int64_t h, int64_t v, int dtype, int reduction_code,
                                         int64_t ignore_index, int64_t exclude_index,
                                         float logit_softcap, float logit_multiplier,
                                         void* grad_hidden, void* grad_weight, float* grad_bias,
                                         int64_t panel_bytes, void* workspace,
                                         int64_t workspace_bytes, void* stream) {
  RowOptions opt;
  opt.logit_scale = logit_multiplier;
  opt.token_weights = token_weights;
  opt.row_count = row_count;
  // d(sum_r w_r loss_r) / d loss_r = w_r: the sum reduction with per-row weights
  return backward_entry(hidden, weight, bias, labels, row_idx, lse, valid_count, grad_output, m,
                        n_out, h, v, dtype, reduction_code, 0, ignore_index, exclude_index,
                        logit_softcap, grad_hidden, grad_weight, grad_bias, panel_bytes, workspace,
                        workspace_bytes, static_cast<hipStream_t>(stream), opt);
}

// ---------------------------------------------------------- soft embedding --

extern "C" int64_t tlce_soft_embedding_workspace_bytes(int64_t m, int64_t h, int64_t v, int dtype,
                                                       int64_t panel_bytes) {
  if (m < 0 || h <= 0 || v <= 0) return -1;
  const Plan fp = make_plan(m, h, v, dtype, false, 0);
  const Plan bp = make_plan(m, h, v, dtype, false, panel_bytes);
  int64_t need = soft_embedding_layout(fp, bp, m, h, dtype).total;
  // the soft cap is not known here: enough for either sequence
  if (fused_gradients_supported(h, v, dtype)) {
    const FusedPlan p = make_fused_plan(m, h, v, dtype, panel_bytes);
    need = std::max(need, fused_layout(p, m, h, dtype, false).total);
  }
  return need;
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
  if (fused_gradients_supported(h, v, dtype) && embedding_scale > 0.0f) {
    // two contractions instead of three: under a soft cap of at most 40 no row maximum is
    // needed at all; otherwise one pass emits entries relative to exact tile maxima
    const bool capped = logit_softcap > 0.0f && logit_softcap <= kSoftEmbeddingMaxCap;
    const FusedPlan p = make_fused_plan(m, h, v, dtype, panel_bytes);
    const int64_t need = fused_layout(p, m, h, dtype, false).total;
    TLCE_REQUIRE(workspace_bytes >= need, "soft_embedding: workspace too small (%lld < %lld)",
                 (long long)workspace_bytes, (long long)need);
    TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0,
                 "soft_embedding: workspace must be 256-byte aligned");
    if (capped) {
      return soft_embedding_fused_impl<MfmaDirect4Engine<__bf16>>(
          p, hidden, weight, m, h, v, dtype, logit_softcap, embedding_scale, out,
          static_cast<char*>(workspace), stream);
    }
    return soft_embedding_emit_impl<MfmaDirect4Engine<__bf16>>(
        p, hidden, weight, m, h, v, dtype, logit_softcap, embedding_scale, out,
        static_cast<char*>(workspace), stream);
  }
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
                               float* teacher_lse, void* teacher_probabilities,
                               int64_t panel_bytes, void* workspace,
                               int64_t workspace_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = kl_validate(draft_hidden, draft_weight, teacher_hidden, teacher_weight, m,
                           h_draft, h_teacher, v, dtype))
    return rc;
  if (m == 0) return 0;
  TLCE_REQUIRE(losses && draft_lse && teacher_lse && workspace, "kl_forward: null pointer");
  TLCE_REQUIRE(((uintptr_t)teacher_probabilities & 255) == 0,
               "kl_forward: teacher_probabilities must be 256-byte aligned");
  const KlPlans k = kl_plans(m, h_draft, h_teacher, v, dtype, panel_bytes);
  TLCE_REQUIRE(workspace_bytes >= k.layout.total, "kl_forward: workspace too small (%lld < %lld)",
               (long long)workspace_bytes, (long long)k.layout.total);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0, "kl_forward: workspace must be 256-byte aligned");
  TLCE_DISPATCH(k.draft, dtype,
                kl_forward_impl<E>(k.draft, k.teacher, k.layout, draft_hidden, draft_weight,
                                   teacher_hidden, teacher_weight, m, h_draft, h_teacher, v, dtype,
                                   logit_softcap, losses, draft_lse, teacher_lse,
                                   static_cast<char*>(workspace), stream,
                                   teacher_probabilities));
}

extern "C" int64_t tlce_kl_teacher_probabilities_bytes(int64_t m, int64_t h_draft,
                                                       int64_t h_teacher, int64_t v, int dtype) {
  if (m <= 0 || h_draft <= 0 || h_teacher <= 0 || v <= 0) return 0;
  const KlPlans k = kl_plans(m, h_draft, h_teacher, v, dtype, 0);
  return k.draft.mp * k.draft.vp * dtype_bytes(dtype);
}

extern "C" int tlce_kl_gradient_in_forward_supported(int64_t m, int64_t h_draft,
                                                     int64_t h_teacher, int64_t v, int dtype,
                                                     float logit_softcap) {
  if (m <= 0 || h_draft <= 0 || h_teacher <= 0 || v <= 0) return 0;
  return kl_gradient_in_forward_supported(m, h_draft, h_teacher, v, dtype, logit_softcap) ? 1 : 0;
}

extern "C" int64_t tlce_kl_forward_with_gradient_workspace_bytes(int64_t m, int64_t h_draft,
                                                                 int64_t h_teacher, int64_t v,
                                                                 int dtype, int64_t panel_bytes) {
  if (!tlce_kl_gradient_in_forward_supported(m, h_draft, h_teacher, v, dtype, 0.0f)) return -1;
  // (the soft cap does not change the layout)
  const int64_t rows = std::min(m, fused_row_block(m, h_draft, v, dtype));   // the largest block
  const KlPlans k = kl_plans(rows, h_draft, h_teacher, v, dtype, panel_bytes);
  return kl_fused_layout(k.layout, k.draft, make_fused_plan(rows, h_draft, v, dtype, 0), h_draft)
      .total;
}

extern "C" int tlce_kl_forward_with_gradient(
    const void* draft_hidden, const void* draft_weight, const void* teacher_hidden,
    const void* teacher_weight, int64_t m, int64_t h_draft, int64_t h_teacher, int64_t v,
    int dtype, float logit_softcap, float* losses, float* draft_lse, float* teacher_lse,
    float* unit_grad_hidden_f32, int64_t panel_bytes, void* workspace, int64_t workspace_bytes,
    void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = kl_validate(draft_hidden, draft_weight, teacher_hidden, teacher_weight, m,
                           h_draft, h_teacher, v, dtype))
    return rc;
  if (m == 0) return 0;
  TLCE_REQUIRE(kl_gradient_in_forward_supported(m, h_draft, h_teacher, v, dtype, logit_softcap),
               "kl_forward_with_gradient: needs bf16 inputs, a soft cap of at most 40 or none, both "
               "hidden sizes and v multiples of 64 (h_draft=%lld, h_teacher=%lld, v=%lld)",
               (long long)h_draft, (long long)h_teacher, (long long)v);
  TLCE_REQUIRE(losses && draft_lse && teacher_lse && unit_grad_hidden_f32 && workspace,
               "kl_forward_with_gradient: null pointer");
  TLCE_REQUIRE(((uintptr_t)unit_grad_hidden_f32 & 15) == 0,
               "kl_forward_with_gradient: the gradient buffer must be 16-byte aligned");
  const int64_t need = tlce_kl_forward_with_gradient_workspace_bytes(m, h_draft, h_teacher, v,
                                                                     dtype, panel_bytes);
  TLCE_REQUIRE(workspace_bytes >= need,
               "kl_forward_with_gradient: workspace too small (%lld < %lld)",
               (long long)workspace_bytes, (long long)need);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0,
               "kl_forward_with_gradient: workspace must be 256-byte aligned");
  // rows are independent: blocks of the panel budget one after the other
  const int64_t block = fused_row_block(m, h_draft, v, dtype);
  const int64_t es = dtype_bytes(dtype);
  for (int64_t r0 = 0; r0 < m; r0 += block) {
    const int64_t rows = std::min(block, m - r0);
    const KlPlans k = kl_plans(rows, h_draft, h_teacher, v, dtype, panel_bytes);
    const FusedPlan fp = make_fused_plan(rows, h_draft, v, dtype, 0);
    if (int rc = kl_forward_with_gradient_impl<MfmaDirect4Engine<__bf16>>(
            k.draft, k.teacher, k.layout, fp,
            static_cast<const char*>(draft_hidden) + r0 * h_draft * es, draft_weight,
            static_cast<const char*>(teacher_hidden) + r0 * h_teacher * es, teacher_weight, rows,
            h_draft, h_teacher, v, dtype, logit_softcap, losses + r0, draft_lse + r0,
            teacher_lse + r0,
            unit_grad_hidden_f32 + r0 * h_draft, static_cast<char*>(workspace), stream))
      return rc;
  }
  return 0;
}

extern "C" int tlce_kl_backward(const void* draft_hidden, const void* draft_weight,
                                const void* teacher_hidden, const void* teacher_weight,
                                const float* draft_lse, const float* teacher_lse,
                                const float* grad_output,
                                const void* teacher_probabilities, int64_t m, int64_t h_draft,
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
                                    static_cast<char*>(workspace), stream,
                                    teacher_probabilities));
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

extern "C" int tlce_ce_topk_gradient_in_forward_supported(int64_t m, int64_t h, int64_t v,
                                                          int dtype) {
  if (m <= 0 || h <= 0 || v <= 0) return 0;
  return topk_gradient_in_forward_supported(m, h, v, dtype) ? 1 : 0;
}

extern "C" int64_t tlce_ce_topk_forward_with_gradient_workspace_bytes(int64_t m, int64_t h,
                                                                      int64_t v, int dtype,
                                                                      int64_t panel_bytes) {
  if (m <= 0 || h <= 0 || v <= 0 || !topk_gradient_in_forward_supported(m, h, v, dtype)) return -1;
  const int64_t rows = std::min(m, fused_row_block(m, h, v, dtype));   // the largest block
  return topk_fused_layout(topk_plan(rows, h, v, dtype, panel_bytes),
                           make_fused_plan(rows, h, v, dtype, 0), h).total;
}

extern "C" int tlce_ce_topk_forward_with_gradient(
    const void* hidden, const void* weight, const int64_t* labels, int64_t m, int64_t h,
    int64_t v, int dtype, int top_k, float output_multiplier, float logit_softcap, float* losses,
    float* probabilities, float* top_values, int64_t* top_ids, float* lse,
    float* unit_grad_hidden_f32, int64_t panel_bytes, void* workspace, int64_t workspace_bytes,
    void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = topk_validate(hidden, weight, labels, m, h, v, dtype, top_k)) return rc;
  if (m == 0) return 0;
  TLCE_REQUIRE(topk_gradient_in_forward_supported(m, h, v, dtype),
               "ce_topk_forward_with_gradient: needs bf16 inputs with h and v multiples of 64 "
               "(h=%lld, v=%lld)", (long long)h, (long long)v);
  TLCE_REQUIRE(losses && probabilities && top_values && top_ids && lse && unit_grad_hidden_f32 &&
                   workspace,
               "ce_topk_forward_with_gradient: null pointer");
  TLCE_REQUIRE(((uintptr_t)unit_grad_hidden_f32 & 15) == 0,
               "ce_topk_forward_with_gradient: the gradient buffer must be 16-byte aligned");
  const int64_t need =
      tlce_ce_topk_forward_with_gradient_workspace_bytes(m, h, v, dtype, panel_bytes);
  TLCE_REQUIRE(workspace_bytes >= need,
               "ce_topk_forward_with_gradient: workspace too small (%lld < %lld)",
               (long long)workspace_bytes, (long long)need);
  TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0,
               "ce_topk_forward_with_gradient: workspace must be 256-byte aligned");
  const int64_t block = fused_row_block(m, h, v, dtype);
  const char* hidden_b = static_cast<const char*>(hidden);
  for (int64_t r0 = 0; r0 < m; r0 += block) {
    const int64_t rows = std::min(block, m - r0);
    const TopkPlan t = topk_plan(rows, h, v, dtype, panel_bytes);
    const FusedPlan p = make_fused_plan(rows, h, v, dtype, 0);
    if (int rc = topk_forward_with_gradient_impl<MfmaDirect4Engine<__bf16>>(
            t, p, hidden_b + r0 * h * dtype_bytes(dtype), weight, labels + r0, rows, h, v, top_k,
            output_multiplier, logit_softcap, losses + r0, probabilities + r0,
            top_values + r0 * top_k, top_ids + r0 * top_k, lse + r0,
            unit_grad_hidden_f32 + r0 * h, static_cast<char*>(workspace), stream))
      return rc;
  }
  return 0;
}

extern "C" int tlce_ce_topk_apply_gradient(const float* unit_grad_hidden_f32, const void* hidden,
                                           const void* weight, const int64_t* labels,
                                           const int64_t* top_ids, const float* ce_scale,
                                           const float* grad_top_values, int64_t m, int64_t h,
                                           int64_t v, int dtype, int top_k,
                                           float output_multiplier, float logit_softcap,
                                           void* grad_hidden, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = topk_validate(hidden, weight, labels, m, h, v, dtype, top_k)) return rc;
  TLCE_REQUIRE(dtype == TLCE_DTYPE_BF16, "ce_topk_apply_gradient: bf16 only");
  if (m == 0) return 0;
  TLCE_REQUIRE(unit_grad_hidden_f32 && top_ids && ce_scale && grad_hidden,
               "ce_topk_apply_gradient: null pointer");
  TopkApplyArgs a;
  a.unit = unit_grad_hidden_f32; a.hidden = hidden; a.weight = weight; a.labels = labels;
  a.top_ids = top_ids; a.ce_scale = ce_scale; a.grad_top_values = grad_top_values;
  a.m = (int)m; a.h = (int)h; a.k = top_k;
  a.softcap = logit_softcap; a.logit_scale = output_multiplier; a.grad_hidden = grad_hidden;
  return launch_topk_apply(a, stream);
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

// ------------------------------------------------ per-sample loss numerators --
extern "C" int tlce_segment_weighted_sum(const float* values, const float* weights,
                                         const int64_t* row_idx, const int64_t* row_count,
                                         int64_t m, int64_t segment_length, int64_t n_segments,
                                         float* out, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  TLCE_REQUIRE(m >= 0 && segment_length > 0 && n_segments >= 0 && n_segments < (1ll << 31),
               "segment_weighted_sum: bad sizes m=%lld segment_length=%lld n_segments=%lld",
               (long long)m, (long long)segment_length, (long long)n_segments);
  if (n_segments == 0) return 0;
  TLCE_REQUIRE(out != nullptr, "segment_weighted_sum: out is null");
  TLCE_REQUIRE(m == 0 || (values != nullptr && row_idx != nullptr),
               "segment_weighted_sum: null pointer");
  ScopedTimer timer(kClassOther, stream);
  lce_segment_weighted_sum_kernel<<<(int)n_segments, 256, 0, stream>>>(
      values, weights, row_idx, row_count, m, segment_length, out);
  TLCE_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------ forward that leaves the gradients ----
extern "C" int tlce_fused_gradients_supported(int64_t h, int64_t v, int dtype) {
  return (h > 0 && v > 0 && fused_gradients_supported(h, v, dtype)) ? 1 : 0;
}

extern "C" int tlce_query_fused_plan(int64_t m, int64_t h, int64_t v, int dtype,
                                     int64_t panel_bytes, int64_t* block_rows, int* n_blocks,
                                     int* grad_hidden_k_splits) {
  TLCE_REQUIRE(m >= 0 && h > 0 && v > 0, "query_fused_plan: bad shape");
  TLCE_REQUIRE(fused_gradients_supported(h, v, dtype),
               "query_fused_plan: needs bf16 inputs with h and v multiples of 64");
  const FusedPlan p = make_fused_plan(m, h, v, dtype, panel_bytes);
  if (block_rows) *block_rows = p.block_rows;
  if (n_blocks) *n_blocks = p.n_blocks;
  if (grad_hidden_k_splits) *grad_hidden_k_splits = p.dh_ksplit;
  return 0;
}

extern "C" int64_t tlce_forward_with_gradients_workspace_bytes(int64_t m, int64_t h, int64_t v,
                                                               int dtype, int compute_weight_grad,
                                                               int64_t panel_bytes) {
  if (m < 0 || h <= 0 || v <= 0 || !fused_gradients_supported(h, v, dtype)) return -1;
  return fused_layout(make_fused_plan(m, h, v, dtype, panel_bytes), m, h, dtype,
                      compute_weight_grad != 0).total;
}

extern "C" int tlce_forward_with_gradients(
    const void* hidden, const void* weight, const int64_t* labels, const int64_t* row_idx,
    const float* token_weights, const int64_t* row_count, int64_t m, int64_t n_out, int64_t h,
    int64_t v, int dtype, int64_t ignore_index, int64_t exclude_index, float logit_softcap,
    float logit_multiplier,
    float* losses, float* lse, float* valid_count, float* grad_hidden_f32, float* grad_weight_f32,
    int64_t panel_bytes, void* workspace, int64_t workspace_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (int rc = validate_common(hidden, weight, m, h, v, dtype)) return rc;
  TLCE_REQUIRE(fused_gradients_supported(h, v, dtype),
               "forward_with_gradients: needs bf16 inputs with h and v multiples of 64 "
               "(h=%lld v=%lld dtype=%d)", (long long)h, (long long)v, dtype);
  TLCE_REQUIRE(valid_count != nullptr, "forward_with_gradients: valid_count is null");
  TLCE_REQUIRE(logit_multiplier > 0.0f,
               "forward_with_gradients: the logit multiplier must be positive");
  TLCE_REQUIRE(n_out >= m, "forward_with_gradients: n_out=%lld < m=%lld", (long long)n_out,
               (long long)m);
  TLCE_REQUIRE(row_idx != nullptr || n_out == m || m == 0,
               "forward_with_gradients: n_out != m without row_idx");
  TLCE_REQUIRE(row_count == nullptr || row_idx != nullptr,
               "forward_with_gradients: a device-side row count needs row_idx");
  TLCE_REQUIRE(((uintptr_t)grad_hidden_f32 & 15) == 0 && ((uintptr_t)grad_weight_f32 & 15) == 0,
               "forward_with_gradients: gradients must be 16-byte aligned");
  // everything that can be refused is refused before the first launch
  const FusedPlan p = make_fused_plan(m, h, v, dtype, panel_bytes);
  if (m > 0) {
    TLCE_REQUIRE(labels && lse && grad_hidden_f32 && workspace,
                 "forward_with_gradients: null pointer");
    const int64_t need = fused_layout(p, m, h, dtype, grad_weight_f32 != nullptr).total;
    TLCE_REQUIRE(workspace_bytes >= need,
                 "forward_with_gradients: workspace too small (%lld < %lld)",
                 (long long)workspace_bytes, (long long)need);
    TLCE_REQUIRE(((uintptr_t)workspace & 255) == 0,
                 "forward_with_gradients: workspace must be 256-byte aligned");
  }
  if (int rc = fill_zero(valid_count, 4, stream)) return rc;
  if (losses != nullptr && (row_idx != nullptr || m == 0)) {
    if (int rc = fill_zero(losses, n_out * 4, stream)) return rc;
  }
  if (m == 0) {
    if (grad_weight_f32 != nullptr) return fill_zero(grad_weight_f32, v * h * 4, stream);
    return 0;
  }
  FusedOptions opt;
  opt.logit_scale = logit_multiplier;
  opt.token_weights = token_weights;
  opt.row_count = row_count;
  return fused_gradients_impl<MfmaDirect4Engine<__bf16>>(
      p, hidden, weight, labels, row_idx, m, h, v, dtype, ignore_index, exclude_index,
      logit_softcap, losses, lse, valid_count, grad_hidden_f32, grad_weight_f32,
      static_cast<char*>(workspace), stream, opt);
}

extern "C" int tlce_apply_grad_output(const float* grad_hidden_f32, const float* grad_weight_f32,
                                      const int64_t* row_idx, const int64_t* row_count,
                                      const float* grad_output,
                                      const float* valid_count, int64_t m, int64_t n_out,
                                      int64_t h, int64_t v, int dtype, int reduction_code,
                                      void* grad_hidden, void* grad_weight, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  TLCE_REQUIRE(dtype == TLCE_DTYPE_BF16, "apply_grad_output: unsupported dtype code %d (bf16 only)",
               dtype);
  TLCE_REQUIRE(m >= 0 && h > 0 && v > 0 && (h % 4) == 0, "apply_grad_output: bad shape");
  TLCE_REQUIRE(reduction_code == TLCE_REDUCTION_SUM || reduction_code == TLCE_REDUCTION_MEAN ||
                   reduction_code == TLCE_REDUCTION_NONE,
               "apply_grad_output: unknown reduction code %d", reduction_code);
  TLCE_REQUIRE(reduction_code != TLCE_REDUCTION_NONE || grad_weight_f32 == nullptr,
               "apply_grad_output: with one upstream gradient per row (reduction none) the "
               "grad_weight contraction has to wait for it (grad_weight_from_panel)");
  TLCE_REQUIRE(n_out >= m, "apply_grad_output: n_out=%lld < m=%lld", (long long)n_out,
               (long long)m);
  TLCE_REQUIRE(row_idx != nullptr || n_out == m || m == 0,
               "apply_grad_output: n_out != m without row_idx");
  TLCE_REQUIRE(row_count == nullptr || row_idx != nullptr,
               "apply_grad_output: a device-side row count needs row_idx");
  TLCE_REQUIRE(grad_hidden != nullptr || n_out == 0, "apply_grad_output: grad_hidden is null");
  TLCE_REQUIRE(grad_output != nullptr, "apply_grad_output: grad_output is null");
  TLCE_REQUIRE(valid_count != nullptr || reduction_code != TLCE_REDUCTION_MEAN,
               "apply_grad_output: the mean reduction needs valid_count");
  TLCE_REQUIRE((grad_weight == nullptr) == (grad_weight_f32 == nullptr),
               "apply_grad_output: grad_weight and its float32 source go together");
  TLCE_REQUIRE((((uintptr_t)grad_hidden | (uintptr_t)grad_weight | (uintptr_t)grad_hidden_f32 |
                 (uintptr_t)grad_weight_f32) & 15) == 0,
               "apply_grad_output: gradients must be 16-byte aligned");
  const int64_t es = dtype_bytes(dtype);
  if (row_idx != nullptr || m == 0) {
    if (int rc = fill_zero(grad_hidden, n_out * h * es, stream)) return rc;
  }
  ScaleCastArgs a;
  a.grad_output = grad_output; a.valid_count = valid_count; a.reduction = reduction_code;
  a.h = (int)h;
  if (m > 0) {
    TLCE_REQUIRE(grad_hidden_f32 != nullptr, "apply_grad_output: null pointer");
    a.in = grad_hidden_f32; a.row_idx = row_idx; a.rows = m; a.out = grad_hidden;
    a.m_dev = row_count;
    if (int rc = launch_scale_cast(a, stream)) return rc;
    a.m_dev = nullptr;
  }
  if (grad_weight != nullptr) {
    a.in = grad_weight_f32; a.row_idx = nullptr; a.rows = v; a.out = grad_weight;
    if (int rc = launch_scale_cast(a, stream)) return rc;
  }
  return 0;
}

extern "C" int tlce_grad_weight_from_panel(const void* hidden, const int64_t* row_idx,
                                           const int64_t* row_count,
                                           const float* grad_output, const float* valid_count,
                                           int64_t m, int64_t h, int64_t v, int dtype,
                                           int reduction_code, void* grad_weight,
                                           int64_t panel_bytes, void* forward_workspace,
                                           int64_t workspace_bytes, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  TLCE_REQUIRE(m >= 0 && h > 0 && v > 0, "grad_weight_from_panel: bad shape");
  TLCE_REQUIRE(fused_gradients_supported(h, v, dtype),
               "grad_weight_from_panel: needs bf16 inputs with h and v multiples of 64");
  TLCE_REQUIRE(reduction_code == TLCE_REDUCTION_SUM || reduction_code == TLCE_REDUCTION_MEAN ||
                   reduction_code == TLCE_REDUCTION_NONE,
               "grad_weight_from_panel: unknown reduction code %d", reduction_code);
  TLCE_REQUIRE(grad_weight != nullptr && grad_output != nullptr,
               "grad_weight_from_panel: null pointer");
  TLCE_REQUIRE(valid_count != nullptr || reduction_code != TLCE_REDUCTION_MEAN,
               "grad_weight_from_panel: the mean reduction needs valid_count");
  TLCE_REQUIRE(((uintptr_t)grad_weight & 15) == 0 && ((uintptr_t)hidden & 15) == 0,
               "grad_weight_from_panel: operands must be 16-byte aligned");
  const FusedPlan p = make_fused_plan(m, h, v, dtype, panel_bytes);
  TLCE_REQUIRE(p.n_blocks == 1,
               "grad_weight_from_panel: the forward took %d blocks of rows; the panel holds all "
               "rows only when there is one", p.n_blocks);
  if (m == 0) return fill_zero(grad_weight, v * h * dtype_bytes(dtype), stream);
  TLCE_REQUIRE(hidden != nullptr && forward_workspace != nullptr,
               "grad_weight_from_panel: null pointer");
  const int64_t need = fused_layout(p, m, h, dtype, true).total;
  TLCE_REQUIRE(workspace_bytes >= need,
               "grad_weight_from_panel: workspace too small (%lld < %lld): size it with "
               "compute_weight_grad = 1", (long long)workspace_bytes, (long long)need);
  TLCE_REQUIRE(((uintptr_t)forward_workspace & 255) == 0,
               "grad_weight_from_panel: workspace must be 256-byte aligned");
  return deferred_grad_weight_impl<MfmaDirect4Engine<__bf16>>(
      p, hidden, m, h, v, dtype, grad_output, valid_count, reduction_code, row_count, row_idx,
      grad_weight, static_cast<char*>(forward_workspace), stream);
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
