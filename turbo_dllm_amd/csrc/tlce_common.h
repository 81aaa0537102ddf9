// Shared host/device helpers for the gfx950 fused linear cross-entropy library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <string.h>

#include <algorithm>

#include "../../include/tlce.h"

namespace tlce {

// ---------------------------------------------------------------- errors ----
// Thread-local message buffer behind tlce_last_error().  The reference raises
// through TORCH_CHECK (fused_linear_ce.cpp:107-111); here every entry point
// returns a code and leaves the text for the host binding to raise.
char* error_buffer();
int fail(const char* fmt, ...);

#define TLCE_HIP(expr)                                                        \
  do {                                                                        \
    hipError_t tlce_err__ = (expr);                                           \
    if (tlce_err__ != hipSuccess) {                                           \
      return ::tlce::fail("%s failed: %s (%s:%d)", #expr,                     \
                          hipGetErrorString(tlce_err__), __FILE__, __LINE__); \
    }                                                                         \
  } while (0)

#define TLCE_REQUIRE(cond, ...)           \
  do {                                    \
    if (!(cond)) {                        \
      return ::tlce::fail(__VA_ARGS__);   \
    }                                     \
  } while (0)

#define TLCE_LAUNCH_CHECK() TLCE_HIP(hipGetLastError())

// ----------------------------------------------------------------- sizes ----
static inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
static inline int64_t ceil_div(int64_t x, int64_t m) { return (x + m - 1) / m; }
static inline int64_t align256(int64_t x) { return round_up(x, 256); }

static inline int dtype_bytes(int dtype) { return dtype == TLCE_DTYPE_F32 ? 4 : 2; }

// Forward launch shape: token tiles x vocabulary splits workgroups, at most (and
// close to) four whole waves of 256 workgroups on a 256-CU MI355X.  Shared by
// the host plan and by the kernels that derive the plan from a row count that
// only the device knows.
constexpr int kTargetWorkgroups = 1024;
__host__ __device__ static inline int forward_vocab_splits(int n_ttiles, int n_vtiles) {
  const int want = n_ttiles > 0 ? kTargetWorkgroups / n_ttiles : kTargetWorkgroups;
  const int s = want < 1 ? 1 : want;
  return s < n_vtiles ? s : n_vtiles;
}

// K splits of the grad_hidden contraction: `tiles` output tiles per panel, each a
// loop of `k_steps` K steps when unsplit; every split accumulates into a float32
// slab of its own (`slab_elems` elements), summed by the final cast.  Picks the
// count in [1, max_split] with the least estimated time, in units of one K step:
//   rounds of 256 workgroups x (K steps per split + 8 for a tile's start and output)
//   + splits x the time the final cast needs to read one more slab.
// Ties go to fewer splits.  Integer arithmetic only: the host plan and the
// kernels that re-plan for a row count known on the device must agree.
__host__ __device__ static inline int grad_hidden_k_splits(int64_t tiles, int max_split,
                                                           int64_t k_steps, int64_t slab_elems) {
  const int64_t per_slab = (slab_elems >> 20) > 1 ? (slab_elems >> 20) : 1;
  int pick = 1;
  int64_t best = -1;
  for (int ks = 1; ks <= max_split; ++ks) {
    const int64_t rounds = (tiles * ks + 255) / 256;
    const int64_t cost = rounds * ((k_steps + ks - 1) / ks + 8) + ks * per_slab;
    if (best < 0 || cost < best) {
      best = cost;
      pick = ks;
    }
  }
  return pick;
}

constexpr int kXcds = 8;  // MI355X: 8 accelerator dies, workgroups dealt round-robin

// ------------------------------------------------------------- device -------
#define TLCE_LOG2E 1.4426950408889634f
#define TLCE_LN2 0.6931471805599453f

// Workgroups are dealt to the 8 XCDs round-robin by blockIdx; each XCD has its
// own L2.  Map the hardware block id to a logical id so that one XCD works on
// a contiguous range of logical ids (launch grids are multiples of 8).
__device__ __forceinline__ int xcd_logical_block(int bid, int nblocks) {
  const int per = nblocks / kXcds;
  return (bid % kXcds) * per + (bid / kXcds);
}

// Rows of a call whose row count lives on the device: `m` is then the
// capacity the launch was sized for and *m_dev (clamped to [0, m]) the real
// count.  m_dev == null: m itself.
__device__ __forceinline__ int effective_rows(int m, const int64_t* m_dev) {
  if (m_dev == nullptr) return m;
  const int64_t c = *m_dev;
  return c < 0 ? 0 : (c < (int64_t)m ? (int)c : m);
}

// Rows of a block of `cap` rows that starts at row `offset` of a matrix whose real
// row count is on the device (null: all `cap`).
__device__ __forceinline__ int effective_block_rows(int cap, const int64_t* m_dev, int64_t offset) {
  if (m_dev == nullptr) return cap;
  const int64_t c = *m_dev - offset;
  return c < 0 ? 0 : (c < (int64_t)cap ? (int)c : cap);
}

// Logical block id when only the first `tiles` of the launched workgroups have
// work (the launch was sized for more rows than there are): the same mapping a
// launch of round_up(tiles, 8) workgroups would get; -1 for the others.
__device__ __forceinline__ int xcd_logical_block_of(int bid, int tiles) {
  const int total = (tiles + kXcds - 1) / kXcds * kXcds;
  if (bid >= total) return -1;
  const int logical = xcd_logical_block(bid, total);
  return logical < tiles ? logical : -1;
}

// Grouped tile order: consecutive logical ids walk `group` tiles along i, then
// step j, so the ~32 workgroups resident on one XCD cover a group x (32/group)
// block of tiles and share both operands through that XCD's L2.
__device__ __forceinline__ void grouped_tile(int logical, int ni, int nj, int group,
                                             int* ti, int* tj) {
  const int width = group * nj;
  const int gid = logical / width;
  const int first = gid * group;
  const int gsize = min(ni - first, group);
  const int within = logical - gid * width;
  *ti = first + within % gsize;
  *tj = within / gsize;
}

// The same order with the groups along i balanced: ceil(ni / group) groups whose
// sizes differ by at most one (13 tiles in groups of at most 4: 4, 3, 3, 3 instead
// of 4, 4, 4, 1), for launches whose ni is small and not a multiple of the group.
__device__ __forceinline__ void balanced_grouped_tile(int logical, int ni, int nj, int group,
                                                      int* ti, int* tj) {
  const int n_groups = (ni + group - 1) / group;
  const int base = ni / n_groups, extra = ni % n_groups;   // the first `extra` groups hold base + 1
  const int big = (base + 1) * nj;
  int first, gsize, within;
  if (logical < extra * big) {
    const int g = logical / big;
    gsize = base + 1;
    first = g * gsize;
    within = logical - g * big;
  } else {
    const int rest = logical - extra * big;
    const int g = rest / (base * nj);
    gsize = base;
    first = extra * (base + 1) + g * base;
    within = rest - g * base * nj;
  }
  *ti = first + within % gsize;
  *tj = within / gsize;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// tanh(x) = 1 - 2 / (1 + e^{2x}); saturates cleanly to +-1 for large |x|.
__device__ __forceinline__ float fast_tanh(float x) {
  const float e = fast_exp2(x * (2.0f * TLCE_LOG2E));
  return 1.0f - 2.0f * fast_rcp(1.0f + e);
}

// Elementwise math by engine.  The float32 engine (float32 inputs, held to the
// reference's 2e-5 bars) takes the library routines: fast_tanh loses relative
// accuracy for small arguments (1 - 2 / (1 + e) cancels), which the soft cap's
// derivative then carries into the gradient.  The 16-bit engines take the
// hardware approximations, whose error is far below the rounding of their inputs.
template <bool kPrecise>
__device__ __forceinline__ float exp2_of(float x) {
  if constexpr (kPrecise) return exp2f(x);
  else return fast_exp2(x);
}
template <bool kPrecise>
__device__ __forceinline__ float log2_of(float x) {
  if constexpr (kPrecise) return log2f(x);
  else return fast_log2(x);
}
template <bool kPrecise>
__device__ __forceinline__ float tanh_of(float x) {
  if constexpr (kPrecise) return tanhf(x);
  else return fast_tanh(x);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

template <typename T>
__device__ __forceinline__ float to_float(T x) { return static_cast<float>(x); }
template <typename T>
__device__ __forceinline__ T from_float(float x) { return static_cast<T>(x); }

// Host-side launch grid: a multiple of 8 so xcd_logical_block is a bijection.
static inline int xcd_grid(int64_t tiles) { return (int)round_up(tiles, kXcds); }

}  // namespace tlce
