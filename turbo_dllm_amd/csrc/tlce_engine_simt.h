// 64x64x16 float32-FMA tile engine: the generic path for float32 inputs and for
// shapes the MFMA engine cannot take (hidden size not a multiple of 8).
//
// Same contract as MfmaEngine: C[i][j] = sum_k A[i][k] * B[j][k] over one tile,
// A and B K-contiguous.  256 threads; thread t owns tile column t%64 and the 16
// consecutive tile rows 16*(t/64) .. +16.  Products are accumulated in float32
// in ascending K order, so results are reproducible run to run.
#pragma once

#include "tlce_common.h"

namespace tlce {

template <typename T_>
struct SimtEngine {
  using T = T_;

  static constexpr int kTile = 64;
  static constexpr int kBK = 16;
  static constexpr int kThreads = 256;
  static constexpr int kPad = kBK + 1;
  static constexpr int kSmemBytes = 2 * kTile * kPad * 4;  // A and B slabs, float32
  static constexpr int kCols = 1;
  static constexpr int kRows = 16;
  static constexpr int kShare = 4;
  static constexpr bool kHasKMajor = false;
  static constexpr bool kPrecise = sizeof(T_) == 4;   // float32 inputs: library exp / tanh

  struct Acc { float c[kRows]; };

  int tid;

  __device__ __forceinline__ SimtEngine() { tid = threadIdx.x; }

  __device__ __forceinline__ int col(int) const { return tid & 63; }
  __device__ __forceinline__ int row(int i) const { return (tid >> 6) * 16 + i; }
  __device__ __forceinline__ int share_slot() const { return tid >> 6; }
  static __device__ __forceinline__ float get(const Acc& a, int, int i) { return a.c[i]; }
  static __device__ __forceinline__ void set(Acc& a, int, int i, float v) { a.c[i] = v; }
  static __device__ __forceinline__ void zero(Acc& a) {
#pragma unroll
    for (int i = 0; i < kRows; ++i) a.c[i] = 0.0f;
  }
  // A wave is 64 lanes = the 64 tile columns of one 16-row band.
  __device__ __forceinline__ float reduce_over_cols(float v) const { return wave_sum(v); }
  __device__ __forceinline__ bool col_leader() const { return (tid & 63) == 0; }
  // every lane of a wave owns a different tile column
  __device__ __forceinline__ float reduce_over_rows_in_wave(float v) const { return v; }
  __device__ __forceinline__ bool row_leader() const { return true; }
  __device__ __forceinline__ void forget_lane_invariants() {}

  __device__ __forceinline__ void mainloop(const T* __restrict__ A, int64_t lda, int a_row0,
                                           int a_rows, const T* __restrict__ B, int64_t ldb,
                                           int b_row0, int b_rows, int k_begin, int k_end,
                                           Acc& acc, char* smem) const {
    float* As = reinterpret_cast<float*>(smem);
    float* Bs = As + kTile * kPad;
    const int my_col = tid & 63;
    const int band = (tid >> 6) * 16;
    for (int k0 = k_begin; k0 < k_end; k0 += kBK) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int e = tid + 256 * q;
        const int r = e >> 4;
        const int kk = e & 15;
        const int k = k0 + kk;
        const int ar = min(a_row0 + r, a_rows - 1);
        const int br = min(b_row0 + r, b_rows - 1);
        As[r * kPad + kk] = (k < k_end) ? to_float<T>(A[(int64_t)ar * lda + k]) : 0.0f;
        Bs[r * kPad + kk] = (k < k_end) ? to_float<T>(B[(int64_t)br * ldb + k]) : 0.0f;
      }
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < kBK; ++kk) {
        const float b = Bs[my_col * kPad + kk];
#pragma unroll
        for (int i = 0; i < kRows; ++i) acc.c[i] = fmaf(As[(band + i) * kPad + kk], b, acc.c[i]);
      }
      __syncthreads();
    }
  }

  // acc = A * B^T (same operands as mainloop).
  __device__ __forceinline__ void mainloop_set(const T* __restrict__ A, int64_t lda, int a_row0,
                                               int a_rows, const T* __restrict__ B, int64_t ldb,
                                               int b_row0, int b_rows, int k_begin, int k_end,
                                               Acc& acc, char* smem) const {
    zero(acc);
    mainloop(A, lda, a_row0, a_rows, B, ldb, b_row0, b_rows, k_begin, k_end, acc, smem);
  }
};

}  // namespace tlce
