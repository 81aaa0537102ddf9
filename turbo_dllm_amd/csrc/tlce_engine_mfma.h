// 256x256 bf16/f16 MFMA tile engines for gfx950 (CDNA4), wave64.
//
// Both compute C[i][j] = sum_k A[i][k] * B[j][k] for one 256x256 tile, A and B both
// K-contiguous (row-major [rows, K]).  512 threads = 8 waves in a 2 (A rows) x
// 4 (B rows) grid; each wave owns a 128x64 sub-tile as 4x2
// v_mfma_f32_32x32x16 blocks (128 fp32 accumulator registers per lane), two
// waves per SIMD.
//
// LDS: two stages of (A 256x64 + B 256x64) 2-byte elements = 2 x 64 KiB of the
// CU's 160 KiB.  A tile row is 128 bytes = eight 16-byte chunks; chunk c of
// row r lives at chunk slot c ^ ((r >> 1) & 7), which makes both the 16-byte
// staging writes and the 16-byte MFMA fragment reads hit all 64 banks.
//
// Accumulator layout of one 32x32 block (lane l, register q of 16):
//   row = 8*(q/4) + 4*(l/32) + q%4,   col = l%32.
// A/B fragment of one block for K-slice ks: lane l supplies row l%32,
// K = 16*ks + 8*(l/32) .. +8  (one 16-byte chunk).
#pragma once

#include <type_traits>

#include "tlce_common.h"

namespace tlce {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

template <typename T> struct MfmaOp;
template <> struct MfmaOp<__bf16> {
  using V8 = bf16x8_t;
  static __device__ __forceinline__ f32x16_t mma(V8 a, V8 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct MfmaOp<_Float16> {
  using V8 = f16x8_t;
  static __device__ __forceinline__ f32x16_t mma(V8 a, V8 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// Thread <-> tile-element mapping shared by the MFMA engines: 2 waves along
// the A rows, kWavesN_ along the B rows, each wave 4 x kTN_ blocks of 32x32
// (8 waves of 128x64, or 4 waves of 128x128).
template <typename T_, int kWavesN_ = 4, int kTN_ = 2>
struct MfmaTileLayout {
  using T = T_;
  using Op = MfmaOp<T>;
  using V8 = typename Op::V8;

  static constexpr int kTile = 256;     // BM == BN
  static constexpr int kWavesN = kWavesN_;   // waves along B rows
  static constexpr int kThreads = 2 * kWavesN * 64;
  static constexpr int kTM = 4;         // 32-row blocks per wave along A rows
  static constexpr int kTN = kTN_;      // 32-col blocks per wave along B rows
  static constexpr int kCols = kTN;          // tile columns owned per thread
  static constexpr int kRows = kTM * 16;     // tile rows held per owned column
  static constexpr int kShare = 4;           // threads that hold the same column
  static_assert(kWavesN * kTN * 32 == kTile, "waves must tile the 256 B rows");

  struct Acc { f32x16_t c[kTM][kTN]; };

  int lane, wave, wm, wn;

  __device__ __forceinline__ MfmaTileLayout() {
    lane = threadIdx.x & 63;
    wave = threadIdx.x >> 6;
    wm = wave / kWavesN;
    wn = wave % kWavesN;
  }

  __device__ __forceinline__ int col(int j) const {
    return wn * (kTN * 32) + j * 32 + (lane & 31);
  }
  __device__ __forceinline__ int row(int i) const {
    return wm * 128 + (i >> 4) * 32 + ((i >> 2) & 3) * 8 + (lane >> 5) * 4 + (i & 3);
  }
  __device__ __forceinline__ int share_slot() const { return wm * 2 + (lane >> 5); }
  static __device__ __forceinline__ float get(const Acc& a, int j, int i) {
    return a.c[i >> 4][j][i & 15];
  }
  static __device__ __forceinline__ void set(Acc& a, int j, int i, float v) {
    a.c[i >> 4][j][i & 15] = v;
  }
  static __device__ __forceinline__ void zero(Acc& a) {
#pragma unroll
    for (int tm = 0; tm < kTM; ++tm)
#pragma unroll
      for (int tn = 0; tn < kTN; ++tn)
#pragma unroll
        for (int q = 0; q < 16; ++q) a.c[tm][tn][q] = 0.0f;
  }
  // Sum over the lanes that hold the same tile row (the 32 lanes of a half-wave).
  __device__ __forceinline__ float reduce_over_cols(float v) const {
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
  }
  __device__ __forceinline__ bool col_leader() const { return (lane & 31) == 0; }
};

// Register-staged engine: global -> VGPR -> LDS, two 64-wide K stages.  Takes
// any K that is a multiple of 8 (zero-fills the tail); used when the hidden
// size is not a multiple of 32.
template <typename T_>
struct MfmaEngine : MfmaTileLayout<T_> {
  using Base = MfmaTileLayout<T_>;
  using T = T_;
  using Op = typename Base::Op;
  using V8 = typename Base::V8;
  using Acc = typename Base::Acc;
  using Base::kTile;
  using Base::kTM;
  using Base::kTN;
  using Base::lane;
  using Base::wm;
  using Base::wn;
  static constexpr int kBK = 64;
  static constexpr int kRowBytes = kBK * 2;                  // 128
  static constexpr int kStageBytes = 2 * kTile * kRowBytes;  // 65536
  static constexpr int kSmemBytes = 2 * kStageBytes;         // 131072

  // acc += A[a_row0 .. +256, k_begin .. k_end) * B[b_row0 .. +256, same K)^T.
  // Rows past a_rows / b_rows are clamped to the last valid row (their results
  // are discarded by the caller); K past k_end is zero-filled.  k_begin and
  // k_end are multiples of 8 and lda/ldb multiples of 8 (16-byte chunks).
  __device__ __forceinline__ void mainloop(const T* __restrict__ A, int64_t lda, int a_row0,
                                           int a_rows, const T* __restrict__ B, int64_t ldb,
                                           int b_row0, int b_rows, int k_begin, int k_end,
                                           Acc& acc, char* smem) const {
    const int tid = threadIdx.x;
    const int c = tid & 7;
    const int r0 = tid >> 3;
    const int pc = c ^ ((tid >> 4) & 7);

    const T* ap[4];
    const T* bp[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int ar = min(a_row0 + r0 + 64 * j, a_rows - 1);
      const int br = min(b_row0 + r0 + 64 * j, b_rows - 1);
      ap[j] = A + (int64_t)ar * lda + k_begin + c * 8;
      bp[j] = B + (int64_t)br * ldb + k_begin + c * 8;
    }
    const int st_off = r0 * kRowBytes + pc * 16;

    const int swz = (lane >> 1) & 7;
    const int hi = lane >> 5;
    const int a_frag = (wm * 128 + (lane & 31)) * kRowBytes;
    const int b_frag = kTile * kRowBytes + (wn * 64 + (lane & 31)) * kRowBytes;

    uint4 ra[4], rb[4];

    // A chunk past k_end re-reads the row's first chunk (always in bounds) and
    // is zeroed in registers, so the loads stay unconditional global loads.
    auto gload = [&](int k0) {
      const bool ok = (k0 + c * 8) < k_end;
      const int64_t back = ok ? 0 : (int64_t)(k0 - k_begin + c * 8);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        ra[j] = *reinterpret_cast<const uint4*>(ap[j] - back);
        rb[j] = *reinterpret_cast<const uint4*>(bp[j] - back);
        if (!ok) {
          ra[j] = make_uint4(0u, 0u, 0u, 0u);
          rb[j] = make_uint4(0u, 0u, 0u, 0u);
        }
        ap[j] += kBK;
        bp[j] += kBK;
      }
    };
    auto sstore = [&](int stage) {
      char* base = smem + stage * kStageBytes + st_off;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        *reinterpret_cast<uint4*>(base + j * 64 * kRowBytes) = ra[j];
        *reinterpret_cast<uint4*>(base + kTile * kRowBytes + j * 64 * kRowBytes) = rb[j];
      }
    };
    auto compute = [&](int stage) {
      const char* base = smem + stage * kStageBytes;
#pragma unroll
      for (int ks = 0; ks < kBK / 16; ++ks) {
        const int slot = ((2 * ks + hi) ^ swz) * 16;
        V8 af[kTM], bf[kTN];
#pragma unroll
        for (int tm = 0; tm < kTM; ++tm)
          af[tm] = __builtin_bit_cast(
              V8, *reinterpret_cast<const uint4*>(base + a_frag + tm * 32 * kRowBytes + slot));
#pragma unroll
        for (int tn = 0; tn < kTN; ++tn)
          bf[tn] = __builtin_bit_cast(
              V8, *reinterpret_cast<const uint4*>(base + b_frag + tn * 32 * kRowBytes + slot));
#pragma unroll
        for (int tm = 0; tm < kTM; ++tm)
#pragma unroll
          for (int tn = 0; tn < kTN; ++tn) acc.c[tm][tn] = Op::mma(af[tm], bf[tn], acc.c[tm][tn]);
      }
    };

    const int nk = (k_end - k_begin + kBK - 1) / kBK;
    gload(k_begin);
    sstore(0);
    __syncthreads();
    for (int it = 0; it < nk; ++it) {
      const int cur = it & 1;
      const bool more = (it + 1) < nk;
      if (more) gload(k_begin + (it + 1) * kBK);
      compute(cur);
      if (more) sstore(cur ^ 1);
      __syncthreads();
    }
  }
};

// Direct-to-LDS engine: the operand tiles go global -> LDS with
// global_load_lds_dwordx4 (no VGPR staging, no ds_write), through a ring of
// four 32-wide K stages (4 x 32 KiB), so a tile is requested three K steps
// before it is consumed and HBM/L2 latency hides behind ~48 MFMAs per wave.
// Needs K (k_end - k_begin) to be a multiple of 32.
//
// A stage row is 64 bytes = four 16-byte chunks; chunk c of row r sits in slot
// c ^ ((r >> 2) & 3): the 16 lanes of one LDS read phase (16 rows, one chunk)
// then cover all 64 banks.  A wave's load instruction fills 1 KiB = 16 rows:
// lane i lands in row i/4, slot i%4, so it fetches logical chunk
// (i%4) ^ ((i>>4)&3) of that row.
//
// Ordering: loads are counted per wave by vmcnt and complete in order.  Before
// using tile k a wave waits until at most the loads of the (up to two) younger
// tiles are outstanding, then the workgroup barrier publishes every wave's
// part of tile k and retires stage (k-1)%4, which the loads of tile k+3 refill.
template <typename T_>
struct MfmaDirectEngine : MfmaTileLayout<T_> {
  using Base = MfmaTileLayout<T_>;
  using T = T_;
  using Op = typename Base::Op;
  using V8 = typename Base::V8;
  using Acc = typename Base::Acc;
  using Base::kTile;
  using Base::kTM;
  using Base::kTN;
  using Base::lane;
  using Base::wave;
  using Base::wm;
  using Base::wn;
  static constexpr int kBK = 32;
  static constexpr int kStages = 4;
  static constexpr int kRowBytes = kBK * 2;                  // 64
  static constexpr int kOperandBytes = kTile * kRowBytes;    // 16384
  static constexpr int kStageBytes = 2 * kOperandBytes;      // 32768
  static constexpr int kSmemBytes = kStages * kStageBytes;   // 131072

  static __device__ __forceinline__ void load_to_lds(unsigned lds_addr, const T* src) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(lds_addr), "v"(src)
                 : "memory", "m0");
  }

  __device__ __forceinline__ void mainloop(const T* __restrict__ A, int64_t lda, int a_row0,
                                           int a_rows, const T* __restrict__ B, int64_t ldb,
                                           int b_row0, int b_rows, int k_begin, int k_end,
                                           Acc& acc, char* smem) const {
    // loader role: this wave fills rows [32*wave, 32*wave+32) of both operands
    const int lrow = lane >> 2;
    const int chunk = (lane & 3) ^ ((lane >> 4) & 3);
    const T* ap[2];
    const T* bp[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int r = wave * 32 + j * 16 + lrow;
      const int ar = min(a_row0 + r, a_rows - 1);
      const int br = min(b_row0 + r, b_rows - 1);
      ap[j] = A + (int64_t)ar * lda + k_begin + chunk * 8;
      bp[j] = B + (int64_t)br * ldb + k_begin + chunk * 8;
    }
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    const unsigned fill =
        __builtin_amdgcn_readfirstlane(lds0 + (unsigned)(wave * 32 * kRowBytes));

    auto issue = [&](int stage) {
      const unsigned dst = fill + (unsigned)(stage * kStageBytes);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        load_to_lds(dst + j * 16 * kRowBytes, ap[j]);
        load_to_lds(dst + kOperandBytes + j * 16 * kRowBytes, bp[j]);
        ap[j] += kBK;
        bp[j] += kBK;
      }
    };

    // consumer role: fragment addresses of this wave's 128x64 sub-tile
    const int swz = (lane >> 2) & 3;
    const int hi = lane >> 5;
    const int a_frag = (wm * 128 + (lane & 31)) * kRowBytes;
    const int b_frag = kOperandBytes + (wn * 64 + (lane & 31)) * kRowBytes;

    // Fragments of one 16-wide K slice: 4 A blocks + 2 B blocks, 24 VGPRs.
    struct Frags { V8 a[kTM]; V8 b[kTN]; };
    auto read_slice = [&](Frags& f, int stage, int ks) {
      const char* base = smem + stage * kStageBytes;
      const int slot = ((2 * ks + hi) ^ swz) * 16;
#pragma unroll
      for (int tm = 0; tm < kTM; ++tm)
        f.a[tm] = __builtin_bit_cast(
            V8, *reinterpret_cast<const uint4*>(base + a_frag + tm * 32 * kRowBytes + slot));
#pragma unroll
      for (int tn = 0; tn < kTN; ++tn)
        f.b[tn] = __builtin_bit_cast(
            V8, *reinterpret_cast<const uint4*>(base + b_frag + tn * 32 * kRowBytes + slot));
    };
    auto mma_slice = [&](const Frags& f) {
#pragma unroll
      for (int tm = 0; tm < kTM; ++tm)
#pragma unroll
        for (int tn = 0; tn < kTN; ++tn) acc.c[tm][tn] = Op::mma(f.a[tm], f.b[tn], acc.c[tm][tn]);
    };

    // Software pipeline: the fragments of the next K slice are always in flight
    // while the MFMAs of the current one issue, also across K steps.  The
    // barrier that publishes tile k+1 sits in the middle of step k, after the
    // last LDS reads of tile k have been issued and before slice 0 of tile k+1
    // is read; the stage refilled after it, (k+3)%4 == (k-1)%4, was last read
    // in step k-1.
    const int nk = (k_end - k_begin) / kBK;
#pragma unroll
    for (int t = 0; t < kStages - 1; ++t)
      if (t < nk) issue(t);
    if (nk >= 3) {
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    } else if (nk == 2) {
      asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    Frags f0, f1;
    read_slice(f0, 0, 0);
    for (int k = 0; k + 1 < nk; ++k) {
      read_slice(f1, k & (kStages - 1), 1);
      __builtin_amdgcn_sched_barrier(0);   // keep the LDS reads ahead of the MFMA batch
      mma_slice(f0);
      // tile k+1 must have landed; tile k+2 (if any) may stay in flight
      if (k + 2 < nk) {
        asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      __syncthreads();
      if (k + kStages - 1 < nk) issue((k + kStages - 1) & (kStages - 1));
      read_slice(f0, (k + 1) & (kStages - 1), 0);
      __builtin_amdgcn_sched_barrier(0);
      mma_slice(f1);
    }
    read_slice(f1, (nk - 1) & (kStages - 1), 1);
    mma_slice(f0);
    mma_slice(f1);
    __syncthreads();
  }
};

// Four-wave direct-to-LDS engine (K multiple of 64): 256 threads, each wave a
// 128x128 sub-tile (4x4 MFMA blocks, 256 accumulator registers, one wave per
// SIMD), which halves the LDS fragment traffic per MFMA of the 8-wave layout.
// Two 64-wide K stages of 64 KiB; stage rows are 128 bytes, so every
// global_load_lds_dwordx4 wave instruction moves eight full 128-byte lines.
//
// Loads use the scalar-base form: the tile's base address and K position live
// in SGPRs, the per-lane byte offsets (row clamp and chunk swizzle folded in)
// are computed once per tile, so a load costs two scalar moves and no VALU work.
//
// Software pipeline of one wave (the only wave on its SIMD): the fragments of
// K slice s+1 are read while the 16 MFMAs of slice s issue; the next tile's
// 16 load instructions are spread over slices 0-2; the barrier that publishes
// the next tile sits in the middle of slice 3, so the first fragments of the
// next tile are in flight under the last 8 MFMAs of the current one.
template <typename T_>
struct MfmaDirect4Engine : MfmaTileLayout<T_, 2, 4> {
  using Base = MfmaTileLayout<T_, 2, 4>;
  using T = T_;
  using Op = typename Base::Op;
  using V8 = typename Base::V8;
  using Acc = typename Base::Acc;
  using Base::kTile;
  using Base::kTM;
  using Base::kTN;
  using Base::lane;
  using Base::wave;
  using Base::wm;
  using Base::wn;
  static constexpr int kBK = 64;
  static constexpr int kRowBytes = kBK * 2;                  // 128
  static constexpr int kOperandBytes = kTile * kRowBytes;    // 32768
  static constexpr int kStageBytes = 2 * kOperandBytes;      // 65536
  static constexpr int kSmemBytes = 2 * kStageBytes;         // 131072
  static constexpr int kLoadsPerOperand = 8;                 // per wave per tile

  static __device__ __forceinline__ void load_to_lds(unsigned lds_addr, unsigned byte_offset,
                                                     const char* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(byte_offset), "s"(base)
                 : "memory", "m0");
  }

  struct Frags { V8 a[kTM]; V8 b[kTN]; };

  __device__ __forceinline__ void mainloop(const T* __restrict__ A, int64_t lda, int a_row0,
                                           int a_rows, const T* __restrict__ B, int64_t ldb,
                                           int b_row0, int b_rows, int k_begin, int k_end,
                                           Acc& acc, char* smem) const {
    // loader role: this wave fills rows [64*wave, 64*wave+64) of both operands,
    // eight rows (1 KiB) per instruction; lane i lands in row i/8, slot i%8
    unsigned aoff[kLoadsPerOperand], boff[kLoadsPerOperand];
#pragma unroll
    for (int j = 0; j < kLoadsPerOperand; ++j) {
      const int r = wave * 64 + j * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ ((r >> 1) & 7);
      const int ar = min(a_row0 + r, a_rows - 1) - a_row0;
      const int br = min(b_row0 + r, b_rows - 1) - b_row0;
      aoff[j] = (unsigned)((int64_t)ar * lda * 2 + chunk * 16);
      boff[j] = (unsigned)((int64_t)br * ldb * 2 + chunk * 16);
    }
    const char* abase = reinterpret_cast<const char*>(A + (int64_t)a_row0 * lda + k_begin);
    const char* bbase = reinterpret_cast<const char*>(B + (int64_t)b_row0 * ldb + k_begin);
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    const unsigned fill =
        __builtin_amdgcn_readfirstlane(lds0 + (unsigned)(wave * 64 * kRowBytes));

    // load number q (0..15) of K tile `tile` into `stage`: even q -> operand A,
    // odd q -> operand B, instruction q/2 of this wave's eight per operand
    auto issue_one = [&](int stage, int tile, int q) {
      const unsigned dst = fill + (unsigned)(stage * kStageBytes) + (unsigned)((q >> 1) * 8 * kRowBytes);
#if defined(TLCE_EXP_SAMELINE)
      // every load re-reads this wave's first 1 KiB: stays in the vector L1
      if (q & 1) load_to_lds(dst + kOperandBytes, (unsigned)(lane * 16), bbase);
      else load_to_lds(dst, (unsigned)(lane * 16), abase);
#elif defined(TLCE_EXP_SAMETILE)
      // no K advance: the tile's first 64-wide slab again (L2 hits)
      if (q & 1) load_to_lds(dst + kOperandBytes, boff[q >> 1], bbase);
      else load_to_lds(dst, aoff[q >> 1], abase);
#else
      if (q & 1) {
        load_to_lds(dst + kOperandBytes, boff[q >> 1], bbase + (int64_t)tile * kRowBytes);
      } else {
        load_to_lds(dst, aoff[q >> 1], abase + (int64_t)tile * kRowBytes);
      }
#endif
    };

    // consumer role: fragment addresses of this wave's 128x128 sub-tile
    const int swz = (lane >> 1) & 7;
    const int hi = lane >> 5;
    const int a_frag = (wm * 128 + (lane & 31)) * kRowBytes;
    const int b_frag = kOperandBytes + (wn * 128 + (lane & 31)) * kRowBytes;

    auto read_a = [&](Frags& f, int stage, int ks, int tm) {
      const int slot = ((2 * ks + hi) ^ swz) * 16;
      f.a[tm] = __builtin_bit_cast(
          V8, *reinterpret_cast<const uint4*>(smem + stage * kStageBytes + a_frag +
                                              tm * 32 * kRowBytes + slot));
    };
    auto read_b = [&](Frags& f, int stage, int ks, int tn) {
      const int slot = ((2 * ks + hi) ^ swz) * 16;
      f.b[tn] = __builtin_bit_cast(
          V8, *reinterpret_cast<const uint4*>(smem + stage * kStageBytes + b_frag +
                                              tn * 32 * kRowBytes + slot));
    };
    // fragment r (0..7) of a slice in the order the next slice consumes them:
    // b0..b3 first (every MFMA group needs all four), then a0..a3
    auto read_frag = [&](Frags& f, int stage, int ks, int r) {
      if (r < 4) read_b(f, stage, ks, r); else read_a(f, stage, ks, r - 4);
    };

    // One K step = 64 MFMAs = 16 groups of 4 (slice sl = g/4, A block q = g%4,
    // B block t = 0..3).  A wave issues in order and an MFMA occupies its pipe
    // for 32 cycles, so everything else has to fit into those shadows a few
    // instructions at a time: after every MFMA at most one LDS fragment read
    // or one load instruction (three scalar + one vector instruction) follows.
    //   reads : the 8 fragments of the next slice, two per group (slots 0, 2);
    //           the next tile's slice 0 is read in the two groups after the
    //           barrier (5 + 3);
    //   loads : of the next tile's 16, six go out right after the barrier of
    //           the previous step, ten in groups 0..9 (slot 1) - the last one
    //           16 MFMAs (~500 cycles) before the barrier that waits for it.
    const int nk = (k_end - k_begin) / kBK;
    auto step = [&](int k, Frags& fa, Frags& fb, auto has_next_tag) {
      constexpr bool kHasNext = decltype(has_next_tag)::value;
      const int cur = k & 1;
      const int nxt = cur ^ 1;
      const bool more = (k + 2 < nk);
#pragma unroll
      for (int g = 0; g < 16; ++g) {
        const int sl = g >> 2;
        const int q = g & 3;
        Frags& fcur = (sl & 1) ? fb : fa;
        Frags& fnext = (sl & 1) ? fa : fb;
        const bool after_barrier = kHasNext && sl == 3 && q >= 2;
        if (kHasNext && sl == 3 && q == 2) {
          // tile k+1 is complete and visible from here on; stage `cur` is free
#ifndef TLCE_EXP_NOWAIT
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
#ifndef TLCE_EXP_NOBARRIER
          __syncthreads();
#endif
        }
#pragma unroll
        for (int t = 0; t < kTN; ++t) {
          acc.c[q][t] = Op::mma(fcur.a[q], fcur.b[t], acc.c[q][t]);
          if (sl < 3) {
            if (t == 0) read_frag(fnext, cur, sl + 1, 2 * q);
            if (t == 2) read_frag(fnext, cur, sl + 1, 2 * q + 1);
#ifndef TLCE_EXP_NOLOAD
            if (kHasNext && t == 1 && g < 10) issue_one(nxt, k + 1, 6 + g);
#endif
          } else if (after_barrier) {
            if (q == 2) {
              if (t == 0) { read_frag(fnext, nxt, 0, 0); read_frag(fnext, nxt, 0, 1); }
              else read_frag(fnext, nxt, 0, t + 1);
            } else {
              if (t < 3) read_frag(fnext, nxt, 0, 5 + t);
            }
#ifndef TLCE_EXP_NOLOAD
            if (t >= 1 && more) issue_one(cur, k + 2, (q - 2) * 3 + (t - 1));
#endif
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    };

#pragma unroll
    for (int q = 0; q < 16; ++q) issue_one(0, 0, q);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (nk > 1) {
#pragma unroll
      for (int q = 0; q < 6; ++q) issue_one(1, 1, q);
    }
    Frags f0, f1;
#pragma unroll
    for (int r = 0; r < 8; ++r) read_frag(f0, 0, 0, r);
    // a step consumes slices from f0,f1,f0,f1 and leaves the next tile's slice 0 in f0
    for (int k = 0; k + 1 < nk; ++k) step(k, f0, f1, std::true_type{});
    step(nk - 1, f0, f1, std::false_type{});
    __syncthreads();
  }
};

}  // namespace tlce
