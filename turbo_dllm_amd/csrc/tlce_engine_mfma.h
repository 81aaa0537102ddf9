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
  static constexpr bool kPrecise = false;    // hardware exp / rcp approximations in the epilogues
  static_assert(kWavesN * kTN * 32 == kTile, "waves must tile the 256 B rows");

  struct Acc { f32x16_t c[kTM][kTN]; };

  int lane, wave, wm, wn;

  __device__ __forceinline__ MfmaTileLayout() {
    lane = threadIdx.x & 63;
    wave = threadIdx.x >> 6;
    wm = wave / kWavesN;
    wn = wave % kWavesN;
  }

  // An empty asm that "modifies" the lane index: values derived from it before
  // this point are not reused after it, so a kernel that loops over tiles can
  // keep the compiler from hoisting (and then spilling) per-lane addresses.
  __device__ __forceinline__ void forget_lane_invariants() { asm volatile("" : "+v"(lane)); }

  __device__ __forceinline__ int col(int j) const {
    return wn * (kTN * 32) + j * 32 + (lane & 31);
  }
  // The tile columns that have owned index j in some thread: number t of them.
  static constexpr int kTokensPerIndex = kWavesN * 32;
  static __device__ __forceinline__ int token_of_index(int j, int t) {
    return (t >> 5) * (kTN * 32) + j * 32 + (t & 31);
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
  // Sum over the lanes of this wave that hold the same tile column (lanes l and
  // l ^ 32 hold different rows of it); other waves keep their own sums.
  __device__ __forceinline__ float reduce_over_rows_in_wave(float v) const {
    return v + __shfl_xor(v, 32, 64);
  }
  __device__ __forceinline__ bool row_leader() const { return lane < 32; }
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
  static constexpr bool kHasKMajor = false;

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

  // acc = A * B^T (same operands as mainloop).
  __device__ __forceinline__ void mainloop_set(const T* __restrict__ A, int64_t lda, int a_row0,
                                               int a_rows, const T* __restrict__ B, int64_t ldb,
                                               int b_row0, int b_rows, int k_begin, int k_end,
                                               Acc& acc, char* smem) const {
    Base::zero(acc);
    mainloop(A, lda, a_row0, a_rows, B, ldb, b_row0, b_rows, k_begin, k_end, acc, smem);
  }
};

// Four-wave direct-to-LDS engine (K multiple of 64): 256 threads, each wave a
// 128x128 sub-tile (4x4 MFMA blocks, 256 accumulator registers, one wave per
// SIMD).  Operands go global -> LDS with global_load_lds_dwordx4 (no VGPR
// staging, no ds_write) into two 64-wide K stages of 64 KiB; every wave load
// instruction moves 1 KiB made of full 128-byte (or 512-byte) row segments.
//
// Either operand can be stored in one of two ways:
//   K-contiguous  X[row][k]  (the projection's hidden and weight rows, the
//                 logit-gradient panel as seen by grad_hidden);
//   K-major       X[k][row]  (weight as seen by grad_hidden, hidden and the
//                 logit-gradient panel as seen by grad_weight), read from LDS
//                 with the transposing ds_read_b64_tr_b16, so no transposed
//                 copy of any matrix is ever made in HBM.
//
// LDS layouts of one operand stage (32 KiB):
//   K-contiguous: 256 rows x 128 B; 16-byte chunk c of row r in slot
//                 c ^ ((r >> 1) & 7).
//   K-major:      64 K rows x 512 B; 16-byte chunk c of K row k in slot
//                 c ^ (4 * (k & 3)): the four K rows x 64 bytes that half a
//                 wave reads at once then fall into four different quarters
//                 of the banks, and 64-byte runs stay contiguous.
// ds_read_b64_tr_b16 works on groups of 16 lanes: lane i of a group addresses
// 4 consecutive elements, and lane l receives element l%4 of the chunks of
// lanes l/4, 4 + l/4, 8 + l/4, 12 + l/4.  With lane i addressing K row i/4,
// columns 4*(i%4).. of a 4 x 16 block, lane l ends up with 4 consecutive K
// values of column l: half an MFMA fragment.
//
// Loads use the scalar-base form: tile base and K position live in SGPRs, the
// per-lane byte offsets (row clamp and slot swizzle folded in) are computed
// once per tile, so a load costs three scalar instructions and no VALU work.
//
// Software pipeline of one wave (the only wave on its SIMD; it issues in
// order and an MFMA occupies its pipe for 32 cycles): one K step = 64 MFMAs
// = 16 groups of 4 (slice sl = g/4, A block q = g%4, B block t).  After every
// MFMA at most one fragment read and one load instruction follow.
//   reads : the fragments of the next slice, spread over the groups of the
//           current one; slice 0 of the next tile is read in the two groups
//           after the barrier, which sits in the middle of slice 3;
//   loads : of the next tile's 16, six go out right after the barrier of the
//           previous step, ten in the first groups of the step (two per group
//           in groups 0..4, or one per group in groups 0..9).
template <typename T>
struct Operand {
  const T* ptr;   // matrix base
  int64_t ld;     // elements between consecutive stored rows
  int row0;       // first tile row (K-contiguous) or first tile column (K-major)
  int rows;       // valid rows / columns of the matrix; accesses beyond are clamped
};

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
  static constexpr int kOperandBytes = kTile * kBK * 2;      // 32768
  static constexpr int kStageBytes = 2 * kOperandBytes;      // 65536
  static constexpr int kSmemBytes = 2 * kStageBytes;         // 131072
  static constexpr int kLoads = 8;                           // per wave, operand and K tile
  static constexpr bool kHasKMajor = true;

  typedef short v4s_t __attribute__((ext_vector_type(4)));
  typedef short v8s_t __attribute__((ext_vector_type(8)));

  static __device__ __forceinline__ void load_to_lds(unsigned lds_addr, unsigned byte_offset,
                                                     const char* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(byte_offset), "s"(base)
                 : "memory", "m0");
  }

  // Loader state of one operand: where this wave's eight 1 KiB pieces of a K
  // tile come from and where they land.
  struct Loader {
    unsigned off[kLoads];   // per-lane byte offsets from the K tile's base
    unsigned fill;          // LDS address of this wave's first piece in stage 0
    const char* next;       // base address of the next K tile to request
    int64_t step;           // bytes between consecutive K tiles
  };

  template <bool kKMajor>
  __device__ __forceinline__ Loader make_loader(const Operand<T>& x, int k_begin, unsigned lds_op,
                                                bool second_operand) const {
    Loader ld;
    (void)second_operand;
    if (!kKMajor) {
      // this wave fills tile rows [64w, 64w+64), eight rows per instruction
#pragma unroll
      for (int j = 0; j < kLoads; ++j) {
        const int r = wave * 64 + j * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((r >> 1) & 7);
        const int rr = min(x.row0 + r, x.rows - 1) - x.row0;
        ld.off[j] = (unsigned)((int64_t)rr * x.ld * 2 + chunk * 16);
      }
      ld.fill = __builtin_amdgcn_readfirstlane(lds_op + (unsigned)(wave * 64 * 128));
      ld.next = reinterpret_cast<const char*>(x.ptr + (int64_t)x.row0 * x.ld + k_begin);
      ld.step = kBK * 2;
    } else {
      // this wave fills K rows [16w, 16w+16) of the slab, two rows per instruction
      const int last_chunk = x.rows / 8 - 1 - x.row0 / 8;   // relative to the tile
#pragma unroll
      for (int j = 0; j < kLoads; ++j) {
        const int kr = wave * 16 + j * 2 + (lane >> 5);
        const int swz = 4 * (kr & 3);
        const int chunk = min((lane & 31) ^ swz, last_chunk);
        ld.off[j] = (unsigned)((int64_t)kr * x.ld * 2 + chunk * 16);
      }
      ld.fill = __builtin_amdgcn_readfirstlane(lds_op + (unsigned)(wave * 16 * 512));
      ld.next = reinterpret_cast<const char*>(x.ptr + (int64_t)k_begin * x.ld + x.row0);
      ld.step = (int64_t)kBK * x.ld * 2;
    }
    return ld;
  }

  // Fragment addressing of one operand for this lane.
  struct Reader {
    int base[4];   // LDS byte offset of block 0..3 within the operand stage
  };

  template <bool kKMajor>
  __device__ __forceinline__ Reader make_reader(int wave_block) const {
    Reader rd;
    if (!kKMajor) {
      const int swz = (lane >> 1) & 7;
      (void)swz;
#pragma unroll
      for (int b = 0; b < 4; ++b) rd.base[b] = (wave_block * 128 + b * 32 + (lane & 31)) * 128;
    } else {
      const int g = lane >> 4;          // 16-lane group
      const int i = lane & 15;
      const int hi = g >> 1;
      const int swz = 4 * (i >> 2);      // = 4 * (K row & 3)
      const int kr = 8 * hi + (i >> 2);  // K row within a 16-wide slice, first half
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int col = wave_block * 128 + b * 32 + 16 * (g & 1) + 4 * (i & 3);
        const int slot = (col >> 3) ^ swz;
        rd.base[b] = kr * 512 + slot * 16 + (col & 7) * 2;
      }
    }
    return rd;
  }

  template <bool kKMajor>
  __device__ __forceinline__ V8 read_frag(const char* op_stage, const Reader& rd, int ks,
                                          int b) const {
    if (!kKMajor) {
      const int slot = ((2 * ks + (lane >> 5)) ^ ((lane >> 1) & 7)) * 16;
      return __builtin_bit_cast(V8, *reinterpret_cast<const uint4*>(op_stage + rd.base[b] + slot));
    } else {
      typedef __attribute__((address_space(3))) v4s_t* lds_v4s_ptr;
      const char* p0 = op_stage + rd.base[b] + ks * 16 * 512;
      const v4s_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (lds_v4s_ptr)(uintptr_t)(unsigned)(uintptr_t)p0);
      const v4s_t hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (lds_v4s_ptr)(uintptr_t)(unsigned)(uintptr_t)(p0 + 4 * 512));
      v8s_t v;
      v[0] = lo[0]; v[1] = lo[1]; v[2] = lo[2]; v[3] = lo[3];
      v[4] = hi4[0]; v[5] = hi4[1]; v[6] = hi4[2]; v[7] = hi4[3];
      return __builtin_bit_cast(V8, v);
    }
  }

  struct Frags { V8 a[kTM]; V8 b[kTN]; };

  // acc += A-tile * B-tile^T over K in [k_begin, k_end), a multiple of 64 wide.
  // K-contiguous operand: tile rows row0 .. row0+256 of x (rows clamped to
  // x.rows - 1).  K-major operand: tile columns row0 .. row0+256 of x (16-byte
  // column chunks clamped to the last valid one; x.rows is a multiple of 8);
  // all K rows in [k_begin, k_end) must exist.
  // kOverwrite: acc = A-tile * B-tile^T instead (the incoming acc is ignored: the
  // first 16 MFMAs take a zero constant as their addend, which saves zeroing
  // 256 accumulator registers per tile).
  template <bool kAKMajor, bool kBKMajor, bool kOverwrite = false>
  __device__ __forceinline__ void mainloop_ex(const Operand<T>& A, const Operand<T>& B,
                                              int k_begin, int k_end, Acc& acc,
                                              char* smem) const {
    const unsigned lds0 = (unsigned)(uintptr_t)smem;
    Loader la = make_loader<kAKMajor>(A, k_begin, lds0, false);
    Loader lb = make_loader<kBKMajor>(B, k_begin, lds0 + kOperandBytes, true);
    const Reader ra = make_reader<kAKMajor>(wm);
    const Reader rb = make_reader<kBKMajor>(wn);

    // load number q (0..15) of the next K tile into `stage`, `ahead` K tiles
    // past the loaders' current position: even q -> A, odd q -> B
    auto issue_one = [&](int stage, int ahead, int q) {
      const unsigned s_off = (unsigned)(stage * kStageBytes) + (unsigned)((q >> 1) * 1024);
      if (q & 1) load_to_lds(lb.fill + s_off, lb.off[q >> 1], lb.next + ahead * lb.step);
      else load_to_lds(la.fill + s_off, la.off[q >> 1], la.next + ahead * la.step);
    };
    // fragment r (0..7) of a slice in the order the next slice consumes them:
    // b0..b3 first (every MFMA group needs all four), then a0..a3
    auto read_one = [&](Frags& f, int stage, int ks, int r) {
      const char* st = smem + stage * kStageBytes;
      if (r < 4) f.b[r] = read_frag<kBKMajor>(st + kOperandBytes, rb, ks, r);
      else f.a[r - 4] = read_frag<kAKMajor>(st, ra, ks, r - 4);
    };

    const int nk = (k_end - k_begin) / kBK;
    constexpr bool kLoadsInPairs = !(kAKMajor && !kBKMajor);
    auto step = [&](int k, Frags& fa, Frags& fb, auto has_next_tag, auto first_tag) {
      constexpr bool kHasNext = decltype(has_next_tag)::value;
      constexpr bool kFirst = decltype(first_tag)::value;   // first step of an overwriting loop
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
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          __syncthreads();
          la.next += la.step;
          lb.next += lb.step;
        }
#pragma unroll
        for (int t = 0; t < kTN; ++t) {
          if (kFirst && sl == 0) {
            const f32x16_t zero = {};
            acc.c[q][t] = Op::mma(fcur.a[q], fcur.b[t], zero);
          } else {
            acc.c[q][t] = Op::mma(fcur.a[q], fcur.b[t], acc.c[q][t]);
          }
          if (sl < 3) {
            if (t == 0) read_one(fnext, cur, sl + 1, 2 * q);
            if (t == 2) read_one(fnext, cur, sl + 1, 2 * q + 1);
            if (kHasNext) {
              // loads 6..15 of the next tile: two per group in groups 0..4 (measured
              // about 1 % faster), except for the K-major x K-contiguous pairing,
              // which does better with one per group in groups 0..9
              if (kLoadsInPairs) {
                if ((t == 1 || t == 3) && g < 5) issue_one(nxt, 0, 6 + 2 * g + (t == 3));
              } else {
                if (t == 1 && g < 10) issue_one(nxt, 0, 6 + g);
              }
            }
          } else if (after_barrier) {
            if (q == 2) {
              if (t == 0) { read_one(fnext, nxt, 0, 0); read_one(fnext, nxt, 0, 1); }
              else read_one(fnext, nxt, 0, t + 1);
            } else {
              if (t < 3) read_one(fnext, nxt, 0, 5 + t);
            }
            if (t >= 1 && more) issue_one(cur, 0, (q - 2) * 3 + (t - 1));
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    };

    // tile 0 entirely, then the first six loads of tile 1 (la.next / lb.next
    // always point at the tile whose loads are being issued)
#pragma unroll
    for (int q = 0; q < 16; ++q) issue_one(0, 0, q);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    la.next += la.step;
    lb.next += lb.step;
    if (nk > 1) {
#pragma unroll
      for (int q = 0; q < 6; ++q) issue_one(1, 0, q);
    }
    Frags f0, f1;
#pragma unroll
    for (int r = 0; r < 8; ++r) read_one(f0, 0, 0, r);
    // a step consumes slices from f0,f1,f0,f1 and leaves the next tile's slice 0 in f0
    if constexpr (kOverwrite) {
      if (nk > 1) {
        step(0, f0, f1, std::true_type{}, std::true_type{});
        for (int k = 1; k + 1 < nk; ++k) step(k, f0, f1, std::true_type{}, std::false_type{});
        step(nk - 1, f0, f1, std::false_type{}, std::false_type{});
      } else {
        step(0, f0, f1, std::false_type{}, std::true_type{});
      }
    } else {
      for (int k = 0; k + 1 < nk; ++k) step(k, f0, f1, std::true_type{}, std::false_type{});
      step(nk - 1, f0, f1, std::false_type{}, std::false_type{});
    }
    __syncthreads();
  }

  __device__ __forceinline__ void mainloop(const T* __restrict__ A, int64_t lda, int a_row0,
                                           int a_rows, const T* __restrict__ B, int64_t ldb,
                                           int b_row0, int b_rows, int k_begin, int k_end,
                                           Acc& acc, char* smem) const {
    const Operand<T> a = {A, lda, a_row0, a_rows};
    const Operand<T> b = {B, ldb, b_row0, b_rows};
    mainloop_ex<false, false>(a, b, k_begin, k_end, acc, smem);
  }

  // acc = A * B^T over a non-empty K range (same operands as mainloop).
  __device__ __forceinline__ void mainloop_set(const T* __restrict__ A, int64_t lda, int a_row0,
                                               int a_rows, const T* __restrict__ B, int64_t ldb,
                                               int b_row0, int b_rows, int k_begin, int k_end,
                                               Acc& acc, char* smem) const {
    const Operand<T> a = {A, lda, a_row0, a_rows};
    const Operand<T> b = {B, ldb, b_row0, b_rows};
    mainloop_ex<false, false, true>(a, b, k_begin, k_end, acc, smem);
  }
};

}  // namespace tlce
