// Shared MFMA mainloop for gfx950 (MI355X): C[m][n] = sum_k A[m][k] * B[n][k].
//
// Both operands are K-contiguous in memory ("NT" GEMM).  One workgroup owns a BM x BN tile of C;
// its waves are arranged WAVES_M x WAVES_N and each wave owns (BM/WAVES_M) x (BN/WAVES_N) as
// 32x32 MFMA blocks.  K is streamed in slabs of BKB bytes per row through an LDS ring that is filled
// by direct global->LDS loads (16 bytes per lane, no VGPR staging): NSTAGE whole slabs, or NSTAGE half
// slabs (one operand each) in the split layout described at GemmCfg.
//
// LDS layout of one operand slab: row-major, BKB bytes per row, the 16-byte chunk index of every
// row XOR-ed with a function of the row number so that the 16-byte MFMA operand reads of 32
// consecutive rows spread over all banks.
//
// Accumulator layout of one 32x32 block (v_mfma_f32_32x32x*): lane l holds column n = l % 32 and
// the 16 rows m = 8*(r/4) + 4*(l/32) + (r%4), r = 0..15.  Epilogues rely on this: everything a lane
// holds belongs to ONE column n per block, so per-column reductions over m are lane-local.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tile_map.hpp"

namespace lce {

typedef __bf16 bf16_t;
typedef bf16_t bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16_t;
typedef f16_t f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef short i16x4_t __attribute__((ext_vector_type(4)));

#define LCE_DEV __device__ __forceinline__

typedef const void __attribute__((address_space(1))) * gptr_t;
typedef void __attribute__((address_space(3))) * lptr_t;

// transposing LDS read of four 16-bit elements per lane (see GemmCore::init_tn for the lane mapping).
// Issued as inline assembly with a 32-bit LDS address: through the builtin the compiler waits for ALL
// outstanding global->LDS loads before every such read (it cannot tell that they do not alias), which
// serialises the ring.  The price: the compiler does not know that the result arrives later, so the
// consumer places the lgkmcnt waits itself (GemmCore::substep).
template <int OFF>
LCE_DEV u32x2_t tr_read(uint32_t lds_addr) {
  u32x2_t v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(lds_addr), "n"(OFF));
  return v;
}

// plain 16-byte LDS read as inline assembly, for loops that place their lgkmcnt waits by hand
template <int OFF>
LCE_DEV u32x4_t lds_read16(uint32_t lds_addr) {
  u32x4_t v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(lds_addr), "n"(OFF));
  return v;
}

template <typename T>
struct Mma;

// one 16-byte chunk (8 bf16 along K) per lane of A and of B -> one 32x32x16 MFMA
template <>
struct Mma<bf16_t> {
  static LCE_DEV void run(f32x16_t& acc, const u32x4_t& a, const u32x4_t& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                  acc, 0, 0, 0);
  }
};

// the same with IEEE half-precision operands
template <>
struct Mma<f16_t> {
  static LCE_DEV void run(f32x16_t& acc, const u32x4_t& a, const u32x4_t& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b),
                                                 acc, 0, 0, 0);
  }
};

// one 16-byte chunk (4 fp32 along K) per lane -> four 32x32x2 MFMAs (true fp32 multiply-add)
template <>
struct Mma<float> {
  static LCE_DEV void run(f32x16_t& acc, const u32x4_t& a, const u32x4_t& b) {
    const f32x4_t af = __builtin_bit_cast(f32x4_t, a);
    const f32x4_t bf = __builtin_bit_cast(f32x4_t, b);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[i], acc, 0, 0, 0);
  }
};

// SPLIT_ (needs BM == BN): the ring holds NSTAGE_ HALF stages, one operand's slab each, in the order
// A0 B0 A1 B1 A2 ...; with five of them a barrier still hands back one A and one B half per slab, but
// the odd half lets the A operand of the slab after next stay in flight ACROSS the barrier, so half of
// the loads get two barrier periods to land instead of one.
// TRANS_ (split ring, 16-bit elements only): 1 = both operands are stored K-major in memory, A[k][m] and B[k][n]
// (C = A^T . B); 2 = only B is (C = A . B with A[m][k], B[k][n]).  A ring slot of a K-major operand holds 64 k-rows
// of 256 columns and its MFMA operand fragments are fetched with the transposing LDS read (ds_read_b64_tr_b16,
// two per fragment).
template <typename TIN_, int BM_, int BN_, int BKB_, int NSTAGE_, int WAVES_M_, int WAVES_N_, int SPLIT_ = 0, int TRANS_ = 0>
struct GemmCfg {
  typedef TIN_ TIN;
  static constexpr bool CORE16 = false;  // (the four-wave 16x16x32 mainloop is GemmCfg16, gemm_core16.hpp)
  static constexpr int BM = BM_, BN = BN_, BKB = BKB_, NSTAGE = NSTAGE_;
  static constexpr int SPLIT = SPLIT_;  // 0 whole stages; 1 split ring, A operand early; 2 split ring, B operand early
  static constexpr int TRANS = TRANS_;
  static constexpr bool TRANS_A = TRANS_ == 1, TRANS_B = TRANS_ != 0;
  static_assert(TRANS_ == 0 || (SPLIT_ != 0 && sizeof(TIN_) == 2 && BM_ == 256 && BN_ == 256 && BKB_ == 128), "transposed operands: split ring, 16-bit, 256x256");
  static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr int NW = WAVES_M * WAVES_N;
  static constexpr int NTHREADS = NW * 64;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int FM = WM / 32, FN = WN / 32;
  static constexpr int BK = BKB / (int)sizeof(TIN);  // K elements per slab
  static constexpr int CH = BKB / 16;                 // 16-byte chunks per row
  static constexpr int KSUB = CH / 2;                 // MFMA k-substeps per slab (2 chunks each)
  static constexpr int ROWS_PER_LOAD = 64 / CH;       // rows one wave-wide 16B/lane load covers
  static constexpr int A_LOADS = BM / ROWS_PER_LOAD / NW;
  static constexpr int B_LOADS = BN / ROWS_PER_LOAD / NW;
  static constexpr int A_BYTES = BM * BKB, B_BYTES = BN * BKB;
  static constexpr int STAGE_BYTES = SPLIT ? A_BYTES : A_BYTES + B_BYTES;  // one ring slot
  static constexpr int LDS_BYTES = STAGE_BYTES * NSTAGE;
  static_assert(!SPLIT || (BM == BN && NSTAGE == 5), "split ring: equal halves, five slots");
  static_assert(BKB == 128 || BKB == 64, "slab rows are 64 or 128 bytes");
  static_assert(BM % (ROWS_PER_LOAD * NW) == 0 && BN % (ROWS_PER_LOAD * NW) == 0, "tile/loader mismatch");
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be whole 32x32 blocks");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
  static_assert(KSUB % 2 == 0 && NSTAGE >= 2 && NSTAGE <= 5, "pipeline shape");

  // XOR pattern applied to the chunk index of a row (uses row bits 0..3 only, so it is the same
  // for rows that differ by a multiple of 32).
  static LCE_DEV int swz(int row) {
    if constexpr (CH == 8) return (row ^ ((row >> 3) & 1)) & 7;
    else return ((row >> 1) ^ (row >> 3)) & 3;
  }
};

// Per-lane addressing state for streaming one operand slab (A or B) from global memory.
template <int NLOADS>
struct SlabLoader {
  uint32_t voff[NLOADS];  // byte offset of this lane's 16-byte chunk relative to the tile's first row, k = 0
};

template <typename Cfg>
struct GemmCore {
  typedef typename Cfg::TIN TIN;

  const char* a_base;  // &A[m0][0]
  const char* b_base;  // &B[n0][0]
  SlabLoader<Cfg::A_LOADS> la;
  SlabLoader<Cfg::B_LOADS> lb;
  int wave, lane, wave_m, wave_n;
  uint32_t a_rd, b_rd;  // LDS byte offsets (within a stage) of this lane's operand rows, swizzle folded in
  int64_t a_slab, b_slab;  // bytes from one K slab to the next in memory (BKB, or 64 rows for K-major operands)
  // mixed mode (only B K-major): memory row inside a slab and chunk offset of each load, rows clamped per slab
  int b_row[Cfg::B_LOADS];
  int64_t b_ld_bytes, b_kvalid;

  // rows beyond the matrix are clamped to its last row (their results are discarded by the epilogue).
  // With `b_rows` given, row n of the B operand is B[b_rows[n]] (a gather; B is then the matrix's first
  // row and every row's byte offset must fit 32 bits).
  LCE_DEV void init(const TIN* A, int64_t lda, int64_t m0, int64_t M, const TIN* B, int64_t ldb, int64_t n0,
                    int64_t N, const int* b_rows = nullptr) {
    wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    lane = threadIdx.x & 63;
    wave_m = wave / Cfg::WAVES_N;
    wave_n = wave % Cfg::WAVES_N;
    a_base = reinterpret_cast<const char*>(A + m0 * lda);
    b_base = reinterpret_cast<const char*>(b_rows ? B : B + n0 * ldb);
    a_slab = b_slab = Cfg::BKB;
    const int rows_a = (int)((M - m0) < (int64_t)Cfg::BM ? (M - m0) : (int64_t)Cfg::BM);
    const int rows_b = (int)((N - n0) < (int64_t)Cfg::BN ? (N - n0) : (int64_t)Cfg::BN);
    const int lr = lane / Cfg::CH, pc = lane % Cfg::CH;
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j) {
      const int row = (j * Cfg::NW + wave) * Cfg::ROWS_PER_LOAD + lr;
      const int c = pc ^ Cfg::swz(row);
      const int crow = row < rows_a ? row : rows_a - 1;
      la.voff[j] = (uint32_t)((int64_t)crow * lda * (int64_t)sizeof(TIN)) + (uint32_t)(c * 16);
    }
#pragma unroll
    for (int j = 0; j < Cfg::B_LOADS; ++j) {
      const int row = (j * Cfg::NW + wave) * Cfg::ROWS_PER_LOAD + lr;
      const int c = pc ^ Cfg::swz(row);
      const int crow = row < rows_b ? row : rows_b - 1;
      const int64_t grow = b_rows ? (int64_t)b_rows[n0 + crow] : (int64_t)crow;
      lb.voff[j] = (uint32_t)(grow * ldb * (int64_t)sizeof(TIN)) + (uint32_t)(c * 16);
    }
    const int r32 = lane & 31, hh = lane >> 5;
    const int x = (hh ^ Cfg::swz(r32)) * 16;
    a_rd = (uint32_t)((wave_m * Cfg::WM + r32) * Cfg::BKB + x);
    b_rd = (uint32_t)((Cfg::SPLIT ? 0 : Cfg::A_BYTES) + (wave_n * Cfg::WN + r32) * Cfg::BKB + x);
  }

  // K-major operands: A[k][m0 + 0..BM), B[k][n0 + 0..BN), row strides lda / ldb (elements).  A ring slot
  // holds 64 k-rows x 512 bytes; the 16-byte chunk c of row r sits at chunk position c ^ ((r % 4) * 4), so the
  // four rows that one transposing read touches fall into different banks.
  LCE_DEV void init_tn(const TIN* A, int64_t lda, int64_t m0, const TIN* B, int64_t ldb, int64_t n0) {
    wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    lane = threadIdx.x & 63;
    wave_m = wave / Cfg::WAVES_N;
    wave_n = wave % Cfg::WAVES_N;
    a_base = reinterpret_cast<const char*>(A + m0);
    b_base = reinterpret_cast<const char*>(B + n0);
    a_slab = 64 * lda * (int64_t)sizeof(TIN);
    b_slab = 64 * ldb * (int64_t)sizeof(TIN);
#pragma unroll
    for (int j = 0; j < Cfg::A_LOADS; ++j) {
      const int row = (j * Cfg::NW + wave) * 2 + lane / 32;  // one wave-wide load covers two 512-byte rows
      const int c = (lane % 32) ^ ((row % 4) * 4);
      la.voff[j] = (uint32_t)((int64_t)row * lda * (int64_t)sizeof(TIN)) + (uint32_t)(c * 16);
      lb.voff[j] = (uint32_t)((int64_t)row * ldb * (int64_t)sizeof(TIN)) + (uint32_t)(c * 16);
    }
    // transposing read: in each group of 16 lanes, lane 4e + q supplies the address of X[k0 + e][x0 + 4q ..]
    // and lane i receives X[k0 .. k0+3][x0 + i]; groups 0/1 take the two 16-column halves of a 32-column
    // block, groups 2/3 the upper half (k + 8) of the 16 k-values of a substep
    const int g = lane / 16, e = (lane % 16) / 4, q = lane % 4;
    const int ma = wave_m * Cfg::WM + 16 * (g % 2) + 4 * q, nb = wave_n * Cfg::WN + 16 * (g % 2) + 4 * q;
    const uint32_t row_off = (uint32_t)((8 * (g / 2) + e) * 512);
    a_rd = row_off + (uint32_t)((((ma / 8) ^ (4 * e)) * 16) + (ma % 8) * 2);
    b_rd = row_off + (uint32_t)((((nb / 8) ^ (4 * e)) * 16) + (nb % 8) * 2);
  }

  // A[m][k] row-major as in init(); B[k][n0 + 0..BN) K-major with row stride ldb.  LDS row r of a slab is memory row
  // perm(r) of the slab (perm: a permutation of 0..63, the order in which A's columns were stored), and memory rows at
  // or beyond `kvalid` are replaced by row kvalid-1 (A is zero there).  B has `ncols` columns from n0 on.
  template <typename Perm>
  LCE_DEV void init_mixed(const TIN* A, int64_t lda, int64_t m0, int64_t M, const TIN* B, int64_t ldb, int64_t n0, int64_t ncols,
                          int64_t kvalid, Perm perm) {
    init(A, lda, m0, M, B, ldb, 0, Cfg::BN);
    b_base = reinterpret_cast<const char*>(B + n0);
    b_slab = 64;  // rows per slab (the byte offset is formed per load, see dma_half)
    b_ld_bytes = ldb * (int64_t)sizeof(TIN);
    b_kvalid = kvalid;
#pragma unroll
    for (int j = 0; j < Cfg::B_LOADS; ++j) {
      const int row = (j * Cfg::NW + wave) * 2 + lane / 32;
      const int c = (lane % 32) ^ ((row % 4) * 4);
      b_row[j] = (int)perm(row);
      // columns beyond the matrix (last N tile of a width that is no multiple of the tile) are fetched from the
      // row's first chunk instead: in bounds, and they only feed output columns that are discarded
      lb.voff[j] = (uint32_t)(((int64_t)c * (16 / (int)sizeof(TIN)) < ncols ? c : 0) * 16);
    }
    const int g = lane / 16, e = (lane % 16) / 4, q = lane % 4;
    const int nb = wave_n * Cfg::WN + 16 * (g % 2) + 4 * q;
    b_rd = (uint32_t)((8 * (g / 2) + e) * 512) + (uint32_t)((((nb / 8) ^ (4 * e)) * 16) + (nb % 8) * 2);
  }

  static constexpr int PER = Cfg::A_LOADS + Cfg::B_LOADS;  // wave-wide DMA loads per slab
  static constexpr int N_READS = Cfg::FM + Cfg::FN;       // LDS operand reads per k-substep
  static constexpr int N_BLK = Cfg::FM * Cfg::FN;         // 32x32 blocks per wave

  // one of the PER wave-wide 16-byte-per-lane global->LDS loads of a slab (A loads first)
  LCE_DEV void dma_one(char* lds, int stage, int64_t kbyte, int idx) const {
    char* sa = lds + stage * Cfg::STAGE_BYTES;
    if (idx < Cfg::A_LOADS) {
      __builtin_amdgcn_global_load_lds((gptr_t)(a_base + kbyte + la.voff[idx]),
                                       (lptr_t)(sa + (idx * Cfg::NW + wave) * 1024), 16, 0, 0);
    } else {
      const int j = idx - Cfg::A_LOADS;
      __builtin_amdgcn_global_load_lds((gptr_t)(b_base + kbyte + lb.voff[j]),
                                       (lptr_t)(sa + Cfg::A_BYTES + (j * Cfg::NW + wave) * 1024), 16, 0, 0);
    }
  }
  // split ring: load j of one operand's half slab into ring slot `slot`
  LCE_DEV void dma_half(char* lds, int slot, int64_t kbyte, bool is_b, int j) const {
    char* sa = lds + slot * Cfg::STAGE_BYTES + (j * Cfg::NW + wave) * 1024;
    // kbyte counts BKB bytes per slab; K-major operands advance by 64 rows per slab instead
    if (is_b) {
      int64_t off = kbyte;
      if constexpr (Cfg::TRANS == 1) off = (kbyte / Cfg::BKB) * b_slab;
      if constexpr (Cfg::TRANS == 2) {
        int64_t row = (kbyte / Cfg::BKB) * 64 + b_row[j];
        row = row < b_kvalid ? row : b_kvalid - 1;
        off = row * b_ld_bytes;
      }
      __builtin_amdgcn_global_load_lds((gptr_t)(b_base + off + lb.voff[j]), (lptr_t)sa, 16, 0, 0);
    } else {
      const int64_t off = Cfg::TRANS_A ? (kbyte / Cfg::BKB) * a_slab : kbyte;
      __builtin_amdgcn_global_load_lds((gptr_t)(a_base + off + la.voff[j]), (lptr_t)sa, 16, 0, 0);
    }
  }
  LCE_DEV void issue_slab(char* lds, int stage, int64_t kbyte) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) dma_one(lds, stage, kbyte, i);
  }

  // one of the N_READS operand reads of k-substep kk, in the order a0, b0..b(FN-1), a1..a(FM-1)
  // (sa, sb: the ring slots holding the A and the B operand; the same pointer unless the ring is split)
  LCE_DEV void read_one(const char* sa, const char* sb, int kk, int idx, u32x4_t (&af)[Cfg::FM], u32x4_t (&bf)[Cfg::FN]) const {
    if constexpr (Cfg::TRANS != 0) {
      const bool is_a = idx == 0 || idx > Cfg::FN;
      const int blk = idx == 0 ? 0 : (idx <= Cfg::FN ? idx - 1 : idx - Cfg::FN);
      u32x4_t v;
      if ((is_a && Cfg::TRANS_A) || (!is_a && Cfg::TRANS_B)) {
        // block i of A / j of B: 32 columns further = 4 chunks = bit 6 / bits 6-7 of the byte offset, which the
        // swizzle XORs; substep kk: 16 rows further; second half of the fragment: 4 rows further
        const uint32_t base = (uint32_t)reinterpret_cast<uintptr_t>(is_a ? sa : sb) + ((is_a ? a_rd : b_rd) ^ (uint32_t)(blk * 64));
        u32x2_t lo, hi;
        if (kk == 0) { lo = tr_read<0>(base); hi = tr_read<2048>(base); }
        else if (kk == 1) { lo = tr_read<8192>(base); hi = tr_read<8192 + 2048>(base); }
        else if (kk == 2) { lo = tr_read<16384>(base); hi = tr_read<16384 + 2048>(base); }
        else { lo = tr_read<24576>(base); hi = tr_read<24576 + 2048>(base); }
        v = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
      } else {
        // row-major operand: block i is 32 rows = 4096 bytes further, substep kk flips chunk bits (see the plain path)
        const uint32_t base = (uint32_t)reinterpret_cast<uintptr_t>(is_a ? sa : sb) + ((is_a ? a_rd : b_rd) ^ (uint32_t)(kk * 32));
        if (blk == 0) v = lds_read16<0>(base);
        else if (blk == 1) v = lds_read16<4096>(base);
        else if (blk == 2) v = lds_read16<8192>(base);
        else v = lds_read16<12288>(base);
      }
      if (is_a) af[blk] = v;
      else bf[blk] = v;
      return;
    }
    const uint32_t ao = a_rd ^ (uint32_t)(kk * 32);
    const uint32_t bo = b_rd ^ (uint32_t)(kk * 32);
    if (idx == 0) af[0] = *reinterpret_cast<const u32x4_t*>(sa + ao);
    else if (idx <= Cfg::FN) bf[idx - 1] = *reinterpret_cast<const u32x4_t*>(sb + bo + (idx - 1) * 32 * Cfg::BKB);
    else af[idx - Cfg::FN] = *reinterpret_cast<const u32x4_t*>(sa + ao + (idx - Cfg::FN) * 32 * Cfg::BKB);
  }
  LCE_DEV void load_frags(const char* sa, const char* sb, int kk, u32x4_t (&af)[Cfg::FM], u32x4_t (&bf)[Cfg::FN]) const {
#pragma unroll
    for (int i = 0; i < N_READS; ++i) read_one(sa, sb, kk, i, af, bf);
  }

  // One k-substep with a hand-placed instruction order (pinned by scheduling barriers): the MFMAs
  // of this substep, with the operand reads of the NEXT substep (from `sa_next` / `sb_next`, substep `kk_next`)
  // and, when DMA is set, the global->LDS loads of a future slab dealt out between them.
  // DMA: 0 none; 1 the loads of a whole stage (unsplit ring); 2 / 3 (split ring) loads [J0, J1) of a B / A half
  template <int DMA, int J0 = 0, int J1 = 0>
  LCE_DEV void substep(f32x16_t (&acc)[Cfg::FM][Cfg::FN], const u32x4_t (&af)[Cfg::FM], const u32x4_t (&bf)[Cfg::FN],
                       const char* sa_next, const char* sb_next, int kk_next, u32x4_t (&af_n)[Cfg::FM],
                       u32x4_t (&bf_n)[Cfg::FN], char* lds, int dma_stage, int64_t dma_kbyte) const {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int b = 0; b < N_BLK; ++b) {
      if constexpr (Cfg::TRANS != 0) {
        // The operand reads are inline assembly (see tr_read), so the waits are placed by hand.  Reads are issued
        // in the order a0, b0 .. b(FN-1), a1 .. (two instructions for a K-major operand, one for a row-major one),
        // one operand after each of the first MFMAs, and LDS reads return in order.  Before MFMA b of this
        // substep, the reads of the NEXT substep issued so far are in flight behind this substep's; the MFMA
        // needs its A block (b / FN) and its B block (b % FN).
        constexpr int CA = Cfg::TRANS_A ? 2 : 1, CB = Cfg::TRANS_B ? 2 : 1;
        constexpr int ALL = CA * Cfg::FM + CB * Cfg::FN;
        // instructions issued up to and including operand read number `idx` of the order above
        auto upto = [](int idx) { return idx < 0 ? 0 : (idx == 0 ? CA : (idx <= Cfg::FN ? CA + CB * idx : CA + CB * Cfg::FN + CA * (idx - Cfg::FN))); };
        const int ia = b / Cfg::FN, ib = b % Cfg::FN;
        const int last = ia == 0 ? 1 + ib : Cfg::FN + ia;  // the last operand read it depends on
        const int allow = (ALL - upto(last)) + upto((b < N_READS ? b : N_READS) - 1);
        static_assert(ALL <= 15, "lgkmcnt range");
        wait_lgkm(allow);
        __builtin_amdgcn_sched_barrier(0);  // the wait stays in front of the MFMA
      }
      Mma<TIN>::run(acc[b / Cfg::FN][b % Cfg::FN], af[b / Cfg::FN], bf[b % Cfg::FN]);
      // reads: spread over the first blocks, one read after every `rstep`-th MFMA
      constexpr int rstep = 1;
      if ((b % rstep) == rstep - 1 && b / rstep < N_READS) read_one(sa_next, sb_next, kk_next, b / rstep, af_n, bf_n);
      if (N_BLK < N_READS && b == N_BLK - 1) {
#pragma unroll
        for (int r = N_BLK; r < N_READS; ++r) read_one(sa_next, sb_next, kk_next, r, af_n, bf_n);
      }
      if constexpr (DMA == 1) {
#pragma unroll
        for (int d = b * PER / N_BLK; d < (b + 1) * PER / N_BLK; ++d) dma_one(lds, dma_stage, dma_kbyte, d);
      } else if constexpr (DMA == 2 || DMA == 3) {
        constexpr int NJ = J1 - J0;
#pragma unroll
        for (int d = b * NJ / N_BLK; d < (b + 1) * NJ / N_BLK; ++d) dma_half(lds, dma_stage, dma_kbyte, DMA == 2, J0 + d);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // Full K loop.  K must be a multiple of Cfg::BK (and > 0).  The k-substeps are software
  // pipelined: operand fragments of substep s+1 are read from LDS while the MFMAs of substep s run,
  // and the workgroup barrier that hands a ring stage back to the loader sits before the LAST
  // substep of a slab, so the matrix pipe keeps working across the barrier.  The loop body is
  // branch-free: past the end of K the loader re-fetches the last slab into a stage nobody reads.
  // Issues the loads of the first NSTAGE slabs.  LDS must be free (every wave past its last read and
  // its loads drained: a workgroup barrier after the previous main()).
  LCE_DEV void prologue(char* lds, int64_t K) const {
    const int nk = (int)(K / Cfg::BK);
    const int64_t last_kbyte = (int64_t)(nk - 1) * Cfg::BKB;
    if constexpr (Cfg::SPLIT) {
      // half slabs 0..3 = E0 L0 E1 L1 (E: the early operand) into slots 0..3
#pragma unroll
      for (int hf = 0; hf < 4; ++hf) {
        const int64_t kb = (int64_t)(hf / 2) * Cfg::BKB;
#pragma unroll
        for (int j = 0; j < Cfg::A_LOADS; ++j) dma_half(lds, hf, kb < last_kbyte ? kb : last_kbyte, (hf & 1) == (Cfg::SPLIT == 1), j);
      }
      return;
    }
#pragma unroll
    for (int s = 0; s < Cfg::NSTAGE; ++s) {
      const int64_t kb = (int64_t)s * Cfg::BKB;
      issue_slab(lds, s, kb < last_kbyte ? kb : last_kbyte);
    }
  }

  LCE_DEV void run(char* lds, int64_t K, f32x16_t (&acc)[Cfg::FM][Cfg::FN]) const {
    prologue(lds, K);
    main(lds, K, acc);
  }

  // The K loop proper; prologue() must have been called for this tile (no other vector memory
  // loads may have been issued by this wave in between: the waits count outstanding loads).
  LCE_DEV void main(char* lds, int64_t K, f32x16_t (&acc)[Cfg::FM][Cfg::FN]) const {
    if constexpr (Cfg::SPLIT) {
      main_split(lds, K, acc);
      return;
    }
    constexpr int NS = Cfg::NSTAGE, KSUB = Cfg::KSUB;
    const int nk = (int)(K / Cfg::BK);
    const int64_t last_kbyte = (int64_t)(nk - 1) * Cfg::BKB;
#pragma unroll
    for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
      for (int j = 0; j < Cfg::FN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    wait_vm<Cfg::SPLIT ? 0 : (NS - 1) * PER>();  // (the split ring has its own loop; this body is still instantiated)
    __builtin_amdgcn_s_barrier();
    u32x4_t af[2][Cfg::FM], bf[2][Cfg::FN];
    load_frags(lds, lds, 0, af[0], bf[0]);
    int stage = 0;
    int64_t kb_next = (int64_t)NS * Cfg::BKB;
    for (int it = 0; it < nk; ++it) {
      const char* s = lds + stage * Cfg::STAGE_BYTES;
#pragma unroll
      for (int kk = 0; kk < KSUB - 1; ++kk) {
        substep<0>(acc, af[kk & 1], bf[kk & 1], s, s, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1], lds, 0, 0);
      }
      // last substep of this slab: its fragments are in registers, so this wave is done with the stage
      const int nstage = stage + 1 == NS ? 0 : stage + 1;
      wait_vm<Cfg::SPLIT ? 0 : (NS - 2) * PER>();  // slab it+1 has landed (only the younger slabs may be in flight)
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's reads of the stage have returned
      __builtin_amdgcn_s_barrier();
      substep<1>(acc, af[(KSUB - 1) & 1], bf[(KSUB - 1) & 1], lds + nstage * Cfg::STAGE_BYTES,
                    lds + nstage * Cfg::STAGE_BYTES, 0, af[0], bf[0], lds, stage, kb_next < last_kbyte ? kb_next : last_kbyte);
      kb_next += Cfg::BKB;
      stage = nstage;
    }
    wait_vm<0>();  // drain the redundant tail fetches before LDS is reused
  }

  // K loop over the split ring.  One operand is "early" (E: A with SPLIT = 1, B with SPLIT = 2), the
  // other "late" (L).  Slab i reads E(i) from slot (2i) % 5 and L(i) from slot (2i+1) % 5.  While slab i
  // computes, its first two k-substeps issue the loads of E(i+2) into the slot that L(i-1) left
  // (slot (2i+4) % 5); after the barrier that ends slab i, its last substep issues L(i+2) into E(i)'s
  // slot.  The barrier needs E(i+1), L(i+1): everything except the youngest A_LOADS loads, E(i+2),
  // which stay in flight across it.  So the burst after the barrier is half as long and half of the
  // loads get two barrier periods to land.  Measured against the 2-stage ring of whole slabs: the
  // load-only loop drops from 1.37 to 1.10 ms (16384 x 16384 x 3584), the full GEMM from 1.59 to 1.54.
  LCE_DEV void main_split(char* lds, int64_t K, f32x16_t (&acc)[Cfg::FM][Cfg::FN]) const {
    constexpr int KSUB = Cfg::KSUB, HL = Cfg::A_LOADS;
    constexpr bool A_EARLY = Cfg::SPLIT == 1;
    constexpr int EARLY = A_EARLY ? 3 : 2, LATE = A_EARLY ? 2 : 3;  // substep DMA modes: 3 loads an A half, 2 a B half
    static_assert(Cfg::A_LOADS == Cfg::B_LOADS && KSUB == 4 && HL % 2 == 0, "equal halves, four k-substeps");
    const int nk = (int)(K / Cfg::BK);
    const int64_t last_kbyte = (int64_t)(nk - 1) * Cfg::BKB;
#pragma unroll
    for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
      for (int j = 0; j < Cfg::FN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    wait_vm<2 * HL>();  // E0, L0 have landed
    __builtin_amdgcn_s_barrier();
    u32x4_t af[2][Cfg::FM], bf[2][Cfg::FN];
    load_frags(lds + (A_EARLY ? 0 : Cfg::STAGE_BYTES), lds + (A_EARLY ? Cfg::STAGE_BYTES : 0), 0, af[0], bf[0]);
    int sa = 0;  // slot of this slab's early half; the late half is in the next slot
    for (int it = 0; it < nk; ++it) {
      const int sb = sa + 1 >= 5 ? sa + 1 - 5 : sa + 1;
      const int na = sa + 2 >= 5 ? sa + 2 - 5 : sa + 2;
      const int nb = sa + 3 >= 5 ? sa + 3 - 5 : sa + 3;
      const int fa = sa + 4 >= 5 ? sa + 4 - 5 : sa + 4;  // free slot: takes E(it+2)
      const char* pa = lds + (A_EARLY ? sa : sb) * Cfg::STAGE_BYTES;
      const char* pb = lds + (A_EARLY ? sb : sa) * Cfg::STAGE_BYTES;
      const int64_t kb2 = (int64_t)(it + 2) * Cfg::BKB;
      const int64_t kb = kb2 < last_kbyte ? kb2 : last_kbyte;
      substep<EARLY, 0, HL / 2>(acc, af[0], bf[0], pa, pb, 1, af[1], bf[1], lds, fa, kb);
      substep<EARLY, HL / 2, HL>(acc, af[1], bf[1], pa, pb, 2, af[0], bf[0], lds, fa, kb);
      substep<0>(acc, af[0], bf[0], pa, pb, 3, af[1], bf[1], lds, 0, 0);
      wait_vm<HL>();                       // slab it+1 has landed; E(it+2) may still be in flight
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's reads of both slots have returned
      __builtin_amdgcn_s_barrier();
      substep<LATE, 0, HL>(acc, af[1], bf[1], lds + (A_EARLY ? na : nb) * Cfg::STAGE_BYTES, lds + (A_EARLY ? nb : na) * Cfg::STAGE_BYTES, 0,
                           af[0], bf[0], lds, sa, kb);
      sa = na;
    }
    wait_vm<0>();  // drain the redundant tail fetches before LDS is reused
  }

  // s_waitcnt lgkmcnt(n) only; n is a constant after unrolling, the switch folds away
  static LCE_DEV void wait_lgkm(int n) {
#define LCE_LGKM(N) case N: __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8)); break;
    switch (n) {
      LCE_LGKM(0) LCE_LGKM(1) LCE_LGKM(2) LCE_LGKM(3) LCE_LGKM(4) LCE_LGKM(5) LCE_LGKM(6) LCE_LGKM(7)
      LCE_LGKM(8) LCE_LGKM(9) LCE_LGKM(10) LCE_LGKM(11) LCE_LGKM(12) LCE_LGKM(13) LCE_LGKM(14)
      default: __builtin_amdgcn_s_waitcnt(0xC07F | (15 << 8)); break;
    }
#undef LCE_LGKM
  }

  template <int N>
  static LCE_DEV void wait_vm() {
    // gfx9 s_waitcnt simm16: vmcnt[3:0] bits 3:0, expcnt bits 6:4, lgkmcnt bits 11:8, vmcnt[5:4] bits 15:14
    static_assert(N < 64, "vmcnt range");
    __builtin_amdgcn_s_waitcnt(((N & 0xF) | ((N >> 4) << 14)) | 0x0F70);
  }
};

}  // namespace lce
