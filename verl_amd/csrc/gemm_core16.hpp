// Second MFMA mainloop for gfx950 (MI355X), 16-bit operands only: four waves, each owning 128 x 128 of a
// 256 x 256 workgroup tile as 8 x 8 blocks of v_mfma_f32_16x16x32.
//
// Why a second one (measured on N(0,1) x N(0,0.02) operands, 16384 x 16384 x 3584, no epilogue, same box):
// the eight-wave 32x32x16 loop of gemm_core.hpp reaches 1.34 PFLOP/s, this one 1.48.  With such data the chip is
// power-limited (a register-resident MFMA loop runs at 1.83 PFLOP/s with 32x32x16 and 1.97 with 16x16x32,
// against 2.48 on all-zero operands), so what counts is energy per FLOP: the 16x16x32 shape moves a fifth less
// register data per FLOP, and a 128 x 128 wave tile needs a third fewer LDS operand reads than 64 x 128.
//
// The accumulators (256 registers per lane) live in AGPRs, the operand fragments (two k-steps of 8 + 8
// fragments, 128 registers) in VGPRs.  The MFMAs and the LDS reads are inline assembly: the compiler moves
// accumulators between the two register classes otherwise, and it cannot interleave what it does not order.
// Consequently the s_waitcnt for the reads are placed by hand (LDS reads return in order).
//
// LDS ring: the split ring of gemm_core.hpp (five half slabs of 32 KB, the B operand early), one workgroup
// barrier per slab, placed between its two k-steps.
//
// Accumulator layout of one 16 x 16 block: lane l holds column n = l % 16 and rows m = 4 * (l / 16) + r,
// r = 0..3.  Block (i, j) of a wave covers rows 16 i .. and columns 16 j .. of its 128 x 128.
#pragma once
#include <utility>

#include "gemm_core.hpp"

namespace lce {

template <typename T>
struct Mma16;
template <>
struct Mma16<bf16_t> {
  static LCE_DEV void run(f32x4_t& acc, const u32x4_t& a, const u32x4_t& b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  }
  // the same instruction as a builtin: the compiler schedules it and knows its latency
  static LCE_DEV f32x4_t known(const f32x4_t& acc, const u32x4_t& a, const u32x4_t& b) {
    typedef __bf16 v8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), acc, 0, 0, 0);
  }
};
template <>
struct Mma16<f16_t> {
  static LCE_DEV void run(f32x4_t& acc, const u32x4_t& a, const u32x4_t& b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  }
  static LCE_DEV f32x4_t known(const f32x4_t& acc, const u32x4_t& a, const u32x4_t& b) {
    typedef _Float16 v8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), acc, 0, 0, 0);
  }
};

template <int... Is, typename F>
LCE_DEV void static_for(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}

// TRANS_: 0 both operands K-contiguous (row-major A[m][k], B[n][k]); 1 both K-major in memory, A[k][m] and
// B[k][n], fetched with the transposing LDS read (two ds_read_b64_tr_b16 per fragment); 2 only A K-major (mixed).
template <typename TIN_, int TRANS_ = 0>
struct GemmCfg16 {
  typedef TIN_ TIN;
  static_assert(sizeof(TIN_) == 2, "16-bit operands");
  static constexpr bool CORE16 = true;
  static constexpr int BM = 256, BN = 256, BKB = 128, BK = 64, NSTAGE = 5, SPLIT = 2, TRANS = TRANS_;
  static constexpr int WAVES_M = 2, WAVES_N = 2, NW = 4, NTHREADS = 256;
  static constexpr int WM = 128, WN = 128;
  static constexpr int NB = 8;                       // 16-row blocks per side of a wave tile
  static constexpr int STAGE_BYTES = 32768;          // one operand's slab: 256 rows x 128 bytes, or 64 k-rows x 512 bytes
  static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;
  static constexpr int HL = 8;                       // wave-wide 16-byte-per-lane loads per wave and half slab
};

template <typename Cfg>
struct GemmCore16 {
  typedef typename Cfg::TIN TIN;
  static constexpr int NB = Cfg::NB, HL = Cfg::HL, SLOT = Cfg::STAGE_BYTES;
  static constexpr bool TN = Cfg::TRANS == 1;
  static constexpr bool TA = Cfg::TRANS != 0, TB = Cfg::TRANS == 1;  // which operand is K-major in memory

  const char* a_base;
  const char* b_base;
  uint32_t va[HL], vb[HL];  // per-lane byte offsets of the loads inside slab 0
  uint32_t a_rd, b_rd;      // per-lane LDS read offsets inside a slot (block 0, k-step 0)
  int64_t a_slab, b_slab;   // bytes from one K slab to the next in memory
  int wave, lane, wave_m, wave_n;
  // mixed mode: row of A inside a slab that each load fetches, A's row stride in bytes and the number of its rows that exist
  uint32_t va_tail[HL];         // mixed mode: va of the last slab of A that has rows, rows beyond them clamped
  int64_t a_ks_full, a_ks_last;  // slabs below a_ks_full have all their 64 rows; a_ks_last: the last slab with any

  LCE_DEV void set_lane() {
    wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    lane = threadIdx.x & 63;
    wave_m = wave >> 1;
    wave_n = wave & 1;
  }

  // Row-major operands.  MFMA rows come from A (rows m0 .. of an M-row matrix), MFMA columns from B (rows n0 .. of
  // an N-row matrix); rows beyond a matrix are clamped to its last row (the epilogue discards them).  With `b_rows`,
  // row n of the B operand is B[b_rows[n]] (a gather; every row's byte offset from B must then fit 32 bits).
  // LDS layout of a slab: row-major, 128 bytes per row, 16-byte chunk c of row r at position c ^ ((r / 2) % 8): the
  // 16 rows x 4 chunks that a quarter wave reads for one fragment then fall into 64 different banks.
  LCE_DEV void init(const TIN* A, int64_t lda, int64_t m0, int64_t M, const TIN* B, int64_t ldb, int64_t n0, int64_t N,
                    const int* b_rows = nullptr) {
    set_lane();
    a_base = reinterpret_cast<const char*>(A + m0 * lda);
    b_base = reinterpret_cast<const char*>(b_rows ? B : B + n0 * ldb);
    a_slab = b_slab = Cfg::BKB;
    const int rows_a = (int)((M - m0) < (int64_t)Cfg::BM ? (M - m0) : (int64_t)Cfg::BM);
    const int rows_b = (int)((N - n0) < (int64_t)Cfg::BN ? (N - n0) : (int64_t)Cfg::BN);
    const int lr = lane >> 3, pc = lane & 7;
#pragma unroll
    for (int j = 0; j < HL; ++j) {
      const int row = (j * Cfg::NW + wave) * 8 + lr;
      const int c = pc ^ ((row >> 1) & 7);
      const int ra = row < rows_a ? row : rows_a - 1;
      const int rb = row < rows_b ? row : rows_b - 1;
      const int64_t gb = b_rows ? (int64_t)b_rows[n0 + rb] : (int64_t)rb;
      va[j] = (uint32_t)((int64_t)ra * lda * 2) + (uint32_t)(c * 16);
      vb[j] = (uint32_t)(gb * ldb * 2) + (uint32_t)(c * 16);
    }
    const int r16 = lane & 15, g = lane >> 4;
    const uint32_t off = (uint32_t)(r16 * 128 + ((g ^ (r16 >> 1)) * 16));
    a_rd = (uint32_t)(wave_m * Cfg::WM * 128) + off;
    b_rd = (uint32_t)(wave_n * Cfg::WN * 128) + off;
  }

  // K-major operands: A[k][m0 + 0..256), B[k][n0 + 0..256) with row strides lda / ldb (elements); both must be
  // allocated in whole 256-column tiles.  A ring slot holds 64 k-rows of 512 bytes; chunk c of row r sits at
  // position c ^ swz(r), swz(r) = 4 (r % 4) ^ 2 ((r / 8) % 2), so that the eight k-rows that half a wave touches
  // in one transposing read fall into different banks.
  // The transposing read: in each group of 16 lanes, lane 4e + q supplies the address of X[k0 + e][x0 + 4q ..] and
  // lane i receives X[k0 .. k0+3][x0 + i]; group g of the wave takes the k-octet 8g of the 32 k-values of a k-step,
  // and a second read 4 rows further completes the octet.
  LCE_DEV void init_tn(const TIN* A, int64_t lda, int64_t m0, const TIN* B, int64_t ldb, int64_t n0) {
    set_lane();
    a_base = reinterpret_cast<const char*>(A + m0);
    b_base = reinterpret_cast<const char*>(B + n0);
    a_slab = 64 * lda * 2;
    b_slab = 64 * ldb * 2;
#pragma unroll
    for (int j = 0; j < HL; ++j) {
      const int row = (j * Cfg::NW + wave) * 2 + (lane >> 5);
      const int c = (lane & 31) ^ tn_swz(row);
      va[j] = (uint32_t)((int64_t)row * lda * 2) + (uint32_t)(c * 16);
      vb[j] = (uint32_t)((int64_t)row * ldb * 2) + (uint32_t)(c * 16);
    }
    const int g = lane >> 4, e = (lane & 15) >> 2, q = lane & 3;
    const int row = 8 * g + e;  // (k-step 0, first half of the octet)
    const uint32_t in_row = (uint32_t)((((q >> 1) ^ tn_swz(row)) * 16) + (q & 1) * 8);
    a_rd = (uint32_t)(row * 512 + wave_m * Cfg::WM * 2) + in_row;
    b_rd = (uint32_t)(row * 512 + wave_n * Cfg::WN * 2) + in_row;
  }
  static LCE_DEV int tn_swz(int row) { return ((row & 3) * 4) ^ (((row >> 3) & 1) * 2); }

  // Mixed: A[k][m0 + 0..256) K-major as in init_tn, B row-major as in init (rows n0 .. of an N-row matrix, clamped).
  // LDS row r of an A slab holds memory row perm(r) of the slab (perm: a permutation of 0..63, the order in which B's
  // K index was stored); rows at or beyond `kvalid` > 0 are replaced by rows that exist (B is zero there), and columns at
  // or beyond `mcols` (a last tile of a width that is no multiple of 256) by the row's first chunk: in bounds, and they
  // feed only results that the epilogue discards.
  template <typename Perm>
  LCE_DEV void init_mixed(const TIN* A, int64_t lda, int64_t m0, int64_t mcols, int64_t kvalid, Perm perm, const TIN* B, int64_t ldb,
                          int64_t n0, int64_t N) {
    static_assert(Cfg::TRANS == 2, "mixed mode");
    set_lane();
    a_base = reinterpret_cast<const char*>(A + m0);
    b_base = reinterpret_cast<const char*>(B + n0 * ldb);
    a_slab = 64 * lda * 2;
    b_slab = Cfg::BKB;
    a_ks_full = kvalid / 64;
    a_ks_last = (kvalid - 1) / 64;
    const int last_row = (int)(kvalid - 1 - a_ks_last * 64);  // of slab a_ks_last
    const int rows_b = (int)((N - n0) < (int64_t)Cfg::BN ? (N - n0) : (int64_t)Cfg::BN);
    const int lr = lane >> 3, pc = lane & 7;
#pragma unroll
    for (int j = 0; j < HL; ++j) {
      const int rowa = (j * Cfg::NW + wave) * 2 + (lane >> 5);
      const int ca = (lane & 31) ^ tn_swz(rowa);
      const int prow = (int)perm(rowa);
      const uint32_t col = (uint32_t)(((int64_t)ca * 8 < mcols ? ca : 0) * 16);
      va[j] = (uint32_t)((int64_t)prow * lda * 2) + col;
      va_tail[j] = (uint32_t)((int64_t)(prow < last_row ? prow : last_row) * lda * 2) + col;
      const int rowb = (j * Cfg::NW + wave) * 8 + lr;
      const int cb = pc ^ ((rowb >> 1) & 7);
      const int rb = rowb < rows_b ? rowb : rows_b - 1;
      vb[j] = (uint32_t)((int64_t)rb * ldb * 2) + (uint32_t)(cb * 16);
    }
    const int g = lane >> 4, e = (lane & 15) >> 2, q = lane & 3;
    const int row = 8 * g + e;
    a_rd = (uint32_t)(row * 512 + wave_m * Cfg::WM * 2) + (uint32_t)((((q >> 1) ^ tn_swz(row)) * 16) + (q & 1) * 8);
    const int r16 = lane & 15;
    b_rd = (uint32_t)(wave_n * Cfg::WN * 128) + (uint32_t)(r16 * 128 + ((g ^ (r16 >> 1)) * 16));
  }

  // ---- instruction-level pieces ----------------------------------------------------------------------------
  // load j of one operand's half slab number `ks` into ring slot `slot`
  LCE_DEV void dma(char* lds, int slot, int64_t ks, bool is_b, int j) const {
    char* dst = lds + slot * SLOT + (j * Cfg::NW + wave) * 1024;
    const char* src;
    if (Cfg::TRANS == 2 && !is_b) {
      // slabs with rows that do not exist take the last slab that has any, with its rows clamped (branch-free: the
      // hand-placed schedule of a k-step must stay one basic block)
      const bool tail = ks >= a_ks_full;
      src = a_base + (tail ? a_ks_last : ks) * a_slab + (tail ? va_tail[j] : va[j]);
    } else {
      src = (is_b ? b_base + ks * b_slab + vb[j] : a_base + ks * a_slab + va[j]);
    }
    __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)dst, 16, 0, 0);
  }

  // Fragments are read in the order a0, b0 .. b7, a1 .. a7 (F = 0 .. 15): the MFMAs walk the A blocks in the outer
  // loop, so the first row of eight needs a0 and every b, the later rows one more a each.
  static constexpr bool frag_is_a(int f) { return f == 0 || f > 8; }
  static constexpr int frag_blk(int f) { return f == 0 ? 0 : (f <= 8 ? f - 1 : f - 8); }
  static constexpr int CA = TA ? 2 : 1, CB = TB ? 2 : 1;  // LDS instructions per fragment of each operand
  // ra / rb: LDS address of the slot plus a_rd / b_rd; S: k-step inside the slab
  template <int F, int S>
  LCE_DEV void read_frag(uint32_t ra, uint32_t rb, u32x4_t (&af)[NB], u32x4_t (&bf)[NB]) const {
    constexpr bool is_a = frag_is_a(F);
    constexpr int blk = frag_blk(F);
    u32x4_t v;
    if constexpr (is_a ? TA : TB) {
      // block: 16 columns = 32 bytes further, inside the swizzled chunk bits; k-step: 32 rows; second half: 4 rows
      const uint32_t base = (is_a ? ra : rb) ^ (uint32_t)(blk * 32);
      const u32x2_t lo = tr_read<S * 16384>(base), hi = tr_read<S * 16384 + 2048>(base);
      v = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
    } else {
      v = lds_read16<blk * 2048>((is_a ? ra : rb) ^ (uint32_t)(S * 64));
    }
    if constexpr (is_a) af[blk] = v;
    else bf[blk] = v;
  }

  // LDS instructions issued up to and including fragment f of a k-step (f = -1: none)
  static constexpr int upto(int f) { return f < 0 ? 0 : (f == 0 ? CA : (f <= 8 ? CA + CB * f : CA + 8 * CB + CA * (f - 8))); }
  static constexpr int ALLI = 8 * (CA + CB);
  // fragments of the next k-step issued before MFMA m of this one: one after each even MFMA of the first half
  static constexpr int frags_before(int m) { return (m + 1) / 2 > 16 ? 16 : (m + 1) / 2; }

  // One k-step: 64 MFMAs on (af, bf); the 16 fragment reads of the next k-step (from ra_n / rb_n, k-step S_N) and HL
  // global->LDS loads are dealt between them.  WAIT: the fragments of this step were read during the previous step
  // and may still be in flight.  DMA_B: the loads fetch the B operand's half slab `dma_ks` (else A's) into `dma_slot`.
  template <bool WAIT, int S_N, bool DMA_B>
  LCE_DEV void kstep(f32x4_t (&acc)[NB][NB], const u32x4_t (&af)[NB], const u32x4_t (&bf)[NB], uint32_t ra_n, uint32_t rb_n,
                     u32x4_t (&af_n)[NB], u32x4_t (&bf_n)[NB], char* lds, int dma_slot, int64_t dma_ks) const {
    static_for(std::make_integer_sequence<int, NB * NB>{}, [&](auto mc) {
      constexpr int m = decltype(mc)::value;
      constexpr int i = m / NB, j = m % NB;
      if constexpr (WAIT && (i == 0 || m % NB == 0)) {
        constexpr int need = i == 0 ? 1 + j : 8 + i;  // the last fragment this MFMA depends on
        constexpr int allow = (ALLI - upto(need)) + upto(frags_before(m) - 1);
        wait_lgkm<(allow > 15 ? 15 : allow)>();
      }
      __builtin_amdgcn_sched_barrier(0);
      Mma16<TIN>::run(acc[i][j], af[i], bf[j]);
      if constexpr ((m & 1) == 0 && m / 2 < 16) read_frag<m / 2, S_N>(ra_n, rb_n, af_n, bf_n);
      if constexpr (m % (NB * NB / HL) == 3) dma(lds, dma_slot, dma_ks, DMA_B, m / (NB * NB / HL));
      __builtin_amdgcn_sched_barrier(0);
    });
  }

  template <int N>
  static LCE_DEV void wait_lgkm() { __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8)); }
  template <int N>
  static LCE_DEV void wait_vm() {
    static_assert(N < 64, "vmcnt range");
    __builtin_amdgcn_s_waitcnt(((N & 0xF) | ((N >> 4) << 14)) | 0x0F70);
  }

  // Issues the loads of the first two slabs (half slabs E0 L0 E1 L1 into slots 0..3; E = the B operand).  LDS must be
  // free: every wave past its last read of the previous tile and its own loads drained (a workgroup barrier after main()).
  LCE_DEV void prologue(char* lds, int64_t K) const {
    const int64_t last = K / Cfg::BK - 1;
#pragma unroll
    for (int hf = 0; hf < 4; ++hf) {
      const int64_t ks = hf / 2 < last ? hf / 2 : last;
#pragma unroll
      for (int j = 0; j < HL; ++j) dma(lds, hf, ks, (hf & 1) == 0, j);
    }
  }

  // The K loop (K a positive multiple of 64); prologue() must have been called for this tile, and no other vector memory
  // load may have been issued by this wave since (the waits count outstanding loads).  Slab i reads B from slot 2i % 5
  // and A from the next slot.  Its first k-step issues the loads of B(i+2) into the slot that A(i-1) left; the barrier
  // between the two k-steps waits for slab i+1 (everything but those youngest loads) and for every wave's reads of slab
  // i; the second k-step then issues A(i+2) into B(i)'s slot and reads the first fragments of slab i+1.  Past the end
  // of K the loader re-fetches the last slab into slots nobody reads (a branch-free body), drained at the end.
  LCE_DEV void main(char* lds, int64_t K, f32x4_t (&acc)[NB][NB]) const {
    const int nk = (int)(K / Cfg::BK);
    const int64_t last = nk - 1;
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    wait_vm<2 * HL>();  // slab 0 has landed
    __builtin_amdgcn_s_barrier();
    const uint32_t lds0 = (uint32_t)reinterpret_cast<uintptr_t>(lds);
    u32x4_t af[2][NB], bf[2][NB];
    static_for(std::make_integer_sequence<int, 16>{}, [&](auto fc) {
      read_frag<decltype(fc)::value, 0>(lds0 + SLOT + a_rd, lds0 + b_rd, af[0], bf[0]);
    });
    int sb = 0;  // slot of this slab's B half; its A half is in the next slot
    for (int it = 0; it < nk; ++it) {
      const int sa = sb + 1 >= 5 ? sb + 1 - 5 : sb + 1;
      const int nb = sb + 2 >= 5 ? sb + 2 - 5 : sb + 2;
      const int na = sb + 3 >= 5 ? sb + 3 - 5 : sb + 3;
      const int fr = sb + 4 >= 5 ? sb + 4 - 5 : sb + 4;  // free slot: takes B(it+2)
      const int64_t ks = it + 2 < last ? it + 2 : last;
      kstep<true, 1, true>(acc, af[0], bf[0], lds0 + sa * SLOT + a_rd, lds0 + sb * SLOT + b_rd, af[1], bf[1], lds, fr, ks);
      wait_vm<HL>();   // slab it+1 has landed; B(it+2) may still be in flight
      wait_lgkm<0>();  // this wave's reads of slab it have returned
      __builtin_amdgcn_s_barrier();
      kstep<false, 0, false>(acc, af[1], bf[1], lds0 + na * SLOT + a_rd, lds0 + nb * SLOT + b_rd, af[0], bf[0], lds, sb, ks);
      sb = nb;
    }
    wait_vm<0>();    // drain the redundant tail fetches before LDS is reused
    wait_lgkm<0>();  // and the reads of the slab after the last
    // The accumulators are read by ordinary instructions from here on: let the last MFMAs retire.  The MFMAs are inline
    // assembly, so the compiler knows nothing of their latency, and it is free to place a copy of an accumulator (for the
    // epilogue, or to spill it) right behind the statement that last wrote it, ahead of this wait (seen in a variant of
    // the forward: accumulators copied to scratch a few instructions behind the last MFMA, wrong statistics).  Only the
    // last blocks of the k-step can still be in the matrix pipe when the loop ends, so the last row of blocks is passed
    // through one more MFMA that the compiler does know (zero operands: acc + 0): behind a builtin it keeps the
    // distance to a read itself, and the matrix pipe orders it behind the assembly MFMA that wrote the same registers.
    asm volatile("s_nop 15\n\ts_nop 7" ::);
    const u32x4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < NB; ++j) acc[NB - 1][j] = Mma16<TIN>::known(acc[NB - 1][j], zero, zero);
  }

  LCE_DEV void run(char* lds, int64_t K, f32x4_t (&acc)[NB][NB]) const {
    prologue(lds, K);
    main(lds, K, acc);
  }
};

}  // namespace lce
