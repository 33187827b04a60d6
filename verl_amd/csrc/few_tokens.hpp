// Gradient GEMMs of a backward with few tokens (at most 128), and d_logits from kept logits; 16-bit inputs, gfx950.
//
// With T <= 128 both products are one streaming pass over a [V, H] matrix and bound by HBM, not by the matrix cores:
//   d_weight[v][h] = sum_t dS[t][v] * hidden[t][h]      writes [V, H] once; its operands (dS, hidden) are small
//   d_hidden[t][h] = sum_v dS[t][v] * W[v][h]           reads W once; its result is small
// The 256 x 256 tiles of the general path spend such a pass waiting: a d_weight tile has a K loop of one or two slabs
// between a cold start and 128 KB of scattered 2-byte stores, and a d_hidden tile keeps two half slabs of W in flight
// per CU.  The kernels here are shaped for the stream instead:
//   * several small workgroups per CU (40-80 KB of LDS, <= 168 registers), so that one workgroup's loads overlap
//     another's MFMAs and stores without a hand-built ring; the next operand tile travels global -> registers while
//     the current one is multiplied, and is written to LDS after it;
//   * d_weight: one workgroup owns 64 vocabulary rows and walks all of H, so dS is fetched once per row block and
//     every store instruction writes 16 rows x 64 contiguous bytes;
//   * d_hidden: the vocabulary is cut into as many K slices as fill the chip twice over (fp32 partials, summed in a
//     fixed order afterwards), and W is read as it lies in memory.
// Both take their K-major operand (hidden[t][.], dS[t][.], W[v][.]) through the transposing LDS read
// ds_read_b64_tr_b16.  Everything is plain HIP with compiler-placed waits.
#pragma once
#include "gemm_core.hpp"
#include "lce_kernels.hpp"

namespace lce {

typedef short i16x4_lds_t __attribute__((ext_vector_type(4)));

// Transposing read.  In each group of 16 lanes, lane 4e + q passes the address of four consecutive 16-bit elements of
// row e, X[e][4q' ..]; lane i of the group receives the i-th of the group's 16 columns for rows 0..3, i.e.
// column (i % 4) of the run that lane (i / 4) pointed at in each row.
LCE_DEV u32x2_t tr_read_b64(const char* lds_addr) {
  const i16x4_lds_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (i16x4_lds_t __attribute__((address_space(3)))*)(uintptr_t)(uint32_t)(uintptr_t)lds_addr);
  u32x2_t r;
  __builtin_memcpy(&r, &v, 8);
  return r;
}

template <typename T>
LCE_DEV void mma16(f32x4_t& acc, const u32x4_t& a, const u32x4_t& b) {
  if constexpr (sizeof(T) == 2 && __is_same(T, bf16_t)) {
    bf16x8_t x, y;
    __builtin_memcpy(&x, &a, 16);
    __builtin_memcpy(&y, &b, 16);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, acc, 0, 0, 0);
  } else {
    f16x8_t x, y;
    __builtin_memcpy(&x, &a, 16);
    __builtin_memcpy(&y, &b, 16);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, acc, 0, 0, 0);
  }
}

// swizzle of the 16-byte chunks of a K-major LDS row of 512 bytes (32 chunks): row r holds chunk c at position
// c ^ fw_swz(r), so that the rows one transposing read touches (r, r+1, r+2, r+3 and the same 8 and 16 rows on) fall
// into different banks (values below 16: valid for rows of 16 chunks and of 32)
LCE_DEV int fw_swz(int r) { return ((r & 3) << 2) ^ ((r >> 3) & 3); }

template <typename TIN>
struct FewArgs {
  const TIN* dS;      // [>= kt rows][ldS]: d_logits of the chunk by (compact) token position; columns in Perm order;
  int64_t ldS;        //   zero rows beyond the tokens that take part, zero columns beyond the chunk's rows
  const TIN* Ht;      // compact copy of hidden, [>= kt rows][ldHt], ldHt >= round_up(H, 256); zero rows beyond the tokens
  int64_t ldHt;
  const TIN* W;       // first row of the chunk, row stride ldw
  int64_t ldw;
  int64_t vrows;      // rows of the chunk
  int64_t ucols;      // columns of dS that are written (vrows rounded up to the permutation group)
  int64_t H;
  int kt;             // token positions summed over by d_weight: a multiple of 32, <= 128
  int nt;             // token rows of d_hidden's result that exist (<= 128)
  const int* n_rows;  // device-side count of the token positions that take part (null: kt)
  void* dW;           // [vrows][H] rows of d_weight of this chunk (TOUT)
  float* dHp;         // fp32 partials of d_hidden: slice s at dHp + s * part_stride, [nt][H]
  int64_t part_stride;
  int ksplit;         // K slices of d_hidden
  int64_t kslice;     // columns of dS per slice, a multiple of 64
  int accumulate;     // d_hidden partials: 0 store, 1 add to what is there (second and later chunks)
  int n_dw;           // workgroups of the d_weight part (they come first in the grid)
};

// ------------------------------------------------------------------------------------------------------------------
// d_weight, few tokens.  Workgroup = 256 threads = 4 waves; it owns dS columns [u0, u0 + 64) and walks H in tiles of
// HW = 256 or 128 columns; a wave multiplies 64 columns of the tile with all 64 dS columns (HW = 256) or with 32 of
// them (HW = 128: two waves side by side along each):  C[m = h][n = u] = sum_t Ht[t][h] * dS[t][u].
// MFMA rows are assigned to h in pairs of blocks: block 2i'+b, row 4g+r  <->  h = 32i' + 8g + 4b + r, so a lane ends
// up with 8 consecutive h for one u.  With 16-bit output a wave's results pass through a tile of its own in LDS and
// leave it as whole 128-byte lines, eight lanes per row (measured on the d_weight workgroups alone, H=3584, V=152064:
// 64 tokens 243 -> 228 us, 4.48 -> 4.78 TB/s; 96 tokens 306 -> 296 us); fp32 output is stored from the registers,
// 16 rows x 128 bytes per instruction.
// ------------------------------------------------------------------------------------------------------------------
template <typename TIN, typename TOUT, typename Perm, int KT, int HW>
LCE_DEV void dw_few_tile(const FewArgs<TIN>& p, int bid, char* lds) {
  static_assert(KT % 32 == 0 && KT <= 128, "token positions: whole k-steps of 32");
  static_assert(HW == 256 || HW == 128, "columns of a hidden tile");
  constexpr int KS = KT / 32;
  constexpr int RB = HW * 2, CPR = HW / 8;  // bytes and 16-byte chunks of a hidden tile's row
  // waves: WAVES_H along the tile's columns x WAVES_U along the 64 dS columns; a wave owns 64 columns of the hidden tile
  // (MI = 4 MFMA row blocks) and NJ blocks of 16 dS columns
  constexpr int WH = 64, MI = 4, WAVES_H = HW / WH, WAVES_U = 4 / WAVES_H, NJ = 4 / WAVES_U;
  constexpr bool STAGE = sizeof(TOUT) == 2;  // 16-bit output: a wave's row piece is one 128-byte line, stored through LDS
  char* sB = lds;                    // dS tile: KT rows x 128 bytes (64 columns), chunk c of row r at c ^ (r & 7)
  char* sA = lds + KT * 128;         // hidden tile: KT rows x RB bytes, chunk c of row r at c ^ fw_swz(r)
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int g = lane >> 4, l16 = lane & 15, e = l16 >> 2, q = l16 & 3;
  const int wh = wave % WAVES_H, wu = wave / WAVES_H;  // this wave's place along the hidden tile and along the dS columns
  const int64_t u0 = (int64_t)bid * 64;

  // dS tile -> LDS (KT * 8 chunks of 16 bytes)
#pragma unroll
  for (int i = 0; i < (KT * 8 + 255) / 256; ++i) {
    const int id = tid + i * 256, r = id >> 3, c = id & 7;
    if (id < KT * 8) {
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(p.dS + (int64_t)r * p.ldS + u0 + c * 8);
      *reinterpret_cast<u32x4_t*>(sB + r * 128 + ((c ^ (r & 7)) * 16)) = v;
    }
  }
  constexpr int AL = KT * CPR / 256;  // 16-byte chunks of a hidden tile per thread
  u32x4_t pre[AL];
  auto fetch = [&](int64_t h0) {
#pragma unroll
    for (int i = 0; i < AL; ++i) {
      const int id = tid + i * 256, r = id / CPR, c = id % CPR;
      pre[i] = *reinterpret_cast<const u32x4_t*>(p.Ht + (int64_t)r * p.ldHt + h0 + c * 8);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < AL; ++i) {
      const int id = tid + i * 256, r = id / CPR, c = id % CPR;
      *reinterpret_cast<u32x4_t*>(sA + r * RB + ((c ^ fw_swz(r)) * 16)) = pre[i];
    }
  };
  fetch(0);
  // output rows of this lane: dS column u0 + 16 NJ wu + 16 j + l16
  int64_t vrow[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int64_t v = Perm::vocab_at(u0 + 16 * NJ * wu + 16 * j + l16);
    vrow[j] = v < p.vrows ? v : -1;
  }
  // token positions that take part (a device-side count may cut the host's): rows beyond them are not read
  int ks_n = p.kt / 32;
  if (p.n_rows) {
    const int k = (*p.n_rows + 31) / 32;
    ks_n = k < ks_n ? k : ks_n;
  }
  // B fragments (dS) are the same for every h tile: they stay in registers (read once the tile has landed) unless 128
  // token positions meet 256-column tiles (registers)
  constexpr bool KEEP_B = KT <= 64 || HW <= 128;
  u32x4_t bf[KEEP_B ? KS : 1][NJ];
  auto read_b = [&](int ks, u32x4_t (&out)[NJ]) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      // lanes (e, q) of group g address row 32 ks + 8 g + e (+4), columns 16 NJ wu + 16 j + 4 q ..
      const int r0 = 32 * ks + 8 * g + e, r1 = r0 + 4, col = 16 * NJ * wu + 16 * j + 4 * q;
      const u32x2_t lo = tr_read_b64(sB + r0 * 128 + (((col >> 3) ^ (r0 & 7)) * 16) + (col & 7) * 2);
      const u32x2_t hi = tr_read_b64(sB + r1 * 128 + (((col >> 3) ^ (r1 & 7)) * 16) + (col & 7) * 2);
      out[j] = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
    }
  };
  const int n_ht = (int)((p.H + HW - 1) / HW);
  for (int ht = 0; ht < n_ht; ++ht) {
    __syncthreads();  // every wave is done with the previous hidden tile
    stash();
    __syncthreads();
    if (KEEP_B && ht == 0) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) read_b(ks, bf[KEEP_B ? ks : 0]);
    }
    if (ht + 1 < n_ht) fetch((int64_t)(ht + 1) * HW);
    f32x4_t acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks >= ks_n) break;
      u32x4_t af[MI];
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        // block i = 2i' + b: the run of lane q starts at column WH wh + 32 i' + 8 q + 4 b
        const int col = WH * wh + 32 * (i >> 1) + 8 * q + 4 * (i & 1);
        const int r0 = 32 * ks + 8 * g + e, r1 = r0 + 4;
        const u32x2_t lo = tr_read_b64(sA + r0 * RB + (((col >> 3) ^ fw_swz(r0)) * 16) + (col & 7) * 2);
        const u32x2_t hi = tr_read_b64(sA + r1 * RB + (((col >> 3) ^ fw_swz(r1)) * 16) + (col & 7) * 2);
        af[i] = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
      }
      if (!KEEP_B) read_b(ks, bf[0]);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) mma16<TIN>(acc[i][j], af[i], bf[KEEP_B ? ks : 0][j]);
    }
    if constexpr (STAGE) {
      // Whole 128-byte lines per store: the wave's 16 NJ rows x 64 columns go through a tile of its own in LDS (16-byte
      // chunk c of row r at c ^ ((r / 2) % 8), so that the 16 rows x 4 chunks of one write fall into different banks)
      // and leave it eight rows at a time, eight lanes per row.  No barrier: LDS operations of one wave complete in order.
      char* sC = lds + KT * 128 + KT * RB + wave * (NJ * 2048);
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int ip = 0; ip < MI / 2; ++ip) {
          float d[8];
#pragma unroll
          for (int x = 0; x < 8; ++x) d[x] = acc[2 * ip + (x >> 2)][j][x & 3];
          const int row = 16 * j + l16, c = 4 * ip + g;
          store_run<TOUT, 8>(reinterpret_cast<TOUT*>(sC + row * 128 + ((c ^ ((row >> 1) & 7)) * 16)), d);
        }
      const int64_t hw0 = (int64_t)ht * HW + WH * wh;
#pragma unroll
      for (int it = 0; it < NJ * 2; ++it) {
        const int row = it * 8 + (lane >> 3), pc = lane & 7, c = pc ^ ((row >> 1) & 7);
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(sC + row * 128 + pc * 16);
        const int64_t vr = Perm::vocab_at(u0 + 16 * NJ * wu + row), h = hw0 + c * 8;
        if (vr < p.vrows && h < p.H) *reinterpret_cast<u32x4_t*>(static_cast<TOUT*>(p.dW) + vr * p.H + h) = v;
      }
      continue;
    }
    // lane (g, l16): rows h = h0 + WH wh + 32 i' + 8 g + (0..7) of output row vrow[j]
    const int64_t hb = (int64_t)ht * HW + WH * wh + 8 * g;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      if (vrow[j] < 0) continue;
#pragma unroll
      for (int ip = 0; ip < MI / 2; ++ip) {
        const int64_t h = hb + 32 * ip;
        if (h >= p.H) continue;  // (H is a multiple of 8)
        float d[8];
#pragma unroll
        for (int x = 0; x < 8; ++x) d[x] = acc[2 * ip + (x >> 2)][j][x & 3];
        store_run<TOUT, 8>(static_cast<TOUT*>(p.dW) + vrow[j] * p.H + h, d);  // (non-temporal stores: 2.9 instead of 4.1 TB/s)
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------------------------
// d_hidden, few tokens.  Workgroup = 256 threads = 4 waves; it owns columns [h0, h0 + 256) of the result for all NT
// token rows and one K slice of the chunk's dS columns; wave w multiplies h0 + 64w .. +63:
//   C[m = h][n = t] = sum_u W[vocab_at(u)][h] * dS[t][u].
// A stage is 64 columns of dS: 64 rows of W (512 bytes of each, fetched in the order of dS's columns) and NT x 128
// bytes of dS.
// ------------------------------------------------------------------------------------------------------------------
template <typename TIN, typename Perm, int NT, int HW>
LCE_DEV void dh_few_tile(const FewArgs<TIN>& p, int bid, char* lds) {
  static_assert(NT == 64 || NT == 128, "token rows of a tile");
  static_assert(HW == 256 || HW == 128, "columns of a tile");
  constexpr int NJ = NT / 16;
  constexpr int RB = HW * 2, CPR = HW / 8;  // bytes and 16-byte chunks of a W stage's row
  constexpr int WH = HW / 4, MI = WH / 16;  // columns and 16-row MFMA blocks of a wave
  constexpr int WL = 64 * CPR / 256;        // chunks of a W stage per thread
  char* sA = lds;              // W stage: 64 rows x RB bytes, chunk c of row r at c ^ fw_swz(r)
  char* sB = lds + 64 * RB;    // dS stage: NT rows x 128 bytes, chunk c of row t at c ^ ((t >> 1) & 7)
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int g = lane >> 4, l16 = lane & 15, e = l16 >> 2, q = l16 & 3;
  const int n_ht = (int)((p.H + HW - 1) / HW);
  const int ht = bid % n_ht, s = bid / n_ht;
  const int64_t h0 = (int64_t)ht * HW;
  const int64_t k_begin = (int64_t)s * p.kslice;
  int64_t k_end = k_begin + p.kslice;
  if (k_end > p.ucols) k_end = p.ucols;
  float* out = p.dHp + (int64_t)s * p.part_stride;

  f32x4_t acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // per thread: WL chunks of the W stage (row r = tid / CPR + (256 / CPR) i, chunk tid % CPR), NT / 32 chunks of the dS stage
  const int wc = tid % CPR;
  const int64_t wcol = (h0 + wc * 8 < p.H) ? h0 + wc * 8 : 0;  // (columns beyond H: any in-bounds address; results are not stored)
  constexpr int BL = NT * 8 / 256;
  u32x4_t pw[WL], pb[BL];
  auto fetch = [&](int64_t k0) {
#pragma unroll
    for (int i = 0; i < WL; ++i) {
      const int r = tid / CPR + (256 / CPR) * i;
      int64_t v = Perm::vocab_at(k0 + r);
      v = v < p.vrows ? v : p.vrows - 1;  // dS is zero in such a column
      pw[i] = *reinterpret_cast<const u32x4_t*>(p.W + v * p.ldw + wcol);
    }
#pragma unroll
    for (int i = 0; i < BL; ++i) {
      const int id = tid + i * 256, t = id >> 3, c = id & 7;
      pb[i] = *reinterpret_cast<const u32x4_t*>(p.dS + (int64_t)t * p.ldS + k0 + c * 8);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < WL; ++i) {
      const int r = tid / CPR + (256 / CPR) * i;
      *reinterpret_cast<u32x4_t*>(sA + r * RB + ((wc ^ fw_swz(r)) * 16)) = pw[i];
    }
#pragma unroll
    for (int i = 0; i < BL; ++i) {
      const int id = tid + i * 256, t = id >> 3, c = id & 7;
      *reinterpret_cast<u32x4_t*>(sB + t * 128 + ((c ^ ((t >> 1) & 7)) * 16)) = pb[i];
    }
  };
  if (k_begin < k_end) fetch(k_begin);
  for (int64_t k0 = k_begin; k0 < k_end; k0 += 64) {
    __syncthreads();
    stash();
    __syncthreads();
    if (k0 + 64 < k_end) fetch(k0 + 64);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      u32x4_t af[MI], bf[NJ];
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int col = WH * wave + 16 * i + 4 * q;
        const int r0 = 32 * ks + 8 * g + e, r1 = r0 + 4;
        const u32x2_t lo = tr_read_b64(sA + r0 * RB + (((col >> 3) ^ fw_swz(r0)) * 16) + (col & 7) * 2);
        const u32x2_t hi = tr_read_b64(sA + r1 * RB + (((col >> 3) ^ fw_swz(r1)) * 16) + (col & 7) * 2);
        af[i] = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
      }
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int t = 16 * j + l16, c = 4 * ks + g;  // k = 32 ks + 8 g .. +7 of token row t
        bf[j] = *reinterpret_cast<const u32x4_t*>(sB + t * 128 + ((c ^ ((t >> 1) & 7)) * 16));
      }
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) mma16<TIN>(acc[i][j], af[i], bf[j]);
    }
  }
  // lane (g, l16): h = h0 + WH wave + 16 i + 4 g + (0..3) of token row 16 j + l16
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int t = 16 * j + l16;
    if (t >= p.nt) continue;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      const int64_t h = h0 + WH * wave + 16 * i + 4 * g;
      if (h >= p.H) continue;  // (H is a multiple of 4)
      float* dst = out + (int64_t)t * p.H + h;
      f32x4_t v = acc[i][j];
      if (p.accumulate) v += *reinterpret_cast<const f32x4_t*>(dst);
      *reinterpret_cast<f32x4_t*>(dst) = v;
    }
  }
}

// KT / NT: token positions (64 up to 64 tokens, else 128); HW: columns of H per tile (256 up to 64 tokens, else 128,
// which keeps the accumulators and the tile in flight within 128 registers a lane)
template <int KT>
struct FewShape {
  static constexpr int NT = KT, HW = KT <= 64 ? 256 : 128, HW_DW = HW;
  static constexpr int DW = KT * 128 + KT * HW_DW * 2 + HW_DW * 128;  // dS tile, hidden tile, the four waves' store tiles
  static constexpr int DH = 64 * HW * 2 + NT * 128;
  static constexpr int LDS_BYTES = DW > DH ? DW : DH;
};

// One launch: the d_weight workgroups (the writers) first, then the d_hidden workgroups (the readers); the two
// streams overlap in time.
template <typename TIN, typename TOUT, typename Perm, int KT>
__global__ __launch_bounds__(256, 2) void lce_bwd_few_kernel(FewArgs<TIN> p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  typedef FewShape<KT> S;
  const int bid = blockIdx.x;
  if (bid < p.n_dw) dw_few_tile<TIN, TOUT, Perm, KT, S::HW_DW>(p, bid, lds);
  else dh_few_tile<TIN, Perm, S::NT, S::HW>(p, bid - p.n_dw, lds);
}

// ------------------------------------------------------------------------------------------------------------------
// d_logits of a vocabulary chunk from logits that the forward kept (tokens up to half the hidden size): what the
// d_logits tiles compute from their accumulators, here from x[t * ldx + v], element by element with the same
// expressions, so the same bits.  One pass over 4 bytes per logit instead of a pass over W.  Workgroup b owns the 64
// columns [64 b, 64 b + 64) of dS, which lie within one group of the vocabulary order Perm (a whole group of the
// eight-wave tiles' order, half a group of the 16x16x32 tiles'), and the first `nrows` compact token positions: rows
// beyond the tokens that take part and columns beyond the chunk's rows (the grid covers whole 256-row tiles) are
// written as zeros, as the tiles write them.  Eight lanes share a position: they read the 256 bytes of its token's
// logits behind the 64 columns and write 128 bytes of dS.
// p: the chunk's DsArgs (W, h, the tile map and the range are not used); x: the kept logit of the chunk's first row
// for token 0.
// ------------------------------------------------------------------------------------------------------------------
template <typename TIN, typename Perm>
__global__ __launch_bounds__(256) void ds_from_logits_kernel(DsArgs<TIN> p, const float* x, int64_t ldx, int nrows) {
  static_assert(sizeof(TIN) == 2 && Perm::GV % 64 == 0, "16-bit d_logits, groups of the vocabulary order in multiples of 64 rows");
  const int tid = threadIdx.x, c = tid & 7;
  const int64_t u0 = (int64_t)blockIdx.x * 64;   // first of this workgroup's 64 columns of dS
  const int64_t g0 = u0 - u0 % Perm::GV;         // first row (= first column) of their group of the vocabulary order
  const int64_t Tc = p.n_rows ? (int64_t)*p.n_rows : p.T;
  for (int pos = tid >> 3; pos < nrows; pos += 32) {
    float lse2 = 0.f, C0 = 0.f, C1 = 0.f, G = 0.f;
    int64_t tok = -1;
    int rel = -1;
    if (pos < Tc) {
      tok = p.rows ? (int64_t)p.rows[pos] : pos;
      const float glp = p.g_lp[tok * p.g_lp_stride] * p.g_lp_scale;
      const float gent = p.g_ent ? p.g_ent[tok] : 0.f;
      const TokenConsts k = token_consts(glp, gent, p.maximum[tok], p.accumulate[tok], p.entropy_b[tok], p.rcp_tau);
      lse2 = k.lse2; G = k.G; C1 = k.C1; C0 = k.C0;
      const int64_t y = p.labels[tok] - p.v0;
      rel = (p.label_outside != 1 && y >= g0 && y < g0 + Perm::GV) ? (int)(y - g0) : -1;
    }
    // columns c * 8 + (0..3) and c * 8 + (4..7) of the workgroup's 64 are two runs of four consecutive vocabulary rows
    // (both orders Perm keep what one lane of a d_logits tile holds together: four consecutive rows per register quad),
    // and the cache's rows are padded to whole groups, so each run is one aligned 16-byte load
    float xv[8];
    int row[8];  // vocabulary row relative to the group's first
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const int r0 = (int)(Perm::vocab_at(u0 + c * 8 + 4 * hf) - g0);
      f32x4_t v = {0.f, 0.f, 0.f, 0.f};
      if (tok >= 0 && g0 + r0 < p.vrows) v = *reinterpret_cast<const f32x4_t*>(x + tok * ldx + g0 + r0);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        row[4 * hf + e] = r0 + e;
        xv[4 * hf + e] = v[e];
      }
    }
    float d[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const bool dead = tok < 0 || g0 + row[e] >= p.vrows;
      d[e] = dlogit<true>(dead ? 0.f : xv[e], p.c, lse2, C0, C1, G, row[e] == rel, dead, p.label_outside == 2);
    }
    store_run<TIN, 8>(p.dS + (int64_t)pos * p.ldS + u0 + c * 8, d);
  }
}

}  // namespace lce
