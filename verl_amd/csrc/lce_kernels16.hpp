// The fused kernels on the four-wave 16x16x32 mainloop (gemm_core16.hpp): same arguments, same results layout
// and the same orientation as lce_kernels.hpp (MFMA rows = vocabulary, MFMA columns = tokens, so a lane owns
// whole tokens), with the accumulator layout of the 16 x 16 blocks: in block (i, j) of a wave tile lane l holds
// token 16 j + l % 16 and the vocabulary rows 16 i + 4 (l / 16) + r, r = 0..3.
#pragma once
#include "gemm_core16.hpp"
#include "lce_kernels.hpp"

namespace lce {

// K order of the backward's private intermediates (see KPerm in lce_kernels.hpp): inside each group of 128
// vocabulary rows (one wave tile) the entries are ordered so that what a lane holds of two neighbouring blocks is one
// 16-byte run and the four lane groups follow each other (64 contiguous bytes per token and store instruction):
// row v = 16 i + 4 g + r  ->  position 32 (i / 2) + 8 g + 4 (i % 2) + r.  Tokens keep their order.
template <typename TIN, int TR>
struct KPerm<GemmCfg16<TIN, TR>> {
  static constexpr int GT = 128, GV = 128;
  static __host__ __device__ __forceinline__ int64_t token(int64_t t) { return t; }
  static __host__ __device__ __forceinline__ int64_t token_at(int64_t u) { return u; }
  static __host__ __device__ __forceinline__ int64_t vocab(int64_t v) {
    const int64_t l = v % GV, i = l / 16, w = l % 16;
    return v - l + (i / 2) * 32 + (w / 4) * 8 + (i % 2) * 4 + (w % 4);
  }
  static __host__ __device__ __forceinline__ int64_t vocab_at(int64_t u) {
    const int64_t l = u % GV, ip = l / 32, rem = l % 32, g = rem / 8, ih = (rem % 8) / 4, r = rem % 4;
    return u - l + (2 * ip + ih) * 16 + 4 * g + r;
  }
};

// ------------------------------------------------------------------------------------------------
// forward
// ------------------------------------------------------------------------------------------------
// folds one finished tile into the running per-token statistics (FULL: no padded vocabulary rows in the tile)
template <typename Cfg, bool FULL>
LCE_DEV void fwd16_fold(const FwdArgs<typename Cfg::TIN>& p, const f32x4_t (&acc)[Cfg::NB][Cfg::NB], float (&m)[Cfg::NB],
                        float (&a)[Cfg::NB], float (&b)[Cfg::NB], const int (&lab)[Cfg::NB], int vbase, int vend, int64_t tok0, int g4,
                        int l16) {
  constexpr int NB = Cfg::NB;
  // The running statistics do not live in registers across the K loop (256 accumulator and 256 ordinary registers are
  // in use there; the compiler keeps them in scratch memory meanwhile).  All of them are asked for here, so that they
  // come back in one batch of loads instead of column by column, each column waiting for its own (forward at 16384
  // tokens: H=896 4.57 -> 4.43 ms, H=1536 6.39 -> 6.28, H=3584 12.91 -> 12.85).
#pragma unroll
  for (int j = 0; j < NB; ++j) asm volatile("" : "+v"(m[j]), "+v"(a[j]), "+v"(b[j]));
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    __builtin_amdgcn_sched_barrier(0);  // one block column at a time (register pressure)
    float x[NB * 4];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = acc[i][j][r];
        if (!FULL && vbase + 16 * i + 4 * g4 + r >= vend) v = -INFINITY;  // padded vocabulary rows
        x[i * 4 + r] = v;
      }
    // four independent chains each for the maximum and the two sums: one wave per SIMD has no neighbour to hide the
    // latency of a dependent chain of 32
    float t4[4] = {x[0], x[1], x[2], x[3]};
#pragma unroll
    for (int q = 4; q < NB * 4; ++q) t4[q & 3] = fmaxf(t4[q & 3], x[q]);
    const float tmax = fmaxf(fmaxf(t4[0], t4[1]), fmaxf(t4[2], t4[3]));
    const float mn = fmaxf(m[j], tmax);
    const float sc = fast_exp2((m[j] - mn) * p.c);
    const float mc = mn * p.c;
    m[j] = mn;
    float a4[4] = {a[j] * sc, 0.f, 0.f, 0.f}, b4[4] = {b[j] * sc, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < NB * 4; ++q) {
      const float e = fast_exp2(__builtin_fmaf(x[q], p.c, -mc));
      a4[q & 3] += e;
      // padded rows: -inf in the log-sum-exp, 0 in the sum of x * exp
      b4[q & 3] = __builtin_fmaf(FULL ? x[q] : (x[q] == -INFINITY ? 0.f : x[q]), e, b4[q & 3]);
    }
    const float aj = (a4[0] + a4[1]) + (a4[2] + a4[3]), bj = (b4[0] + b4[1]) + (b4[2] + b4[3]);
    a[j] = aj;
    b[j] = bj;
    // label logit: rare (a token's label falls in this wave tile with probability WM / V)
    const int rel = lab[j] - vbase;
    const bool mine = lab[j] >= 0 && lab[j] < vend && rel >= 0 && rel < Cfg::WM && (((rel >> 2) & 3) == g4);
    if (__builtin_amdgcn_ballot_w64(mine) != 0) {
      float pick = 0.f;
#pragma unroll
      for (int q = 0; q < NB * 4; ++q)
        if (mine && 16 * (q >> 2) + (q & 3) == (rel & ~12)) pick = x[q];
      // exactly one lane in the whole grid owns a token's label: plain store, no merge needed
      if (mine) p.xlabel[tok0 + j * 16 + l16] = pick;
    }
  }
}

// KEEP: the tiles also write their logits to p.xcache (FwdArgs), for a backward that then does not recompute them
template <typename Cfg, bool KEEP>
LCE_DEV void fwd16_body(const FwdArgs<typename Cfg::TIN>& p, char* lds) {
  constexpr int NB = Cfg::NB;
  int tt, s;
  if (!p.map.decode(blockIdx.x, tt, s)) return;
  const int64_t n0 = (int64_t)tt * Cfg::BN;
  const int lane = threadIdx.x & 63, g4 = lane >> 4, l16 = lane & 15;
  GemmCore16<Cfg> g;
  g.set_lane();

  float m[NB], a[NB], b[NB];
  int lab[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    m[j] = kNegBig;
    a[j] = 0.f;
    b[j] = 0.f;
    const int64_t t = n0 + g.wave_n * Cfg::WN + j * 16 + l16;
    const int64_t y = t < p.T ? p.labels[t] - p.label_offset : -1;
    lab[j] = (y >= 0 && y < p.V) ? (int)y : -1;
  }

  f32x4_t acc[NB][NB];
  const int64_t row0 = (int64_t)s * p.split_stride;
  const int64_t vend64 = row0 + p.split_span < p.V ? row0 + p.split_span : p.V;
  const int vend = (int)vend64;
  g.init(p.W, p.ldw, row0, vend64, p.h, p.ldh, n0, p.T);
  g.prologue(lds, p.H);
  for (int64_t m0 = row0; m0 < vend64; m0 += p.tile_step) {
    g.main(lds, p.H, acc);
    const int vbase = (int)m0 + g.wave_m * Cfg::WM;  // vocabulary index of this wave's first row
    const bool full = m0 + Cfg::BM <= vend64;
    if constexpr (KEEP) {
      // a lane holds four consecutive vocabulary rows of a token per block: one 16-byte store.  Issued AHEAD of the next
      // tile's first loads: the K loop waits on counts of outstanding vector-memory operations, and with the stores older
      // than every load it waits for, those counts mean what they say.  The count is a 6-bit field: the stores are
      // issued 16 at a time and so many are waited for that, with the prologue's 32 loads behind them, fewer than 64
      // operations are ever in flight.
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int64_t t = n0 + g.wave_n * Cfg::WN + j * 16 + l16;
        if (t < p.T) {
          float* dst = p.xcache + t * p.ldx;
#pragma unroll
          for (int i = 0; i < NB; ++i) {
            const int v = vbase + 16 * i + 4 * g4;
            if (v + 3 < vend) {
              *reinterpret_cast<f32x4_t*>(dst + v) = acc[i][j];
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r)
                if (v + r < vend) dst[v + r] = acc[i][j][r];
            }
          }
        }
        if (!full) {  // (a tile at the end of its split: up to four single stores per block)
          __builtin_amdgcn_sched_barrier(0);
          GemmCore16<Cfg>::template wait_vm<0>();
        } else if (j % 2 == 1 && j >= 3) {
          __builtin_amdgcn_sched_barrier(0);
          if (j == NB - 1) GemmCore16<Cfg>::template wait_vm<24>();
          else GemmCore16<Cfg>::template wait_vm<32>();
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // the next tile's first slabs fly while this tile's statistics are folded in
    __syncthreads();  // every wave is past its last LDS read and has drained its own loads
    if (m0 + p.tile_step < vend64) {
      g.init(p.W, p.ldw, m0 + p.tile_step, vend64, p.h, p.ldh, n0, p.T);
      g.prologue(lds, p.H);
    }
    if (full) fwd16_fold<Cfg, true>(p, acc, m, a, b, lab, vbase, vend, n0 + g.wave_n * Cfg::WN, g4, l16);
    else fwd16_fold<Cfg, false>(p, acc, m, a, b, lab, vbase, vend, n0 + g.wave_n * Cfg::WN, g4, l16);
  }
  __syncthreads();

  // merge the four lane groups (same token, different vocabulary rows), then the two waves along the vocabulary
  f32x4_t* red = reinterpret_cast<f32x4_t*>(lds);  // [WAVES_M][BN]
#pragma unroll
  for (int j = 0; j < NB; ++j) {
#pragma unroll
    for (int off = 16; off <= 32; off <<= 1) {
      const float m2 = __shfl_xor(m[j], off), a2 = __shfl_xor(a[j], off), b2 = __shfl_xor(b[j], off);
      merge_stats(m[j], a[j], b[j], m2, a2, b2, p.c);
    }
    if (g4 == 0) {
      const f32x4_t v = {m[j], a[j], b[j], 0.f};
      red[g.wave_m * Cfg::BN + g.wave_n * Cfg::WN + j * 16 + l16] = v;
    }
  }
  __syncthreads();
  for (int t = threadIdx.x; t < Cfg::BN; t += Cfg::NTHREADS) {
    const f32x4_t v0 = red[t];
    float vm = v0[0], va = v0[1], vb = v0[2];
#pragma unroll
    for (int w = 1; w < Cfg::WAVES_M; ++w) {
      const f32x4_t u = red[w * Cfg::BN + t];
      merge_stats(vm, va, vb, u[0], u[1], u[2], p.c);
    }
    const int64_t tok = n0 + t;
    const f32x4_t v = {vm, va, vb, 0.f};
    if (tok < p.T) p.parts[(int64_t)s * p.T + tok] = v;
  }
}

// ------------------------------------------------------------------------------------------------
// backward: d_logits tiles
// ------------------------------------------------------------------------------------------------
// per-position constants of the d_logits tiles (see DsArgs::tokc)
inline __global__ void ds_token_consts_kernel(const int* rows, const int* n_rows, int64_t T, int64_t tpad, const float* g_lp, int64_t g_lp_stride,
                                       float g_lp_scale, const float* g_ent, const float* maximum, const float* accumulate,
                                       const float* entropy_b, const int64_t* labels, int64_t vocab_offset, int64_t V, float rcp_tau,
                                       f32x4_t* tokc, int* tokl) {
  const int64_t pos = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (pos >= tpad) return;
  const int64_t Tc = n_rows ? (int64_t)*n_rows : T;
  f32x4_t c = {1.0e30f, 0.f, 0.f, 0.f};
  int lab = -1;
  if (pos < Tc) {
    const int64_t tok = rows ? (int64_t)rows[pos] : pos;
    const float glp = g_lp[tok * g_lp_stride] * g_lp_scale;
    const float gent = g_ent ? g_ent[tok] : 0.f;
    const TokenConsts k = token_consts(glp, gent, maximum[tok], accumulate[tok], entropy_b[tok], rcp_tau);
    c[0] = k.lse2;
    c[1] = k.C0;
    c[2] = k.C1;
    c[3] = k.G;
    const int64_t y = labels[tok] - vocab_offset;
    lab = (y >= 0 && y < V) ? (int)y : -1;
  }
  tokc[pos] = c;
  tokl[pos] = lab;
}

// One finished tile: d_logits of the wave's 128 tokens x 128 vocabulary entries, written to dS straight from the
// registers: a lane holds 8 consecutive positions of the wave tile's vocabulary order per pair of blocks, the four lane
// groups 64 contiguous bytes of a token's row.  (Staging the tile through LDS for whole 256-byte runs per instruction
// was measured 9% slower on the pass: 3.64 against 3.31 ms per 38144-row chunk of config 2.)
// LABEL: some token of the wave tile has its label among the tile's rows: the one lane that holds that entry patches
// it after the common arithmetic (zero when the label's entry is kept out of the tiles, + G when everything is inside).
// EDGE: the tile reaches beyond the chunk's last row; those entries are zeros.
template <typename Cfg, bool LABEL, bool EDGE>
LCE_DEV void ds16_epilogue(const DsArgs<typename Cfg::TIN>& p, const f32x4_t (&acc)[Cfg::NB][Cfg::NB], const f32x4_t (&tc)[Cfg::NB],
                           const int (&lab)[Cfg::NB], int64_t tok0, int vloc0, int g4, int l16) {
  typedef typename Cfg::TIN TIN;
  constexpr int NB = Cfg::NB;
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const float lse2 = tc[j][0], C0 = tc[j][1], C1 = tc[j][2], G = tc[j][3];
    // the label's entry: block pair rel / 32, lane group (rel / 4) % 4, value 4 ((rel / 16) % 2) + rel % 4 of the run
    const int rel = (LABEL && p.label_outside != 1) ? lab[j] - (int)p.lab0 - vloc0 : -1;  // (1: the tiles hold the softmax terms only)
    const int own_ip = (rel >= 0 && rel < Cfg::WM && ((rel >> 2) & 3) == g4) ? rel >> 5 : -1;
    const int own_q = ((rel >> 4) & 1) * 4 + (rel & 3);
    const int64_t tok = tok0 + j * 16 + l16;
#pragma unroll
    for (int ip = 0; ip < NB / 2; ++ip) {
      float d[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const int i = 2 * ip + (q >> 2), r = q & 3;
        d[q] = dlogit<false>(acc[i][j][r], p.c, lse2, C0, C1, G, false, false, false);
        if (EDGE && vloc0 + 16 * i + 4 * g4 + r >= p.vrows) d[q] = 0.f;
      }
      if (LABEL) {
        const bool mine = own_ip == ip;
        if (__builtin_amdgcn_ballot_w64(mine) != 0) {
#pragma unroll
          for (int q = 0; q < 8; ++q)
            if (mine && q == own_q) d[q] = p.label_outside == 2 ? 0.f : d[q] + G;
        }
      }
      // rows of positions without a token are zeros (their constants make them so); they pad the d_weight GEMM's K
      if (tok < p.tpad) store_run<TIN, 8>(p.dS + tok * p.ldS + vloc0 + ip * 32 + g4 * 8, d);
    }
  }
}

// One workgroup per tile.  (Workgroups that walk strips of 2, 4 or 8 consecutive vocabulary tiles, with the first loads
// of the next tile in flight while the finished one is written out, took the same time on the pass alone and more inside
// the backward's combined launch, whose tail then is a strip long.)
template <typename Cfg>
LCE_DEV void ds16_tile(const DsArgs<typename Cfg::TIN>& p, int bid, char* lds) {
  constexpr int NB = Cfg::NB;
  const int64_t Tc = p.n_rows ? (int64_t)*p.n_rows : p.T;  // tokens that take part
  int tt, vt;
  const TileMap map = p.n_rows ? p.map.with_rows((int)((Tc + Cfg::BN - 1) / Cfg::BN)) : p.map;
  if (!map.decode(bid, tt, vt)) return;
  const int64_t n0 = (int64_t)tt * Cfg::BN;
  const int lane = threadIdx.x & 63, g4 = lane >> 4, l16 = lane & 15;
  GemmCore16<Cfg> g;
  g.set_lane();
  const int64_t tok0 = n0 + g.wave_n * Cfg::WN;  // first position of this wave's group
  f32x4_t tc[NB];
  int lab[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int64_t pos = tok0 + j * 16 + l16;
    tc[j] = f32x4_t{1.0e30f, 0.f, 0.f, 0.f};
    lab[j] = -1;
    if (pos < p.tpad) {
      tc[j] = p.tokc[pos];
      lab[j] = p.tokl[pos];
    }
  }
  g.init(p.W, p.ldw, (int64_t)vt * Cfg::BM, p.vrows, p.h, p.ldh, n0, Tc, p.rows);
  f32x4_t acc[NB][NB];
  g.run(lds, p.H, acc);
  const int vloc0 = vt * Cfg::BM + g.wave_m * Cfg::WM;  // chunk-local vocabulary index of this wave's first row
  // fast path: no padded vocabulary rows and no label in the wave tile
  bool has_label = false;
  if (p.label_outside != 1) {
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int rel = lab[j] - (int)p.lab0 - vloc0;
      has_label |= (rel >= 0 && rel < Cfg::WM);
    }
  }
  const bool labels_here = __builtin_amdgcn_ballot_w64(has_label) != 0;
  // Labels kept out of the tiles altogether (label_outside == 2, the default): the tile is written by the common
  // path, and the lane that stored a label's entry then overwrites it with a zero (same lane, same address, later
  // store).  Measured on a 38144-column chunk of config 2, where one wave tile in nine holds a label: 3.71 -> 3.58 ms
  // against patching inside the common arithmetic.  With the one-hot part inside the tile (0) the patch adds G there.
  const bool in_tile = labels_here && p.label_outside == 0;
  const bool edge = vloc0 + Cfg::WM > p.vrows;
  if (edge && in_tile) ds16_epilogue<Cfg, true, true>(p, acc, tc, lab, tok0, vloc0, g4, l16);
  else if (edge) ds16_epilogue<Cfg, false, true>(p, acc, tc, lab, tok0, vloc0, g4, l16);
  else if (in_tile) ds16_epilogue<Cfg, true, false>(p, acc, tc, lab, tok0, vloc0, g4, l16);
  else ds16_epilogue<Cfg, false, false>(p, acc, tc, lab, tok0, vloc0, g4, l16);
  if (labels_here && p.label_outside == 2) {
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int rel = lab[j] - (int)p.lab0 - vloc0;  // = 16 i + 4 g + r inside the wave tile
      const int64_t tok = tok0 + j * 16 + l16;
      if (rel >= 0 && rel < Cfg::WM && ((rel >> 2) & 3) == g4 && tok < p.tpad)
        p.dS[tok * p.ldS + vloc0 + (rel >> 5) * 32 + g4 * 8 + ((rel >> 4) & 1) * 4 + (rel & 3)] = (typename Cfg::TIN)0.f;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// plain GEMMs.  The MFMA rows are taken from the operand that indexes the CONTIGUOUS dimension of C, so that
// the four accumulator registers of a block are four neighbours in a row of C (one 16-byte or 8-byte access):
// for C[m][n] = sum_k A[m][k] B[n][k] lane l holds m = 16 j + l % 16 and n = 16 i + 4 (l / 16) + r.
// ------------------------------------------------------------------------------------------------
template <typename Cfg, int MODE, bool EDGE>
LCE_DEV void gemm16_epilogue(const GemmArgs<typename Cfg::TIN>& p, const f32x4_t (&acc)[Cfg::NB][Cfg::NB], int64_t mw, int64_t nw) {
  typedef typename Cfg::TIN TIN;
  // mw, nw: this lane's row of block column 0 and its first column of block row 0
  // accumulate modes: the old values of block column j + 1 are fetched before column j is added and stored, so that
  // a lane always has eight 16-byte loads in flight (measured on the d_hidden GEMM of one 8192-column chunk, 16384 x
  // 3584 x 8192: 0.900 -> 0.875 ms; the same GEMM storing without reading takes 0.837)
  f32x4_t prev[2][Cfg::NB];
  auto fetch = [&](int j) {
    const int64_t m = mw + j * 16;
#pragma unroll
    for (int i = 0; i < Cfg::NB; ++i) {
      const int64_t n = nw + i * 16;
      prev[j & 1][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (!(EDGE && (m >= p.M || n >= p.N))) prev[j & 1][i] = *reinterpret_cast<const f32x4_t*>(p.Cf + m * p.ldcf + n);
    }
  };
  if (MODE & 1) fetch(0);
#pragma unroll
  for (int j = 0; j < Cfg::NB; ++j) {
    const int64_t m = mw + j * 16;
    if ((MODE & 1) && j + 1 < Cfg::NB) fetch(j + 1);
    if (EDGE && m >= p.M) continue;
#pragma unroll
    for (int i = 0; i < Cfg::NB; ++i) {
      const int64_t n = nw + i * 16;
      if (EDGE && n >= p.N) continue;  // (N is a multiple of 4)
      f32x4_t v = acc[i][j];
      if (MODE & 1) {
        v += prev[j & 1][i];
      }
      if (MODE & 2) {
        typedef typename VecOf<TIN, 4>::type vec_t;
        vec_t o;
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = (TIN)v[r];
        *reinterpret_cast<vec_t*>(p.Ct + m * p.ldct + n) = o;
      } else {
        *reinterpret_cast<f32x4_t*>(p.Cf + m * p.ldcf + n) = v;
      }
    }
  }
}

// CoreCfg: Cfg itself, or its mixed twin GemmCfg16<TIN, 2>: then B is K-major as it lies in memory, B[k][n] with row
// stride ldb, its rows in the order KPerm<Cfg>::vocab_at of A's columns (the d_hidden GEMM reading W in place: no W^T);
// rows of B at or beyond p.b_rows_valid do not exist (A is zero in those columns).
template <typename Cfg, typename CoreCfg = Cfg>
LCE_DEV void gemm16_tile(const GemmArgs<typename Cfg::TIN>& pin, int bid, char* lds) {
  GemmArgs<typename Cfg::TIN> p = pin;
  if (p.m_dev) {
    const int64_t m = *p.m_dev;
    p.M = m < p.M ? m : p.M;
  }
  if (p.k_dev) {
    const int64_t k = ((int64_t)*p.k_dev + p.k_gran - 1) / p.k_gran * p.k_gran;
    p.K = k < p.K ? k : p.K;
  }
  int64_t k0 = 0, k1 = p.K;
  if (p.ksplit > 1) {
    const int s = bid / p.map.total;  // (the grid holds ksplit copies of the host-sized map)
    bid -= s * p.map.total;
    k0 = s * p.kslice;
    k1 = k0 + p.kslice < p.K ? k0 + p.kslice : p.K;
    p.Cf += s * p.cf_split_stride;
  }
  int tm, tn;
  const TileMap map = p.m_dev ? p.map.with_rows((int)((p.M + Cfg::BM - 1) / Cfg::BM)) : p.map;
  if (!map.decode(bid, tm, tn)) return;
  const int64_t m0 = (int64_t)tm * Cfg::BM, n0 = (int64_t)tn * Cfg::BN;
  GemmCore16<CoreCfg> g;
  f32x4_t acc[Cfg::NB][Cfg::NB];
  if (k0 < k1 && (CoreCfg::TRANS != 2 || k0 < p.b_rows_valid)) {
    // MFMA rows = n, MFMA columns = m
    if constexpr (CoreCfg::TRANS == 2)
      g.init_mixed(p.B + k0 * p.ldb, p.ldb, n0, p.N - n0, p.b_rows_valid - k0, [](int r) { return KPerm<Cfg>::vocab_at(r); }, p.A + k0, p.lda,
                   m0, p.M);
    else
      g.init(p.B + k0, p.ldb, n0, p.N, p.A + k0, p.lda, m0, p.M);
    g.run(lds, k1 - k0, acc);
  } else {  // empty K range: contributes zero (and still initialises what it owns)
    if (p.out_mode == 1) return;
    g.set_lane();
#pragma unroll
    for (int i = 0; i < Cfg::NB; ++i)
#pragma unroll
      for (int j = 0; j < Cfg::NB; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  const int64_t mw = m0 + g.wave_n * Cfg::WN + (g.lane & 15), nw = n0 + g.wave_m * Cfg::WM + 4 * (g.lane >> 4);
  const bool edge = m0 + Cfg::BM > p.M || n0 + Cfg::BN > p.N;
#define LCE_EPI16(MODE)                                             \
  if (edge) gemm16_epilogue<Cfg, MODE, true>(p, acc, mw, nw);       \
  else gemm16_epilogue<Cfg, MODE, false>(p, acc, mw, nw)
  switch (p.out_mode) {
    case 0: LCE_EPI16(0); break;
    case 1: LCE_EPI16(1); break;
    case 2: LCE_EPI16(2); break;
    default: LCE_EPI16(3); break;
  }
#undef LCE_EPI16
}

// C[m][n] = sum_k A[k][m] * B[k][n], both operands K-major and allocated in whole 256-column tiles, K (or *k_dev
// rounded up to k_gran) a multiple of 64.  out_mode 0: Cf = acc; out_mode 2: Ct[PermCfg's vocab_at(m)][n] = (TIN)acc
// (the rows of C are A's columns, which the d_logits epilogue leaves in KPerm::vocab order).
template <typename Cfg, typename PermCfg>
LCE_DEV void gemm16_tn_tile(const GemmArgs<typename Cfg::TIN>& pin, int bid, char* lds) {
  typedef typename Cfg::TIN TIN;
  GemmArgs<TIN> p = pin;
  if (p.k_dev) {
    const int64_t k = ((int64_t)*p.k_dev + p.k_gran - 1) / p.k_gran * p.k_gran;
    p.K = k < p.K ? k : p.K;
  }
  int tm, tn;
  if (!p.map.decode(bid, tm, tn)) return;
  const int64_t m0 = (int64_t)tm * Cfg::BM, n0 = (int64_t)tn * Cfg::BN;
  GemmCore16<Cfg> g;
  f32x4_t acc[Cfg::NB][Cfg::NB];
  if (p.K > 0) {
    g.init_tn(p.B, p.ldb, n0, p.A, p.lda, m0);  // MFMA rows = n, MFMA columns = m
    g.run(lds, p.K, acc);
  } else {
    g.set_lane();
#pragma unroll
    for (int i = 0; i < Cfg::NB; ++i)
#pragma unroll
      for (int j = 0; j < Cfg::NB; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  const int64_t nw = n0 + g.wave_m * Cfg::WM + 4 * (g.lane >> 4);
#pragma unroll
  for (int j = 0; j < Cfg::NB; ++j) {
    const int u = g.wave_n * Cfg::WN + j * 16 + (g.lane & 15);  // row inside the tile, in the operand's column order
    const int64_t m = m0 + ((p.out_mode == 2 || p.perm_rows) ? (int64_t)KPerm<PermCfg>::vocab_at(u) : (int64_t)u);
    if (m >= p.M) continue;
#pragma unroll
    for (int i = 0; i < Cfg::NB; ++i) {
      const int64_t n = nw + i * 16;
      if (n >= p.N) continue;  // (N is a multiple of 4)
      if (p.out_mode == 2) {
        typedef typename VecOf<TIN, 4>::type vec_t;
        vec_t o;
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = (TIN)acc[i][j][r];
        *reinterpret_cast<vec_t*>(p.Ct + m * p.ldct + n) = o;
      } else {
        *reinterpret_cast<f32x4_t*>(p.Cf + m * p.ldcf + n) = acc[i][j];
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// kernels
// ------------------------------------------------------------------------------------------------
template <typename Cfg, bool KEEP = false>
__global__ __launch_bounds__(Cfg::NTHREADS) void lce_fwd16_kernel(FwdArgs<typename Cfg::TIN> p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  fwd16_body<Cfg, KEEP>(p, lds);
}

template <typename Cfg>
__global__ __launch_bounds__(Cfg::NTHREADS) void gemm16_nt_kernel(GemmArgs<typename Cfg::TIN> p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  gemm16_tile<Cfg>(p, blockIdx.x, lds);
}

template <typename Cfg>
__global__ __launch_bounds__(Cfg::NTHREADS) void gemm16_tn_kernel(GemmArgs<typename Cfg::TIN> p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  gemm16_tn_tile<GemmCfg16<typename Cfg::TIN, 1>, Cfg>(p, blockIdx.x, lds);
}

template <typename Cfg>
LCE_DEV void any_gemm16_tile(const GemmArgs<typename Cfg::TIN>& p, int bid, char* lds) {
  if (p.tn == 1) gemm16_tn_tile<GemmCfg16<typename Cfg::TIN, 1>, Cfg>(p, bid, lds);
  else if (p.tn == 2) gemm16_tile<Cfg, GemmCfg16<typename Cfg::TIN, 2>>(p, bid, lds);
  else gemm16_tile<Cfg>(p, bid, lds);
}

// one launch of the backward's steady state (see lce_bwd_chunk_kernel)
template <typename Cfg>
__global__ __launch_bounds__(Cfg::NTHREADS) void lce_bwd_chunk16_kernel(BwdChunkArgs<typename Cfg::TIN> p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int bid = blockIdx.x;
  if (bid < p.n_gw) any_gemm16_tile<Cfg>(p.gw, bid, lds);
  else if (bid < p.n_gw + p.n_gh) any_gemm16_tile<Cfg>(p.gh, bid - p.n_gw, lds);
  else ds16_tile<Cfg>(p.ds, bid - p.n_gw - p.n_gh, lds);
}

}  // namespace lce
