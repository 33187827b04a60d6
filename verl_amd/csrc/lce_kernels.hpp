// Device kernels of the fused lm-head log-prob + entropy path (gfx950).
//
// Orientation used by the fused kernels: the MFMA "A" operand is the weight tile (rows = vocabulary)
// and the "B" operand is the hidden tile (rows = tokens), so the accumulator holds S^T[vocab][token].
// With the 32x32 accumulator layout each lane then owns ONE token per block and 16 vocabulary
// entries of it: max / sum-exp / sum x*exp over the vocabulary are lane-local, and per-token
// constants (statistics, upstream gradients, label) are per-lane scalars.
#pragma once
#include "gemm_core.hpp"

namespace lce {

static constexpr float kLog2e = 1.4426950408889634f;
static constexpr float kLn2 = 0.6931471805599453f;
static constexpr float kNegBig = -1.0e30f;  // running-max seed: finite so that (seed - seed) is 0, not NaN

LCE_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// (m, a, b) partial statistics in raw-accumulator units x (logit = x / tau), c = log2(e) / tau:
// a = sum 2^((x - m) c), b = sum x 2^((x - m) c)
LCE_DEV void merge_stats(float& m, float& a, float& b, float m2, float a2, float b2, float c) {
  const float mn = fmaxf(m, m2);
  const float s1 = fast_exp2((m - mn) * c), s2 = fast_exp2((m2 - mn) * c);
  a = a * s1 + a2 * s2;
  b = b * s1 + b2 * s2;
  m = mn;
}

// vocabulary index (relative to the wave tile's first row) of accumulator register r in block row i
LCE_DEV int acc_row(int i, int r, int hh) { return i * 32 + 8 * (r >> 2) + 4 * hh + (r & 3); }

// ------------------------------------------------------------------------------------------------
// forward: partial statistics per (vocabulary split, token)
// ------------------------------------------------------------------------------------------------
template <typename TIN>
struct FwdArgs {
  const TIN* W;
  int64_t ldw;
  const TIN* h;
  int64_t ldh;
  const int64_t* labels;
  int64_t T, V, H;
  float c;           // log2(e) / temperature
  f32x4_t* parts;    // [S][T] of (m, a, b, unused)
  float* xlabel;     // [T] raw accumulator value at the label: written by the one lane that owns it, left as it was for a
                     // token whose label is not a row of W (the merge kernels do not read it then)
  int S;             // vocabulary splits
  // Split s owns the tiles that start at rows s * split_stride + i * tile_step (i = 0, 1, ...) below its end row
  // min(V, s * split_stride + split_span).  Two layouts: tiles dealt round robin (split_stride = BM, tile_step =
  // S * BM, split_span = V: concurrently running workgroups stay on neighbouring tiles), or one contiguous row
  // range per split (split_stride = split_span = rows per split, tile_step = BM: every split reads the same
  // number of rows of W whatever V is; its last tile is partial).
  int64_t split_stride, tile_step, split_span;
  TileMap map;       // rows = token tiles, cols = splits
  int64_t label_offset;  // W holds vocabulary rows [label_offset, label_offset + V) of a larger vocabulary (0 = all of it)
  // When not null (offered while the tokens are at most half the hidden size), the raw logits h . W[v] (fp32, before the division by the
  // temperature) are kept for the backward, xcache[t * ldx + v] for t < T, v < V (ldx a multiple of 4).
  float* xcache;
  int64_t ldx;
};

template <typename Cfg>
__global__ __launch_bounds__(Cfg::NTHREADS) void lce_fwd_kernel(FwdArgs<typename Cfg::TIN> p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  int tt, s;
  if (!p.map.decode(blockIdx.x, tt, s)) return;
  const int64_t n0 = (int64_t)tt * Cfg::BN;
  const int lane = threadIdx.x & 63, hh = lane >> 5, ln = lane & 31;
  GemmCore<Cfg> g;

  float m[Cfg::FN], a[Cfg::FN], b[Cfg::FN];
  int lab[Cfg::FN];
  {
    const int wave = threadIdx.x >> 6;
    const int wave_n = wave % Cfg::WAVES_N;
#pragma unroll
    for (int j = 0; j < Cfg::FN; ++j) {
      m[j] = kNegBig;
      a[j] = 0.f;
      b[j] = 0.f;
      const int64_t t = n0 + wave_n * Cfg::WN + j * 32 + ln;
      const int64_t y = t < p.T ? p.labels[t] - p.label_offset : -1;
      lab[j] = (y >= 0 && y < p.V) ? (int)y : -1;
    }
  }

  f32x16_t acc[Cfg::FM][Cfg::FN];
  const int64_t row0 = (int64_t)s * p.split_stride;
  const int64_t vend64 = row0 + p.split_span < p.V ? row0 + p.split_span : p.V;
  const int vend = (int)vend64;
  g.init(p.W, p.ldw, row0, vend64, p.h, p.ldh, n0, p.T);
  g.prologue(lds, p.H);
  for (int64_t m0 = row0; m0 < vend64; m0 += p.tile_step) {
    g.main(lds, p.H, acc);
    const int vbase = (int)m0 + g.wave_m * Cfg::WM;  // vocabulary index of this wave's first row
    const bool full = m0 + Cfg::BM <= vend64;
    __builtin_amdgcn_sched_barrier(0);
    {
      // the logits of this tile, for a backward that then has no need to recompute them: a lane holds four consecutive
      // vocabulary rows of a token in four consecutive registers, 16 bytes of that token's row of the cache; the lanes'
      // pieces of a 128-byte line meet in L2.  Issued AHEAD of the next tile's first loads: the K loop waits on counts
      // of outstanding vector-memory operations, and with the stores older than every load it waits for, those counts
      // mean what they say (64 tokens: 209 instead of 187 us, the same as with the stores behind those loads).
      if (p.xcache) {
#pragma unroll
        for (int j = 0; j < Cfg::FN; ++j) {
          const int64_t t = n0 + g.wave_n * Cfg::WN + j * 32 + ln;
          if (t >= p.T) continue;
          float* dst = p.xcache + t * p.ldx;
#pragma unroll
          for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int v = vbase + acc_row(i, 4 * q, hh);
              if (v + 3 < vend) {
                const f32x4_t x4 = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                *reinterpret_cast<f32x4_t*>(dst + v) = x4;  // (non-temporal stores: 222 instead of 209 us)
              } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  if (v + e < vend) dst[v + e] = acc[i][j][4 * q + e];
              }
            }
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // start fetching the next tile's first slabs now: the loads fly while this tile's statistics are
    // folded in (the epilogue touches neither LDS nor vector memory on its common path)
    __syncthreads();  // every wave is past its last LDS read and has drained its own loads
    if (m0 + p.tile_step < vend64) {
      g.init(p.W, p.ldw, m0 + p.tile_step, vend64, p.h, p.ldh, n0, p.T);
      g.prologue(lds, p.H);
    }
    if (!full) {
#pragma unroll
      for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::FN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (vbase + acc_row(i, r, hh) >= vend) acc[i][j][r] = -INFINITY;
    }
#pragma unroll
    for (int j = 0; j < Cfg::FN; ++j) {
      __builtin_amdgcn_sched_barrier(0);  // keep one block column in flight at a time (register pressure)
      float tmax = -INFINITY;
#pragma unroll
      for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, acc[i][j][r]);
      __builtin_amdgcn_sched_barrier(0);
      const float mn = fmaxf(m[j], tmax);
      const float sc = fast_exp2((m[j] - mn) * p.c);
      const float mc = mn * p.c;
      float aj = a[j] * sc, bj = b[j] * sc;
      m[j] = mn;
      if (full) {
#pragma unroll
        for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float x = acc[i][j][r];
            const float e = fast_exp2(__builtin_fmaf(x, p.c, -mc));
            aj += e;
            bj = __builtin_fmaf(x, e, bj);
          }
      } else {
        // padded vocabulary rows: -inf in the log-sum-exp, 0 in the sum of x * exp
#pragma unroll
        for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float x = acc[i][j][r];
            const float e = fast_exp2(__builtin_fmaf(x, p.c, -mc));
            aj += e;
            bj = __builtin_fmaf(x == -INFINITY ? 0.f : x, e, bj);
          }
      }
      a[j] = aj;
      b[j] = bj;
      // label logit: rare (a token's label falls in this wave tile with probability WM / V)
      const int rel = lab[j] - vbase;
      const bool mine = lab[j] >= 0 && lab[j] < vend && rel >= 0 && rel < Cfg::WM && (((rel >> 2) & 1) == hh);
      if (__builtin_amdgcn_ballot_w64(mine) != 0) {
        float pick = 0.f;
#pragma unroll
        for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (mine && acc_row(i, r, hh) == rel) pick = acc[i][j][r];
        // exactly one lane in the whole grid owns a token's label: plain store, no merge needed
        if (mine) p.xlabel[n0 + g.wave_n * Cfg::WN + j * 32 + ln] = pick;
      }
    }
  }
  __syncthreads();

  // merge the two lane halves (same token, different vocabulary rows), then the WAVES_M waves
  f32x4_t* red = reinterpret_cast<f32x4_t*>(lds);  // [WAVES_M][BN]
#pragma unroll
  for (int j = 0; j < Cfg::FN; ++j) {
    const float m2 = __shfl_xor(m[j], 32), a2 = __shfl_xor(a[j], 32), b2 = __shfl_xor(b[j], 32);
    merge_stats(m[j], a[j], b[j], m2, a2, b2, p.c);
    if (hh == 0) {
      f32x4_t v = {m[j], a[j], b[j], 0.f};
      red[g.wave_m * Cfg::BN + g.wave_n * Cfg::WN + j * 32 + ln] = v;
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

// raw logit at the label of token t: what the forward tiles left in xlabel[t], or 0 when the label is not one of the V
// rows of W that start at vocabulary id label_offset (no lane owns such a token, and xlabel[t] holds whatever the
// workspace held before the call)
LCE_DEV float label_logit(const float* xlabel, const int64_t* labels, int64_t label_offset, int64_t V, int64_t t) {
  const int64_t y = labels[t] - label_offset;
  return (y >= 0 && y < V) ? xlabel[t] : 0.f;
}

// merge the S partials of every token and emit the five per-token outputs; LANES (a power of two up
// to 64) threads share a token: each merges every LANES-th partial, then a fixed shuffle tree joins
// them (with few tokens there are hundreds of splits per token and only a handful of tokens)
template <int LANES>
__global__ void lce_fwd_merge_kernel(const f32x4_t* parts, const float* xlabel, const int64_t* labels, int64_t label_offset, int64_t V,
                                     int S, int64_t T, float c, float rcp_tau, float* logprobs, float* entropy, float* maximum, float* accumulate,
                                     float* entropy_b) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t t = gid / LANES;
  const int sub = (int)(gid % LANES);
  const bool live = t < T;
  float vm = kNegBig, va = 0.f, vb = 0.f;
  if (live) {
    for (int s = sub; s < S; s += LANES) {
      const f32x4_t u = parts[(int64_t)s * T + t];
      merge_stats(vm, va, vb, u[0], u[1], u[2], c);
    }
  }
#pragma unroll
  for (int off = LANES / 2; off > 0; off >>= 1) {
    const float m2 = __shfl_xor(vm, off), a2 = __shfl_xor(va, off), b2 = __shfl_xor(vb, off);
    merge_stats(vm, va, vb, m2, a2, b2, c);
  }
  if (!live || sub != 0) return;
  const float vz = label_logit(xlabel, labels, label_offset, V, t);
  const float mz = vm * rcp_tau;
  const float lse = mz + logf(va);
  const float eb = (vb / va) * rcp_tau;
  maximum[t] = mz;
  accumulate[t] = va;
  entropy_b[t] = eb;
  entropy[t] = lse - eb;
  logprobs[t] = vz * rcp_tau - lse;
}

// Vocabulary-parallel building block: the same merge, but the result stays a partial for exchange
// between the owners of the vocabulary shards: out[t] = (max logit, sum exp(logit - max),
// sum logit * exp(logit - max), label logit or 0), in logit units (after the division by temperature).
template <int LANES>
__global__ void lce_fwd_shard_merge_kernel(const f32x4_t* parts, const float* xlabel, const int64_t* labels, int64_t label_offset,
                                           int64_t V, int S, int64_t T, float c, float rcp_tau, f32x4_t* out) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t t = gid / LANES;
  const int sub = (int)(gid % LANES);
  const bool live = t < T;
  float vm = kNegBig, va = 0.f, vb = 0.f;
  if (live) {
    for (int s = sub; s < S; s += LANES) {
      const f32x4_t u = parts[(int64_t)s * T + t];
      merge_stats(vm, va, vb, u[0], u[1], u[2], c);
    }
  }
#pragma unroll
  for (int off = LANES / 2; off > 0; off >>= 1) {
    const float m2 = __shfl_xor(vm, off), a2 = __shfl_xor(va, off), b2 = __shfl_xor(vb, off);
    merge_stats(vm, va, vb, m2, a2, b2, c);
  }
  if (!live || sub != 0) return;
  const f32x4_t v = {vm * rcp_tau, va, vb * rcp_tau, label_logit(xlabel, labels, label_offset, V, t) * rcp_tau};
  out[t] = v;
}

// merges the partials of R vocabulary shards (shard-major [R][T]) in the fixed order r = 0, 1, ... and
// emits the five per-token outputs
inline __global__ void lce_merge_shards_kernel(const f32x4_t* partials, int R, int64_t T, float* logprobs, float* entropy,
                                        float* maximum, float* accumulate, float* entropy_b) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  float vm = kNegBig, va = 0.f, vb = 0.f, vz = 0.f;
  for (int r = 0; r < R; ++r) {
    const f32x4_t u = partials[(int64_t)r * T + t];
    merge_stats(vm, va, vb, u[0], u[1], u[2], kLog2e);
    vz += u[3];  // the label lives in at most one shard; the others hold 0
  }
  const float lse = vm + logf(va);
  const float eb = vb / va;
  maximum[t] = vm;
  accumulate[t] = va;
  entropy_b[t] = eb;
  entropy[t] = lse - eb;
  logprobs[t] = vz - lse;
}

// deterministic single-workgroup sum of x[0..n) * scale -> out[0]
inline __global__ void lce_reduce_sum_kernel(const float* x, int64_t n, float scale, float* out) {
  __shared__ double sh[1024];
  double acc = 0.0;
  for (int64_t i = threadIdx.x; i < n; i += blockDim.x) acc += (double)x[i];
  sh[threadIdx.x] = acc;
  __syncthreads();
  for (int s = blockDim.x >> 1; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) sh[threadIdx.x] += sh[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[0] = (float)(sh[0] * (double)scale);
}

// ------------------------------------------------------------------------------------------------
// backward, stage 1: recompute a [vocab chunk] x [tokens] logit tile and write d_logits in both
// layouts (token-major for d_hidden's GEMM, vocab-major for d_weight's GEMM)
// ------------------------------------------------------------------------------------------------
template <typename TIN>
struct DsArgs {
  const TIN* W;  // first row of the chunk
  int64_t ldw;
  const TIN* h;
  int64_t ldh;
  const int64_t* labels;
  int64_t T, H;
  int64_t v0;     // vocabulary index of the chunk's first row (global: labels are matched against v0 + row)
  int64_t vrows;  // valid rows in the chunk
  float c, rcp_tau;
  const float* maximum;
  const float* accumulate;
  const float* entropy_b;
  const float* g_lp;  // [T] or [1]
  int64_t g_lp_stride;  // 1 or 0
  float g_lp_scale;     // 1, or 1/T for mean
  const float* g_ent;   // [T] or null
  TIN* dS;              // [T][ldS]      (token-major)
  int64_t ldS;
  TIN* dST;             // [vchunk][ldST] (vocab-major); null when the d_weight GEMM reads dS with transposing LDS reads
  int64_t ldST;
  int64_t tpad;         // tokens rounded up to the GEMM K granule: columns [T, tpad) of dST / rows [T, tpad) of dS are written as zeros
  TileMap map;          // rows = token tiles, cols = vocab tiles of the chunk
  // Token compaction (both null = off): only tokens with a non-zero upstream gradient take part.
  // rows[k] is the token behind compact position k < *n_rows; dS / dS^T are indexed by k, while
  // hidden, labels, the statistics and the upstream gradients are read at rows[k].
  const int* rows;
  const int* n_rows;
  int label_outside;  // 1: the tiles hold the softmax terms only; the one-hot part g_lp / tau * 1[v == label] is added
                      // elsewhere in fp32 (label_rows.hpp); 2: the label's whole entry is left out of the tiles (zero
                      // there) and added elsewhere in fp32; 0: everything inside the tiles
  // Per-position constants prepared once per backward (ds_token_consts_kernel; used by the 16x16x32 tiles):
  // tokc[k] = (logsumexp * log2 e, C0, C1, G) of the token at compact position k < tpad (positions without a token
  // hold (1e30, 0, 0, 0), which makes every entry of their rows zero), tokl[k] = its label as a row of this call's
  // weight or -1; lab0 = the chunk's first row in the same numbering.
  const f32x4_t* tokc;
  const int* tokl;
  int64_t lab0;
  int64_t range_rows;  // few tokens: > 0 = every workgroup of lce_bwd_ds_kernel takes that many vocabulary rows (a multiple of the wave tile's)
};

// The two gradient GEMMs sum over the vocabulary (d_hidden) and over the tokens (d_weight); any
// permutation of the summation index is allowed as long as both operands of a GEMM use the same one.
// The intermediates (dS, dS^T, W^T, h^T) are private to the backward, so their K order is chosen to
// suit the producer: inside each group of WN tokens / WM vocabulary rows (one wave tile) the index is
// re-ordered so that everything ONE lane of the d_logits epilogue holds is contiguous, and the
// epilogue stores 16-byte / 8-byte vectors instead of single elements.
template <typename Cfg>
struct KPerm {
  static constexpr int GT = Cfg::WN, GV = Cfg::WM;
  // token t (lane ln = t % 32 of block column j = (t % GT) / 32)  ->  ln * FN + j
  static __host__ __device__ __forceinline__ int64_t token(int64_t t) {
    const int64_t l = t % GT;
    return t - l + (l % 32) * Cfg::FN + l / 32;
  }
  // vocabulary row v = i*32 + 8*(r/4) + 4*hh + r%4 of its group  ->  hh * 16*FM + i*16 + r
  static __host__ __device__ __forceinline__ int64_t vocab(int64_t v) {
    const int64_t l = v % GV;
    const int64_t i = l / 32, w = l % 32, hh = (w >> 2) & 1, r = (w >> 3) * 4 + (w & 3);
    return v - l + hh * 16 * Cfg::FM + i * 16 + r;
  }
  // inverses: which token / vocabulary row sits at position u
  static __host__ __device__ __forceinline__ int64_t token_at(int64_t u) {
    const int64_t l = u % GT;
    return u - l + (l % Cfg::FN) * 32 + l / Cfg::FN;
  }
  static __host__ __device__ __forceinline__ int64_t vocab_at(int64_t u) {
    const int64_t l = u % GV;
    const int64_t hh = l / (16 * Cfg::FM), rem = l % (16 * Cfg::FM), i = rem / 16, r = rem % 16;
    return u - l + i * 32 + 8 * (r >> 2) + 4 * hh + (r & 3);
  }
};

template <typename T, int N>
struct VecOf;
template <int N>
struct VecOf<float, N> { typedef float type __attribute__((ext_vector_type(N))); };
template <int N>
struct VecOf<bf16_t, N> { typedef bf16_t type __attribute__((ext_vector_type(N))); };
template <int N>
struct VecOf<f16_t, N> { typedef f16_t type __attribute__((ext_vector_type(N))); };

// store N consecutive elements (N * sizeof(T) <= 16 bytes per store; wider runs are split);
// STREAM: non-temporal stores, for data that this kernel does not read back
// The fp32 value that is rounded to 16 bits is made opaque to the optimiser first: where it is a product, the compiler
// otherwise fuses the multiplication and the conversion into one v_fma_mixlo_f16 in some kernels and not in others, and
// the single rounding of the exact product differs from the two roundings (to fp32, then to fp16) at ties (found as one
// fp16 d_logits entry in 260000 that differed between the tiles and d_logits computed from kept logits).
template <typename T>
LCE_DEV T round_to(float x) {
  if constexpr (__is_same(T, f16_t)) asm("" : "+v"(x));  // (no instruction fuses arithmetic with a conversion to bf16)
  return (T)x;
}

template <typename T, int N, bool STREAM = false>
LCE_DEV void store_run(T* dst, const float (&v)[N]) {
  constexpr int PER = (16 / (int)sizeof(T)) < N ? (16 / (int)sizeof(T)) : N;
  typedef typename VecOf<T, PER>::type vec_t;
#pragma unroll
  for (int k = 0; k < N; k += PER) {
    vec_t out;
#pragma unroll
    for (int e = 0; e < PER; ++e) out[e] = round_to<T>(v[k + e]);
    if (STREAM) __builtin_nontemporal_store(out, reinterpret_cast<vec_t*>(dst + k));
    else *reinterpret_cast<vec_t*>(dst + k) = out;
  }
}

// The per-token constants of d_logits: with p = exp2(x c - lse2), dz = p (C0 + C1 x) (+ G at the label).  ONE function
// with floating-point contraction switched off for every kernel that needs them (the d_logits tiles of both mainloops, the
// per-position table of the 16x16x32 tiles, the label coefficients, d_logits from kept logits), so that the compiler
// cannot fuse `a * b + c` in one kernel and not in the next and leave a token with constants that differ in their last bit.
// glp: upstream gradient of the log-prob, already scaled for the reduction; gent: of the entropy.
struct TokenConsts {
  float lse2, C0, C1, G;
};
LCE_DEV TokenConsts token_consts(float glp, float gent, float maximum, float accumulate, float entropy_b, float rcp_tau) {
#pragma clang fp contract(off)
  TokenConsts k;
  k.lse2 = (maximum + logf(accumulate)) * kLog2e;
  k.G = glp * rcp_tau;
  k.C1 = -gent * rcp_tau * rcp_tau;
  k.C0 = -k.G + gent * entropy_b * rcp_tau;
  return k;
}

// d_logits of one accumulator element; SLOW adds the label one-hot and masks padded rows / tokens
// (drop: the label's entry is not part of the tile at all, it is added elsewhere in fp32)
template <bool SLOW>
LCE_DEV float dlogit(float x, float c, float lse2, float C0, float C1, float G, bool hit, bool dead, bool drop) {
#pragma clang fp contract(off)
  const float pr = fast_exp2(__builtin_fmaf(x, c, -lse2));
  float dv = pr * __builtin_fmaf(x, C1, C0);
  if (SLOW) {
    if (hit) dv = drop ? 0.f : dv + G;
    if (dead) dv = 0.f;
  }
  return dv;
}

// dS (token-major) leaves the wave through a wave-private LDS staging tile so that every store
// instruction writes whole 128-byte lines (8 lanes x 16 bytes per token row); written straight from
// the accumulator layout each lane would hit a different row, which costs ~25% of the kernel.
// 16-byte chunks of a staged row are XOR-swizzled with the row number (conflict-free both ways).
template <typename Cfg>
struct DsStage {
  typedef typename Cfg::TIN TIN;
  static constexpr bool kEnabled = sizeof(TIN) == 2;                 // fp32 tiles do not fit; they store directly
  static constexpr int ROW_BYTES = Cfg::WM * (int)sizeof(TIN);       // one token's slice of the wave tile
  static constexpr int CPR = ROW_BYTES / 16;                          // 16-byte chunks per row
  static constexpr int WAVE_BYTES = Cfg::WN * ROW_BYTES;
  static_assert(!kEnabled || WAVE_BYTES * Cfg::NW <= Cfg::LDS_BYTES, "staging tile must fit the mainloop's LDS");
  static LCE_DEV int swz(int row) { return (row ^ ((row >> 3) & 1)) & 7; }
};

template <typename Cfg, bool SLOW>
LCE_DEV void ds_epilogue(const DsArgs<typename Cfg::TIN>& p, const f32x16_t (&acc)[Cfg::FM][Cfg::FN], int64_t tok0,
                         int64_t Tc, int vloc0, int hh, int ln, char* stage_lds) {
  typedef typename Cfg::TIN TIN;
  typedef DsStage<Cfg> Stg;
  constexpr int FM = Cfg::FM, FN = Cfg::FN;
  float lse2[FN], C0[FN], C1[FN], G[FN];
  int rel[FN];
  bool tok_ok[FN];
#pragma unroll
  for (int j = 0; j < FN; ++j) {
    const int64_t pos = tok0 + j * 32 + ln;  // position in dS / dS^T
    tok_ok[j] = pos < Tc;
    lse2[j] = C0[j] = C1[j] = G[j] = 0.f;
    rel[j] = -1;
    if (tok_ok[j]) {
      const int64_t tok = p.rows ? (int64_t)p.rows[pos] : pos;
      const float glp = p.g_lp[tok * p.g_lp_stride] * p.g_lp_scale;
      const float gent = p.g_ent ? p.g_ent[tok] : 0.f;
      const TokenConsts k = token_consts(glp, gent, p.maximum[tok], p.accumulate[tok], p.entropy_b[tok], p.rcp_tau);
      lse2[j] = k.lse2; G[j] = k.G; C1[j] = k.C1; C0[j] = k.C0;
      const int64_t y = p.labels[tok] - p.v0;
      rel[j] = (p.label_outside != 1 && y >= vloc0 && y < vloc0 + Cfg::WM) ? (int)(y - vloc0) : -1;
    }
  }
  const bool tok_group_live = p.dST != nullptr && tok0 < p.tpad;  // the whole token group is inside dS^T's columns
  TIN* dst_t = p.dST + (tok0 + (int64_t)ln * FN);            // + vocab row * ldST   (token order: ln*FN + j)
  TIN* dst_s = p.dS + (vloc0 + hh * 16 * FM);                // + token * ldS + i*16 + r (vocab order: hh, i, r)
#pragma unroll
  for (int i = 0; i < FM; ++i) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      __builtin_amdgcn_sched_barrier(0);  // bound the live range of the staged values
      float stage[FN][8];
#pragma unroll
      for (int rr = 0; rr < 8; ++rr) {
        const int r = half * 8 + rr;
        const int row = acc_row(i, r, hh);  // wave-tile-local vocabulary row
        float d[FN];
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          d[j] = dlogit<SLOW>(acc[i][j][r], p.c, lse2[j], C0[j], C1[j], G[j], row == rel[j],
                              !tok_ok[j] || vloc0 + row >= p.vrows, p.label_outside == 2);
          stage[j][rr] = d[j];
        }
        if (tok_group_live) store_run<TIN, FN>(dst_t + (int64_t)(vloc0 + row) * p.ldST, d);
      }
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        if constexpr (Stg::kEnabled) {
          // logical 16-byte chunk of this run inside the token's row: (hh*16*FM + i*16 + half*8) elements
          const int c = hh * 2 * FM + i * 2 + half, row = j * 32 + ln;
          store_run<TIN, 8>(reinterpret_cast<TIN*>(stage_lds + row * Stg::ROW_BYTES + ((c ^ Stg::swz(row)) * 16)), stage[j]);
        } else {
          if (tok_ok[j])
            store_run<TIN, 8>(dst_s + (tok0 + j * 32 + ln) * p.ldS + i * 16 + half * 8, stage[j]);
        }
      }
    }
  }
  if constexpr (Stg::kEnabled) {
    // the staging tile is private to this wave: LDS operations of one wave complete in order
    const int lane = hh * 32 + ln;
#pragma unroll
    for (int it = 0; it < Stg::WAVE_BYTES / 1024; ++it) {
      const int q = it * 64 + lane, row = q / Stg::CPR, pc = q % Stg::CPR;
      const int c = pc ^ Stg::swz(row);
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(stage_lds + row * Stg::ROW_BYTES + pc * 16);
      const int64_t tok = tok0 + row;
      // rows of tokens that do not take part are zeros (the staged values are); they pad the d_weight GEMM's K
      if (tok < p.tpad) *reinterpret_cast<u32x4_t*>(p.dS + tok * p.ldS + vloc0 + c * 8) = v;
    }
  }
}

// One 256-row vocabulary tile of the d_logits pass for the token tile at n0: rows m0 .. of the chunk, of which the
// workgroup owns those below own_end (a multiple of the wave tile's rows; the rest belongs to a neighbour and is
// neither read beyond the clamp nor written).
template <typename Cfg>
LCE_DEV void ds_tile_at(const DsArgs<typename Cfg::TIN>& p, int64_t n0, int64_t m0, int64_t own_end, int64_t Tc, char* lds) {
  const int lane = threadIdx.x & 63, hh = lane >> 5, ln = lane & 31;
  GemmCore<Cfg> g;
  g.init(p.W, p.ldw, m0, own_end < p.vrows ? own_end : p.vrows, p.h, p.ldh, n0, Tc, p.rows);
  f32x16_t acc[Cfg::FM][Cfg::FN];
  g.run(lds, p.H, acc);

  const int vloc0 = (int)m0 + g.wave_m * Cfg::WM;      // chunk-local vocabulary index of this wave's first row
  const int64_t tok0 = n0 + g.wave_n * Cfg::WN;         // first token of this wave's group
  // fast path: the wave tile is interior (no padded rows or tokens) and holds no label
  bool has_label = false;
#pragma unroll
  for (int j = 0; j < Cfg::FN; ++j) {
    const int64_t tok = tok0 + j * 32 + ln;
    if (tok < Tc && p.label_outside != 1) {
      const int64_t y = p.labels[p.rows ? p.rows[tok] : tok] - p.v0;
      has_label |= (y >= vloc0 && y < vloc0 + Cfg::WM);
    }
  }
  const bool interior = vloc0 + Cfg::WM <= p.vrows && tok0 + Cfg::WN <= Tc;
  __syncthreads();  // every wave's slab loads have landed and its operand reads are done: LDS is free
  if (vloc0 >= own_end) return;  // (a whole wave tile of the neighbour's rows; the caller's barriers are outside)
  char* stage_lds = lds + g.wave * DsStage<Cfg>::WAVE_BYTES;
  if (interior && __builtin_amdgcn_ballot_w64(has_label) == 0) ds_epilogue<Cfg, false>(p, acc, tok0, Tc, vloc0, hh, ln, stage_lds);
  else ds_epilogue<Cfg, true>(p, acc, tok0, Tc, vloc0, hh, ln, stage_lds);
}

template <typename Cfg>
LCE_DEV void ds_tile(const DsArgs<typename Cfg::TIN>& p, int bid, char* lds) {
  const int64_t Tc = p.n_rows ? (int64_t)*p.n_rows : p.T;  // tokens that take part
  if (p.range_rows > 0) {
    // Few tokens (one token tile, HBM-bound): every workgroup takes one contiguous range of range_rows vocabulary rows,
    // the same length for all, instead of whole 256-row tiles (594 tiles over 256 CUs would be 3 against 2).  The last
    // tile of a range is clamped at the range's end: its surplus rows are repeats of one row in the loads, and the
    // waves that hold only such rows store nothing.
    if (Tc <= 0) return;  // no token takes part: nothing to read (the operand loads clamp to the last token) or to write
    const int64_t pad_end = (p.vrows + Cfg::WM - 1) / Cfg::WM * Cfg::WM;  // (rows up to the wave tile are written as zeros)
    const int64_t r0 = (int64_t)bid * p.range_rows;
    const int64_t r1 = r0 + p.range_rows < pad_end ? r0 + p.range_rows : pad_end;
    // Walked from the range's end: the forward, which ran last, walked the same ranges from their start, so what the
    // memory-side cache still holds of W is read first (64 tokens, H=3584, V=152064: 8 us of 207)
    const int64_t ntile = (r1 - r0 + Cfg::BM - 1) / Cfg::BM;
    for (int64_t i = ntile - 1; i >= 0; --i) {
      if (i < ntile - 1) __syncthreads();  // the staging tiles of the previous tile's epilogue are read out
      ds_tile_at<Cfg>(p, 0, r0 + i * Cfg::BM, r1, Tc, lds);
    }
    return;
  }
  int tt, vt;
  // with a device-side token count the XCD-aware map is rebuilt over the token tiles that exist, so
  // that they spread evenly over the XCDs (the host's map would leave whole XCDs without work)
  const TileMap map = p.n_rows ? p.map.with_rows((int)((Tc + Cfg::BN - 1) / Cfg::BN)) : p.map;
  if (!map.decode(bid, tt, vt)) return;
  ds_tile_at<Cfg>(p, (int64_t)tt * Cfg::BN, (int64_t)vt * Cfg::BM, (int64_t)1 << 40, Tc, lds);
}

// ------------------------------------------------------------------------------------------------
// plain NT GEMM with the shared mainloop: C[m][n] = sum_k A[m][k] B[n][k]
//   out_mode 0: Cf = acc           1: Cf += acc
//            2: Ct = (TIN)acc      3: Ct = (TIN)(Cf + acc)
// ------------------------------------------------------------------------------------------------
template <typename TIN>
struct GemmArgs {
  const TIN* A;
  int64_t lda;
  const TIN* B;
  int64_t ldb;
  int64_t M, N, K;
  float* Cf;
  int64_t ldcf;
  TIN* Ct;
  int64_t ldct;
  int out_mode;
  TileMap map;  // rows = M tiles, cols = N tiles
  // split K: workgroup `bid` computes tile bid % map.total over k in [s * kslice, min(K, (s + 1) * kslice)),
  // s = bid / map.total < ksplit, into the fp32 partial Cf + s * cf_split_stride (out_mode 0 or 1 only)
  int ksplit;
  int64_t kslice, cf_split_stride;
  // sizes known only on the device (null = use M / K): rows that exist, M = min(M, *m_dev), and the
  // reduction length, K = min(K, *k_dev rounded up to k_gran); K = 0 gives C = 0
  const int* m_dev;
  const int* k_dev;
  int k_gran;
  // operands K-major, A[k][m] and B[k][n] (gemm_tn_tile); the rows of C are then A's columns, which the d_logits
  // epilogue leaves in KPerm::vocab order: row u of the tile is written to row KPerm::vocab_at(u) of C
  int tn;  // 0 NT (gemm_tile); 1 both operands K-major (gemm_tn_tile); 2 only B K-major, its rows in KPerm::vocab order (gemm_nb_tile)
  int64_t b_rows_valid;  // tn == 2: rows of B that exist (K may be rounded up beyond them; A is zero there)
  int perm_rows;  // tn == 1 with fp32 output: row u of the tile goes to row KPerm::vocab_at(u) of Cf as well (out_mode 2 always does)
};

template <typename Cfg, int MODE, bool EDGE>
LCE_DEV void gemm_epilogue(const GemmArgs<typename Cfg::TIN>& p, const f32x16_t (&acc)[Cfg::FM][Cfg::FN], int64_t m0,
                           int64_t n0, int wave_m, int wave_n, int hh, int ln) {
  typedef typename Cfg::TIN TIN;
  const int64_t mw = m0 + wave_m * Cfg::WM + 4 * hh;  // row of register 0 of block row 0
#pragma unroll
  for (int j = 0; j < Cfg::FN; ++j) {
    const int64_t n = n0 + wave_n * Cfg::WN + j * 32 + ln;
    if (EDGE && n >= p.N) continue;
#pragma unroll
    for (int i = 0; i < Cfg::FM; ++i) {
      __builtin_amdgcn_sched_barrier(0);  // one 32x32 block at a time (register pressure)
      float* cf = (MODE != 2) ? p.Cf + (mw + i * 32) * p.ldcf + n : nullptr;
      TIN* ct = (MODE & 2) ? p.Ct + (mw + i * 32) * p.ldct + n : nullptr;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (EDGE && mw + i * 32 + 8 * q + u >= p.M) continue;
          float v = acc[i][j][q * 4 + u];
          if (MODE & 1) v += cf[(8 * q + u) * p.ldcf];
          if (MODE & 2) ct[(8 * q + u) * p.ldct] = (TIN)v;
          else cf[(8 * q + u) * p.ldcf] = v;
        }
      }
    }
  }
}

template <typename Cfg>
LCE_DEV void gemm_tile(const GemmArgs<typename Cfg::TIN>& pin, int bid, char* lds) {
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
  const int lane = threadIdx.x & 63, hh = lane >> 5, ln = lane & 31;
  GemmCore<Cfg> g;
  g.init(p.A + k0, p.lda, m0, p.M, p.B + k0, p.ldb, n0, p.N);
  f32x16_t acc[Cfg::FM][Cfg::FN];
  if (k0 < k1) {
    g.run(lds, k1 - k0, acc);
  } else {  // empty K range: contributes zero (and still initialises what it owns)
    if (p.out_mode == 1) return;
#pragma unroll
    for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
      for (int j = 0; j < Cfg::FN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  }
  const bool edge = m0 + Cfg::BM > p.M || n0 + Cfg::BN > p.N;
#define LCE_EPI(MODE)                                                                           \
  if (edge) gemm_epilogue<Cfg, MODE, true>(p, acc, m0, n0, g.wave_m, g.wave_n, hh, ln);         \
  else gemm_epilogue<Cfg, MODE, false>(p, acc, m0, n0, g.wave_m, g.wave_n, hh, ln)
  switch (p.out_mode) {
    case 0: LCE_EPI(0); break;
    case 1: LCE_EPI(1); break;
    case 2: LCE_EPI(2); break;
    default: LCE_EPI(3); break;
  }
#undef LCE_EPI
}

// C[m][n] = sum_k A[k][m] * B[k][n]: both operands K-major (Cfg::TRANS); A and B are allocated in whole
// 256-column tiles, K (or *k_dev rounded up to k_gran) a multiple of 64.  out_mode 0: Cf = acc;
// out_mode 2: Ct[KPerm::vocab_at(m)][n] = (TIN)acc (see GemmArgs::tn).
template <typename Cfg, typename PermCfg, int MODE, bool EDGE>
LCE_DEV void gemm_tn_epilogue(const GemmArgs<typename Cfg::TIN>& p, const f32x16_t (&acc)[Cfg::FM][Cfg::FN], int64_t m0, int64_t n0,
                              int wave_m, int wave_n, int hh, int ln) {
  typedef typename Cfg::TIN TIN;
#pragma unroll
  for (int j = 0; j < Cfg::FN; ++j) {
    const int64_t n = n0 + wave_n * Cfg::WN + j * 32 + ln;
    if (EDGE && n >= p.N) continue;
#pragma unroll
    for (int i = 0; i < Cfg::FM; ++i) {
      __builtin_amdgcn_sched_barrier(0);  // one 32x32 block at a time (register pressure)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int u = acc_row(i, r, hh);  // row inside the wave tile
        const int um = (MODE == 2 || p.perm_rows) ? (int)KPerm<PermCfg>::vocab_at(u) : u;
        const int64_t m = m0 + wave_m * Cfg::WM + um;
        if (EDGE && m >= p.M) continue;
        if (MODE == 2) p.Ct[m * p.ldct + n] = (TIN)acc[i][j][r];
        else p.Cf[m * p.ldcf + n] = acc[i][j][r];
      }
    }
  }
}

template <typename Cfg, typename PermCfg>
LCE_DEV void gemm_tn_tile(const GemmArgs<typename Cfg::TIN>& pin, int bid, char* lds) {
  GemmArgs<typename Cfg::TIN> p = pin;
  if (p.k_dev) {
    const int64_t k = ((int64_t)*p.k_dev + p.k_gran - 1) / p.k_gran * p.k_gran;
    p.K = k < p.K ? k : p.K;
  }
  int tm, tn;
  if (!p.map.decode(bid, tm, tn)) return;
  const int64_t m0 = (int64_t)tm * Cfg::BM, n0 = (int64_t)tn * Cfg::BN;
  const int lane = threadIdx.x & 63, hh = lane >> 5, ln = lane & 31;
  GemmCore<Cfg> g;
  g.init_tn(p.A, p.lda, m0, p.B, p.ldb, n0);
  f32x16_t acc[Cfg::FM][Cfg::FN];
  if (p.K > 0) {
    g.run(lds, p.K, acc);
  } else {
#pragma unroll
    for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
      for (int j = 0; j < Cfg::FN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  }
  const bool edge = m0 + Cfg::BM > p.M || n0 + Cfg::BN > p.N;
  if (p.out_mode == 2) {
    if (edge) gemm_tn_epilogue<Cfg, PermCfg, 2, true>(p, acc, m0, n0, g.wave_m, g.wave_n, hh, ln);
    else gemm_tn_epilogue<Cfg, PermCfg, 2, false>(p, acc, m0, n0, g.wave_m, g.wave_n, hh, ln);
  } else {
    if (edge) gemm_tn_epilogue<Cfg, PermCfg, 0, true>(p, acc, m0, n0, g.wave_m, g.wave_n, hh, ln);
    else gemm_tn_epilogue<Cfg, PermCfg, 0, false>(p, acc, m0, n0, g.wave_m, g.wave_n, hh, ln);
  }
}

template <typename Cfg>
__global__ __launch_bounds__(Cfg::NTHREADS) void gemm_tn_kernel(GemmArgs<typename Cfg::TIN> p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  gemm_tn_tile<Cfg, Cfg>(p, blockIdx.x, lds);
}

template <typename Cfg>
__global__ __launch_bounds__(Cfg::NTHREADS) void lce_bwd_ds_kernel(DsArgs<typename Cfg::TIN> p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  ds_tile<Cfg>(p, blockIdx.x, lds);
}

template <typename Cfg>
__global__ __launch_bounds__(Cfg::NTHREADS) void gemm_nt_kernel(GemmArgs<typename Cfg::TIN> p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  gemm_tile<Cfg>(p, blockIdx.x, lds);
}

// One launch of the backward's steady state: the two gradient GEMMs of vocabulary chunk c-1 and the
// d_logits tiles of chunk c (which go to the other buffer pair) share a grid, longest tiles first,
// so the tail of one sub-problem is filled by the next instead of idling the CUs.
// Sub-grid sizes are multiples of 32, which keeps (block id % 8) -> XCD intact for every sub-problem.
template <typename TIN>
struct BwdChunkArgs {
  // the two gradient GEMMs of chunk c-1, the one with the longer K loop per tile in the first slot:
  //   d_weight[chunk c-1] = dS^T . h^T   (K = T)   and   d_hidden (+)= dS . W^T[chunk c-1]   (K = chunk width / K splits)
  GemmArgs<TIN> gw;
  GemmArgs<TIN> gh;
  DsArgs<TIN> ds;    // d_logits of chunk c                     (K = H, heavy epilogue)
  int n_gw, n_gh, n_ds;
};

// C[m][n] (+)= sum_k A[m][k] * B[k][n]: A row-major, B K-major as it lies in memory (Cfg::TRANS == 2).  Column k of A
// holds the product partner of B's row KPerm::vocab_at(k) (the order the d_logits epilogue stores its columns in).
// Split K, device-side M and the fp32 output modes 0 / 1 as in gemm_tile.
template <typename Cfg, typename PermCfg>
LCE_DEV void gemm_nb_tile(const GemmArgs<typename Cfg::TIN>& pin, int bid, char* lds) {
  GemmArgs<typename Cfg::TIN> p = pin;
  if (p.m_dev) {
    const int64_t m = *p.m_dev;
    p.M = m < p.M ? m : p.M;
  }
  int64_t k0 = 0, k1 = p.K;
  if (p.ksplit > 1) {
    const int s = bid / p.map.total;
    bid -= s * p.map.total;
    k0 = s * p.kslice;
    k1 = k0 + p.kslice < p.K ? k0 + p.kslice : p.K;
    p.Cf += s * p.cf_split_stride;
  }
  int tm, tn;
  const TileMap map = p.m_dev ? p.map.with_rows((int)((p.M + Cfg::BM - 1) / Cfg::BM)) : p.map;
  if (!map.decode(bid, tm, tn)) return;
  const int64_t m0 = (int64_t)tm * Cfg::BM, n0 = (int64_t)tn * Cfg::BN;
  const int lane = threadIdx.x & 63, hh = lane >> 5, ln = lane & 31;
  GemmCore<Cfg> g;
  f32x16_t acc[Cfg::FM][Cfg::FN];
  if (k0 < k1 && k0 < p.b_rows_valid) {
    g.init_mixed(p.A + k0, p.lda, m0, p.M, p.B + k0 * p.ldb, p.ldb, n0, p.N - n0, p.b_rows_valid - k0,
                 [](int r) { return KPerm<PermCfg>::vocab_at(r); });
    g.run(lds, k1 - k0, acc);
  } else {  // empty K range: contributes zero (and still initialises what it owns)
    if (p.out_mode == 1) return;
    g.init(p.A, p.lda, m0, p.M, p.A, p.lda, 0, Cfg::BN);  // (wave_m / wave_n for the epilogue)
#pragma unroll
    for (int i = 0; i < Cfg::FM; ++i)
#pragma unroll
      for (int j = 0; j < Cfg::FN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  }
  const bool edge = m0 + Cfg::BM > p.M || n0 + Cfg::BN > p.N;
  if (p.out_mode == 0) {
    if (edge) gemm_epilogue<Cfg, 0, true>(p, acc, m0, n0, g.wave_m, g.wave_n, hh, ln);
    else gemm_epilogue<Cfg, 0, false>(p, acc, m0, n0, g.wave_m, g.wave_n, hh, ln);
  } else {
    if (edge) gemm_epilogue<Cfg, 1, true>(p, acc, m0, n0, g.wave_m, g.wave_n, hh, ln);
    else gemm_epilogue<Cfg, 1, false>(p, acc, m0, n0, g.wave_m, g.wave_n, hh, ln);
  }
}

// the mainloop configuration for K-major operands that goes with Cfg (same tile and wave layout, split ring)
template <typename Cfg>
struct TransOf {
  typedef GemmCfg<typename Cfg::TIN, Cfg::BM, Cfg::BN, 128, 5, Cfg::WAVES_M, Cfg::WAVES_N, 2, 1> type;   // A and B K-major
  typedef GemmCfg<typename Cfg::TIN, Cfg::BM, Cfg::BN, 128, 5, Cfg::WAVES_M, Cfg::WAVES_N, 2, 2> mixed;  // only B
};

template <typename Cfg>
LCE_DEV void any_gemm_tile(const GemmArgs<typename Cfg::TIN>& p, int bid, char* lds) {
  if constexpr (sizeof(typename Cfg::TIN) == 2 && Cfg::BM == 256 && Cfg::BN == 256 && Cfg::WAVES_M == 4 && Cfg::WAVES_N == 2) {
    if (p.tn == 1) {
      gemm_tn_tile<typename TransOf<Cfg>::type, Cfg>(p, bid, lds);
      return;
    }
    if (p.tn == 2) {
      gemm_nb_tile<typename TransOf<Cfg>::mixed, Cfg>(p, bid, lds);
      return;
    }
  }
  gemm_tile<Cfg>(p, bid, lds);
}

template <typename Cfg>
__global__ __launch_bounds__(Cfg::NTHREADS) void lce_bwd_chunk_kernel(BwdChunkArgs<typename Cfg::TIN> p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int bid = blockIdx.x;
  if (bid < p.n_gw) any_gemm_tile<Cfg>(p.gw, bid, lds);
  else if (bid < p.n_gw + p.n_gh) any_gemm_tile<Cfg>(p.gh, bid - p.n_gw, lds);
  else ds_tile<Cfg>(p.ds, bid - p.n_gw - p.n_gh, lds);
}

// how the one-hot part of d_logits is evaluated per token when it is kept out of the d_logits tiles
struct LabelTerm {
  const int64_t* labels;  // null: the one-hot part is inside the tiles (nothing to add)
  int64_t v0, V;          // this call's weight rows are vocabulary ids [v0, v0 + V)
  const float* g_lp;
  int64_t g_stride;       // 0: one value shared by all tokens (sum / mean reduction)
  float scale;            // g_lp * scale = G, the coefficient of 1[v == label] in d_logits
};

// d_hidden[t][:] = (T)(sum over s < S of part[s * stride + pos(t) * H + :]) with pos(t) = inv[t] (t itself
// without `inv`), or zeros where inv[t] < 0 (token without upstream gradient).  The sum runs in the
// fixed order s = 0, 1, ..., so the result does not depend on scheduling.  H a multiple of 4.
// With a label term, G_t * W[label_t][:] is added in fp32 before the one rounding.
// (bid of nblocks workgroups: the kernel's own grid, or the part of a larger grid that does this work)
template <typename T, typename TOUT>
LCE_DEV void dh_finish_body(const float* part, int S, int64_t stride, const int* inv, int64_t ntok, int64_t H, TOUT* out,
                            const LabelTerm& lt, const T* W, int64_t ldw, int64_t bid, int64_t nblocks) {
  const int64_t per_row = H / 4, n = ntok * per_row;
  for (int64_t q = bid * blockDim.x + threadIdx.x; q < n; q += nblocks * blockDim.x) {
    const int64_t t = q / per_row, c = (q - t * per_row) * 4;
    const int64_t pos = inv ? (int64_t)inv[t] : t;
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    if (pos >= 0) {
      const float* src = part + pos * H + c;
      a = *reinterpret_cast<const float4*>(src);
      for (int s = 1; s < S; ++s) {
        const float4 b = *reinterpret_cast<const float4*>(src + s * stride);
        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
      }
      if (lt.labels) {
        const float G = lt.g_lp[t * lt.g_stride] * lt.scale;
        const int64_t y = lt.labels[t] - lt.v0;
        if (G != 0.f && y >= 0 && y < lt.V) {
          const T* w = W + y * ldw + c;
          a.x = __builtin_fmaf(G, (float)w[0], a.x); a.y = __builtin_fmaf(G, (float)w[1], a.y);
          a.z = __builtin_fmaf(G, (float)w[2], a.z); a.w = __builtin_fmaf(G, (float)w[3], a.w);
        }
      }
    }
    TOUT* dst = out + t * H + c;
    dst[0] = round_to<TOUT>(a.x); dst[1] = round_to<TOUT>(a.y); dst[2] = round_to<TOUT>(a.z); dst[3] = round_to<TOUT>(a.w);
  }
}

template <typename T, typename TOUT>
__global__ void dh_finish_kernel(const float* part, int S, int64_t stride, const int* inv, int64_t ntok, int64_t H, TOUT* out,
                                 LabelTerm lt, const T* W, int64_t ldw) {
  dh_finish_body<T, TOUT>(part, S, stride, inv, ntok, H, out, lt, W, ldw, (int64_t)blockIdx.x, (int64_t)gridDim.x);
}

// Tokens whose upstream gradients are both zero add nothing to either gradient.  The others are listed in order:
// rows[k] = k-th such token, inv[t] = its position k or -1, *n_rows = how many.  g_lp has stride 0 when one value is
// shared by all tokens (sum / mean reduction).  Two launches over blocks of kActiveBlock tokens: the first counts each
// block's tokens, the second adds up the counts of the blocks before its own and numbers its tokens with wave ballots
// (coalesced reads; 262144 tokens: 0.66 ms as one workgroup walking 256 tokens per thread, now two launches of a few us).
constexpr int kActiveBlock = 4096;

LCE_DEV bool token_is_active(const float* g_lp, int64_t g_lp_stride, const float* g_ent, int64_t t) {
  return (g_lp[t * g_lp_stride] != 0.f) || (g_ent && g_ent[t] != 0.f);
}

inline __global__ __launch_bounds__(256) void active_count_kernel(const float* g_lp, int64_t g_lp_stride, const float* g_ent, int64_t T,
                                                           int* block_counts) {
  __shared__ int part[4];
  const int64_t base = (int64_t)blockIdx.x * kActiveBlock;
  int n = 0;
  for (int k = 0; k < kActiveBlock / 256; ++k) {
    const int64_t t = base + k * 256 + threadIdx.x;
    const bool on = t < T && token_is_active(g_lp, g_lp_stride, g_ent, t);
    n += (int)__popcll(__builtin_amdgcn_ballot_w64(on));  // (the same value in every lane of the wave)
  }
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = n;
  __syncthreads();
  if (threadIdx.x == 0) block_counts[blockIdx.x] = part[0] + part[1] + part[2] + part[3];
}

inline __global__ __launch_bounds__(256) void active_rows_kernel(const float* g_lp, int64_t g_lp_stride, const float* g_ent, int64_t T,
                                                          const int* block_counts, int* rows, int* inv, int* n_rows) {
  __shared__ int part[4];
  __shared__ int before;
  // tokens listed by the blocks before this one
  int acc = 0;
  for (int b = threadIdx.x; b < (int)blockIdx.x; b += 256) acc += block_counts[b];
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) before = part[0] + part[1] + part[2] + part[3];
  __syncthreads();
  int pos0 = before;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t base = (int64_t)blockIdx.x * kActiveBlock;
  for (int k = 0; k < kActiveBlock / 256; ++k) {
    const int64_t t = base + k * 256 + threadIdx.x;
    const bool on = t < T && token_is_active(g_lp, g_lp_stride, g_ent, t);
    const unsigned long long m = __builtin_amdgcn_ballot_w64(on);
    __syncthreads();  // part[] of the previous round has been read
    if (lane == 0) part[wave] = (int)__popcll(m);
    __syncthreads();
    int pre = pos0;
    for (int w = 0; w < wave; ++w) pre += part[w];
    const int pos = pre + (int)__popcll(m & ((1ull << lane) - 1ull));
    if (t < T) {
      inv[t] = on ? pos : -1;
      if (on) rows[pos] = (int)t;
    }
    pos0 += part[0] + part[1] + part[2] + part[3];
  }
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) *n_rows = pos0;
}

inline __global__ void fill_zero_kernel(uint32_t* p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0u;
}

// out[r][:C] = in[rows[r]][:C] (in[r] without `rows`) for r < R = *n_rows (R without), zeros for the rows up to the next
// multiple of 64 (the K granule of the d_weight GEMM); one 16-byte chunk per thread, C a multiple of 16 bytes
template <typename T>
__global__ void gather_rows_kernel(const T* in, int64_t ldi, int64_t R, int64_t C, T* out, int64_t ldo, int64_t rpad, const int* rows,
                                   const int* n_rows) {
  constexpr int N = 16 / (int)sizeof(T);
  typedef typename VecOf<T, N>::type vec_t;
  if (n_rows) R = *n_rows;
  const int64_t rend = (R + 63) / 64 * 64 < rpad ? (R + 63) / 64 * 64 : rpad;
  const int64_t per_row = C / N, n = rend * per_row;
  for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < n; q += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = q / per_row, c = (q - r * per_row) * N;
    vec_t v;
#pragma unroll
    for (int e = 0; e < N; ++e) v[e] = (T)0.f;
    if (r < R) v = *reinterpret_cast<const vec_t*>(in + (rows ? (int64_t)rows[r] : r) * ldi + c);
    *reinterpret_cast<vec_t*>(out + r * ldo + c) = v;
  }
}

// out[c][perm(r)] = in[r][c] for r < R, c < C; out has `ldo` columns, columns perm(r) with r in
// [R, rpad) are zero-filled (rpad a multiple of the permutation's group).  PERM: 0 none,
// 1 KPerm::token, 2 KPerm::vocab.  Grid: (ceil(rpad/128), ceil(C/64)), 256 threads; a workgroup moves
// 128 rows x 64 columns through LDS with 16-byte loads and stores on both sides.
// `in` rows and `out` rows must be 16-byte aligned (ldi, ldo, C multiples of 16 bytes).
// With `rows` / `n_rows` (device), row r of the input is in[rows[r]] for r < *n_rows and R = *n_rows.
template <typename Cfg, int PERM>
__global__ __launch_bounds__(256) void transpose_pad_kernel(const typename Cfg::TIN* in, int64_t ldi, int64_t R, int64_t C,
                                                            typename Cfg::TIN* out, int64_t ldo, int64_t rpad,
                                                            const int* rows = nullptr, const int* n_rows = nullptr) {
  typedef typename Cfg::TIN TIN;
  constexpr int N = 16 / (int)sizeof(TIN);   // elements per 16-byte vector
  constexpr int RB = 128, CB = 64;
  constexpr int PITCH = CB + (sizeof(TIN) == 2 ? 2 : 1);  // odd number of 32-bit words per tile row
  static_assert(KPerm<Cfg>::GT <= RB && KPerm<Cfg>::GV <= RB && RB % KPerm<Cfg>::GT == 0 && RB % KPerm<Cfg>::GV == 0, "group size");
  typedef typename VecOf<TIN, N>::type vec_t;
  __shared__ TIN tile[RB][PITCH];
  const int64_t r0 = (int64_t)blockIdx.x * RB, c0 = (int64_t)blockIdx.y * CB;
  if (n_rows) {
    R = *n_rows;
    if (r0 >= (R + 255) / 256 * 256) return;  // beyond the last K granule that any GEMM reads
  }
  {
    constexpr int LPR = CB / N;            // lanes per row
    constexpr int RPP = 256 / LPR;         // rows per pass
    const int lr = threadIdx.x / LPR, lc = (threadIdx.x % LPR) * N;
#pragma unroll
    for (int k = 0; k < RB / RPP; ++k) {
      const int i = k * RPP + lr;
      const int64_t r = r0 + i, c = c0 + lc;
      vec_t v;
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = (TIN)0.f;
      if (r < R && c < C) {
        const int64_t src = rows ? (int64_t)rows[r] : r;
        v = *reinterpret_cast<const vec_t*>(in + src * ldi + c);
      }
#pragma unroll
      for (int e = 0; e < N; ++e) tile[i][lc + e] = v[e];
    }
  }
  __syncthreads();
  {
    constexpr int LPR = RB / N;            // lanes per output row segment
    constexpr int CPP = 256 / LPR;         // output rows per pass
    const int q = (threadIdx.x % LPR) * N, lc = threadIdx.x / LPR;
#pragma unroll
    for (int k = 0; k < CB / CPP; ++k) {
      const int ci = k * CPP + lc;
      const int64_t c = c0 + ci, u0 = r0 + q;
      if (c >= C || u0 >= rpad) continue;
      vec_t v;
#pragma unroll
      for (int e = 0; e < N; ++e) {
        const int64_t u = u0 + e;
        const int64_t r = PERM == 1 ? KPerm<Cfg>::token_at(u) : (PERM == 2 ? KPerm<Cfg>::vocab_at(u) : u);
        v[e] = tile[(int)(r - r0)][ci];
      }
      __builtin_nontemporal_store(v, reinterpret_cast<vec_t*>(out + c * ldo + u0));  // read back only by later launches
    }
  }
}

// ------------------------------------------------------------------------------------------------
// unfused twins on materialised logits: one workgroup per row, one pass
// ------------------------------------------------------------------------------------------------
template <typename TIN>
LCE_DEV float load_as_float(const TIN* p, int64_t i) { return (float)p[i]; }

// A row is walked as [head | 16-byte vectors | tail]: `head` elements bring the pointer to a 16-byte
// boundary, then every lane loads whole vectors (8 bf16 / 4 fp32), two per trip so that two loads
// are in flight per lane.
template <typename TIN>
struct RowSplit {
  static constexpr int N = 16 / (int)sizeof(TIN);
  typedef typename VecOf<TIN, N>::type vec_t;
  int64_t head, nvec, tail0;
  LCE_DEV RowSplit(const TIN* row, int64_t V) {
    const uint64_t mis = reinterpret_cast<uint64_t>(row) & 15;
    head = (int64_t)(((16 - mis) & 15) / sizeof(TIN));
    if (head > V) head = V;
    nvec = (V - head) / N;
    tail0 = head + nvec * N;
  }
};

// per-row online (max, sum exp, sum z exp): the block leaves m = max, a = sum exp(z - m), b = sum z exp(z - m);
// with SQ the third sum is sum exp(z - m)^2 instead (it rescales with the square of the factor)
template <typename TIN, int NT, bool SQ = false>
LCE_DEV void row_stats(const TIN* row, int64_t V, float& m, float& a, float& b, float* sh) {
  typedef RowSplit<TIN> RS;
  typedef typename RS::vec_t vec_t;
  constexpr int N = RS::N;
  float tm = kNegBig, ta = 0.f, tb = 0.f;
  auto add_one = [&](float z) {
    if (z > tm) {
      const float sc = fast_exp2((tm - z) * kLog2e);
      ta *= sc;
      tb *= SQ ? sc * sc : sc;
      tm = z;
    }
    const float e = fast_exp2((z - tm) * kLog2e);
    ta += e;
    tb = __builtin_fmaf(SQ ? e : z, e, tb);
  };
  auto add_vec = [&](const vec_t& v) {
    float z[N];
    float vm = (float)v[0];
#pragma unroll
    for (int e = 0; e < N; ++e) {
      z[e] = (float)v[e];
      vm = fmaxf(vm, z[e]);
    }
    if (vm > tm) {  // one rescale per vector
      const float sc = fast_exp2((tm - vm) * kLog2e);
      ta *= sc;
      tb *= SQ ? sc * sc : sc;
      tm = vm;
    }
    const float ntm2 = -tm * kLog2e;
#pragma unroll
    for (int e = 0; e < N; ++e) {
      const float ex = fast_exp2(__builtin_fmaf(z[e], kLog2e, ntm2));
      ta += ex;
      tb = __builtin_fmaf(SQ ? ex : z[e], ex, tb);
    }
  };
  auto merge = [&](float& m1, float& a1, float& b1, float m2, float a2, float b2) {
    if (!SQ) return merge_stats(m1, a1, b1, m2, a2, b2, kLog2e);
    const float mn = fmaxf(m1, m2);
    const float s1 = fast_exp2((m1 - mn) * kLog2e), s2 = fast_exp2((m2 - mn) * kLog2e);
    a1 = a1 * s1 + a2 * s2;
    b1 = b1 * s1 * s1 + b2 * s2 * s2;
    m1 = mn;
  };
  const RS rs(row, V);
  for (int64_t v = threadIdx.x; v < rs.head; v += NT) add_one(load_as_float(row, v));
  const vec_t* vp = reinterpret_cast<const vec_t*>(row + rs.head);
  int64_t i = threadIdx.x;
  for (; i + NT < rs.nvec; i += 2 * NT) {
    const vec_t v0 = vp[i], v1 = vp[i + NT];
    add_vec(v0);
    add_vec(v1);
  }
  if (i < rs.nvec) add_vec(vp[i]);
  for (int64_t v = rs.tail0 + threadIdx.x; v < V; v += NT) add_one(load_as_float(row, v));
  // wave reduce
  for (int off = 32; off > 0; off >>= 1) {
    const float m2 = __shfl_xor(tm, off), a2 = __shfl_xor(ta, off), b2 = __shfl_xor(tb, off);
    merge(tm, ta, tb, m2, a2, b2);
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) {
    sh[wave * 3 + 0] = tm;
    sh[wave * 3 + 1] = ta;
    sh[wave * 3 + 2] = tb;
  }
  __syncthreads();
  tm = sh[0];
  ta = sh[1];
  tb = sh[2];
  for (int w = 1; w < NT / 64; ++w) merge(tm, ta, tb, sh[w * 3], sh[w * 3 + 1], sh[w * 3 + 2]);
  m = tm;
  a = ta;
  b = tb;
  __syncthreads();
}

// stats (optional, [R][2]): logsumexp and sum softmax * logit of each row, kept for the backward
template <typename TIN, int NT>
__global__ __launch_bounds__(NT) void logits_fwd_kernel(const TIN* logits, int64_t ldl, const int64_t* labels, int64_t V,
                                                        float* logprobs, float* entropy, float* stats) {
  __shared__ float sh[3 * NT / 64];
  const int64_t r = blockIdx.x;
  const TIN* row = logits + r * ldl;
  float m, a, b;
  row_stats<TIN, NT>(row, V, m, a, b, sh);
  if (threadIdx.x == 0) {
    const float lse = m + logf(a);
    if (entropy) entropy[r] = lse - b / a;
    if (logprobs) {
      const int64_t y = labels[r];
      const float zy = (y >= 0 && y < V) ? load_as_float(row, y) : 0.f;
      logprobs[r] = zy - lse;
    }
    if (stats) {
      stats[2 * r] = lse;
      stats[2 * r + 1] = b / a;
    }
  }
}

// sum over the vocabulary of softmax(row)^2 = sum exp(z - m)^2 / (sum exp(z - m))^2, one pass
// stats (optional, [R]): the row's logsumexp, kept for the backward
template <typename TIN, int NT>
__global__ __launch_bounds__(NT) void logits_pi2_kernel(const TIN* logits, int64_t ldl, int64_t V, float* out, float* stats) {
  __shared__ float sh[3 * NT / 64];
  const int64_t r = blockIdx.x;
  float m, a, q;
  row_stats<TIN, NT, true>(logits + r * ldl, V, m, a, q, sh);
  if (threadIdx.x == 0) {
    out[r] = q / (a * a);
    if (stats) stats[r] = m + logf(a);
  }
}

// gradient of S = sum_v p_v^2 with respect to the logits: dS/dz_k = 2 p_k (p_k - S); d_logits = g * that.
// lse / S: per-row logsumexp and sum of squares from the forward (either may be null: recomputed from the row).
template <typename TIN, int NT>
__global__ __launch_bounds__(NT) void logits_pi2_bwd_kernel(const TIN* logits, int64_t ldl, int64_t V, const float* lse_in, const float* s_in,
                                                            const float* g, TIN* dl, int64_t ldd) {
  typedef RowSplit<TIN> RS;
  typedef typename RS::vec_t vec_t;
  constexpr int N = RS::N;
  __shared__ float sh[3 * NT / 64];
  const int64_t r = blockIdx.x;
  const TIN* row = logits + r * ldl;
  float lse, S;
  if (lse_in && s_in) {
    lse = lse_in[r];
    S = s_in[r];
  } else {
    float m, a, q;
    row_stats<TIN, NT, true>(row, V, m, a, q, sh);
    lse = m + logf(a);
    S = q / (a * a);
  }
  const float lse2 = lse * kLog2e, g2 = 2.f * g[r];
  TIN* out = dl + r * ldd;
  auto value = [&](float z) {
    const float pr = fast_exp2(__builtin_fmaf(z, kLog2e, -lse2));
    return g2 * pr * (pr - S);
  };
  const RS rs(row, V);
  const bool same = ((reinterpret_cast<uint64_t>(out) ^ reinterpret_cast<uint64_t>(row)) & 15) == 0;  // vector stores line up too
  if (!same) {
    for (int64_t v = threadIdx.x; v < V; v += NT) out[v] = (TIN)value(load_as_float(row, v));
    return;
  }
  for (int64_t v = threadIdx.x; v < rs.head; v += NT) out[v] = (TIN)value(load_as_float(row, v));
  const vec_t* vp = reinterpret_cast<const vec_t*>(row + rs.head);
  vec_t* op = reinterpret_cast<vec_t*>(out + rs.head);
  auto vec = [&](int64_t i, const vec_t& v) {
    vec_t o;
#pragma unroll
    for (int e = 0; e < N; ++e) o[e] = (TIN)value((float)v[e]);
    __builtin_nontemporal_store(o, &op[i]);  // written once, never re-read by this kernel
  };
  int64_t i = threadIdx.x;
  for (; i + 3 * NT < rs.nvec; i += 4 * NT) {  // four loads in flight per lane
    const vec_t a0 = vp[i], a1 = vp[i + NT], a2 = vp[i + 2 * NT], a3 = vp[i + 3 * NT];
    vec(i, a0);
    vec(i + NT, a1);
    vec(i + 2 * NT, a2);
    vec(i + 3 * NT, a3);
  }
  for (; i < rs.nvec; i += NT) vec(i, vp[i]);
  for (int64_t v = rs.tail0 + threadIdx.x; v < V; v += NT) out[v] = (TIN)value(load_as_float(row, v));
}

template <typename TIN, int NT>
__global__ __launch_bounds__(NT) void logits_bwd_kernel(const TIN* logits, int64_t ldl, const int64_t* labels, int64_t V,
                                                        const float* stats, const float* g_lp, const float* g_ent, TIN* dl,
                                                        int64_t ldd) {
  typedef RowSplit<TIN> RS;
  typedef typename RS::vec_t vec_t;
  constexpr int N = RS::N;
  __shared__ float sh[3 * NT / 64];
  const int64_t r = blockIdx.x;
  const TIN* row = logits + r * ldl;
  float lse, eb;
  if (stats) {
    lse = stats[2 * r];
    eb = stats[2 * r + 1];
  } else {
    float m, a, b;
    row_stats<TIN, NT>(row, V, m, a, b, sh);
    lse = m + logf(a);
    eb = b / a;
  }
  const float lse2 = lse * kLog2e;
  const float glp = g_lp ? g_lp[r] : 0.f;
  const float gent = g_ent ? g_ent[r] : 0.f;
  const int64_t y = (g_lp && labels) ? labels[r] : -1;
  TIN* out = dl + r * ldd;
  // d = p * (-glp - gent * (z - eb)) = p * (c0 + c1 * z)
  const float c0 = -glp + gent * eb, c1 = -gent;
  auto one = [&](int64_t v) {
    const float z = load_as_float(row, v);
    float d = fast_exp2(__builtin_fmaf(z, kLog2e, -lse2)) * __builtin_fmaf(z, c1, c0);
    if (v == y) d += glp;
    out[v] = (TIN)d;
  };
  const RS rs(row, V);
  const bool same = ((reinterpret_cast<uint64_t>(out) ^ reinterpret_cast<uint64_t>(row)) & 15) == 0;  // vector stores line up too
  if (!same) {
    for (int64_t v = threadIdx.x; v < V; v += NT) one(v);
    return;
  }
  for (int64_t v = threadIdx.x; v < rs.head; v += NT) one(v);
  const vec_t* vp = reinterpret_cast<const vec_t*>(row + rs.head);
  vec_t* op = reinterpret_cast<vec_t*>(out + rs.head);
  auto vec = [&](int64_t i, const vec_t& v) {
    vec_t o;
    const int64_t v0 = rs.head + i * N;
#pragma unroll
    for (int e = 0; e < N; ++e) {
      const float z = (float)v[e];
      float d = fast_exp2(__builtin_fmaf(z, kLog2e, -lse2)) * __builtin_fmaf(z, c1, c0);
      if (v0 + e == y) d += glp;
      o[e] = (TIN)d;
    }
    __builtin_nontemporal_store(o, &op[i]);  // written once, never re-read by this kernel
  };
  int64_t i = threadIdx.x;
  for (; i + 3 * NT < rs.nvec; i += 4 * NT) {  // four loads in flight per lane
    const vec_t a0 = vp[i], a1 = vp[i + NT], a2 = vp[i + 2 * NT], a3 = vp[i + 3 * NT];
    vec(i, a0);
    vec(i + NT, a1);
    vec(i + 2 * NT, a2);
    vec(i + 3 * NT, a3);
  }
  for (; i < rs.nvec; i += NT) vec(i, vp[i]);
  for (int64_t v = rs.tail0 + threadIdx.x; v < V; v += NT) one(v);
}

// ------------------------------------------------------------------------------------------------
// consumer of the path's outputs: clipped PPO policy loss + entropy bonus + KL penalty against a reference
// policy, every aggregation mode of agg_loss
// ------------------------------------------------------------------------------------------------
enum { PPO_KL_NONE = 0, PPO_KL_K1 = 1, PPO_KL_ABS = 2, PPO_KL_K2 = 3, PPO_KL_K3 = 4 };
enum { PPO_TOKEN_MEAN = 0, PPO_TOKEN_SUM = 1, PPO_SEQ_MEAN_TOKEN_SUM = 2, PPO_SEQ_MEAN_TOKEN_SUM_NORM = 3,
       PPO_SEQ_MEAN_TOKEN_MEAN = 4 };

struct PpoArgs {
  const float* log_prob;  // null: no policy term (plain aggregation of `entropy`)
  const float* entropy;   // may be null
  const float* old_log_prob;
  const float* advantages;
  const float* mask;
  const float* is_weights;  // may be null: per-token factor on the policy loss (rollout correction), a constant
  const float* ref_log_prob;  // with kl_type != PPO_KL_NONE
  int kl_type;
  int kl_straight_through;  // the estimator's value with the gradient of 0.5 * (log_prob - ref_log_prob)^2
  float kl_coef;
  int64_t rows, row_len;    // [rows][row_len], row-major, contiguous
  int segs;                 // workgroups per row
  int64_t seg_len;          // elements per workgroup (the last one of a row may be short)
  float clip_low, clip_high, clip_c, entropy_coeff;
  float* g_log_prob;  // unscaled d(sum of masked losses)/d log_prob
  float* g_entropy;   // may be null
  float* partials;    // [rows * segs][8]
  // Packed model outputs (both null: log_prob, entropy and the two gradients are [rows][row_len] like everything else).
  // Otherwise log_prob / entropy / g_log_prob / g_entropy are [total_nnz] vectors over the packed sequences and element
  // (row, c) lives at pk_start[row] + c for c < pk_len[row]; beyond that the value is the padding constant 0 and there is
  // no gradient to write (the response slice of verl/workers/utils/padding.py:97-141, left-shifted by one token:
  // pk_start = end of the sequence - response length - 1).
  const int64_t* pk_start;
  const int64_t* pk_len;
  int64_t total_nnz;
};

// index of element (row, c) in the model-output vectors, or -1 for a padding position of the packed layout
LCE_DEV int64_t ppo_out_index(const PpoArgs& p, int64_t row, int64_t c) {
  if (!p.pk_start) return row * p.row_len + c;
  const int64_t i = p.pk_start[row] + c;
  return (c < p.pk_len[row] && i >= 0 && i < p.total_nnz) ? i : -1;
}

// Per-token terms and unscaled gradients; workgroup (row, seg) reduces its segment of one row to
// partials[row * segs + seg][0..6] = sums of (loss, entropy, clipped, -log ratio, dual-clipped, 1, kl) x mask.
inline __global__ void ppo_terms_kernel(PpoArgs p) {
  __shared__ float sh[8][256];
  float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int64_t row = (int64_t)blockIdx.x / p.segs;
  const int64_t c0 = ((int64_t)blockIdx.x % p.segs) * p.seg_len;
  const int64_t c1 = c0 + p.seg_len < p.row_len ? c0 + p.seg_len : p.row_len;
  for (int64_t c = c0 + threadIdx.x; c < c1; c += blockDim.x) {
    const int64_t t = row * p.row_len + c;
    const int64_t to = ppo_out_index(p, row, c);
    const float m = p.mask[t];
    const bool on = m != 0.f;  // values outside the mask never reach a sum (NaNs there are harmless)
    float loss = 0.f, dloss = 0.f, nkl = 0.f, clipped = 0.f, dual_clipped = 0.f;
    if (p.log_prob) {
      const float lp = to >= 0 ? p.log_prob[to] : 0.f, A = p.advantages[t];
      const float d = lp - p.old_log_prob[t];
      nkl = fminf(fmaxf(d, -20.f), 20.f);
      const float r = __expf(nkl);
      // (the clamps pass the gradient ON their bounds, as torch.clamp's backward does, and the maximum / minimum split
      // it evenly at a tie, as torch.maximum / torch.min do: the reference's autograd at the kinks)
      const float dr = (d >= -20.f && d <= 20.f) ? r : 0.f;        // d ratio / d log_prob
      const float rc = fminf(fmaxf(r, 1.f - p.clip_low), 1.f + p.clip_high);
      const float drc = (r >= 1.f - p.clip_low && r <= 1.f + p.clip_high) ? dr : 0.f;
      const float l1 = -A * r, l2 = -A * rc, l3 = -A * p.clip_c;
      const float lc1 = fmaxf(l1, l2);
      const float dlc1 = l1 > l2 ? -A * dr : (l2 > l1 ? -A * drc : -A * 0.5f * (dr + drc));
      const bool dual = A < 0.f;
      const float isw = p.is_weights ? p.is_weights[t] : 1.f;
      loss = (dual ? fminf(l3, lc1) : lc1) * isw;
      dloss = (dual ? (l3 < lc1 ? 0.f : (l3 == lc1 ? 0.5f * dlc1 : dlc1)) : dlc1) * isw;
      clipped = l2 > l1 ? 1.f : 0.f;
      dual_clipped = (lc1 > l3 && dual) ? 1.f : 0.f;
      float kl = 0.f;
      if (p.kl_type != PPO_KL_NONE) {
        const float e = lp - p.ref_log_prob[t];
        float dkl;
        if (p.kl_type == PPO_KL_K1) {
          kl = e;
          dkl = 1.f;
        } else if (p.kl_type == PPO_KL_ABS) {
          kl = fabsf(e);
          dkl = e > 0.f ? 1.f : (e < 0.f ? -1.f : 0.f);
        } else if (p.kl_type == PPO_KL_K2) {
          kl = 0.5f * e * e;
          dkl = e;
        } else {  // k3 = exp(q) - q - 1, q = clamp(ref - log_prob, +-20), clamped to +-10
          const float q = fminf(fmaxf(-e, -20.f), 20.f);
          const float em1 = expm1f(q);  // (exp(q) - 1 - q without cancellation near q = 0, where it is q^2 / 2)
          const float k = em1 - q;
          kl = fminf(fmaxf(k, -10.f), 10.f);
          dkl = (-e >= -20.f && -e <= 20.f && k >= -10.f && k <= 10.f) ? -em1 : 0.f;
        }
        if (p.kl_straight_through) dkl = e;
        dloss += p.kl_coef * dkl;
      }
      if (to >= 0) p.g_log_prob[to] = on ? dloss * m : 0.f;
      if (on) s[6] += kl * m;
    }
    float ent = 0.f;
    if (p.entropy) {
      ent = to >= 0 ? p.entropy[to] : 0.f;
      if (to >= 0) p.g_entropy[to] = on ? -p.entropy_coeff * m : 0.f;
    }
    if (on) {
      s[0] += loss * m;
      s[1] += ent * m;
      s[2] += clipped * m;
      s[3] += -nkl * m;
      s[4] += dual_clipped * m;
    }
    s[5] += m;
  }
#pragma unroll
  for (int k = 0; k < 8; ++k) sh[k][threadIdx.x] = s[k];
  __syncthreads();
  for (int w = blockDim.x >> 1; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w)
#pragma unroll
      for (int k = 0; k < 8; ++k) sh[k][threadIdx.x] += sh[k][threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x < 8) p.partials[(int64_t)blockIdx.x * 8 + threadIdx.x] = sh[threadIdx.x][0];
}

struct PpoAgg {
  int mode;
  float dp_size;            // factor on every mode
  float batch_num_tokens;   // token-mean denominator, <= 0: sum(mask)
  float global_batch_size;  // seq-mean denominator, <= 0: number of rows with sum(mask) > 0
  float loss_scale_factor;  // seq-mean-token-sum-norm divisor, <= 0: row_len
  float entropy_coeff, kl_coef;
};

// fixed-order sum of NV doubles per thread over the workgroup (256 threads); result valid in every thread
template <int NV>
__device__ inline void ppo_block_sum(double (&v)[NV], double (*sh)[256]) {
  __syncthreads();
#pragma unroll
  for (int k = 0; k < NV; ++k) sh[k][threadIdx.x] = v[k];
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w)
#pragma unroll
      for (int k = 0; k < NV; ++k) sh[k][threadIdx.x] += sh[k][threadIdx.x + w];
    __syncthreads();
  }
#pragma unroll
  for (int k = 0; k < NV; ++k) v[k] = sh[k][0];
}

// One workgroup of 256 threads.  Row totals from the segment partials (ascending segment), the weight each
// row's token sums carry under the aggregation mode, the loss and the metrics.
// row_tot [rows][4] double (loss, entropy, mask, kl), row_weight [rows] float.
// out: [0] loss = pg_loss - entropy_coeff * entropy_loss + kl_coef * kl_loss, [1] pg_loss, [2] entropy_loss,
//      [3] pg_clipfrac, [4] ppo_kl, [5] pg_clipfrac_lower, [6] sum(mask),
//      [7] dp_size / denominator of the mode (1 / tokens or 1 / sequences included), [8] kl_loss
inline __global__ void ppo_finish_kernel(const float* partials, int64_t rows, int segs, int64_t row_len, PpoAgg g,
                                  double* row_tot, float* row_weight, float* out) {
  __shared__ double sh[5][256];
  double a[5] = {0.0, 0.0, 0.0, 0.0, 0.0};  // clipped, -log ratio, dual-clipped, sum(mask), rows with tokens
  for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) {
    double t[7] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
    for (int sgm = 0; sgm < segs; ++sgm)
#pragma unroll
      for (int k = 0; k < 7; ++k) t[k] += (double)partials[(r * segs + sgm) * 8 + k];
    row_tot[r * 4 + 0] = t[0];
    row_tot[r * 4 + 1] = t[1];
    row_tot[r * 4 + 2] = t[5];
    row_tot[r * 4 + 3] = t[6];
    a[0] += t[2];
    a[1] += t[3];
    a[2] += t[4];
    a[3] += t[5];
    a[4] += t[5] > 0.0 ? 1.0 : 0.0;
  }
  ppo_block_sum(a, sh);
  const double n_tok = a[3];
  const double tok_den = g.batch_num_tokens > 0.f ? (double)g.batch_num_tokens : n_tok;
  const double seq_den = g.global_batch_size > 0.f ? (double)g.global_batch_size : a[4];
  const double norm = g.loss_scale_factor > 0.f ? (double)g.loss_scale_factor : (double)row_len;
  double base;
  switch (g.mode) {
    case PPO_TOKEN_MEAN: base = (double)g.dp_size / tok_den; break;
    case PPO_TOKEN_SUM: base = (double)g.dp_size; break;
    case PPO_SEQ_MEAN_TOKEN_SUM_NORM: base = (double)g.dp_size / seq_den / norm; break;
    default: base = (double)g.dp_size / seq_den; break;
  }
  const bool per_seq = g.mode >= PPO_SEQ_MEAN_TOKEN_SUM;
  double b[3] = {0.0, 0.0, 0.0};
  for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) {
    const double cnt = row_tot[r * 4 + 2];
    double w = base;
    if (per_seq && !(cnt > 0.0)) w = 0.0;  // rows without tokens are excluded from a sequence mean
    if (g.mode == PPO_SEQ_MEAN_TOKEN_MEAN) w /= cnt + 1e-8;
    row_weight[r] = (float)w;
    b[0] += w * row_tot[r * 4 + 0];
    b[1] += w * row_tot[r * 4 + 1];
    b[2] += w * row_tot[r * 4 + 3];
  }
  ppo_block_sum(b, sh);
  if (threadIdx.x == 0) {
    out[0] = (float)(b[0] - (double)g.entropy_coeff * b[1] + (double)g.kl_coef * b[2]);
    out[1] = (float)b[0];
    out[2] = (float)b[1];
    out[3] = (float)(a[0] / (n_tok + 1e-8));
    out[4] = (float)(a[1] / (n_tok + 1e-8));
    out[5] = (float)(a[2] / (n_tok + 1e-8));
    out[6] = (float)n_tok;
    out[7] = (float)base;
    out[8] = (float)b[2];
  }
}

inline __global__ void ppo_scale_kernel(PpoArgs p, const float* row_weight) {
  const int64_t row = (int64_t)blockIdx.x / p.segs;
  const int64_t c0 = ((int64_t)blockIdx.x % p.segs) * p.seg_len;
  const int64_t c1 = c0 + p.seg_len < p.row_len ? c0 + p.seg_len : p.row_len;
  const float scale = row_weight[row];
  for (int64_t c = c0 + threadIdx.x; c < c1; c += blockDim.x) {
    const int64_t t = ppo_out_index(p, row, c);
    if (t < 0) continue;
    if (p.g_log_prob) p.g_log_prob[t] *= scale;
    if (p.g_entropy) p.g_entropy[t] *= scale;
  }
}

}  // namespace lce
