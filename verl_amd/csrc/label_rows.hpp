// The one-hot part of the gradient of the logits, carried outside the 16-bit d_logits tiles.
//
// d_logits[t][v] = G_t * 1[v == label_t] + (terms proportional to softmax_t[v]),  G_t = g_logprob_t / temperature.
// The softmax terms are small everywhere; G_t is O(1..10) and sits in one column per token.  Rounded to bf16
// with the rest of the tile it carries an error of up to 2^-9 * |G_t| into d_hidden[t] and into the label's row
// of d_weight, where several tokens with the same label and gradients of opposite sign leave a small difference
// of large terms.  So the tiles hold the softmax terms only, and the one-hot part is added in fp32:
//   d_hidden[t][:]        += G_t * W[label_t][:]        (when the fp32 partials are summed and rounded)
//   d_weight[label][:]    += sum over tokens t with that label, in ascending t, of G_t * hidden[t][:]
//                            (after the GEMMs have written the softmax terms)
// The second sum needs the tokens grouped by label in a fixed order: a stable LSD radix sort of
// (label row, position in the token list) pairs, 8 bits per pass, written here (no float atomics anywhere, and
// no library call that a captured graph could not replay).
// In the default mode G_t above is replaced by the label's whole entry of d_logits, softmax part included
// (label_coef_kernel), and the tiles hold zero at the label.
#pragma once

#include "lce_kernels.hpp"

namespace lce {

constexpr int kSortBlock = 1024;      // items per workgroup of a sort pass: 4 rounds of 256 threads
constexpr uint32_t kNoRow = 0xFFFFFFFFu;  // key of a token that contributes no one-hot term; sorts last

// label row of `tok` inside this call's weight, or kNoRow when the label is elsewhere or G is zero
LCE_DEV uint32_t label_row(const LabelTerm& lt, int64_t tok, float& G) {
  G = lt.g_lp[tok * lt.g_stride] * lt.scale;
  const int64_t y = lt.labels[tok] - lt.v0;
  return (G != 0.f && y >= 0 && y < lt.V) ? (uint32_t)y : kNoRow;
}

// coef[t] = d_logits[t][label_t] in fp32, the whole entry: p * (C0 + C1 * x) + G with x = hidden[t] . W[label_t]
// recomputed here (one wave per token, 16-byte loads, a fixed shuffle tree), p = exp(x / tau - logsumexp_t).  With it
// the tiles leave the label's entry out altogether, so that for a token that is certain of its label the small
// number G * (1 - p) is formed in fp32 instead of as the difference of G (fp32) and G * p (rounded to 16 bits).
// Zero for tokens without upstream gradient and for labels outside this call's rows of W.  H a multiple of 8.
template <typename T>
struct CoefArgs {
  const T* h;
  int64_t ldh;
  const T* W;
  int64_t ldw;
  const int64_t* labels;
  int64_t v0, V;      // this call's rows of W are vocabulary ids [v0, v0 + V)
  int64_t ntok, H;
  const float* maximum;
  const float* accumulate;
  const float* entropy_b;
  const float* g_lp;  // upstream gradient of the log-probabilities, stride 0 when all tokens share one value
  int64_t g_stride;
  float g_scale;      // 1, or 1 / tokens for the mean
  const float* g_ent; // upstream gradient of the entropy, or null
  float rcp_tau, c;   // 1 / temperature, log2(e) / temperature
  float* coef;        // [ntok]
};

// the coefficient of token t, computed by one whole wave (the same value in every lane)
template <typename T>
LCE_DEV float label_coef_wave(const CoefArgs<T>& a, int64_t t) {
  static_assert(sizeof(T) == 2, "16-bit inputs");
  typedef typename VecOf<T, 8>::type vec_t;
  const int lane = threadIdx.x & 63;
  const float glp = a.g_lp[t * a.g_stride] * a.g_scale;
  const float gent = a.g_ent ? a.g_ent[t] : 0.f;
  const int64_t y = a.labels[t] - a.v0;
  float out = 0.f;
  if ((glp != 0.f || gent != 0.f) && y >= 0 && y < a.V) {  // (uniform over the wave)
    const T* hr = a.h + t * a.ldh;
    const T* wr = a.W + y * a.ldw;
    float x = 0.f;
    for (int64_t k = (int64_t)lane * 8; k < a.H; k += 64 * 8) {
      const vec_t u = *reinterpret_cast<const vec_t*>(hr + k);
      const vec_t w = *reinterpret_cast<const vec_t*>(wr + k);
#pragma unroll
      for (int e = 0; e < 8; ++e) x = __builtin_fmaf((float)u[e], (float)w[e], x);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off);
    const TokenConsts k = token_consts(glp, gent, a.maximum[t], a.accumulate[t], a.entropy_b[t], a.rcp_tau);
    out = dlogit<true>(x, a.c, k.lse2, k.C0, k.C1, k.G, true, false, false);  // the label's own entry: p (C0 + C1 x) + G
  }
  return out;
}

template <typename T>
__global__ __launch_bounds__(256) void label_coef_kernel(CoefArgs<T> a) {
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= a.ntok) return;
  const float out = label_coef_wave(a, t);
  if ((threadIdx.x & 63) == 0) a.coef[t] = out;
}

// keys[k] = label row of the k-th listed token (rows[k], or k itself without a list), vals[k] = that token;
// positions from the list's length up to n_items are filled with kNoRow.
inline __global__ __launch_bounds__(256) void label_keys_kernel(LabelTerm lt, const int* rows, const int* n_rows, int64_t T, int n_items,
                                                         uint32_t* keys, int* vals) {
  const int k = blockIdx.x * 256 + threadIdx.x;
  if (k >= n_items) return;
  const int64_t n = n_rows ? (int64_t)*n_rows : T;
  uint32_t key = kNoRow;
  int tok = -1;
  if (k < n) {
    tok = rows ? rows[k] : k;
    float G;
    key = label_row(lt, tok, G);
  }
  keys[k] = key;
  vals[k] = tok;
}

// ---- one radix pass over `nblocks` blocks of kSortBlock items: histogram, scan, stable scatter ----

// gh[digit * nblocks + block] = number of items of `block` whose digit is `digit`
LCE_DEV void sort_hist_block(const uint32_t* keys, int shift, int block, int nblocks, int* gh, int* h /* LDS [256] */) {
  const int tid = threadIdx.x;
  h[tid] = 0;
  __syncthreads();
#pragma unroll
  for (int q = 0; q < kSortBlock / 256; ++q) atomicAdd(&h[(keys[block * kSortBlock + q * 256 + tid] >> shift) & 255], 1);
  __syncthreads();
  gh[tid * nblocks + block] = h[tid];
}

// Items keep their order inside a digit: the item at position q * 256 + tid of a block ranks behind all items of
// earlier rounds q, earlier waves and lower lanes with the same digit.
LCE_DEV void sort_scatter_block(const uint32_t* kin, const int* vin, uint32_t* kout, int* vout, int shift, int block,
                                int nblocks, const int* gh, int* base /* LDS [256] */) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  base[tid] = gh[tid * nblocks + block];
  __syncthreads();
#pragma unroll
  for (int q = 0; q < kSortBlock / 256; ++q) {
    const int i = block * kSortBlock + q * 256 + tid;
    const uint32_t key = kin[i];
    const int val = vin[i];
    const int d = (int)((key >> shift) & 255);
    uint64_t peers = ~0ull;  // lanes of this wave with the same digit
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const uint64_t bal = __builtin_amdgcn_ballot_w64((d >> b) & 1);
      peers &= ((d >> b) & 1) ? bal : ~bal;
    }
    const int rank = __builtin_popcountll(peers & ((1ull << lane) - 1ull));
    const int cnt = __builtin_popcountll(peers);
    int off = 0;
    for (int w = 0; w < 4; ++w) {
      if (wave == w) {
        off = base[d];                     // every lane of the group reads the running offset ...
        __builtin_amdgcn_wave_barrier();
        if (rank == 0) base[d] = off + cnt;  // ... before its first lane moves it on
      }
      __syncthreads();
    }
    kout[off + rank] = key;
    vout[off + rank] = val;
  }
}

inline __global__ __launch_bounds__(256) void sort_hist_kernel(const uint32_t* keys, int shift, int nblocks, int* gh) {
  __shared__ int h[256];
  sort_hist_block(keys, shift, blockIdx.x, nblocks, gh, h);
}

// exclusive scan of gh[0 .. n) in place, one workgroup of 1024 threads
inline __global__ __launch_bounds__(1024) void sort_scan_kernel(int* gh, int n) {
  __shared__ int part[1024];
  const int tid = threadIdx.x;
  const int per = (n + 1023) / 1024;
  const int i0 = tid * per, i1 = i0 + per < n ? i0 + per : n;
  int s = 0;
  for (int i = i0; i < i1; ++i) s += gh[i];
  part[tid] = s;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    const int v = tid >= off ? part[tid - off] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  int run = part[tid] - s;
  for (int i = i0; i < i1; ++i) {
    const int v = gh[i];
    gh[i] = run;
    run += v;
  }
}

inline __global__ __launch_bounds__(256) void sort_scatter_kernel(const uint32_t* kin, const int* vin, uint32_t* kout, int* vout, int shift,
                                                           int nblocks, const int* gh) {
  __shared__ int base[256];
  sort_scatter_block(kin, vin, kout, vout, shift, blockIdx.x, nblocks, gh, base);
}

// Up to kSortBlock tokens: keys and all passes in one workgroup (buffers 0 / 1 alternate; `passes` is even or
// odd, the caller reads the result from buffer passes % 2).
inline __global__ __launch_bounds__(256) void label_sort_single_kernel(LabelTerm lt, const int* rows, const int* n_rows, int64_t T, int passes,
                                                                uint32_t* keys0, int* vals0, uint32_t* keys1, int* vals1) {
  __shared__ int tab[256];
  __shared__ int gh[256];
  const int tid = threadIdx.x;
  const int64_t n = n_rows ? (int64_t)*n_rows : T;
  if (n <= 256) {
    // few tokens: every thread ranks its own item among all of them (stable: ties by position), one pass, no radix
    // passes (16 -> 4 us with 64 tokens, where the whole backward takes 0.7 ms)
    uint32_t key = kNoRow;
    int tok = -1;
    if (tid < n) {
      tok = rows ? rows[tid] : tid;
      float G;
      key = label_row(lt, tok, G);
    }
    tab[tid] = (int)key;  // (bit pattern; compared as unsigned below)
    __syncthreads();
    int rank = 0;
    for (int j = 0; j < 256; ++j) {
      const uint32_t kj = (uint32_t)tab[j];
      rank += (kj < key || (kj == key && j < tid)) ? 1 : 0;
    }
    uint32_t* kout = (passes & 1) ? keys1 : keys0;  // where the caller reads the result of `passes` radix passes
    int* vout = (passes & 1) ? vals1 : vals0;
    kout[rank] = key;
    vout[rank] = tok;
    for (int k = 256 + tid; k < kSortBlock; k += 256) {
      kout[k] = kNoRow;
      vout[k] = -1;
    }
    return;
  }
  for (int k = tid; k < kSortBlock; k += 256) {
    uint32_t key = kNoRow;
    int tok = -1;
    if (k < n) {
      tok = rows ? rows[k] : k;
      float G;
      key = label_row(lt, tok, G);
    }
    keys0[k] = key;
    vals0[k] = tok;
  }
  __syncthreads();
  for (int p = 0; p < passes; ++p) {
    const uint32_t* kin = (p & 1) ? keys1 : keys0;
    const int* vin = (p & 1) ? vals1 : vals0;
    uint32_t* kout = (p & 1) ? keys0 : keys1;
    int* vout = (p & 1) ? vals0 : vals1;
    sort_hist_block(kin, 8 * p, 0, 1, gh, tab);
    __syncthreads();
    // exclusive scan of the 256 digit counts
    const int own = gh[tid];
    tab[tid] = own;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
      const int v = tid >= off ? tab[tid - off] : 0;
      __syncthreads();
      tab[tid] += v;
      __syncthreads();
    }
    gh[tid] = tab[tid] - own;
    __syncthreads();
    sort_scatter_block(kin, vin, kout, vout, 8 * p, 0, 1, gh, tab);
    __syncthreads();
  }
}

// d_weight[row][:] += sum of G_t * hidden[t][:] over the run of sorted positions with key == row, in order.
// One workgroup per sorted position; only the first position of a run works.  Runs after the d_weight GEMMs:
// the rows are read back in the output dtype (rounded once by the GEMM that wrote the softmax terms, which are
// small next to the one-hot sums on all but a few rows) and rounded once more with the sum added in fp32.
// (TOUT: the dtype d_weight is returned in, the input dtype or fp32)
template <typename T, typename TOUT>
__global__ __launch_bounds__(256) void dw_label_rows_kernel(const uint32_t* keys, const int* toks, int n_items, LabelTerm lt, const T* h,
                                                            int64_t ldh, int64_t H, TOUT* dW) {
  constexpr int N = 16 / (int)sizeof(T);
  typedef typename VecOf<T, N>::type vec_t;
  const int i = blockIdx.x;
  const uint32_t key = keys[i];
  if (key == kNoRow || (i > 0 && keys[i - 1] == key)) return;
  TOUT* row = dW + (int64_t)key * H;
  for (int64_t c = (int64_t)threadIdx.x * N; c < H; c += 256 * N) {
    typedef typename VecOf<TOUT, N>::type ovec_t;
    const ovec_t cur = *reinterpret_cast<const ovec_t*>(row + c);
    float acc[N];
#pragma unroll
    for (int e = 0; e < N; ++e) acc[e] = 0.f;
    for (int j = i; j < n_items && keys[j] == key; ++j) {
      const int64_t tok = toks[j];
      const float G = lt.g_lp[tok * lt.g_stride] * lt.scale;
      const vec_t hv = *reinterpret_cast<const vec_t*>(h + tok * ldh + c);
#pragma unroll
      for (int e = 0; e < N; ++e) acc[e] = __builtin_fmaf(G, (float)hv[e], acc[e]);
    }
#pragma unroll
    for (int e = 0; e < N; ++e) acc[e] += (float)cur[e];
    ovec_t out;
#pragma unroll
    for (int e = 0; e < N; ++e) out[e] = round_to<TOUT>(acc[e]);
    *reinterpret_cast<ovec_t*>(row + c) = out;
  }
}

// ------------------------------------------------------------------------------------------------------------------
// Few tokens (at most 128, 16-bit inputs): a backward of well under a millisecond, where every small launch costs
// 5 us or more.  One launch before the d_logits pass and one after the gradient GEMMs replace eight:
//   few_prep_kernel    the list of tokens with a gradient (active_count / active_rows), the label coefficients
//                      (label_coef) and the compact copy of hidden (gather_rows);
//   few_finish_kernel  d_hidden from its partials (dh_finish) and the one-hot rows of d_weight (dw_label_rows), which
//                      finds the tokens that share a label by comparing all pairs instead of sorting them.
// Results are the same bits as from the separate kernels: same expressions, same order of every sum.
// ------------------------------------------------------------------------------------------------------------------

// Workgroup b: every workgroup lists the tokens itself (ballots over at most 128 gradients); workgroup 0 stores the
// list; workgroup b then owns compact position b: the row of hidden it copies to Ht[b] (zeros from the list's end up to
// the next multiple of 64, the K granule of the d_weight product) and that token's label coefficient (wave 0).
// Grid: tokens rounded up to 64, at most rpad.  a.coef may be null (no coefficients wanted).
template <typename T>
__global__ __launch_bounds__(256) void few_prep_kernel(CoefArgs<T> a, T* Ht, int64_t ldHt, int64_t rpad, int* rows, int* inv, int* n_rows) {
  static_assert(sizeof(T) == 2, "16-bit inputs");
  typedef typename VecOf<T, 8>::type vec_t;
  __shared__ int list[128];
  __shared__ int cnt[2];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  bool on = false;
  int before = 0;
  if (wave < 2) {
    on = tid < a.ntok && token_is_active(a.g_lp, a.g_stride, a.g_ent, tid);
    const unsigned long long m = __builtin_amdgcn_ballot_w64(on);
    before = (int)__popcll(m & ((1ull << lane) - 1ull));
    if (lane == 0) cnt[wave] = (int)__popcll(m);
  }
  __syncthreads();
  const int n = cnt[0] + cnt[1];
  if (wave < 2) {
    const int pos = (wave ? cnt[0] : 0) + before;
    if (on) list[pos] = tid;
    if (blockIdx.x == 0 && tid < a.ntok) {
      inv[tid] = on ? pos : -1;
      if (on) rows[pos] = tid;
      else if (a.coef) a.coef[tid] = 0.f;
    }
  }
  if (blockIdx.x == 0 && tid == 0) *n_rows = n;
  __syncthreads();
  const int k = blockIdx.x;
  const int64_t rend = ((int64_t)n + 63) / 64 * 64 < rpad ? ((int64_t)n + 63) / 64 * 64 : rpad;
  if (k >= rend) return;
  const int64_t tok = k < n ? list[k] : -1;
  for (int64_t c = (int64_t)tid * 8; c < a.H; c += 256 * 8) {
    vec_t v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (T)0.f;
    if (tok >= 0) v = *reinterpret_cast<const vec_t*>(a.h + tok * a.ldh + c);
    *reinterpret_cast<vec_t*>(Ht + (int64_t)k * ldHt + c) = v;
  }
  if (tok >= 0 && a.coef && wave == 0) {
    const float out = label_coef_wave(a, tok);
    if (lane == 0) a.coef[tok] = out;
  }
}

// Workgroups [0, n_dh): d_hidden, as dh_finish_kernel with that many workgroups.  Workgroup n_dh + i: compact position
// i of the token list; the first position of each label adds sum of G_t * hidden[t][:] over the positions with that
// label, in order, to the label's row of d_weight (as dw_label_rows_kernel does over a sorted run).
template <typename T, typename TOUT>
__global__ __launch_bounds__(256) void few_finish_kernel(const float* part, int S, int64_t stride, const int* inv, int64_t ntok, int64_t H,
                                                         TOUT* d_hidden, LabelTerm lt, const T* W, int64_t ldw, int n_dh, const int* rows,
                                                         const int* n_rows, const T* h, int64_t ldh, TOUT* dW) {
  if ((int)blockIdx.x < n_dh) {
    dh_finish_body<T, TOUT>(part, S, stride, inv, ntok, H, d_hidden, lt, W, ldw, (int64_t)blockIdx.x, (int64_t)n_dh);
    return;
  }
  constexpr int N = 16 / (int)sizeof(T);
  typedef typename VecOf<T, N>::type vec_t;
  __shared__ uint32_t keys[128];
  __shared__ float coefs[128];
  __shared__ int toks[128];
  const int i = (int)blockIdx.x - n_dh, tid = threadIdx.x;
  const int n = *n_rows;
  if (i >= n) return;
  if (tid < n && tid < 128) {
    const int tok = rows[tid];
    float G;
    keys[tid] = label_row(lt, tok, G);
    coefs[tid] = G;
    toks[tid] = tok;
  }
  __syncthreads();
  const uint32_t key = keys[i];
  if (key == kNoRow) return;
  for (int j = 0; j < i; ++j)
    if (keys[j] == key) return;  // (the same for every thread) an earlier position owns this row
  TOUT* row = dW + (int64_t)key * H;
  for (int64_t c = (int64_t)tid * N; c < H; c += 256 * N) {
    typedef typename VecOf<TOUT, N>::type ovec_t;
    const ovec_t cur = *reinterpret_cast<const ovec_t*>(row + c);
    float acc[N];
#pragma unroll
    for (int e = 0; e < N; ++e) acc[e] = 0.f;
    for (int j = i; j < n; ++j) {
      if (keys[j] != key) continue;
      const float G = coefs[j];
      const vec_t hv = *reinterpret_cast<const vec_t*>(h + (int64_t)toks[j] * ldh + c);
#pragma unroll
      for (int e = 0; e < N; ++e) acc[e] = __builtin_fmaf(G, (float)hv[e], acc[e]);
    }
#pragma unroll
    for (int e = 0; e < N; ++e) acc[e] += (float)cur[e];
    ovec_t out;
#pragma unroll
    for (int e = 0; e < N; ++e) out[e] = round_to<TOUT>(acc[e]);
    *reinterpret_cast<ovec_t*>(row + c) = out;
  }
}

}  // namespace lce
