// Host-side launch logic of liblce_gfx950.so shared by its translation units: tuning state, timing scopes, tile
// variants, workspace layouts and the templated forward / backward launchers.  The library is compiled as one object per
// (element type, direction) from lce_dtype.hip plus the C ABI in lce_abi.hip, so everything here sits in an anonymous
// namespace (one private copy per object) except the mutable state, which lce_abi.hip defines once.
#pragma once
#include "../../include/lce_abi.h"

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include <mutex>
#include <utility>
#include <vector>

#include "label_rows.hpp"
#include "lce_kernels.hpp"
#include "lce_kernels16.hpp"
#include "few_tokens.hpp"

using namespace lce;

// ---- state shared by every object of the library; defined in lce_abi.hip ----
namespace lce_shared {
extern thread_local char err[512];  // message of the calling thread's last failure (lce_last_error)
struct ProfRec { int cls; hipEvent_t a, b; };
extern std::mutex prof_mu;
extern bool prof_on;
extern std::vector<ProfRec> prof_recs;
extern std::vector<hipEvent_t> prof_pool;

// Defaults of the 32x32x16 loops: the backward's long-K GEMMs gain 3% from the split ring; the forward gains from it
// only up to 8192 tokens and beyond that fetches twice as much through the fabric with it at the same speed (the XCD's
// workgroups drift apart and lose L2 sharing), so large fp32 forwards keep the 2-stage ring.  16-bit inputs run the
// four-wave 16x16x32 loop (variant 3) above the token counts below.
constexpr int kDefaultVariantFwd = 2, kDefaultVariantBwd = 1, kVariantCore16 = 3;
// variant 3 is the default above these token counts (measured at H=3584, V=152064: the forward gains 2-6% from 1024
// tokens on; forward + backward is 2% slower with it at 1024 tokens, 2% faster at 1536 and 2048, 4% at 3072)
constexpr int64_t kCore16MinTokensFwd = 512, kCore16MinTokensBwd = 1280;
struct Tuning {
  int variant_fwd = kDefaultVariantFwd, variant_bwd = kDefaultVariantBwd;
  bool variant_forced = false;   // lce_set_variant was called: no size-based choice of the tile
  int split_bwd = 0;             // diagnostic: launch the three sub-problems of a backward chunk separately
  int ds_tokens_first = -1;      // tile order of the d_logits pass; -1: by size
  int label_outside = 2;         // 16-bit inputs: the label's entry of d_logits added in fp32 outside the d_logits tiles (1: only its one-hot part)
  int dh_ksplit = 0;             // K slices of the d_hidden GEMM; 0: chosen by shape
  int64_t ws_budget = 0;         // byte budget of the backward workspace; 0: the built-in bound
  int64_t keep_logits_tokens = LCE_KEEP_LOGITS_NO_LIMIT;  // a lower limit than half the hidden size for lce_logits_cache_bytes (0: never)
  int few_token_gemms = 1;       // gradient GEMMs of a backward with at most 128 tokens: the streaming kernels of few_tokens.hpp
};

// tile selectors of the per-type launchers: 0..3 are the variants of lce_set_variant, then the two few-token forward tiles
enum { kSelT64 = 4, kSelT128 = 5 };

// The launchers of one element type each (lce_dtype.hip compiles them as separate objects).  `sel` is a tile selector;
// the other arguments are those of forward_impl / backward_impl / launch_gemm below with untyped pointers.
#define LCE_FWD_PARAMS                                                                                                      \
  const void *h, int64_t ldh, const void *W, int64_t ldw, const int64_t *labels, int64_t T, int64_t H, int64_t V,          \
      float temperature, int reduction, float *lp, float *ent, float *mx, float *ac, float *eb, char *ws, hipStream_t st,   \
      int64_t label_offset, float *shard_out, int max_splits, float *xcache
#define LCE_BWD_PARAMS                                                                                                      \
  const void *h, int64_t ldh, const void *W, int64_t ldw, const int64_t *labels, int64_t T, int64_t H, int64_t V,          \
      float temperature, int reduction, const float *mx, const float *ac, const float *eb, const float *glp,               \
      const float *gent, void *dh, void *dw, bool grads_f32, char *ws, int64_t vchunk, hipStream_t st,                     \
      int64_t vocab_offset, const Tuning &tu, const float *xcache
#define LCE_GEMM_PARAMS                                                                                                     \
  const void *A, int64_t lda, const void *B, int64_t ldb, float *C, int64_t ldc, int64_t M, int64_t N, int64_t K,          \
      hipStream_t st
int forward_bf16(int sel, LCE_FWD_PARAMS);
int forward_f16(int sel, LCE_FWD_PARAMS);
int forward_f32(int sel, LCE_FWD_PARAMS);
int backward_bf16(int sel, LCE_BWD_PARAMS);
int backward_f16(int sel, LCE_BWD_PARAMS);
int backward_f32(int sel, LCE_BWD_PARAMS);
int gemm_nt_bf16(int sel, LCE_GEMM_PARAMS);
int gemm_nt_f16(int sel, LCE_GEMM_PARAMS);
int gemm_nt_f32(int sel, LCE_GEMM_PARAMS);
// C[M,N] fp32 = A^T B for K-major bf16 operands A [K, lda], B [K, ldb]; core16: on the 16x16x32 loop
int gemm_tn_bf16(bool core16, LCE_GEMM_PARAMS);
}  // namespace lce_shared
using namespace lce_shared;

namespace {

bool known_dtype(int dtype) { return dtype == LCE_DTYPE_BF16 || dtype == LCE_DTYPE_F32 || dtype == LCE_DTYPE_F16; }
size_t esize(int dtype) { return dtype == LCE_DTYPE_F32 ? 4 : 2; }

// the mainloop variant a backward over T tokens of `esz`-byte elements runs with.  The backward is built on two of the
// mainloops: the four-wave 16x16x32 loop (variant 3) and the eight-wave split ring with the B operand early (variant 1,
// which a forced variant 0 or 2 also selects: those two differ from it only in ways that matter to the forward).
int bwd_variant(const Tuning& tu, int64_t T, size_t esz) {
  if (tu.variant_forced) return tu.variant_bwd == kVariantCore16 ? kVariantCore16 : kDefaultVariantBwd;
  return (esz == 2 && T > kCore16MinTokensBwd) ? kVariantCore16 : kDefaultVariantBwd;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(lce_shared::err, sizeof(lce_shared::err), fmt, ap);
  va_end(ap);
  return code;
}

// ---- optional per-kernel-class timing with HIP events (off by default; used by the benchmark) ----
enum { PC_FWD = 0, PC_FWD_MERGE, PC_BWD_DS, PC_GEMM_DH, PC_GEMM_DW, PC_TRANSPOSE, PC_LOGITS_FWD, PC_LOGITS_BWD, PC_BWD_CHUNK, PC_ACTIVE_ROWS, PC_DH_FINISH, PC_LABEL_ROWS, PC_COUNT };

hipEvent_t prof_event() {
  if (!lce_shared::prof_pool.empty()) { hipEvent_t e = lce_shared::prof_pool.back(); lce_shared::prof_pool.pop_back(); return e; }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}
struct ProfScope {
  bool on; int cls; hipStream_t st; hipEvent_t a;
  ProfScope(int c, hipStream_t s) : on(lce_shared::prof_on), cls(c), st(s), a(nullptr) {
    if (on) { std::lock_guard<std::mutex> l(lce_shared::prof_mu); a = prof_event(); (void)hipEventRecord(a, st); }
  }
  ~ProfScope() {
    if (on) { std::lock_guard<std::mutex> l(lce_shared::prof_mu); hipEvent_t b = prof_event(); (void)hipEventRecord(b, st); lce_shared::prof_recs.push_back({cls, a, b}); }
  }
};

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(LCE_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return LCE_OK;
}

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// tile configurations of the mainloop, selectable for tuning (lce_set_variant)
//            TIN     BM   BN   BKB NSTAGE WAVES_M WAVES_N SPLIT
template <typename TIN> struct Variant0 { typedef GemmCfg<TIN, 256, 256, 128, 5, 4, 2, 1> Cfg; };  // split ring of five half stages, A early
template <typename TIN> struct Variant1 { typedef GemmCfg<TIN, 256, 256, 128, 5, 4, 2, 2> Cfg; };  // split ring of five half stages, B early
template <typename TIN> struct Variant2 { typedef GemmCfg<TIN, 256, 256, 128, 2, 4, 2> Cfg; };     // two whole stages
// four waves of 128x128 on v_mfma_f32_16x16x32 (16-bit inputs; fp32 inputs run the split-ring 32x32x2 loop instead)
template <typename TIN> struct Variant3 { typedef GemmCfg16<TIN> Cfg; };
template <> struct Variant3<float> { typedef GemmCfg<float, 256, 256, 128, 5, 4, 2, 2> Cfg; };
// forward with few tokens (one pass over W, HBM-bound): narrow token tiles leave LDS for a deeper ring
template <typename TIN> struct VariantT64 { typedef GemmCfg<TIN, 256, 64, 128, 4, 4, 2> Cfg; };
template <typename TIN> struct VariantT128 { typedef GemmCfg<TIN, 256, 128, 128, 3, 4, 2> Cfg; };
constexpr int kNumVariants = 4;

template <typename K>
void allow_lds(K kernel, int bytes) {
  // dynamic LDS above 64 KiB has to be enabled per kernel; cheap and idempotent
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

int block_rows(int nrow_tiles) { return TileMap::block_rows(nrow_tiles); }

// ---------------------------------------------------------------------------------------------
template <typename Cfg>
GemmArgs<typename Cfg::TIN> make_gemm_args(const typename Cfg::TIN* A, int64_t lda, const typename Cfg::TIN* B, int64_t ldb,
                                           int64_t M, int64_t N, int64_t K, float* Cf, int64_t ldcf, typename Cfg::TIN* Ct,
                                           int64_t ldct, int out_mode) {
  GemmArgs<typename Cfg::TIN> p;
  p.A = A; p.lda = lda; p.B = B; p.ldb = ldb; p.M = M; p.N = N; p.K = K;
  p.Cf = Cf; p.ldcf = ldcf; p.Ct = Ct; p.ldct = ldct; p.out_mode = out_mode;
  p.ksplit = 1; p.kslice = K; p.cf_split_stride = 0;
  p.m_dev = nullptr; p.k_dev = nullptr; p.k_gran = 1; p.tn = 0; p.b_rows_valid = 0; p.perm_rows = 0;
  const int tm = (int)((M + Cfg::BM - 1) / Cfg::BM), tn = (int)((N + Cfg::BN - 1) / Cfg::BN);
  p.map = TileMap::make(tm, tn, block_rows(tm), 1);
  return p;
}

template <typename Cfg>
int launch_gemm(const typename Cfg::TIN* A, int64_t lda, const typename Cfg::TIN* B, int64_t ldb, int64_t M, int64_t N,
                int64_t K, float* Cf, int64_t ldcf, typename Cfg::TIN* Ct, int64_t ldct, int out_mode,
                hipStream_t st, int prof_cls = PC_GEMM_DH) {
  typedef typename Cfg::TIN TIN;
  if (M <= 0 || N <= 0) return LCE_OK;
  if (K <= 0 || K % Cfg::BK != 0) return fail(LCE_E_ARG, "gemm: K=%lld must be a positive multiple of %d", (long long)K, Cfg::BK);
  const GemmArgs<TIN> p = make_gemm_args<Cfg>(A, lda, B, ldb, M, N, K, Cf, ldcf, Ct, ldct, out_mode);
  ProfScope prof(prof_cls, st);
  if constexpr (Cfg::CORE16) {
    if (N % 4 != 0) return fail(LCE_E_ARG, "gemm: N=%lld must be a multiple of 4", (long long)N);
    allow_lds(gemm16_nt_kernel<Cfg>, Cfg::LDS_BYTES);
    hipLaunchKernelGGL(gemm16_nt_kernel<Cfg>, dim3(p.map.total), dim3(Cfg::NTHREADS), Cfg::LDS_BYTES, st, p);
  } else {
    allow_lds(gemm_nt_kernel<Cfg>, Cfg::LDS_BYTES);
    hipLaunchKernelGGL(gemm_nt_kernel<Cfg>, dim3(p.map.total), dim3(Cfg::NTHREADS), Cfg::LDS_BYTES, st, p);
  }
  return check_launch("gemm_nt_kernel");
}

// Vocabulary splits of the forward with 256-token tiles.  A workgroup owns one (token tile, split) pair and walks the
// split's vocabulary tiles itself, and the tile map gives every XCD the same number of workgroups, so the launch takes
// ceil(workgroups / CUs) rounds of ceil(tiles / splits) tiles each: pick the split count with the fewest tile-times,
// counting a quarter of a tile per workgroup for its ramp-up and its partial results (so ties go to fewer splits), from
// the XCD block's width `bc` on: the 32 workgroups that share an L2 then cover 32 / bc token tiles x bc splits and fetch
// each operand slab once for several of them.  (One split per token tile, which ties on tile-times from 256 token tiles
// on, leaves every workgroup of an XCD with its own 256 rows of hidden: measured 440 instead of 1300 TFLOP/s at 65536
// and at 262144 tokens.)  With 48 token tiles (12288 tokens) eight splits are 384 workgroups = two rounds of 75 tiles;
// sixteen splits give three rounds of 38.
constexpr int kNumCUs = 256;
constexpr int kMaxSplits = 256;
int forward_splits_256(int ntt, int nvt, int max_splits = kMaxSplits) {
  const int bc = 32 / block_rows(ntt);
  if (max_splits < bc) return max_splits > 1 ? max_splits : 1;  // (a caller with very little room for partial results)
  auto cost_of = [&](int S, int64_t* tiles_out) {
    const int64_t per_xcd = ((int64_t)ntt * S + 7) / 8;
    const int64_t rounds = (per_xcd + kNumCUs / 8 - 1) / (kNumCUs / 8);
    const int64_t tiles = (nvt + S - 1) / S;
    if (tiles_out) *tiles_out = tiles;
    return rounds * (4 * tiles + 1);
  };
  int best = bc;
  int64_t best_cost = -1;
  for (int S = bc; S <= max_splits && (S <= nvt || S == bc); ++S) {
    const int64_t cost = cost_of(S, nullptr);
    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best = S; }
  }
  // Among the split counts within 2 % of the fewest tile-times, one that makes a workgroup walk 48 to 96 tiles is
  // preferred: the longer the walk, the further the 32 workgroups of an XCD drift apart and the fewer of them share a
  // fetched slab; the shorter, the more the rounds' ramp-up shows.  Measured, forward launch (tiles per workgroup: ms):
  // T=16384, H=3584, V=152064: 149: 13.47, 75: 13.30, 50: 13.26, 38: 13.51, fetched through the fabric 59.6 -> 30.8 GB;
  // T=32768, H=4096, V=128256: 126: 25.23, 63: 24.88, 42: 24.69, 32: 24.97; T=65536, H=5120: 149: 74.8, 75: 72.6, 50: 73.4.
  int pick = -1;
  int64_t pick_cost = -1;
  for (int S = bc; S <= max_splits && (S <= nvt || S == bc); ++S) {
    int64_t tiles;
    const int64_t cost = cost_of(S, &tiles);
    if (cost * 100 > best_cost * 102 || tiles < 48 || tiles > 96) continue;
    if (pick_cost < 0 || cost < pick_cost) { pick_cost = cost; pick = S; }
  }
  if (pick > 0) best = pick;
  return best;
}

// Kept logits: fp32 [T][logits_cache_row(V)], element [t][v] = hidden[t] . W[v].  A backward that is given them
// computes d_logits from 4 bytes per logit instead of from a pass over W and a T x V x H product.  Offered for 16-bit
// inputs while the cache is no larger than the weight it came from: T * V * 4 <= V * H * 2, i.e. up to H / 2 tokens;
// beyond that nothing of size T x V is ever kept.
int64_t logits_cache_row(int64_t V) { return round_up(V, 64); }
int64_t logits_cache_max_tokens(int64_t H, size_t esz) { return esz == 2 ? H / 2 : 0; }

template <typename Cfg>
int forward_impl(const typename Cfg::TIN* h, int64_t ldh, const typename Cfg::TIN* W, int64_t ldw, const int64_t* labels,
                 int64_t T, int64_t H, int64_t V, float temperature, int reduction, float* logprobs, float* entropy,
                 float* maximum, float* accumulate, float* entropy_b, char* ws, hipStream_t st, int64_t label_offset = 0,
                 float* shard_out = nullptr, int max_splits = kMaxSplits, float* xcache = nullptr) {
  // shard_out: W is one shard of a larger vocabulary starting at row label_offset; instead of the five
  // outputs the per-token partial (max, sum exp, sum logit*exp, label logit) goes to shard_out [T][4]
  typedef typename Cfg::TIN TIN;
  const int ntt = (int)((T + Cfg::BN - 1) / Cfg::BN);
  const int nvt = (int)((V + Cfg::BM - 1) / Cfg::BM);
  // splits: enough workgroups to fill 256 CUs, in multiples of the XCD block width
  const int br = block_rows(ntt), bc = 32 / br;
  const int nrb = (ntt + br - 1) / br;
  // max_splits: the caller's workspace holds partial results of at most that many splits
  int S = Cfg::BN == 256 ? forward_splits_256(ntt, nvt, max_splits) : bc * ((8 + nrb - 1) / nrb);
  if (S > nvt) S = nvt;
  if (S > max_splits) S = max_splits;
  // The narrow token tiles serve the HBM-bound case (up to 128 tokens: one streaming read of W).  There each
  // split takes one contiguous range of rows, the same length for all, instead of whole tiles dealt round robin
  // (594 tiles over 256 splits would be 3 against 2, and a split's tiles would lie 256 tiles apart).  Measured
  // on the kernel, H=3584, V=152064: T=1 203 -> 187 us, T=64 209 -> 190, T=128 221 -> 211; H=4096, V=128256,
  // T=64: 227 -> 181.  Ranges in multiples of 64 rows did best or within 3% of the best in all of these.
  int64_t rows_per_split = 0;
  if (Cfg::BN <= 128 && nvt < 8 * S) {
    rows_per_split = round_up((V + S - 1) / S, 64);
    S = (int)((V + rows_per_split - 1) / rows_per_split);
  }
  FwdArgs<TIN> p;
  p.W = W; p.ldw = ldw; p.h = h; p.ldh = ldh; p.labels = labels; p.T = T; p.V = V; p.H = H;
  p.c = kLog2e / temperature;
  p.parts = reinterpret_cast<f32x4_t*>(ws);
  p.xlabel = reinterpret_cast<float*>(ws + align256((size_t)S * T * 16));
  p.S = S;
  p.split_stride = rows_per_split ? rows_per_split : Cfg::BM;
  p.tile_step = rows_per_split ? Cfg::BM : (int64_t)S * Cfg::BM;
  p.split_span = rows_per_split ? rows_per_split : V;
  p.label_offset = label_offset;
  // xcache: the raw logits are kept for the backward
  p.xcache = xcache; p.ldx = logits_cache_row(V);
  p.map = TileMap::make(ntt, S, br, 1);
  float* lp_tok = reduction == LCE_REDUCTION_NONE ? logprobs : reinterpret_cast<float*>(ws + align256((size_t)S * T * 16) + align256((size_t)T * 4));
  int rc;
  {
    ProfScope prof(PC_FWD, st);
    if constexpr (Cfg::CORE16) {
      if (xcache) {
        allow_lds((lce_fwd16_kernel<Cfg, true>), Cfg::LDS_BYTES);
        hipLaunchKernelGGL((lce_fwd16_kernel<Cfg, true>), dim3(p.map.total), dim3(Cfg::NTHREADS), Cfg::LDS_BYTES, st, p);
      } else {
        allow_lds((lce_fwd16_kernel<Cfg, false>), Cfg::LDS_BYTES);
        hipLaunchKernelGGL((lce_fwd16_kernel<Cfg, false>), dim3(p.map.total), dim3(Cfg::NTHREADS), Cfg::LDS_BYTES, st, p);
      }
    } else {
      allow_lds(lce_fwd_kernel<Cfg>, Cfg::LDS_BYTES);
      hipLaunchKernelGGL(lce_fwd_kernel<Cfg>, dim3(p.map.total), dim3(Cfg::NTHREADS), Cfg::LDS_BYTES, st, p);
    }
    rc = check_launch("lce_fwd_kernel");
  }
  if (rc) return rc;
  if (shard_out) {
    ProfScope prof(PC_FWD_MERGE, st);
    f32x4_t* out = reinterpret_cast<f32x4_t*>(shard_out);
    if (S >= 64)
      hipLaunchKernelGGL(lce_fwd_shard_merge_kernel<64>, dim3((unsigned)((T * 64 + 255) / 256)), dim3(256), 0, st, p.parts, p.xlabel, labels, label_offset, V, S,
                         T, p.c, 1.0f / temperature, out);
    else if (S >= 8)
      hipLaunchKernelGGL(lce_fwd_shard_merge_kernel<8>, dim3((unsigned)((T * 8 + 255) / 256)), dim3(256), 0, st, p.parts, p.xlabel, labels, label_offset, V, S, T,
                         p.c, 1.0f / temperature, out);
    else
      hipLaunchKernelGGL(lce_fwd_shard_merge_kernel<1>, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, st, p.parts, p.xlabel, labels, label_offset, V, S, T,
                         p.c, 1.0f / temperature, out);
    return check_launch("lce_fwd_shard_merge_kernel");
  }
  {
    ProfScope prof(PC_FWD_MERGE, st);
    if (S >= 64)
      hipLaunchKernelGGL(lce_fwd_merge_kernel<64>, dim3((unsigned)((T * 64 + 255) / 256)), dim3(256), 0, st, p.parts, p.xlabel, labels, label_offset, V, S, T,
                         p.c, 1.0f / temperature, lp_tok, entropy, maximum, accumulate, entropy_b);
    else if (S >= 8)
      hipLaunchKernelGGL(lce_fwd_merge_kernel<8>, dim3((unsigned)((T * 8 + 255) / 256)), dim3(256), 0, st, p.parts, p.xlabel, labels, label_offset, V, S, T,
                         p.c, 1.0f / temperature, lp_tok, entropy, maximum, accumulate, entropy_b);
    else
      hipLaunchKernelGGL(lce_fwd_merge_kernel<1>, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, st, p.parts, p.xlabel, labels, label_offset, V, S, T, p.c,
                         1.0f / temperature, lp_tok, entropy, maximum, accumulate, entropy_b);
    rc = check_launch("lce_fwd_merge_kernel");
  }
  if (rc) return rc;
  if (reduction != LCE_REDUCTION_NONE) {
    const float scale = reduction == LCE_REDUCTION_MEAN ? 1.0f / (float)T : 1.0f;
    hipLaunchKernelGGL(lce_reduce_sum_kernel, dim3(1), dim3(1024), 0, st, lp_tok, T, scale, logprobs);
    rc = check_launch("lce_reduce_sum_kernel");
  }
  return rc;
}

// upper bound of the number of vocabulary splits forward_impl picks, over the token-tile widths in use
int forward_splits_upper_bound(int64_t T, int64_t V, int max_splits = kMaxSplits) {
  int best = forward_splits_256((int)((T + 255) / 256), (int)((V + 255) / 256), max_splits);
  for (int bn = 64; bn <= 128; bn <<= 1) {
    const int ntt = (int)((T + bn - 1) / bn);
    const int br = block_rows(ntt), bc = 32 / br, nrb = (ntt + br - 1) / br;
    const int S = bc * ((8 + nrb - 1) / nrb);
    if (S > best) best = S;
  }
  return best < max_splits ? best : max_splits;
}

struct BwdLayout {
  int64_t vchunk, tpad, vpad, ldS, ldST, ldWt, ldHt;
  size_t off_dS[2], off_dST[2], off_Wt, off_Ht, off_dHacc, off_rows, off_inv, off_nrows, off_acounts, off_coef, off_keys[2], off_vals[2], off_hist, off_tokc, off_tokl, total;
  int sort_items, sort_passes;  // label sort (0 items: the one-hot part stays inside the d_logits tiles)
  int nchunks;
  int ksplit;  // K splits of the d_hidden GEMM (each with its own fp32 partial)
  bool tn;     // the gradient GEMMs read dS, a compact copy of hidden and W as they lie in memory (transposing LDS
               // reads for the K-major operands): no dS^T, no h^T
  bool tn_dh;  // ... and the d_hidden GEMM reads W as it lies in memory too: no W^T
  bool few;    // at most 128 tokens, 16-bit inputs: both gradient GEMMs run as the streaming kernels of few_tokens.hpp
};

// The d_weight GEMM takes the token-major d_logits and hidden as they are where transposing LDS reads exist (16-bit
// elements); for fp32 a vocab-major copy of the d_logits and a transposed hidden are built for it.
bool dw_transposed_reads(size_t esz) { return esz == 2; }

// The d_hidden GEMM has only ceil(T/256) * ceil(H/256) output tiles, each with a K loop as long as the
// vocabulary chunk.  With few tokens one such tile takes longer than a CU's share of the whole launch
// (d_logits tiles + both GEMMs) and would set the launch's duration; the K range is then cut into
// slices, with an fp32 partial each, so that a tile takes at most about half of that share.
int64_t few_tile_columns(int64_t T) { return T <= 64 ? FewShape<64>::HW : FewShape<128>::HW; }

int dh_ksplit(int64_t T, int64_t H, int64_t vchunk) {
  const int64_t ntt = (T + 255) / 256, nht = (H + 255) / 256, nvt = (vchunk + 255) / 256;
  const int64_t work = ntt * nvt * H + nvt * nht * ntt * 256 + ntt * nht * vchunk;  // in K elements of 256x256 tiles
  const int64_t share = work / 256 / 2;
  const int64_t s = share > 0 ? (vchunk + share - 1) / share : 16;
  return (int)(s < 1 ? 1 : s > 16 ? 16 : s);
}

// layout for a given chunk width
BwdLayout bwd_layout_for(const Tuning& tu, int64_t T, int64_t H, int64_t V, size_t esz, int64_t vchunk, int64_t gt, int64_t gv) {
  BwdLayout L;
  const int variant = bwd_variant(tu, T, esz);
  L.tn = dw_transposed_reads(esz);
  // Measured: reading W through the transposing LDS reads costs the d_hidden GEMM about 2% of its rate, and
  // saves one transpose of W per call.  The transpose is the larger cost up to some thousands of tokens
  // (T=64: 1.95 -> 1.43 ms per forward + backward, T=4096: 15.7 -> 14.7 ms at H=3584, V=152064), the GEMM
  // rate beyond that (T=16384: +0.5 ms).
  // (on the 16x16x32 loop the transposing reads of one operand cost under 1 %: W is always read in place there)
  L.tn_dh = L.tn && (variant == kVariantCore16 || T <= 8192);
  vchunk = round_up(vchunk, 256);
  if (vchunk > round_up(V, 256)) vchunk = round_up(V, 256);
  L.vchunk = vchunk;
  L.ksplit = tu.dh_ksplit > 0 ? tu.dh_ksplit : dh_ksplit(T, H, vchunk);
  L.few = tu.few_token_gemms && L.tn && T <= 128;
  if (L.few) {
    // K slices of the streaming d_hidden kernel: its workgroups (column tiles x slices) fill the chip about twice
    // over, which is what two resident workgroups per CU take in one round; at least 1024 columns per slice
    const int64_t n_ht = (H + few_tile_columns(T) - 1) / few_tile_columns(T);
    int64_t ks = (2 * kNumCUs) / n_ht;
    const int64_t most = (vchunk + 1023) / 1024;
    ks = ks > most ? most : ks;
    L.ksplit = tu.dh_ksplit > 0 ? tu.dh_ksplit : (int)(ks < 1 ? 1 : ks > 40 ? 40 : ks);
    L.tn_dh = true;  // W is read in place
  }
  L.nchunks = (int)((V + vchunk - 1) / vchunk);
  // Row strides are kept away from large powers of two (+128 bytes): with a 16 or 32 KiB stride the
  // 256 rows of an operand tile would all fall into the same L2 channel.
  // tokens / vocabulary rounded up to the K-permutation groups (gt, gv: at most one workgroup tile,
  // which is what the size query assumes; the launch passes the tile variant's wave-tile sizes)
  L.tpad = round_up(T, gt);
  L.vpad = round_up(V, gv);
  L.ldS = vchunk + 64;
  L.ldST = L.tpad + 64;
  L.ldWt = vchunk + 64;  // one chunk of W^T at a time
  L.ldHt = L.tn ? round_up(H, 256) + 64 : L.tpad + 64;  // tn: row stride of the compact copy of hidden [tpad][.]
  size_t o = 0;
  // the d_logits pair is double buffered when there is more than one chunk: chunk c is produced
  // while the GEMMs of chunk c-1 consume the other pair
  for (int b = 0; b < 2; ++b) {
    L.off_dS[b] = o;
    if (b == 0 || L.nchunks > 1) o += align256((size_t)L.tpad * L.ldS * esz);
    L.off_dST[b] = o;
    if (!L.tn && (b == 0 || L.nchunks > 1)) o += align256((size_t)vchunk * L.ldST * esz);
  }
  L.off_Wt = o;    o += L.tn_dh ? 0 : align256((size_t)H * L.ldWt * esz);
  L.off_Ht = o;    o += L.tn ? align256((size_t)L.tpad * L.ldHt * esz) : align256((size_t)H * L.ldHt * esz);
  L.off_dHacc = o; o += (size_t)L.ksplit * align256((size_t)T * H * 4);
  // list of the tokens with a non-zero upstream gradient, its inverse, and its length
  L.off_rows = o;  o += align256((size_t)L.tpad * 4);
  L.off_inv = o;   o += align256((size_t)T * 4);
  L.off_nrows = o; o += 256;
  L.off_acounts = o; o += align256((size_t)((T + kActiveBlock - 1) / kActiveBlock) * 4);  // per-block counts of the token list
  // (label row, token) pairs, two buffers each, and the per-block digit counts of one radix pass
  L.sort_items = (esz == 2 && tu.label_outside && T <= ((int64_t)1 << 30)) ? (int)round_up(T, kSortBlock) : 0;
  int vbits = 1;
  while (vbits < 32 && ((int64_t)1 << vbits) < V) ++vbits;
  L.sort_passes = (vbits + 1 + 7) / 8;
  for (int b = 0; b < 2; ++b) {
    L.off_keys[b] = o; o += align256((size_t)L.sort_items * 4);
    L.off_vals[b] = o; o += align256((size_t)L.sort_items * 4);
  }
  L.off_hist = o;  o += align256((size_t)(L.sort_items / kSortBlock) * 256 * 4);
  // per-token coefficient of the label's entry of d_logits, when the whole entry is kept out of the tiles
  L.off_coef = o;  o += (L.sort_items && tu.label_outside == 2) ? align256((size_t)T * 4) : 0;
  // per-position constants of the d_logits tiles (16-bit inputs): 16 + 4 bytes per position
  L.off_tokc = o;  o += esz == 2 ? align256((size_t)L.tpad * 16) : 0;
  L.off_tokl = o;  o += esz == 2 ? align256((size_t)L.tpad * 4) : 0;
  L.total = o;
  return L;
}

// vchunk <= 0 picks the default chunk width: as wide as possible (fewer, longer launches; the whole vocabulary
// in one chunk where that fits, which it does up to about 8192 tokens) while the whole workspace stays below a
// quarter of one [T, V] tile plus one fp32 [V, H],
//   (2 or 4)*T*vc*esz + esz*vc*H + (esz + 4*ksplit)*T*H (+ padding)  <=  0.25*T*V*esz + 4*V*H,
// then evened out over the number of chunks that width needs.
// gt, gv: K-permutation groups that tokens / vocabulary are rounded up to (at most one workgroup
// tile, which is what the size query assumes; the launch passes the tile variant's wave-tile sizes).
BwdLayout bwd_layout(const Tuning& tu, int64_t T, int64_t H, int64_t V, size_t esz, int64_t vchunk, int64_t gt = 256, int64_t gv = 256) {
  if (vchunk <= 0) {
    // Upper bound of the whole workspace: a quarter of one [T, V] tile plus one fp32 [V, H].  Below it the default is
    // a chunk of 16384 columns, wider while one d_logits buffer stays within 256 MiB (few tokens: the whole vocabulary
    // in one chunk, which saves a pass over W per chunk), narrower once two such buffers would pass 4 GiB.  Measured on
    // one box, three interleaved runs each: T=16384, H=3584, V=152064: 8192 columns 54.80 ms per step, 16384 columns
    // 54.27, 24576 columns 54.26 (each halving of the chunk count halves the fp32 read-modify-write passes over d_hidden
    // and the launch boundaries; 0.15 ms on another box); T=32768, H=4096, V=128256: 66.67 against 65.97; 4096 columns
    // cost 6 %; up to 8192 tokens the width makes no difference from 16384 columns on.  T=65536, H=5120, V=152064, where a
    // buffer of 16384 columns takes 2 GiB: 229.1 ms for the backward's launches with 8192 columns, 234.7 with 15360.  A byte budget (LCE_OPT_WORKSPACE_BUDGET) replaces the default
    // rule: the widest chunk whose workspace fits it, but never fewer than 2048 columns.
    double gate = 0.25 * (double)T * V * esz + 4.0 * (double)V * H;
    vchunk = round_up(V, 256);
    if (tu.ws_budget > 0) {
      if ((double)tu.ws_budget < gate) gate = (double)tu.ws_budget;
    } else {
      int64_t cols = (((int64_t)256 << 20) / (T * (int64_t)esz)) / 256 * 256;
      if (cols < 16384) {
        // many tokens: 16384 columns while one d_logits buffer stays within 1 GiB, never fewer than 8192
        cols = (((int64_t)1 << 30) / (T * (int64_t)esz)) / 256 * 256;
        cols = cols > 16384 ? 16384 : cols < 8192 ? 8192 : cols;
      }
      // very many tokens: the two d_logits buffers stay within 4 GiB (at 262144 tokens chunks of 4096 columns take as
      // long as chunks of 8192, 567.1 against 567.2 ms per actor step, with 10.1 instead of 14.1 GiB of workspace: a
      // launch is long enough there for its fixed costs not to show)
      const int64_t cap = (((int64_t)2 << 30) / (T * (int64_t)esz)) / 256 * 256;
      if (cols > cap) cols = cap < 2048 ? 2048 : cap;
      if (cols < vchunk) vchunk = cols;
    }
    while (vchunk > 2048 && (double)bwd_layout_for(tu, T, H, V, esz, vchunk, 256, 256).total + 512.0 > gate) vchunk -= 1024;
    if (vchunk < 2048) vchunk = 2048;
    const int64_t n = (V + vchunk - 1) / vchunk;
    vchunk = round_up((V + n - 1) / n, 256);
  }
  return bwd_layout_for(tu, T, H, V, esz, vchunk, gt, gv);
}

// The d_logits tiles of a backward with few tokens stream W once, like the forward with few tokens, and gain from
// the same narrow token tiles with a deeper ring.  SmallCfg must permute the vocabulary inside a wave tile as Cfg
// does (same WM), because the gradient GEMMs that read dS run with Cfg.
template <typename SmallCfg, typename Cfg>
int launch_ds_few_tokens(DsArgs<typename Cfg::TIN> d, int64_t T, int nvt, hipStream_t st) {
  static_assert(SmallCfg::WM == Cfg::WM && SmallCfg::FM == Cfg::FM && SmallCfg::BM == Cfg::BM, "same vocabulary order in dS");
  const int ntt = (int)((T + SmallCfg::BN - 1) / SmallCfg::BN);
  d.map = TileMap::make(ntt, nvt, block_rows(ntt), 0);
  unsigned grid = (unsigned)d.map.total;
  if (ntt == 1) {
    // one contiguous range of rows per workgroup, the same length for all and at most one workgroup per CU (measured
    // on the kernel, 64 tokens, H=3584, V=152064: 594 tiles on 256 CUs, 3 against 2, took 215 us)
    const int64_t pad_end = round_up(d.vrows, SmallCfg::WM);
    d.range_rows = round_up((pad_end + kNumCUs - 1) / kNumCUs, SmallCfg::WM);
    grid = (unsigned)((pad_end + d.range_rows - 1) / d.range_rows);
  }
  allow_lds(lce_bwd_ds_kernel<SmallCfg>, SmallCfg::LDS_BYTES);
  hipLaunchKernelGGL(lce_bwd_ds_kernel<SmallCfg>, dim3(grid), dim3(SmallCfg::NTHREADS), SmallCfg::LDS_BYTES, st, d);
  return check_launch("lce_bwd_ds_kernel");
}

// Both gradient GEMMs of one vocabulary chunk of a backward with at most 128 tokens, as one launch of the streaming
// kernels (few_tokens.hpp): d_weight rows of the chunk in the output dtype, d_hidden as L.ksplit fp32 partials.
template <typename Cfg, typename TOUT, int KT>
int launch_few_gemms(const FewArgs<typename Cfg::TIN>& q, bool with_dh, hipStream_t st) {
  typedef typename Cfg::TIN TIN;
  typedef FewShape<KT> S;
  const int n_ht = (int)((q.H + S::HW - 1) / S::HW);
  auto kern = lce_bwd_few_kernel<TIN, TOUT, KPerm<Cfg>, KT>;
  allow_lds(kern, S::LDS_BYTES);
  // (q.n_dw = 0: no d_weight workgroups; without d_hidden the grid ends after them)
  hipLaunchKernelGGL(kern, dim3((unsigned)(q.n_dw + (with_dh ? n_ht * q.ksplit : 0))), dim3(256), S::LDS_BYTES, st, q);
  return check_launch("lce_bwd_few_kernel");
}

template <typename Cfg>
int backward_impl(const typename Cfg::TIN* h, int64_t ldh, const typename Cfg::TIN* W, int64_t ldw, const int64_t* labels,
                  int64_t T, int64_t H, int64_t V, float temperature, int reduction, const float* maximum,
                  const float* accumulate, const float* entropy_b, const float* dlogprobs, const float* dentropy,
                  void* d_hidden, void* d_weight, bool grads_f32, char* ws, int64_t vchunk, hipStream_t st,
                  int64_t vocab_offset, const Tuning& tu, const float* xcache = nullptr) {
  // vocab_offset: W is the shard [vocab_offset, vocab_offset + V) of a larger vocabulary (labels are global ids)
  // d_hidden or d_weight may be null (not both): that gradient is not wanted (a frozen lm-head, an input without
  // gradient) and its GEMM, a third of the backward's work, is left out
  typedef typename Cfg::TIN TIN;
  const bool need_dh = d_hidden != nullptr, need_dw = d_weight != nullptr;
  const BwdLayout L = bwd_layout(tu, T, H, V, sizeof(TIN), vchunk, KPerm<Cfg>::GT, KPerm<Cfg>::GV);
  TIN* dS[2] = {reinterpret_cast<TIN*>(ws + L.off_dS[0]), reinterpret_cast<TIN*>(ws + L.off_dS[1])};
  TIN* dST[2] = {reinterpret_cast<TIN*>(ws + L.off_dST[0]), reinterpret_cast<TIN*>(ws + L.off_dST[1])};
  TIN* Wt = reinterpret_cast<TIN*>(ws + L.off_Wt);
  TIN* Ht = reinterpret_cast<TIN*>(ws + L.off_Ht);
  float* dHacc = reinterpret_cast<float*>(ws + L.off_dHacc);
  int rc;
  // Tokens with zero upstream gradients (prompt and padding positions of a PPO batch) add nothing to
  // either gradient: list the others on the device and run everything below on that list.  Nothing
  // comes back to the host, so grids are sized for all T tokens and surplus workgroups exit at once.
  // (The gather addresses rows of `hidden` with 32-bit byte offsets; larger inputs run uncompacted.)
  const bool compact = (uint64_t)T * (uint64_t)ldh * sizeof(TIN) < (1ull << 32);
  int* rows = compact ? reinterpret_cast<int*>(ws + L.off_rows) : nullptr;
  int* inv = compact ? reinterpret_cast<int*>(ws + L.off_inv) : nullptr;
  int* n_rows = compact ? reinterpret_cast<int*>(ws + L.off_nrows) : nullptr;
  // tokens grouped by label for the one-hot part of d_weight (added after the GEMMs)
  LabelTerm lt;
  lt.labels = nullptr; lt.v0 = vocab_offset; lt.V = V; lt.g_lp = dlogprobs;
  lt.g_stride = reduction == LCE_REDUCTION_NONE ? 1 : 0;
  lt.scale = (reduction == LCE_REDUCTION_MEAN ? 1.0f / (float)T : 1.0f) / temperature;
  uint32_t* skeys[2] = {reinterpret_cast<uint32_t*>(ws + L.off_keys[0]), reinterpret_cast<uint32_t*>(ws + L.off_keys[1])};
  int* svals[2] = {reinterpret_cast<int*>(ws + L.off_vals[0]), reinterpret_cast<int*>(ws + L.off_vals[1])};
  CoefArgs<TIN> ca;
  ca.h = h; ca.ldh = ldh; ca.W = W; ca.ldw = ldw; ca.labels = labels; ca.v0 = vocab_offset; ca.V = V; ca.ntok = T; ca.H = H;
  ca.maximum = maximum; ca.accumulate = accumulate; ca.entropy_b = entropy_b; ca.g_lp = dlogprobs; ca.g_stride = lt.g_stride;
  ca.g_scale = reduction == LCE_REDUCTION_MEAN ? 1.0f / (float)T : 1.0f; ca.g_ent = dentropy; ca.rcp_tau = 1.0f / temperature;
  ca.c = kLog2e / temperature;
  const bool with_coef = sizeof(TIN) == 2 && L.sort_items && tu.label_outside == 2;
  ca.coef = with_coef ? reinterpret_cast<float*>(ws + L.off_coef) : nullptr;
  if (L.sort_items) lt.labels = labels;
  if (with_coef) { lt.g_lp = ca.coef; lt.g_stride = 1; lt.scale = 1.0f; }
  // few tokens: the token list, the label coefficients and the compact copy of hidden come from one launch, and the
  // one-hot rows of d_weight need no sorted list (few_finish_kernel at the end)
  const bool few_prep = L.few && compact;
  if (few_prep) {
    if constexpr (sizeof(TIN) == 2) {
      ProfScope prof(PC_ACTIVE_ROWS, st);
      const int64_t r64 = round_up(T, 64);
      hipLaunchKernelGGL(few_prep_kernel<TIN>, dim3((unsigned)(r64 < L.tpad ? r64 : L.tpad)), dim3(256), 0, st, ca, Ht, L.ldHt, L.tpad, rows,
                         inv, n_rows);
      if ((rc = check_launch("few_prep_kernel"))) return rc;
    }
  } else if (compact) {
    ProfScope prof(PC_ACTIVE_ROWS, st);
    int* acounts = reinterpret_cast<int*>(ws + L.off_acounts);
    const unsigned nblk = (unsigned)((T + kActiveBlock - 1) / kActiveBlock);
    hipLaunchKernelGGL(active_count_kernel, dim3(nblk), dim3(256), 0, st, dlogprobs, ca.g_stride, dentropy, T, acounts);
    if ((rc = check_launch("active_count_kernel"))) return rc;
    hipLaunchKernelGGL(active_rows_kernel, dim3(nblk), dim3(256), 0, st, dlogprobs, ca.g_stride, dentropy, T, acounts, rows, inv, n_rows);
    if ((rc = check_launch("active_rows_kernel"))) return rc;
  }
  if (L.sort_items && !few_prep) {
    ProfScope prof(PC_LABEL_ROWS, st);
    if constexpr (sizeof(TIN) == 2) if (with_coef) {
      hipLaunchKernelGGL(label_coef_kernel<TIN>, dim3((unsigned)((T + 3) / 4)), dim3(256), 0, st, ca);
      if ((rc = check_launch("label_coef_kernel"))) return rc;
    }
    const int nblocks = L.sort_items / kSortBlock;
    if (!need_dw) {
      // (the tokens grouped by label serve the one-hot rows of d_weight only)
    } else if (nblocks == 1) {
      hipLaunchKernelGGL(label_sort_single_kernel, dim3(1), dim3(256), 0, st, lt, rows, n_rows, T, L.sort_passes, skeys[0], svals[0],
                         skeys[1], svals[1]);
      if ((rc = check_launch("label_sort_single_kernel"))) return rc;
    } else {
      int* hist = reinterpret_cast<int*>(ws + L.off_hist);
      hipLaunchKernelGGL(label_keys_kernel, dim3(L.sort_items / 256), dim3(256), 0, st, lt, rows, n_rows, T, L.sort_items, skeys[0], svals[0]);
      if ((rc = check_launch("label_keys_kernel"))) return rc;
      for (int ps = 0; ps < L.sort_passes; ++ps) {
        const int in = ps & 1, out = in ^ 1;
        hipLaunchKernelGGL(sort_hist_kernel, dim3(nblocks), dim3(256), 0, st, skeys[in], 8 * ps, nblocks, hist);
        hipLaunchKernelGGL(sort_scan_kernel, dim3(1), dim3(1024), 0, st, hist, 256 * nblocks);
        hipLaunchKernelGGL(sort_scatter_kernel, dim3(nblocks), dim3(256), 0, st, skeys[in], svals[in], skeys[out], svals[out], 8 * ps,
                           nblocks, hist);
        if ((rc = check_launch("label sort pass"))) return rc;
      }
    }
  }
  f32x4_t* tokc = nullptr;
  int* tokl = nullptr;
  if constexpr (Cfg::CORE16) {
    tokc = reinterpret_cast<f32x4_t*>(ws + L.off_tokc);
    tokl = reinterpret_cast<int*>(ws + L.off_tokl);
    ProfScope prof(PC_ACTIVE_ROWS, st);
    hipLaunchKernelGGL(ds_token_consts_kernel, dim3((unsigned)((L.tpad + 255) / 256)), dim3(256), 0, st, rows, n_rows, T, L.tpad, dlogprobs,
                       (int64_t)(reduction == LCE_REDUCTION_NONE ? 1 : 0), reduction == LCE_REDUCTION_MEAN ? 1.0f / (float)T : 1.0f,
                       dentropy, maximum, accumulate, entropy_b, labels, vocab_offset, V, 1.0f / temperature, tokc, tokl);
    if ((rc = check_launch("ds_token_consts_kernel"))) return rc;
  }
  // second operand of the d_weight GEMM (W^T for d_hidden follows chunk by chunk): the listed rows of hidden,
  // as they are (K-major, for the transposing reads), or transposed to h^T [H][T]
  if (few_prep) {
    // (few_prep_kernel has written the compact copy)
  } else if (L.tn) {
    ProfScope prof(PC_TRANSPOSE, st);
    hipLaunchKernelGGL(gather_rows_kernel<TIN>, dim3(2048), dim3(256), 0, st, h, ldh, T, H, Ht, L.ldHt, L.tpad, rows, n_rows);
    if ((rc = check_launch("gather_rows_kernel"))) return rc;
  } else {
    ProfScope prof(PC_TRANSPOSE, st);
    hipLaunchKernelGGL((transpose_pad_kernel<Cfg, 1>), dim3((unsigned)((L.tpad + 127) / 128), (unsigned)((H + 63) / 64)), dim3(256), 0,
                       st, h, ldh, T, H, Ht, L.ldHt, L.tpad, rows, n_rows);
    if ((rc = check_launch("transpose h"))) return rc;
  }

  const int ntt = (int)((T + Cfg::BN - 1) / Cfg::BN);
  // (the K-major d_weight tiles use the 160 KB split ring whatever ring the variant itself uses)
  const int chunk_lds = L.tn && Cfg::LDS_BYTES < 160 * 1024 ? 160 * 1024 : Cfg::LDS_BYTES;
  auto launch_chunk = [&](const BwdChunkArgs<TIN>& q) {
    if constexpr (Cfg::CORE16) {
      allow_lds(lce_bwd_chunk16_kernel<Cfg>, chunk_lds);
      hipLaunchKernelGGL(lce_bwd_chunk16_kernel<Cfg>, dim3(q.n_gw + q.n_gh + q.n_ds), dim3(Cfg::NTHREADS), chunk_lds, st, q);
    } else {
      allow_lds(lce_bwd_chunk_kernel<Cfg>, chunk_lds);
      hipLaunchKernelGGL(lce_bwd_chunk_kernel<Cfg>, dim3(q.n_gw + q.n_gh + q.n_ds), dim3(Cfg::NTHREADS), chunk_lds, st, q);
    }
  };
  // launch c (0 <= c <= nchunks): d_logits of chunk c (if any) + the two gradient GEMMs of chunk c-1 (if any)
  for (int c = 0; c <= L.nchunks; ++c) {
    BwdChunkArgs<TIN> p;
    p.n_gw = p.n_gh = p.n_ds = 0;
    bool swapped = false;
    if (c < L.nchunks) {
      const int64_t v0 = (int64_t)c * L.vchunk;
      const int64_t vrows = (V - v0) < L.vchunk ? (V - v0) : L.vchunk;
      DsArgs<TIN>& d = p.ds;
      d.W = W + v0 * ldw; d.ldw = ldw; d.h = h; d.ldh = ldh; d.labels = labels; d.T = T; d.H = H;
      d.v0 = vocab_offset + v0; d.vrows = vrows; d.rcp_tau = 1.0f / temperature; d.c = kLog2e / temperature;
      d.maximum = maximum; d.accumulate = accumulate; d.entropy_b = entropy_b;
      d.g_lp = dlogprobs; d.g_lp_stride = reduction == LCE_REDUCTION_NONE ? 1 : 0;
      d.g_lp_scale = reduction == LCE_REDUCTION_MEAN ? 1.0f / (float)T : 1.0f;
      d.g_ent = dentropy;
      d.dS = dS[c & 1]; d.ldS = L.ldS; d.dST = L.tn ? nullptr : dST[c & 1]; d.ldST = L.ldST; d.tpad = L.tpad;
      d.rows = rows; d.n_rows = n_rows;
      d.label_outside = lt.labels != nullptr ? tu.label_outside : 0;
      d.tokc = tokc; d.tokl = tokl; d.lab0 = v0;
      d.range_rows = 0;
      if (Cfg::CORE16 && L.tn) {
        // the compact copy of hidden built for the d_weight GEMM: the tiles read it without a row gather
        d.h = Ht; d.ldh = L.ldHt; d.rows = nullptr;
      }
      const int nvt = (int)((vrows + Cfg::BM - 1) / Cfg::BM);
      // Order in which an XCD's consecutive blocks walk the chunk.  Measured: along the vocabulary is 2-3%
      // faster on the launch while `hidden` is small enough to stay in the memory-side cache next to the
      // chunk's other operands (T=16384, H=3584: 117 MB), along the tokens is 2% faster beyond that
      // (T=32768, H=4096 and T=65536, H=5120).
      const int tokens_first = tu.ds_tokens_first >= 0 ? tu.ds_tokens_first : ((size_t)T * H * sizeof(TIN) > ((size_t)128 << 20));
      d.map = TileMap::make(ntt, nvt, block_rows(ntt), tokens_first);
      p.n_ds = d.map.total;
    }
    if (c > 0) {
      const int cc = c - 1;
      const int64_t v0 = (int64_t)cc * L.vchunk;
      const int64_t vrows = (V - v0) < L.vchunk ? (V - v0) : L.vchunk;
      // fp32 d_hidden partial [T][H] (+)= dS[T][Kc] . W[v0 : v0 + Kc][H]  (rows = listed tokens)
      const int64_t kc = round_up(vrows, KPerm<Cfg>::GV);
      bool few_done = false;  // (then nothing is left for the tile kernels but the d_logits of the next chunk)
      if constexpr (sizeof(TIN) == 2) {
        if (L.few) {
          FewArgs<TIN> q;
          q.dS = dS[cc & 1]; q.ldS = L.ldS; q.Ht = Ht; q.ldHt = L.ldHt; q.W = W + v0 * ldw; q.ldw = ldw;
          q.vrows = vrows; q.ucols = kc; q.H = H;
          q.kt = T <= 64 ? 64 : 128; q.nt = (int)T; q.n_rows = n_rows;
          q.dW = !need_dw ? nullptr
                 : grads_f32 ? static_cast<void*>(static_cast<float*>(d_weight) + v0 * H) : static_cast<void*>(static_cast<TIN*>(d_weight) + v0 * H);
          q.dHp = dHacc; q.part_stride = (int64_t)(align256((size_t)T * H * 4) / 4);
          q.ksplit = L.ksplit; q.kslice = round_up((q.ucols + L.ksplit - 1) / L.ksplit, 64);
          q.accumulate = cc == 0 ? 0 : 1;
          q.n_dw = need_dw ? (int)(q.ucols / 64) : 0;
          ProfScope prof(PC_BWD_CHUNK, st);
          if (T <= 64) rc = grads_f32 ? launch_few_gemms<Cfg, float, 64>(q, need_dh, st) : launch_few_gemms<Cfg, TIN, 64>(q, need_dh, st);
          else rc = grads_f32 ? launch_few_gemms<Cfg, float, 128>(q, need_dh, st) : launch_few_gemms<Cfg, TIN, 128>(q, need_dh, st);
          if (rc) return rc;
          few_done = true;
        }
      }
      if (!few_done) {
        if (!need_dh) {
          // (no d_hidden GEMM)
        } else if (L.tn_dh) {
          // W as it lies in memory (K-major for this product), fetched with transposing LDS reads
          p.gh = make_gemm_args<Cfg>(dS[cc & 1], L.ldS, W + v0 * ldw, ldw, T, H, kc, dHacc, H, nullptr, 0, cc == 0 ? 0 : 1);
          p.gh.tn = 2;
          p.gh.b_rows_valid = vrows;
        } else {
          // Wt = this chunk of W, transposed just before the launch (the previous launch, the last reader of the
          // buffer, is complete by then)
          ProfScope prof(PC_TRANSPOSE, st);
          hipLaunchKernelGGL((transpose_pad_kernel<Cfg, 2>), dim3((unsigned)((kc + 127) / 128), (unsigned)((H + 63) / 64)), dim3(256), 0,
                             st, W + v0 * ldw, ldw, vrows, H, Wt, L.ldWt, kc);
          if ((rc = check_launch("transpose W"))) return rc;
          p.gh = make_gemm_args<Cfg>(dS[cc & 1], L.ldS, Wt, L.ldWt, T, H, kc, dHacc, H, nullptr, 0, cc == 0 ? 0 : 1);
        }
        if (need_dh) p.gh.m_dev = n_rows;
        if (need_dh && L.ksplit > 1) {
          p.gh.ksplit = L.ksplit;
          p.gh.kslice = round_up((kc + L.ksplit - 1) / L.ksplit, Cfg::BK);
          p.gh.cf_split_stride = (int64_t)(align256((size_t)T * H * 4) / 4);
        }
        // d_weight[v0 : v0 + vrows][H] = dST[vrows][Tpad] . Ht[H][Tpad]^T   (written in the input dtype, or as fp32)
        float* dw_f32 = need_dw && grads_f32 ? static_cast<float*>(d_weight) + v0 * H : nullptr;
        TIN* dw_t = need_dw && !grads_f32 ? static_cast<TIN*>(d_weight) + v0 * H : nullptr;
        if (!need_dw) {
          // (no d_weight GEMM)
        } else if (L.tn) {
          // d_weight[v0 : v0 + vrows][H] = dS[tokens][vrows]^T . hidden[tokens][H], both operands K-major
          p.gw = make_gemm_args<Cfg>(dS[cc & 1], L.ldS, Ht, L.ldHt, vrows, H, round_up(T, 64), dw_f32, H, dw_t, H, grads_f32 ? 0 : 2);
          p.gw.tn = 1;
          p.gw.perm_rows = 1;
          p.gw.k_dev = n_rows; p.gw.k_gran = 64;
        } else {
          p.gw = make_gemm_args<Cfg>(dST[cc & 1], L.ldST, Ht, L.ldHt, vrows, H, L.tpad, dw_f32, H, dw_t, H, grads_f32 ? 0 : 2);
          p.gw.k_dev = n_rows; p.gw.k_gran = KPerm<Cfg>::GT;
        }
        p.n_gh = need_dh ? p.gh.map.total * L.ksplit : 0;
        p.n_gw = need_dw ? p.gw.map.total : 0;
        if (need_dh && need_dw && p.gh.kslice > p.gw.K) {  // longer tiles go first
          std::swap(p.gh, p.gw);
          std::swap(p.n_gh, p.n_gw);
          swapped = true;
        } else if (!need_dw) {  // an only GEMM sits in the first slot
          p.gw = p.gh;
          p.n_gw = p.n_gh;
          p.n_gh = 0;
          swapped = true;
        }
      }
    }
    if (p.n_gw + p.n_gh + p.n_ds == 0) continue;
    if (tu.split_bwd) {
      const int n[3] = {p.n_gw, p.n_gh, p.n_ds};
      const int cls[3] = {swapped ? PC_GEMM_DH : PC_GEMM_DW, swapped ? PC_GEMM_DW : PC_GEMM_DH, PC_BWD_DS};
      for (int k = 0; k < 3; ++k) {
        if (n[k] == 0) continue;
        BwdChunkArgs<TIN> q = p;
        if (k == 1) q.gw = p.gh;  // sub-problem k is moved to the front slot of a single-problem launch
        if (k == 2) { q.n_gw = 0; q.n_gh = 0; } else { q.n_gw = n[k]; q.n_gh = 0; q.n_ds = 0; }
        ProfScope prof(cls[k], st);
        launch_chunk(q);
        if ((rc = check_launch("lce_bwd_chunk_kernel(split)"))) return rc;
      }
      continue;
    }
    if constexpr (sizeof(TIN) == 2 && Cfg::BM == 256) {
      if (xcache && L.tn && p.n_ds > 0) {
        // d_logits of this chunk from the logits the forward kept: no pass over W, no T x V x H product
        const int64_t ldx = logits_cache_row(V);
        const int nrows = L.few ? ((int)(T <= 64 ? 64 : 128) < (int)L.tpad ? (int)(T <= 64 ? 64 : 128) : (int)L.tpad) : (int)L.tpad;
        const int64_t c0 = p.ds.v0 - vocab_offset;  // the chunk's first row of W
        {
          ProfScope prof(PC_BWD_DS, st);
          DsArgs<TIN> dq = p.ds;
          dq.rows = rows;  // (the 16x16x32 tiles read the compact copy of hidden and no list; the cache is indexed by token)
          hipLaunchKernelGGL((ds_from_logits_kernel<TIN, KPerm<Cfg>>), dim3((unsigned)(round_up(p.ds.vrows, 256) / 64)), dim3(256), 0, st, dq,
                             xcache + c0, ldx, nrows);
          if ((rc = check_launch("ds_from_logits_kernel"))) return rc;
        }
        p.n_ds = 0;  // (what is left for the launch below: the gradient GEMMs of the previous chunk)
        if (p.n_gw + p.n_gh == 0) continue;
      }
    }
    ProfScope prof(PC_BWD_CHUNK, st);
    if constexpr (sizeof(TIN) == 2 && Cfg::BM == 256 && Cfg::WAVES_M == 4) {
      if (p.n_gw + p.n_gh == 0 && L.tn && T <= 128) {  // the first launch: d_logits tiles only
        const int nvt = (int)((p.ds.vrows + Cfg::BM - 1) / Cfg::BM);
        rc = T <= 64 ? launch_ds_few_tokens<typename VariantT64<TIN>::Cfg, Cfg>(p.ds, T, nvt, st)
                     : launch_ds_few_tokens<typename VariantT128<TIN>::Cfg, Cfg>(p.ds, T, nvt, st);
        if (rc) return rc;
        continue;
      }
    }
    launch_chunk(p);
    if ((rc = check_launch("lce_bwd_chunk_kernel"))) return rc;
  }
  if (few_prep) {
    // d_hidden and the one-hot rows of d_weight (every row holds its softmax terms by now), one launch
    if constexpr (sizeof(TIN) == 2) {
      ProfScope prof(PC_DH_FINISH, st);
      const int n_dh = need_dh ? (int)((T * (H / 4) + 255) / 256) : 0;
      const int n_lr = (L.sort_items && need_dw) ? (int)T : 0;
      const int64_t part_stride = (int64_t)(align256((size_t)T * H * 4) / 4);
      if (n_dh + n_lr > 0) {
        if (grads_f32)
          hipLaunchKernelGGL((few_finish_kernel<TIN, float>), dim3((unsigned)(n_dh + n_lr)), dim3(256), 0, st, dHacc, L.ksplit, part_stride, inv,
                             T, H, static_cast<float*>(d_hidden), lt, W, ldw, n_dh, rows, n_rows, h, ldh, static_cast<float*>(d_weight));
        else
          hipLaunchKernelGGL((few_finish_kernel<TIN, TIN>), dim3((unsigned)(n_dh + n_lr)), dim3(256), 0, st, dHacc, L.ksplit, part_stride, inv,
                             T, H, static_cast<TIN*>(d_hidden), lt, W, ldw, n_dh, rows, n_rows, h, ldh, static_cast<TIN*>(d_weight));
        if ((rc = check_launch("few_finish_kernel"))) return rc;
      }
    }
    return LCE_OK;
  }
  if (need_dh) {
    // d_hidden = ordered sum of the fp32 partials, rounded once; zero rows for tokens without gradient
    ProfScope prof(PC_DH_FINISH, st);
    int64_t blocks = (T * (H / 4) + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    const int64_t part_stride = (int64_t)(align256((size_t)T * H * 4) / 4);
    if (grads_f32)
      hipLaunchKernelGGL((dh_finish_kernel<TIN, float>), dim3((unsigned)blocks), dim3(256), 0, st, dHacc, L.ksplit, part_stride, inv, T, H,
                         static_cast<float*>(d_hidden), lt, W, ldw);
    else
      hipLaunchKernelGGL((dh_finish_kernel<TIN, TIN>), dim3((unsigned)blocks), dim3(256), 0, st, dHacc, L.ksplit, part_stride, inv, T, H,
                         static_cast<TIN*>(d_hidden), lt, W, ldw);
    if ((rc = check_launch("dh_finish_kernel"))) return rc;
  }
  if (L.sort_items && need_dw) {
    // one-hot part of d_weight: every chunk's rows hold their softmax terms by now
    ProfScope prof(PC_LABEL_ROWS, st);
    const int res = L.sort_passes & 1;
    if (grads_f32)
      hipLaunchKernelGGL((dw_label_rows_kernel<TIN, float>), dim3(L.sort_items), dim3(256), 0, st, skeys[res], svals[res], L.sort_items, lt, h,
                         ldh, H, static_cast<float*>(d_weight));
    else
      hipLaunchKernelGGL((dw_label_rows_kernel<TIN, TIN>), dim3(L.sort_items), dim3(256), 0, st, skeys[res], svals[res], L.sort_items, lt, h,
                         ldh, H, static_cast<TIN*>(d_weight));
    if ((rc = check_launch("dw_label_rows_kernel"))) return rc;
  }
  return LCE_OK;
}


}  // namespace
