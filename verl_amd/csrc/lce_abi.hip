// C ABI of liblce_gfx950.so (see include/lce_abi.h): argument checks, the choice of the tile variant, and the kernels
// that do not depend on the GEMM element type.  The forward / backward launchers are compiled per element type in
// lce_dtype.hip.  Nothing here allocates device memory: callers bring the workspace.
#include "lce_host.hpp"

namespace lce_shared {
thread_local char err[512] = "";
std::mutex prof_mu;
bool prof_on = false;
std::vector<ProfRec> prof_recs;
std::vector<hipEvent_t> prof_pool;
}  // namespace lce_shared

namespace {

// Tuning state.  Every entry point takes ONE snapshot of it under the mutex and works from that copy, so a setter
// running on another thread can never change the workspace layout between a call's own size check and its launches.
// (A setter between lce_backward_workspace_bytes and lce_backward can still make the two disagree: lce_backward
// re-derives the size from its own snapshot and returns LCE_E_WORKSPACE instead of overrunning the buffer.)
std::mutex g_tuning_mu;
Tuning g_tuning;
Tuning tuning_snapshot() {
  std::lock_guard<std::mutex> l(g_tuning_mu);
  return g_tuning;
}

// the per-type launchers (one object of the library each), indexed by LCE_DTYPE_*
typedef int (*ForwardFn)(int, LCE_FWD_PARAMS);
typedef int (*BackwardFn)(int, LCE_BWD_PARAMS);
typedef int (*GemmFn)(int, LCE_GEMM_PARAMS);
ForwardFn const kForward[3] = {forward_bf16, forward_f32, forward_f16};
BackwardFn const kBackward[3] = {backward_bf16, backward_f32, backward_f16};
GemmFn const kGemmNt[3] = {gemm_nt_bf16, gemm_nt_f32, gemm_nt_f16};
static_assert(LCE_DTYPE_BF16 == 0 && LCE_DTYPE_F32 == 1 && LCE_DTYPE_F16 == 2, "order of the launcher tables");

int check_common(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                 int64_t H, int64_t V, int dtype, float temperature, int reduction) {
  if (!known_dtype(dtype)) return fail(LCE_E_ARG, "unsupported dtype %d", dtype);
  const int64_t kmul = esize(dtype) == 2 ? 64 : 32, ldmul = esize(dtype) == 2 ? 8 : 4;
  if (T < 0 || H <= 0 || V <= 0) return fail(LCE_E_ARG, "bad shape T=%lld H=%lld V=%lld", (long long)T, (long long)H, (long long)V);
  if (V >= (1LL << 31) || T >= (1LL << 31)) return fail(LCE_E_ARG, "T and V must be below 2^31");
  if (H % kmul != 0) return fail(LCE_E_ARG, "hidden size %lld must be a multiple of %lld", (long long)H, (long long)kmul);
  if (ldh < H || ldw < H || ldh % ldmul != 0 || ldw % ldmul != 0) return fail(LCE_E_ARG, "bad row strides ldh=%lld ldw=%lld", (long long)ldh, (long long)ldw);
  // the loads address a 256-row tile with 32-bit byte offsets from its first row
  const int64_t esz = esize(dtype);
  if (ldh * esz * 256 >= (1LL << 32) || ldw * esz * 256 >= (1LL << 32))
    return fail(LCE_E_ARG, "row strides ldh=%lld ldw=%lld too large: 256 rows must span less than 4 GiB", (long long)ldh, (long long)ldw);
  if (T > 0 && (!hidden || !weight || !labels)) return fail(LCE_E_ARG, "null input pointer");
  if (!aligned16(hidden) || !aligned16(weight)) return fail(LCE_E_ARG, "hidden and weight must be 16-byte aligned");
  if (!(temperature > 0.f)) return fail(LCE_E_ARG, "temperature must be positive");
  if (reduction < 0 || reduction > 2) return fail(LCE_E_ARG, "Invalid reduction: %d", reduction);
  return LCE_OK;
}

}  // namespace

// Scratch memory of lce_forward_static: device memory that lives in the library's own image, so that the entry point
// needs no caller workspace and allocates nothing.  Every GPU that runs the library holds its own copy of the array at
// its own address (found once per device with hipGetSymbolAddress); the array's name itself is only a host-side
// stand-in and is never passed to a kernel.
static __device__ __align__(256) unsigned char scratch[LCE_STATIC_SCRATCH_BYTES];
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
// per device: the address of `scratch`, and who used it last (the stream, and an event recorded behind that call's last
// kernel) so that a call on ANOTHER stream while that one is still running is refused instead of racing for the buffer
struct StaticUse {
  void* ptr = nullptr;
  hipEvent_t done = nullptr;
  hipStream_t last_stream = nullptr;
  bool recorded = false;
};
StaticUse g_static[kMaxDevices];
// set-up of the current device's entry (once per device; the caller holds g_scratch_mu)
int static_scratch(StaticUse** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(LCE_E_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(LCE_E_ARG, "device index %d out of range", dev);
  StaticUse& u = g_static[dev];
  if (!u.ptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return fail(LCE_E_LAUNCH, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    e = hipEventCreateWithFlags(&u.done, hipEventDisableTiming);
    if (e != hipSuccess) return fail(LCE_E_LAUNCH, "hipEventCreateWithFlags: %s", hipGetErrorString(e));
    u.ptr = ptr;
  }
  *out = &u;
  return LCE_OK;
}
}  // namespace

extern "C" {


int lce_abi_version(void) { return LCE_ABI_VERSION; }
const char* lce_last_error(void) { return lce_shared::err; }
int lce_num_variants(void) { return kNumVariants; }
int lce_set_variant(int variant) {
  if (variant < -1 || variant >= kNumVariants) return fail(LCE_E_ARG, "variant %d out of range", variant);
  std::lock_guard<std::mutex> l(g_tuning_mu);
  g_tuning.variant_forced = variant >= 0;
  g_tuning.variant_fwd = variant < 0 ? kDefaultVariantFwd : variant;
  g_tuning.variant_bwd = variant < 0 ? kDefaultVariantBwd : variant;
  return LCE_OK;
}
int lce_set_option(int key, int64_t value) {
  std::lock_guard<std::mutex> l(g_tuning_mu);
  Tuning& t = g_tuning;
  switch (key) {
    case LCE_OPT_SPLIT_BACKWARD_LAUNCHES: t.split_bwd = value != 0; return LCE_OK;
    case LCE_OPT_LABEL_TERM_OUTSIDE:
      if (value < 0 || value > 2) return fail(LCE_E_ARG, "LCE_OPT_LABEL_TERM_OUTSIDE takes 0, 1 or 2");
      t.label_outside = (int)value;
      return LCE_OK;
    case LCE_OPT_DLOGITS_TOKENS_FIRST: t.ds_tokens_first = value < 0 ? -1 : (value != 0); return LCE_OK;
    case LCE_OPT_DHIDDEN_KSPLIT:
      if (value < 0 || value > 16) return fail(LCE_E_ARG, "LCE_OPT_DHIDDEN_KSPLIT takes 0..16");
      t.dh_ksplit = (int)value;
      return LCE_OK;
    case LCE_OPT_FEW_TOKEN_GEMMS: t.few_token_gemms = value != 0; return LCE_OK;
    case LCE_OPT_WORKSPACE_BUDGET:
      if (value < 0) return fail(LCE_E_ARG, "LCE_OPT_WORKSPACE_BUDGET takes a byte count (0 = the built-in default)");
      t.ws_budget = value;
      return LCE_OK;
    case LCE_OPT_KEEP_LOGITS_TOKENS:
      if (value < 0) return fail(LCE_E_ARG, "LCE_OPT_KEEP_LOGITS_TOKENS takes a token count >= 0 (0: no logits are kept)");
      t.keep_logits_tokens = value;
      return LCE_OK;
    default: return fail(LCE_E_ARG, "unknown option %d", key);
  }
}

int lce_profile_enable(int on) {
  std::lock_guard<std::mutex> l(lce_shared::prof_mu);
  lce_shared::prof_on = on != 0;
  return LCE_OK;
}
int lce_profile_num_classes(void) { return PC_COUNT; }
const char* lce_profile_class_name(int cls) {
  static const char* names[PC_COUNT] = {"lce_fwd_kernel", "lce_fwd_merge_kernel", "lce_bwd_ds_kernel", "gemm_nt_kernel(d_hidden)",
                                        "gemm_nt_kernel(d_weight)", "transpose_pad_kernel", "logits_fwd_kernel", "logits_bwd_kernel",
                                        "lce_bwd_chunk_kernel", "active_rows_kernel", "dh_finish_kernel", "label_rows_kernels"};
  return (cls >= 0 && cls < PC_COUNT) ? names[cls] : "";
}
int lce_profile_read(double* total_ms, int64_t* launches, int reset) {
  std::lock_guard<std::mutex> l(lce_shared::prof_mu);
  for (int c = 0; c < PC_COUNT; ++c) { total_ms[c] = 0.0; launches[c] = 0; }
  for (const ProfRec& r : lce_shared::prof_recs) {
    if (hipEventSynchronize(r.b) != hipSuccess) return fail(LCE_E_LAUNCH, "profile: event synchronize failed");
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, r.a, r.b) != hipSuccess) return fail(LCE_E_LAUNCH, "profile: elapsed time failed");
    total_ms[r.cls] += ms;
    launches[r.cls] += 1;
  }
  if (reset) {
    for (const ProfRec& r : lce_shared::prof_recs) { lce_shared::prof_pool.push_back(r.a); lce_shared::prof_pool.push_back(r.b); }
    lce_shared::prof_recs.clear();
  }
  return LCE_OK;
}

// bytes of forward workspace when at most max_splits vocabulary splits are used: their partial statistics [S][T][4] fp32,
// the label logits [T] and (for the reductions) the per-token log-probs [T]
static size_t forward_workspace_need(int64_t T, int64_t V, int max_splits) {
  if (T <= 0) return 256;
  return align256((size_t)forward_splits_upper_bound(T, V > 0 ? V : 1, max_splits) * (size_t)T * 16) + 2 * align256((size_t)T * 4);
}

size_t lce_forward_workspace_bytes(int64_t T, int64_t H, int64_t V, int dtype) {
  (void)H; (void)dtype;
  return forward_workspace_need(T, V, kMaxSplits);
}

// shared body of lce_forward and lce_forward_shard
static int forward_entry(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                         int64_t H, int64_t V, int dtype, float temperature, int reduction, float* logprobs, float* entropy,
                         float* maximum, float* accumulate, float* entropy_b, void* workspace, size_t workspace_bytes,
                         void* stream, int64_t label_offset, float* shard_out, int max_splits = kMaxSplits, float* xcache = nullptr) {
  int rc = check_common(hidden, ldh, weight, ldw, labels, T, H, V, dtype, temperature, reduction);
  if (rc) return rc;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (T == 0) {
    if (!shard_out && reduction != LCE_REDUCTION_NONE && logprobs) {
      hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, st, reinterpret_cast<uint32_t*>(logprobs), (int64_t)1);
      return check_launch("fill_zero_kernel");
    }
    return LCE_OK;
  }
  if (!shard_out && (!logprobs || !entropy || !maximum || !accumulate || !entropy_b)) return fail(LCE_E_ARG, "null output pointer");
  if (!workspace || workspace_bytes < forward_workspace_need(T, V, max_splits))
    return fail(LCE_E_WORKSPACE, "forward workspace too small: %zu < %zu", workspace_bytes, forward_workspace_need(T, V, max_splits));
  char* ws = static_cast<char*>(workspace);
  const Tuning tu = tuning_snapshot();
  int sel = tu.variant_fwd;
  if (!tu.variant_forced) {
    if (T <= 64) sel = kSelT64;
    else if (T <= 128) sel = kSelT128;
    else if (T <= 512) sel = 0;  // W (the A operand) streams from HBM: give it the early slot
    else if (esize(dtype) == 2 && T > kCore16MinTokensFwd) sel = kVariantCore16;
    // the split ring: measured 4-7% faster than the 2-stage ring up to 8192 tokens, equal (+-1%) beyond, and
    // 4.5% faster again once `hidden` is far larger than the memory-side cache (T=65536, H=5120: 671 MB)
    else if (T <= 8192 || (uint64_t)T * (uint64_t)H * esize(dtype) > (512ull << 20)) sel = 1;
  }
  if (xcache && sel != kSelT64 && sel != kSelT128 && sel != 0 && !(sel == kVariantCore16 && esize(dtype) == 2))
    return fail(LCE_E_ARG, "forward: tile selector %d cannot keep the logits", sel);
  return kForward[dtype](sel, hidden, ldh, weight, ldw, labels, T, H, V, temperature, reduction, logprobs, entropy, maximum,
                         accumulate, entropy_b, ws, st, label_offset, shard_out, max_splits, xcache);
}

int64_t lce_logits_cache_max_tokens(int64_t H, int dtype) {
  if (!known_dtype(dtype) || H <= 0) return 0;
  const Tuning tu = tuning_snapshot();
  if (tu.variant_forced) return 0;  // (a forced tile variant may be one that cannot write the cache)
  const int64_t most = logits_cache_max_tokens(H, esize(dtype));
  return most < tu.keep_logits_tokens ? most : tu.keep_logits_tokens;
}

size_t lce_logits_cache_bytes(int64_t T, int64_t H, int64_t V, int dtype) {
  if (V <= 0 || T < 1 || T > lce_logits_cache_max_tokens(H, dtype)) return 0;
  return (size_t)T * (size_t)logits_cache_row(V) * 4;
}

int lce_forward_keep_logits(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                            int64_t H, int64_t V, int dtype, float temperature, int reduction, float* logprobs, float* entropy,
                            float* maximum, float* accumulate, float* entropy_b, void* workspace, size_t workspace_bytes,
                            void* logits_cache, size_t logits_cache_bytes, void* stream) {
  if (logits_cache) {
    const size_t need = known_dtype(dtype) ? lce_logits_cache_bytes(T, H, V, dtype) : 0;
    if (need == 0) return fail(LCE_E_ARG, "lce_forward_keep_logits: no logits are kept for this shape (lce_logits_cache_bytes is 0): pass NULL");
    if (logits_cache_bytes < need) return fail(LCE_E_WORKSPACE, "logits cache too small: %zu < %zu", logits_cache_bytes, need);
    if (reinterpret_cast<size_t>(logits_cache) % 16 != 0) return fail(LCE_E_ARG, "logits cache must be 16-byte aligned");
  }
  return forward_entry(hidden, ldh, weight, ldw, labels, T, H, V, dtype, temperature, reduction, logprobs, entropy, maximum,
                       accumulate, entropy_b, workspace, workspace_bytes, stream, 0, nullptr, kMaxSplits, static_cast<float*>(logits_cache));
}

int lce_forward(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                int64_t H, int64_t V, int dtype, float temperature, int reduction, float* logprobs, float* entropy,
                float* maximum, float* accumulate, float* entropy_b, void* workspace, size_t workspace_bytes,
                void* stream) {
  return forward_entry(hidden, ldh, weight, ldw, labels, T, H, V, dtype, temperature, reduction, logprobs, entropy, maximum,
                       accumulate, entropy_b, workspace, workspace_bytes, stream, 0, nullptr);
}

int lce_forward_static(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T, int64_t H,
                       int64_t V, int dtype, float temperature, int reduction, float* logprobs, float* entropy, float* maximum,
                       float* accumulate, float* entropy_b, void* stream) {
  if (!known_dtype(dtype)) return fail(LCE_E_ARG, "unsupported dtype %d", dtype);
  // as many vocabulary splits as the buffer has room for (16 bytes per token and split, 8 more per token); the forward
  // wants at least the four that fill an XCD's tile block
  int max_splits = kMaxSplits;
  if (T > 0) {
    const size_t fixed = 2 * align256((size_t)T * 4) + 256;
    const size_t room = (size_t)LCE_STATIC_SCRATCH_BYTES > fixed ? ((size_t)LCE_STATIC_SCRATCH_BYTES - fixed) / ((size_t)T * 16) : 0;
    if (room < 4)
      return fail(LCE_E_WORKSPACE, "lce_forward_static: T=%lld needs %zu bytes of scratch, the built-in buffer holds %zu; use lce_forward with a workspace",
                  (long long)T, fixed + (size_t)T * 64, (size_t)LCE_STATIC_SCRATCH_BYTES);
    if (room < (size_t)kMaxSplits) max_splits = (int)room;
  }
  // One call at a time per device on the host side: the check below, the launches and the record behind them are one step.
  std::lock_guard<std::mutex> l(g_scratch_mu);
  StaticUse* use = nullptr;
  int rc = static_scratch(&use);
  if (rc) return rc;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  // (a capturing stream records nothing here and is not checked: inside a graph the order of the nodes is the caller's)
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  const bool capturing = hipStreamIsCapturing(st, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone;
  if (!capturing && use->recorded && use->last_stream != st && hipEventQuery(use->done) == hipErrorNotReady)
    return fail(LCE_E_BUSY, "lce_forward_static: the previous call on this GPU, on another stream, is still running and owns the "
                            "built-in scratch buffer; order the two streams, or use lce_forward with a workspace of your own");
  // (nothing in the buffer has to start at zero, and nothing of the previous call's contents is read)
  rc = forward_entry(hidden, ldh, weight, ldw, labels, T, H, V, dtype, temperature, reduction, logprobs, entropy, maximum,
                     accumulate, entropy_b, use->ptr, (size_t)LCE_STATIC_SCRATCH_BYTES, stream, 0, nullptr, max_splits);
  if (rc == LCE_OK && !capturing && T > 0) {
    if (hipEventRecord(use->done, st) != hipSuccess) return fail(LCE_E_LAUNCH, "lce_forward_static: hipEventRecord failed");
    use->last_stream = st;
    use->recorded = true;
  }
  return rc;
}

int lce_forward_shard(const void* hidden, int64_t ldh, const void* weight_shard, int64_t ldw, const int64_t* labels, int64_t T,
                      int64_t H, int64_t V_local, int64_t vocab_offset, int dtype, float temperature, float* partials,
                      void* workspace, size_t workspace_bytes, void* stream) {
  if (!partials && T > 0) return fail(LCE_E_ARG, "null partials pointer");
  if (vocab_offset < 0) return fail(LCE_E_ARG, "vocab_offset must be >= 0");
  return forward_entry(hidden, ldh, weight_shard, ldw, labels, T, H, V_local, dtype, temperature, LCE_REDUCTION_NONE, nullptr,
                       nullptr, nullptr, nullptr, nullptr, workspace, workspace_bytes, stream, vocab_offset, partials);
}

int lce_merge_shards(const float* partials, int R, int64_t T, int reduction, float* logprobs, float* entropy, float* maximum,
                     float* accumulate, float* entropy_b, void* workspace, size_t workspace_bytes, void* stream) {
  if (R <= 0 || T < 0) return fail(LCE_E_ARG, "bad shard count or token count");
  if (reduction < 0 || reduction > 2) return fail(LCE_E_ARG, "Invalid reduction: %d", reduction);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (T == 0) {
    if (reduction != LCE_REDUCTION_NONE && logprobs) {
      hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, st, reinterpret_cast<uint32_t*>(logprobs), (int64_t)1);
      return check_launch("fill_zero_kernel");
    }
    return LCE_OK;
  }
  if (!partials || !logprobs || !entropy || !maximum || !accumulate || !entropy_b) return fail(LCE_E_ARG, "null pointer");
  float* lp_tok = logprobs;
  if (reduction != LCE_REDUCTION_NONE) {
    if (!workspace || workspace_bytes < (size_t)T * 4) return fail(LCE_E_WORKSPACE, "merge workspace too small: need %zu bytes", (size_t)T * 4);
    lp_tok = static_cast<float*>(workspace);
  }
  hipLaunchKernelGGL(lce_merge_shards_kernel, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, st,
                     reinterpret_cast<const f32x4_t*>(partials), R, T, lp_tok, entropy, maximum, accumulate, entropy_b);
  int rc = check_launch("lce_merge_shards_kernel");
  if (rc) return rc;
  if (reduction != LCE_REDUCTION_NONE) {
    const float scale = reduction == LCE_REDUCTION_MEAN ? 1.0f / (float)T : 1.0f;
    hipLaunchKernelGGL(lce_reduce_sum_kernel, dim3(1), dim3(1024), 0, st, lp_tok, T, scale, logprobs);
    rc = check_launch("lce_reduce_sum_kernel");
  }
  return rc;
}

size_t lce_backward_workspace_bytes(int64_t T, int64_t H, int64_t V, int dtype, int64_t vchunk) {
  if (T <= 0 || H <= 0 || V <= 0) return 256;
  return bwd_layout(tuning_snapshot(), T, H, V, esize(dtype), vchunk).total + 256;
}

// shared body of lce_backward and lce_backward_shard
static int backward_entry(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                          int64_t H, int64_t V, int dtype, float temperature, int reduction, const float* maximum,
                          const float* accumulate, const float* entropy_b, const float* dlogprobs, const float* dentropy,
                          void* d_hidden, void* d_weight, void* workspace, size_t workspace_bytes, int64_t vchunk,
                          void* stream, int64_t vocab_offset, bool grads_f32 = false, const float* xcache = nullptr) {
  int rc = check_common(hidden, ldh, weight, ldw, labels, T, H, V, dtype, temperature, reduction);
  if (rc) return rc;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const size_t esz = esize(dtype);
  if (!d_weight && !d_hidden) return fail(LCE_E_ARG, "null d_hidden and d_weight: nothing to compute");
  if (T == 0) {
    if (!d_weight) return LCE_OK;
    const int64_t words = (int64_t)((size_t)V * H * (grads_f32 ? 4 : esz) / 4);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(1024), dim3(256), 0, st, reinterpret_cast<uint32_t*>(d_weight), words);
    return check_launch("fill_zero_kernel");
  }
  if (!maximum || !accumulate || !entropy_b || !dlogprobs) return fail(LCE_E_ARG, "null pointer");
  if (!aligned16(d_hidden) || !aligned16(d_weight)) return fail(LCE_E_ARG, "gradients must be 16-byte aligned");
  if (vchunk < 0) return fail(LCE_E_ARG, "vchunk must be >= 0");
  const Tuning tu = tuning_snapshot();
  const size_t need = bwd_layout(tu, T, H, V, esz, vchunk).total + 256;
  if (!workspace || workspace_bytes < need) return fail(LCE_E_WORKSPACE, "backward workspace too small: %zu < %zu", workspace_bytes, need);
  char* ws = reinterpret_cast<char*>(align256(reinterpret_cast<size_t>(workspace)));
  return kBackward[dtype](bwd_variant(tu, T, esz), hidden, ldh, weight, ldw, labels, T, H, V, temperature, reduction, maximum,
                          accumulate, entropy_b, dlogprobs, dentropy, d_hidden, d_weight, grads_f32, ws, vchunk, st, vocab_offset,
                          tu, xcache);
}

int lce_backward_from_logits(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                             int64_t H, int64_t V, int dtype, float temperature, int reduction, const float* maximum,
                             const float* accumulate, const float* entropy_b, const float* dlogprobs, const float* dentropy,
                             void* d_hidden, void* d_weight, int grads_fp32, void* workspace, size_t workspace_bytes, int64_t vchunk,
                             const void* logits_cache, size_t logits_cache_bytes, void* stream) {
  if (logits_cache) {
    const size_t need = known_dtype(dtype) ? lce_logits_cache_bytes(T, H, V, dtype) : 0;
    if (need == 0) return fail(LCE_E_ARG, "lce_backward_from_logits: no logits are kept for this shape (lce_logits_cache_bytes is 0): pass NULL");
    if (logits_cache_bytes < need) return fail(LCE_E_WORKSPACE, "logits cache too small: %zu < %zu", logits_cache_bytes, need);
    if (reinterpret_cast<size_t>(logits_cache) % 16 != 0) return fail(LCE_E_ARG, "logits cache must be 16-byte aligned");
  }
  return backward_entry(hidden, ldh, weight, ldw, labels, T, H, V, dtype, temperature, reduction, maximum, accumulate, entropy_b,
                        dlogprobs, dentropy, d_hidden, d_weight, workspace, workspace_bytes, vchunk, stream, 0, grads_fp32 != 0,
                        static_cast<const float*>(logits_cache));
}

int lce_backward(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T,
                 int64_t H, int64_t V, int dtype, float temperature, int reduction, const float* maximum,
                 const float* accumulate, const float* entropy_b, const float* dlogprobs, const float* dentropy,
                 void* d_hidden, void* d_weight, void* workspace, size_t workspace_bytes, int64_t vchunk,
                 void* stream) {
  return backward_entry(hidden, ldh, weight, ldw, labels, T, H, V, dtype, temperature, reduction, maximum, accumulate, entropy_b,
                        dlogprobs, dentropy, d_hidden, d_weight, workspace, workspace_bytes, vchunk, stream, 0);
}

int lce_backward_f32(const void* hidden, int64_t ldh, const void* weight, int64_t ldw, const int64_t* labels, int64_t T, int64_t H,
                     int64_t V, int dtype, float temperature, int reduction, const float* maximum, const float* accumulate,
                     const float* entropy_b, const float* dlogprobs, const float* dentropy, float* d_hidden, float* d_weight,
                     void* workspace, size_t workspace_bytes, int64_t vchunk, void* stream) {
  return backward_entry(hidden, ldh, weight, ldw, labels, T, H, V, dtype, temperature, reduction, maximum, accumulate, entropy_b,
                        dlogprobs, dentropy, d_hidden, d_weight, workspace, workspace_bytes, vchunk, stream, 0, true);
}

int lce_backward_shard(const void* hidden, int64_t ldh, const void* weight_shard, int64_t ldw, const int64_t* labels, int64_t T,
                       int64_t H, int64_t V_local, int64_t vocab_offset, int dtype, float temperature, int reduction,
                       const float* maximum, const float* accumulate, const float* entropy_b, const float* dlogprobs,
                       const float* dentropy, void* d_hidden_partial, void* d_weight_shard, void* workspace,
                       size_t workspace_bytes, int64_t vchunk, void* stream) {
  if (vocab_offset < 0) return fail(LCE_E_ARG, "vocab_offset must be >= 0");
  return backward_entry(hidden, ldh, weight_shard, ldw, labels, T, H, V_local, dtype, temperature, reduction, maximum, accumulate,
                        entropy_b, dlogprobs, dentropy, d_hidden_partial, d_weight_shard, workspace, workspace_bytes, vchunk, stream,
                        vocab_offset);
}

int lce_gemm_nt(const void* A, int64_t lda, const void* B, int64_t ldb, float* C, int64_t ldc, int64_t M, int64_t N,
                int64_t K, int dtype, int variant, void* stream) {
  if (!known_dtype(dtype)) return fail(LCE_E_ARG, "unsupported dtype %d", dtype);
  if (!A || !B || !C || !aligned16(A) || !aligned16(B)) return fail(LCE_E_ARG, "bad pointer");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (variant < 0 || variant >= kNumVariants) return fail(LCE_E_ARG, "variant %d out of range", variant);
  return kGemmNt[dtype](variant, A, lda, B, ldb, C, ldc, M, N, K, st);
}

int lce_gemm_tn(const void* A, int64_t lda, const void* B, int64_t ldb, float* C, int64_t ldc, int64_t M, int64_t N, int64_t K,
                int variant, void* stream) {
  if (!A || !B || !C || !aligned16(A) || !aligned16(B)) return fail(LCE_E_ARG, "bad pointer");
  if (M <= 0 || N <= 0 || K <= 0 || K % 64 != 0 || lda % 8 != 0 || ldb % 8 != 0) return fail(LCE_E_ARG, "gemm_tn: bad shape");
  if (lda < round_up(M, 256) || ldb < round_up(N, 256)) return fail(LCE_E_ARG, "gemm_tn: rows must be allocated in whole 256-column tiles");
  const bool core16 = variant == kVariantCore16;  // the same product on the four-wave 16x16x32 loop
  if (core16 && N % 4 != 0) return fail(LCE_E_ARG, "gemm_tn: N must be a multiple of 4");
  return gemm_tn_bf16(core16, A, lda, B, ldb, C, ldc, M, N, K, reinterpret_cast<hipStream_t>(stream));
}

int lce_logits_forward(const void* logits, int64_t ldl, const int64_t* labels, int64_t R, int64_t V, int dtype,
                       float* logprobs, float* entropy, float* stats, void* stream) {
  if (!known_dtype(dtype)) return fail(LCE_E_ARG, "unsupported dtype %d", dtype);
  if (R < 0 || V <= 0 || ldl < V) return fail(LCE_E_ARG, "bad shape R=%lld V=%lld ldl=%lld", (long long)R, (long long)V, (long long)ldl);
  if (R == 0) return LCE_OK;
  if (!logits || (logprobs && !labels)) return fail(LCE_E_ARG, "null pointer");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  constexpr int NT = 512;
  ProfScope prof(PC_LOGITS_FWD, st);
  if (dtype == LCE_DTYPE_BF16)
    hipLaunchKernelGGL((logits_fwd_kernel<bf16_t, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const bf16_t*)logits, ldl, labels, V, logprobs, entropy, stats);
  else if (dtype == LCE_DTYPE_F16)
    hipLaunchKernelGGL((logits_fwd_kernel<f16_t, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const f16_t*)logits, ldl, labels, V, logprobs, entropy, stats);
  else
    hipLaunchKernelGGL((logits_fwd_kernel<float, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const float*)logits, ldl, labels, V, logprobs, entropy, stats);
  return check_launch("logits_fwd_kernel");
}

int lce_logits_sum_pi_squared(const void* logits, int64_t ldl, int64_t R, int64_t V, int dtype, float* out, float* lse_out, void* stream) {
  if (!known_dtype(dtype)) return fail(LCE_E_ARG, "unsupported dtype %d", dtype);
  if (R < 0 || V <= 0 || ldl < V) return fail(LCE_E_ARG, "bad shape R=%lld V=%lld ldl=%lld", (long long)R, (long long)V, (long long)ldl);
  if (R == 0) return LCE_OK;
  if (!logits || !out) return fail(LCE_E_ARG, "null pointer");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  constexpr int NT = 512;
  ProfScope prof(PC_LOGITS_FWD, st);
  if (dtype == LCE_DTYPE_BF16)
    hipLaunchKernelGGL((logits_pi2_kernel<bf16_t, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const bf16_t*)logits, ldl, V, out, lse_out);
  else if (dtype == LCE_DTYPE_F16)
    hipLaunchKernelGGL((logits_pi2_kernel<f16_t, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const f16_t*)logits, ldl, V, out, lse_out);
  else
    hipLaunchKernelGGL((logits_pi2_kernel<float, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const float*)logits, ldl, V, out, lse_out);
  return check_launch("logits_pi2_kernel");
}

int lce_logits_sum_pi_squared_backward(const void* logits, int64_t ldl, int64_t R, int64_t V, int dtype, const float* lse, const float* sum_pi2,
                                       const float* g, void* d_logits, int64_t ldd, void* stream) {
  if (!known_dtype(dtype)) return fail(LCE_E_ARG, "unsupported dtype %d", dtype);
  if (R < 0 || V <= 0 || ldl < V || ldd < V)
    return fail(LCE_E_ARG, "bad shape R=%lld V=%lld ldl=%lld ldd=%lld", (long long)R, (long long)V, (long long)ldl, (long long)ldd);
  if (R == 0) return LCE_OK;
  if (!logits || !g || !d_logits) return fail(LCE_E_ARG, "null pointer");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  constexpr int NT = 512;
  ProfScope prof(PC_LOGITS_BWD, st);
  if (dtype == LCE_DTYPE_BF16)
    hipLaunchKernelGGL((logits_pi2_bwd_kernel<bf16_t, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const bf16_t*)logits, ldl, V, lse, sum_pi2, g,
                       (bf16_t*)d_logits, ldd);
  else if (dtype == LCE_DTYPE_F16)
    hipLaunchKernelGGL((logits_pi2_bwd_kernel<f16_t, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const f16_t*)logits, ldl, V, lse, sum_pi2, g,
                       (f16_t*)d_logits, ldd);
  else
    hipLaunchKernelGGL((logits_pi2_bwd_kernel<float, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const float*)logits, ldl, V, lse, sum_pi2, g,
                       (float*)d_logits, ldd);
  return check_launch("logits_pi2_bwd_kernel");
}

// geometry of the PPO loss launches: workgroups per row and elements per workgroup
static void ppo_geometry(int64_t rows, int64_t row_len, int* segs, int64_t* seg_len) {
  int64_t want = (row_len + 1023) / 1024;        // about 4 elements per thread
  int64_t cap = rows >= 4096 ? 1 : 4096 / rows;  // bounds what the single finishing workgroup walks
  int64_t s = want < cap ? want : cap;
  if (s < 1) s = 1;
  *seg_len = (row_len + s - 1) / s;
  *segs = (int)((row_len + *seg_len - 1) / *seg_len);
}

static size_t ppo_align(size_t x) { return (x + 255) & ~(size_t)255; }

size_t lce_ppo_loss_workspace_bytes(int64_t rows, int64_t row_len) {
  if (rows <= 0 || row_len <= 0) return 0;
  int segs;
  int64_t seg_len;
  ppo_geometry(rows, row_len, &segs, &seg_len);
  return ppo_align((size_t)rows * segs * 8 * sizeof(float)) + ppo_align((size_t)rows * 4 * sizeof(double)) +
         ppo_align((size_t)rows * sizeof(float));
}

// shared body of lce_ppo_loss and lce_ppo_loss_packed
static int ppo_entry(const float* log_prob, const float* entropy, const int64_t* pk_start, const int64_t* pk_len, int64_t total_nnz,
                     const float* old_log_prob, const float* advantages, const float* mask, const float* is_weights,
                     const float* ref_log_prob, int kl_type, float kl_coef, int64_t rows, int64_t row_len, int agg_mode, float clip_low,
                     float clip_high, float clip_c, float entropy_coeff, float dp_size, float batch_num_tokens,
                     float global_batch_size, float loss_scale_factor, float* out, float* g_log_prob, float* g_entropy,
                     void* workspace, size_t workspace_bytes, void* stream) {
  if (rows <= 0 || row_len <= 0) return fail(LCE_E_ARG, "ppo loss: rows and row_len must be positive");
  if (rows > ((int64_t)1 << 30) || row_len > ((int64_t)1 << 40) / rows) return fail(LCE_E_ARG, "ppo loss: too many elements");
  if (!mask || !out) return fail(LCE_E_ARG, "null pointer");
  if (log_prob) {
    if (!old_log_prob || !advantages || !g_log_prob) return fail(LCE_E_ARG, "null pointer");
    if (!(clip_c > 1.f)) return fail(LCE_E_ARG, "clip_ratio_c must be greater than 1");
  } else if (!entropy || g_log_prob || kl_type != LCE_PPO_KL_NONE) {
    return fail(LCE_E_ARG, "without log_prob the call aggregates `entropy` alone");
  }
  if ((entropy == nullptr) != (g_entropy == nullptr)) return fail(LCE_E_ARG, "entropy and g_entropy go together");
  if ((pk_start == nullptr) != (pk_len == nullptr)) return fail(LCE_E_ARG, "packed layout: starts and lengths go together");
  if (pk_start && total_nnz < 0) return fail(LCE_E_ARG, "packed layout: total_nnz must be >= 0");
  const int kl_base = kl_type & ~LCE_PPO_KL_STRAIGHT_THROUGH;
  if (kl_base < LCE_PPO_KL_NONE || kl_base > LCE_PPO_KL_K3 || (kl_base == LCE_PPO_KL_NONE && kl_type != LCE_PPO_KL_NONE))
    return fail(LCE_E_ARG, "ppo loss: unknown kl_type %d", kl_type);
  if (kl_base != LCE_PPO_KL_NONE && !ref_log_prob) return fail(LCE_E_ARG, "the KL penalty needs ref_log_prob");
  if (agg_mode < PPO_TOKEN_MEAN || agg_mode > PPO_SEQ_MEAN_TOKEN_MEAN) return fail(LCE_E_ARG, "Invalid loss_agg_mode: %d", agg_mode);
  if (!(dp_size > 0.f)) return fail(LCE_E_ARG, "ppo loss: dp_size must be positive");
  if (!workspace || workspace_bytes < lce_ppo_loss_workspace_bytes(rows, row_len))
    return fail(LCE_E_WORKSPACE, "ppo workspace too small");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  PpoArgs p;
  ppo_geometry(rows, row_len, &p.segs, &p.seg_len);
  const int64_t blocks = rows * p.segs;
  if (blocks > 0x7fffffff) return fail(LCE_E_ARG, "ppo loss: too many rows");
  char* ws = static_cast<char*>(workspace);
  p.partials = reinterpret_cast<float*>(ws);
  ws += ppo_align((size_t)blocks * 8 * sizeof(float));
  double* row_tot = reinterpret_cast<double*>(ws);
  ws += ppo_align((size_t)rows * 4 * sizeof(double));
  float* row_weight = reinterpret_cast<float*>(ws);
  p.log_prob = log_prob; p.entropy = entropy; p.old_log_prob = old_log_prob; p.advantages = advantages; p.mask = mask;
  p.is_weights = is_weights; p.rows = rows; p.row_len = row_len;
  p.ref_log_prob = ref_log_prob; p.kl_type = kl_base; p.kl_coef = kl_coef;
  // (k2's own gradient is already the straight-through one, verl/trainer/ppo/core_algos.py:2203-2204)
  p.kl_straight_through = (kl_type & LCE_PPO_KL_STRAIGHT_THROUGH) != 0 && kl_base != LCE_PPO_KL_K2;
  p.clip_low = clip_low; p.clip_high = clip_high; p.clip_c = clip_c; p.entropy_coeff = entropy_coeff;
  p.g_log_prob = g_log_prob; p.g_entropy = g_entropy;
  p.pk_start = pk_start; p.pk_len = pk_len; p.total_nnz = total_nnz;
  PpoAgg g;
  g.mode = agg_mode; g.dp_size = dp_size; g.batch_num_tokens = batch_num_tokens; g.global_batch_size = global_batch_size;
  g.loss_scale_factor = loss_scale_factor; g.entropy_coeff = entropy_coeff;
  g.kl_coef = kl_base != LCE_PPO_KL_NONE ? kl_coef : 0.f;
  int rc;
  if (pk_start && total_nnz > 0) {
    // packed gradients: the positions no response token maps to (prompts, the last token of each sequence) are zeros
    for (float* gp : {g_log_prob, g_entropy}) {
      if (!gp) continue;
      hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((total_nnz + 1023) / 1024 < 4096 ? (total_nnz + 1023) / 1024 : 4096)), dim3(256), 0, st,
                         reinterpret_cast<uint32_t*>(gp), total_nnz);
      if ((rc = check_launch("fill_zero_kernel"))) return rc;
    }
  }
  hipLaunchKernelGGL(ppo_terms_kernel, dim3((unsigned)blocks), dim3(256), 0, st, p);
  if ((rc = check_launch("ppo_terms_kernel"))) return rc;
  hipLaunchKernelGGL(ppo_finish_kernel, dim3(1), dim3(256), 0, st, p.partials, rows, p.segs, row_len, g, row_tot,
                     row_weight, out);
  if ((rc = check_launch("ppo_finish_kernel"))) return rc;
  hipLaunchKernelGGL(ppo_scale_kernel, dim3((unsigned)blocks), dim3(256), 0, st, p, row_weight);
  return check_launch("ppo_scale_kernel");
}

int lce_ppo_loss(const float* log_prob, const float* entropy, const float* old_log_prob, const float* advantages,
                 const float* mask, const float* is_weights, const float* ref_log_prob, int kl_type, float kl_coef,
                 int64_t rows, int64_t row_len, int agg_mode,
                 float clip_low, float clip_high, float clip_c, float entropy_coeff, float dp_size,
                 float batch_num_tokens, float global_batch_size, float loss_scale_factor, float* out,
                 float* g_log_prob, float* g_entropy, void* workspace, size_t workspace_bytes, void* stream) {
  return ppo_entry(log_prob, entropy, nullptr, nullptr, 0, old_log_prob, advantages, mask, is_weights, ref_log_prob, kl_type, kl_coef, rows,
                   row_len, agg_mode, clip_low, clip_high, clip_c, entropy_coeff, dp_size, batch_num_tokens, global_batch_size,
                   loss_scale_factor, out, g_log_prob, g_entropy, workspace, workspace_bytes, stream);
}

int lce_ppo_loss_packed(const float* log_prob_packed, const float* entropy_packed, int64_t total_nnz, const int64_t* response_start,
                        const int64_t* response_len, const float* old_log_prob, const float* advantages, const float* mask,
                        const float* is_weights, const float* ref_log_prob, int kl_type, float kl_coef, int64_t rows, int64_t row_len,
                        int agg_mode, float clip_low, float clip_high, float clip_c, float entropy_coeff, float dp_size,
                        float batch_num_tokens, float global_batch_size, float loss_scale_factor, float* out,
                        float* g_log_prob_packed, float* g_entropy_packed, void* workspace, size_t workspace_bytes, void* stream) {
  if (!log_prob_packed || !response_start || !response_len) return fail(LCE_E_ARG, "ppo loss (packed): null pointer");
  return ppo_entry(log_prob_packed, entropy_packed, response_start, response_len, total_nnz, old_log_prob, advantages, mask, is_weights,
                   ref_log_prob, kl_type, kl_coef, rows, row_len, agg_mode, clip_low, clip_high, clip_c, entropy_coeff, dp_size,
                   batch_num_tokens, global_batch_size, loss_scale_factor, out, g_log_prob_packed, g_entropy_packed, workspace,
                   workspace_bytes, stream);
}

int lce_logits_backward(const void* logits, int64_t ldl, const int64_t* labels, int64_t R, int64_t V, int dtype,
                        const float* stats, const float* dlogprobs, const float* dentropy, void* d_logits, int64_t ldd,
                        void* stream) {
  if (!known_dtype(dtype)) return fail(LCE_E_ARG, "unsupported dtype %d", dtype);
  if (R < 0 || V <= 0 || ldl < V || ldd < V) return fail(LCE_E_ARG, "bad shape");
  if (R == 0) return LCE_OK;
  if (!logits || !d_logits || (dlogprobs && !labels)) return fail(LCE_E_ARG, "null pointer");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  constexpr int NT = 512;
  ProfScope prof(PC_LOGITS_BWD, st);
  if (dtype == LCE_DTYPE_BF16)
    hipLaunchKernelGGL((logits_bwd_kernel<bf16_t, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const bf16_t*)logits, ldl, labels, V, stats, dlogprobs, dentropy, (bf16_t*)d_logits, ldd);
  else if (dtype == LCE_DTYPE_F16)
    hipLaunchKernelGGL((logits_bwd_kernel<f16_t, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const f16_t*)logits, ldl, labels, V, stats, dlogprobs, dentropy, (f16_t*)d_logits, ldd);
  else
    hipLaunchKernelGGL((logits_bwd_kernel<float, NT>), dim3((unsigned)R), dim3(NT), 0, st, (const float*)logits, ldl, labels, V, stats, dlogprobs, dentropy, (float*)d_logits, ldd);
  return check_launch("logits_bwd_kernel");
}

}  // extern "C"
