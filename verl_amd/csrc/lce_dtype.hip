// One object of liblce_gfx950.so: the launchers of ONE element type (LCE_TU_DTYPE = LCE_DTYPE_BF16 / _F32 / _F16) in ONE
// direction (LCE_TU_PART = 0: forward and the plain NT GEMM; 1: backward, and for bf16 the TN GEMM), instantiated for every
// tile variant.  The build compiles the six combinations side by side; lce_abi.hip calls them through the declarations in
// lce_host.hpp.
#include "lce_host.hpp"

#if !defined(LCE_TU_DTYPE) || !defined(LCE_TU_PART)
#error "compile with -DLCE_TU_DTYPE=<LCE_DTYPE_*> -DLCE_TU_PART=<0|1>"
#endif

#if LCE_TU_DTYPE == 0
typedef bf16_t TuT;
#define TU_FN(name) name##_bf16
#elif LCE_TU_DTYPE == 1
typedef float TuT;
#define TU_FN(name) name##_f32
#elif LCE_TU_DTYPE == 2
typedef f16_t TuT;
#define TU_FN(name) name##_f16
#else
#error "unknown LCE_TU_DTYPE"
#endif

namespace lce_shared {

#if LCE_TU_PART == 0

int TU_FN(forward)(int sel, LCE_FWD_PARAMS) {
#define LCE_RUN(Vt)                                                                                                          \
  return forward_impl<typename Vt<TuT>::Cfg>((const TuT*)h, ldh, (const TuT*)W, ldw, labels, T, H, V, temperature, reduction, \
                                             lp, ent, mx, ac, eb, ws, st, label_offset, shard_out, max_splits, xcache)
  switch (sel) {
    case 0: LCE_RUN(Variant0);
    case 1: LCE_RUN(Variant1);
    case 2: LCE_RUN(Variant2);
    case 3: LCE_RUN(Variant3);
    case kSelT64: LCE_RUN(VariantT64);
    case kSelT128: LCE_RUN(VariantT128);
  }
#undef LCE_RUN
  return fail(LCE_E_ARG, "tile selector %d out of range", sel);
}

int TU_FN(gemm_nt)(int sel, LCE_GEMM_PARAMS) {
#define LCE_RUN(Vt) \
  return launch_gemm<typename Vt<TuT>::Cfg>((const TuT*)A, lda, (const TuT*)B, ldb, M, N, K, C, ldc, nullptr, 0, 0, st)
  switch (sel) {
    case 0: LCE_RUN(Variant0);
    case 1: LCE_RUN(Variant1);
    case 2: LCE_RUN(Variant2);
    case 3: LCE_RUN(Variant3);
  }
#undef LCE_RUN
  return fail(LCE_E_ARG, "variant %d out of range", sel);
}

#else  // LCE_TU_PART == 1

int TU_FN(backward)(int sel, LCE_BWD_PARAMS) {
#define LCE_RUN(Vt)                                                                                                           \
  return backward_impl<typename Vt<TuT>::Cfg>((const TuT*)h, ldh, (const TuT*)W, ldw, labels, T, H, V, temperature, reduction, \
                                              mx, ac, eb, glp, gent, dh, dw, grads_f32, ws, vchunk, st, vocab_offset, tu, xcache)
  // (bwd_variant() hands over one of the two mainloops the backward is built on)
  switch (sel) {
    case kDefaultVariantBwd: LCE_RUN(Variant1);
    case kVariantCore16: LCE_RUN(Variant3);
  }
#undef LCE_RUN
  return fail(LCE_E_ARG, "variant %d out of range", sel);
}

#if LCE_TU_DTYPE == 0
int gemm_tn_bf16(bool core16, LCE_GEMM_PARAMS) {
  typedef GemmCfg<bf16_t, 256, 256, 128, 5, 4, 2, 2, 1> Cfg;
  GemmArgs<bf16_t> p = make_gemm_args<Cfg>((const bf16_t*)A, lda, (const bf16_t*)B, ldb, M, N, K, C, ldc, nullptr, 0, 0);
  ProfScope prof(PC_GEMM_DW, st);
  if (core16) {
    typedef GemmCfg16<bf16_t> C16;
    allow_lds(gemm16_tn_kernel<C16>, C16::LDS_BYTES);
    hipLaunchKernelGGL(gemm16_tn_kernel<C16>, dim3(p.map.total), dim3(C16::NTHREADS), C16::LDS_BYTES, st, p);
    return check_launch("gemm16_tn_kernel");
  }
  allow_lds(gemm_tn_kernel<Cfg>, Cfg::LDS_BYTES);
  hipLaunchKernelGGL(gemm_tn_kernel<Cfg>, dim3(p.map.total), dim3(Cfg::NTHREADS), Cfg::LDS_BYTES, st, p);
  return check_launch("gemm_tn_kernel");
}
#endif

#endif

}  // namespace lce_shared
