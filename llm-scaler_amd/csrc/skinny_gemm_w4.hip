// Entry points of the weight-streaming GEMV / small-M GEMM for the 4-bit formats: INT4 group 128
// and GGUF Q4_K (repacked).  The FP8 entry points are in skinny_gemm.hip.
#include "skinny_run.hpp"

using namespace qlin;

extern "C" {

int mi_gemv_int4_multi(const void* x, int nmat, const void* const* w, const void* const* scale,
                       const void* const* zp, void* const* out, const int* N, int M, int K,
                       int act_dtype, void* stream) {
  if (nmat < 1 || nmat > kMaxMat || !w || !scale || !out || !N) return MI_ERR_ARG;
  SkinnyArgs a{};
  a.x = x; a.nmat = nmat; a.M = M; a.K = K;
  for (int i = 0; i < nmat; ++i) {
    if (!scale[i]) return MI_ERR_ARG;
    a.w[i] = w[i]; a.s[i] = scale[i]; a.z[i] = zp ? zp[i] : nullptr; a.out[i] = out[i]; a.N[i] = N[i];
  }
  return run<1, 0>(a, act_dtype, (hipStream_t)stream);
}

int mi_gemv_int4(const void* x, const void* w, const void* scale, const void* zp, void* out, int M,
                 int N, int K, int act_dtype, void* stream) {
  const void* zps[1] = {zp};
  return mi_gemv_int4_multi(x, 1, &w, &scale, zp ? zps : nullptr, &out, &N, M, K, act_dtype, stream);
}

int mi_gemv_q4k(const void* x, const void* ql, const void* scale, const void* qmin, void* out, int M,
                int N, int K, void* stream) {
  if (!scale || !qmin) return MI_ERR_ARG;
  SkinnyArgs a{};
  a.x = x; a.nmat = 1; a.M = M; a.K = K;
  a.w[0] = ql; a.s[0] = scale; a.z[0] = qmin; a.out[0] = out; a.N[0] = N;
  return run<2, 0>(a, DT_F16, (hipStream_t)stream);
}

}  // extern "C"
