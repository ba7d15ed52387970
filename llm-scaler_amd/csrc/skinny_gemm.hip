// Entry points of the weight-streaming GEMV / small-M GEMM for FP8 (per-channel, per-tensor,
// 128x128 block): M <= 4 takes the one-wavefront-per-row kernel (gemv_rows.hpp), larger M the
// MFMA kernels (kslice_kernel.hpp, skinny_kernel.hpp), M > 64 the tiled GEMM.  The INT4 and
// Q4_K entry points are in skinny_gemm_w4.hip.
#include "skinny_run.hpp"

using namespace qlin;

extern "C" {

int mi_gemm_fp8_pern_multi(const void* x, int nmat, const void* const* w, const void* const* scale,
                           void* const* out, const int* N, int M, int K, int act_dtype,
                           int scale_is_f16, void* stream) {
  if (nmat < 1 || nmat > kMaxMat || !w || !scale || !out || !N) return MI_ERR_ARG;
  SkinnyArgs a{};
  a.x = x; a.nmat = nmat; a.M = M; a.K = K; a.scale_f16 = scale_is_f16;
  for (int i = 0; i < nmat; ++i) {
    if (!scale[i]) return MI_ERR_ARG;
    a.w[i] = w[i]; a.s[i] = scale[i]; a.out[i] = out[i]; a.N[i] = N[i];
  }
  return run<0, SC_PERN>(a, act_dtype, (hipStream_t)stream);
}

int mi_gemm_fp8_pern(const void* x, const void* w, const void* scale, void* out, int M, int N, int K,
                     int act_dtype, int scale_is_f16, void* stream) {
  return mi_gemm_fp8_pern_multi(x, 1, &w, &scale, &out, &N, M, K, act_dtype, scale_is_f16, stream);
}

int mi_gemm_fp8_pert_multi(const void* x, int nmat, const void* const* w, const float* const* scale,
                           void* const* out, const int* N, int M, int K, int act_dtype, void* stream) {
  if (nmat < 1 || nmat > kMaxMat || !w || !scale || !out || !N) return MI_ERR_ARG;
  SkinnyArgs a{};
  a.x = x; a.nmat = nmat; a.M = M; a.K = K;
  for (int i = 0; i < nmat; ++i) {
    if (!scale[i]) return MI_ERR_ARG;
    a.w[i] = w[i]; a.s[i] = scale[i]; a.out[i] = out[i]; a.N[i] = N[i];
  }
  return run<0, SC_PERT>(a, act_dtype, (hipStream_t)stream);
}

int mi_gemm_fp8_pert(const void* x, const void* w, const float* scale, void* out, int M, int N, int K,
                     int act_dtype, void* stream) {
  return mi_gemm_fp8_pert_multi(x, 1, &w, &scale, &out, &N, M, K, act_dtype, stream);
}

int mi_gemm_fp8_blockscale_multi(const void* x, int nmat, const void* const* w,
                                 const float* const* scale, void* const* out, const int* N, int M,
                                 int K, int act_dtype, void* stream) {
  if (nmat < 1 || nmat > kMaxMat || !w || !scale || !out || !N) return MI_ERR_ARG;
  if (K % 128) return MI_ERR_SHAPE;
  SkinnyArgs a{};
  a.x = x; a.nmat = nmat; a.M = M; a.K = K;
  for (int i = 0; i < nmat; ++i) {
    if (!scale[i]) return MI_ERR_ARG;
    a.w[i] = w[i]; a.s[i] = scale[i]; a.out[i] = out[i]; a.N[i] = N[i];
  }
  return run<0, SC_BLOCK>(a, act_dtype, (hipStream_t)stream);
}

int mi_gemm_fp8_blockscale(const void* x, const void* w, const float* scale, void* out, int M, int N,
                           int K, int act_dtype, void* stream) {
  return mi_gemm_fp8_blockscale_multi(x, 1, &w, &scale, &out, &N, M, K, act_dtype, stream);
}

}  // extern "C"
