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

int mi_moe_gemv_fp8_block_routed(const void* x, int x_div, int x_silu, const void* w, const float* w_scale,
                                 void* out, long long out_stride, const int32_t* route_expert,
                                 const void* route_weight, int routes, int num_experts, const void* shared_w,
                                 const float* shared_scale, int shared_rows, int shared_x_first, int N, int K,
                                 int act_dtype, void* stream) {
  if (!x || !w || !w_scale || !out || !route_expert) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (x_div < 1 || num_experts < 1 || x_silu < 0 || x_silu > 1) return MI_ERR_ARG;
  if ((shared_w != nullptr) != (shared_scale != nullptr) || shared_rows < 0 || shared_x_first < 0) return MI_ERR_ARG;
  if (!shared_w) shared_rows = 0;
  if (routes < 0 || N < 0 || K <= 0 || (K % 128) || out_stride < N) return MI_ERR_SHAPE;
  if ((uint64_t)N * (uint64_t)K >= (1ull << 31) || (long)routes + shared_rows > 65535) return MI_ERR_SHAPE;
  if (rows_lds_bytes(RF_FP8, 1, K) > 64 * 1024) return MI_ERR_SHAPE;
  if (!(routes + shared_rows) || !N) return MI_OK;
  RowsArgs r{};
  r.x = x; r.nmat = 1; r.M = 1; r.K = K;
  r.r_expert = route_expert; r.r_out_mul = route_weight; r.r_num_experts = num_experts; r.r_x_div = x_div;
  r.r_out_stride = out_stride;
  r.w[0] = w; r.s[0] = w_scale; r.out[0] = out; r.N[0] = N;
  r.r_w_stride[0] = (long long)N * K;
  r.r_s_stride[0] = (long long)((N + 127) / 128) * (K / 128) * 4;
  if (shared_rows) { r.r_alt_w = shared_w; r.r_alt_s = shared_scale; r.r_alt_from = routes; r.r_alt_x_first = shared_x_first; }
  const int total = routes + shared_rows;
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == DT_F16) {
    if (x_silu) launch_rows_routed<ActF16, RF_FP8, RS_BLOCK, 2>(r, total, st);
    else launch_rows_routed<ActF16, RF_FP8, RS_BLOCK, 1>(r, total, st);
  } else {
    if (x_silu) launch_rows_routed<ActBF16, RF_FP8, RS_BLOCK, 2>(r, total, st);
    else launch_rows_routed<ActBF16, RF_FP8, RS_BLOCK, 1>(r, total, st);
  }
  return launch_status();
}

int mi_gemm_fp8_blockscale(const void* x, const void* w, const float* scale, void* out, int M, int N,
                           int K, int act_dtype, void* stream) {
  return mi_gemm_fp8_blockscale_multi(x, 1, &w, &scale, &out, &N, M, K, act_dtype, stream);
}

}  // extern "C"
