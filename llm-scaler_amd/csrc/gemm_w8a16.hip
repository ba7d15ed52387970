// Prefill GEMMs on FP8 (per-channel / per-tensor / 128x128 block scales) and GGUF Q4_K weights
// for more than 64 activation rows: the tiled matrix-core GEMM of gemm_tiled.hpp with the FP8
// and Q4_K weight formats.  Each weight byte is read once per 256 (or 128) activation rows
// instead of once per 64 as the weight-streaming kernels would.
#include "gemm_tiled.hpp"
#include "scratch.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

template <class Act, int BN> using WFp8Plain = WFp8<Act, BN, false>;
template <class Act, int BN> using WFp8Block = WFp8<Act, BN, true>;

static inline bool tiled_shape_ok(int M, int N, int K, int wbytes_per_k_num, int wbytes_per_k_den) {
  if (M <= 0 || N <= 0 || K <= 0 || (K % 128)) return false;
  if ((uint64_t)(M + 15) * (uint64_t)K * 2 >= (1ull << 31)) return false;
  return (uint64_t)N * (uint64_t)K * wbytes_per_k_num / wbytes_per_k_den < (1ull << 31);
}

}  // namespace qlin

using namespace qlin;

extern "C" {

int mi_gemm_tiled_workspace(int M, int K, long long* bytes) {
  if (!bytes) return MI_ERR_ARG;
  if (M < 0 || K <= 0) return MI_ERR_SHAPE;
  *bytes = (long long)((M + 15) & ~15) * K * 2;
  return MI_OK;
}

int mi_gemm_fp8_tiled_ws(const void* x, const void* w, const void* scale, int scale_mode, int scale_is_f16,
                         void* out, void* workspace, long long workspace_bytes, int M, int N, int K,
                         int act_dtype, void* stream) {
  if (!x || !w || !scale || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (scale_mode < 0 || scale_mode > 2) return MI_ERR_ARG;
  if (M < 0 || N < 0) return MI_ERR_SHAPE;
  if (!M || !N) return MI_OK;
  if (!tiled_shape_ok(M, N, K, 1, 1)) return MI_ERR_SHAPE;
  if (!workspace || workspace_bytes < (long long)((M + 15) & ~15) * K * 2) return MI_ERR_ARG;
  GemmArgs p{};
  p.w = w; p.scale = scale; p.out = out; p.M = M; p.N = N; p.K = K;
  p.scale_mode = scale_mode; p.scale_f16 = scale_is_f16;
  hipStream_t st = (hipStream_t)stream;
  if (scale_mode == 2)
    return act_dtype == DT_F16 ? run_gemm_tiled<ActF16, WFp8Block>(p, x, workspace, st)
                               : run_gemm_tiled<ActBF16, WFp8Block>(p, x, workspace, st);
  return act_dtype == DT_F16 ? run_gemm_tiled<ActF16, WFp8Plain>(p, x, workspace, st)
                             : run_gemm_tiled<ActBF16, WFp8Plain>(p, x, workspace, st);
}

int mi_gemm_q4k_tiled_ws(const void* x, const void* ql, const void* scale, const void* qmin, void* out,
                         void* workspace, long long workspace_bytes, int M, int N, int K, void* stream) {
  if (!x || !ql || !scale || !qmin || !out) return MI_ERR_ARG;
  if (M < 0 || N < 0) return MI_ERR_SHAPE;
  if (!M || !N) return MI_OK;
  if (!tiled_shape_ok(M, N, K, 1, 2)) return MI_ERR_SHAPE;
  if (!workspace || workspace_bytes < (long long)((M + 15) & ~15) * K * 2) return MI_ERR_ARG;
  GemmArgs p{};
  p.w = ql; p.scale = scale; p.zp = qmin; p.out = out; p.M = M; p.N = N; p.K = K;
  return run_gemm_tiled<ActF16, WQ4K>(p, x, workspace, (hipStream_t)stream);
}

}  // extern "C"
