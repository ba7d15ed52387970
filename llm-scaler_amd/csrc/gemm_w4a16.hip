// Prefill W4A16 GEMM: out[M,N] = x[M,K] @ dequant(w[N,K])^T, int4 weights in groups of 128 along K
// with fp16 scales and optional per-group zero-points, fp16 / bf16 activations.  The kernel is the
// tiled matrix-core GEMM of gemm_tiled.hpp with the INT4 weight format.
#include "gemm_tiled.hpp"
#include "scratch.hpp"
#include "../../include/mi355x_qlinear.h"

using namespace qlin;

extern "C" {

int mi_gemm_int4_workspace(int M, int N, int K, long long* bytes) {
  if (!bytes) return MI_ERR_ARG;
  if (M < 0 || N < 0 || K <= 0 || (K % 128)) return MI_ERR_SHAPE;
  *bytes = (M <= 64 || !N) ? 0 : (long long)((M + 15) & ~15) * K * 2;
  return MI_OK;
}

int mi_gemm_int4_ws(const void* x, const void* w, const void* scale, const void* zp, void* out,
                    void* workspace, long long workspace_bytes, int M, int N, int K, int act_dtype,
                    void* stream) {
  if (!x || !w || !scale || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (M < 0 || N < 0 || K <= 0 || (K % 128)) return MI_ERR_SHAPE;
  if ((uint64_t)(M + 15) * (uint64_t)K * 2 >= (1ull << 31) || (uint64_t)N * (uint64_t)K / 2 >= (1ull << 31))
    return MI_ERR_SHAPE;
  if (!M || !N) return MI_OK;
  if (M <= 64) return mi_gemv_int4(x, w, scale, zp, out, M, N, K, act_dtype, stream);
  const int Mp = (M + 15) & ~15;
  if (!workspace || workspace_bytes < (long long)Mp * K * 2) return MI_ERR_ARG;
  GemmArgs p{};
  p.w = w; p.scale = scale; p.zp = zp; p.out = out; p.M = M; p.N = N; p.K = K;
  return act_dtype == DT_F16 ? run_gemm_tiled<ActF16, WInt4>(p, x, workspace, (hipStream_t)stream)
                             : run_gemm_tiled<ActBF16, WInt4>(p, x, workspace, (hipStream_t)stream);
}

int mi_gemm_int4(const void* x, const void* w, const void* scale, const void* zp, void* out, int M, int N,
                 int K, int act_dtype, void* stream) {
  long long bytes = 0;
  const int rc = mi_gemm_int4_workspace(M, N, K, &bytes);
  if (rc != MI_OK) return rc;
  if (!bytes) return mi_gemm_int4_ws(x, w, scale, zp, out, nullptr, 0, M, N, K, act_dtype, stream);
  // scratch for the re-tiled activations: this stream's grow-only buffer (the first
  // call of a size allocates; callers that must never allocate pass their own
  // workspace through mi_gemm_int4_ws)
  void* ws = scratch_get((hipStream_t)stream, (size_t)bytes);
  if (!ws) return MI_ERR_LAUNCH;
  return mi_gemm_int4_ws(x, w, scale, zp, out, ws, bytes, M, N, K, act_dtype, stream);
}

}  // extern "C"
