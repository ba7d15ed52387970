// GPTQ / AWQ style W4A16 operands -> the resident group-128 layout of the INT4 kernels.
//
// The reference's asymmetric W4A16 linear is a third-party op called as
// int4_gemm_w4a16(x, qweight[K/8, N] int32, bias, scales[K/g, N], qzeros, g, g_idx)
// (vllm/patches/vllm_for_multi_arc.patch:5492-5500, AWQ :5002-5010, GPTQ :5080-5088): the
// reduction index is the OUTER one of every operand, and zero-points are packed eight to an
// int32 along N.  The kernels here read weights, scales and zero-points N-major.  These
// kernels turn one into the other on the device, bit for bit:
//   w_out [N, K/8] int32 : w_out[n][i] = qweight[i][n]       (nibble z of a word = element 8i + z, both sides)
//   s_out [N, K/128] fp16: s_out[n][g] = scales[g][n]
//   zp_out[N, K/128] u8  : zp_out[n][g] = ((qzeros[g][n / 8] >> 4 (n % 8)) & 15) + zero_bias,
//                          or qzeros[0] for every (n, g) when the zero-point is one scalar
//                          (the symmetric case, where the caller's qzeros holds the value 8).
#include "qlinear_common.hpp"
#include "../../include/mi355x_qlinear.h"

using namespace qlin;

namespace {

constexpr int kTile = 64;

// int32 matrix transpose through LDS: in [R, C] -> out [C, R]; 64 x 64 tiles, 256 threads
__global__ __launch_bounds__(256) void w4_transpose_kernel(const int32_t* __restrict__ in, int32_t* __restrict__ out,
                                                           int R, int C) {
  __shared__ int32_t tile[kTile][kTile + 1];
  const int c0 = blockIdx.x * kTile, r0 = blockIdx.y * kTile;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < kTile; r += 4) {
    const int rr = r0 + r, cc = c0 + tx;
    if (rr < R && cc < C) tile[r][tx] = in[(size_t)rr * C + cc];
  }
  __syncthreads();
  for (int c = ty; c < kTile; c += 4) {
    const int cc = c0 + c, rr = r0 + tx;
    if (cc < C && rr < R) out[(size_t)cc * R + rr] = tile[tx][c];
  }
}

// scales [G, N] -> [N, G]; zero-points [G, N/8] int32 (or one scalar) -> [N, G] bytes.  One thread per
// (g, n), n fastest, so the reads coalesce; the tables are a few hundred KiB.
__global__ __launch_bounds__(256) void w4_side_kernel(const uint16_t* __restrict__ scales,
                                                      const int32_t* __restrict__ qzeros, int zero_scalar,
                                                      int zero_bias, uint16_t* __restrict__ s_out,
                                                      uint8_t* __restrict__ zp_out, int N, int G) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)N * G) return;
  const int g = (int)(i / N), n = (int)(i % N);
  s_out[(size_t)n * G + g] = scales[i];
  if (zp_out) {
    int z;
    if (zero_scalar) z = qzeros[0];
    else z = ((qzeros[(size_t)g * (N / 8) + (n >> 3)] >> (4 * (n & 7))) & 15) + zero_bias;
    zp_out[(size_t)n * G + g] = (uint8_t)z;
  }
}

template <class Act>
__global__ __launch_bounds__(256) void add_bias_kernel(typename Act::elem* __restrict__ out,
                                                       const typename Act::elem* __restrict__ bias, long total, int N) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  out[i] = Act::from_f32(Act::to_f32(out[i]) + Act::to_f32(bias[i % N]));
}

}  // namespace

extern "C" {

int mi_w4a16_kmajor_prepare(const int32_t* qweight, const void* scales, const int32_t* qzeros, int zero_scalar,
                            int zero_bias, void* w_out, void* s_out, uint8_t* zp_out, int N, int K, void* stream) {
  if (!scales || !s_out) return MI_ERR_ARG;
  if ((zp_out && !qzeros) || (qweight && !w_out)) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 128)) return MI_ERR_SHAPE;
  if (zp_out && !zero_scalar && (N % 8)) return MI_ERR_SHAPE;        // eight zero-points per word along N
  if (zero_bias < 0 || zero_bias > 1) return MI_ERR_ARG;
  if ((uint64_t)N * (uint64_t)K / 2 >= (1ull << 31)) return MI_ERR_SHAPE;
  if (!N) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  const int K8 = K / 8, G = K / 128;
  if (qweight) {
    const dim3 grid((N + kTile - 1) / kTile, (K8 + kTile - 1) / kTile);
    hipLaunchKernelGGL(w4_transpose_kernel, grid, dim3(256), 0, st, qweight, (int32_t*)w_out, K8, N);
  }
  const long total = (long)N * G;
  hipLaunchKernelGGL(w4_side_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, (const uint16_t*)scales,
                     qzeros, zero_scalar, zero_bias, (uint16_t*)s_out, zp_out, N, G);
  return launch_status();
}

int mi_add_bias(void* out, const void* bias, int M, int N, int act_dtype, void* stream) {
  if (!out || !bias) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (M < 0 || N < 0) return MI_ERR_SHAPE;
  const long total = (long)M * N;
  if (!total) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)((total + 255) / 256));
  if (act_dtype == DT_F16)
    hipLaunchKernelGGL(add_bias_kernel<ActF16>, grid, dim3(256), 0, st, (ActF16::elem*)out, (const ActF16::elem*)bias, total, N);
  else
    hipLaunchKernelGGL(add_bias_kernel<ActBF16>, grid, dim3(256), 0, st, (ActBF16::elem*)out, (const ActBF16::elem*)bias, total, N);
  return launch_status();
}

}  // extern "C"
