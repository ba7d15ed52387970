// Dequant-only kernels and the GGUF Q4_K repack.
//
// These materialise the dequantized weights with the very same in-register
// routines the fused GEMV / GEMM kernels use (qlinear_common.hpp), so that
// bit-exactness of the dequantization can be checked directly.  They are also
// the load-time step for callers that want a dense copy.  All are trivially
// HBM-bound elementwise kernels: one lane handles 8 consecutive k.
#include "qlinear_common.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

template <class Act>
__global__ __launch_bounds__(256) void dequant_int4_kernel(const uint32_t* __restrict__ w,
                                                           const _Float16* __restrict__ scale,
                                                           const uint8_t* __restrict__ zp,
                                                           typename Act::v8* __restrict__ out,
                                                           int N, int K) {
  const size_t words = (size_t)N * (K >> 3);
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= words) return;
  const int wpr = K >> 3;
  const int n = (int)(i / wpr);
  const int k = (int)(i % wpr) * 8;
  const size_t gidx = (size_t)n * (K >> 7) + (k >> 7);
  const float s = (float)scale[gidx];
  const float z = zp ? (float)zp[gidx] : 8.0f;
  if constexpr (Act::dt == DT_F16) {
    out[i] = int4x8_to_f16(w[i], (_Float16)s, (_Float16)(1024.0f + z));
  } else {
    out[i] = int4x8_to_bf16(w[i], s, z);
  }
}

// mode: 0 per-channel fp32, 1 per-channel fp16, 2 per-tensor, 3 128x128 block
__global__ __launch_bounds__(256) void dequant_fp8_kernel(const uint8_t* __restrict__ w,
                                                          const void* __restrict__ scale, int mode,
                                                          float* __restrict__ out, int N, int K) {
  const size_t total = (size_t)N * K;
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int n = (int)(i / K), k = (int)(i % K);
  float s;
  if (mode == 0) s = ((const float*)scale)[n];
  else if (mode == 1) s = (float)((const _Float16*)scale)[n];
  else if (mode == 2) s = ((const float*)scale)[0];
  else s = ((const float*)scale)[(size_t)(n >> 7) * ((K + 127) >> 7) + (k >> 7)];
  out[i] = fp8_to_f32(w[i]) * s;
}

template <class Act>
__global__ __launch_bounds__(256) void decode_e4m3_kernel(const u32x2* __restrict__ w,
                                                          typename Act::v8* __restrict__ out,
                                                          size_t groups) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  const u32x2 v = w[i];
  out[i] = fp8x8_to_act<Act>(v[0], v[1]);
}

__global__ __launch_bounds__(256) void dequant_q4k_kernel(const uint32_t* __restrict__ ql,
                                                          const _Float16* __restrict__ scale,
                                                          const _Float16* __restrict__ qmin,
                                                          f16x8* __restrict__ out, int N, int K) {
  const size_t words = (size_t)N * (K >> 3);
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= words) return;
  const int wpr = K >> 3;
  const int n = (int)(i / wpr);
  const int k = (int)(i % wpr) * 8;
  const size_t b = (size_t)n * (K >> 5) + (k >> 5);
  out[i] = q4kx8_to_f16(ql[i], scale[b], qmin[b]);
}

// Raw GGUF block_q4_K {fp16 d, fp16 dmin, u8 scales[12], u8 qs[128]} -> the
// interleaved-nibble representation.  One thread per output byte of ql, plus
// one thread per (row, super-block, sub-block) for scale / min.
__global__ __launch_bounds__(256) void q4k_repack_ql_kernel(const uint8_t* __restrict__ raw,
                                                            uint8_t* __restrict__ ql, int N, int K) {
  const size_t total = (size_t)N * (K >> 1);
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int half = K >> 1;
  const int n = (int)(i / half);
  const int e = (int)(i % half) * 2;                 // first of the two elements
  const int sb = e >> 8, r = e & 255;
  const int il = r >> 6, hi = (r >> 5) & 1, p = r & 31;
  const uint8_t* qs = raw + ((size_t)n * (K >> 8) + sb) * 144 + 16 + 32 * il + p;
  const uint32_t a = qs[0], b = qs[1];
  ql[i] = hi ? (uint8_t)((a >> 4) | ((b >> 4) << 4)) : (uint8_t)((a & 0xF) | ((b & 0xF) << 4));
}

__global__ __launch_bounds__(256) void q4k_repack_sm_kernel(const uint8_t* __restrict__ raw,
                                                            _Float16* __restrict__ scale,
                                                            _Float16* __restrict__ qmin, int N, int K) {
  const size_t total = (size_t)N * (K >> 5);
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int j = (int)(i & 7);
  const uint8_t* blk = raw + (i >> 3) * 144;
  const _Float16 d = *(const _Float16*)(blk);
  const _Float16 dmin = *(const _Float16*)(blk + 2);
  const uint8_t* q = blk + 4;
  uint32_t sc, mn;
  if (j < 4) {
    sc = q[j] & 63u;
    mn = q[j + 4] & 63u;
  } else {
    sc = (q[j + 4] & 0xFu) | ((uint32_t)(q[j - 4] >> 6) << 4);
    mn = (uint32_t)(q[j + 4] >> 4) | ((uint32_t)(q[j] >> 6) << 4);
  }
  scale[i] = (_Float16)((float)d * (float)sc);
  qmin[i] = (_Float16)((float)dmin * (float)mn);
}

static inline dim3 grid1d(size_t n, int bs = 256) { return dim3((unsigned)((n + bs - 1) / bs)); }

}  // namespace qlin

using namespace qlin;

extern "C" {

int mi_dequant_int4(const void* w, const void* scale, const void* zp, void* out, int N, int K,
                    int out_dtype, void* stream) {
  if (!w || !scale || !out) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 128)) return MI_ERR_SHAPE;
  const size_t words = (size_t)N * (K >> 3);
  if (!words) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == DT_F16)
    hipLaunchKernelGGL(dequant_int4_kernel<ActF16>, grid1d(words), dim3(256), 0, st, (const uint32_t*)w,
                       (const _Float16*)scale, (const uint8_t*)zp, (f16x8*)out, N, K);
  else if (out_dtype == DT_BF16)
    hipLaunchKernelGGL(dequant_int4_kernel<ActBF16>, grid1d(words), dim3(256), 0, st, (const uint32_t*)w,
                       (const _Float16*)scale, (const uint8_t*)zp, (bf16x8*)out, N, K);
  else
    return MI_ERR_ARG;
  return launch_status();
}

int mi_dequant_fp8(const void* w, const void* scale, int scale_mode, float* out, int N, int K,
                   void* stream) {
  if (!w || !scale || !out) return MI_ERR_ARG;
  if (scale_mode < 0 || scale_mode > 3) return MI_ERR_ARG;
  if (N < 0 || K <= 0) return MI_ERR_SHAPE;
  const size_t total = (size_t)N * K;
  if (!total) return MI_OK;
  hipLaunchKernelGGL(dequant_fp8_kernel, grid1d(total), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)w, scale, scale_mode, out, N, K);
  return launch_status();
}

int mi_decode_e4m3(const void* codes, void* out, long long count, int out_dtype, void* stream) {
  if (!codes || !out) return MI_ERR_ARG;
  if (count < 0 || (count % 8)) return MI_ERR_SHAPE;
  const size_t groups = (size_t)count / 8;
  if (!groups) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == DT_F16)
    hipLaunchKernelGGL(decode_e4m3_kernel<ActF16>, grid1d(groups), dim3(256), 0, st, (const u32x2*)codes,
                       (f16x8*)out, groups);
  else if (out_dtype == DT_BF16)
    hipLaunchKernelGGL(decode_e4m3_kernel<ActBF16>, grid1d(groups), dim3(256), 0, st, (const u32x2*)codes,
                       (bf16x8*)out, groups);
  else
    return MI_ERR_ARG;
  return launch_status();
}

int mi_dequant_q4k(const void* ql, const void* scale, const void* qmin, void* out, int N, int K,
                   void* stream) {
  if (!ql || !scale || !qmin || !out) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 32)) return MI_ERR_SHAPE;
  const size_t words = (size_t)N * (K >> 3);
  if (!words) return MI_OK;
  hipLaunchKernelGGL(dequant_q4k_kernel, grid1d(words), dim3(256), 0, (hipStream_t)stream,
                     (const uint32_t*)ql, (const _Float16*)scale, (const _Float16*)qmin, (f16x8*)out, N, K);
  return launch_status();
}

int mi_q4k_repack(const void* raw, void* ql, void* scale, void* qmin, int N, int K, void* stream) {
  if (!raw || !ql || !scale || !qmin) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 256)) return MI_ERR_SHAPE;
  if (!N) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(q4k_repack_ql_kernel, grid1d((size_t)N * (K >> 1)), dim3(256), 0, st,
                     (const uint8_t*)raw, (uint8_t*)ql, N, K);
  hipLaunchKernelGGL(q4k_repack_sm_kernel, grid1d((size_t)N * (K >> 5)), dim3(256), 0, st,
                     (const uint8_t*)raw, (_Float16*)scale, (_Float16*)qmin, N, K);
  return launch_status();
}

}  // extern "C"
