// GEMV on 16-bit (unquantized) weights for the small projections that sit next to the
// quantized ones in a decode step (routers, the GDN b/a projection): out = x @ w^T, w [N, K]
// in the activation type, a few activation rows.  One workgroup (4 wavefronts) per output
// row, so that even a 32-row router fills some of the device and K = 2048 is one step:
// every lane reads 16 contiguous bytes of the weight row per step (non-temporal) and the
// matching 16 bytes of each activation row (from L2), accumulates with v_dot2_f32; DPP sums
// inside the wavefronts, LDS across them.  With GELU the workgroup owns gate row n and up
// row n + N of a [2N, K] weight and writes gelu_tanh(gate) * up.
#include "gemv_rows.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

constexpr int kW16Rows = 8;                           // activation rows per pass

template <class Act, bool GELU>
__global__ __launch_bounds__(256) void gemv_w16_kernel(const typename Act::elem* __restrict__ x,
                                                       const typename Act::elem* __restrict__ w,
                                                       typename Act::elem* __restrict__ out, int M, int N, int K) {
  __shared__ float red[2][4][kW16Rows];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = blockIdx.x;
  const int rows_w = GELU ? 2 * N : N;
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(w, (uint32_t)rows_w * (uint32_t)K * 2u);
  const __amdgpu_buffer_rsrc_t xr = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);
  for (int m0 = 0; m0 < M; m0 += kW16Rows) {
    float acc[kW16Rows], acc2[kW16Rows];
#pragma unroll
    for (int m = 0; m < kW16Rows; ++m) { acc[m] = 0.f; acc2[m] = 0.f; }
    for (int k = (int)threadIdx.x * 8; k < K; k += 2048) {
      const u32x4 wg = __builtin_amdgcn_raw_buffer_load_b128(wr, ((uint32_t)n * (uint32_t)K + (uint32_t)k) * 2u, 0, 2);
      u32x4 wu = {0u, 0u, 0u, 0u};
      if constexpr (GELU)
        wu = __builtin_amdgcn_raw_buffer_load_b128(wr, ((uint32_t)(n + N) * (uint32_t)K + (uint32_t)k) * 2u, 0, 2);
      u32x4 xv[kW16Rows];
#pragma unroll
      for (int m = 0; m < kW16Rows; ++m)               // rows past M read zeros through the dead offset
        xv[m] = __builtin_amdgcn_raw_buffer_load_b128(
            xr, m0 + m < M ? ((uint32_t)(m0 + m) * (uint32_t)K + (uint32_t)k) * 2u : 0x80000000u, 0, 0);
#pragma unroll
      for (int m = 0; m < kW16Rows; ++m)
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          acc[m] = Dot2<Act>::run(wg[d], xv[m][d], acc[m]);
          if constexpr (GELU) acc2[m] = Dot2<Act>::run(wu[d], xv[m][d], acc2[m]);
        }
    }
#pragma unroll
    for (int m = 0; m < kW16Rows; ++m) {
      const float v = wave_sum(acc[m]);
      if (lane == 0) red[0][wave][m] = v;
      if constexpr (GELU) {
        const float u = wave_sum(acc2[m]);
        if (lane == 0) red[1][wave][m] = u;
      }
    }
    __syncthreads();
    if ((int)threadIdx.x < kW16Rows && m0 + (int)threadIdx.x < M) {
      const int m = threadIdx.x;
      float v = (red[0][0][m] + red[0][1][m]) + (red[0][2][m] + red[0][3][m]);
      if constexpr (GELU) {
        const float u = (red[1][0][m] + red[1][1][m]) + (red[1][2][m] + red[1][3][m]);
        float two_z = 2.0f * (0.7978845608f * (v + 0.044715f * (v * v * v)));
        two_z = fminf(fmaxf(two_z, -30.0f), 30.0f);
        const float ex = __expf(two_z);
        v = 0.5f * v * (1.0f + (ex - 1.0f) / (ex + 1.0f)) * u;
      }
      out[(size_t)(m0 + m) * N + n] = Act::from_f32(v);
    }
    __syncthreads();                                   // red is rewritten by the next pass
  }
}

}  // namespace qlin

using namespace qlin;

extern "C" {

int mi_gemv_w16(const void* x, const void* w, void* out, int M, int N, int K, int gelu_mul, int act_dtype,
                void* stream) {
  if (!x || !w || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (M < 0 || N <= 0 || K <= 0 || (K % 8)) return MI_ERR_SHAPE;
  if ((uint64_t)N * (gelu_mul ? 2 : 1) * (uint64_t)K * 2 >= (1ull << 32) || (uint64_t)M * (uint64_t)K * 2 >= (1ull << 31))
    return MI_ERR_SHAPE;
  if (!M) return MI_OK;
  const dim3 grid((unsigned)N);
  hipStream_t st = (hipStream_t)stream;
#define QLIN_W16(ACT, T, G) \
  hipLaunchKernelGGL((gemv_w16_kernel<ACT, G>), grid, dim3(256), 0, st, (const T*)x, (const T*)w, (T*)out, M, N, K)
  if (act_dtype == DT_F16) { if (gelu_mul) QLIN_W16(ActF16, _Float16, true); else QLIN_W16(ActF16, _Float16, false); }
  else { if (gelu_mul) QLIN_W16(ActBF16, __bf16, true); else QLIN_W16(ActBF16, __bf16, false); }
#undef QLIN_W16
  return launch_status();
}

}  // extern "C"
