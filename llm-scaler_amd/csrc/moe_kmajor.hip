// Decode MoE on K-major FP8 expert weights, gfx950.
//
// The per-tensor FP8 MoE of the reference keeps the routed experts' weights with the
// reduction index outermost: gate_up [E, H, 2I] and down [E, I, H], one fp32 scale per
// expert.  A weight row is then one k: out[n] = sum_k a[k] * W[k][n] is a sum of scaled
// ROWS, so no lane-to-lane reduction is needed — a lane owns 16 adjacent output columns
// (one 16-byte load per k), a wavefront 1024, and K is what gets split: over the four
// wavefronts of a workgroup (LDS reduction) and over `splits` workgroups, each of which
// stores an fp32 partial row.  The partial rows are added in a fixed order by the
// consumer: the down kernel's prologue sums the up partials, applies the expert scale
// and SiLU(gate) * up (rounded to the activation type, as a stored intermediate would
// be), and the finalize kernel sums the down partials over splits and routes with the
// routing weights and adds the shared expert.  With one token and top-10 routing only
// ten experts are read, so the split over K is what fills the device.
#include "qlinear_common.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

constexpr int kKmWaves = 4;
constexpr int kKmBatch = 8;                           // rows in flight per wavefront

// acc[0..15] += a * (16 e4m3 codes of v)
__device__ __forceinline__ void km_fma16(float (&acc)[16], const u32x4 v, const float a) {
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[d], false);
    const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[d], true);
    acc[4 * d + 0] = fmaf(a, lo[0], acc[4 * d + 0]);
    acc[4 * d + 1] = fmaf(a, lo[1], acc[4 * d + 1]);
    acc[4 * d + 2] = fmaf(a, hi[0], acc[4 * d + 2]);
    acc[4 * d + 3] = fmaf(a, hi[1], acc[4 * d + 3]);
  }
}

// Rows [k_lo, k_hi) of one expert's [K, N] matrix against the multipliers in LDS
// (mult[k - k_lo]); columns [c0 + 16 lane, +16).  The partial row goes to `dst` (fp32, N wide).
// `fill` computes the multipliers into `mult` (it ends with a workgroup barrier); it runs after
// the first batch of weight loads has been issued, so that its own loads wait together with
// them instead of in front of them.
template <class Fill>
__device__ __forceinline__ void km_stream(const uint8_t* __restrict__ wexp, const float* mult, float* red,
                                          float* __restrict__ dst, int k_lo, int k_hi, int N, int c0, Fill&& fill) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = c0 + lane * 16;
  const bool live = col < N;                          // N % 16 == 0: a lane's 16 columns are all in or all out
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(wexp, (uint32_t)k_hi * (uint32_t)N);
  const uint32_t dead = live ? 0u : 0x80000000u;
  float acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  auto load_batch = [&](u32x4 (&v)[kKmBatch], int k0) {
#pragma unroll
    for (int b = 0; b < kKmBatch; ++b) {
      const int k = k0 + b;
      const uint32_t off = k < k_hi ? ((uint32_t)k * (uint32_t)N + (uint32_t)col) | dead : 0x80000000u;
      v[b] = __builtin_amdgcn_raw_buffer_load_b128(wr, off, 0, 2);
    }
  };
  u32x4 v[kKmBatch];
  int k0 = k_lo + wave * kKmBatch;
  load_batch(v, k0);
  __builtin_amdgcn_sched_barrier(0);
  fill();
  for (; k0 < k_hi; k0 += kKmWaves * kKmBatch) {
#pragma unroll
    for (int b = 0; b < kKmBatch; ++b) {
      const int k = k0 + b;
      const float a = k < k_hi ? mult[k - k_lo] : 0.f;
      km_fma16(acc, v[b], a);
    }
    if (k0 + kKmWaves * kKmBatch < k_hi) load_batch(v, k0 + kKmWaves * kKmBatch);
  }
  // reduce the four wavefronts' partial rows through LDS: red[wave][i][lane]
#pragma unroll
  for (int i = 0; i < 16; ++i) red[(wave * 16 + i) * 64 + lane] = acc[i];
  __syncthreads();
  if (wave == 0 && live) {
    float out[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float s = red[i * 64 + lane];
#pragma unroll
      for (int w = 1; w < kKmWaves; ++w) s += red[(w * 16 + i) * 64 + lane];
      out[i] = s;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<f32x4*>(dst + col + 4 * q) = f32x4{out[4 * q], out[4 * q + 1], out[4 * q + 2], out[4 * q + 3]};
  }
}

// grid = routes * splits * column blocks.  partial[route][split][two_i] = sum over the split's
// rows k of x[token][k] * W[e][k][:]   (unscaled)
template <class Act>
__global__ __launch_bounds__(kKmWaves * 64) void km_up_kernel(const typename Act::elem* __restrict__ x,
                                                              const uint8_t* __restrict__ w,
                                                              const int32_t* __restrict__ route_expert,
                                                              float* __restrict__ partial, int top_k, int H,
                                                              int two_i, int splits, int rows_per_split, int cblocks,
                                                              int E) {
  __shared__ float mult[1024];
  __shared__ float red[kKmWaves * 16 * 64];
  const int cb = blockIdx.x % cblocks;
  const int sp = (blockIdx.x / cblocks) % splits;
  const int route = blockIdx.x / (cblocks * splits);
  int e = route_expert[route];
  const bool valid = (unsigned)e < (unsigned)E;       // an id outside [0, E) contributes zeros
  if (!valid) e = 0;
  const int k_lo = sp * rows_per_split;
  const int k_hi = valid ? min(H, k_lo + rows_per_split) : k_lo;
  const typename Act::elem* xr = x + (size_t)(route / top_k) * H;
  km_stream(w + (size_t)e * H * two_i, mult, red, partial + ((size_t)route * splits + sp) * two_i, k_lo, k_hi, two_i,
            cb * 1024, [&]() {
              for (int i = threadIdx.x; i < k_hi - k_lo; i += kKmWaves * 64) mult[i] = Act::to_f32(xr[k_lo + i]);
              __syncthreads();
            });
}

// Activation between a K-major up projection and an N-major down projection:
// inter[route][i] = act(s_e * gate[i]) * (s_e * up[i]), gate / up summed over the up partials in
// split order, the product rounded once to the activation type.  One thread per (route, i).
template <class Act>
__global__ __launch_bounds__(256) void km_act_kernel(const float* __restrict__ up_partial, int up_splits,
                                                      const float* __restrict__ up_scale,
                                                      const int32_t* __restrict__ route_expert,
                                                      typename Act::elem* __restrict__ inter, int I, int iblocks,
                                                      int gelu, int E) {
  const int route = blockIdx.x / iblocks;
  const int i = (blockIdx.x - route * iblocks) * 256 + (int)threadIdx.x;
  if (i >= I) return;
  const int e = route_expert[route];
  float g = 0.f, u = 0.f;
  if ((unsigned)e < (unsigned)E) {                    // a route outside [0, E) yields zeros
    const float* up = up_partial + (size_t)route * up_splits * 2 * I;
    for (int s = 0; s < up_splits; ++s) {
      g += up[(size_t)s * 2 * I + i];
      u += up[(size_t)s * 2 * I + I + i];
    }
    const float se = up_scale[e];
    g *= se;
    u *= se;
  }
  float a;
  if (gelu) {
    float two_z = 2.0f * (0.7978845608f * (g + 0.044715f * (g * g * g)));
    two_z = fminf(fmaxf(two_z, -30.0f), 30.0f);
    const float ex = __expf(two_z);
    a = 0.5f * g * (1.0f + (ex - 1.0f) / (ex + 1.0f));
  } else {
    a = g / (1.0f + __expf(-g));
  }
  inter[(size_t)route * I + i] = Act::from_f32(a * u);
}

// grid = routes * splits * column blocks.  The multipliers are the route's intermediate
// values inter[i] = act(s_e * gate[i]) * (s_e * up[i]), gate / up summed over the up partials,
// rounded to the activation type.  partial[route][split][H] (unscaled by the down scale).
template <class Act>
__global__ __launch_bounds__(kKmWaves * 64) void km_down_kernel(const float* __restrict__ up_partial, int up_splits,
                                                                const float* __restrict__ up_scale,
                                                                const uint8_t* __restrict__ w2,
                                                                const int32_t* __restrict__ route_expert,
                                                                float* __restrict__ partial, int I, int H, int splits,
                                                                int rows_per_split, int cblocks, int gelu, int E) {
  __shared__ float mult[1024];
  __shared__ float red[kKmWaves * 16 * 64];
  const int cb = blockIdx.x % cblocks;
  const int sp = (blockIdx.x / cblocks) % splits;
  const int route = blockIdx.x / (cblocks * splits);
  int e = route_expert[route];
  const bool valid = (unsigned)e < (unsigned)E;
  if (!valid) e = 0;
  const int k_lo = sp * rows_per_split;
  const int k_hi = valid ? min(I, k_lo + rows_per_split) : k_lo;
  const float se = up_scale[e];
  const float* up = up_partial + (size_t)route * up_splits * 2 * I;
  auto fill = [&]() {
  // gate / up sums over the up partials: nq threads share one row (each a strided subset of the
  // splits, eight loads in flight), and the nq sub-sums are added in a fixed order
  __shared__ float gsum[kKmWaves * 64], usum[kKmWaves * 64];
  const int rows = k_hi - k_lo;
  const int nq = rows > 0 && rows <= kKmWaves * 32 ? (kKmWaves * 64) / rows : 1;
  for (int i0 = 0; i0 < rows; i0 += kKmWaves * 64) {
    const int i = i0 + (nq > 1 ? (int)threadIdx.x % rows : (int)threadIdx.x);
    const int q = nq > 1 ? (int)threadIdx.x / rows : 0;
    const bool mine = i < rows && q < nq;
    float g = 0.f, u = 0.f;
    if (mine) {
      for (int s0 = q; s0 < up_splits; s0 += 8 * nq) {
        float gv[8], uv[8];
#pragma unroll
        for (int b = 0; b < 8; ++b) {
          const bool ok = s0 + b * nq < up_splits;
          const size_t row = (size_t)(ok ? s0 + b * nq : 0) * 2 * I + k_lo + i;
          gv[b] = ok ? up[row] : 0.f;
          uv[b] = ok ? up[row + I] : 0.f;
        }
#pragma unroll
        for (int b = 0; b < 8; ++b) { g += gv[b]; u += uv[b]; }
      }
    }
    if (nq > 1) {
      gsum[threadIdx.x] = g;
      usum[threadIdx.x] = u;
      __syncthreads();
      if (q == 0 && i < rows) {
        for (int qq = 1; qq < nq; ++qq) { g += gsum[qq * rows + i]; u += usum[qq * rows + i]; }
      }
    }
    if (q == 0 && i < rows) {
      g *= se;
      u *= se;
      float a;
      if (gelu) {
        float two_z = 2.0f * (0.7978845608f * (g + 0.044715f * (g * g * g)));
        two_z = fminf(fmaxf(two_z, -30.0f), 30.0f);
        const float ex = __expf(two_z);
        a = 0.5f * g * (1.0f + (ex - 1.0f) / (ex + 1.0f));
      } else {
        a = g / (1.0f + __expf(-g));
      }
      mult[i] = Act::to_f32(Act::from_f32(a * u));
    }
  }
  __syncthreads();
  };
  km_stream(w2 + (size_t)e * I * H, mult, red, partial + ((size_t)route * splits + sp) * H, k_lo, k_hi, H, cb * 1024, fill);
}

// out[t][h] = sum_j w[t][j] * s2[e(t,j)] * sum_s partial[(t,j)][s][h]  (+ gate[t] * shared[t][h])
// One workgroup per (token, 256 columns): lane = 4 columns, the (route, split) pairs are dealt
// round-robin to the sixteen wavefronts (eight independent loads in flight each), whose sums are
// added in wave order through LDS, so the result does not depend on timing.
constexpr int kKmFinWaves = 16;
template <class Act>
__global__ __launch_bounds__(kKmFinWaves * 64) void km_finalize_kernel(
    const float* __restrict__ partial, int splits, const float* __restrict__ down_scale,
    const int32_t* __restrict__ route_expert, const typename Act::elem* __restrict__ top_w,
    const typename Act::elem* __restrict__ shared, const float* __restrict__ gate, typename Act::elem* __restrict__ out,
    int T, int top_k, int H, int cblocks, int E) {
  __shared__ f32x4 red[kKmFinWaves][64];
  __shared__ float coef[64];                          // routing weight x down scale per route (top_k <= 64)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int t = blockIdx.x / cblocks;
  const int h = ((blockIdx.x % cblocks) * 64 + lane) * 4;
  const bool live = h < H;
  if ((int)threadIdx.x < top_k) {
    const int route = t * top_k + threadIdx.x;
    const int e = route_expert[route];
    coef[threadIdx.x] = (unsigned)e < (unsigned)E ? Act::to_f32(top_w[route]) * down_scale[e] : 0.f;
  }
  __syncthreads();
  const int pairs = top_k * splits;
  const float* base = partial + (size_t)t * pairs * H + (live ? h : 0);
  f32x4 sum = {0.f, 0.f, 0.f, 0.f};
  for (int p0 = wave; p0 < pairs; p0 += kKmFinWaves * 8) {
    f32x4 v[8];
    float c[8];
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const int p = p0 + kKmFinWaves * b;
      const bool ok = p < pairs;
      const int pc = ok ? p : 0;
      v[b] = *reinterpret_cast<const f32x4*>(base + (size_t)pc * H);
      c[b] = ok ? coef[pc / splits] : 0.f;
    }
#pragma unroll
    for (int b = 0; b < 8; ++b) sum += v[b] * c[b];
  }
  red[wave][lane] = sum;
  __syncthreads();
  if (wave != 0 || !live) return;
  sum = red[0][lane];
#pragma unroll
  for (int w = 1; w < kKmFinWaves; ++w) sum += red[w][lane];
  if (shared) {
    const float gt = gate ? gate[t] : 1.0f;
#pragma unroll
    for (int v = 0; v < 4; ++v) sum[v] += gt * Act::to_f32(shared[(size_t)t * H + h + v]);
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) out[(size_t)t * H + h + v] = Act::from_f32(sum[v]);
}

static int km_rows_per_split(int K, int splits) {
  int rows = (K + splits - 1) / splits;
  return (rows + 7) & ~7;
}

}  // namespace qlin

using namespace qlin;

extern "C" {

int mi_moe_kmajor_up(const void* x, const void* w, const int32_t* route_expert, float* partial, int routes,
                     int top_k, int num_experts, int H, int two_i, int splits, int act_dtype, void* stream) {
  if (!x || !w || !route_expert || !partial) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (routes < 0 || top_k <= 0 || num_experts <= 0 || H <= 0 || two_i <= 0 || (two_i % 32) || splits <= 0) return MI_ERR_SHAPE;
  if ((uint64_t)H * (uint64_t)two_i >= (1ull << 31)) return MI_ERR_SHAPE;
  const int rows = km_rows_per_split(H, splits);
  if (rows > 1024) return MI_ERR_SHAPE;
  if (!routes) return MI_OK;
  const int cblocks = (two_i + 1023) / 1024;
  const dim3 grid((unsigned)routes * splits * cblocks);
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == DT_F16)
    hipLaunchKernelGGL(km_up_kernel<ActF16>, grid, dim3(kKmWaves * 64), 0, st, (const _Float16*)x, (const uint8_t*)w,
                       route_expert, partial, top_k, H, two_i, splits, rows, cblocks, num_experts);
  else
    hipLaunchKernelGGL(km_up_kernel<ActBF16>, grid, dim3(kKmWaves * 64), 0, st, (const __bf16*)x, (const uint8_t*)w,
                       route_expert, partial, top_k, H, two_i, splits, rows, cblocks, num_experts);
  return launch_status();
}

int mi_moe_kmajor_down(const float* up_partial, int up_splits, const float* up_scale, const void* w2,
                       const int32_t* route_expert, float* partial, int routes, int num_experts, int I, int H,
                       int splits, int gelu, int act_dtype, void* stream) {
  if (!up_partial || !up_scale || !w2 || !route_expert || !partial) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (routes < 0 || num_experts <= 0 || up_splits <= 0 || I <= 0 || H <= 0 || (H % 16) || splits <= 0) return MI_ERR_SHAPE;
  if ((uint64_t)H * (uint64_t)I >= (1ull << 31)) return MI_ERR_SHAPE;
  const int rows = km_rows_per_split(I, splits);
  if (rows > 1024) return MI_ERR_SHAPE;
  if (!routes) return MI_OK;
  const int cblocks = (H + 1023) / 1024;
  const dim3 grid((unsigned)routes * splits * cblocks);
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == DT_F16)
    hipLaunchKernelGGL(km_down_kernel<ActF16>, grid, dim3(kKmWaves * 64), 0, st, up_partial, up_splits, up_scale,
                       (const uint8_t*)w2, route_expert, partial, I, H, splits, rows, cblocks, gelu, num_experts);
  else
    hipLaunchKernelGGL(km_down_kernel<ActBF16>, grid, dim3(kKmWaves * 64), 0, st, up_partial, up_splits, up_scale,
                       (const uint8_t*)w2, route_expert, partial, I, H, splits, rows, cblocks, gelu, num_experts);
  return launch_status();
}

int mi_moe_kmajor_act(const float* up_partial, int up_splits, const float* up_scale, const int32_t* route_expert,
                      void* inter, int routes, int num_experts, int I, int gelu, int act_dtype, void* stream) {
  if (!up_partial || !up_scale || !route_expert || !inter) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (routes < 0 || num_experts <= 0 || up_splits <= 0 || I <= 0) return MI_ERR_SHAPE;
  if (!routes) return MI_OK;
  const int iblocks = (I + 255) / 256;
  const dim3 grid((unsigned)routes * iblocks);
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == DT_F16)
    hipLaunchKernelGGL(km_act_kernel<ActF16>, grid, dim3(256), 0, st, up_partial, up_splits, up_scale, route_expert,
                       (_Float16*)inter, I, iblocks, gelu, num_experts);
  else
    hipLaunchKernelGGL(km_act_kernel<ActBF16>, grid, dim3(256), 0, st, up_partial, up_splits, up_scale, route_expert,
                       (__bf16*)inter, I, iblocks, gelu, num_experts);
  return launch_status();
}

int mi_moe_kmajor_finalize(const float* partial, int splits, const float* down_scale, const int32_t* route_expert,
                           const void* top_w, const void* shared, const float* gate, void* out, int T, int top_k,
                           int num_experts, int H, int act_dtype, void* stream) {
  if (!partial || !down_scale || !route_expert || !top_w || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (T < 0 || top_k <= 0 || top_k > 64 || num_experts <= 0 || H <= 0 || (H % 4) || splits <= 0) return MI_ERR_SHAPE;
  if (!T) return MI_OK;
  const int cblocks = (H + 255) / 256;
  const dim3 grid((unsigned)T * cblocks);
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == DT_F16)
    hipLaunchKernelGGL(km_finalize_kernel<ActF16>, grid, dim3(kKmFinWaves * 64), 0, st, partial, splits, down_scale, route_expert,
                       (const _Float16*)top_w, (const _Float16*)shared, gate, (_Float16*)out, T, top_k, H, cblocks, num_experts);
  else
    hipLaunchKernelGGL(km_finalize_kernel<ActBF16>, grid, dim3(kKmFinWaves * 64), 0, st, partial, splits, down_scale, route_expert,
                       (const __bf16*)top_w, (const __bf16*)shared, gate, (__bf16*)out, T, top_k, H, cblocks, num_experts);
  return launch_status();
}

}  // extern "C"
