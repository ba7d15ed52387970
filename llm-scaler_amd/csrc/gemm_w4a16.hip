// Prefill W4A16 GEMM for gfx950: out[M,N] = x[M,K] @ dequant(w[N,K])^T, int4
// weights in groups of 128 along K with fp16 scales and optional per-group
// zero-points, fp16 / bf16 activations.
//
// MFMA-bound regime (M in the thousands).  A workgroup of 4 wavefronts (2 x 2)
// owns a BM x BN output tile and walks K in steps of 64.  Per step the
// activation tile is copied global -> registers -> LDS with 128-bit accesses
// and the weight tile is dequantized on the way (the same in-register routines
// the dequant-only kernel uses, so the LDS image holds the bit-exact 16-bit
// weights) — each weight is dequantized once per workgroup and reused by all BM
// rows.  LDS is double buffered: the global loads of step k+1 are issued before
// the MFMAs of step k and written to the other buffer after them, one barrier
// per step.  LDS rows are padded by 16 bytes (row pitch 144 B) so that the
// 16-lane groups of a ds_read_b128 in MFMA operand layout touch 64 distinct
// banks.  Each wavefront computes a (BM/2) x (BN/2) sub-tile with
// v_mfma_f32_16x16x32_{bf16,f16}; the weights are the MFMA A operand, so a lane
// ends up with 4 consecutive output columns of one row and stores them as 8 bytes.
#include "qlinear_common.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

struct GemmArgs {
  const void* x;
  const void* w;
  const void* scale;
  const void* zp;
  void* out;
  int M, N, K;
  int tiles_m, tiles_n;
};

constexpr int kBK = 64;
constexpr int kPitch = kBK + 8;                      // elements per LDS row (144 bytes)

template <class Act, int BM, int BN>
__global__ __launch_bounds__(256) void gemm_w4a16_kernel(const GemmArgs p) {
  using V8 = typename Act::v8;
  using Elem = typename Act::elem;
  constexpr int WM = BM / 2, WN = BN / 2;             // wave sub-tile
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int A_CH = BM * 8 / 256;                  // 16-byte chunks of the x tile per thread
  constexpr int B_CH = BN * 2 / 256;                  // 16-byte chunks (32 nibbles) of the w tile per thread
  static_assert(A_CH >= 1 && B_CH >= 1, "tile too small for 256 threads");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  Elem* As = reinterpret_cast<Elem*>(smem);                                   // [2][BM][kPitch]
  Elem* Bs = As + 2 * BM * kPitch;                                            // [2][BN][kPitch]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 15, g = lane >> 4;
  const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;

  // tile order: consecutive workgroups share the weight tile (same n-tile) so that
  // the 8 XCDs, which take workgroups round-robin, each keep re-using one slab of x
  const int tn = blockIdx.x / p.tiles_m;
  const int tm = blockIdx.x - tn * p.tiles_m;
  const int m0 = tm * BM, n0 = tn * BN;
  const int M = p.M, N = p.N, K = p.K;
  const int Kg = K >> 7;

  const __amdgpu_buffer_rsrc_t xr = make_rsrc(p.x, (uint32_t)M * (uint32_t)K * 2u);
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(p.w, (uint32_t)N * ((uint32_t)K >> 1));
  const _Float16* sc = (const _Float16*)p.scale;
  const uint8_t* zp = (const uint8_t*)p.zp;

  f32x4 acc[TN][TM];
#pragma unroll
  for (int a = 0; a < TN; ++a)
#pragma unroll
    for (int b = 0; b < TM; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 areg[A_CH];
  u32x4 breg[B_CH];
  float bs[B_CH], bz[B_CH];

  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      const int c = tid + i * 256;
      const int row = c >> 3, kc = c & 7;
      const uint32_t dead = (uint32_t)(!(m0 + row < M)) << 31;
      areg[i] = buf_load16(xr, (((uint32_t)(m0 + row) * (uint32_t)K + (uint32_t)(k0 + kc * 8)) * 2u) | dead);
    }
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      const int c = tid + i * 256;
      const int row = c >> 1, kc = c & 1;             // 2 chunks of 32 k per row
      const int n = n0 + row;
      const uint32_t dead = (uint32_t)(!(n < N)) << 31;
      breg[i] = buf_load16(wr, ((uint32_t)n * ((uint32_t)K >> 1) + (uint32_t)((k0 + kc * 32) >> 1)) | dead);
      const int nc = n < N ? n : N - 1;
      const size_t gi = (size_t)nc * Kg + (k0 >> 7);
      bs[i] = (float)sc[gi];
      bz[i] = zp ? (float)zp[gi] : 8.0f;
    }
  };
  auto store_lds = [&](int buf) {
    Elem* Ab = As + buf * BM * kPitch;
    Elem* Bb = Bs + buf * BN * kPitch;
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
      const int c = tid + i * 256;
      const int row = c >> 3, kc = c & 7;
      *reinterpret_cast<u32x4*>(Ab + row * kPitch + kc * 8) = areg[i];
    }
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      const int c = tid + i * 256;
      const int row = c >> 1, kc = c & 1;
      V8* dst = reinterpret_cast<V8*>(Bb + row * kPitch + kc * 32);
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        if constexpr (Act::dt == DT_F16)
          dst[d] = int4x8_to_f16(breg[i][d], (_Float16)bs[i], (_Float16)(1024.0f + bz[i]));
        else
          dst[d] = int4x8_to_bf16(breg[i][d], bs[i], bz[i]);
      }
    }
  };
  auto compute = [&](int buf) {
    const Elem* Ab = As + buf * BM * kPitch;
    const Elem* Bb = Bs + buf * BN * kPitch;
#pragma unroll
    for (int s = 0; s < kBK / 32; ++s) {
      V8 xa[TM], wb[TN];
#pragma unroll
      for (int b = 0; b < TM; ++b)
        xa[b] = *reinterpret_cast<const V8*>(Ab + (wm0 + b * 16 + j) * kPitch + s * 32 + g * 8);
#pragma unroll
      for (int a = 0; a < TN; ++a)
        wb[a] = *reinterpret_cast<const V8*>(Bb + (wn0 + a * 16 + j) * kPitch + s * 32 + g * 8);
#pragma unroll
      for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b) acc[a][b] = Act::mfma(wb[a], xa[b], acc[a][b]);
    }
  };

  const int KT = K / kBK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const bool more = kt + 1 < KT;
    if (more) load_global((kt + 1) * kBK);
    compute(kt & 1);
    if (more) store_lds((kt + 1) & 1);
    __syncthreads();
  }

  // D = W-tile (rows n) x X-tile^T: lane holds n = 4 g + v (v = 0..3), m = j
  Elem* out = (Elem*)p.out;
#pragma unroll
  for (int b = 0; b < TM; ++b) {
    const int m = m0 + wm0 + b * 16 + j;
    if (m < M) {
#pragma unroll
      for (int a = 0; a < TN; ++a) {
        const int n = n0 + wn0 + a * 16 + g * 4;
        Elem v4[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) v4[v] = Act::from_f32(acc[a][b][v]);
        Elem* dst = out + (size_t)m * N + n;
        if (n + 3 < N && (N & 3) == 0) {
          *reinterpret_cast<uint64_t*>(dst) = *reinterpret_cast<const uint64_t*>(v4);
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (n + v < N) dst[v] = v4[v];
        }
      }
    }
  }
}

template <class Act, int BM, int BN>
static int launch_gemm(GemmArgs p, hipStream_t st) {
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const size_t lds = (size_t)2 * (BM + BN) * kPitch * 2;
  auto kern = gemm_w4a16_kernel<Act, BM, BN>;
  if (lds > 64 * 1024) {
    static bool raised = false;                       // opt in to > 64 KiB of dynamic LDS once
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds) != hipSuccess)
        return MI_ERR_LAUNCH;
      raised = true;
    }
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(256), lds, st, p);
  return launch_status();
}

}  // namespace qlin

using namespace qlin;

extern "C" {

int mi_gemm_int4(const void* x, const void* w, const void* scale, const void* zp, void* out, int M, int N,
                 int K, int act_dtype, void* stream) {
  if (!x || !w || !scale || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (M < 0 || N < 0 || K <= 0 || (K % 128)) return MI_ERR_SHAPE;
  if ((uint64_t)M * (uint64_t)K * 2 >= (1ull << 31) || (uint64_t)N * (uint64_t)K / 2 >= (1ull << 31))
    return MI_ERR_SHAPE;
  if (!M || !N) return MI_OK;
  if (M <= 64) return mi_gemv_int4(x, w, scale, zp, out, M, N, K, act_dtype, stream);
  GemmArgs p{};
  p.x = x; p.w = w; p.scale = scale; p.zp = zp; p.out = out; p.M = M; p.N = N; p.K = K;
  hipStream_t st = (hipStream_t)stream;
  const bool big = (long)M * N >= (long)256 * 256 * 256;       // enough 256x256 tiles to fill the chip
  if (act_dtype == DT_F16)
    return big ? launch_gemm<ActF16, 256, 256>(p, st) : launch_gemm<ActF16, 128, 128>(p, st);
  return big ? launch_gemm<ActBF16, 256, 256>(p, st) : launch_gemm<ActBF16, 128, 128>(p, st);
}

}  // extern "C"
