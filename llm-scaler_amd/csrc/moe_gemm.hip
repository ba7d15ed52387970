// Grouped (per-expert) FP8 block-scaled GEMM for MoE, gfx950.
//
// Rows arrive expert-contiguous: expert e owns rows [start[e], start[e+1]) of the
// activation matrix (optionally through a row-gather map).  With top-k routing
// over many experts each expert sees only a few dozen rows, so the op is bound
// by streaming every expert's weights once from HBM, not by the matrix cores:
// one workgroup owns (expert, a few 16-row weight tiles) and all of K, its
// wavefronts interleave 128-wide K granules (= one scale block) and reduce
// through LDS, and the expert's rows ride along as MFMA A-operand tiles
// (16 rows each, up to 64 rows per pass).  Workgroups of experts with no rows
// exit at once and read nothing.
//
// Two arithmetic modes:
//   A8  : activations pre-quantised to E4M3 per row per 128-k group (scale xs);
//         native v_mfma_f32_16x16x32_fp8_fp8, and the product of the two block
//         scales is applied to each granule's fp32 partial:
//             acc += (A8 . W8)_granule * xs[row, g] * ws[n / 128, g]
//   A16 : fp16 / bf16 activations (w8a16, the reference's mode): weights are
//         converted exactly to 16 bit and ws is applied to the granule partial.
// Optional fused epilogue: SiLU(gate) * up, where a workgroup pairs weight row n
// (gate) with row n + N/2 (up) and writes N/2 columns.
#include "qlinear_common.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

struct MoeGemmArgs {
  const void* a;              // activations: fp8 [rows, K] (A8) or 16-bit [rows, K]
  const float* a_scale;       // A8: [rows, K/128]
  const int32_t* row_map;     // optional: sorted position -> source row of `a` / `a_scale`
  const void* w;              // [E, N, K] e4m3
  const float* w_scale;       // [E, ceil(N/128), K/128]
  const int32_t* start;       // [E+1]
  void* out;                  // [total_rows, N_out], activation dtype or fp32 (out_f32)
  int out_f32;
  int E, N, K;                // N = weight rows per expert
  int n_out;                  // output columns (N, or N/2 with the fused SiLU*mul)
  int tiles_per_expert;       // workgroups per expert
  int a_rows;                 // rows in `a` (bounds the buffer)
  int total_rows;             // rows in `out`
};

template <class Act, bool A8, bool SILU, int RT, int NW>
__global__ __launch_bounds__(NW * 64) void moe_gemm_kernel(const MoeGemmArgs p) {
  using V8 = typename Act::v8;
  using Elem = typename Act::elem;
  constexpr int MT = 4;                               // up to 64 rows per pass
  __shared__ f32x4 red[NW > 1 ? NW - 1 : 1][RT][MT][64];

  const int e = blockIdx.x / p.tiles_per_expert;
  const int tile = blockIdx.x - e * p.tiles_per_expert;
  const int r0 = p.start[e];
  const int cnt = p.start[e + 1] - r0;
  if (cnt <= 0) return;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15, g = lane >> 4;
  const int K = p.K, N = p.N;
  const int G = K >> 7;
  const int half = N >> 1;
  // weight rows of this workgroup: tile t covers rows nbase[t] .. +16
  int nbase[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if constexpr (SILU)
      nbase[t] = (t & 1) * half + (tile * (RT / 2) + (t >> 1)) * 16;   // (gate, up) pairs
    else
      nbase[t] = (tile * RT + t) * 16;
  }
  const int nlimit = SILU ? half : N;                 // valid column range per tile family

  const uint8_t* wexp = (const uint8_t*)p.w + (size_t)e * N * K;
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(wexp, (uint32_t)N * (uint32_t)K);
  const uint32_t a_esz = A8 ? 1u : 2u;
  const __amdgpu_buffer_rsrc_t ar = make_rsrc(p.a, (uint32_t)p.a_rows * (uint32_t)K * a_esz);
  const int Kb = G;
  const int Nb = (N + 127) >> 7;
  const float* wsc = p.w_scale + (size_t)e * Nb * Kb;

  for (int mc = 0; mc < cnt; mc += 16 * MT) {
    const int rows_here = min(16 * MT, cnt - mc);
    const int mtiles = (rows_here + 15) >> 4;
    // source row of this lane's A fragment, per m-tile
    uint32_t arow[MT];
    bool avalid[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mc + mt * 16 + j;
      avalid[mt] = m < cnt;
      const int pos = r0 + (avalid[mt] ? m : 0);
      arow[mt] = (uint32_t)(p.row_map ? p.row_map[pos] : pos);
    }
    // rows whose activation scale this lane needs in the D layout: mt*16 + 4g + v
    uint32_t srow[MT][4];
    if constexpr (A8) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int m = mc + mt * 16 + g * 4 + v;
          const int pos = r0 + (m < cnt ? m : 0);
          srow[mt][v] = (uint32_t)(p.row_map ? p.row_map[pos] : pos);
        }
    }

    f32x4 acc[RT][MT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int gi = wave; gi < G; gi += NW) {
      const uint32_t kl = (uint32_t)gi * 128u + (uint32_t)g * 32u;
      u32x4 wa[RT], wb[RT];
      float ws[RT];
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const uint32_t n = (uint32_t)(nbase[t] + j);
        const uint32_t dead = (uint32_t)(!((nbase[t] + j - (SILU ? (t & 1) * half : 0)) < nlimit)) << 31;
        const uint32_t off = (n * (uint32_t)K + kl) | dead;
        wa[t] = __builtin_amdgcn_raw_buffer_load_b128(wr, off, 0, 2);
        wb[t] = __builtin_amdgcn_raw_buffer_load_b128(wr, off + 16u, 0, 2);
        const int nb = min(nbase[t] >> 7, Nb - 1);
        ws[t] = wsc[(size_t)nb * Kb + gi];
      }
      // A fragments
      u32x4 af[MT][A8 ? 2 : 4];
      float xs[MT][4];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt < mtiles) {                             // wave-uniform
          const uint32_t dead = (uint32_t)(!avalid[mt]) << 31;
          const uint32_t off = ((arow[mt] * (uint32_t)K + kl) * a_esz) | dead;
#pragma unroll
          for (int i = 0; i < (A8 ? 2 : 4); ++i) af[mt][i] = buf_load16(ar, off + 16u * i);
          if constexpr (A8) {
#pragma unroll
            for (int v = 0; v < 4; ++v) xs[mt][v] = p.a_scale[(size_t)srow[mt][v] * Kb + gi];
          }
        }
      }
      V8 b16[RT][4];
      if constexpr (!A8) {
#pragma unroll
        for (int t = 0; t < RT; ++t) {
          b16[t][0] = fp8x8_to_act<Act>(wa[t][0], wa[t][1]);
          b16[t][1] = fp8x8_to_act<Act>(wa[t][2], wa[t][3]);
          b16[t][2] = fp8x8_to_act<Act>(wb[t][0], wb[t][1]);
          b16[t][3] = fp8x8_to_act<Act>(wb[t][2], wb[t][3]);
        }
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (mt < mtiles) {
#pragma unroll
          for (int t = 0; t < RT; ++t) {
            f32x4 tt = f32x4{0.f, 0.f, 0.f, 0.f};
            if constexpr (A8) {
              const long a0 = (long)(((uint64_t)af[mt][0][1] << 32) | af[mt][0][0]);
              const long a1 = (long)(((uint64_t)af[mt][0][3] << 32) | af[mt][0][2]);
              const long a2 = (long)(((uint64_t)af[mt][1][1] << 32) | af[mt][1][0]);
              const long a3 = (long)(((uint64_t)af[mt][1][3] << 32) | af[mt][1][2]);
              const long b0 = (long)(((uint64_t)wa[t][1] << 32) | wa[t][0]);
              const long b1 = (long)(((uint64_t)wa[t][3] << 32) | wa[t][2]);
              const long b2 = (long)(((uint64_t)wb[t][1] << 32) | wb[t][0]);
              const long b3 = (long)(((uint64_t)wb[t][3] << 32) | wb[t][2]);
              tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a0, b0, tt, 0, 0, 0);
              tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a1, b1, tt, 0, 0, 0);
              tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a2, b2, tt, 0, 0, 0);
              tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a3, b3, tt, 0, 0, 0);
#pragma unroll
              for (int v = 0; v < 4; ++v) acc[t][mt][v] += tt[v] * (xs[mt][v] * ws[t]);
            } else {
#pragma unroll
              for (int i = 0; i < 4; ++i) tt = Act::mfma(as_v8<V8>(af[mt][i]), b16[t][i], tt);
              acc[t][mt] += tt * ws[t];
            }
          }
        }
      }
    }

    // ---- reduce across the NW wavefronts ----
    if constexpr (NW > 1) {
      if (wave > 0) {
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) red[wave - 1][t][mt][lane] = acc[t][mt];
      }
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int w = 0; w < NW - 1; ++w)
#pragma unroll
          for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[t][mt] += red[w][t][mt][lane];
      }
    }
    if (wave == 0) {
      Elem* out = (Elem*)p.out;
      float* out32 = (float*)p.out;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int m = mc + mt * 16 + g * 4 + v;
          if (m < cnt) {
            const size_t orow = (size_t)(r0 + m) * p.n_out;
            if constexpr (SILU) {
#pragma unroll
              for (int t = 0; t < RT; t += 2) {
                const int n = nbase[t] + j;            // gate row == output column
                if (n < half) {
                  const float gate = acc[t][mt][v], up = acc[t + 1][mt][v];
                  const float r = gate / (1.0f + expf(-gate)) * up;
                  if (p.out_f32) out32[orow + n] = r; else out[orow + n] = Act::from_f32(r);
                }
              }
            } else {
#pragma unroll
              for (int t = 0; t < RT; ++t) {
                const int n = nbase[t] + j;
                if (n < N) {
                  if (p.out_f32) out32[orow + n] = acc[t][mt][v]; else out[orow + n] = Act::from_f32(acc[t][mt][v]);
                }
              }
            }
          }
        }
    }
    if constexpr (NW > 1) __syncthreads();            // red[] is reused by the next pass
  }
}

template <class Act, bool A8, bool SILU, int RT, int NW>
static int launch_moe(MoeGemmArgs p, hipStream_t st) {
  const int cols = SILU ? p.N / 2 : p.N;
  const int cols_per_wg = SILU ? (RT / 2) * 16 : RT * 16;
  p.tiles_per_expert = (cols + cols_per_wg - 1) / cols_per_wg;
  p.n_out = cols;
  const long wgs = (long)p.E * p.tiles_per_expert;
  if (wgs <= 0) return MI_OK;
  hipLaunchKernelGGL((moe_gemm_kernel<Act, A8, SILU, RT, NW>), dim3((unsigned)wgs), dim3(NW * 64), 0, st, p);
  return launch_status();
}

template <class Act, bool A8>
static int dispatch_moe(const MoeGemmArgs& p, int fuse_silu, hipStream_t st) {
  // a workgroup should stream on the order of 64 KiB of weights
  if (fuse_silu) return launch_moe<Act, A8, true, 2, 4>(p, st);
  if (p.K <= 1024) return launch_moe<Act, A8, false, 4, 2>(p, st);
  return launch_moe<Act, A8, false, 2, 4>(p, st);
}

}  // namespace qlin

using namespace qlin;

extern "C" {

int mi_moe_gemm_fp8_block(const void* a, const float* a_scale, const int32_t* row_map, const void* w,
                          const float* w_scale, const int32_t* expert_start, void* out, int a_rows,
                          int total_rows, int E, int N, int K, int fuse_silu_mul, int act_dtype,
                          int out_f32, void* stream) {
  if (!a || !w || !w_scale || !expert_start || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (E < 0 || N <= 0 || K <= 0 || (K % 128) || a_rows < 0 || total_rows < 0) return MI_ERR_SHAPE;
  if (fuse_silu_mul && (N % 2)) return MI_ERR_SHAPE;
  if ((uint64_t)N * (uint64_t)K >= (1ull << 31) || (uint64_t)a_rows * (uint64_t)K * 2 >= (1ull << 31))
    return MI_ERR_SHAPE;
  if (!E || !total_rows) return MI_OK;
  MoeGemmArgs p{};
  p.a = a; p.a_scale = a_scale; p.row_map = row_map; p.w = w; p.w_scale = w_scale;
  p.start = expert_start; p.out = out; p.E = E; p.N = N; p.K = K; p.a_rows = a_rows;
  p.total_rows = total_rows;
  p.out_f32 = out_f32;
  hipStream_t st = (hipStream_t)stream;
  if (a_scale) {
    return act_dtype == DT_F16 ? dispatch_moe<ActF16, true>(p, fuse_silu_mul, st)
                               : dispatch_moe<ActBF16, true>(p, fuse_silu_mul, st);
  }
  return act_dtype == DT_F16 ? dispatch_moe<ActF16, false>(p, fuse_silu_mul, st)
                             : dispatch_moe<ActBF16, false>(p, fuse_silu_mul, st);
}

}  // extern "C"
