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

// One pass over K for a chunk of MTC 16-row activation tiles.  The weights are the
// MFMA A operand and the activations the B operand, so a lane ends up holding
// ONE activation row (mt*16 + j) and four consecutive weight rows (4 g + v): the
// per-row activation scale is then a single value per lane, tile and granule.
// Granules are software-pipelined through two register buffers; loads of a
// granule (weights first, then activations, then scales) are issued together so
// that the in-order memory counter lets granule i be consumed while granule
// i + 1 is still in flight.
template <class Act, bool A8, int RT, int NW, int MTC>
__device__ __forceinline__ void moe_chunk(const MoeGemmArgs& p, f32x4 (&acc)[RT][4],
                                          __amdgpu_buffer_rsrc_t wr, __amdgpu_buffer_rsrc_t ar,
                                          const float* wsc, const int (&nbase)[RT],
                                          const uint32_t (&wdead)[RT], const uint32_t (&arow)[4],
                                          const uint32_t (&adead)[4], int wave, int j, int g) {
  using V8 = typename Act::v8;
  constexpr int NA = A8 ? 2 : 4;                      // 16-byte loads per activation row per granule
  const int K = p.K;
  const int G = K >> 7;
  const int Kb = G;
  const int Nb = (p.N + 127) >> 7;
  const uint32_t a_esz = A8 ? 1u : 2u;

  struct Frag {
    u32x4 wa[RT], wb[RT];
    u32x4 af[MTC][NA];
    float ws[RT];
    float xs[MTC];
  };
  auto load_frag = [&](Frag& f, int gi) {
    const uint32_t gdead = (uint32_t)(gi >= G) << 31;
    const int gic = gi < G ? gi : G - 1;
    const uint32_t kl = (uint32_t)gic * 128u + (uint32_t)g * 32u;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const uint32_t off = ((uint32_t)(nbase[t] + j) * (uint32_t)K + kl) | wdead[t] | gdead;
      f.wa[t] = __builtin_amdgcn_raw_buffer_load_b128(wr, off, 0, 2);
      f.wb[t] = __builtin_amdgcn_raw_buffer_load_b128(wr, off + 16u, 0, 2);
    }
#pragma unroll
    for (int mt = 0; mt < MTC; ++mt) {
      const uint32_t off = ((arow[mt] * (uint32_t)K + kl) * a_esz) | adead[mt] | gdead;
#pragma unroll
      for (int i = 0; i < NA; ++i) f.af[mt][i] = buf_load16(ar, off + 16u * i);
    }
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int nb = min(nbase[t] >> 7, Nb - 1);
      f.ws[t] = wsc[(size_t)nb * Kb + gic];
    }
    if constexpr (A8) {
#pragma unroll
      for (int mt = 0; mt < MTC; ++mt) f.xs[mt] = p.a_scale[(size_t)arow[mt] * Kb + gic];
    }
  };
  auto compute = [&](const Frag& f) {
    V8 w16[RT][4];
    if constexpr (!A8) {
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        w16[t][0] = fp8x8_to_act<Act>(f.wa[t][0], f.wa[t][1]);
        w16[t][1] = fp8x8_to_act<Act>(f.wa[t][2], f.wa[t][3]);
        w16[t][2] = fp8x8_to_act<Act>(f.wb[t][0], f.wb[t][1]);
        w16[t][3] = fp8x8_to_act<Act>(f.wb[t][2], f.wb[t][3]);
      }
    }
#pragma unroll
    for (int mt = 0; mt < MTC; ++mt) {
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        f32x4 tt = f32x4{0.f, 0.f, 0.f, 0.f};
        if constexpr (A8) {
          const long x0 = (long)(((uint64_t)f.af[mt][0][1] << 32) | f.af[mt][0][0]);
          const long x1 = (long)(((uint64_t)f.af[mt][0][3] << 32) | f.af[mt][0][2]);
          const long x2 = (long)(((uint64_t)f.af[mt][1][1] << 32) | f.af[mt][1][0]);
          const long x3 = (long)(((uint64_t)f.af[mt][1][3] << 32) | f.af[mt][1][2]);
          const long w0 = (long)(((uint64_t)f.wa[t][1] << 32) | f.wa[t][0]);
          const long w1 = (long)(((uint64_t)f.wa[t][3] << 32) | f.wa[t][2]);
          const long w2 = (long)(((uint64_t)f.wb[t][1] << 32) | f.wb[t][0]);
          const long w3 = (long)(((uint64_t)f.wb[t][3] << 32) | f.wb[t][2]);
          tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w0, x0, tt, 0, 0, 0);
          tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w1, x1, tt, 0, 0, 0);
          tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w2, x2, tt, 0, 0, 0);
          tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w3, x3, tt, 0, 0, 0);
          acc[t][mt] += tt * (f.xs[mt] * f.ws[t]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) tt = Act::mfma(w16[t][i], as_v8<V8>(f.af[mt][i]), tt);
          acc[t][mt] += tt * f.ws[t];
        }
      }
    }
  };

  Frag fa, fb;
  int gi = wave;
  load_frag(fa, gi);
  while (gi < G) {
    load_frag(fb, gi + NW);
    compute(fa);
    gi += NW;
    if (gi >= G) break;
    load_frag(fa, gi + NW);
    compute(fb);
    gi += NW;
  }
}

template <class Act, bool A8, bool SILU, int RT, int NW>
__global__ __launch_bounds__(NW * 64) void moe_gemm_kernel(const MoeGemmArgs p) {
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
  const int half = N >> 1;
  // weight rows of this workgroup: tile t covers rows nbase[t] .. +16
  int nbase[RT];
  uint32_t wdead[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if constexpr (SILU) {
      const int col = (tile * (RT / 2) + (t >> 1)) * 16;       // (gate, up) pairs share a column
      nbase[t] = (t & 1) * half + col;
      wdead[t] = (uint32_t)(!(col + j < half)) << 31;
    } else {
      nbase[t] = (tile * RT + t) * 16;
      wdead[t] = (uint32_t)(!(nbase[t] + j < N)) << 31;
    }
  }

  const uint8_t* wexp = (const uint8_t*)p.w + (size_t)e * N * K;
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(wexp, (uint32_t)N * (uint32_t)K);
  const uint32_t a_esz = A8 ? 1u : 2u;
  const __amdgpu_buffer_rsrc_t ar = make_rsrc(p.a, (uint32_t)p.a_rows * (uint32_t)K * a_esz);
  const int Nb = (N + 127) >> 7;
  const float* wsc = p.w_scale + (size_t)e * Nb * (K >> 7);

  for (int mc = 0; mc < cnt; mc += 16 * MT) {
    const int rows_here = min(16 * MT, cnt - mc);
    const int mtiles = (rows_here + 15) >> 4;
    // source row of this lane's activation fragment, per m-tile
    uint32_t arow[MT], adead[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mc + mt * 16 + j;
      const bool ok = m < cnt;
      adead[mt] = (uint32_t)(!ok) << 31;
      const int pos = r0 + (ok ? m : 0);
      arow[mt] = (uint32_t)(p.row_map ? p.row_map[pos] : pos);
    }

    f32x4 acc[RT][MT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    switch (mtiles) {                                  // wave-uniform
      case 1: moe_chunk<Act, A8, RT, NW, 1>(p, acc, wr, ar, wsc, nbase, wdead, arow, adead, wave, j, g); break;
      case 2: moe_chunk<Act, A8, RT, NW, 2>(p, acc, wr, ar, wsc, nbase, wdead, arow, adead, wave, j, g); break;
      case 3: moe_chunk<Act, A8, RT, NW, 3>(p, acc, wr, ar, wsc, nbase, wdead, arow, adead, wave, j, g); break;
      default: moe_chunk<Act, A8, RT, NW, 4>(p, acc, wr, ar, wsc, nbase, wdead, arow, adead, wave, j, g); break;
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
    // D layout: lane holds activation row mt*16 + j and weight rows nbase + 4 g + v
    if (wave == 0) {
      Elem* out = (Elem*)p.out;
      float* out32 = (float*)p.out;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = mc + mt * 16 + j;
        if (m < cnt) {
          const size_t orow = (size_t)(r0 + m) * p.n_out;
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            if constexpr (SILU) {
#pragma unroll
              for (int t = 0; t < RT; t += 2) {
                const int n = nbase[t] + g * 4 + v;      // gate row == output column
                if (n < half) {
                  const float gate = acc[t][mt][v], up = acc[t + 1][mt][v];
                  const float r = gate / (1.0f + expf(-gate)) * up;
                  if (p.out_f32) out32[orow + n] = r; else out[orow + n] = Act::from_f32(r);
                }
              }
            } else {
#pragma unroll
              for (int t = 0; t < RT; ++t) {
                const int n = nbase[t] + g * 4 + v;
                if (n < N) {
                  if (p.out_f32) out32[orow + n] = acc[t][mt][v]; else out[orow + n] = Act::from_f32(acc[t][mt][v]);
                }
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
