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

// LDS staging geometry.  A wavefront stages one K granule (128 k) of its weight
// tiles and of the expert's activation rows in a private LDS region: global
// loads are row-coalesced (8 or 16 consecutive lanes read one row's contiguous
// 128 / 256 bytes — loading the MFMA operand layout directly, where consecutive
// lanes hit different rows, halves the L1 rate once the activation stream from
// L2 is added to the weight stream), and the operands are then read back in MFMA
// layout.  Rows are padded by 16 bytes so that the 16 lanes of an operand read
// (row stride 144 / 272 bytes) fall into distinct banks.
constexpr int kWPitch = 128 + 16;                    // fp8 weight / activation row of one granule
constexpr int kA16Pitch = 256 + 16;                  // 16-bit activation row of one granule

template <bool A8, int RT>
__host__ __device__ constexpr int moe_stage_bytes() {
  return RT * 16 * kWPitch + 64 * (A8 ? kWPitch : kA16Pitch);
}

// One pass over K for a chunk of MTC 16-row activation tiles.  The weights are the
// MFMA A operand and the activations the B operand, so a lane ends up holding
// ONE activation row (mt*16 + j) and four consecutive weight rows (4 g + v): the
// per-row activation scale is then a single value per lane, tile and granule.
// The global loads of granule i+1 are issued right after granule i has been
// written to LDS, so they are in flight while granule i is multiplied.
template <class Act, bool A8, int RT, int NW, int MTC>
__device__ __forceinline__ void moe_chunk(const MoeGemmArgs& p, f32x4 (&acc)[RT][4],
                                          __amdgpu_buffer_rsrc_t wr, __amdgpu_buffer_rsrc_t ar,
                                          const float* wsc, const int (&nbase)[RT],
                                          const uint32_t (&woff)[RT][2], const uint32_t (&aoff)[16],
                                          const uint32_t (&arow)[4], unsigned char* stage, int wave,
                                          int lane) {
  static_assert(MTC >= 1 && MTC <= 4, "one to four activation tiles");
  using V8 = typename Act::v8;
  constexpr int NAI = A8 ? 2 * MTC : 4 * MTC;         // activation staging loads per granule
  constexpr int APitch = A8 ? kWPitch : kA16Pitch;
  constexpr uint32_t AGran = A8 ? 128u : 256u;        // activation bytes per row per granule
  const int j = lane & 15, g = lane >> 4;
  const int K = p.K;
  const int G = K >> 7;
  const int Kb = G;
  const int Nb = (p.N + 127) >> 7;
  unsigned char* wl = stage;
  unsigned char* al = stage + RT * 16 * kWPitch;
  // staging slots of this lane
  const int wrow = lane >> 3, wch = lane & 7;          // weights and fp8 activations: 8 lanes per row
  const int a16row = lane >> 4, a16ch = lane & 15;     // 16-bit activations: 16 lanes per row

  struct Regs {                                       // one granule in flight
    u32x4 w[RT][2];
    u32x4 a[NAI];
    float ws[RT], xs[MTC];
  };
  // The granule index enters every address as a scalar offset, so a load costs no
  // vector ALU work.  A prefetch past the last granule re-reads the last one
  // (clamped index); its data is never staged.
  const __amdgpu_buffer_rsrc_t xsr = make_rsrc(p.a_scale, A8 ? (uint32_t)p.a_rows * (uint32_t)Kb * 4u : 0u);
  uint32_t xsoff[MTC];
#pragma unroll
  for (int mt = 0; mt < MTC; ++mt) xsoff[mt] = arow[mt] * (uint32_t)Kb * 4u;
  auto load_granule = [&](Regs& r, int gi) {
    const int gic = gi < G ? gi : G - 1;
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int i = 0; i < 2; ++i)
        r.w[t][i] = __builtin_amdgcn_raw_buffer_load_b128(wr, woff[t][i], (uint32_t)gic * 128u, 2);
#pragma unroll
    for (int i = 0; i < NAI; ++i)
      r.a[i] = __builtin_amdgcn_raw_buffer_load_b128(ar, aoff[i], (uint32_t)gic * AGran, 0);
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int nb = min(nbase[t] >> 7, Nb - 1);
      r.ws[t] = wsc[(size_t)nb * Kb + gic];
    }
    if constexpr (A8) {
#pragma unroll
      for (int mt = 0; mt < MTC; ++mt)
        r.xs[mt] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xsr, xsoff[mt], (uint32_t)gic * 4u, 0));
    }
  };
  // stage granule `r` into LDS, start the load of granule `next` into the same
  // registers, then multiply out of LDS
  auto step = [&](Regs& r, int next) {
    float wsc_cur[RT], xsc_cur[MTC];
#pragma unroll
    for (int t = 0; t < RT; ++t) wsc_cur[t] = r.ws[t];
#pragma unroll
    for (int mt = 0; mt < MTC; ++mt) xsc_cur[mt] = A8 ? r.xs[mt] : 1.0f;
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int i = 0; i < 2; ++i)
        *reinterpret_cast<u32x4*>(wl + (t * 16 + wrow + 8 * i) * kWPitch + wch * 16) = r.w[t][i];
#pragma unroll
    for (int i = 0; i < NAI; ++i) {
      if constexpr (A8)
        *reinterpret_cast<u32x4*>(al + (wrow + 8 * i) * APitch + wch * 16) = r.a[i];
      else
        *reinterpret_cast<u32x4*>(al + (a16row + 4 * i) * APitch + a16ch * 16) = r.a[i];
    }
    load_granule(r, next);                            // prefetch; dead beyond the last granule
    // operands back in MFMA layout
    u32x4 wf[RT][2];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int i = 0; i < 2; ++i)
        wf[t][i] = *reinterpret_cast<const u32x4*>(wl + (t * 16 + j) * kWPitch + g * 32 + i * 16);
    V8 w16[RT][4];
    if constexpr (!A8) {
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        w16[t][0] = fp8x8_to_act<Act>(wf[t][0][0], wf[t][0][1]);
        w16[t][1] = fp8x8_to_act<Act>(wf[t][0][2], wf[t][0][3]);
        w16[t][2] = fp8x8_to_act<Act>(wf[t][1][0], wf[t][1][1]);
        w16[t][3] = fp8x8_to_act<Act>(wf[t][1][2], wf[t][1][3]);
      }
    }
#pragma unroll
    for (int mt = 0; mt < MTC; ++mt) {
      if constexpr (A8) {
        const u32x4 x0 = *reinterpret_cast<const u32x4*>(al + (mt * 16 + j) * APitch + g * 32);
        const u32x4 x1 = *reinterpret_cast<const u32x4*>(al + (mt * 16 + j) * APitch + g * 32 + 16);
        const long xa = (long)(((uint64_t)x0[1] << 32) | x0[0]);
        const long xb = (long)(((uint64_t)x0[3] << 32) | x0[2]);
        const long xc = (long)(((uint64_t)x1[1] << 32) | x1[0]);
        const long xd = (long)(((uint64_t)x1[3] << 32) | x1[2]);
#pragma unroll
        for (int t = 0; t < RT; ++t) {
          const long w0 = (long)(((uint64_t)wf[t][0][1] << 32) | wf[t][0][0]);
          const long w1 = (long)(((uint64_t)wf[t][0][3] << 32) | wf[t][0][2]);
          const long w2 = (long)(((uint64_t)wf[t][1][1] << 32) | wf[t][1][0]);
          const long w3 = (long)(((uint64_t)wf[t][1][3] << 32) | wf[t][1][2]);
          f32x4 tt = f32x4{0.f, 0.f, 0.f, 0.f};
          tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w0, xa, tt, 0, 0, 0);
          tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w1, xb, tt, 0, 0, 0);
          tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w2, xc, tt, 0, 0, 0);
          tt = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w3, xd, tt, 0, 0, 0);
          acc[t][mt] += tt * (xsc_cur[mt] * wsc_cur[t]);
        }
      } else {
        V8 xf[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          xf[i] = *reinterpret_cast<const V8*>(al + (mt * 16 + j) * APitch + g * 64 + i * 16);
#pragma unroll
        for (int t = 0; t < RT; ++t) {
          f32x4 tt = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int i = 0; i < 4; ++i) tt = Act::mfma(w16[t][i], xf[i], tt);
          acc[t][mt] += tt * wsc_cur[t];
        }
      }
    }
  };

  // two granules in flight per wavefront
  Regs r0, r1;
  int gi = wave;
  load_granule(r0, gi);
  load_granule(r1, gi + NW);
  while (gi < G) {
    step(r0, gi + 2 * NW);
    gi += NW;
    if (gi >= G) break;
    step(r1, gi + 2 * NW);
    gi += NW;
  }
}

template <class Act, bool A8, bool SILU, int RT, int NW>
__global__ __launch_bounds__(NW * 64) void moe_gemm_kernel(const MoeGemmArgs p) {
  using Elem = typename Act::elem;
  constexpr int MT = 4;                               // up to 64 rows per pass
  constexpr int kStage = moe_stage_bytes<A8, RT>();
  constexpr int kRed = NW * RT * MT * 64 * 16;
  constexpr int kLds = NW * kStage > kRed ? NW * kStage : kRed;
  // the cross-wave reduction buffer overlays the staging regions (used after a barrier)
  __shared__ __attribute__((aligned(16))) unsigned char smem[kLds];
  f32x4 (*red)[RT][MT][64] = reinterpret_cast<f32x4 (*)[RT][MT][64]>(smem);

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
  uint32_t woff[RT][2];                               // staging offsets (granule 0), dead bit for ragged N
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    int col;
    if constexpr (SILU) {
      col = (tile * (RT / 2) + (t >> 1)) * 16;        // (gate, up) pairs share a column
      nbase[t] = (t & 1) * half + col;
    } else {
      col = (tile * RT + t) * 16;
      nbase[t] = col;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = (lane >> 3) + 8 * i;
      const bool ok = col + row < (SILU ? half : N);
      woff[t][i] = ((uint32_t)(nbase[t] + row) * (uint32_t)K + (uint32_t)(lane & 7) * 16u) | ((uint32_t)(!ok) << 31);
    }
  }

  const uint8_t* wexp = (const uint8_t*)p.w + (size_t)e * N * K;
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(wexp, (uint32_t)N * (uint32_t)K);
  const uint32_t a_esz = A8 ? 1u : 2u;
  const __amdgpu_buffer_rsrc_t ar = make_rsrc(p.a, (uint32_t)p.a_rows * (uint32_t)K * a_esz);
  const int Nb = (N + 127) >> 7;
  const float* wsc = p.w_scale + (size_t)e * Nb * (K >> 7);
  unsigned char* stage = smem + wave * kStage;

  for (int mc = 0; mc < cnt; mc += 16 * MT) {
    const int rows_here = min(16 * MT, cnt - mc);
    const int mtiles = (rows_here + 15) >> 4;
    // source rows: in MFMA layout (for the activation scales) and in staging layout
    uint32_t arow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mc + mt * 16 + j;
      const int pos = r0 + (m < cnt ? m : 0);
      arow[mt] = (uint32_t)(p.row_map ? p.row_map[pos] : pos);
    }
    uint32_t aoff[16];
#pragma unroll
    for (int i = 0; i < (A8 ? 8 : 16); ++i) {
      const int row = A8 ? (lane >> 3) + 8 * i : (lane >> 4) + 4 * i;
      const int m = mc + row;
      const bool ok = m < cnt;
      const int pos = r0 + (ok ? m : 0);
      const uint32_t src = (uint32_t)(p.row_map ? p.row_map[pos] : pos);
      const uint32_t ch = A8 ? (uint32_t)(lane & 7) : (uint32_t)(lane & 15);
      aoff[i] = (src * (uint32_t)K * a_esz + ch * 16u) | ((uint32_t)(!ok) << 31);
    }

    f32x4 acc[RT][MT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    switch (mtiles) {                                  // wave-uniform
      case 1: moe_chunk<Act, A8, RT, NW, 1>(p, acc, wr, ar, wsc, nbase, woff, aoff, arow, stage, wave, lane); break;
      case 2: moe_chunk<Act, A8, RT, NW, 2>(p, acc, wr, ar, wsc, nbase, woff, aoff, arow, stage, wave, lane); break;
      case 3: moe_chunk<Act, A8, RT, NW, 3>(p, acc, wr, ar, wsc, nbase, woff, aoff, arow, stage, wave, lane); break;
      default: moe_chunk<Act, A8, RT, NW, 4>(p, acc, wr, ar, wsc, nbase, woff, aoff, arow, stage, wave, lane); break;
    }

    // ---- reduce across the NW wavefronts (buffer overlays the staging regions) ----
    // Every wave deposits its partial tiles; wave w then sums and stores the
    // activation tiles mt = w, w + NW, ... so the epilogue is spread over the
    // whole workgroup instead of serialising on one wave.
    if constexpr (NW > 1) {
      __syncthreads();
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          if (mt < mtiles) red[wave][t][mt][lane] = acc[t][mt];
      __syncthreads();
    }
    // D layout: lane holds activation row mt*16 + j and weight rows nbase + 4 g + v
    {
      Elem* out = (Elem*)p.out;
      float* out32 = (float*)p.out;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = mc + mt * 16 + j;
        const bool mine = (NW == 1) || ((mt % NW) == wave);
        if (mine && mt < mtiles) {
          f32x4 sum[RT];
#pragma unroll
          for (int t = 0; t < RT; ++t) {
            if constexpr (NW > 1) {
              sum[t] = red[0][t][mt][lane];
#pragma unroll
              for (int w = 1; w < NW; ++w) sum[t] += red[w][t][mt][lane];
            } else {
              sum[t] = acc[t][mt];
            }
          }
          if (m < cnt) {
            const size_t orow = (size_t)(r0 + m) * p.n_out;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              if constexpr (SILU) {
#pragma unroll
                for (int t = 0; t < RT; t += 2) {
                  const int n = nbase[t] + g * 4 + v;      // gate row == output column
                  if (n < half) {
                    const float gate = sum[t][v], up = sum[t + 1][v];
                    const float r = gate / (1.0f + __expf(-gate)) * up;
                    if (p.out_f32) out32[orow + n] = r; else out[orow + n] = Act::from_f32(r);
                  }
                }
              } else {
#pragma unroll
                for (int t = 0; t < RT; ++t) {
                  const int n = nbase[t] + g * 4 + v;
                  if (n < N) {
                    if (p.out_f32) out32[orow + n] = sum[t][v]; else out[orow + n] = Act::from_f32(sum[t][v]);
                  }
                }
              }
            }
          }
        }
      }
    }
    if constexpr (NW > 1) __syncthreads();            // the overlay is reused by the next pass
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
