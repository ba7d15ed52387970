// Weight-streaming ("skinny") quantized GEMV / small-M GEMM for gfx950.
//
// Regime: M <= 64 rows of activations against an [N, K] quantized weight.  The
// weight is read exactly once at full HBM rate; everything else (activations,
// scales) comes out of L2.  One workgroup owns up to 64 output columns (weight
// rows, in 16-row tiles) and all of K; its NW wavefronts interleave 128-wide K granules so that the
// workgroup as a whole walks each weight row front to back, and every lane
// issues 128-bit loads.  Weights are dequantized in registers to the activation
// type and fed to v_mfma_f32_16x16x32_{f16,bf16} with the activations as the A
// operand (M padded to 16 inside the matrix core — free while HBM-bound).  The
// NW partial accumulators are reduced through LDS.
//
// Global loads are row-coalesced: consecutive lanes read one row's contiguous
// bytes of a granule (loading MFMA operand layout directly makes every lane touch
// a different 16-byte piece, and the texture addresser, not HBM, becomes the
// limit), and a wave-private LDS tile turns them into operand layout.  The
// weights always take this path (non-temporal loads); the activations from 17 rows
// on — up to 16 rows their direct loads are cheaper than the extra LDS traffic
// (INT4, N = 14336, K = 4096: 12.7 against 13.5 us at M = 8; 17.7 against 16.6 us at
// M = 32, 11.9 against 9.8 us for N = 4096).
//
// Lane mapping inside one granule (128 k): lane = (j = lane % 16, g = lane / 16)
// holds the 32 consecutive k  [128 gi + 32 g, +32)  of weight row n0 + j and of
// activation row j.  MFMA i (0..3) consumes the i-th 8-k slice of both.
#pragma once
#include "qlinear_common.hpp"
#include "gemv_rows.hpp"

namespace qlin {

constexpr int kMaxMat = 3;
constexpr int kSkinnyXLdsFrom = 2;                  // 16-row activation tiles from which x is staged through LDS
constexpr bool kXLdsOf(int mt) { return mt >= kSkinnyXLdsFrom; }

struct SkinnyArgs {
  const void* x;
  const void* w[kMaxMat];
  const void* s[kMaxMat];     // scales (format specific)
  const void* z[kMaxMat];     // int4: zero-points (may be null); q4k / q5k: mins
  const void* h[kMaxMat];     // q5k / q6k: tile-shuffled high bits
  void* out[kMaxMat];
  int N[kMaxMat];
  int tiles[kMaxMat];         // 16-row tiles per matrix
  int nmat;
  int M, K;
  int rpw;                    // weight rows owned by one workgroup (<= 16 RT)
  int scale_f16;              // fp8 per-channel: scale is fp16 instead of fp32
  // msplit > 1: the rows of x are split over msplit workgroups per weight row block (16 MT rows
  // each); tiles_total = row blocks of all matrices.
  int msplit, tiles_total;
  // Grouped launches (GRP instantiations): one (expert, first row, rows) triple per chunk; the
  // chunk's rows of x are rows t0 .. t0 + nt - 1, or tok_ids[t0 ..] when given; output row t0 + m,
  // out_stride elements apart; the expert's tables sit *_stride bytes after the previous expert's.
  const int32_t* chunks;
  const int32_t* tok_ids;
  int num_chunks, num_experts, x_rows, out_rows;
  int cgroup;                 // consecutive chunks that share an XCD (>= 1)
  long long out_stride, w_stride, s_stride, z_stride, h_stride;
};

enum : int { SC_PERN = 0, SC_PERT = 1, SC_BLOCK = 2 };

// ---------------------------------------------------------------- kernel
// FMT: 0 = fp8 (SC selects the scale mode), 1 = int4 g128, 2 = Q4_K repacked, 3 = Q4_0,
// 4 = Q8_0, 5 = Q5_K, 6 = Q6_K (the GGUF formats in their repacked representation, fp16);
// 7 = Q5_K, 8 = Q6_K with the high bits in element order (the MoE down stacks: Q5_K byte j bit b =
// fifth bit of element 8j + b, Q6_K byte j field p = top two bits of element 4j + p).
// MT = 16-row activation tiles (M <= 16 MT), RT = 16-row weight tiles per
// workgroup, NW = wavefronts splitting K, UN = granules in flight per wave.
// SL: the scales (and mins / zero-points) of the workgroup's rows are staged once in LDS instead
// of being fetched per tile and granule with scattered 16-bit loads: per-32 tables for Q4_K,
// Q5_K, Q4_0, Q8_0 (needs K % 256 == 0), per-128 tables for INT4; chosen when the tables fit
// beside the staging tiles.
// GRP: the grid is (row blocks x chunks), see SkinnyArgs; all workgroups of a chunk run on one XCD.
// The body: `tile` = row block over all matrices, m0 = first row of x (dense), {eid, t0, mrows} = the chunk (GRP).
template <class Act, int FMT, int SC, int MT, int RT, int NW, int UN, bool SL, bool GRP>
__device__ __forceinline__ void skinny_body(const SkinnyArgs& a, int tile, const int m0, const int eid, const int t0,
                                            const int mrows) {
  using V8 = typename Act::v8;
  using Elem = typename Act::elem;
  constexpr bool kIsFp8 = (FMT == 0);
  constexpr bool kIsInt4 = (FMT == 1);
  constexpr bool kIsQ4K = (FMT == 2);
  constexpr bool kIsQ40 = (FMT == 3);
  constexpr bool kIsQ80 = (FMT == 4);
  constexpr bool kIsQ5K = (FMT == 5 || FMT == 7);
  constexpr bool kIsQ6K = (FMT == 6 || FMT == 8);
  constexpr bool kPlainH = (FMT == 7 || FMT == 8);    // high bits in element order
  constexpr bool kByteW = kIsFp8 || kIsQ80;           // one byte per weight: 128 bytes per row and granule
  constexpr bool kHigh = kIsQ5K || kIsQ6K;            // extra high bits per weight
  constexpr bool kBlock = kIsFp8 && SC == SC_BLOCK;
  constexpr bool kSide32 = kIsQ4K || kIsQ5K || kIsQ40 || kIsQ80;   // one fp16 scale per 32 k
  constexpr bool kHasMin = kIsQ4K || kIsQ5K;
  static_assert(!SL || kSide32 || kIsInt4, "LDS-staged scales are for the formats with per-32 or per-128 scales");

  // wave-private staging tiles for the weights (one 16-row tile = 16 rows of one
  // granule, padded pitch); the cross-wave reduction buffer overlays them at the end
  constexpr int kWRowB = kByteW ? 128 : 64;           // weight bytes per row per granule
  constexpr int kWP = kWRowB + 16;                    // LDS pitch: operand reads hit distinct banks
  constexpr int kXP = 256 + 16;                       // activation tile pitch
  constexpr bool kXLds = MT >= kSkinnyXLdsFrom;                    // stage the activations through LDS too
  constexpr int kWStage = NW * RT * 16 * kWP;         // activation tiles follow the weight tiles
  constexpr int kTiles = kWStage + (kXLds ? NW * 16 * kXP : 0);   // one tile per wavefront, reused by its MT tiles; SL: the scale tables follow
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  f32x4 (*red)[RT][MT][64] = reinterpret_cast<f32x4 (*)[RT][MT][64]>(smem);

  int mat = 0;
#pragma unroll
  for (int i = 0; i + 1 < kMaxMat; ++i) {
    if (mat == i && i + 1 < a.nmat && tile >= a.tiles[i]) { tile -= a.tiles[i]; mat = i + 1; }
  }
  const int N = a.N[mat];
  const int K = a.K, M = GRP ? mrows : min(a.M - m0, MT * 16);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int j = lane & 15, g = lane >> 4;
  const int n0 = tile * a.rpw;
  const int nend = min(N, n0 + a.rpw);                // rows past it belong to the next workgroup
  const int G = (K + 127) >> 7;

  const uint32_t wrow = kByteW ? (uint32_t)K : ((uint32_t)K >> 1);
  const uint32_t hrow = kIsQ5K ? ((uint32_t)K >> 3) : ((uint32_t)K >> 2);   // high-bit bytes per row
  // the expert's tables (GRP); null stays null
  const char* hbase = (const char*)a.h[mat];
  const char* wbase = (const char*)a.w[mat];
  const char* sbase = (const char*)a.s[mat];
  const char* zbase = (const char*)a.z[mat];
  if constexpr (GRP) {
    wbase += (long long)eid * a.w_stride;
    sbase += (long long)eid * a.s_stride;
    if (zbase) zbase += (long long)eid * a.z_stride;
    if (hbase) hbase += (long long)eid * a.h_stride;
  }
  const __amdgpu_buffer_rsrc_t hr = make_rsrc(hbase, kHigh ? (uint32_t)N * hrow : 0u);
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(wbase, (uint32_t)N * wrow);
  const __amdgpu_buffer_rsrc_t xr = GRP ? make_rsrc(a.x, (uint32_t)a.x_rows * (uint32_t)K * 2u)
                                        : make_rsrc((const char*)a.x + (size_t)m0 * K * 2, (uint32_t)M * (uint32_t)K * 2u);
  // GRP: byte offset of the row of x behind each row slot this lane loads (past the end: reads zeros)
  constexpr int kXSlots = kXLdsOf(MT) ? 4 : 1;
  uint32_t xro[MT][kXSlots];
  if constexpr (GRP) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < kXSlots; ++i) {
        const int m = mt * 16 + (kXLdsOf(MT) ? (lane >> 4) + 4 * i : j);
        const int pos = t0 + min(m, M - 1);
        const int tok = a.tok_ids ? a.tok_ids[pos] : pos;
        xro[mt][i] = (m < M && tok >= 0 && tok < a.x_rows) ? (uint32_t)tok * (uint32_t)K * 2u : kOOB;
      }
  }

  const _Float16* s16 = (const _Float16*)sbase;
  const float* s32 = (const float*)sbase;
  const uint8_t* zp = (const uint8_t*)zbase;
  const _Float16* qmin = (const _Float16*)zbase;
  const int Kg = K >> 7;                             // int4 groups per row
  const int Kb32 = K >> 5;                           // q4k sub-blocks per row
  const int Kb = G;                                  // fp8 block columns

  f32x4 acc[RT][MT];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // FP8 per-channel / per-tensor: the output scales of the columns this wavefront finishes (see the
  // end), requested first of all and kept as raw bits; fetched where they are used they are one more
  // round trip at the very end of the launch.
  constexpr int kOutIters = (RT * MT + NW - 1) / NW;
  uint32_t os_raw[kOutIters];
#pragma unroll
  for (int it = 0; it < kOutIters; ++it) os_raw[it] = 0;
  float os_pert = 1.0f;
  if constexpr (kIsFp8 && SC == SC_PERT) os_pert = s32[0];
  if constexpr (kIsFp8 && SC == SC_PERN) {
#pragma unroll
    for (int it = 0; it < kOutIters; ++it) {
      const int n = min(n0 + ((wave + it * NW) / MT) * 16 + j, N - 1);
      os_raw[it] = a.scale_f16 ? (uint32_t)reinterpret_cast<const uint16_t*>(s16)[n] : reinterpret_cast<const uint32_t*>(s32)[n];
    }
  }

  // Out-of-range granules / lanes / rows load zeros for both operands, so the
  // loop body needs no branches: a zero weight times a zero activation adds 0.
  //
  // A stage = U granules of this wavefront (gbase, gbase + NW, ...): their loads, and
  // later their conversion + MFMAs.  With UN >= 2 the granules of a turn are split into
  // two stages in a ring, so that the loads of the next stage are in flight while the
  // current one is consumed (continuous streaming instead of load bursts).
  constexpr int US = UN >= 2 ? UN / 2 : UN;           // granules per stage
  struct Stage {
    u32x4 wa[US][RT], wb[US][RT];
    u32x4 xa[US][MT][4];
    u32x4 ha[US][RT][(kHigh && !kPlainH) ? 2 : 1];    // q5k / q6k: the lane's 32 high-bit bytes (element order: 4 / 8 bytes)
    uint32_t sc[US][RT];                              // raw bits: int4 / q4k scale (fp16), block scale (fp32)
    uint32_t zz[US][RT];                              // raw: int4 zero-point byte / q4k min (fp16)
  };
  const uint16_t* s16u = reinterpret_cast<const uint16_t*>(s16);
  const uint16_t* qminu = reinterpret_cast<const uint16_t*>(qmin);
  const uint8_t* zsrc = zp ? zp : reinterpret_cast<const uint8_t*>(s16);   // always a readable address
  const bool has_zp = zp != nullptr;

  auto load_stage = [&](Stage& st, int gbase) {
#pragma unroll
    for (int u = 0; u < US; ++u) {
      const int gi = gbase + u * NW;
      const int kl = gi * 128 + g * 32;
      const bool ok = (gi < G) && (kl < K);
      const int gic = gi < G ? gi : G - 1;
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        const int n = n0 + t * 16 + j;
        const int nc = n < N ? n : N - 1;
        // weights: row-coalesced (consecutive lanes read one row's contiguous bytes);
        // they are turned into operand layout through LDS before use
        if constexpr (kByteW) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int r = (lane >> 3) + 8 * h, c = lane & 7;
            const int nr = n0 + t * 16 + r;
            const bool okw = gi < G && gi * 128 + c * 16 < K && nr < nend;
            // non-temporal: the weights are used once and should not displace x in L2
            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(
                wr, okw ? (uint32_t)nr * wrow + (uint32_t)(gi * 128 + c * 16) : kOOB, 0, 2);
            if (h == 0) st.wa[u][t] = v; else st.wb[u][t] = v;
          }
        } else {
          const int r = lane >> 2, c = lane & 3;
          const int nr = n0 + t * 16 + r;
          const bool okw = gi < G && gi * 128 + c * 32 < K && nr < nend;
          st.wa[u][t] = __builtin_amdgcn_raw_buffer_load_b128(
              wr, okw ? (uint32_t)nr * wrow + (uint32_t)(gi * 64 + c * 16) : kOOB, 0, 2);
        }
        // side data stays raw until it is used: a conversion here would wait for the load,
        // and with it for every older load in flight
        if constexpr (kIsInt4 && !SL) {
          st.sc[u][t] = s16u[(size_t)nc * Kg + gic];
          st.zz[u][t] = zsrc[(size_t)nc * Kg + gic];
        } else if constexpr (SL) {
          // read from the LDS tables when the stage is consumed
        } else if constexpr (kIsQ4K || kIsQ5K) {
          const int sb = gic * 4 + g;
          const int sbc = sb < Kb32 ? sb : Kb32 - 1;
          st.sc[u][t] = s16u[(size_t)nc * Kb32 + sbc];
          st.zz[u][t] = qminu[(size_t)nc * Kb32 + sbc];
        } else if constexpr (kIsQ40 || kIsQ80) {
          const int sb = gic * 4 + g;
          const int sbc = sb < Kb32 ? sb : Kb32 - 1;
          st.sc[u][t] = s16u[(size_t)nc * Kb32 + sbc];
        } else if constexpr (kIsQ6K) {
          // two 16-wide groups per lane: both fp16 scales in one 32-bit load
          const int sb = gic * 4 + g;
          const int sbc = sb < Kb32 ? sb : Kb32 - 1;
          st.sc[u][t] = reinterpret_cast<const uint32_t*>(s16)[(size_t)nc * Kb32 + sbc];
        } else if constexpr (kBlock) {
          st.sc[u][t] = reinterpret_cast<const uint32_t*>(s32)[(size_t)(min(n0 + t * 16, N - 1) >> 7) * Kb + gic];
        }
        if constexpr (kHigh) {
          if constexpr (kPlainH) {
            // element order: this lane's 32 consecutive k are 4 (Q5_K) or 8 (Q6_K) consecutive bytes
            const uint32_t ho = ok && n < nend ? (uint32_t)n * hrow + (uint32_t)gic * (kIsQ5K ? 16u : 32u) + (uint32_t)g * (kIsQ5K ? 4u : 8u) : kOOB;
            if constexpr (kIsQ5K) {
              st.ha[u][t][0] = u32x4{__builtin_amdgcn_raw_buffer_load_b32(hr, ho, 0, 0), 0u, 0u, 0u};
            } else {
              const u32x2 two = __builtin_amdgcn_raw_buffer_load_b64(hr, ho, 0, 0);
              st.ha[u][t][0] = u32x4{two[0], two[1], 0u, 0u};
            }
          } else {
          // per 512-k tile the high bits of element b*64 + t' (Q5_K) / p*128 + t' (Q6_K) sit in
          // byte t': this lane's 32 consecutive k are 32 consecutive bytes, one bit field
          const uint32_t tile = (uint32_t)gic >> 2;
          const uint32_t within = kIsQ5K ? ((uint32_t)g & 1u) * 32u : (uint32_t)g * 32u;
          const uint32_t ho = ok && n < nend ? (uint32_t)n * hrow + tile * (kIsQ5K ? 64u : 128u) + within : kOOB;
          st.ha[u][t][0] = __builtin_amdgcn_raw_buffer_load_b128(hr, ho, 0, 0);
          st.ha[u][t][1] = __builtin_amdgcn_raw_buffer_load_b128(hr, ho == kOOB ? kOOB : ho + 16u, 0, 0);
          }
        }
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if constexpr (kXLds) {
          // many rows: row-coalesced as well (16 lanes read one row's 256 contiguous
          // bytes of the granule), transposed through LDS before use
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int r = (lane >> 4) + 4 * i, c = lane & 15;
            const int m = mt * 16 + r;
            const bool okx = gi < G && gi * 128 + c * 8 < K && m < M;
            if constexpr (GRP) st.xa[u][mt][i] = buf_load16(xr, okx ? xro[mt][i] + (uint32_t)(gi * 128 + c * 8) * 2u : kOOB);
            else st.xa[u][mt][i] = buf_load16(xr, okx ? ((uint32_t)m * (uint32_t)K + (uint32_t)(gi * 128 + c * 8)) * 2u : kOOB);
          }
        } else {
          // few rows: straight into operand layout (lane (j, g): row j, 32 consecutive k)
          const uint32_t xoff = !ok ? kOOB : (GRP ? xro[mt][0] + (uint32_t)kl * 2u : ((uint32_t)(mt * 16 + j) * (uint32_t)K + (uint32_t)kl) * 2u);
#pragma unroll
          for (int i = 0; i < 4; ++i) st.xa[u][mt][i] = buf_load16(xr, ok ? xoff + 16u * i : kOOB);
        }
      }
    }
  };

  auto compute_stage = [&](Stage& st, int gbase_of_stage) {
#pragma unroll
    for (int u = 0; u < US; ++u) {
      // activations through this wavefront's staging tile into MFMA operand layout:
      // lane (j, g) ends up with row j, k = 32 g + 8 i .. + 7 of the granule
#pragma unroll
      for (int mt = 0; mt < (kXLds ? MT : 0); ++mt) {
        unsigned char* xl = smem + kWStage + wave * 16 * kXP;   // the wavefront's LDS operations retire in order
#pragma unroll
        for (int i = 0; i < 4; ++i)
          *reinterpret_cast<u32x4*>(xl + ((lane >> 4) + 4 * i) * kXP + (lane & 15) * 16) = st.xa[u][mt][i];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          st.xa[u][mt][i] = *reinterpret_cast<const u32x4*>(xl + j * kXP + g * 64 + i * 16);
      }
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        // through this wavefront's staging tile into MFMA operand layout
        unsigned char* wl = smem + (wave * RT + t) * 16 * kWP;
        u32x4 wa = st.wa[u][t], wb = st.wb[u][t];
        if constexpr (kByteW) {
          *reinterpret_cast<u32x4*>(wl + (lane >> 3) * kWP + (lane & 7) * 16) = wa;
          *reinterpret_cast<u32x4*>(wl + ((lane >> 3) + 8) * kWP + (lane & 7) * 16) = wb;
          wa = *reinterpret_cast<const u32x4*>(wl + j * kWP + g * 32);
          wb = *reinterpret_cast<const u32x4*>(wl + j * kWP + g * 32 + 16);
        } else {
          *reinterpret_cast<u32x4*>(wl + (lane >> 2) * kWP + (lane & 3) * 16) = wa;
          wa = *reinterpret_cast<const u32x4*>(wl + j * kWP + g * 16);
        }
        if constexpr (SL && kIsInt4) {
          const int gq = min(gbase_of_stage + u * NW, Kg - 1);
          const uint16_t* ts = reinterpret_cast<const uint16_t*>(smem + kTiles);
          const uint8_t* tz = reinterpret_cast<const uint8_t*>(ts + RT * 16 * Kg);
          st.sc[u][t] = ts[(t * 16 + j) * Kg + gq];
          st.zz[u][t] = tz[(t * 16 + j) * Kg + gq];
        } else if constexpr (SL) {
          const int gi_here = gbase_of_stage + u * NW;
          const int sb = min(gi_here * 4 + g, Kb32 - 1);
          const uint16_t* tab = reinterpret_cast<const uint16_t*>(smem + kTiles);
          st.sc[u][t] = tab[(t * 16 + j) * Kb32 + sb];
          if constexpr (kHasMin) st.zz[u][t] = tab[(RT * 16 + t * 16 + j) * Kb32 + sb];
        }
        V8 b[4];
        float scf = 0.f;
        if constexpr (kIsFp8) {
          b[0] = fp8x8_to_act<Act>(wa[0], wa[1]);
          b[1] = fp8x8_to_act<Act>(wa[2], wa[3]);
          b[2] = fp8x8_to_act<Act>(wb[0], wb[1]);
          b[3] = fp8x8_to_act<Act>(wb[2], wb[3]);
          if constexpr (kBlock) scf = __builtin_bit_cast(float, st.sc[u][t]);
        } else if constexpr (kIsInt4) {
          const float sf = (float)__builtin_bit_cast(_Float16, (uint16_t)st.sc[u][t]);
          const float zf = has_zp ? (float)st.zz[u][t] : 8.0f;
          if constexpr (Act::dt == DT_F16) {
            const _Float16 s = (_Float16)sf;
            const _Float16 z = (_Float16)(1024.0f + zf);
#pragma unroll
            for (int i = 0; i < 4; ++i) b[i] = int4x8_to_f16(wa[i], s, z);
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) b[i] = int4x8_to_bf16(wa[i], sf, zf);
          }
        } else if constexpr (kIsQ4K) {
          if constexpr (Act::dt == DT_F16) {
            const _Float16 s = __builtin_bit_cast(_Float16, (uint16_t)st.sc[u][t]);
            const _Float16 mn = __builtin_bit_cast(_Float16, (uint16_t)st.zz[u][t]);
#pragma unroll
            for (int i = 0; i < 4; ++i) b[i] = q4kx8_to_f16(wa[i], s, mn);
          }
        } else if constexpr (kIsQ40) {
          if constexpr (Act::dt == DT_F16) {
            const _Float16 s = __builtin_bit_cast(_Float16, (uint16_t)st.sc[u][t]);
#pragma unroll
            for (int i = 0; i < 4; ++i) b[i] = int4x8_to_f16(wa[i], s, (_Float16)1032.0f);   // (nib - 8) * d
          }
        } else if constexpr (kIsQ80) {
          if constexpr (Act::dt == DT_F16) {
            const _Float16 s = __builtin_bit_cast(_Float16, (uint16_t)st.sc[u][t]);
            b[0] = i8x8_to_f16(wa[0], wa[1], s);
            b[1] = i8x8_to_f16(wa[2], wa[3], s);
            b[2] = i8x8_to_f16(wb[0], wb[1], s);
            b[3] = i8x8_to_f16(wb[2], wb[3], s);
          }
        } else if constexpr (kHigh) {
          if constexpr (Act::dt == DT_F16) {
            // granule gi of its 512-k tile: Q5_K bit 2 (gi % 4) + g / 2, Q6_K field gi % 4
            const int gi_here = gbase_of_stage + u * NW;
            const uint32_t shift = kIsQ5K ? (uint32_t)((gi_here & 3) * 2 + (g >> 1)) : (uint32_t)((gi_here & 3) * 2);
            const _Float16 s0 = __builtin_bit_cast(_Float16, (uint16_t)(st.sc[u][t] & 0xFFFFu));
            const _Float16 s1 = __builtin_bit_cast(_Float16, (uint16_t)(st.sc[u][t] >> 16));
            const _Float16 mn = __builtin_bit_cast(_Float16, (uint16_t)st.zz[u][t]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              if constexpr (kPlainH && kIsQ5K) {
                // byte i of the word: one bit per element 8 i + b; spread to one bit per byte
                const uint32_t hb = (st.ha[u][t][0][0] >> (8 * i)) & 0xFFu;
                const uint32_t hA = ((hb & 0xFu) * 0x00204081u) & 0x01010101u;
                const uint32_t hB = ((hb >> 4) * 0x00204081u) & 0x01010101u;
                b[i] = kqx8_to_f16<1>(wa[i], hA, hB, 0u, s0, mn);
              } else if constexpr (kPlainH) {
                // 16 bits: a 2-bit field per element 8 i + p; spread to one field per byte
                const uint32_t hw = (st.ha[u][t][0][i >> 1] >> (16 * (i & 1))) & 0xFFFFu;
                auto spread = [](uint32_t x) {
                  return (((x & 0x33u) * 0x1001u) & 0x00030003u) | (((((x >> 2) & 0x33u) * 0x1001u) & 0x00030003u) << 8);
                };
                b[i] = kqx8_to_f16<2>(wa[i], spread(hw & 0xFFu), spread(hw >> 8), 0u, i < 2 ? s0 : s1, (_Float16)0.0f);
              } else {
              const uint32_t hA = st.ha[u][t][i >> 1][(i & 1) * 2], hB = st.ha[u][t][i >> 1][(i & 1) * 2 + 1];
              if constexpr (kIsQ5K) b[i] = kqx8_to_f16<1>(wa[i], hA, hB, shift, s0, mn);
              else b[i] = kqx8_to_f16<2>(wa[i], hA, hB, shift, i < 2 ? s0 : s1, (_Float16)0.0f);
              }
            }
          }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          if constexpr (kBlock) {
            f32x4 tt = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < 4; ++i) tt = Act::mfma(as_v8<V8>(st.xa[u][mt][i]), b[i], tt);
            acc[t][mt] += tt * scf;
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              acc[t][mt] = Act::mfma(as_v8<V8>(st.xa[u][mt][i]), b[i], acc[t][mt]);
          }
        }
      }
    }
  };

  if constexpr (SL && kIsInt4) {
    // tables [RT * 16 rows][K / 128]: fp16 scales, then zero-point bytes; rows past the range are zeros
    uint16_t* ts = reinterpret_cast<uint16_t*>(smem + kTiles);
    uint8_t* tz = reinterpret_cast<uint8_t*>(ts + RT * 16 * Kg);
    const int total = RT * 16 * Kg;
    constexpr int FI = 4;
    for (int c0 = 0; c0 < total; c0 += NW * 64 * FI) {
      uint16_t sv[FI];
      uint8_t zv[FI];
#pragma unroll
      for (int i = 0; i < FI; ++i) {
        const int c = c0 + i * NW * 64 + (int)threadIdx.x;
        const int r = min(c, total - 1) / Kg, cc = min(c, total - 1) - r * Kg;
        const int n = min(n0 + r, N - 1);
        sv[i] = s16u[(size_t)n * Kg + cc];
        zv[i] = zsrc[(size_t)n * Kg + cc];
      }
#pragma unroll
      for (int i = 0; i < FI; ++i) {
        const int c = c0 + i * NW * 64 + (int)threadIdx.x;
        if (c < total) {
          const bool ok = n0 + c / Kg < nend;
          ts[c] = ok ? sv[i] : (uint16_t)0;
          tz[c] = ok ? zv[i] : (uint8_t)0;
        }
      }
    }
    __syncthreads();
  } else if constexpr (SL) {
    // tables [RT * 16 rows][K / 32] of scales, then of mins; rows past the workgroup's range are zeros
    const __amdgpu_buffer_rsrc_t sr = make_rsrc(sbase, (uint32_t)N * (uint32_t)Kb32 * 2u);
    const __amdgpu_buffer_rsrc_t mr = make_rsrc(zbase, kHasMin ? (uint32_t)N * (uint32_t)Kb32 * 2u : 0u);
    const int cpr = Kb32 >> 3;                        // 16-byte chunks per row
    u32x4* tab = reinterpret_cast<u32x4*>(smem + kTiles);
    const int total = RT * 16 * cpr;
    constexpr int FI = 4;                             // chunks in flight per thread and table
    for (int c0 = 0; c0 < total; c0 += NW * 64 * FI) {
      u32x4 sv[FI], mv[FI];
#pragma unroll
      for (int i = 0; i < FI; ++i) {
        const int c = c0 + i * NW * 64 + (int)threadIdx.x;
        const int r = c / cpr, cc = c - r * cpr;
        const int n = n0 + r;
        const uint32_t off = (c < total && n < nend) ? ((uint32_t)n * (uint32_t)Kb32 + (uint32_t)cc * 8u) * 2u : kOOB;
        sv[i] = buf_load16(sr, off);
        if constexpr (kHasMin) mv[i] = buf_load16(mr, off);
      }
#pragma unroll
      for (int i = 0; i < FI; ++i) {
        const int c = c0 + i * NW * 64 + (int)threadIdx.x;
        if (c < total) {
          tab[c] = sv[i];
          if constexpr (kHasMin) tab[total + c] = mv[i];
        }
      }
    }
    __syncthreads();
  }

  if constexpr (UN >= 2) {
    // two-stage ring; the only exit is at the bottom (stages past the end load zeros)
    Stage s0, s1;
    load_stage(s0, wave);
    for (int gbase = wave; gbase < G; gbase += NW * UN) {
      load_stage(s1, gbase + NW * US);
      __builtin_amdgcn_sched_barrier(0);
      compute_stage(s0, gbase);
      load_stage(s0, gbase + NW * UN);
      __builtin_amdgcn_sched_barrier(0);
      compute_stage(s1, gbase + NW * US);
    }
  } else {
    Stage s0;
    for (int gbase = wave; gbase < G; gbase += NW * UN) {
      load_stage(s0, gbase);
      __builtin_amdgcn_sched_barrier(0);
      compute_stage(s0, gbase);
    }
  }

  // ---- the NW partial tiles meet in LDS; the wavefronts share the output tiles ----
  __syncthreads();                                    // the buffer overlays the staging tiles
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[wave][t][mt][lane] = acc[t][mt];
  __syncthreads();
  // D layout: lane holds output column n0 + 16 t + j, rows mt*16 + 4 g + v.
  const size_t opitch = GRP ? (size_t)a.out_stride : (size_t)N;
  Elem* out = (Elem*)a.out[mat] + (GRP ? (size_t)t0 * opitch : (size_t)m0 * N);
#pragma unroll
  for (int it = 0; it < kOutIters; ++it) {
    const int o = wave + it * NW;
    if (o >= RT * MT) break;
    const int t = o / MT, mt = o - t * MT;
    const int n = n0 + t * 16 + j;
    f32x4 sum = red[0][t][mt][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) sum += red[w][t][mt][lane];
    if (n < nend) {
      float os = 1.0f;
      if constexpr (kIsFp8 && SC == SC_PERN)
        os = a.scale_f16 ? (float)__builtin_bit_cast(_Float16, (uint16_t)os_raw[it]) : __builtin_bit_cast(float, os_raw[it]);
      if constexpr (kIsFp8 && SC == SC_PERT) os = os_pert;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int m = mt * 16 + g * 4 + v;
        if (m < M) out[(size_t)m * opitch + n] = Act::from_f32(sum[v] * os);
      }
    }
  }
}

// Grouped launches: which chunk and row block a workgroup takes.  Workgroups are dealt to the 8 XCDs in turn;
// an XCD walks groups of `cgroup` consecutive chunks (the caller lists an expert's chunks one after the other)
// row block by row block, so that a chunk's rows of x enter one L2 and the chunks of a group find their
// expert's row block there.
__device__ __forceinline__ int grouped_chunk_of(const SkinnyArgs& a, int& tile) {
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int per = a.cgroup * a.tiles_total;
  const int unit = slot / per, r = slot - unit * per;
  tile = r / a.cgroup;
  return (unit * 8 + xcd) * a.cgroup + (r - tile * a.cgroup);
}

template <class Act, int FMT, int SC, int MT, int RT, int NW, int UN, bool SL = false, bool GRP = false>
__global__ __launch_bounds__(NW * 64) void skinny_kernel(const SkinnyArgs a) {
  int tile = blockIdx.x;
  int m0 = 0;                                         // first row of x of this workgroup
  int eid = 0, t0 = 0, mrows = 0;
  if constexpr (GRP) {
    const int cid = grouped_chunk_of(a, tile);
    if (cid >= a.num_chunks) return;
    eid = a.chunks[3 * cid];
    t0 = a.chunks[3 * cid + 1];
    const int nt = a.chunks[3 * cid + 2];
    if (nt <= 0 || eid < 0 || eid >= a.num_experts || t0 < 0 || t0 >= a.out_rows) return;
    mrows = min(min(nt, MT * 16), a.out_rows - t0);   // rows past 16 MT are not computed
  }
  if (!GRP && a.msplit > 1) {
    // The workgroups of a row block sit 8 apart: workgroups are dealt to the 8 XCDs in turn, so
    // the block's weights come from HBM once and from that XCD's L2 afterwards.
    const int grp = blockIdx.x / (8 * a.msplit), rem = blockIdx.x - grp * 8 * a.msplit;
    m0 = (rem >> 3) * (MT * 16);
    tile = grp * 8 + (rem & 7);
    if (tile >= a.tiles_total || m0 >= a.M) return;
  }
  skinny_body<Act, FMT, SC, MT, RT, NW, UN, SL, GRP>(a, tile, m0, eid, t0, mrows);
}

// Grouped launch whose workgroups pick the number of 16-row tiles of x from their chunk's rows (up to 64):
// a chunk of 20 rows costs two tiles' loads, LDS traffic and MFMAs instead of four.  One granule in flight.
template <class Act, int FMT, int RT, int NW, bool SL>
__global__ __launch_bounds__(NW * 64) void skinny_grouped_kernel(const SkinnyArgs a) {
  int tile;
  const int cid = grouped_chunk_of(a, tile);
  if (cid >= a.num_chunks) return;
  const int eid = a.chunks[3 * cid];
  const int t0 = a.chunks[3 * cid + 1];
  const int nt = a.chunks[3 * cid + 2];
  if (nt <= 0 || eid < 0 || eid >= a.num_experts || t0 < 0 || t0 >= a.out_rows) return;
  const int mrows = min(min(nt, 64), a.out_rows - t0);  // rows past 64 are not computed
  if (mrows <= 16) skinny_body<Act, FMT, 0, 1, RT, NW, 1, SL, true>(a, tile, 0, eid, t0, mrows);
  else if (mrows <= 32) skinny_body<Act, FMT, 0, 2, RT, NW, 1, SL, true>(a, tile, 0, eid, t0, mrows);
  else if (mrows <= 48) skinny_body<Act, FMT, 0, 3, RT, NW, 1, SL, true>(a, tile, 0, eid, t0, mrows);
  else skinny_body<Act, FMT, 0, 4, RT, NW, 1, SL, true>(a, tile, 0, eid, t0, mrows);
}

// Bytes of the LDS scale tables of an SL instantiation (0: the format has none).
template <int FMT, int RT>
static inline int skinny_table_bytes(int K) {
  if (FMT == 1) return (RT * 16 * (K / 128) * 3 + 15) & ~15;   // fp16 scales + zero-point bytes
  const bool side32 = FMT == 2 || FMT == 5 || FMT == 7 || FMT == 3 || FMT == 4;
  if (!side32) return 0;
  return RT * 16 * (K / 32) * 2 * ((FMT == 2 || FMT == 5 || FMT == 7) ? 2 : 1);
}

template <class Act, int FMT, int SC, int MT, int RT, int NW, int UN, bool SL = false>
static void launch_one(SkinnyArgs a, int rpw, hipStream_t st) {
  int tiles = 0;
  a.rpw = rpw;
  for (int i = 0; i < a.nmat; ++i) {
    a.tiles[i] = (a.N[i] + rpw - 1) / rpw;
    tiles += a.tiles[i];
  }
  if (tiles == 0) return;
  a.tiles_total = tiles;
  const int wgs = a.msplit > 1 ? ((tiles + 7) / 8) * 8 * a.msplit : tiles;
  constexpr int kStage = NW * RT * 16 * (((FMT == 0 || FMT == 4) ? 128 : 64) + 16) + (MT >= kSkinnyXLdsFrom ? NW * 16 * (256 + 16) : 0);
  constexpr int kRed = NW * RT * MT * 1024;
  static_assert((kStage > kRed ? kStage : kRed) <= 160 * 1024, "staging tiles exceed the 160 KiB of LDS per workgroup");
  const int with_tables = kStage + (SL ? skinny_table_bytes<FMT, RT>(a.K) : 0);
  const int lds = with_tables > kRed ? with_tables : kRed;
  auto kern = skinny_kernel<Act, FMT, SC, MT, RT, NW, UN, SL>;
  if (lds > 64 * 1024) {
    static int raised = 0;                            // opt in to > 64 KiB of dynamic LDS (grows with K)
    if (raised < lds) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      raised = lds;
    }
  }
  hipLaunchKernelGGL(kern, dim3(wgs), dim3(NW * 64), lds, st, a);
}

// The SL instantiation when the format has per-32 scales, K allows whole 16-byte chunks per row
// and the tables fit beside the staging tiles; the plain one otherwise.
template <int FMT, int MT, int RT, int NW>
static inline bool skinny_tables_fit(int K) {
  if constexpr (FMT == 1 || FMT == 2 || FMT == 3 || FMT == 4 || FMT == 5 || FMT == 7) {
    constexpr int kStage = NW * RT * 16 * (((FMT == 0 || FMT == 4) ? 128 : 64) + 16) + (MT >= kSkinnyXLdsFrom ? NW * 16 * (256 + 16) : 0);
    return (FMT == 1 || K % 256 == 0) && kStage + skinny_table_bytes<FMT, RT>(K) <= 160 * 1024;
  }
  return false;
}

template <class Act, int FMT, int SC, int MT, int RT, int NW, int UN>
static void launch_pick(const SkinnyArgs& a, int rpw, hipStream_t st) {
  if constexpr (FMT == 1 || FMT == 2 || FMT == 3 || FMT == 4 || FMT == 5) {
    if (skinny_tables_fit<FMT, MT, RT, NW>(a.K)) return launch_one<Act, FMT, SC, MT, RT, NW, UN, true>(a, rpw, st);
  }
  launch_one<Act, FMT, SC, MT, RT, NW, UN, false>(a, rpw, st);
}

template <class Act, int FMT, int SC>
static int launch_mt(const SkinnyArgs& a, hipStream_t st) {
  if (a.M == 0) return MI_OK;
  {
    // One workgroup per CU and round, R weight rows each (a multiple of 8, at most
    // 64): wide workgroups re-read the activations from L2 least often, and an
    // exact multiple of the CU count leaves no partial last round.  Rows of a
    // workgroup's last 16-row tile beyond R are dead lanes that load nothing.
    long ntot = 0;
    for (int i = 0; i < a.nmat; ++i) ntot += a.N[i];
    const int cus = device_cu_count();
    int rounds = (int)((ntot + (long)cus * 64 - 1) / ((long)cus * 64));
    if (rounds < 1) rounds = 1;
    int rpw = (int)((ntot + (long)cus * rounds - 1) / ((long)cus * rounds));
    // block scales: tiles must not straddle a 128-row scale block
    rpw = (FMT == 0 && SC == SC_BLOCK) ? ((rpw + 15) & ~15) : ((rpw + 7) & ~7);
    if (rpw > 64) rpw = 64;
    // 33 .. 64 rows against at most 32 weight rows per CU: every workgroup would stage all of x
    // through its LDS for one or two weight tiles.  Two workgroups per (twice as tall) row block
    // take 32 rows of x each instead: half the x traffic and LDS work per weight row; the second
    // reads the block's weights from L2.  FP8 and INT4 only (K = 4096, M = 64: FP8 N = 5120 17.3 ->
    // 12.4 us, INT4 N = 4096 13.5 -> 11.9 us); the formats with per-32 scale tables lose, since both
    // workgroups stage the block's tables (Q4_K K = N = 5120: 17.8 -> 19.7 us).
    if ((FMT == 0 || FMT == 1) && a.M > 32 && rounds == 1 && rpw <= 32 && ntot >= 16L * cus) {
      SkinnyArgs h = a;
      h.msplit = 2;
      int r2 = (int)((2 * ntot + cus - 1) / cus);
      r2 = (FMT == 0 && SC == SC_BLOCK) ? ((r2 + 15) & ~15) : ((r2 + 7) & ~7);
      if (r2 <= 32) launch_pick<Act, FMT, SC, 2, 2, 8, 2>(h, r2, st);
      else if (r2 <= 48) launch_pick<Act, FMT, SC, 2, 3, 8, 2>(h, r2, st);
      else launch_pick<Act, FMT, SC, 2, 4, 8, 1>(h, r2 > 64 ? 64 : r2, st);
      return launch_status();
    }
    if (rpw <= 16) {
      if (a.M <= 16) launch_pick<Act, FMT, SC, 1, 1, 8, 4>(a, rpw, st);
      else if (a.M <= 32) launch_pick<Act, FMT, SC, 2, 1, 8, 2>(a, rpw, st);
      else launch_pick<Act, FMT, SC, 4, 1, 8, 1>(a, rpw, st);
    } else if (rpw <= 32) {
      if (a.M <= 16) {
        // more than 32 granules: six per wavefront in flight cover K in one turn of the ring
        // (Q4_K K = N = 5120: M=8 13.5 -> 12.7 us, M=16 15.5 -> 13.9 us)
        // (not for Q5_K / Q6_K: with their high-bit registers six granules spill)
        bool six = false;
        if constexpr (FMT != 5 && FMT != 6) {
          six = a.K > 4096 && a.K <= 6144;
          if (six) launch_pick<Act, FMT, SC, 1, 2, 8, 6>(a, rpw, st);
        }
        if (!six) launch_pick<Act, FMT, SC, 1, 2, 8, 4>(a, rpw, st);
      } else if (a.M <= 32) launch_pick<Act, FMT, SC, 2, 2, 8, 2>(a, rpw, st);
      else if constexpr (FMT == 0 || FMT == 4) launch_pick<Act, FMT, SC, 4, 2, 8, 1>(a, rpw, st);
      else if (skinny_tables_fit<FMT, 4, 2, 6>(a.K)) launch_pick<Act, FMT, SC, 4, 2, 6, 1>(a, rpw, st);
      else launch_one<Act, FMT, SC, 4, 2, 8, 1>(a, rpw, st);   // nibble formats: eight waves' tiles fit the LDS
      // (cfg4 M=64, Q4_K: 24.1 us with four waves, 21.9 with eight, 18.6 with six + the LDS tables)
    } else {
      if (a.M <= 16) launch_pick<Act, FMT, SC, 1, 4, 8, 2>(a, rpw, st);
      else if (a.M <= 32) launch_pick<Act, FMT, SC, 2, 4, 8, 1>(a, rpw, st);
      // eight wavefronts since the activations pass through one LDS tile per wavefront (four would
      // leave one per SIMD and nothing to overlap its load -> LDS -> MFMA chain with): K=4096 N=14336
      // M=64 FP8 24.2 -> 21.9 us, INT4 25.7 -> 21.1 us
      else launch_pick<Act, FMT, SC, 4, 4, 8, 1>(a, rpw, st);
    }
  }
  return launch_status();
}

}  // namespace qlin
