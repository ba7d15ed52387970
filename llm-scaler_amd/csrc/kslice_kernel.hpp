// Small-M weight-only GEMM (FP8 E4M3, INT4 group 128, GGUF Q4_K / Q4_0 / Q8_0) with the
// activations resident in registers.
//
// Regime: 3 <= M <= 32 rows (up to 64 for K <= 2048) against an [N, K] quantized weight, M * K
// small enough that a workgroup can hold all of x in its register file (x is the matrix-core
// operand that never changes while the weight streams past).  One workgroup owns up to 64 weight
// rows; its 8 wavefronts split K into 8 contiguous slices instead of interleaving granules, so that
//   - a wavefront loads its slice of x ONCE, before any weight load is issued (x comes from L2;
//     the vector-memory counter retires in order, so these loads never queue behind the weight
//     stream),
//   - the loop is weight loads -> wave-private LDS transpose -> decode -> MFMA, with the
//     next 16-row tile in flight while the current one is consumed: no barrier, no x traffic,
//   - the 8 partial tiles meet once, at the end, in LDS.
// Weight loads are row-contiguous (one instruction reads 1 KiB of consecutive slice bytes, row
// after row: operand-layout loads whose lanes read 64-byte pieces of 16 rows were measured
// about 3 us slower on a 56 MB weight); the wavefront's own LDS tile (pitch + 16 bytes) turns
// them into operand layout.  The slice of x is loaded the same way.
//
// k assignment inside a slice: step q (0 .. NQ-1) of lane (j = lane % 16, g = lane / 16) covers
// k = 64 q + 16 g .. + 15 of weight row n0 + 16 t + j (16 bytes of a byte format, 8 bytes of a
// nibble format); MFMA 2 q + h consumes its k = 8 h .. 8 h + 7 against
// x[j][slice + 64 q + 16 g + 8 h .. + 7].
// Side data travels with the tile as a few small loads per lane: INT4 the fp16 scales and
// zero-point bytes of the row's NQ / 2 groups inside the slice, the GGUF formats the fp16 scales
// (Q4_K: and mins) of its 2 NQ sub-blocks.  The weights are decoded with the scale folded in
// (the routines of the dequantization kernels), so the sums need no factor; FP8 per-channel /
// per-tensor scales multiply the finished sums, block scales each 128-wide partial.
#pragma once
#include "skinny_kernel.hpp"

namespace qlin {

constexpr int kKsliceWaves = 8;
// 16-row weight tiles per workgroup: four, or what the partial tiles of four activation tiles
// leave of the LDS
constexpr int kslice_max_tiles(int MT) { return MT <= 3 ? 4 : 3; }

template <int MT, int NQ>
constexpr int kslice_lds_bytes() {
  return kKsliceWaves * 16 * (64 * NQ + 16) + kKsliceWaves * kslice_max_tiles(MT) * MT * 1024;
}

// FMT = 0: FP8 E4M3, 1: INT4 group 128, 2: GGUF Q4_K (repacked; fp16 scale and min per 32 k),
// 3: Q4_0, 4: Q8_0 (repacked; fp16 scale per 32 k).  MT = 16-row activation tiles (M <= 16 MT),
// NQ = 64-wide k steps per slice (slice = 64 NQ k; byte formats: NQ 16-byte loads per lane and
// tile, nibble formats: NQ / 2),
// BLOCK = 128x128 block scales (FP8; otherwise one scale per output channel or per tensor,
// applied to the finished sum).
template <class Act, int FMT, bool BLOCK, int MT, int NQ>
__global__ __launch_bounds__(kKsliceWaves * 64) void kslice_kernel(const SkinnyArgs a, const int scale_mode) {
  using V8 = typename Act::v8;
  using Elem = typename Act::elem;
  constexpr bool kInt4 = FMT == 1;
  constexpr bool kQ4K = FMT == 2;
  constexpr bool kQ40 = FMT == 3;
  constexpr bool kQ80 = FMT == 4;
  constexpr bool kSide32 = kQ4K || kQ40 || kQ80;      // one fp16 scale (Q4_K: and min) per 32 k
  constexpr bool kNib = kInt4 || kQ4K || kQ40;        // two weights per byte
  static_assert(!kInt4 || (NQ % 4 == 0 && !BLOCK), "INT4: whole pairs of groups per slice");
  static_assert(!kSide32 || (NQ % 2 == 0 && !BLOCK && Act::dt == DT_F16), "the GGUF formats run in fp16");
  constexpr int NW = kKsliceWaves;
  constexpr int kMaxTiles = kslice_max_tiles(MT);
  constexpr int kSliceB = 64 * NQ;                    // k of a slice = bytes of half a slice row of x
  constexpr int kPitch = kSliceB + 16;                // LDS row pitch: operand reads hit distinct banks
  constexpr int kStage = 16 * kPitch;                 // one wavefront's staging tile
  constexpr int kCPR = kSliceB / 16;                  // 16-byte chunks per row of the tile (x halves, FP8 weights)
  constexpr int kWRowB = kNib ? kSliceB / 2 : kSliceB;   // bytes of one weight row inside a slice
  constexpr int kWPitch = kWRowB + 16;
  constexpr int kWCPR = kWRowB / 16;
  constexpr int NL = kNib ? NQ / 2 : NQ;              // 16-byte weight loads per lane and tile
  // side words per lane and tile: INT4 one per pair of groups (two fp16 scales / two zero-point
  // bytes), Q4_K one per step (the fp16 scales / mins of its two 32-wide sub-blocks)
  constexpr int NS = kInt4 ? NQ / 4 : (kSide32 ? NQ : 1);
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // the partial tiles live beside the staging tiles
  f32x4 (*red)[kMaxTiles][MT][64] = reinterpret_cast<f32x4 (*)[kMaxTiles][MT][64]>(smem + NW * kStage);

  int tile = blockIdx.x;
  int mat = 0;
#pragma unroll
  for (int i = 0; i + 1 < kMaxMat; ++i) {
    if (mat == i && i + 1 < a.nmat && tile >= a.tiles[i]) { tile -= a.tiles[i]; mat = i + 1; }
  }
  const int N = a.N[mat];
  const int K = a.K, M = a.M;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int j = lane & 15, g = lane >> 4;
  const int n0 = tile * a.rpw;
  const int nend = min(N, n0 + a.rpw);
  const int ntiles = (nend - n0 + 15) >> 4;           // <= kMaxTiles
  const int kbase = wave * kSliceB;                   // first k of this wavefront's slice

  const uint32_t wrow = kNib ? (uint32_t)K >> 1 : (uint32_t)K;   // weight bytes per row
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(a.w[mat], (uint32_t)N * wrow);
  // INT4 side data: fp16 scales and (optional) zero-point bytes per 128-wide group
  const int Kg = K >> 7;
  const bool has_zp = kInt4 && a.z[mat] != nullptr;
  const int Kc = K >> 5;                              // Q4_K: fp16 scale and min per 32-wide sub-block
  const __amdgpu_buffer_rsrc_t sr =
      make_rsrc(a.s[mat], kInt4 ? (uint32_t)N * (uint32_t)Kg * 2u : (kSide32 ? (uint32_t)N * (uint32_t)Kc * 2u : 0u));
  const __amdgpu_buffer_rsrc_t zr =
      make_rsrc((has_zp || kQ4K) ? a.z[mat] : a.s[mat],
                has_zp ? (uint32_t)N * (uint32_t)Kg : (kQ4K ? (uint32_t)N * (uint32_t)Kc * 2u : 0u));
  const __amdgpu_buffer_rsrc_t xr = make_rsrc(a.x, (uint32_t)M * (uint32_t)K * 2u);

  // The 64 NQ 16-byte chunks of a 16-row tile (16 rows x kCPR chunks) are walked row-major: load i
  // takes chunks 64 i .. 64 i + 63, i.e. 1 KiB of consecutive bytes, row after row.
  auto chunk_of = [&](int i, int& r, int& c) {
    const int f = i * 64 + lane;
    r = f / kCPR;
    c = f - r * kCPR;
  };
  unsigned char* stage = smem + wave * kStage;

  // ---- x: the wavefront's slice of every row, once ----
  // Loaded like the weights, row-contiguous: x is read by every workgroup, and an instruction
  // whose lanes gather 16-byte operand pieces from 16 rows takes the L1 four times as long as
  // one that reads 1 KiB in a row (measured: 256 workgroups x 32 rows x 4096, 6.5 against 1.6 us).
  // A 16-row tile of the slice is two LDS tiles wide (16-bit elements), so it is staged in two
  // halves; slot [mt][hx NQ/2 + i / 2][i % 2] holds load i of half hx until the transposition.
  u32x4 xq[MT][NQ][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int hx = 0; hx < 2; ++hx)
#pragma unroll
      for (int i = 0; i < NQ; ++i) {
        int r, c;
        chunk_of(i, r, c);
        const int m = mt * 16 + r;
        const int k = kbase + hx * (kSliceB / 2) + 8 * c;
        xq[mt][hx * (NQ / 2) + i / 2][i & 1] =
            buf_load16(xr, (m < M && k < K) ? ((uint32_t)m * (uint32_t)K + (uint32_t)k) * 2u : kOOB);
      }
  // registers (row-contiguous) -> LDS tile -> registers (operand layout: lane (j, g) of slot
  // [mt][q][h] holds x[16 mt + j][slice + 64 q + 16 g + 8 h .. + 7])
  auto transpose_x = [&]() {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int hx = 0; hx < 2; ++hx) {
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
          int r, c;
          chunk_of(i, r, c);
          *reinterpret_cast<u32x4*>(stage + r * kPitch + c * 16) = xq[mt][hx * (NQ / 2) + i / 2][i & 1];
        }
#pragma unroll
        for (int q = 0; q < NQ / 2; ++q)
#pragma unroll
          for (int h = 0; h < 2; ++h)
            xq[mt][hx * (NQ / 2) + q][h] =
                *reinterpret_cast<const u32x4*>(stage + j * kPitch + 128 * q + 32 * g + 16 * h);
      }
  };

  // ---- weights: two 16-row tiles in flight in registers ----
  // A tile in registers: NL 16-byte loads per lane (row-contiguous until the transposition, then
  // step q's bytes: FP8 w[q], INT4 dwords 2 (q % 2) and 2 (q % 2) + 1 of w[q / 2]); INT4 also the
  // lane's row's scales (two fp16 per word) and zero-points (two bytes per word) of the slice.
  struct Tile {
    u32x4 w[NL];
    uint32_t s[NS], z[NS];
  };
  auto wchunk_of = [&](int i, int& r, int& c) {
    const int f = i * 64 + lane;
    r = f / kWCPR;
    c = f - r * kWCPR;
  };
  auto load_tile = [&](Tile& tl, int t) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      int r, c;
      wchunk_of(i, r, c);
      const int n = n0 + t * 16 + r;
      const int k = kbase + (kNib ? 32 : 16) * c;     // first k of the chunk
      const bool ok = t < ntiles && n < nend && k < K;
      tl.w[i] = __builtin_amdgcn_raw_buffer_load_b128(
          wr, ok ? (uint32_t)n * wrow + (uint32_t)(kNib ? k >> 1 : k) : kOOB, 0, 2 /* nt */);
    }
    if constexpr (kInt4) {
      const int n = n0 + t * 16 + j;
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        const int grp = (kbase >> 7) + 2 * i;         // K % 256 == 0: a pair of groups never straddles the row end
        const bool ok = t < ntiles && n < nend && grp < Kg;
        const uint32_t e = (uint32_t)n * (uint32_t)Kg + (uint32_t)grp;
        tl.s[i] = __builtin_amdgcn_raw_buffer_load_b32(sr, ok ? e * 2u : kOOB, 0, 0);
        tl.z[i] = has_zp ? (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(zr, ok ? e : kOOB, 0, 0) : 0x0808u;
      }
    }
    if constexpr (kSide32) {
      // the row's 2 NQ sub-blocks inside the slice, four entries (one step pair) per 64-bit load
      const int n = n0 + t * 16 + j;
#pragma unroll
      for (int i = 0; i < NQ / 2; ++i) {
        const int sb = (kbase >> 5) + 4 * i;          // K % 256 == 0: four entries never straddle the row end
        const bool ok = t < ntiles && n < nend && sb < Kc;
        const uint32_t off = ok ? ((uint32_t)n * (uint32_t)Kc + (uint32_t)sb) * 2u : kOOB;
        const u32x2 sv = __builtin_amdgcn_raw_buffer_load_b64(sr, off, 0, 0);
        tl.s[2 * i] = sv[0]; tl.s[2 * i + 1] = sv[1];
        if constexpr (kQ4K) {
          const u32x2 mv = __builtin_amdgcn_raw_buffer_load_b64(zr, off, 0, 0);
          tl.z[2 * i] = mv[0]; tl.z[2 * i + 1] = mv[1];
        }
      }
    }
  };
  // registers (row-contiguous) -> this wavefront's LDS tile -> registers (operand layout)
  auto transpose_tile = [&](Tile& tl) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      int r, c;
      wchunk_of(i, r, c);
      *reinterpret_cast<u32x4*>(stage + r * kWPitch + c * 16) = tl.w[i];
    }
    if constexpr (kNib) {
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(stage + j * kWPitch + 32 * q + 8 * g);
        tl.w[q >> 1][(q & 1) * 2] = v[0];
        tl.w[q >> 1][(q & 1) * 2 + 1] = v[1];
      }
    } else {
#pragma unroll
      for (int q = 0; q < NQ; ++q) tl.w[q] = *reinterpret_cast<const u32x4*>(stage + j * kWPitch + 64 * q + 16 * g);
    }
  };
  // the 8 k of MFMA 2 q + h as the activation type
  auto operand = [&](const Tile& tl, int q, int h) -> V8 {
    if constexpr (kInt4) {
      const uint32_t dw = tl.w[q >> 1][(q & 1) * 2 + h];
      const int gq = q >> 1;                          // group inside the slice
      const uint32_t sbits = (tl.s[gq >> 1] >> (16 * (gq & 1))) & 0xFFFFu;
      const float zf = (float)((tl.z[gq >> 1] >> (8 * (gq & 1))) & 0xFFu);
      const float sf = (float)__builtin_bit_cast(_Float16, (uint16_t)sbits);
      if constexpr (Act::dt == DT_F16) return int4x8_to_f16(dw, (_Float16)sf, (_Float16)(1024.0f + zf));
      else return int4x8_to_bf16(dw, sf, zf);
    } else if constexpr (kQ4K) {
      // step q covers sub-blocks 2 q (lanes g = 0, 1) and 2 q + 1 (g = 2, 3) of the slice
      const uint32_t dw = tl.w[q >> 1][(q & 1) * 2 + h];
      const uint32_t sh = (uint32_t)(g >> 1) * 16u;
      const _Float16 sc = __builtin_bit_cast(_Float16, (uint16_t)(tl.s[q] >> sh));
      const _Float16 mn = __builtin_bit_cast(_Float16, (uint16_t)(tl.z[q] >> sh));
      if constexpr (Act::dt == DT_F16) return q4kx8_to_f16(dw, sc, mn);
      else return V8{};
    } else if constexpr (kQ40) {
      const uint32_t dw = tl.w[q >> 1][(q & 1) * 2 + h];
      const _Float16 sc = __builtin_bit_cast(_Float16, (uint16_t)(tl.s[q] >> ((uint32_t)(g >> 1) * 16u)));
      if constexpr (Act::dt == DT_F16) return int4x8_to_f16(dw, sc, (_Float16)1032.0f);   // (nib - 8) * d
      else return V8{};
    } else if constexpr (kQ80) {
      const _Float16 sc = __builtin_bit_cast(_Float16, (uint16_t)(tl.s[q] >> ((uint32_t)(g >> 1) * 16u)));
      if constexpr (Act::dt == DT_F16) return i8x8_to_f16(tl.w[q][2 * h], tl.w[q][2 * h + 1], sc);
      else return V8{};
    } else {
      return fp8x8_to_act<Act>(tl.w[q][2 * h], tl.w[q][2 * h + 1]);
    }
  };
  const float* s32 = (const float*)a.s[mat];
  const int Kb = (K + 127) >> 7;
  auto compute_tile = [&](Tile& w, int t) {
    transpose_tile(w);
    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    if constexpr (BLOCK) {
      // two reads = one 128-wide scale block; its partial sum is scaled before it joins the total
      const int nb = min(n0 + t * 16, N - 1) >> 7;
#pragma unroll
      for (int q2 = 0; q2 < NQ / 2; ++q2) {
        const int kb = min((kbase >> 7) + q2, Kb - 1);
        const float sc = s32[(size_t)nb * Kb + kb];
        f32x4 part[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) part[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) {
          const int q = q2 * 2 + qq;
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const V8 b = operand(w, q, h);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) part[mt] = Act::mfma(as_v8<V8>(xq[mt][q][h]), b, part[mt]);
          }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[mt] += part[mt] * sc;
      }
    } else {
#pragma unroll
      for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const V8 b = operand(w, q, h);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[mt] = Act::mfma(as_v8<V8>(xq[mt][q][h]), b, acc[mt]);
        }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[wave][t][mt][lane] = acc[mt];
  };

  Tile w0, w1;
  load_tile(w0, 0);
  load_tile(w1, 1);
  __builtin_amdgcn_sched_barrier(0);
  // The output scales of the columns this wavefront finishes (see the end), requested behind the
  // first weight tiles and kept as raw bits: fetched where they are used they are one more round
  // trip at the very end of the launch, with nothing left to hide it.  (Not ahead of the weight
  // loads: the compiler may pick the pending scale register as the don't-care half of a 64-bit
  // address multiply-add, and the first weight load then waits for the scale.)
  constexpr int kOutIters = (kMaxTiles * MT + NW - 1) / NW;
  uint32_t os_raw[kOutIters];
#pragma unroll
  for (int it = 0; it < kOutIters; ++it) os_raw[it] = 0;
  float os_pert = 1.0f;
  if constexpr (FMT == 0 && !BLOCK) {
    if (scale_mode == SC_PERT) os_pert = ((const float*)a.s[mat])[0];
    if (scale_mode != SC_PERT) {
#pragma unroll
      for (int it = 0; it < kOutIters; ++it) {
        const int o = wave + it * NW;
        const int n = min(n0 + (o / MT) * 16 + j, N - 1);
        os_raw[it] = a.scale_f16 ? (uint32_t)((const uint16_t*)a.s[mat])[n] : ((const uint32_t*)a.s[mat])[n];
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  transpose_x();
  // Tiles 0 .. 3 with static register slots.  Every load is issued unconditionally (a tile past
  // the workgroup's range loads nothing), so the wait counts stay exact on every path; only the
  // arithmetic of a missing tile is skipped.
  compute_tile(w0, 0);
  load_tile(w0, 2);
  __builtin_amdgcn_sched_barrier(0);
  if (ntiles > 1) compute_tile(w1, 1);
  load_tile(w1, 3);
  __builtin_amdgcn_sched_barrier(0);
  if (ntiles > 2) compute_tile(w0, 2);
  if constexpr (kMaxTiles > 3) {
    if (ntiles > 3) compute_tile(w1, 3);
  }

  // ---- the 8 slices meet: wavefront w finishes output tile (t, mt) = w ----
  __syncthreads();
#pragma unroll
  for (int it = 0; it < kOutIters; ++it) {
    const int o = wave + it * NW;
    if (o >= ntiles * MT) break;
    const int t = o / MT, mt = o - t * MT;
    f32x4 sum = red[0][t][mt][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) sum += red[w][t][mt][lane];
    // D layout: lane holds output column n0 + 16 t + j, rows 16 mt + 4 g + v
    const int n = n0 + t * 16 + j;
    if (n < nend) {
      float os = 1.0f;
      if constexpr (FMT == 0 && !BLOCK) {
        if (scale_mode == SC_PERT) os = os_pert;
        else os = a.scale_f16 ? (float)__builtin_bit_cast(_Float16, (uint16_t)os_raw[it]) : __builtin_bit_cast(float, os_raw[it]);
      }
      Elem* out = (Elem*)a.out[mat];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int m = mt * 16 + g * 4 + v;
        if (m < M) out[(size_t)m * N + n] = Act::from_f32(sum[v] * os);
      }
    }
  }
}

// Whether the register-resident path covers a problem (0: no; else the steps per slice): 3 .. 64
// rows, the slice of x within 128 registers per lane; fmt 0 (FP8): 16-byte aligned rows; fmt 1
// (INT4): K a multiple of 512, so that a slice holds whole pairs of groups and the side loads are
// aligned; fmt 2 (Q4_K): K a multiple of 256, and a scale and a min word per step on top of x;
// fmt 3, 4 (Q4_0, Q8_0): K a multiple of 128.
static inline int kslice_loads(int M, int K, int fmt = 0) {
  if (M < 3 || M > 64 || (K % 16) || (fmt == 1 && (K % 512)) || (fmt == 2 && (K % 256)) ||
      ((fmt == 3 || fmt == 4) && (K % 128)))
    return 0;
  const int mt = (M + 15) / 16;
  int nq = (K + 64 * kKsliceWaves - 1) / (64 * kKsliceWaves);   // steps to cover K with 8 slices
  nq = fmt == 1 ? ((nq + 3) & ~3) : ((nq + 1) & ~1);            // FP8: whole 128-wide scale blocks
  const int choices[] = {2, 4, 6, 8, 10, 12};          // 16 steps spill
  for (int c : choices)
    if (c >= nq) {
      if (fmt >= 2) return (mt * c + c <= 20) ? c : 0;          // GGUF: scale (and min) words per step and tile on top
      return (mt * c <= 16) ? c : 0;                            // x registers: mt * c * 8 <= 128
    }
  return 0;
}

// true when a kernel was launched; false when no instantiation covers (MT, nq, FMT), in which case
// the caller reports MI_ERR_SHAPE and leaves the output untouched
template <class Act, int FMT, bool BLOCK, int MT>
static bool kslice_launch_nq(const SkinnyArgs& a, int nq, int tiles, int scale_mode, hipStream_t st) {
  const dim3 grid(tiles), block(kKsliceWaves * 64);
#define QLIN_KSLICE(NQ_)                                                                                       \
  case NQ_:                                                                                                    \
    if constexpr (MT * NQ_ <= 16 && (FMT != 1 || NQ_ % 4 == 0) && (FMT < 2 || MT * NQ_ + NQ_ <= 20))           \
    {                                                                                                          \
      auto kern = kslice_kernel<Act, FMT, BLOCK, MT, NQ_>;                                                     \
      constexpr int lds = kslice_lds_bytes<MT, NQ_>();                                                         \
      static_assert(lds <= 160 * 1024, "staging tiles exceed the LDS");                                        \
      static bool raised = false;                                                                              \
      if (lds > 64 * 1024 && !raised) {                                                                        \
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds); \
        raised = true;                                                                                         \
      }                                                                                                        \
      hipLaunchKernelGGL(kern, grid, block, lds, st, a, scale_mode);                                           \
      return true;                                                                                             \
    }                                                                                                          \
    break;
  switch (nq) {
    QLIN_KSLICE(2) QLIN_KSLICE(4) QLIN_KSLICE(6) QLIN_KSLICE(8) QLIN_KSLICE(10) QLIN_KSLICE(12)
    default: break;
  }
#undef QLIN_KSLICE
  return false;
}

// scale_mode (FP8): SC_PERN / SC_PERT / SC_BLOCK.  Rows per workgroup as in the skinny kernel: one
// workgroup per CU and round, a multiple of 16 rows, at most 64.
template <class Act, int FMT = 0>
static int kslice_launch(SkinnyArgs a, int scale_mode, int nq, hipStream_t st) {
  long ntot = 0;
  for (int i = 0; i < a.nmat; ++i) ntot += a.N[i];
  const int cus = device_cu_count();
  const int max_rows = 16 * kslice_max_tiles((a.M + 15) / 16);
  int rounds = (int)((ntot + (long)cus * max_rows - 1) / ((long)cus * max_rows));
  if (rounds < 1) rounds = 1;
  int rpw = (int)((ntot + (long)cus * rounds - 1) / ((long)cus * rounds));
  rpw = scale_mode == SC_BLOCK ? ((rpw + 15) & ~15) : ((rpw + 7) & ~7);
  if (rpw > max_rows) rpw = max_rows;
  if (rpw < 8) rpw = 8;
  a.rpw = rpw;
  int tiles = 0;
  for (int i = 0; i < a.nmat; ++i) {
    a.tiles[i] = (a.N[i] + rpw - 1) / rpw;
    tiles += a.tiles[i];
  }
  if (!tiles) return MI_OK;
  const bool block = FMT == 0 && scale_mode == SC_BLOCK;
#define QLIN_KSLICE_MT(MT_)                                                              \
  case MT_:                                                                              \
    if constexpr (FMT != 0) launched = kslice_launch_nq<Act, FMT, false, MT_>(a, nq, tiles, scale_mode, st);   \
    else if (block) launched = kslice_launch_nq<Act, 0, true, MT_>(a, nq, tiles, scale_mode, st);   \
    else launched = kslice_launch_nq<Act, 0, false, MT_>(a, nq, tiles, scale_mode, st);             \
    break;
  bool launched = false;
  switch ((a.M + 15) / 16) {
    QLIN_KSLICE_MT(1) QLIN_KSLICE_MT(2) QLIN_KSLICE_MT(3) QLIN_KSLICE_MT(4)
    default: return MI_ERR_SHAPE;
  }
#undef QLIN_KSLICE_MT
  if (!launched) return MI_ERR_SHAPE;      // kslice_loads() and the instantiation guards disagree
  return launch_status();
}

}  // namespace qlin
