// Prefill GEMM for gfx950 on quantized weights: out[M,N] = x[M,K] @ dequant(w[N,K])^T with
// fp16 / bf16 activations, templated on the weight format (INT4 group 128, FP8 E4M3 with
// per-channel / per-tensor / 128x128 block scales, GGUF Q4_K in its repacked representation).
//
// MFMA-bound regime (M in the hundreds or thousands).  A workgroup of 4 wavefronts (2 x 2)
// owns a BM x BN output tile; each wavefront computes a (BM/2) x (BN/2) sub-tile with
// v_mfma_f32_16x16x32_{bf16,f16}, accumulators in the AGPR half of the register file.  What
// limits this kernel is LDS bandwidth (a CU sustains about 130 B/ns of ds_read_b128 and
// 75 B/ns of LDS writes, against ~1 us of MFMA work per 64-wide K step), so only the operand
// that has to be shared goes through LDS:
//   * weights: each 64-wide K step of the BN weight rows is loaded once per workgroup (128-bit
//     loads), dequantized to the activation type in registers and written to a double-buffered
//     LDS tile (row pitch 144 B, so the 16 rows of an MFMA operand read fall into distinct
//     banks); every weight is dequantized once per workgroup and reused by all BM rows;
//   * activations: never touch LDS.  A small pre-pass re-tiles x into MFMA operand order (one
//     1 KiB block per 16 rows x 32 k, lane l's 16 bytes at l * 16), so that a wavefront fetches
//     an operand with one fully contiguous 128-bit load per lane straight from global memory /
//     L2 into a 4-deep register ring, 3 K steps of 32 ahead of its use.  (Read from the
//     row-major matrix, the 64 lanes of an operand hit 64 different 16-byte pieces of 16 rows
//     and the texture addresser becomes the bottleneck.)  The re-tiled copy lives in a caller-
//     provided workspace of roundup(M, 16) * K * 2 bytes.
// The dequantization is cut into small pieces that are placed behind individual MFMAs, so the
// vector ALU works in the shadow of the matrix pipe.  One barrier per 64-wide K step.  The
// weights are the MFMA A operand, so a lane ends up with 4 consecutive output columns of one
// row and stores them as 8 bytes.
//
// A weight format is a policy class: how a 64-wide K step of a weight row is cut into 16-byte
// chunks, which side loads (scales, zero-points, mins) a chunk needs, the dequantization of a
// chunk as a sequence of small pieces, and an optional factor on the finished sums.
#pragma once
#include "qlinear_common.hpp"
#include <type_traits>

namespace qlin {

struct GemmArgs {
  const void* x;              // activations re-tiled into MFMA operand order (the workspace)
  const void* w;
  const void* scale;
  const void* zp;             // int4: zero-points (may be null); Q4_K: mins
  void* out;
  int M, N, K;
  int tiles_m, tiles_n;
  int xcd_m;                  // dense launches: the 8 XCDs form an xcd_m x (8 / xcd_m) grid over the tiles (0: none)
  int scale_mode;             // fp8: 0 = per output channel, 1 = per tensor / expert, 2 = 128x128 blocks,
                              // 3 = two per expert: weight rows below n_half, rows from n_half on
  int scale_f16;              // fp8 per channel: the scales are fp16 instead of fp32
  // Grouped launch (GROUPED kernels): M-tile i of the grid belongs to expert g_tile[4 i] and covers
  // the rows [g_tile[4 i + 1], + g_tile[4 i + 2]) of the expert-sorted order; its activations
  // start at 16-row block g_tile[4 i + 3] of the re-tiled copy (every expert's rows are padded
  // to whole blocks there).  g_count[0] = number of M-tiles; M = rows of x (all experts).
  // The matrices of expert e start e * g_w_stride bytes into w and e * g_s_stride bytes into
  // scale.  out rows: sorted position, or out_map[position]; optional factor row_weight[row].
  const int32_t* g_tile;
  const int32_t* g_count;
  long long g_w_stride, g_s_stride;
  const int32_t* out_map;
  const void* row_weight;
  int x_blocks;               // 16-row blocks in the re-tiled activations
  int n_half;                 // FUSE: weight row n (gate) pairs with row n + n_half (up); N = 2 n_half
  int gelu;                   // FUSE: tanh-GELU instead of SiLU
  int out_rows;               // rows of out (bounds mapped rows)
  int out_packed;             // GROUPED: out is written in the re-tiled operand order of x (16-row blocks of the
                              // tile table, n_out / 32 steps each) for a following grouped GEMM; out_rows = 16 x blocks
};

// MFMA with the accumulator pinned to the AGPR half of the register file and updated in place.
// Left to the register allocator, the 224-256 accumulator registers of a 128 x 128 wave tile
// get split and copied around the loop; the constraint keeps them where they are.  The
// operands of every call come from LDS / global loads (never from a vector-ALU result), and
// results are only read after the explicit wait at the end of the K loop.
template <class Act>
__device__ __forceinline__ void mfma_agpr(f32x4& acc, u32x4 a, u32x4 b) {
  if constexpr (Act::dt == DT_F16)
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  else
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

constexpr int kBK = 64;
constexpr int kPitch = kBK + 8;                      // elements per LDS row (144 bytes)

// ------------------------------------------------------------------ INT4 group 128
// 32 nibbles per 16-byte chunk, two chunks per row and step; fp16 scale and optional zero-point
// byte per group of 128.  A nibble 0..15 read as an E4M3 code is nib * 2^-9 (codes below 16 are
// the subnormals and the first binade, same spacing), so one v_cvt_pk_f32_fp8 turns two nibbles
// into floats; fma(nib * 2^-9, 512 s, -z s) in fp32 is exact ((nib - z) * s has at most 16
// significant bits), then one RNE to the activation type: the same value as rne((nib - z) * s),
// only the sign of a zero can differ from the subtract-then-multiply form, which no product
// notices.  (A packed-fp16 formulation — plant the nibble in the mantissa of 1024, v_pk_add_f16,
// v_pk_mul_f16 — measured 1.5x slower for the whole kernel, with or without v_perm_b32: the
// packed 16-bit instructions do not hide behind the MFMAs the way the fp32 ones do.)
template <class Act, int BN>
struct WInt4 {
  static constexpr int CPR = 2;                       // chunks per row and 64-wide step
  static constexpr double kWeightBytesPerK = 0.5;
  static constexpr int B_CH = (BN * CPR + 255) / 256; // chunks per thread
  static constexpr int LPC = 3;                       // load instructions per chunk
  static constexpr int kPieces = B_CH * 4 * 8;        // 8 pieces per packed dword of 8 nibbles
  static constexpr bool kOutScale = false;
  static constexpr bool kPermK = false;
  struct Res {
    __amdgpu_buffer_rsrc_t wr, sr, zr;
    bool has_zp;
    int Kg;
  };
  struct Stage {
    u32x4 b[B_CH];
    uint32_t s[B_CH], z[B_CH];                        // fp16 scale bits, zero-point: 32-bit slots, one register each
  };
  struct Dq {
    uint32_t e, o;
    f32x2 fe, fo;
    u32x4 outv;
    float sf[B_CH], nzs[B_CH];                        // 512 * scale and -z * scale (exact)
  };
  static __device__ __forceinline__ Res make(const GemmArgs& p, int = 0) {
    Res r;
    r.Kg = p.K >> 7;
    r.wr = make_rsrc(p.w, (uint32_t)p.N * ((uint32_t)p.K >> 1));
    r.sr = make_rsrc(p.scale, (uint32_t)p.N * (uint32_t)r.Kg * 2u);
    r.zr = make_rsrc(p.zp, p.zp ? (uint32_t)p.N * (uint32_t)r.Kg : 0u);
    r.has_zp = p.zp != nullptr;
    return r;
  }
  // byte offset of chunk kc of row n at k = 0, and the row's first side-table entry
  static __device__ __forceinline__ void chunk_addr(const Res& r, int n, int kc, int K, uint32_t& boff, uint32_t& soff) {
    boff = (uint32_t)n * ((uint32_t)K >> 1) + (uint32_t)(kc * 16);
    soff = (uint32_t)n * (uint32_t)r.Kg;              // in groups; x2 for the fp16 scale
  }
  static __device__ __forceinline__ void load1(const Res& r, Stage& st, const uint32_t (&boff)[B_CH],
                                               const uint32_t (&soff)[B_CH], int kt, uint32_t dead, int idx) {
    const uint32_t k0 = (uint32_t)kt * kBK;
    const int i = idx / 3, kind = idx % 3;
    if (kind == 0)
      st.b[i] = __builtin_amdgcn_raw_buffer_load_b128(r.wr, boff[i] | dead, k0 >> 1, 0);
    else if (kind == 1)
      st.s[i] = __builtin_amdgcn_raw_buffer_load_b16(r.sr, ((soff[i] & 0x7fffffffu) * 2u) | (soff[i] & 0x80000000u) | dead,
                                                     (k0 >> 7) * 2u, 0);
    else          // without zero-points the resource is empty and the load returns 0
      st.z[i] = __builtin_amdgcn_raw_buffer_load_b8(r.zr, soff[i] | dead, k0 >> 7, 0);
  }
  static __device__ __forceinline__ void begin(const Res& r, const Stage& st, Dq& q) {
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      const _Float16 sc = __builtin_bit_cast(_Float16, (uint16_t)st.s[i]);
      const float z = r.has_zp ? (float)st.z[i] : 8.0f;
      q.sf[i] = (float)sc * 512.0f;
      q.nzs[i] = -z * (float)sc;
    }
  }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    if constexpr (Act::dt == DT_F16) {
      const f16x2 r = {(_Float16)a, (_Float16)b};
      return __builtin_bit_cast(uint32_t, r);
    } else {
      const bf16x2 r = {(__bf16)a, (__bf16)b};
      return __builtin_bit_cast(uint32_t, r);
    }
  }
  // piece I of the stage; dst[i] = LDS address of chunk i's 64 output bytes in the target buffer
  static __device__ __forceinline__ void piece(const Stage& st, Dq& q, int I, unsigned char* const (&dst)[B_CH]) {
    const int dword = I >> 3, part = I & 7;
    const int i = dword / 4, dw = dword % 4;
    auto pair = [&](float a, float b) {
      return pack2(__builtin_fmaf(a, q.sf[i], q.nzs[i]), __builtin_fmaf(b, q.sf[i], q.nzs[i]));
    };
    if (part == 0) {
      const uint32_t w = st.b[i][dw];
      q.e = w & 0x0F0F0F0Fu;
      q.o = (w >> 4) & 0x0F0F0F0Fu;
    } else if (part == 7) {
      *reinterpret_cast<u32x4*>(dst[i] + dw * 16) = q.outv;
    } else if (part == 1) {
      q.fe = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.e, false);
      q.fo = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.o, false);
    } else if (part == 4) {
      q.fe = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.e, true);
      q.fo = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.o, true);
    } else if (part == 2) q.outv[0] = pair(q.fe[0], q.fo[0]);
    else if (part == 3) q.outv[1] = pair(q.fe[1], q.fo[1]);
    else if (part == 5) q.outv[2] = pair(q.fe[0], q.fo[0]);
    else q.outv[3] = pair(q.fe[1], q.fo[1]);
  }
  static __device__ __forceinline__ float out_scale(const Res&, const GemmArgs&, int) { return 1.0f; }
};

// ------------------------------------------------------------------ GGUF Q4_K (repacked)
// The int4 nibble layout with an fp16 scale and an fp16 min per 32 k = per chunk:
// w = fp16(fp16(nib * scale) - min), the product rounded before the subtraction (two roundings,
// as the dense dequantization does).  The product is formed in fp32 (exact: 4 x 11 significant
// bits) and rounded once to fp16, which is the fp16 product; the subtraction is the one packed
// fp16 instruction left per pair (packed 16-bit arithmetic does not hide behind the MFMAs, see
// INT4 above).  fp16 activations only.
template <class Act, int BN>
struct WQ4K {
  static_assert(Act::dt == DT_F16, "Q4_K runs in fp16");
  static constexpr int CPR = 2;
  static constexpr double kWeightBytesPerK = 0.5;
  static constexpr int B_CH = (BN * CPR + 255) / 256;
  static constexpr int LPC = 3;
  static constexpr int PPD = 12;                      // pieces per dword of 8 nibbles
  static constexpr int kPieces = B_CH * 4 * PPD;
  static constexpr bool kOutScale = false;
  static constexpr bool kPermK = false;
  struct Res {
    __amdgpu_buffer_rsrc_t wr, sr, mr;
    int Kc;
  };
  struct Stage {
    u32x4 b[B_CH];
    uint32_t s[B_CH], m[B_CH];                        // fp16 bits (32-bit slots: 16-bit members end up on the stack)
  };
  struct Dq {
    uint32_t e, o, t;
    f32x2 fe, fo;
    u32x4 outv;
    float sf[B_CH];                                   // 512 * scale
    f16x2 mv[B_CH];
  };
  static __device__ __forceinline__ Res make(const GemmArgs& p, int = 0) {
    Res r;
    r.Kc = p.K >> 5;
    r.wr = make_rsrc(p.w, (uint32_t)p.N * ((uint32_t)p.K >> 1));
    r.sr = make_rsrc(p.scale, (uint32_t)p.N * (uint32_t)r.Kc * 2u);
    r.mr = make_rsrc(p.zp, (uint32_t)p.N * (uint32_t)r.Kc * 2u);
    return r;
  }
  static __device__ __forceinline__ void chunk_addr(const Res& r, int n, int kc, int K, uint32_t& boff, uint32_t& soff) {
    boff = (uint32_t)n * ((uint32_t)K >> 1) + (uint32_t)(kc * 16);
    soff = ((uint32_t)n * (uint32_t)r.Kc + (uint32_t)kc) * 2u;   // bytes: one fp16 per 32 k
  }
  static __device__ __forceinline__ void load1(const Res& r, Stage& st, const uint32_t (&boff)[B_CH],
                                               const uint32_t (&soff)[B_CH], int kt, uint32_t dead, int idx) {
    const uint32_t k0 = (uint32_t)kt * kBK;
    const int i = idx / 3, kind = idx % 3;
    if (kind == 0) st.b[i] = __builtin_amdgcn_raw_buffer_load_b128(r.wr, boff[i] | dead, k0 >> 1, 0);
    else if (kind == 1) st.s[i] = __builtin_amdgcn_raw_buffer_load_b16(r.sr, soff[i] | dead, (k0 >> 5) * 2u, 0);
    else st.m[i] = __builtin_amdgcn_raw_buffer_load_b16(r.mr, soff[i] | dead, (k0 >> 5) * 2u, 0);
  }
  static __device__ __forceinline__ void begin(const Res&, const Stage& st, Dq& q) {
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      const _Float16 mn = __builtin_bit_cast(_Float16, (uint16_t)st.m[i]);
      q.sf[i] = (float)__builtin_bit_cast(_Float16, (uint16_t)st.s[i]) * 512.0f;   // exact: a power of two
      q.mv[i] = f16x2{mn, mn};
    }
  }
  static __device__ __forceinline__ void piece(const Stage& st, Dq& q, int I, unsigned char* const (&dst)[B_CH]) {
#pragma clang fp contract(off)
    const int dword = I / PPD, part = I % PPD;
    const int i = dword / 4, dw = dword % 4;
    // nib * 2^-9 times 512 s = nib * s exactly in fp32; one RNE to fp16 = the fp16 product
    auto prod = [&](float a, float b) {
      const f16x2 r = {(_Float16)(a * q.sf[i]), (_Float16)(b * q.sf[i])};
      return __builtin_bit_cast(uint32_t, r);
    };
    auto sub_min = [&](uint32_t v) { return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, v) - q.mv[i]); };
    if (part == 0) {
      const uint32_t w = st.b[i][dw];
      q.e = w & 0x0F0F0F0Fu;
      q.o = (w >> 4) & 0x0F0F0F0Fu;
    } else if (part == 1) {
      q.fe = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.e, false);
      q.fo = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.o, false);
    } else if (part == 6) {
      q.fe = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.e, true);
      q.fo = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.o, true);
    } else if (part == 2 || part == 7) q.t = prod(q.fe[0], q.fo[0]);
    else if (part == 4 || part == 9) q.t = prod(q.fe[1], q.fo[1]);
    else if (part == 3) q.outv[0] = sub_min(q.t);
    else if (part == 5) q.outv[1] = sub_min(q.t);
    else if (part == 8) q.outv[2] = sub_min(q.t);
    else if (part == 10) q.outv[3] = sub_min(q.t);
    else *reinterpret_cast<u32x4*>(dst[i] + dw * 16) = q.outv;
  }
  static __device__ __forceinline__ float out_scale(const Res&, const GemmArgs&, int) { return 1.0f; }
};

// ------------------------------------------------------------------ FP8 E4M3
// 16 codes per 16-byte chunk, four chunks per row and step.  BLOCK = false: the decode is exact
// (every E4M3 value is a 16-bit float) and the per-channel or per-tensor scale multiplies the
// finished sum.  BLOCK = true: one fp32 scale per 128 x 128 block, folded into the weight
// (decode to fp32, multiply, one rounding to the activation type) because the accumulators
// cannot be rescaled per K block.
template <class Act, int BN, bool BLOCK>
struct WFp8 {
  static constexpr int CPR = 4;
  static constexpr double kWeightBytesPerK = 1.0;
  static constexpr int B_CH = (BN * CPR + 255) / 256;
  static constexpr int LPC = BLOCK ? 2 : 1;
  static constexpr int kPPC = BLOCK ? 10 : 4;         // pieces per chunk
  static constexpr int kPieces = B_CH * kPPC;
  static constexpr bool kOutScale = !BLOCK;
  static constexpr bool kPermK = false;
  struct Res {
    __amdgpu_buffer_rsrc_t wr, sr;
    const void* se;                                   // this expert's scales
    int Kb;
  };
  struct Stage {
    u32x4 b[B_CH];
    uint32_t s[BLOCK ? B_CH : 1];                     // block scale, fp32 bits
  };
  struct Dq {
    u32x4 outv;
  };
  // e: expert of a grouped launch (its matrices start e * stride bytes in)
  static __device__ __forceinline__ Res make(const GemmArgs& p, int e = 0) {
    Res r;
    r.Kb = (p.K + 127) >> 7;
    r.wr = make_rsrc((const char*)p.w + (long long)e * p.g_w_stride, (uint32_t)p.N * (uint32_t)p.K);
    r.sr = make_rsrc((const char*)p.scale + (long long)e * p.g_s_stride,
                     BLOCK ? (uint32_t)((p.N + 127) >> 7) * (uint32_t)r.Kb * 4u : 0u);
    r.se = (const char*)p.scale + (long long)e * p.g_s_stride;
    return r;
  }
  static __device__ __forceinline__ void chunk_addr(const Res& r, int n, int kc, int K, uint32_t& boff, uint32_t& soff) {
    boff = (uint32_t)n * (uint32_t)K + (uint32_t)(kc * 16);
    soff = (uint32_t)(n >> 7) * (uint32_t)r.Kb * 4u;  // bytes: the row block's first scale
  }
  static __device__ __forceinline__ void load1(const Res& r, Stage& st, const uint32_t (&boff)[B_CH],
                                               const uint32_t (&soff)[B_CH], int kt, uint32_t dead, int idx) {
    const uint32_t k0 = (uint32_t)kt * kBK;
    const int i = idx / LPC, kind = idx % LPC;
    if (kind == 0) st.b[i] = __builtin_amdgcn_raw_buffer_load_b128(r.wr, boff[i] | dead, k0, 0);
    else st.s[i] = __builtin_amdgcn_raw_buffer_load_b32(r.sr, soff[i] | dead, (k0 >> 7) * 4u, 0);
  }
  static __device__ __forceinline__ void begin(const Res&, const Stage&, Dq&) {}
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    if constexpr (Act::dt == DT_F16) {
      const f16x2 r = {(_Float16)a, (_Float16)b};
      return __builtin_bit_cast(uint32_t, r);
    } else {
      const bf16x2 r = {(__bf16)a, (__bf16)b};
      return __builtin_bit_cast(uint32_t, r);
    }
  }
  static __device__ __forceinline__ void piece(const Stage& st, Dq& q, int I, unsigned char* const (&dst)[B_CH]) {
    const int i = I / kPPC, part = I % kPPC;
    if constexpr (!BLOCK) {
      // piece = one dword of four codes -> two packed pairs; a 16-byte write after every second
      const uint32_t w = st.b[i][part];
      uint32_t p0, p1;
      if constexpr (Act::dt == DT_F16) {
        p0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false));
        p1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true));
      } else {
        p0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
        p1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true));
      }
      q.outv[(part & 1) * 2] = p0;
      q.outv[(part & 1) * 2 + 1] = p1;
      if (part & 1) *reinterpret_cast<u32x4*>(dst[i] + (part >> 1) * 16) = q.outv;
    } else {
      // pieces 0-3 and 5-8: half a dword (two codes) -> fp32, scale, one rounding; 4 and 9: write
      const int half = part / 5, sub = part % 5;
      if (sub == 4) {
        *reinterpret_cast<u32x4*>(dst[i] + half * 16) = q.outv;
      } else {
        const uint32_t w = st.b[i][half * 2 + (sub >> 1)];
        const f32x2 f = (sub & 1) ? __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true)
                                  : __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
        const float sc = __builtin_bit_cast(float, st.s[i]);
        q.outv[sub] = pack2(f[0] * sc, f[1] * sc);
      }
    }
  }
  static __device__ __forceinline__ float out_scale(const Res& r, const GemmArgs& p, int n) {
    if (p.scale_mode == 1) return ((const float*)r.se)[0];
    if (p.scale_mode == 3) return ((const float*)r.se)[n >= p.n_half ? 1 : 0];
    return p.scale_f16 ? (float)((const _Float16*)r.se)[n] : ((const float*)r.se)[n];
  }
};

// ------------------------------------------------------------------ kernel
// GROUPED: the M-tiles come from a device-built table of (expert, rows) instead of a regular grid
// (MoE: rows sorted by expert, one weight matrix per expert).  FUSE: the tile's weight rows
// alternate, 16 at a time, between a gate block and the up block n_half rows further on, and the
// epilogue writes act(gate) * up (N / 2 output columns).
template <class Act, class Fmt, int BM, int BN, bool GROUPED = false, bool FUSE = false>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const GemmArgs p) {
  using Elem = typename Act::elem;
  constexpr int WM = BM / 2, WN = BN / 2;             // wave sub-tile
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int B_CH = Fmt::B_CH;                     // 16-byte weight chunks of the tile per thread
  constexpr int CPR = Fmt::CPR;
  constexpr int BNP = B_CH * 256 / CPR;               // LDS rows of the weight tile (>= BN)
  constexpr int kLoads = Fmt::LPC * B_CH;             // load instructions per stage and thread
  static_assert(WM % 16 == 0 && WN % 16 == 0 && BNP >= BN, "tile shape");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  Elem* Bs = reinterpret_cast<Elem*>(smem);                                   // [2][BNP][kPitch]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 15, g = lane >> 4;
  const int wn0 = (wave & 1) * WN;

  // Tile order.  The 8 XCDs take workgroups round-robin and each has its own L2, so the tile of a
  // workgroup is derived from (XCD = id % 8, slot on that XCD = id / 8):
  //   dense: the XCDs form an xcd_m x (8 / xcd_m) grid over the tile matrix and each walks its
  //     block of it M-tile first, so that the workgroups resident on an XCD share a few weight
  //     tiles and a few slabs of x and every operand byte is fetched by as few L2s as possible
  //     (xcd_m = 0: plain order, consecutive workgroups share the weight tile);
  //   grouped: XCD x owns one M-tile of every 8 and walks the N-tiles of one M-tile
  //     back to back, so an M-tile's activations are fetched into one L2 once (its N-tiles read
  //     different weight rows: there is nothing else to share).
  int tm, tn;
  if constexpr (GROUPED) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int round = slot / p.tiles_n;               // rotate, so that no XCD gets all the experts' short last tiles
    tm = round * 8 + ((xcd + round) & 7);
    tn = slot - round * p.tiles_n;
  } else if (p.xcd_m) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int per_m = p.tiles_m / p.xcd_m, per_n = p.tiles_n / (8 / p.xcd_m);
    tm = (xcd % p.xcd_m) * per_m + slot % per_m;
    tn = (xcd / p.xcd_m) * per_n + slot / per_m;
  } else {
    tn = blockIdx.x / p.tiles_m;
    tm = blockIdx.x - tn * p.tiles_m;
  }
  int m0 = tm * BM;
  const int n0 = FUSE ? tn * (BN / 2) : tn * BN;      // FUSE: first gate row of the tile
  int M = p.M;
  const int N = p.N, K = p.K;
  const int KT = K / kBK;                             // 64-wide steps (even: K % 128 == 0)
  const int Q = K / 32;                               // 32-wide MFMA steps
  int expert = 0, row0 = 0, xblk0 = 0;
  if constexpr (GROUPED) {
    if (tm >= p.g_count[0]) return;                   // the grid is an upper bound of the tile count
    expert = p.g_tile[4 * tm];
    row0 = p.g_tile[4 * tm + 1];
    M = p.g_tile[4 * tm + 2];                         // rows of this tile
    xblk0 = p.g_tile[4 * tm + 3];
    m0 = 0;
  }

  const int Mp = (p.M + 15) & ~15;
  const uint32_t xtiles = GROUPED ? (uint32_t)p.x_blocks : (uint32_t)(Mp >> 4);
  const __amdgpu_buffer_rsrc_t xr = make_rsrc(p.x, xtiles * 16u * (uint32_t)K * 2u);
  const typename Fmt::Res res = Fmt::make(p, expert);
  // 16-row activation tile b of this wavefront inside the BM-row tile.  GROUPED: the two wavefront
  // rows take the tiles alternately and a wavefront multiplies only the first TM, TM / 2 or TM / 4 of
  // its tiles, whichever covers the `live` ones with rows of the expert in them (the K loop exists
  // in these three lengths; a branch per MFMA costs more than it saves), so a short last tile of an
  // expert costs a fraction of the matrix-core time.
  const int wr = wave >> 1;
  auto mtile = [&](int b) { return GROUPED ? 2 * b + wr : wr * TM + b; };
  int live = TM;
  if constexpr (GROUPED) live = __builtin_amdgcn_readfirstlane((((M + 15) >> 4) - wr + 1) >> 1);
  // weight row of row r of the LDS tile
  auto tile_row = [&](int r) { return FUSE ? n0 + (r >> 5) * 16 + (r & 15) + ((r >> 4) & 1) * p.n_half : n0 + r; };

  f32x4 acc[TN][TM];
#pragma unroll
  for (int a = 0; a < TN; ++a)
#pragma unroll
    for (int b = 0; b < TM; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- activations: register ring.  Block (16-row tile t, 32-wide step q) of the
  // re-tiled x sits at (t * Q + q) * 1024; tile and step enter as a scalar offset.
  const uint32_t xlane = (uint32_t)lane * 16u;
  const uint32_t xtile0 = (uint32_t)xblk0 + (uint32_t)(m0 >> 4);
  u32x4 xring[4][TM];
  uint32_t xtoff[TM];                                 // scalar: byte offset of tile b's block row
#pragma unroll
  for (int b = 0; b < TM; ++b) {
    const uint32_t t = xtile0 + mtile(b) < xtiles ? xtile0 + mtile(b) : xtiles - 1;   // tiles past M: any valid block
    xtoff[b] = __builtin_amdgcn_readfirstlane(t * (uint32_t)Q * 1024u);
  }
  auto load_x1 = [&](int slot, int b, int q) {        // a step beyond the last re-reads the last (never used)
    const uint32_t qc = (uint32_t)(q < Q ? q : Q - 1);
    xring[slot][b] = __builtin_amdgcn_raw_buffer_load_b128(xr, xlane, xtoff[b] + qc * 1024u, 0);
  };
  auto load_x = [&](int slot, int q) {
#pragma unroll
    for (int b = 0; b < TM; ++b) load_x1(slot, b, q);
  };

  // ---- weights: per-thread chunk addresses at k = 0
  uint32_t boff[B_CH], soff[B_CH];
  unsigned char* blds[B_CH];
#pragma unroll
  for (int i = 0; i < B_CH; ++i) {
    const int c = tid + i * 256;
    const int row = c / CPR, kc = c % CPR;
    const int n = tile_row(row);
    const bool live = FUSE ? (n0 + (row >> 5) * 16 + (row & 15) < p.n_half) : (n < N);
    const uint32_t dead = (uint32_t)(!(live && row < BN)) << 31;
    Fmt::chunk_addr(res, n, kc, K, boff[i], soff[i]);
    boff[i] |= dead;
    soff[i] |= dead;
    blds[i] = smem + (row * kPitch + kc * (kBK / CPR)) * 2;
  }
  using StageB = typename Fmt::Stage;                 // weight chunks of one 64-wide step, in registers
  // One of the loads of a stage, so that the main loop can issue them one at a time between
  // MFMAs: a wavefront that issues vector-memory instructions back to back stalls ~35 cycles
  // on each.
  auto load_b1 = [&](StageB& st, int kt, int idx) {
    const uint32_t dead = kt < KT ? 0u : 0x80000000u;
    Fmt::load1(res, st, boff, soff, kt, dead, idx);
  };
  auto load_b = [&](StageB& st, int kt) {
#pragma unroll
    for (int idx = 0; idx < kLoads; ++idx) load_b1(st, kt, idx);
  };

  constexpr int kPieces = Fmt::kPieces;
  using DqState = typename Fmt::Dq;
  constexpr size_t kBufBytes = (size_t)BNP * kPitch * 2;
  auto dq_piece = [&](const StageB& st, int buf, int I, DqState& q) {
    unsigned char* dst[B_CH];
#pragma unroll
    for (int i = 0; i < B_CH; ++i) dst[i] = blds[i] + buf * kBufBytes;
    Fmt::piece(st, q, I, dst);
  };

  // One 64-wide K step: multiply out of LDS buffer `buf` (two 32-wide MFMA steps,
  // ring slots slot0 and slot0 + 1) while the next step's weights (`cur`, loaded one
  // step earlier) are dequantized into the other buffer and the weights two steps
  // ahead are fetched into `nxt`.
  // pieces are spread evenly over the MFMAs of the step: piece I goes behind the
  // first MFMA slot with (slot + 1) * kPieces / kMfmas > I
  auto step64 = [&](auto live_c, int kt, int buf, int slot0, StageB& cur, StageB& nxt) __attribute__((always_inline)) {
    constexpr int L = decltype(live_c)::value;        // activation tiles multiplied (<= TM)
    constexpr int kMfmas = 2 * TN * L;
    const Elem* Bb = Bs + buf * BNP * kPitch;
    DqState q;
    Fmt::begin(res, cur, q);
    auto rd_w = [&](int a, int s) {
      return *reinterpret_cast<const u32x4*>(Bb + (wn0 + a * 16 + j) * kPitch + s * 32 + g * 8);
    };
    // the weight operand of row a + 1 is fetched from LDS while row a is multiplied
    u32x4 wnext = rd_w(0, 0);
    constexpr int kHalf = TN * L;                     // MFMAs per 32-wide step
    constexpr int kXEvery = kHalf / L;                // one activation load per kXEvery MFMAs
    constexpr int kBEvery = kHalf / kLoads > 0 ? kHalf / kLoads : 1;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
      for (int a = 0; a < TN; ++a) {
        const u32x4 wcur = wnext;
        if (a + 1 < TN) wnext = rd_w(a + 1, s);
        else if (s == 0) wnext = rd_w(0, 1);
#pragma unroll
        for (int b = 0; b < L; ++b) {
          mfma_agpr<Act>(acc[a][b], wcur, xring[slot0 + s][b]);
          const int m = a * L + b;                    // MFMA index inside this 32-wide step
          const int slot = s * kHalf + m;
          const int p0 = slot * kPieces / kMfmas, p1 = (slot + 1) * kPieces / kMfmas;
#pragma unroll
          for (int I = p0; I < p1; ++I) dq_piece(cur, buf ^ 1, I, q);
          // global loads, one at a time: the ring slot multiplied in the previous
          // 32-wide step is refilled 3 steps ahead, and in the first half the weight
          // chunks two 64-wide steps ahead are fetched
          if (m % kXEvery == kXEvery / 2 && m / kXEvery < L)
            load_x1((slot0 + s + 3) & 3, m / kXEvery, 2 * kt + s + 3);
          if (s == 0 && m % kBEvery == 0 && m / kBEvery < kLoads) load_b1(nxt, kt + 2, m / kBEvery);
          // keep MFMAs, vector-ALU pieces and memory accesses in this order
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    __syncthreads();
  };

  StageB s0, s1;
  load_b(s0, 0);
  __builtin_amdgcn_sched_barrier(0);
  load_b(s1, 1);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    __builtin_amdgcn_sched_barrier(0);               // keep the ring's loads in issue order
    load_x(r, r);
  }
  {
    DqState q;
    Fmt::begin(res, s0, q);
#pragma unroll
    for (int I = 0; I < kPieces; ++I) dq_piece(s0, 0, I, q);
  }
  __syncthreads();
  auto k_loop = [&](auto live_c) __attribute__((always_inline)) {
    for (int kt = 0; kt < KT; kt += 2) {
      step64(live_c, kt, 0, 0, s1, s0);
      step64(live_c, kt + 1, 1, 2, s0, s1);
    }
  };
  if constexpr (!GROUPED) {
    k_loop(std::integral_constant<int, TM>{});
  } else {
    if (live > TM / 2) k_loop(std::integral_constant<int, TM>{});
    else if (live > TM / 4) k_loop(std::integral_constant<int, TM / 2>{});
    else k_loop(std::integral_constant<int, (TM / 4 > 0 ? TM / 4 : 1)>{});
  }

  // the last MFMAs are still in the matrix pipe: wait before reading their results
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  // D = W-tile (rows n) x X-tile^T: lane holds n = 4 g + v (v = 0..3), m = j
  Elem* out = (Elem*)p.out;
  const int n_out = FUSE ? p.n_half : N;              // output columns
  // output row of this lane's row of activation tile b, or -1
  int orow[TM];
  float rw[TM];
#pragma unroll
  for (int b = 0; b < TM; ++b) {
    const int m = m0 + mtile(b) * 16 + j;
    orow[b] = m < M ? m : -1;
    rw[b] = 1.0f;
    if constexpr (GROUPED) {
      if (m < M) {
        const int pos = row0 + m;
        const int dst = p.out_map ? p.out_map[pos] : pos;
        orow[b] = (unsigned)dst < (unsigned)p.out_rows ? dst : -1;   // a mapped row outside the output is dropped
        if (p.row_weight && orow[b] >= 0) rw[b] = Act::to_f32(((const Elem*)p.row_weight)[dst]);
      }
    }
  }
  constexpr int TNO = FUSE ? TN / 2 : TN;             // output column tiles of this wavefront
  // first of this lane's 4 output columns in column tile ao; FUSE: gate tile 2 ao pairs with up tile 2 ao + 1
  auto col_of = [&](int ao) { return FUSE ? n0 + (wn0 >> 1) + ao * 16 + g * 4 : n0 + wn0 + ao * 16 + g * 4; };
  [[maybe_unused]] float os_all[Fmt::kOutScale ? TNO : 1][4];
  [[maybe_unused]] float os_up = 1.0f;
  if constexpr (Fmt::kOutScale) {
    if constexpr (FUSE) os_up = Fmt::out_scale(res, p, p.n_half);
#pragma unroll
    for (int ao = 0; ao < TNO; ++ao)
#pragma unroll
      for (int v = 0; v < 4; ++v) os_all[ao][v] = Fmt::out_scale(res, p, col_of(ao) + v < N ? col_of(ao) + v : N - 1);
  }
  const bool two_scales = p.scale_mode == 3;
  // the lane's 4 results of (row tile b, column tile ao), before the rounding
  auto result4 = [&](auto gelu_c, int b, int ao, float (&r)[4]) __attribute__((always_inline)) {
    const int a = FUSE ? 2 * ao : ao;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const float osv = Fmt::kOutScale ? os_all[Fmt::kOutScale ? ao : 0][v] : 1.0f;
      if constexpr (FUSE) {
        // one factor per tensor / expert, or one for the gate rows and one for the up rows
        const float gate = acc[a][b][v] * osv, up = acc[a + 1][b][v] * (two_scales ? os_up : osv);
        if constexpr (decltype(gelu_c)::value) {
          float two_z = 2.0f * (0.7978845608f * (gate + 0.044715f * (gate * gate * gate)));
          two_z = fminf(fmaxf(two_z, -30.0f), 30.0f);
          const float ex = __expf(two_z);
          r[v] = 0.5f * gate * (1.0f + (ex - 1.0f) / (ex + 1.0f)) * up;
        } else {
          r[v] = gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up;   // reciprocal to 1 ulp, before a 16-bit rounding
        }
      } else {
        r[v] = Fmt::kOutScale ? acc[a][b][v] * osv : acc[a][b][v];
      }
      if constexpr (GROUPED) r[v] *= rw[b];
    }
  };
  const size_t out_bytes = (size_t)(GROUPED ? p.out_rows : p.M) * (size_t)n_out * 2u;
  constexpr int WNO = FUSE ? WN / 2 : WN;             // output columns of this wavefront
  constexpr int LPR = WNO / 8;                        // lanes, 16 bytes each, per output row of the wave tile
  constexpr int RPP = 64 / LPR;                       // rows per store instruction
  constexpr int PASSES = (16 + RPP - 1) / RPP;
  constexpr int OPITCH = WNO * 2 + 16;                // a row of the wave tile + a slot for the row's offset
  static_assert(WNO % 8 == 0 && 4 * 16 * OPITCH <= 2 * BNP * kPitch * 2, "output staging tile");
  if ((n_out & 7) == 0 && out_bytes < (1ull << 31) && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0) {
    // Each 16-row tile of results is rounded, turned through a tile in LDS that belongs to this
    // wavefront alone (the weight tiles are free after the K loop's last barrier; the LDS queue of a
    // wavefront runs in order, so no barrier) and leaves as 16 bytes per lane, a row's columns in
    // adjacent lanes: a store instruction writes RPP rows of WNO * 2 contiguous bytes instead of 32
    // bytes in each of 16 rows — the workgroup's path to L2 takes a request per row piece, whatever
    // its size.  Rows and column groups outside the output get an offset past the buffer and are dropped.
    const __amdgpu_buffer_rsrc_t orsrc = make_rsrc(p.out, (uint32_t)out_bytes);
    unsigned char* otile = smem + wave * (16 * OPITCH);
    unsigned char* wr_at = otile + j * OPITCH + g * 8;
    const int rr = lane / LPR, cc = lane - rr * LPR;
    const int colr = (FUSE ? n0 + (wn0 >> 1) : n0 + wn0) + cc * 8;     // this lane's 8 columns when it stores
    const bool lane_ok = rr < RPP && colr < n_out;
    auto emit = [&](auto gelu_c) __attribute__((always_inline)) {
#pragma unroll
      for (int b = 0; b < TM; ++b) {
        if (GROUPED && b >= live) break;              // uniform: the tiles past the expert's rows
        *reinterpret_cast<uint32_t*>(otile + j * OPITCH + WNO * 2) =
            orow[b] >= 0 ? (uint32_t)orow[b] * (uint32_t)n_out * 2u : kOOB;
#pragma unroll
        for (int ao = 0; ao < TNO; ++ao) {
          float r[4];
          result4(gelu_c, b, ao, r);
          u32x2 d;
          if constexpr (Act::dt == DT_F16) {
            d[0] = __builtin_bit_cast(uint32_t, f16x2{(_Float16)r[0], (_Float16)r[1]});
            d[1] = __builtin_bit_cast(uint32_t, f16x2{(_Float16)r[2], (_Float16)r[3]});
          } else {
            d[0] = __builtin_bit_cast(uint32_t, bf16x2{(__bf16)r[0], (__bf16)r[1]});
            d[1] = __builtin_bit_cast(uint32_t, bf16x2{(__bf16)r[2], (__bf16)r[3]});
          }
          *reinterpret_cast<u32x2*>(wr_at + ao * 32) = d;
        }
        if constexpr (GROUPED && WNO % 32 == 0) {
          if (p.out_packed) {
            // block (activation tile, 32-wide step) = 1 KiB in operand order: lane 16 g + j holds row j,
            // columns 8 g .. 8 g + 7 of the step; rows past the expert's last are zeros here (their
            // activations were) as the re-tiling pass would write them
            const uint32_t tile = (uint32_t)xblk0 + (uint32_t)mtile(b);
            const int cb = FUSE ? n0 + (wn0 >> 1) : n0 + wn0;
#pragma unroll
            for (int qq = 0; qq < WNO / 32; ++qq) {
              const u32x4 v = *reinterpret_cast<const u32x4*>(otile + j * OPITCH + (qq * 32 + g * 8) * 2);
              const uint32_t q = (uint32_t)(cb >> 5) + qq;
              __builtin_amdgcn_raw_buffer_store_b128(
                  v, orsrc, cb + qq * 32 < n_out ? (tile * (uint32_t)(n_out >> 5) + q) * 1024u + (uint32_t)lane * 16u : kOOB, 0, 0);
            }
            continue;
          }
        }
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
          const int row = ps * RPP + rr;
          const unsigned char* src = otile + (row < 16 ? row : 15) * OPITCH;
          const u32x4 v = *reinterpret_cast<const u32x4*>(src + cc * 16);
          const uint32_t ro = *reinterpret_cast<const uint32_t*>(src + WNO * 2);
          const bool ok = lane_ok && row < 16;
          __builtin_amdgcn_raw_buffer_store_b128(v, orsrc, ok ? ro + (uint32_t)colr * 2u : kOOB, 0, 0);
        }
      }
    };
    if (FUSE && p.gelu) emit(std::true_type{});
    else emit(std::false_type{});
  } else {
    auto emit = [&](auto gelu_c) __attribute__((always_inline)) {
#pragma unroll
      for (int b = 0; b < TM; ++b) {
        if (orow[b] < 0) continue;
#pragma unroll
        for (int ao = 0; ao < TNO; ++ao) {
          const int n = col_of(ao);
          float r[4];
          result4(gelu_c, b, ao, r);
          Elem* dst = out + (size_t)orow[b] * n_out + n;
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (n + v < n_out) dst[v] = Act::from_f32(r[v]);
        }
      }
    };
    if (FUSE && p.gelu) emit(std::true_type{});
    else emit(std::false_type{});
  }
}

// Re-tile x [M, K] (16-bit, row-major) into MFMA operand order: block (t, q) holds
// rows 16 t .. 16 t + 15, k = 32 q .. 32 q + 31; lane l = 16 g + j of the block
// (16 bytes at l * 16) holds row 16 t + j, k = 32 q + 8 g .. + 7.  Rows past M are
// zero.  One workgroup writes four blocks, contiguously.  (Reading the rows contiguously and
// turning them through an LDS tile, as the grouped variant does, was measured slower here:
// 9.1 against 7.3 us for 2048 x 4096.)
// perm_k: the 8 elements of a lane leave in the order 0 4 1 5 2 6 3 7 (weight formats whose
// dequantization produces that order).
constexpr int kPackQ = 16;                            // grouped variant: 32-wide steps per workgroup
constexpr int kPackPitch = kPackQ * 64 + 16;          // and its LDS row pitch (operand reads hit distinct banks)
static __global__ __launch_bounds__(256) void pack_x_kernel(const uint16_t* __restrict__ x, u32x4* __restrict__ xp,
                                                            int M, int K, int Q, int perm_k) {
  const int l = threadIdx.x & 63;
  const int nq4 = (Q + 3) >> 2;                       // flat grid: 4 steps of one row tile per workgroup
  const int t = blockIdx.x / nq4;
  const int q = (blockIdx.x - t * nq4) * 4 + (threadIdx.x >> 6);
  if (q >= Q) return;
  const int m = t * 16 + (l & 15);
  u32x4 v = {0u, 0u, 0u, 0u};
  if (m < M) v = *reinterpret_cast<const u32x4*>(x + (size_t)m * K + q * 32 + (l >> 4) * 8);
  if (perm_k) {
    // dwords hold (x0 x1)(x2 x3)(x4 x5)(x6 x7) -> (x0 x4)(x1 x5)(x2 x6)(x3 x7)
    const uint32_t d0 = v[0], d1 = v[1], d2 = v[2], d3 = v[3];
    v = u32x4{__builtin_amdgcn_perm(d2, d0, 0x05040100u), __builtin_amdgcn_perm(d2, d0, 0x07060302u),
              __builtin_amdgcn_perm(d3, d1, 0x05040100u), __builtin_amdgcn_perm(d3, d1, 0x07060302u)};
  }
  xp[((size_t)t * Q + q) * 64 + l] = v;
}

template <class Act, class Fmt, int BM, int BN>
static int launch_gemm_tiled(GemmArgs p, hipStream_t st) {
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  // XCD grid: among the splits that divide both tile counts, the one with the least operand
  // traffic (a weight tile is fetched by xcd_m L2s, a slab of x by 8 / xcd_m)
  p.xcd_m = 0;
  {
    const double wbytes = (double)p.N * p.K * Fmt::kWeightBytesPerK, xbytes = (double)p.M * p.K * 2.0;
    double best = 0.0;
    for (int a = 1; a <= 8; a *= 2) {
      if (p.tiles_m % a || p.tiles_n % (8 / a)) continue;
      const double cost = a * wbytes + (8 / a) * xbytes;
      if (!p.xcd_m || cost < best) { best = cost; p.xcd_m = a; }
    }
  }
  const size_t lds = (size_t)2 * (Fmt::B_CH * 256 / Fmt::CPR) * kPitch * 2;
  auto kern = gemm_tiled_kernel<Act, Fmt, BM, BN>;
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

// Per K step a workgroup pays for its tile's columns (MFMAs) plus a part that does not shrink with
// the tile (activation loads, barrier, pipeline fill): measured on 5120 x 5120 and 14336 x 4096
// weights, 160- and 192-column tiles cost about (BN + 48) / (256 + 48) of a 256-column tile.
constexpr long kTileFixedCols = 48;

static inline long device_cu_count_gemm() {
  static int cus = 0;
  if (!cus) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      cus = prop.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

// Re-tiles x into `workspace` and runs the tile shape that fits the problem: 128 x 128 tiles
// while 256-row tiles would leave more than half of the chip idle, else 256 rows x 256 / 224 /
// 192 / 160 columns, whichever needs the least time over its rounds of resident workgroups (a
// 5120-column weight is 32 tiles of 160: with 8 row tiles exactly one round of 256 workgroups,
// where 256-column tiles fill 160 of the 256 CUs).  FMT is a template taking (Act, BN).
template <class Act, template <class, int> class FMT>
static int run_gemm_tiled(GemmArgs p, const void* x, void* workspace, hipStream_t st) {
  const int Mp = (p.M + 15) & ~15;
  const int Q = p.K / 32;
  hipLaunchKernelGGL(pack_x_kernel, dim3((unsigned)(((Q + 3) / 4) * (Mp / 16))), dim3(256), 0, st, (const uint16_t*)x,
                     (u32x4*)workspace, p.M, p.K, Q, FMT<Act, 128>::kPermK ? 1 : 0);
  p.x = workspace;
  // 256-row tiles once they occupy more than half of the CUs (a 128 x 128 tile does a quarter of the
  // work per weight and activation byte it moves and runs at about a third of the rate)
  const long cus = device_cu_count_gemm();
  const long tiles_m = (p.M + 255) / 256;
  const bool big = p.M > 128 && tiles_m * ((p.N + 255) / 256) * 2 > cus;
  if (!big) return launch_gemm_tiled<Act, FMT<Act, 128>, 128, 128>(p, st);
  // time ~ rounds of resident workgroups x (columns of a tile + a fixed part per K step)
  auto cost = [&](long bn) { return ((tiles_m * ((p.N + bn - 1) / bn) + cus - 1) / cus) * (bn + kTileFixedCols); };
  long best = 256;
  for (long bn : {224L, 192L, 160L})
    if (cost(bn) < cost(best)) best = bn;
  if (best == 160) return launch_gemm_tiled<Act, FMT<Act, 160>, 256, 160>(p, st);
  if (best == 192) return launch_gemm_tiled<Act, FMT<Act, 192>, 256, 192>(p, st);
  if (best == 224) return launch_gemm_tiled<Act, FMT<Act, 224>, 256, 224>(p, st);
  return launch_gemm_tiled<Act, FMT<Act, 256>, 256, 256>(p, st);
}

}  // namespace qlin
