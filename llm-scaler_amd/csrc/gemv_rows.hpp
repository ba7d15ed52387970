// Decode GEMV for M <= 4 activation rows: one wavefront per weight row.
//
// HBM-bound design.  A wavefront streams whole weight rows with perfectly
// coalesced 128-bit loads (64 lanes x 16 B = 1 KiB contiguous per instruction),
// keeps RW rows in flight, and accumulates with v_dot2_f32_{f16,bf16} (two
// multiply-adds per instruction, fp32 accumulate).  The activations are staged
// once per workgroup in LDS, already laid out in the order the lanes consume
// them, so the inner loop touches global memory for weights only.  The K
// reduction finishes inside the wavefront with cross-lane adds; no LDS
// reduction, no barrier after the staging one.  When a whole activation row fits
// in one batch (K <= SPU spans) and M <= 2, every wavefront keeps its share of
// the activations in registers instead (XREG): no LDS, no barrier at all.
//
// Per-format arithmetic (x = activation, all sums in fp32):
//   fp8   : sum x * e4m3(w), exact conversion to 16 bit, scale applied per row
//           (per-channel / per-tensor) or per lane chunk (128x128 block scale);
//   int4  : nibbles are planted into the mantissa of a 16-bit constant
//           (fp16: 0x6400|nib = 1024+nib, and 0x6400|nib<<4 = 1024+16 nib for
//           odd nibbles, matched by x/16 in LDS; bf16: 0x4300|nib = 128+nib),
//           the constant's contribution  C1 = sum bias_k x_k  and the
//           zero-point's  z * C2, C2 = sum x_k  are precomputed per 32-k chunk
//           at staging time, and the group scale multiplies the corrected
//           partial:  acc += s * (dot - C1 - z C2);
//   Q4_K  : same planting; acc += s * (dot - C1) - min * C2;
//   Q4_0  : the Q4_K path with min = 8 s (32-wide groups, w = (nib - 8) s);
//   Q5_K  : Q4_K plus the fifth bit, OR-ed into the planted constant (bit 4 for
//           even, bit 8 for odd nibbles) from the tile-shuffled qh bytes (dense GEMV) or
//           from element-order qh (routed launches: byte j bit b = element 8j + b for
//           Q5_K, byte j field p = element 4j + p for Q6_K, any K % 32 == 0);
//   Q6_K  : two high bits OR-ed in the same way, the constant and the zero point
//           32 removed exactly in 16 bit before the dot product, one scale per 16;
//   Q8_0  : bytes planted as 0x6400 | (q ^ 0x80) = 1152 + q, 1152 removed exactly
//           in 16 bit, one scale per 32.
// The dequantized weight is therefore never rounded to 16 bit here; against a
// reference that rounds it the difference is below 2^-9 relative per weight.
#pragma once
#include "qlinear_common.hpp"

namespace qlin {

constexpr int kRowsMaxMat = 3;

struct RowsArgs {
  const void* x;
  const void* w[kRowsMaxMat];
  const void* s[kRowsMaxMat];
  const void* z[kRowsMaxMat];
  const void* h[kRowsMaxMat];     // Q5_K / Q6_K high bits (tile-shuffled; element order in routed launches)
  void* out[kRowsMaxMat];
  int N[kRowsMaxMat];
  int groups[kRowsMaxMat];     // row groups (RW rows each) per matrix
  int nmat;
  int M, K;
  int nspan;                   // ceil(K / span_k)
  int total_waves;             // persistent grid size in wavefronts
  int scale_f16;
  // Fused RMS norm of the activation row (NORM kernels, M == 1):
  //   a = x (+ residual);  x' = a * rsqrt(mean_head(a^2) + eps) * weight[k % n_len] (* silu(gate))
  // per head of n_len elements (n_len == K: the whole row).  The workgroup that
  // arrives last writes `residual` (the rounded sum, in place) and `n_out`.
  const void* n_res;
  const void* n_gate;
  const void* n_weight;
  void* n_out;
  unsigned int* n_arrive;      // zeroed counter; the kernel leaves it at zero again
  int n_len;
  float n_eps;
  float n_rscale;              // factor on x + residual before it is stored and normalised
  // Routed launch (ROUTED kernels, M == 1): blockIdx.y is a route r with expert
  // e = r_expert[r] (ids outside [0, r_num_experts) are clamped into range); the matrices of
  // expert e start e * r_*_stride[i] bytes into w / s / z / h, the activation row is row
  // r / r_x_div of x, the output row is r (r_out_stride elements apart) and is multiplied by
  // r_out_mul[r] when that is given.
  // r_alt_w (optional): routes r >= r_alt_from run against this one matrix (scales r_alt_s) instead
  // of an expert's -- a layer's shared expert in the same launch; their activation row is
  // r_alt_x_first + (r - r_alt_from) and they are not multiplied by r_out_mul.
  // ROUTED == 2: a row of x holds 2 K elements, gate then up, and the activation is silu(gate) * up.
  const void* r_alt_w;
  const void* r_alt_s;
  int r_alt_from, r_alt_x_first;
  const int32_t* r_expert;
  const void* r_out_mul;
  int r_num_experts, r_x_div;
  long long r_out_stride;
  long long r_w_stride[kRowsMaxMat], r_s_stride[kRowsMaxMat], r_z_stride[kRowsMaxMat], r_h_stride[kRowsMaxMat];
};

enum : int { RF_FP8 = 0, RF_INT4 = 1, RF_Q4K = 2, RF_Q40 = 3, RF_Q80 = 4, RF_Q5K = 5, RF_Q6K = 6 };
constexpr bool rows_byte_fmt(int fmt) { return fmt == RF_FP8 || fmt == RF_Q80; }   // one byte per weight
enum : int { RS_PERN = 0, RS_PERT = 1, RS_BLOCK = 2 };
// INT4 reuses the scale-mode slot of the template: RS_ZP = the weights come with zero-points
// (their byte is then loaded per group; without them no load is issued at all).
enum : int { RS_ZP = 1 };

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}

template <class Act> struct Dot2;
template <> struct Dot2<ActF16> {
  static __device__ __forceinline__ float run(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
  }
};
template <> struct Dot2<ActBF16> {
  static __device__ __forceinline__ float run(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
  }
};

template <class Act>
__device__ __forceinline__ void fp8x4_to_pairs(uint32_t w, uint32_t& p0, uint32_t& p1) {
  if constexpr (Act::dt == DT_F16) {
    p0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false));
    p1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true));
  } else {
    p0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false));
    p1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true));
  }
}

// LDS image: 16-byte pieces.  Piece index for (span s, piece i, lane l) is
// (s * PPL + i) * 64 + l, PPL = pieces per lane per span (2 for fp8, 4 for the
// nibble formats), so that the 64 lanes of one ds_read_b128 hit consecutive
// addresses.  One piece = 8 consecutive k of one activation row.
//
// The grid is persistent: `a.total_waves` wavefronts walk the flat list of row
// groups (RW rows each, all matrices concatenated) with a fixed stride, and the
// weight loads of the next batch are in flight while the current one is
// consumed (two register buffers).  Weight loads carry the non-temporal hint:
// every byte is used exactly once.
template <class Act, int FMT, int SC, int MR, int NWV, int RW, int SPU, int NBUF, bool MULTI, bool XREG,
          bool NORM = false, int ROUTED = 0>
__global__ __launch_bounds__(NWV * 64) void gemv_rows_kernel(const RowsArgs a_in) {
  static_assert(!NORM || (MR == 1 && !XREG), "the fused norm stages one activation row through LDS");
  static_assert(!ROUTED || (MR == 1 && !NORM), "routed launches take one activation row per route");
  // ROUTED: a private copy of the arguments with this route's bases; otherwise `a` is the
  // kernel argument itself.
  [[maybe_unused]] RowsArgs a_route;
  [[maybe_unused]] float route_mul = 1.0f;
  if constexpr (ROUTED) {
    a_route = a_in;
    const int r = blockIdx.y;
    const bool alt = a_in.r_alt_w != nullptr && r >= a_in.r_alt_from;   // uniform
    int e = a_in.r_expert[alt ? 0 : r];
    e = e < 0 ? 0 : (e >= a_in.r_num_experts ? a_in.r_num_experts - 1 : e);
#pragma unroll
    for (int i = 0; i < kRowsMaxMat; ++i) {
      a_route.w[i] = (const char*)a_in.w[i] + (long long)e * a_in.r_w_stride[i];
      a_route.s[i] = a_in.s[i] ? (const char*)a_in.s[i] + (long long)e * a_in.r_s_stride[i] : nullptr;
      a_route.z[i] = a_in.z[i] ? (const char*)a_in.z[i] + (long long)e * a_in.r_z_stride[i] : nullptr;
      a_route.h[i] = a_in.h[i] ? (const char*)a_in.h[i] + (long long)e * a_in.r_h_stride[i] : nullptr;
      a_route.out[i] = a_in.out[i] ? (char*)a_in.out[i] + (long long)r * a_in.r_out_stride * 2 : nullptr;
    }
    if (alt) { a_route.w[0] = a_in.r_alt_w; a_route.s[0] = a_in.r_alt_s; }
    const long long xrow = alt ? a_in.r_alt_x_first + (r - a_in.r_alt_from) : r / a_in.r_x_div;
    a_route.x = (const char*)a_in.x + xrow * a_in.K * (ROUTED == 2 ? 4 : 2);
    if (a_in.r_out_mul && !alt) route_mul = Act::to_f32(((const typename Act::elem*)a_in.r_out_mul)[r]);
  }
  const RowsArgs& a = ROUTED ? a_route : a_in;
  constexpr bool kFp8 = FMT == RF_FP8;
  constexpr bool kByte = rows_byte_fmt(FMT);
  constexpr bool kNib = !kByte;
  constexpr bool kHigh = FMT == RF_Q5K || FMT == RF_Q6K;
  constexpr bool kSums = kNib && FMT != RF_Q6K;       // formats that use the per-chunk sums
  constexpr int PPL = kByte ? 2 : 4;
  constexpr int SPAN_K = 64 * PPL * 8;               // k covered by one wave load: 1024 / 2048
  constexpr int SPAN_B = kByte ? SPAN_K : SPAN_K / 2; // bytes of one weight row per span
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

  const int K = a.K, M = a.M;
  const int nspan = a.nspan;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // provably uniform
  const int pieces_per_row = nspan * PPL * 64;       // padded to whole spans
  u32x4* xs = reinterpret_cast<u32x4*>(smem);        // [MR][pieces_per_row]
  float* c1 = reinterpret_cast<float*>(smem + (size_t)MR * pieces_per_row * 16);   // [MR][nspan*64]
  float* c2 = c1 + MR * nspan * 64;
  float* nrm = reinterpret_cast<float*>(smem + (size_t)MR * pieces_per_row * 16 + (kByte ? 0 : (size_t)2 * MR * nspan * 64 * 4));   // NORM: [K/8] piece sums, [NWV] wave sums, flag

  const uint32_t wrow = kByte ? (uint32_t)K : ((uint32_t)K >> 1);
  const int nbatch = (nspan + SPU - 1) / SPU;        // batches per row group
  const int stride = a.total_waves;
  const int ngroups = a.groups[0] + a.groups[1] + a.groups[2];

  struct Batch {                                     // one batch = RW rows x SPU spans
    u32x4 w[RW][SPU];
    u32x4 h[RW][SPU][kHigh ? 2 : 1];   // the lane's 32 high-bit bytes (Q5_K / Q6_K)
    // per-lane side data of the chunk, kept as the raw loaded bits: converting here would
    // make the load's first use sit right behind it, and a wait for one load is a wait for
    // every older load in flight (the previous batch's weights)
    uint32_t s[RW][SPU];       // scale: fp16 bits (int4 group, GGUF sub-block; Q6_K: two), fp32 bits (fp8 block)
    uint32_t z[RW][SPU];       // int4 zero-point byte / Q4_K, Q5_K min fp16 bits
    uint32_t os_lo[RW], os_hi[RW];   // fp8 per-channel scale of the row, raw halves (fp32 or fp16)
  };

  // Kernel arguments are selected with uniform compares, never indexed
  // dynamically: a dynamic index would turn into memory loads whose waits
  // serialize behind the weight prefetch.
#define QLIN_PICK(field, mat) \
  (MULTI ? ((mat) == 0 ? a.field[0] : ((mat) == 1 ? a.field[1] : a.field[2])) : a.field[0])
  auto locate = [&](int g, int& mat, int& row0) {
    mat = 0;
    if constexpr (MULTI) {
      if (g >= a.groups[0]) { g -= a.groups[0]; mat = 1; }
      if (mat == 1 && g >= a.groups[1]) { g -= a.groups[1]; mat = 2; }
    }
    row0 = g * RW;
  };

  // Branch-free: an out-of-range group / row / span turns into out-of-range
  // buffer offsets (reads zero) and clamped side-table indices.
  auto load_batch = [&](Batch& b, int g, int sb) {
    const bool live = g < ngroups;
    int mat, row0;
    locate(live ? g : 0, mat, row0);
    const int N = QLIN_PICK(N, mat);
    const __amdgpu_buffer_rsrc_t wr = make_rsrc(QLIN_PICK(w, mat), (uint32_t)N * wrow);
    const __amdgpu_buffer_rsrc_t hr =
        make_rsrc(QLIN_PICK(h, mat), kHigh ? (uint32_t)N * (FMT == RF_Q5K ? ((uint32_t)K >> 3) : ((uint32_t)K >> 2)) : 0u);
    const _Float16* s16 = (const _Float16*)QLIN_PICK(s, mat);
    const float* s32 = (const float*)QLIN_PICK(s, mat);
    const uint8_t* zp = (const uint8_t*)QLIN_PICK(z, mat);
    const uint16_t* qminu = (const uint16_t*)QLIN_PICK(z, mat);
    const uint16_t* s16u = reinterpret_cast<const uint16_t*>(s16);
    const uint8_t* zsrc = zp ? zp : reinterpret_cast<const uint8_t*>(s16);   // always a readable address
    if constexpr (kFp8 && SC == RS_PERN) {
#pragma unroll
      for (int r = 0; r < RW; ++r) {
        const int nc = (row0 + r) < N ? (row0 + r) : N - 1;
        // Two 16-bit loads with uniformly selected offsets cover both scale
        // types without a branch and without converting here: a conversion
        // would wait on the load, and with it on every weight load in flight.
        const uint16_t* sraw = reinterpret_cast<const uint16_t*>(s16);
        const size_t e = a.scale_f16 ? (size_t)nc : (size_t)nc * 2;
        b.os_lo[r] = sraw[e];
        b.os_hi[r] = sraw[e + (a.scale_f16 ? 0 : 1)];
      }
    }
#pragma unroll
    for (int r = 0; r < RW; ++r) {
      const int nc = (row0 + r) < N ? (row0 + r) : N - 1;
#pragma unroll
      for (int sp = 0; sp < SPU; ++sp) {
        const int s = sb * SPU + sp;
        const int chunk = s * 64 + lane;            // 32-k chunk index (nibble formats)
        if constexpr (FMT == RF_INT4) {
          const int Kg = K >> 7;
          int gi = chunk >> 2;
          gi = gi < Kg ? gi : Kg - 1;
          b.s[r][sp] = s16u[(size_t)nc * Kg + gi];
          if constexpr (SC == RS_ZP) b.z[r][sp] = zsrc[(size_t)nc * Kg + gi];
        } else if constexpr (FMT == RF_Q4K || FMT == RF_Q5K) {
          const int Kc = K >> 5;
          const int ci = chunk < Kc ? chunk : Kc - 1;
          b.s[r][sp] = s16u[(size_t)nc * Kc + ci];
          b.z[r][sp] = qminu[(size_t)nc * Kc + ci];
        } else if constexpr (FMT == RF_Q40) {
          const int Kc = K >> 5;
          const int ci = chunk < Kc ? chunk : Kc - 1;
          b.s[r][sp] = s16u[(size_t)nc * Kc + ci];
        } else if constexpr (FMT == RF_Q6K) {
          // the lane's 32 k span two 16-wide groups: both fp16 scales in one 32-bit load
          const int Kc = K >> 5;
          const int ci = chunk < Kc ? chunk : Kc - 1;
          b.s[r][sp] = reinterpret_cast<const uint32_t*>(s16)[(size_t)nc * Kc + ci];
        } else if constexpr (FMT == RF_Q80) {
          const int Kc = K >> 5;
          const int c8 = (s * SPAN_K + lane * 16) >> 5;
          b.s[r][sp] = s16u[(size_t)nc * Kc + (c8 < Kc ? c8 : Kc - 1)];
        } else if constexpr (SC == RS_BLOCK) {
          const int Kb = (K + 127) >> 7;
          const int kblk = (s * SPAN_K + lane * 16) >> 7;
          b.s[r][sp] = reinterpret_cast<const uint32_t*>(s32)[(size_t)(nc >> 7) * Kb + (kblk < Kb ? kblk : Kb - 1)];
        }
      }
    }
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
      for (int sp = 0; sp < SPU; ++sp) {
        const uint32_t kb = (uint32_t)(sb * SPU + sp) * SPAN_B + lane * 16u;   // byte in row
        // in-range offsets stay below 2^31; setting the top bit pushes a dead
        // lane past the buffer's bound (arithmetic, so no branch is formed)
        const uint32_t dead = (uint32_t)(!(live && (row0 + r < N) && (kb < wrow))) << 31;
        b.w[r][sp] = __builtin_amdgcn_raw_buffer_load_b128(
            wr, ((uint32_t)(row0 + r) * wrow + kb) | dead, 0, 2 /* nt */);
        if constexpr (kHigh && ROUTED) {
          // element-order high bits: the lane's 32 consecutive k are 4 (Q5_K) or 8 (Q6_K)
          // consecutive bytes of the row
          const uint32_t hrow = FMT == RF_Q5K ? ((uint32_t)K >> 3) : ((uint32_t)K >> 2);
          const uint32_t hb = FMT == RF_Q5K ? kb >> 2 : kb >> 1;
          const uint32_t ho = ((uint32_t)(row0 + r) * hrow + hb) | dead;
          b.h[r][sp][1] = u32x4{0u, 0u, 0u, 0u};
          if constexpr (FMT == RF_Q5K) {
            b.h[r][sp][0] = u32x4{__builtin_amdgcn_raw_buffer_load_b32(hr, ho, 0, 2), 0u, 0u, 0u};
          } else {
            const u32x2 two = __builtin_amdgcn_raw_buffer_load_b64(hr, ho, 0, 2);
            b.h[r][sp][0] = u32x4{two[0], two[1], 0u, 0u};
          }
        } else if constexpr (kHigh) {
          // per 512-k tile the high bits of element b*64 + t (Q5_K, 1 bit) or
          // p*128 + t (Q6_K, 2 bits) sit in byte t: the lane's 32 consecutive k
          // are 32 consecutive bytes, one bit field
          constexpr uint32_t tile_b = FMT == RF_Q5K ? 64u : 128u;
          const uint32_t hrow = FMT == RF_Q5K ? ((uint32_t)K >> 3) : ((uint32_t)K >> 2);
          const uint32_t tile = (uint32_t)(sb * SPU + sp) * 4u + ((uint32_t)lane >> 4);
          const uint32_t within = FMT == RF_Q5K ? ((uint32_t)lane & 1u) * 32u : ((uint32_t)lane & 3u) * 32u;
          const uint32_t ho = ((uint32_t)(row0 + r) * hrow + tile * tile_b + within) | dead;
          b.h[r][sp][0] = __builtin_amdgcn_raw_buffer_load_b128(hr, ho, 0, 2);
          b.h[r][sp][1] = __builtin_amdgcn_raw_buffer_load_b128(hr, ho + 16u, 0, 2);
        }
      }
  };

  // ---- stage activations ----
  // The vector-memory counter retires in order, so the activation loads are
  // issued BEFORE the weight prefetch: waiting for them then leaves the weight
  // loads in flight.  XPRE loads per thread go out up front; anything beyond
  // that (large M x K) is fetched after the prefetch and waits for it.
  constexpr bool XACT = ROUTED == 2;                  // the activation is silu(gate) * up of a 2 K wide row
  static_assert(!XACT || !XREG, "the fused activation goes through the LDS staging");
  const __amdgpu_buffer_rsrc_t xr = make_rsrc(a.x, (uint32_t)M * (uint32_t)K * (XACT ? 4u : 2u));
  const int total = MR * pieces_per_row;
  constexpr int XPRE = 4;
  // eight gate and eight up values -> eight activations, fp32 inside, one rounding (what
  // silu_mul_kernel computes)
  auto act_mul = [&](u32x4 gv, u32x4 uv) -> u32x4 {
    const typename Act::v8 g8 = as_v8<typename Act::v8>(gv), u8 = as_v8<typename Act::v8>(uv);
    typename Act::v8 o8;
#pragma unroll
    for (int e2 = 0; e2 < 8; ++e2) {
      const float gf = Act::to_f32(g8[e2]), uf = Act::to_f32(u8[e2]);
      o8[e2] = Act::from_f32(gf / (1.0f + expf(-gf)) * uf);
    }
    return __builtin_bit_cast(u32x4, o8);
  };
  auto x_offset = [&](int p) -> uint32_t {
    const int m = (p >= pieces_per_row) + (p >= 2 * pieces_per_row) + (p >= 3 * pieces_per_row);
    const int q = p - m * pieces_per_row;          // (s*PPL + i)*64 + l
    const int l = q & 63;
    const int si = q >> 6;
    const int s = si / PPL, i = si - s * PPL;
    const int k = s * SPAN_K + (l * PPL + i) * 8;
    const uint32_t dead = (uint32_t)(!(p < total && m < M && k < K)) << 31;
    return (((uint32_t)m * K + k) * 2u) | dead;
  };
  auto x_arrange = [&](u32x4 v) -> u32x4 {
    if constexpr (kNib) {
      // natural pairs (x0 x1)(x2 x3)(x4 x5)(x6 x7) -> (x0 x4)(x1 x5)(x2 x6)(x3 x7)
      const uint32_t d0 = v[0], d1 = v[1], d2 = v[2], d3 = v[3];
      uint32_t e0 = __builtin_amdgcn_perm(d2, d0, 0x05040100u);   // lo(d0), lo(d2)
      uint32_t e1 = __builtin_amdgcn_perm(d2, d0, 0x07060302u);   // hi(d0), hi(d2)
      uint32_t e2 = __builtin_amdgcn_perm(d3, d1, 0x05040100u);
      uint32_t e3 = __builtin_amdgcn_perm(d3, d1, 0x07060302u);
      if constexpr (Act::dt == DT_F16) {
        // odd nibbles are planted 4 bits up (1024 + 16 nib): feed them x / 16
        const f16x2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
        e1 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, e1) * sixteenth);
        e3 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, e3) * sixteenth);
      }
      v = u32x4{e0, e1, e2, e3};
    }
    return v;
  };
  auto x_store = [&](int p, u32x4 v) {
    if (p < total) xs[p] = x_arrange(v);
  };
  // what the planted constants contribute (c1) and sum x (c2) over one 32-k
  // chunk = four arranged pieces, summed in a fixed order
  auto chunk_sums = [&](const u32x4 (&pc)[4], float& k1, float& k2) {
    float lo = 0.f, hi = 0.f;
    auto pair_sum = [](uint32_t bits) -> float {
      if constexpr (Act::dt == DT_F16) {
        const f16x2 h = __builtin_bit_cast(f16x2, bits);
        return (float)h[0] + (float)h[1];
      } else {
        const bf16x2 h = __builtin_bit_cast(bf16x2, bits);
        return (float)h[0] + (float)h[1];
      }
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo += pair_sum(pc[i][0]);
      hi += pair_sum(pc[i][1]);
      lo += pair_sum(pc[i][2]);
      hi += pair_sum(pc[i][3]);
    }
    if constexpr (Act::dt == DT_F16) {
      k1 = 1024.0f * (lo + hi);                      // hi already holds x / 16
      k2 = lo + 16.0f * hi;
    } else {
      k1 = 128.0f * (lo + hi);
      k2 = lo + hi;
    }
  };
  // XREG: the lane's own pieces of every span, loaded straight into registers
  constexpr int XM = XREG ? MR : 1, XS = XREG ? SPU : 1;
  u32x4 xreg[XM][XS][PPL];
  float c1r[XM][XS], c2r[XM][XS];
  if constexpr (XREG) {
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
      for (int sp = 0; sp < SPU; ++sp)
#pragma unroll
        for (int i = 0; i < PPL; ++i) {
          const int k = sp * SPAN_K + (lane * PPL + i) * 8;
          const uint32_t dead = (uint32_t)(!(m < M && k < K)) << 31;
          xreg[m][sp][i] = buf_load16(xr, (((uint32_t)m * K + k) * 2u) | dead);
        }
  }
  u32x4 xpre[XPRE];
  [[maybe_unused]] u32x4 upre[XACT ? XPRE : 1];
  if constexpr (!XREG) {
#pragma unroll
    for (int t = 0; t < XPRE; ++t) xpre[t] = buf_load16(xr, x_offset(threadIdx.x + t * NWV * 64));
    if constexpr (XACT) {
#pragma unroll
      for (int t = 0; t < XPRE; ++t) upre[t] = buf_load16(xr, x_offset(threadIdx.x + t * NWV * 64) + (uint32_t)K * 2u);
    }
  }
  // NORM: residual, gate and norm weight of the same pieces (a null operand reads zeros)
  u32x4 nres[NORM ? XPRE : 1], ngate[NORM ? XPRE : 1], nwgt[NORM ? XPRE : 1];
  if constexpr (NORM) {
    const __amdgpu_buffer_rsrc_t rr = make_rsrc(a.n_res, a.n_res ? (uint32_t)K * 2u : 0u);
    const __amdgpu_buffer_rsrc_t gr = make_rsrc(a.n_gate, a.n_gate ? (uint32_t)K * 2u : 0u);
    const __amdgpu_buffer_rsrc_t wr_n = make_rsrc(a.n_weight, (uint32_t)a.n_len * 2u);
#pragma unroll
    for (int t = 0; t < XPRE; ++t) {
      nres[t] = ngate[t] = nwgt[t] = u32x4{0u, 0u, 0u, 0u};
      if (t * NWV * 64 < total) {                     // uniform: this group of pieces exists
        const uint32_t off = x_offset(threadIdx.x + t * NWV * 64);
        const uint32_t k0 = (off & 0x7FFFFFFFu) >> 1;
        const uint32_t kw = a.n_len == K ? k0 : k0 % (uint32_t)a.n_len;
        nres[t] = buf_load16(rr, off);
        ngate[t] = buf_load16(gr, off);
        nwgt[t] = buf_load16(wr_n, (kw * 2u) | (off & 0x80000000u));
      }
    }
  }
  unsigned int n_prev = 0;                            // NORM: workgroups that arrived before this one

  auto advance = [&](int& g, int& sb) {
    if (++sb == nbatch) { sb = 0; g += stride; }
  };
  // ring of NBUF register buffers: NBUF - 1 batches are in flight while one is consumed
  Batch buf[NBUF];
  int gq[NBUF], sq[NBUF];
  int g_next = blockIdx.x * NWV + wave, sb_next = 0;
#pragma unroll
  for (int i = 0; i < NBUF - 1; ++i) {
    gq[i] = g_next; sq[i] = sb_next;
    load_batch(buf[i], g_next, sb_next);
    advance(g_next, sb_next);
  }
  // nothing below may be scheduled above the prefetch: the weight loads go out first
  __builtin_amdgcn_sched_barrier(0);
  // one per-tensor scale per fused matrix (scalars, so they stay in registers)
  float pert0 = 1.0f, pert1 = 1.0f, pert2 = 1.0f;
  if constexpr (kFp8 && SC == RS_PERT) {
    pert0 = ((const float*)a.s[0])[0];
    if constexpr (MULTI) {
      if (a.nmat > 1) pert1 = ((const float*)a.s[1])[0];
      if (a.nmat > 2) pert2 = ((const float*)a.s[2])[0];
    }
  }

  u32x4 res_new[NORM ? XPRE : 1], normed[NORM ? XPRE : 1];   // NORM: what the last workgroup writes back
  if constexpr (XREG) {
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
      for (int sp = 0; sp < SPU; ++sp) {
#pragma unroll
        for (int i = 0; i < PPL; ++i) xreg[m][sp][i] = x_arrange(xreg[m][sp][i]);
        if constexpr (kSums) chunk_sums(xreg[m][sp], c1r[m][sp], c2r[m][sp]);
      }
  } else if constexpr (NORM) {
    using E = typename Act::elem;
    const int V = a.n_len;
    float av[XPRE][8];
    float ssp[XPRE];
#pragma unroll
    for (int t = 0; t < XPRE; ++t) {
      ssp[t] = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) av[t][e] = 0.f;
      if (t * NWV * 64 >= total) continue;            // uniform
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const E h = __builtin_bit_cast(E, (uint16_t)(xpre[t][e >> 1] >> (16 * (e & 1))));
        const E r = __builtin_bit_cast(E, (uint16_t)(nres[t][e >> 1] >> (16 * (e & 1))));
        av[t][e] = (Act::to_f32(h) + Act::to_f32(r)) * a.n_rscale;
        ssp[t] += av[t][e] * av[t][e];
      }
    }
    const bool whole = V == K;
    if (whole) {
      const float ws = wave_sum((ssp[0] + ssp[1]) + (ssp[2] + ssp[3]));
      if (lane == 0) nrm[(K >> 3) + wave] = ws;
    } else {
#pragma unroll
      for (int t = 0; t < XPRE; ++t) {
        const int pidx = threadIdx.x + t * NWV * 64;
        const uint32_t off = x_offset(pidx);
        if (!(off >> 31)) nrm[(off >> 4)] = ssp[t];   // natural piece index k0 / 8
      }
    }
    __syncthreads();                                  // every thread has consumed its loads
    // Arrival count: whoever comes last knows that all workgroups hold their copy of the
    // row in registers, and may overwrite the residual.  The final count is looked at only
    // at the end of the kernel.
    // Relaxed is enough: the barrier above already orders every thread's (completed) loads
    // before the increment, the last workgroup reads nothing the others wrote, and its
    // stores depend on the value it gets back.  A release / acquire pair would add cache
    // write-backs and a wait for every load in flight.
    // Two levels keep the chain of same-address read-modify-writes short (each takes tens of
    // nanoseconds at the memory side): 16 counters by workgroup index, then one on top.
    if (threadIdx.x == 0) {
      const unsigned int sub = blockIdx.x & 15u;
      const unsigned int members = (gridDim.x - sub + 15u) >> 4;
      unsigned int* c1p = a.n_arrive + sub * 16u;       // 64 bytes apart
      const unsigned int p1 = __hip_atomic_fetch_add(c1p, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      n_prev = 0xFFFFFFFFu;
      if (p1 == members - 1) {                          // last of its group: report to the top counter
        __hip_atomic_store(c1p, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        n_prev = __hip_atomic_fetch_add(a.n_arrive + 256, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    float wtot = 0.f;
    if (whole) {
#pragma unroll
      for (int w = 0; w < NWV; ++w) wtot += nrm[(K >> 3) + w];
    }
#pragma unroll
    for (int t = 0; t < XPRE; ++t) {
      if (t * NWV * 64 >= total) continue;
      const uint32_t off = x_offset(threadIdx.x + t * NWV * 64);
      float tot = wtot;
      if (!whole) {
        tot = 0.f;
        const int k0 = (int)((off & 0x7FFFFFFFu) >> 1);
        const int hp = (k0 / V) * (V >> 3);
        if (!(off >> 31))
          for (int jj = 0; jj < (V >> 3); ++jj) tot += nrm[hp + jj];
      }
      const float inv = rsqrtf(tot / (float)V + a.n_eps);
#pragma unroll
      for (int e2 = 0; e2 < 4; ++e2) {
        uint32_t rw = 0, nw = 0;
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          const int e = e2 * 2 + h2;
          const E wv = __builtin_bit_cast(E, (uint16_t)(nwgt[t][e2] >> (16 * h2)));
          float v = av[t][e] * inv * Act::to_f32(wv);
          if (a.n_gate) {
            const float z = Act::to_f32(__builtin_bit_cast(E, (uint16_t)(ngate[t][e2] >> (16 * h2))));
            v *= z / (1.0f + __expf(-z));
          }
          rw |= (uint32_t)__builtin_bit_cast(uint16_t, Act::from_f32(av[t][e])) << (16 * h2);
          nw |= (uint32_t)__builtin_bit_cast(uint16_t, Act::from_f32(v)) << (16 * h2);
        }
        res_new[t][e2] = rw;
        normed[t][e2] = nw;
      }
      x_store(threadIdx.x + t * NWV * 64, normed[t]);
    }
    if constexpr (kSums) {
      __syncthreads();
      const int chunks = nspan * 64;
      for (int c = threadIdx.x; c < chunks; c += NWV * 64) {
        const int s = c >> 6, l = c & 63;
        u32x4 pc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) pc[i] = xs[(s * 4 + i) * 64 + l];
        chunk_sums(pc, c1[c], c2[c]);
      }
    }
    __syncthreads();
  } else {
#pragma unroll
    for (int t = 0; t < XPRE; ++t) x_store(threadIdx.x + t * NWV * 64, XACT ? act_mul(xpre[t], upre[t]) : xpre[t]);
    for (int p = threadIdx.x + XPRE * NWV * 64; p < total; p += NWV * 64) {
      const u32x4 xv = buf_load16(xr, x_offset(p));
      if constexpr (XACT) x_store(p, act_mul(xv, buf_load16(xr, x_offset(p) + (uint32_t)K * 2u)));
      else x_store(p, xv);
    }
    if constexpr (kSums) {
      // per 32-k chunk sums, from the staged image
      __syncthreads();
      const int chunks = MR * nspan * 64;
      for (int c = threadIdx.x; c < chunks; c += NWV * 64) {
        const int m = c / (nspan * 64);
        const int sl = c - m * (nspan * 64);
        const int s = sl >> 6, l = sl & 63;
        u32x4 pc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) pc[i] = xs[m * pieces_per_row + (s * 4 + i) * 64 + l];
        chunk_sums(pc, c1[c], c2[c]);
      }
    }
    __syncthreads();
  }

  float acc[RW][MR];
#pragma unroll
  for (int r = 0; r < RW; ++r)
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[r][m] = 0.f;

  constexpr bool has_zp = FMT == RF_INT4 && SC == RS_ZP;     // zero-points come for all matrices or for none
  auto compute = [&](const Batch& b, int sb) {
#pragma unroll
    for (int sp = 0; sp < SPU; ++sp) {
      const int s = sb * SPU + sp;
      // wave-uniform.  With the activations in registers a span past the row's end holds
      // zero weights and zero activations and is simply computed: the loop body then has
      // no branches, which keeps the wait counts of the loads in flight exact.
      if (XREG || s < nspan) {
        u32x4 xp[MR][PPL];
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
          for (int i = 0; i < PPL; ++i) {
            if constexpr (XREG) xp[m][i] = xreg[m][sp][i];
            else xp[m][i] = xs[m * pieces_per_row + (s * PPL + i) * 64 + lane];
          }
#pragma unroll
        for (int r = 0; r < RW; ++r) {
          const u32x4 w = b.w[r][sp];
          float part[MR];
#pragma unroll
          for (int m = 0; m < MR; ++m) part[m] = 0.f;
          if constexpr (kFp8) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              uint32_t p0, p1;
              fp8x4_to_pairs<Act>(w[d], p0, p1);
#pragma unroll
              for (int m = 0; m < MR; ++m) {
                part[m] = Dot2<Act>::run(p0, xp[m][d >> 1][(d & 1) * 2], part[m]);
                part[m] = Dot2<Act>::run(p1, xp[m][d >> 1][(d & 1) * 2 + 1], part[m]);
              }
            }
            if constexpr (SC == RS_BLOCK) {
#pragma unroll
              for (int m = 0; m < MR; ++m) acc[r][m] += part[m] * __builtin_bit_cast(float, b.s[r][sp]);
            } else {
#pragma unroll
              for (int m = 0; m < MR; ++m) acc[r][m] += part[m];
            }
          } else if constexpr (FMT == RF_Q80) {
            // int8 -> fp16 exactly: 0x6400 | (q ^ 0x80) = 1152 + q, minus 1152
            const f16x2 k1152 = {(_Float16)1152.0f, (_Float16)1152.0f};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              const uint32_t u = w[d] ^ 0x80808080u;
              const uint32_t p0 = __builtin_bit_cast(
                  uint32_t, __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - k1152);
              const uint32_t p1 = __builtin_bit_cast(
                  uint32_t, __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - k1152);
#pragma unroll
              for (int m = 0; m < MR; ++m) {
                part[m] = Dot2<Act>::run(p0, xp[m][d >> 1][(d & 1) * 2], part[m]);
                part[m] = Dot2<Act>::run(p1, xp[m][d >> 1][(d & 1) * 2 + 1], part[m]);
              }
            }
#pragma unroll
            for (int m = 0; m < MR; ++m) acc[r][m] += part[m] * f16_bits_to_f32(b.s[r][sp]);
          } else {
            float part_hi[MR];                       // Q6_K: second 16-wide group of the lane
#pragma unroll
            for (int m = 0; m < MR; ++m) part_hi[m] = 0.f;
            // bit field of the lane inside its high-bit bytes (the same for every span:
            // a span covers whole 512-k tiles)
            const uint32_t hshift = FMT == RF_Q5K ? (((uint32_t)lane & 15u) >> 1) : ((((uint32_t)lane & 15u) >> 2) * 2u);
            constexpr uint32_t hmask = FMT == RF_Q5K ? 0x01010101u : 0x03030303u;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              uint32_t t0, t1, t2, t3;
              if constexpr (Act::dt == DT_F16) {
                const uint32_t w8 = w[d] >> 8;
                t0 = (w[d] & 0x000F000Fu) | 0x64006400u;     // 1024 + nib0 , nib4
                t1 = (w[d] & 0x00F000F0u) | 0x64006400u;     // 1024 + 16 nib1 , nib5
                t2 = (w8 & 0x000F000Fu) | 0x64006400u;       // nib2 , nib6
                t3 = (w8 & 0x00F000F0u) | 0x64006400u;       // nib3 , nib7
              } else {
                t0 = (w[d] & 0x000F000Fu) | 0x43004300u;     // 128 + nib0 , nib4
                t1 = ((w[d] >> 4) & 0x000F000Fu) | 0x43004300u;
                t2 = ((w[d] >> 8) & 0x000F000Fu) | 0x43004300u;
                t3 = ((w[d] >> 12) & 0x000F000Fu) | 0x43004300u;
              }
              if constexpr (kHigh && ROUTED && Act::dt == DT_F16) {
                if constexpr (FMT == RF_Q5K) {
                  // byte d of the lane's word: bit e = fifth bit of element 8d + e.  A second copy
                  // 12 bits up puts bits 4..7 at 16..19, beside the upper halves' nibbles.
                  const uint32_t hb = (b.h[r][sp][0][0] >> (8 * d)) & 0xFFu;
                  const uint32_t spv = hb | (hb << 12);
                  t0 |= (spv << 4) & 0x00100010u;          // elements 0, 4 -> bits 4, 20
                  t1 |= (spv << 7) & 0x01000100u;          // elements 1, 5 -> bits 8, 24
                  t2 |= (spv << 2) & 0x00100010u;          // elements 2, 6
                  t3 |= (spv << 5) & 0x01000100u;          // elements 3, 7
                } else {
                  // 16 bits per 8 elements, field e at bits 2e: low byte -> byte 0, high byte -> byte 2
                  const uint32_t spv = __builtin_amdgcn_perm(0u, b.h[r][sp][0][d >> 1], (d & 1) ? 0x0C030C02u : 0x0C010C00u);
                  t0 |= (spv << 4) & 0x00300030u;          // fields 0, 4 -> bits 4..5, 20..21
                  t1 |= (spv << 6) & 0x03000300u;          // fields 1, 5 -> bits 8..9, 24..25
                  t2 |= spv & 0x00300030u;                 // fields 2, 6
                  t3 |= (spv << 2) & 0x03000300u;          // fields 3, 7
                }
              } else if constexpr (kHigh && Act::dt == DT_F16) {
                // elements 8d .. 8d+3 have their high bits in bytes of hA, 8d+4 .. 8d+7 in hB;
                // pair (i, i+4) takes byte i of each, moved to bit 4 (even) / bit 8 (odd nibbles)
                const uint32_t hA = (b.h[r][sp][d >> 1][(d & 1) * 2] >> hshift) & hmask;
                const uint32_t hB = (b.h[r][sp][d >> 1][(d & 1) * 2 + 1] >> hshift) & hmask;
                t0 |= __builtin_amdgcn_perm(hB, hA, 0x0C040C00u) << 4;
                t1 |= __builtin_amdgcn_perm(hB, hA, 0x0C050C01u) << 8;
                t2 |= __builtin_amdgcn_perm(hB, hA, 0x0C060C02u) << 4;
                t3 |= __builtin_amdgcn_perm(hB, hA, 0x0C070C03u) << 8;
              }
              if constexpr (FMT == RF_Q6K && Act::dt == DT_F16) {
                // exact in fp16: (1024 + v6) - 1056 = v6 - 32, (1024 + 16 v6) - 1536 = 16 (v6 - 32)
                const f16x2 ke = {(_Float16)1056.0f, (_Float16)1056.0f};
                const f16x2 ko = {(_Float16)1536.0f, (_Float16)1536.0f};
                t0 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, t0) - ke);
                t1 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, t1) - ko);
                t2 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, t2) - ke);
                t3 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, t3) - ko);
              }
#pragma unroll
              for (int m = 0; m < MR; ++m) {
                float& pt = (FMT == RF_Q6K && d >= 2) ? part_hi[m] : part[m];
                pt = Dot2<Act>::run(t0, xp[m][d][0], pt);
                pt = Dot2<Act>::run(t1, xp[m][d][1], pt);
                pt = Dot2<Act>::run(t2, xp[m][d][2], pt);
                pt = Dot2<Act>::run(t3, xp[m][d][3], pt);
              }
            }
            if constexpr (FMT == RF_Q6K) {
              const uint32_t two = b.s[r][sp];
              const float s_lo = f16_bits_to_f32(two & 0xFFFFu);
              const float s_hi = f16_bits_to_f32(two >> 16);
#pragma unroll
              for (int m = 0; m < MR; ++m) acc[r][m] += s_lo * part[m] + s_hi * part_hi[m];
            }
            const float sc = f16_bits_to_f32(b.s[r][sp]);
            const float zz = FMT == RF_Q40    ? 8.0f * sc
                             : FMT == RF_INT4 ? (has_zp ? (float)b.z[r][sp] : 8.0f)
                                              : f16_bits_to_f32(b.z[r][sp]);
#pragma unroll
            for (int m = 0; m < (FMT == RF_Q6K ? 0 : MR); ++m) {
              float k1, k2;
              if constexpr (XREG) {
                k1 = c1r[m][sp]; k2 = c2r[m][sp];
              } else {
                k1 = c1[(m * nspan + s) * 64 + lane];
                k2 = c2[(m * nspan + s) * 64 + lane];
              }
              if constexpr (FMT == RF_INT4)
                acc[r][m] += sc * (part[m] - k1 - zz * k2);
              else
                acc[r][m] += sc * (part[m] - k1) - zz * k2;
            }
          }
        }
      }
    }
  };

  // finish the K reduction inside the wavefront, lane 0 stores, accumulators reset.
  // The stored values keep their registers until the next batch's loads have been issued
  // (see the loop): stores and loads retire through one in-order counter, so reusing a
  // store's data register any earlier would make the compiler wait for every load in flight.
  using Elem = typename Act::elem;
  // The RW rows of a batch are adjacent outputs: lane r keeps row r's value and one store per
  // activation row writes them all (a store costs the memory pipeline an instruction slot, like
  // a load, whatever its size).
  uint32_t stored[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) stored[m] = 0u;
  auto finish = [&](const Batch& b, int g) {
    int mat, row0;
    locate(g, mat, row0);
    const int N = QLIN_PICK(N, mat);
    Elem* out = (Elem*)QLIN_PICK(out, mat);
#pragma unroll
    for (int r = 0; r < RW; ++r) {
      float os = 1.0f;
      if constexpr (kFp8 && SC == RS_PERN)
        os = a.scale_f16 ? (float)__builtin_bit_cast(_Float16, (uint16_t)b.os_lo[r])
                         : __builtin_bit_cast(float, b.os_lo[r] | (b.os_hi[r] << 16));
      if constexpr (kFp8 && SC == RS_PERT) os = mat == 0 ? pert0 : (mat == 1 ? pert1 : pert2);
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        const float v = wave_sum(acc[r][m]);
        acc[r][m] = 0.f;
        const uint32_t bits = (uint32_t)__builtin_bit_cast(uint16_t, Act::from_f32(ROUTED ? v * os * route_mul : v * os));
        stored[m] = lane == r ? bits : stored[m];
        if (r == RW - 1) {
          asm volatile("" : "+v"(stored[m]));         // the store below reads exactly this register
          if (lane < RW && row0 + lane < N && m < M)
            out[(size_t)m * N + row0 + lane] = __builtin_bit_cast(Elem, (uint16_t)stored[m]);
        }
      }
    }
  };

  // ---- walk the wave's batches; buffer indices are static after unrolling ----
  // Both halves of a ring turn always issue their loads (a batch past the end loads
  // nothing) and the only way out is at the bottom: an exit in the middle would reach the
  // loop header with the other slot's loads still in flight, and the compiler would then
  // have to drain every load there on every turn.
  while (gq[0] < ngroups) {
#pragma unroll
    for (int i = 0; i < NBUF; ++i) {
      const int j = (i + NBUF - 1) % NBUF;
      gq[j] = g_next; sq[j] = sb_next;
      load_batch(buf[j], g_next, sb_next);
      // the next batch's loads are issued before the current batch is consumed: without
      // the fence the compiler rotates the loop (compute first), which halves the prefetch
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < MR; ++m) asm volatile("" ::"v"(stored[m]));
      advance(g_next, sb_next);
      if (gq[i] < ngroups) {                          // uniform; rejoins before the next loads
        compute(buf[i], sq[i]);
        if (sq[i] == nbatch - 1) finish(buf[i], gq[i]);
      }
    }
  }
  if constexpr (NORM) {
    float* flag = nrm + (K >> 3) + NWV;
    if (threadIdx.x == 0) {
      const unsigned int groups = gridDim.x < 16u ? gridDim.x : 16u;
      const bool last = n_prev == groups - 1;
      if (last) __hip_atomic_store(a.n_arrive + 256, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *flag = last ? 1.0f : 0.0f;
    }
    __syncthreads();
    if (*flag != 0.0f) {
#pragma unroll
      for (int t = 0; t < XPRE; ++t) {
        if (t * NWV * 64 >= total) continue;
        const uint32_t off = x_offset(threadIdx.x + t * NWV * 64);
        if (!(off >> 31)) {
          if (a.n_res) *reinterpret_cast<u32x4*>((char*)const_cast<void*>(a.n_res) + off) = res_new[t];
          if (a.n_out) *reinterpret_cast<u32x4*>((char*)a.n_out + off) = normed[t];
        }
      }
    }
  }
#undef QLIN_PICK
}

// LDS bytes the kernel needs for a given shape.
static inline size_t rows_lds_bytes(int fmt, int MR, int K) {
  const int ppl = rows_byte_fmt(fmt) ? 2 : 4;
  const int span_k = 64 * ppl * 8;
  const int nspan = (K + span_k - 1) / span_k;
  size_t b = (size_t)MR * nspan * ppl * 64 * 16;
  if (!rows_byte_fmt(fmt)) b += (size_t)2 * MR * nspan * 64 * 4;
  return b;
}

// extra LDS of the fused norm: one partial sum per 8-k piece, one per wavefront, one flag
static inline size_t rows_norm_lds_bytes(int K) { return ((size_t)(K >> 3) + 16) * 4; }

// rows the fused norm can stage: XPRE (4) pieces of 8 k per thread, 512 threads
constexpr int kRowsNormMaxK = 4 * 512 * 8;

static inline int device_cu_count() {
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

template <class Act, int FMT, int SC, int MR, int RW, int SPU, bool XREG, bool NORM = false, int ROUTED = 0>
static void launch_rows_rw(RowsArgs a, hipStream_t st, int routes = 1) {
  constexpr int NWV = 8;
  constexpr int NBUF = 2;
  int groups = 0;
  for (int i = 0; i < kRowsMaxMat; ++i) {
    a.groups[i] = i < a.nmat ? (a.N[i] + RW - 1) / RW : 0;
    groups += a.groups[i];
  }
  if (!groups) return;
  // persistent grid: the workgroup count (per CU) that wastes the fewest wave slots
  const int cus = device_cu_count();
  int best_wgs = 0;
  double best_eff = -1.0;
  for (int per_cu = 1; per_cu <= 4; ++per_cu) {
    const long waves = (long)cus * per_cu * NWV;
    const long iters = (groups + waves - 1) / waves;
    const double eff = (double)groups / (double)(iters * waves);
    if (eff > best_eff + 1e-9) { best_eff = eff; best_wgs = cus * per_cu; }
  }
  const int needed = (groups + NWV - 1) / NWV;
  int wgs = needed < best_wgs ? needed : best_wgs;
  if constexpr (ROUTED) {
    // the routes share the device: about two workgroups per CU over all of them, so that a
    // wavefront walks several rows and the next row loads while the current one is consumed
    const int cap = (2 * cus + routes - 1) / routes;
    if (wgs > cap) wgs = cap;
  }
  a.total_waves = wgs * NWV;
  const size_t lds = XREG ? 0 : rows_lds_bytes(FMT, MR, a.K) + (NORM ? rows_norm_lds_bytes(a.K) : 0);
  if (a.nmat == 1 || ROUTED)                          // routed launches take one matrix
    hipLaunchKernelGGL((gemv_rows_kernel<Act, FMT, SC, MR, NWV, RW, SPU, NBUF, false, XREG, NORM, ROUTED>),
                       dim3(wgs, ROUTED ? routes : 1), dim3(NWV * 64), lds, st, a);
  else if constexpr (!ROUTED)
    hipLaunchKernelGGL((gemv_rows_kernel<Act, FMT, SC, MR, NWV, RW, SPU, NBUF, true, XREG, NORM, false>), dim3(wgs),
                       dim3(NWV * 64), lds, st, a);
}

// Routed launch (one activation row per route, expert-indexed matrices): one row per batch,
// activations staged through LDS; the routes are the grid's second dimension.
template <class Act, int FMT, int SC = 0, int ROUTED = 1>
static void launch_rows_routed(RowsArgs a, int routes, hipStream_t st) {
  constexpr bool kByte = rows_byte_fmt(FMT);
  constexpr int ppl = kByte ? 2 : 4;
  constexpr int span_k = 64 * ppl * 8;
  constexpr int SPU = kByte ? 4 : 2;
  a.nspan = (a.K + span_k - 1) / span_k;
  if (a.nspan == 1) return launch_rows_rw<Act, FMT, SC, 1, 1, 1, false, false, ROUTED>(a, st, routes);
  if constexpr (kByte) {
    // a batch of exactly the row's spans: an empty span slot would still cost a dead load and a pass
    // of arithmetic on zeros
    if (a.nspan == 2) return launch_rows_rw<Act, FMT, SC, 1, 1, 2, false, false, ROUTED>(a, st, routes);
    if (a.nspan == 3) return launch_rows_rw<Act, FMT, SC, 1, 1, 3, false, false, ROUTED>(a, st, routes);
  }
  launch_rows_rw<Act, FMT, SC, 1, 1, SPU, false, false, ROUTED>(a, st, routes);
}

// Batch shape by row length.  Rows of up to one batch (fp8: 4 spans = 4096 k,
// nibble formats: 2 or 3 spans = 4096 / 6144 k) with M <= 2 keep the
// activations in registers; longer rows stage them in LDS.
template <class Act, int FMT, int SC, int MR>
static void launch_rows(RowsArgs a, hipStream_t st) {
  constexpr bool kByte = rows_byte_fmt(FMT);
  constexpr bool kHigh = FMT == RF_Q5K || FMT == RF_Q6K;   // three loads per row and span: fewer rows in flight
  constexpr int ppl = kByte ? 2 : 4;
  constexpr int span_k = 64 * ppl * 8;
  constexpr int SPU = kByte ? 4 : 2;
  constexpr bool kRegOk = MR <= 2;
  constexpr int RW2 = kHigh ? 1 : 2;
  a.nspan = (a.K + span_k - 1) / span_k;
  // Few rows (fewer than about four per wavefront): one row per batch.  A wavefront then walks
  // several small batches, so the next one loads while the current one is consumed and the work
  // left after the last load arrives is half as long; with many rows two rows per batch stream
  // better (measured: N = 4096..5120 gain 8-15 %, N >= 14336 lose 3-9 % with one row).
  long ntot = 0;
  for (int i = 0; i < a.nmat; ++i) ntot += a.N[i];
  const bool few = ntot < 4L * device_cu_count() * 8;
  if constexpr (!kByte && !kHigh && kRegOk) {
    if (a.nspan == 3) {
      if (few) return launch_rows_rw<Act, FMT, SC, MR, 1, 3, true>(a, st);
      return launch_rows_rw<Act, FMT, SC, MR, 2, 3, true>(a, st);
    }
  }
  if constexpr (kByte && MR == 1) {
    // K = 5120: five spans in registers instead of two batches (4 + 1) through LDS
    if (a.nspan == 5 && ntot >= 4096) return launch_rows_rw<Act, FMT, SC, MR, 1, 5, true>(a, st);
  }
  if constexpr (kRegOk) {
    // Rows shorter than the widest batch get a batch of exactly their own spans: an empty span
    // slot would still cost a (dead) load instruction and a pass of arithmetic on zeros.
    if (a.nspan == 1) {
      if (few) return launch_rows_rw<Act, FMT, SC, MR, 1, 1, true>(a, st);
      return launch_rows_rw<Act, FMT, SC, MR, 2, 1, true>(a, st);
    }
    if constexpr (kByte) {
      if (a.nspan == 2) {
        if (few) return launch_rows_rw<Act, FMT, SC, MR, 1, 2, true>(a, st);
        return launch_rows_rw<Act, FMT, SC, MR, 2, 2, true>(a, st);
      }
      if (a.nspan == 3) {
        if (few) return launch_rows_rw<Act, FMT, SC, MR, 1, 3, true>(a, st);
        return launch_rows_rw<Act, FMT, SC, MR, 2, 3, true>(a, st);
      }
    }
  }
  const int per_batch = a.nspan < SPU ? a.nspan : SPU;     // loads per row per batch
  const bool one_batch = kRegOk && a.nspan <= SPU;
  if (per_batch >= 4) {
    if constexpr (kRegOk) { if (one_batch) return launch_rows_rw<Act, FMT, SC, MR, 1, SPU, true>(a, st); }
    launch_rows_rw<Act, FMT, SC, MR, 1, SPU, false>(a, st);
  } else if (per_batch >= 2) {
    if (few) {
      if constexpr (kRegOk) { if (one_batch) return launch_rows_rw<Act, FMT, SC, MR, 1, SPU, true>(a, st); }
      return launch_rows_rw<Act, FMT, SC, MR, 1, SPU, false>(a, st);
    }
    if constexpr (kRegOk) { if (one_batch) return launch_rows_rw<Act, FMT, SC, MR, RW2, SPU, true>(a, st); }
    launch_rows_rw<Act, FMT, SC, MR, RW2, SPU, false>(a, st);
  } else {
    // rows of one span: two per batch (four were 15-30 % slower up to N = 16384 and equal
    // beyond), one when there are few rows
    if constexpr (kRegOk) {
      if (one_batch && few) return launch_rows_rw<Act, FMT, SC, MR, 1, SPU, true>(a, st);
      if (one_batch) return launch_rows_rw<Act, FMT, SC, MR, 2, SPU, true>(a, st);
    }
    launch_rows_rw<Act, FMT, SC, MR, 2, SPU, false>(a, st);
  }
}

// M == 1 with the RMS norm fused into the activation staging (LDS path).
template <class Act, int FMT, int SC>
static void launch_rows_norm(RowsArgs a, hipStream_t st) {
  constexpr bool kByte = rows_byte_fmt(FMT);
  constexpr int ppl = kByte ? 2 : 4;
  constexpr int span_k = 64 * ppl * 8;
  constexpr int SPU = kByte ? 4 : 2;
  a.nspan = (a.K + span_k - 1) / span_k;
  long ntot = 0;
  for (int i = 0; i < a.nmat; ++i) ntot += a.N[i];
  const bool few = ntot < 4L * device_cu_count() * 8;
  // short rows: batches of exactly their own spans, one row per batch when there are few rows
  if (a.nspan == 1) {
    if (few) return launch_rows_rw<Act, FMT, SC, 1, 1, 1, false, true>(a, st);
    return launch_rows_rw<Act, FMT, SC, 1, 2, 1, false, true>(a, st);
  }
  if constexpr (kByte) {
    if (a.nspan == 2) {
      if (few) return launch_rows_rw<Act, FMT, SC, 1, 1, 2, false, true>(a, st);
      return launch_rows_rw<Act, FMT, SC, 1, 2, 2, false, true>(a, st);
    }
    if (a.nspan == 3) {
      if (few) return launch_rows_rw<Act, FMT, SC, 1, 1, 3, false, true>(a, st);
      return launch_rows_rw<Act, FMT, SC, 1, 2, 3, false, true>(a, st);
    }
  } else {
    if (a.nspan == 2 && few) return launch_rows_rw<Act, FMT, SC, 1, 1, 2, false, true>(a, st);
  }
  const int per_batch = a.nspan < SPU ? a.nspan : SPU;
  if (per_batch >= 4)
    launch_rows_rw<Act, FMT, SC, 1, 1, SPU, false, true>(a, st);
  else if (per_batch >= 2)
    launch_rows_rw<Act, FMT, SC, 1, 2, SPU, false, true>(a, st);
  else
    launch_rows_rw<Act, FMT, SC, 1, 4, SPU, false, true>(a, st);
}

template <class Act, int FMT, int SC>
static void launch_rows_m(const RowsArgs& a, hipStream_t st) {
  switch (a.M) {
    case 1: launch_rows<Act, FMT, SC, 1>(a, st); break;
    case 2: launch_rows<Act, FMT, SC, 2>(a, st); break;
    default: launch_rows<Act, FMT, SC, 4>(a, st); break;
  }
}

}  // namespace qlin
