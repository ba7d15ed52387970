// Shared device helpers for the gfx950 quantized-linear kernels.
//
// Everything here is written for CDNA4 only: 64-wide wavefronts, the
// 16x16x32 MFMA shapes, raw buffer loads (out-of-range lanes read zero) and
// the gfx950 FP8 (OCP e4m3fn) conversion instructions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qlin {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) int32_t i32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

enum : int { DT_F16 = 0, DT_BF16 = 1 };

// Error codes returned by every C-ABI entry point.
enum : int {
  MI_OK = 0,
  MI_ERR_ARG = -1,        // null pointer / bad enum
  MI_ERR_SHAPE = -2,      // shape or divisibility the kernels do not cover
  MI_ERR_LAUNCH = -3,     // hipGetLastError() after the launch
  MI_ERR_LIMIT = -4,      // size beyond the fixed capacity of a no-allocation entry point
  MI_ERR_BUSY = -5,       // the static scratch is claimed by another stream
};

// ---- raw buffer loads -------------------------------------------------------
// A buffer resource bounds every access: lanes whose byte offset lies past
// `bytes` read zeros, so ragged N / M / K tails need no branches.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
}
constexpr uint32_t kOOB = 0x80000000u;   // an offset no buffer here reaches

// ---- activation element types ----------------------------------------------
struct ActF16 {
  using elem = _Float16;
  using v8 = f16x8;
  static constexpr int dt = DT_F16;
  static __device__ __forceinline__ f32x4 mfma(v8 a, v8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ elem from_f32(float f) { return (_Float16)f; }
  static __device__ __forceinline__ float to_f32(elem e) { return (float)e; }
};
struct ActBF16 {
  using elem = __bf16;
  using v8 = bf16x8;
  static constexpr int dt = DT_BF16;
  static __device__ __forceinline__ f32x4 mfma(v8 a, v8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ elem from_f32(float f) { return (__bf16)f; }
  static __device__ __forceinline__ float to_f32(elem e) { return (float)e; }
};

template <class V8>
__device__ __forceinline__ V8 as_v8(u32x4 r) {
  return __builtin_bit_cast(V8, r);
}

// ---- E4M3 -> 16-bit, exact ---------------------------------------------------
// Every finite E4M3 value (subnormals included) is representable in fp16 and in
// bf16, so the conversion is exact; NaN codes stay NaN.
template <class Act>
__device__ __forceinline__ typename Act::v8 fp8x8_to_act(uint32_t lo, uint32_t hi);

template <>
__device__ __forceinline__ f16x8 fp8x8_to_act<ActF16>(uint32_t lo, uint32_t hi) {
  f16x2 a = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, false);
  f16x2 b = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, true);
  f16x2 c = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, false);
  f16x2 d = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, true);
  return f16x8{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}
template <>
__device__ __forceinline__ bf16x8 fp8x8_to_act<ActBF16>(uint32_t lo, uint32_t hi) {
  bf16x2 a = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false);
  bf16x2 b = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
  bf16x2 c = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false);
  bf16x2 d = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
  return bf16x8{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

__device__ __forceinline__ float fp8_to_f32(uint32_t byte) {
  return __builtin_amdgcn_cvt_f32_fp8(byte, 0);
}

// ---- INT4 (offset-binary nibbles, low nibble = even k) -> 16-bit, exact ------
// One dword holds 8 consecutive k.  Result element i = rne((nib_i - z) * s).
//
// fp16: nib is planted in the mantissa of 1024.0 (0x6400 | nib), (1024 + z) is
// subtracted exactly, and one v_pk_mul_f16 rounds the exact product once — the
// same single rounding as f32(nib - z) * f32(s) -> fp16.
__device__ __forceinline__ f16x8 int4x8_to_f16(uint32_t w, _Float16 s, _Float16 z1024) {
  const uint32_t e = w & 0x0F0F0F0Fu;
  const uint32_t o = (w >> 4) & 0x0F0F0F0Fu;
  f16x2 sv = {s, s};
  f16x2 zv = {z1024, z1024};
  f16x8 out;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const uint32_t sel = 0x0C000C00u | ((4u + p) << 16) | (uint32_t)p;
    const uint32_t bits = __builtin_amdgcn_perm(o, e, sel) | 0x64006400u;
    f16x2 v = __builtin_bit_cast(f16x2, bits);
    v = (v - zv) * sv;
    out[2 * p] = v[0];
    out[2 * p + 1] = v[1];
  }
  return out;
}

// bf16: (nib - z) is an exact small integer and its product with the fp16 scale
// is exact in fp32 (5 x 11 significant bits), so the only rounding is the RNE to
// bf16.  Subtract-then-multiply (not an fma with -z*s) keeps the sign of a zero
// result: (8 - 8) * negative scale is -0.
__device__ __forceinline__ bf16x8 int4x8_to_bf16(uint32_t w, float s, float z) {
  bf16x8 out;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float nib = (float)((w >> (4 * i)) & 0xFu);
    out[i] = (__bf16)((nib - z) * s);
  }
  return out;
}

// ---- Q4_K repacked sub-block -> fp16, two roundings ---------------------------
// w = fp16(fp16(nib * scale) - min): the product is rounded before the
// subtraction, exactly as two separate fp16 ops do; contraction into an fma
// would change about one value in five.
__device__ __forceinline__ f16x8 q4kx8_to_f16(uint32_t w, _Float16 s, _Float16 m) {
#pragma clang fp contract(off)
  const uint32_t e = w & 0x0F0F0F0Fu;
  const uint32_t o = (w >> 4) & 0x0F0F0F0Fu;
  f16x2 sv = {s, s};
  f16x2 mv = {m, m};
  f16x2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
  f16x8 out;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const uint32_t sel = 0x0C000C00u | ((4u + p) << 16) | (uint32_t)p;
    const uint32_t bits = __builtin_amdgcn_perm(o, e, sel) | 0x64006400u;
    f16x2 v = __builtin_bit_cast(f16x2, bits);
    v = v - k1024;
    f16x2 prod = v * sv;
    // keep the product as its own rounded value
    asm volatile("" : "+v"(prod));
    v = prod - mv;
    out[2 * p] = v[0];
    out[2 * p + 1] = v[1];
  }
  return out;
}

// Q8_0: eight signed bytes -> fp16(q) * s, one rounding.  0x6400 | (q ^ 0x80) = 1152 + q
// exactly; the subtraction is exact, the product rounds once.
__device__ __forceinline__ f16x8 i8x8_to_f16(uint32_t w0, uint32_t w1, _Float16 s) {
#pragma clang fp contract(off)
  const f16x2 k1152 = {(_Float16)1152.0f, (_Float16)1152.0f};
  const f16x2 sv = {s, s};
  f16x8 out;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const uint32_t u = (p < 2 ? w0 : w1) ^ 0x80808080u;
    const uint32_t sel = (p & 1) ? 0x04030402u : 0x04010400u;
    f16x2 v = __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(0x64646464u, u, sel));
    v = (v - k1152) * sv;
    out[2 * p] = v[0];
    out[2 * p + 1] = v[1];
  }
  return out;
}

// Q5_K (BITS = 1) / Q6_K (BITS = 2): eight nibbles in w plus their high bits — bytes of hA
// (elements 0..3) and hB (elements 4..7), the field starting at bit `shift` of each byte.
//   Q5_K: fp16(fp16(v * s) - m) with v = nib + 16 h (two roundings, like Q4_K);
//   Q6_K: (v - 32) * s with v = nib + 16 h (exact difference, one rounding; m unused).
template <int BITS>
__device__ __forceinline__ f16x8 kqx8_to_f16(uint32_t w, uint32_t hA, uint32_t hB, uint32_t shift, _Float16 s,
                                             _Float16 m) {
#pragma clang fp contract(off)
  constexpr uint32_t mask = BITS == 1 ? 0x01010101u : 0x03030303u;
  const uint32_t e = w & 0x0F0F0F0Fu;
  const uint32_t o = (w >> 4) & 0x0F0F0F0Fu;
  const uint32_t a = (hA >> shift) & mask, bq = (hB >> shift) & mask;
  const f16x2 sv = {s, s};
  const f16x2 mv = {m, m};
  const f16x2 base = BITS == 1 ? f16x2{(_Float16)1024.0f, (_Float16)1024.0f} : f16x2{(_Float16)1056.0f, (_Float16)1056.0f};
  f16x8 out;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const uint32_t sel = 0x0C000C00u | ((4u + p) << 16) | (uint32_t)p;
    // elements 2p, 2p+1: their high-bit bytes are bytes (2p % 4), (2p % 4) + 1 of hA (p < 2) or hB
    const uint32_t hsrc = p < 2 ? a : bq;
    const uint32_t hsel = (p & 1) ? 0x0C030C02u : 0x0C010C00u;
    const uint32_t hi = __builtin_amdgcn_perm(hsrc, hsrc, hsel) << 4;
    const uint32_t bits = __builtin_amdgcn_perm(o, e, sel) | 0x64006400u | hi;
    f16x2 v = __builtin_bit_cast(f16x2, bits) - base;
    f16x2 prod = v * sv;
    if constexpr (BITS == 1) {
      asm volatile("" : "+v"(prod));                  // keep the product as its own rounded value
      prod = prod - mv;
    }
    out[2 * p] = prod[0];
    out[2 * p + 1] = prod[1];
  }
  return out;
}

// Sum over the 64 lanes with DPP (cross-lane operands inside the VALU, no LDS
// round trips): butterfly inside each row of 16 lanes, then the four row totals
// are read out with v_readlane.  Every lane returns the same total.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
  return v + __builtin_bit_cast(float, moved);
}
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);     // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);     // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);    // row_half_mirror
  v = dpp_add<0x140>(v);    // row_mirror
  const int b = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return (r0 + r1) + (r2 + r3);
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

static inline int launch_status() {
  return hipGetLastError() == hipSuccess ? MI_OK : MI_ERR_LAUNCH;
}

}  // namespace qlin
