// Weight preparation and decode GEMV for the other GGUF formats (Q4_0, Q8_0,
// Q5_K, Q6_K) and the on-device group-128 Q4_0 quantizer.
//
// Repack: raw GGML blocks -> the resident representation the reference's ops
// read (interleaved nibbles, split scales, tile-shuffled high bits).  One
// thread per output byte / scale; the raw blocks (18 / 34 / 176 / 210 bytes)
// are not 16-byte aligned, so they are read bytewise through the cache.
// Dequant: resident representation -> dense fp16 with the reference's fp16
// roundings.  GEMV: the one-wavefront-per-row decode kernel, fp16 only.
#include "gemv_rows.hpp"
#include "gguf_skinny.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

static inline dim3 grid_for(size_t n, int block = 256) { return dim3((unsigned)((n + block - 1) / block)); }

__device__ __forceinline__ _Float16 ld_f16(const uint8_t* p) {
  return __builtin_bit_cast(_Float16, (uint16_t)(p[0] | (p[1] << 8)));
}

// the 6-bit (scale, min) pair j of a K-quant super-block's 12-byte field
__device__ __forceinline__ void scale_min_k4(int j, const uint8_t* q, int& sc, int& mn) {
  if (j < 4) {
    sc = q[j] & 63;
    mn = q[j + 4] & 63;
  } else {
    sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
    mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
  }
}

// ---------------------------------------------------------------- Q4_0 ----
// block = {fp16 d; u8 qs[16]}, byte j = elem j | elem j+16 << 4
__global__ __launch_bounds__(256) void q4_0_repack_kernel(const uint8_t* __restrict__ raw,
                                                          uint8_t* __restrict__ packed,
                                                          _Float16* __restrict__ scale, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;     // output byte
  const size_t total = (size_t)N * (K >> 1);
  if (i >= total) return;
  const int half = K >> 1, nb = K >> 5;
  const int n = (int)(i / half), j = (int)(i % half);
  const int blk = j >> 4, jj = j & 15;                                // elements 2jj, 2jj+1 of the block
  const uint8_t* b = raw + ((size_t)n * nb + blk) * 18;
  auto elem = [&](int e) -> uint32_t {
    const uint32_t byte = b[2 + (e & 15)];
    return e < 16 ? (byte & 0xF) : (byte >> 4);
  };
  packed[i] = (uint8_t)(elem(2 * jj) | (elem(2 * jj + 1) << 4));
  if (jj == 0) scale[(size_t)n * nb + blk] = ld_f16(b);
}

// ---------------------------------------------------------------- Q8_0 ----
__global__ __launch_bounds__(256) void q8_0_repack_kernel(const uint8_t* __restrict__ raw,
                                                          uint8_t* __restrict__ qs,
                                                          _Float16* __restrict__ scale, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;     // output byte = element
  const size_t total = (size_t)N * K;
  if (i >= total) return;
  const int nb = K >> 5;
  const int n = (int)(i / K), k = (int)(i % K);
  const int blk = k >> 5, e = k & 31;
  const uint8_t* b = raw + ((size_t)n * nb + blk) * 34;
  qs[i] = b[2 + e];
  if (e == 0) scale[(size_t)n * nb + blk] = ld_f16(b);
}

// ---------------------------------------------------------------- Q5_K ----
// super-block = {fp16 d, dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]} per 256.
// element e = 64 il + 32 half + p: nibble of qs[32 il + p] (low / high), fifth
// bit = bit (2 il + half) of qh[p].
__device__ __forceinline__ uint32_t q5k_value(const uint8_t* sb, int e) {
  const int il = e >> 6, half = (e >> 5) & 1, p = e & 31;
  const uint32_t byte = sb[48 + 32 * il + p];
  const uint32_t nib = half ? (byte >> 4) : (byte & 0xF);
  return nib | (((sb[16 + p] >> (2 * il + half)) & 1u) << 4);
}

__global__ __launch_bounds__(256) void q5k_repack_ql_kernel(const uint8_t* __restrict__ raw,
                                                            uint8_t* __restrict__ ql, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)N * (K >> 1);
  if (i >= total) return;
  const int half = K >> 1, nsb = K >> 8;
  const int n = (int)(i / half), j = (int)(i % half);
  const int e = 2 * j;
  const uint8_t* sb = raw + ((size_t)n * nsb + (e >> 8)) * 176;
  ql[i] = (uint8_t)((q5k_value(sb, e & 255) & 0xF) | ((q5k_value(sb, (e & 255) + 1) & 0xF) << 4));
}

// qh byte (tile, t): bit b = fifth bit of element tile*512 + b*64 + t
__global__ __launch_bounds__(256) void q5k_repack_qh_kernel(const uint8_t* __restrict__ raw,
                                                            uint8_t* __restrict__ qh, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)N * (K >> 3);
  if (i >= total) return;
  const int per = K >> 3, nsb = K >> 8;
  const int n = (int)(i / per), j = (int)(i % per);
  const int tile = j >> 6, t = j & 63;
  uint32_t byte = 0;
#pragma unroll
  for (int b = 0; b < 8; ++b) {
    const int e = tile * 512 + b * 64 + t;
    const uint8_t* sb = raw + ((size_t)n * nsb + (e >> 8)) * 176;
    byte |= ((q5k_value(sb, e & 255) >> 4) & 1u) << b;
  }
  qh[i] = (uint8_t)byte;
}

// element-order qh (what the MoE down stacks carry): bit b of byte j = fifth bit of element 8j + b
__global__ __launch_bounds__(256) void q5k_repack_qh_plain_kernel(const uint8_t* __restrict__ raw,
                                                                  uint8_t* __restrict__ qh, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)N * (K >> 3);
  if (i >= total) return;
  const int per = K >> 3, nsb = K >> 8;
  const int n = (int)(i / per), j = (int)(i % per);
  const uint8_t* sb = raw + ((size_t)n * nsb + (j >> 5)) * 176;
  uint32_t byte = 0;
#pragma unroll
  for (int b = 0; b < 8; ++b) byte |= ((q5k_value(sb, ((8 * j) & 255) + b) >> 4) & 1u) << b;
  qh[i] = (uint8_t)byte;
}

// scale = fp16(f32(d) * sc6), min = fp16(f32(dmin) * mn6); RAWB = 144 (Q4_K) or 176 (Q5_K)
__global__ __launch_bounds__(256) void kquant_scale_min_kernel(const uint8_t* __restrict__ raw, int rawb,
                                                               _Float16* __restrict__ scale,
                                                               _Float16* __restrict__ qmin, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)N * (K >> 5);
  if (i >= total) return;
  const int per = K >> 5, nsb = K >> 8;
  const int n = (int)(i / per), c = (int)(i % per);
  const uint8_t* sb = raw + ((size_t)n * nsb + (c >> 3)) * rawb;
  int sc, mn;
  scale_min_k4(c & 7, sb + 4, sc, mn);
  scale[i] = (_Float16)((float)ld_f16(sb) * (float)sc);
  qmin[i] = (_Float16)((float)ld_f16(sb + 2) * (float)mn);
}

// ---------------------------------------------------------------- Q6_K ----
// super-block = {u8 ql[128]; u8 qh[64]; i8 scales[16]; fp16 d} per 256.
// element e = 128 ip + 32 quarter + l: nibble of ql[64 ip + 32 (quarter & 1) + l]
// (low for quarter < 2), top bits = field `quarter` of qh[32 ip + l].
__device__ __forceinline__ uint32_t q6k_value(const uint8_t* sb, int e) {
  const int ip = e >> 7, quarter = (e >> 5) & 3, l = e & 31;
  const uint32_t byte = sb[64 * ip + 32 * (quarter & 1) + l];
  const uint32_t nib = quarter >= 2 ? (byte >> 4) : (byte & 0xF);
  return nib | (((sb[128 + 32 * ip + l] >> (2 * quarter)) & 3u) << 4);
}

__global__ __launch_bounds__(256) void q6k_repack_ql_kernel(const uint8_t* __restrict__ raw,
                                                            uint8_t* __restrict__ ql, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)N * (K >> 1);
  if (i >= total) return;
  const int half = K >> 1, nsb = K >> 8;
  const int n = (int)(i / half), j = (int)(i % half);
  const int e = 2 * j;
  const uint8_t* sb = raw + ((size_t)n * nsb + (e >> 8)) * 210;
  ql[i] = (uint8_t)((q6k_value(sb, e & 255) & 0xF) | ((q6k_value(sb, (e & 255) + 1) & 0xF) << 4));
}

// qh byte (tile, t): 2-bit field p = top bits of element tile*512 + p*128 + t
__global__ __launch_bounds__(256) void q6k_repack_qh_kernel(const uint8_t* __restrict__ raw,
                                                            uint8_t* __restrict__ qh, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)N * (K >> 2);
  if (i >= total) return;
  const int per = K >> 2, nsb = K >> 8;
  const int n = (int)(i / per), j = (int)(i % per);
  const int tile = j >> 7, t = j & 127;
  uint32_t byte = 0;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int e = tile * 512 + p * 128 + t;
    const uint8_t* sb = raw + ((size_t)n * nsb + (e >> 8)) * 210;
    byte |= ((q6k_value(sb, e & 255) >> 4) & 3u) << (2 * p);
  }
  qh[i] = (uint8_t)byte;
}

// element-order qh: 2-bit field p of byte j = top bits of element 4j + p
__global__ __launch_bounds__(256) void q6k_repack_qh_plain_kernel(const uint8_t* __restrict__ raw,
                                                                  uint8_t* __restrict__ qh, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)N * (K >> 2);
  if (i >= total) return;
  const int per = K >> 2, nsb = K >> 8;
  const int n = (int)(i / per), j = (int)(i % per);
  const uint8_t* sb = raw + ((size_t)n * nsb + (j >> 6)) * 210;
  uint32_t byte = 0;
#pragma unroll
  for (int p = 0; p < 4; ++p) byte |= ((q6k_value(sb, ((4 * j) & 255) + p) >> 4) & 3u) << (2 * p);
  qh[i] = (uint8_t)byte;
}

__global__ __launch_bounds__(256) void q6k_scale_kernel(const uint8_t* __restrict__ raw,
                                                        _Float16* __restrict__ scale, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)N * (K >> 4);
  if (i >= total) return;
  const int per = K >> 4, nsb = K >> 8;
  const int n = (int)(i / per), c = (int)(i % per);
  const uint8_t* sb = raw + ((size_t)n * nsb + (c >> 4)) * 210;
  scale[i] = (_Float16)((float)ld_f16(sb + 208) * (float)(int8_t)sb[192 + (c & 15)]);
}

// ------------------------------------------------------------- dequant ----
// One thread per 8 consecutive k = one 32-bit word of interleaved nibbles (or 8 bytes).
__global__ __launch_bounds__(256) void dequant_q4_0_kernel(const uint32_t* __restrict__ packed,
                                                           const _Float16* __restrict__ scale,
                                                           f16x8* __restrict__ out, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)N * (K >> 3)) return;
  const int wpr = K >> 3;
  const int n = (int)(i / wpr), k = (int)(i % wpr) * 8;
  // (nib - 8) * d: exact difference, one rounding
  out[i] = int4x8_to_f16(packed[i], scale[(size_t)n * (K >> 5) + (k >> 5)], (_Float16)1032.0f);
}

__global__ __launch_bounds__(256) void dequant_q8_0_kernel(const u32x2* __restrict__ qs,
                                                           const _Float16* __restrict__ scale,
                                                           f16x8* __restrict__ out, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)N * (K >> 3)) return;
  const int wpr = K >> 3;
  const int n = (int)(i / wpr), k = (int)(i % wpr) * 8;
  const _Float16 s = scale[(size_t)n * (K >> 5) + (k >> 5)];
  const u32x2 v = qs[i];
  f16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int q = (int)(int8_t)((v[e >> 2] >> (8 * (e & 3))) & 0xFF);
    o[e] = (_Float16)q * s;                          // fp16(q) exact, one rounding
  }
  out[i] = o;
}

// high bits of elements k .. k+7 (k % 8 == 0) from the tile-shuffled qh
__device__ __forceinline__ void high8(const uint8_t* __restrict__ qh_row, int k, int bits, uint32_t (&h)[8]) {
  const int tile = k >> 9, r = k & 511;
  if (bits == 1) {
    const int b = r >> 6, t = r & 63;
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = (qh_row[tile * 64 + t + e] >> b) & 1u;
  } else {
    const int p = r >> 7, t = r & 127;
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = (qh_row[tile * 128 + t + e] >> (2 * p)) & 3u;
  }
}

__global__ __launch_bounds__(256) void dequant_q5k_kernel(const uint32_t* __restrict__ ql,
                                                          const uint8_t* __restrict__ qh,
                                                          const _Float16* __restrict__ scale,
                                                          const _Float16* __restrict__ qmin,
                                                          f16x8* __restrict__ out, int N, int K) {
#pragma clang fp contract(off)
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)N * (K >> 3)) return;
  const int wpr = K >> 3;
  const int n = (int)(i / wpr), k = (int)(i % wpr) * 8;
  const size_t c = (size_t)n * (K >> 5) + (k >> 5);
  const _Float16 s = scale[c], m = qmin[c];
  uint32_t h[8];
  high8(qh + (size_t)n * (K >> 3), k, 1, h);
  const uint32_t w = ql[i];
  f16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const _Float16 v = (_Float16)(float)(((w >> (4 * e)) & 0xF) | (h[e] << 4));
    _Float16 prod = v * s;                           // rounded on its own, then the subtraction
    asm volatile("" : "+v"(prod));
    o[e] = prod - m;
  }
  out[i] = o;
}

__global__ __launch_bounds__(256) void dequant_q6k_kernel(const uint32_t* __restrict__ ql,
                                                          const uint8_t* __restrict__ qh,
                                                          const _Float16* __restrict__ scale,
                                                          f16x8* __restrict__ out, int N, int K) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)N * (K >> 3)) return;
  const int wpr = K >> 3;
  const int n = (int)(i / wpr), k = (int)(i % wpr) * 8;
  const _Float16 s = scale[(size_t)n * (K >> 4) + (k >> 4)];
  uint32_t h[8];
  high8(qh + (size_t)n * (K >> 2), k, 2, h);
  const uint32_t w = ql[i];
  f16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int v = (int)(((w >> (4 * e)) & 0xF) | (h[e] << 4)) - 32;
    o[e] = (_Float16)(float)v * s;                   // (v6 - 32) exact, one rounding
  }
  out[i] = o;
}

// ------------------------------------------------- group-128 quantizer ----
// GGML quantize_row_q4_0 on 128-wide blocks: 16 lanes per block, 8 consecutive
// elements per lane.  max = first element of largest magnitude (sign kept);
// d = max / -8; id = 1 / d in fp32 (0 for an all-zero block); q = min(15,
// trunc(x * id + 8.5)), product and sum rounded separately.
template <class Act>
__global__ __launch_bounds__(256) void q4_0_quantize_kernel(const typename Act::v8* __restrict__ x,
                                                            uint32_t* __restrict__ qweight,
                                                            _Float16* __restrict__ scale,
                                                            size_t nblocks) {
#pragma clang fp contract(off)   // x * id and + 8.5 round separately, as the CPU rule does
  const size_t gi = (size_t)blockIdx.x * blockDim.x + threadIdx.x;    // 8-element group
  const size_t blk = gi >> 4;
  const int sub = (int)(gi & 15);
  const bool live = blk < nblocks;
  float v[8];
  if (live) {
    const typename Act::v8 in = x[gi];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (float)in[e];
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.f;
  }
  // key = (|v| bits, 127 - index, sign): the maximum is the largest magnitude, lowest index
  uint64_t key = 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, v[e]);
    const uint64_t k = ((uint64_t)(bits & 0x7FFFFFFFu) << 32) | ((uint64_t)(127 - (sub * 8 + e)) << 1) | (bits >> 31);
    key = k > key ? k : key;
  }
#pragma unroll
  for (int off = 1; off < 16; off <<= 1) {
    const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)key, off, 16);
    const uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(key >> 32), off, 16);
    const uint64_t other = ((uint64_t)hi << 32) | lo;
    key = other > key ? other : key;
  }
  const float amax = __builtin_bit_cast(float, (uint32_t)(key >> 32));
  const float mx = (key & 1) ? -amax : amax;
  const float d = mx * -0.125f;                       // max / -8, exact scaling
  // correctly rounded reciprocal (through fp64: a rounded fp64 quotient never sits on an
  // fp32 rounding boundary unless it is exact); the fast fp32 reciprocal is an ulp off at times
  const float id = d != 0.f ? (float)(1.0 / (double)d) : 0.f;
  uint32_t word = 0;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float prod = v[e] * id;
    asm volatile("" : "+v"(prod));               // keep the rounded product: no fused multiply-add
    const float t = prod + 8.5f;
    int q = (int)t;                                   // truncation, t >= 0.5
    q = q < 0 ? 0 : (q > 15 ? 15 : q);
    word |= (uint32_t)q << (4 * e);
  }
  if (live) {
    qweight[gi] = word;
    if (sub == 0) scale[blk] = (_Float16)d;
  }
}

// ----------------------------------------------------------------- GEMV ----
template <int FMT>
static int run_gguf_gemv(RowsArgs r, int M, hipStream_t st) {
  if (!r.x || !r.w[0] || !r.s[0] || !r.out[0]) return MI_ERR_ARG;
  if (M < 0 || r.N[0] < 0 || r.K <= 0) return MI_ERR_SHAPE;
  if ((uint64_t)r.N[0] * (uint64_t)r.K >= (1ull << 31)) return MI_ERR_SHAPE;
  if (M == 0 || r.N[0] == 0) return MI_OK;
  // more than four rows: the MFMA kernels (64 rows per pass); Q4_0 from three rows when x fits the
  // registers (K=N=5120: 10.0 against 11.6-11.9 us on the row kernel)
  if (M > 4 || (FMT == 3 && M > 2 && gguf_skinny_resident(FMT, M, r.K)))
    return gguf_skinny(FMT, r.x, r.w[0], r.h[0], r.s[0], r.z[0], r.out[0], M, r.N[0], r.K, st);
  // rows per launch: as many (4, 2, 1) as the staged activations allow in 64 KiB of LDS
  int step = 4;
  while (step > 1 && rows_lds_bytes(FMT, step, r.K) > 64 * 1024) step >>= 1;
  if (rows_lds_bytes(FMT, step, r.K) > 64 * 1024) return MI_ERR_SHAPE;
  const char* x = (const char*)r.x;
  char* out = (char*)r.out[0];
  for (int m0 = 0; m0 < M; m0 += step) {
    RowsArgs c = r;
    c.M = (M - m0) < step ? (M - m0) : step;
    c.x = x + (size_t)m0 * r.K * 2;
    c.out[0] = out + (size_t)m0 * r.N[0] * 2;
    launch_rows_m<ActF16, FMT, RS_PERN>(c, st);
  }
  return launch_status();
}

// Routed decode GEMVs of a GGUF MoE layer: one launch over all (token, expert) routes.
template <int FMT>
static int run_gguf_routed(RowsArgs r, int routes, hipStream_t st) {
  if (rows_lds_bytes(FMT, 1, r.K) > 64 * 1024) return MI_ERR_SHAPE;
  launch_rows_routed<ActF16, FMT>(r, routes, st);
  return launch_status();
}

}  // namespace qlin

using namespace qlin;

extern "C" {

int mi_moe_gguf_gemv(int fmt, const void* x, int x_div, int nmat, const void* const* ql, const void* const* qh,
                     const void* const* scale, const void* const* qmin, void* const* out, long long out_stride,
                     const int32_t* route_expert, const void* route_weight, int routes, int num_experts, int N,
                     int K, void* stream) {
  if (!x || !ql || !scale || !out || !route_expert) return MI_ERR_ARG;
  if (fmt != RF_Q4K && fmt != RF_Q5K && fmt != RF_Q6K) return MI_ERR_ARG;
  if (nmat < 1 || nmat > 2 || x_div < 1 || num_experts < 1) return MI_ERR_ARG;
  if (routes < 0 || N < 0 || K <= 0 || out_stride < N) return MI_ERR_SHAPE;
  if (K % 32) return MI_ERR_SHAPE;
  if ((uint64_t)N * (uint64_t)K >= (1ull << 31) || routes > 65535) return MI_ERR_SHAPE;
  if (!routes || !N) return MI_OK;
  const long long nk = (long long)N * K;
  for (int i = 0; i < nmat; ++i) {
    if (!ql[i] || !scale[i] || !out[i]) return MI_ERR_ARG;
    if (fmt != RF_Q6K && (!qmin || !qmin[i])) return MI_ERR_ARG;
    if (fmt != RF_Q4K && (!qh || !qh[i])) return MI_ERR_ARG;
  }
  hipStream_t st = (hipStream_t)stream;
  // one launch per matrix: with several matrices in one routed launch the per-route copy of the
  // arguments is indexed by matrix and ends up in memory (measured 116 us against 2 x 6.6 us)
  for (int i = 0; i < nmat; ++i) {
    RowsArgs r{};
    r.x = x; r.nmat = 1; r.M = 1; r.K = K;
    r.r_expert = route_expert; r.r_out_mul = route_weight; r.r_num_experts = num_experts; r.r_x_div = x_div;
    r.r_out_stride = out_stride;
    r.w[0] = ql[i]; r.s[0] = scale[i]; r.out[0] = out[i]; r.N[0] = N;
    r.z[0] = fmt != RF_Q6K ? qmin[i] : nullptr;
    r.h[0] = fmt != RF_Q4K ? qh[i] : nullptr;
    r.r_w_stride[0] = nk / 2;
    r.r_s_stride[0] = fmt == RF_Q6K ? nk / 16 * 2 : nk / 32 * 2;
    r.r_z_stride[0] = nk / 32 * 2;
    r.r_h_stride[0] = fmt == RF_Q5K ? nk / 8 : nk / 4;
    const int rc = fmt == RF_Q4K ? run_gguf_routed<RF_Q4K>(r, routes, st)
                                 : (fmt == RF_Q5K ? run_gguf_routed<RF_Q5K>(r, routes, st)
                                                  : run_gguf_routed<RF_Q6K>(r, routes, st));
    if (rc != MI_OK) return rc;
  }
  return MI_OK;
}

int mi_q4_0_repack(const void* raw, void* packed, void* scale, int N, int K, void* stream) {
  if (!raw || !packed || !scale) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 32)) return MI_ERR_SHAPE;
  if (N == 0) return MI_OK;
  const size_t n = (size_t)N * (K >> 1);
  hipLaunchKernelGGL(q4_0_repack_kernel, grid_for(n), dim3(256), 0, (hipStream_t)stream, (const uint8_t*)raw,
                     (uint8_t*)packed, (_Float16*)scale, N, K);
  return launch_status();
}

int mi_q8_0_repack(const void* raw, void* qs, void* scale, int N, int K, void* stream) {
  if (!raw || !qs || !scale) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 32)) return MI_ERR_SHAPE;
  if (N == 0) return MI_OK;
  hipLaunchKernelGGL(q8_0_repack_kernel, grid_for((size_t)N * K), dim3(256), 0, (hipStream_t)stream,
                     (const uint8_t*)raw, (uint8_t*)qs, (_Float16*)scale, N, K);
  return launch_status();
}

int mi_q5k_repack(const void* raw, void* ql, void* qh, void* scale, void* qmin, int N, int K, void* stream) {
  if (!raw || !ql || !qh || !scale || !qmin) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 512)) return MI_ERR_SHAPE;
  if (N == 0) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(q5k_repack_ql_kernel, grid_for((size_t)N * (K >> 1)), dim3(256), 0, st, (const uint8_t*)raw,
                     (uint8_t*)ql, N, K);
  hipLaunchKernelGGL(q5k_repack_qh_kernel, grid_for((size_t)N * (K >> 3)), dim3(256), 0, st, (const uint8_t*)raw,
                     (uint8_t*)qh, N, K);
  hipLaunchKernelGGL(kquant_scale_min_kernel, grid_for((size_t)N * (K >> 5)), dim3(256), 0, st, (const uint8_t*)raw,
                     176, (_Float16*)scale, (_Float16*)qmin, N, K);
  return launch_status();
}

int mi_q6k_repack(const void* raw, void* ql, void* qh, void* scale, int N, int K, void* stream) {
  if (!raw || !ql || !qh || !scale) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 512)) return MI_ERR_SHAPE;
  if (N == 0) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(q6k_repack_ql_kernel, grid_for((size_t)N * (K >> 1)), dim3(256), 0, st, (const uint8_t*)raw,
                     (uint8_t*)ql, N, K);
  hipLaunchKernelGGL(q6k_repack_qh_kernel, grid_for((size_t)N * (K >> 2)), dim3(256), 0, st, (const uint8_t*)raw,
                     (uint8_t*)qh, N, K);
  hipLaunchKernelGGL(q6k_scale_kernel, grid_for((size_t)N * (K >> 4)), dim3(256), 0, st, (const uint8_t*)raw,
                     (_Float16*)scale, N, K);
  return launch_status();
}

int mi_q5k_repack_plain(const void* raw, void* ql, void* qh, void* scale, void* qmin, int N, int K, void* stream) {
  if (!raw || !ql || !qh || !scale || !qmin) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 256)) return MI_ERR_SHAPE;
  if (N == 0) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(q5k_repack_ql_kernel, grid_for((size_t)N * (K >> 1)), dim3(256), 0, st, (const uint8_t*)raw,
                     (uint8_t*)ql, N, K);
  hipLaunchKernelGGL(q5k_repack_qh_plain_kernel, grid_for((size_t)N * (K >> 3)), dim3(256), 0, st,
                     (const uint8_t*)raw, (uint8_t*)qh, N, K);
  hipLaunchKernelGGL(kquant_scale_min_kernel, grid_for((size_t)N * (K >> 5)), dim3(256), 0, st, (const uint8_t*)raw,
                     176, (_Float16*)scale, (_Float16*)qmin, N, K);
  return launch_status();
}

int mi_q6k_repack_plain(const void* raw, void* ql, void* qh, void* scale, int N, int K, void* stream) {
  if (!raw || !ql || !qh || !scale) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 256)) return MI_ERR_SHAPE;
  if (N == 0) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(q6k_repack_ql_kernel, grid_for((size_t)N * (K >> 1)), dim3(256), 0, st, (const uint8_t*)raw,
                     (uint8_t*)ql, N, K);
  hipLaunchKernelGGL(q6k_repack_qh_plain_kernel, grid_for((size_t)N * (K >> 2)), dim3(256), 0, st,
                     (const uint8_t*)raw, (uint8_t*)qh, N, K);
  hipLaunchKernelGGL(q6k_scale_kernel, grid_for((size_t)N * (K >> 4)), dim3(256), 0, st, (const uint8_t*)raw,
                     (_Float16*)scale, N, K);
  return launch_status();
}

int mi_dequant_q4_0(const void* packed, const void* scale, void* out, int N, int K, void* stream) {
  if (!packed || !scale || !out) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 32)) return MI_ERR_SHAPE;
  if (N == 0) return MI_OK;
  hipLaunchKernelGGL(dequant_q4_0_kernel, grid_for((size_t)N * (K >> 3)), dim3(256), 0, (hipStream_t)stream,
                     (const uint32_t*)packed, (const _Float16*)scale, (f16x8*)out, N, K);
  return launch_status();
}

int mi_dequant_q8_0(const void* qs, const void* scale, void* out, int N, int K, void* stream) {
  if (!qs || !scale || !out) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 32)) return MI_ERR_SHAPE;
  if (N == 0) return MI_OK;
  hipLaunchKernelGGL(dequant_q8_0_kernel, grid_for((size_t)N * (K >> 3)), dim3(256), 0, (hipStream_t)stream,
                     (const u32x2*)qs, (const _Float16*)scale, (f16x8*)out, N, K);
  return launch_status();
}

int mi_dequant_q5k(const void* ql, const void* qh, const void* scale, const void* qmin, void* out, int N, int K,
                   void* stream) {
  if (!ql || !qh || !scale || !qmin || !out) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 512)) return MI_ERR_SHAPE;
  if (N == 0) return MI_OK;
  hipLaunchKernelGGL(dequant_q5k_kernel, grid_for((size_t)N * (K >> 3)), dim3(256), 0, (hipStream_t)stream,
                     (const uint32_t*)ql, (const uint8_t*)qh, (const _Float16*)scale, (const _Float16*)qmin,
                     (f16x8*)out, N, K);
  return launch_status();
}

int mi_dequant_q6k(const void* ql, const void* qh, const void* scale, void* out, int N, int K, void* stream) {
  if (!ql || !qh || !scale || !out) return MI_ERR_ARG;
  if (N < 0 || K <= 0 || (K % 512)) return MI_ERR_SHAPE;
  if (N == 0) return MI_OK;
  hipLaunchKernelGGL(dequant_q6k_kernel, grid_for((size_t)N * (K >> 3)), dim3(256), 0, (hipStream_t)stream,
                     (const uint32_t*)ql, (const uint8_t*)qh, (const _Float16*)scale, (f16x8*)out, N, K);
  return launch_status();
}

int mi_q4_0_quantize(const void* x, void* qweight, void* scale, int rows, int K, int in_dtype, void* stream) {
  if (!x || !qweight || !scale) return MI_ERR_ARG;
  if (in_dtype != DT_F16 && in_dtype != DT_BF16) return MI_ERR_ARG;
  if (rows < 0 || K <= 0 || (K % 128)) return MI_ERR_SHAPE;
  if (rows == 0) return MI_OK;
  const size_t nblocks = (size_t)rows * (K >> 7);
  const dim3 grid = grid_for(nblocks * 16);
  if (in_dtype == DT_F16)
    hipLaunchKernelGGL(q4_0_quantize_kernel<ActF16>, grid, dim3(256), 0, (hipStream_t)stream,
                       (const ActF16::v8*)x, (uint32_t*)qweight, (_Float16*)scale, nblocks);
  else
    hipLaunchKernelGGL(q4_0_quantize_kernel<ActBF16>, grid, dim3(256), 0, (hipStream_t)stream,
                       (const ActBF16::v8*)x, (uint32_t*)qweight, (_Float16*)scale, nblocks);
  return launch_status();
}

int mi_gemv_q4_0(const void* x, const void* packed, const void* scale, void* out, int M, int N, int K,
                 void* stream) {
  if (K % 32) return MI_ERR_SHAPE;
  RowsArgs r{};
  r.x = x; r.w[0] = packed; r.s[0] = scale; r.out[0] = out; r.N[0] = N; r.nmat = 1; r.K = K;
  return run_gguf_gemv<RF_Q40>(r, M, (hipStream_t)stream);
}

int mi_gemv_q8_0(const void* x, const void* qs, const void* scale, void* out, int M, int N, int K, void* stream) {
  if (K % 32) return MI_ERR_SHAPE;
  RowsArgs r{};
  r.x = x; r.w[0] = qs; r.s[0] = scale; r.out[0] = out; r.N[0] = N; r.nmat = 1; r.K = K;
  return run_gguf_gemv<RF_Q80>(r, M, (hipStream_t)stream);
}

int mi_gemv_q5k(const void* x, const void* ql, const void* qh, const void* scale, const void* qmin, void* out,
                int M, int N, int K, void* stream) {
  if (!qh || !qmin) return MI_ERR_ARG;
  if (K % 512) return MI_ERR_SHAPE;
  RowsArgs r{};
  r.x = x; r.w[0] = ql; r.h[0] = qh; r.s[0] = scale; r.z[0] = qmin; r.out[0] = out; r.N[0] = N; r.nmat = 1;
  r.K = K;
  return run_gguf_gemv<RF_Q5K>(r, M, (hipStream_t)stream);
}

int mi_gemv_q6k(const void* x, const void* ql, const void* qh, const void* scale, void* out, int M, int N, int K,
                void* stream) {
  if (!qh) return MI_ERR_ARG;
  if (K % 512) return MI_ERR_SHAPE;
  RowsArgs r{};
  r.x = x; r.w[0] = ql; r.h[0] = qh; r.s[0] = scale; r.out[0] = out; r.N[0] = N; r.nmat = 1; r.K = K;
  return run_gguf_gemv<RF_Q6K>(r, M, (hipStream_t)stream);
}

}  // extern "C"
