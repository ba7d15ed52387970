// Prefill W4A16 GEMM for gfx950: out[M,N] = x[M,K] @ dequant(w[N,K])^T, int4
// weights in groups of 128 along K with fp16 scales and optional per-group
// zero-points, fp16 / bf16 activations.
//
// MFMA-bound regime (M in the thousands).  A workgroup of 4 wavefronts (2 x 2)
// owns a BM x BN output tile; each wavefront computes a (BM/2) x (BN/2) sub-tile
// with v_mfma_f32_16x16x32_{bf16,f16}, accumulators in the AGPR half of the
// register file.  What limits this kernel is LDS bandwidth (a CU sustains about
// 130 B/ns of ds_read_b128 and 75 B/ns of LDS writes, against ~1 us of MFMA work
// per 64-wide K step), so only the operand that has to be shared goes through LDS:
//   * weights: each 64-wide K step of the BN weight rows is loaded once per
//     workgroup (128-bit loads of 32 nibbles), dequantized to the activation type
//     in registers and written to a double-buffered LDS tile (row pitch 144 B, so
//     the 16 rows of an MFMA operand read fall into distinct banks); every weight
//     is dequantized once per workgroup and reused by all BM rows;
//   * activations: never touch LDS.  A small pre-pass re-tiles x into MFMA operand
//     order (one 1 KiB block per 16 rows x 32 k, lane l's 16 bytes at l * 16), so
//     that a wavefront fetches an operand with one fully contiguous 128-bit load
//     per lane straight from global memory / L2 into a 4-deep register ring, 3 K
//     steps of 32 ahead of its use.  (Read from the row-major matrix, the 64 lanes
//     of an operand hit 64 different 16-byte pieces of 16 rows and the texture
//     addresser becomes the bottleneck.)  The re-tiled copy lives in a caller-
//     provided workspace of roundup(M, 16) * K * 2 bytes.
// The dequantization is cut into small pieces that are placed behind individual
// MFMAs, so the vector ALU works in the shadow of the matrix pipe.  One barrier
// per 64-wide K step.  The weights are the MFMA A operand, so a lane ends up with
// 4 consecutive output columns of one row and stores them as 8 bytes.
#include "qlinear_common.hpp"
#include "scratch.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

struct GemmArgs {
  const void* x;              // activations re-tiled into MFMA operand order (the workspace)
  const void* w;
  const void* scale;
  const void* zp;
  void* out;
  int M, N, K;
  int tiles_m, tiles_n;
};

// MFMA with the accumulator pinned to the AGPR half of the register file and
// updated in place.  Left to the register allocator, the 224-256 accumulator
// registers of a 128 x 128 wave tile get split and copied around the loop; the
// constraint keeps them where they are.  The operands of every call come from
// LDS / global loads (never from a vector-ALU result), and results are only read
// after the explicit wait at the end of the K loop.
template <class Act>
__device__ __forceinline__ void mfma_agpr(f32x4& acc, u32x4 a, u32x4 b) {
  if constexpr (Act::dt == DT_F16)
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  else
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

constexpr int kBK = 64;
constexpr int kPitch = kBK + 8;                      // elements per LDS row (144 bytes)

template <class Act, int BM, int BN>
__global__ __launch_bounds__(256) void gemm_w4a16_kernel(const GemmArgs p) {
  using Elem = typename Act::elem;
  constexpr int WM = BM / 2, WN = BN / 2;             // wave sub-tile
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int B_CH = (BN * 2 + 255) / 256;          // 16-byte chunks (32 nibbles) of the w tile per thread
  constexpr int BNP = B_CH * 128;                     // LDS rows of the weight tile (>= BN)
  static_assert(WM % 16 == 0 && WN % 16 == 0, "tile shape");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  Elem* Bs = reinterpret_cast<Elem*>(smem);                                   // [2][BNP][kPitch]

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
  const int KT = K / kBK;                             // 64-wide steps (even: K % 128 == 0)
  const int Q = K / 32;                               // 32-wide MFMA steps

  const int Mp = (M + 15) & ~15;
  const __amdgpu_buffer_rsrc_t xr = make_rsrc(p.x, (uint32_t)Mp * (uint32_t)K * 2u);
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(p.w, (uint32_t)N * ((uint32_t)K >> 1));
  const __amdgpu_buffer_rsrc_t sr = make_rsrc(p.scale, (uint32_t)N * (uint32_t)Kg * 2u);
  const __amdgpu_buffer_rsrc_t zr = make_rsrc(p.zp, p.zp ? (uint32_t)N * (uint32_t)Kg : 0u);
  const bool has_zp = p.zp != nullptr;

  f32x4 acc[TN][TM];
#pragma unroll
  for (int a = 0; a < TN; ++a)
#pragma unroll
    for (int b = 0; b < TM; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- activations: register ring.  Block (16-row tile t, 32-wide step q) of the
  // re-tiled x sits at (t * Q + q) * 1024; tile and step enter as a scalar offset.
  const uint32_t xlane = (uint32_t)lane * 16u;
  const uint32_t xtile0 = (uint32_t)((m0 + wm0) >> 4);
  const uint32_t xtiles = (uint32_t)(Mp >> 4);
  u32x4 xring[4][TM];
  uint32_t xtoff[TM];                                 // scalar: byte offset of tile b's block row
#pragma unroll
  for (int b = 0; b < TM; ++b) {
    const uint32_t t = xtile0 + b < xtiles ? xtile0 + b : xtiles - 1;     // tiles past M: any valid block
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
    const int row = c >> 1, kc = c & 1;               // 2 chunks of 32 k per row
    const int n = n0 + row;
    const uint32_t dead = (uint32_t)(!(n < N && row < BN)) << 31;
    boff[i] = ((uint32_t)n * ((uint32_t)K >> 1) + (uint32_t)(kc * 16)) | dead;
    soff[i] = ((uint32_t)n * (uint32_t)Kg) | dead;    // in groups; x2 for the fp16 scale
    blds[i] = smem + (row * kPitch + kc * 32) * 2;
  }
  struct StageB {                                     // weight chunks of one 64-wide step, in registers
    u32x4 b[B_CH];
    uint16_t s[B_CH];
    uint8_t z[B_CH];
  };
  // One of the 3 B_CH loads of a stage (idx = 3 i + kind), so that the main loop can
  // issue them one at a time between MFMAs: a wavefront that issues vector-memory
  // instructions back to back stalls ~35 cycles on each.
  auto load_b1 = [&](StageB& st, int kt, int idx) {
    const uint32_t dead = kt < KT ? 0u : 0x80000000u;
    const uint32_t k0 = (uint32_t)kt * kBK;
    const int i = idx / 3, kind = idx % 3;
    if (kind == 0)
      st.b[i] = __builtin_amdgcn_raw_buffer_load_b128(wr, boff[i] | dead, k0 >> 1, 0);
    else if (kind == 1)
      st.s[i] = __builtin_amdgcn_raw_buffer_load_b16(sr, ((soff[i] & 0x7fffffffu) * 2u) | (soff[i] & 0x80000000u) | dead,
                                                     (k0 >> 7) * 2u, 0);
    else          // without zero-points the resource is empty and the load returns 0
      st.z[i] = __builtin_amdgcn_raw_buffer_load_b8(zr, soff[i] | dead, k0 >> 7, 0);
  };
  auto load_b = [&](StageB& st, int kt) {
#pragma unroll
    for (int idx = 0; idx < 3 * B_CH; ++idx) load_b1(st, kt, idx);
  };

  // Dequantization of one stage in kPieces pieces of at most 4 vector-ALU
  // instructions (8 pieces per packed dword of 8 nibbles).
  //   fp16: d = (0x6400 | nib) - (1024 + z) exactly, one packed multiply rounds d * s once.
  //   bf16: a nibble 0..15 read as an E4M3 code is nib * 2^-9 (codes below 16 are the
  //         subnormals and the first binade, same spacing), so one v_cvt_pk_f32_fp8
  //         turns two nibbles into floats; fma(nib * 2^-9, 512 s, -z s) in fp32 is exact
  //         ((nib - z) * s has at most 16 significant bits), then one RNE to bf16.
  // Both give the same value as rne((nib - z) * s); only the sign of a zero can
  // differ from the subtract-then-multiply form, which no product notices.
  constexpr int kPieces = B_CH * 4 * 8;
  struct DqState {
    uint32_t e, o;
    f32x2 fe, fo;
    u32x4 outv;
    float sf[B_CH], nzs[B_CH];                        // bf16: 512 * scale and -z * scale (exact)
    f16x2 sv[B_CH], zv[B_CH];                         // fp16: packed scale and 1024 + z
  };
  auto dq_begin = [&](const StageB& st, DqState& q) {
#pragma unroll
    for (int i = 0; i < B_CH; ++i) {
      const _Float16 sc = __builtin_bit_cast(_Float16, st.s[i]);
      const float z = has_zp ? (float)st.z[i] : 8.0f;
      if constexpr (Act::dt == DT_F16) {
        const _Float16 z1024 = (_Float16)(1024.0f + z);
        q.sv[i] = f16x2{sc, sc};
        q.zv[i] = f16x2{z1024, z1024};
      } else {
        q.sf[i] = (float)sc * 512.0f;
        q.nzs[i] = -z * (float)sc;
      }
    }
  };
  constexpr size_t kBufBytes = (size_t)BNP * kPitch * 2;
  auto dq_piece = [&](const StageB& st, int buf, int I, DqState& q) {
    const int dword = I >> 3, part = I & 7;
    const int i = dword / 4, dw = dword % 4;
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    auto bf_pair = [&](float a, float b) {
      const bf16x2_t r = {(__bf16)__builtin_fmaf(a, q.sf[i], q.nzs[i]), (__bf16)__builtin_fmaf(b, q.sf[i], q.nzs[i])};
      return __builtin_bit_cast(uint32_t, r);
    };
    auto f16_pair = [&](int pp) {
      const uint32_t sel = 0x0C000C00u | ((4u + pp) << 16) | (uint32_t)pp;
      const uint32_t bits = __builtin_amdgcn_perm(q.o, q.e, sel) | 0x64006400u;
      return __builtin_bit_cast(uint32_t, (__builtin_bit_cast(f16x2, bits) - q.zv[i]) * q.sv[i]);
    };
    if (part == 0) {
      const uint32_t w = st.b[i][dw];
      q.e = w & 0x0F0F0F0Fu;
      q.o = (w >> 4) & 0x0F0F0F0Fu;
    } else if (part == 7) {
      *reinterpret_cast<u32x4*>(blds[i] + buf * kBufBytes + dw * 16) = q.outv;
    } else if constexpr (Act::dt == DT_F16) {
      if (part <= 4) q.outv[part - 1] = f16_pair(part - 1);
    } else {
      if (part == 1) {
        q.fe = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.e, false);
        q.fo = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.o, false);
      } else if (part == 4) {
        q.fe = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.e, true);
        q.fo = __builtin_amdgcn_cvt_pk_f32_fp8((int)q.o, true);
      } else if (part == 2) q.outv[0] = bf_pair(q.fe[0], q.fo[0]);
      else if (part == 3) q.outv[1] = bf_pair(q.fe[1], q.fo[1]);
      else if (part == 5) q.outv[2] = bf_pair(q.fe[0], q.fo[0]);
      else q.outv[3] = bf_pair(q.fe[1], q.fo[1]);
    }
  };

  // One 64-wide K step: multiply out of LDS buffer `buf` (two 32-wide MFMA steps,
  // ring slots slot0 and slot0 + 1) while the next step's weights (`cur`, loaded one
  // step earlier) are dequantized into the other buffer and the weights two steps
  // ahead are fetched into `nxt`.
  constexpr int kMfmas = 2 * TN * TM;
  // pieces are spread evenly over the MFMAs of the step: piece I goes behind the
  // first MFMA slot with (slot + 1) * kPieces / kMfmas > I
  auto step64 = [&](int kt, int buf, int slot0, StageB& cur, StageB& nxt) {
    const Elem* Bb = Bs + buf * BNP * kPitch;
    DqState q;
    dq_begin(cur, q);
    auto rd_w = [&](int a, int s) {
      return *reinterpret_cast<const u32x4*>(Bb + (wn0 + a * 16 + j) * kPitch + s * 32 + g * 8);
    };
    // the weight operand of row a + 1 is fetched from LDS while row a is multiplied
    u32x4 wnext = rd_w(0, 0);
    constexpr int kHalf = TN * TM;                    // MFMAs per 32-wide step
    constexpr int kXEvery = kHalf / TM;               // one activation load per kXEvery MFMAs
    constexpr int kBEvery = kHalf / (3 * B_CH) > 0 ? kHalf / (3 * B_CH) : 1;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
      for (int a = 0; a < TN; ++a) {
        const u32x4 wcur = wnext;
        if (a + 1 < TN) wnext = rd_w(a + 1, s);
        else if (s == 0) wnext = rd_w(0, 1);
#pragma unroll
        for (int b = 0; b < TM; ++b) {
          mfma_agpr<Act>(acc[a][b], wcur, xring[slot0 + s][b]);
          const int m = a * TM + b;                   // MFMA index inside this 32-wide step
          const int slot = s * kHalf + m;
          const int p0 = slot * kPieces / kMfmas, p1 = (slot + 1) * kPieces / kMfmas;
#pragma unroll
          for (int I = p0; I < p1; ++I) dq_piece(cur, buf ^ 1, I, q);
          // global loads, one at a time: the ring slot multiplied in the previous
          // 32-wide step is refilled 3 steps ahead, and in the first half the weight
          // chunks two 64-wide steps ahead are fetched
          if (m % kXEvery == kXEvery / 2 && m / kXEvery < TM)
            load_x1((slot0 + s + 3) & 3, m / kXEvery, 2 * kt + s + 3);
          if (s == 0 && m % kBEvery == 0 && m / kBEvery < 3 * B_CH) load_b1(nxt, kt + 2, m / kBEvery);
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
    dq_begin(s0, q);
#pragma unroll
    for (int I = 0; I < kPieces; ++I) dq_piece(s0, 0, I, q);
  }
  __syncthreads();
  for (int kt = 0; kt < KT; kt += 2) {
    step64(kt, 0, 0, s1, s0);
    step64(kt + 1, 1, 2, s0, s1);
  }

  // the last MFMAs are still in the matrix pipe: wait before reading their results
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
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

// Re-tile x [M, K] (16-bit, row-major) into MFMA operand order: block (t, q) holds
// rows 16 t .. 16 t + 15, k = 32 q .. 32 q + 31; lane l = 16 g + j of the block
// (16 bytes at l * 16) holds row 16 t + j, k = 32 q + 8 g .. + 7.  Rows past M are
// zero.  One workgroup writes four blocks, contiguously.
__global__ __launch_bounds__(256) void pack_x_kernel(const uint16_t* __restrict__ x, u32x4* __restrict__ xp,
                                                     int M, int K, int Q) {
  const int l = threadIdx.x & 63;
  const int q = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int t = blockIdx.y;
  if (q >= Q) return;
  const int m = t * 16 + (l & 15);
  u32x4 v = {0u, 0u, 0u, 0u};
  if (m < M) v = *reinterpret_cast<const u32x4*>(x + (size_t)m * K + q * 32 + (l >> 4) * 8);
  xp[((size_t)t * Q + q) * 64 + l] = v;
}

template <class Act, int BM, int BN>
static int launch_gemm(GemmArgs p, hipStream_t st) {
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const size_t lds = (size_t)2 * (((BN * 2 + 255) / 256) * 128) * kPitch * 2;
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

}  // namespace qlin

using namespace qlin;

extern "C" {

int mi_gemm_int4_workspace(int M, int N, int K, long long* bytes) {
  if (!bytes) return MI_ERR_ARG;
  if (M < 0 || N < 0 || K <= 0 || (K % 128)) return MI_ERR_SHAPE;
  *bytes = (M <= 64 || !N) ? 0 : (long long)((M + 15) & ~15) * K * 2;
  return MI_OK;
}

int mi_gemm_int4_ws(const void* x, const void* w, const void* scale, const void* zp, void* out,
                    void* workspace, long long workspace_bytes, int M, int N, int K, int act_dtype,
                    void* stream) {
  if (!x || !w || !scale || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (M < 0 || N < 0 || K <= 0 || (K % 128)) return MI_ERR_SHAPE;
  if ((uint64_t)(M + 15) * (uint64_t)K * 2 >= (1ull << 31) || (uint64_t)N * (uint64_t)K / 2 >= (1ull << 31))
    return MI_ERR_SHAPE;
  if (!M || !N) return MI_OK;
  if (M <= 64) return mi_gemv_int4(x, w, scale, zp, out, M, N, K, act_dtype, stream);
  const int Mp = (M + 15) & ~15;
  if (!workspace || workspace_bytes < (long long)Mp * K * 2) return MI_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  const int Q = K / 32;
  hipLaunchKernelGGL(pack_x_kernel, dim3((Q + 3) / 4, Mp / 16), dim3(256), 0, st, (const uint16_t*)x,
                     (u32x4*)workspace, M, K, Q);
  GemmArgs p{};
  p.x = workspace; p.w = w; p.scale = scale; p.zp = zp; p.out = out; p.M = M; p.N = N; p.K = K;
  const bool big = (long)M * N >= (long)256 * 256 * 256;       // enough 256-row tiles to fill the chip
  if (!big)
    return act_dtype == DT_F16 ? launch_gemm<ActF16, 128, 128>(p, st) : launch_gemm<ActBF16, 128, 128>(p, st);
  // 256 x 256 or 256 x 224 tiles: whichever leaves the last round of workgroups fuller
  const long cus = device_cu_count_gemm();
  const long tiles_m = (M + 255) / 256;
  auto cost = [&](long bn) { return ((tiles_m * ((N + bn - 1) / bn) + cus - 1) / cus) * bn; };
  const bool narrow = cost(224) < cost(256);
  if (act_dtype == DT_F16)
    return narrow ? launch_gemm<ActF16, 256, 224>(p, st) : launch_gemm<ActF16, 256, 256>(p, st);
  return narrow ? launch_gemm<ActBF16, 256, 224>(p, st) : launch_gemm<ActBF16, 256, 256>(p, st);
}

int mi_gemm_int4(const void* x, const void* w, const void* scale, const void* zp, void* out, int M, int N,
                 int K, int act_dtype, void* stream) {
  long long bytes = 0;
  const int rc = mi_gemm_int4_workspace(M, N, K, &bytes);
  if (rc != MI_OK) return rc;
  if (!bytes) return mi_gemm_int4_ws(x, w, scale, zp, out, nullptr, 0, M, N, K, act_dtype, stream);
  // scratch for the re-tiled activations: this stream's grow-only buffer (the first
  // call of a size allocates; callers that must never allocate pass their own
  // workspace through mi_gemm_int4_ws)
  void* ws = scratch_get((hipStream_t)stream, (size_t)bytes);
  if (!ws) return MI_ERR_LAUNCH;
  return mi_gemm_int4_ws(x, w, scale, zp, out, ws, bytes, M, N, K, act_dtype, stream);
}

}  // extern "C"
