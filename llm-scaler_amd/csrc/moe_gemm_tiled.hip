// Grouped (per-expert) FP8 weight GEMM for MoE prefill: experts with hundreds of rows.
//
// The weight-streaming grouped kernel (moe_gemm.hip) is built for a few dozen rows per expert;
// with hundreds it is bound by LDS traffic, not by the matrix cores.  Here the expert-sorted rows
// run through the tiled matrix-core GEMM of gemm_tiled.hpp instead (w8a16: fp16 / bf16
// activations, FP8 weights with 128x128 block scales or one scale per expert):
//   1. one small workgroup turns expert_start into a table of M-tiles (expert, first row, rows)
//      and of 16-row activation blocks, every expert padded to whole blocks;
//   2. the activations are gathered (row_map) and re-tiled into MFMA operand order per block;
//   3. the GEMM runs one workgroup per (M-tile, N-tile); the grid is the host-side upper bound
//      of the tile count and surplus workgroups exit at once.
// Optional fused epilogue act(gate) * up (SiLU or tanh-GELU), output row map and per-row factor
// as in the weight-streaming kernel.  The expert MLP as one call (gate_up, act(gate) * up, down)
// shares steps 1 and 2 between its two GEMMs: the first writes its result straight into the
// operand order the second reads, so the intermediate is never re-tiled (nor stored row-major).
#include "gemm_tiled.hpp"
#include "scratch.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

template <class Act, int BN> using WFp8PlainG = WFp8<Act, BN, false>;
template <class Act, int BN> using WFp8BlockG = WFp8<Act, BN, true>;

constexpr int kMapThreads = 1024;

// exclusive scans of two values per thread over the workgroup (whole wavefronts): inside a wavefront by
// shuffles, across the wavefronts through their totals
__device__ __forceinline__ void map_scan2(int& a, int& b, int (*wsum)[2], int tid, int& total_a, int& total_b) {
  const int lane = tid & 63, w = tid >> 6, nw = blockDim.x >> 6;
  int ia = a, ib = b;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int ta = __shfl_up(ia, off), tb = __shfl_up(ib, off);
    if (lane >= off) { ia += ta; ib += tb; }
  }
  if (lane == 63) { wsum[w][0] = ia; wsum[w][1] = ib; }
  __syncthreads();
  int ba = 0, bb = 0;
  total_a = 0; total_b = 0;
  for (int i = 0; i < nw; ++i) {
    if (i < w) { ba += wsum[i][0]; bb += wsum[i][1]; }
    total_a += wsum[i][0]; total_b += wsum[i][1];
  }
  a = ba + ia - a;
  b = bb + ib - b;
}

// g_tile[4 i] = {expert, first sorted row, rows, first activation block} per M-tile of `bm` rows;
// blk[2 b] = {first sorted row, rows} per 16-row activation block; counts[0] = M-tiles,
// counts[1] = blocks.  One workgroup, E <= 1024: thread e scans expert e's counts, then all threads
// share the table entries (entry -> expert by bisection of the scanned offsets).
__global__ __launch_bounds__(kMapThreads) void moe_tile_map_kernel(const int32_t* __restrict__ start, int E, int bm,
                                                                   int32_t* __restrict__ g_tile,
                                                                   int32_t* __restrict__ blk,
                                                                   int32_t* __restrict__ counts) {
  __shared__ int wsum[kMapThreads / 64][2];
  __shared__ int s_boff[kMapThreads + 1], s_toff[kMapThreads + 1], s_r0[kMapThreads], s_cnt[kMapThreads];
  const int e = threadIdx.x;
  const int r0 = e < E ? start[e] : 0;
  const int cnt = e < E ? max(start[e + 1] - r0, 0) : 0;
  int boff = (cnt + 15) >> 4, toff = (cnt + bm - 1) / bm, blocks, tiles;
  map_scan2(boff, toff, wsum, e, blocks, tiles);
  s_boff[e] = boff;
  s_toff[e] = toff;
  s_r0[e] = r0;
  s_cnt[e] = cnt;
  __syncthreads();
  // last expert whose first entry is at or before i (experts without rows share their successor's offset)
  auto owner = [&](const int* off, int i) {
    int lo = 0, hi = E - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (off[mid] <= i) lo = mid; else hi = mid - 1;
    }
    return lo;
  };
  for (int i = e; i < tiles; i += kMapThreads) {
    const int x = owner(s_toff, i), k = i - s_toff[x];
    int32_t* t = g_tile + 4 * i;
    t[0] = x;
    t[1] = s_r0[x] + k * bm;
    t[2] = min(bm, s_cnt[x] - k * bm);
    t[3] = s_boff[x] + k * (bm >> 4);
  }
  for (int b = e; b < blocks; b += kMapThreads) {
    const int x = owner(s_boff, b), k = b - s_boff[x];
    blk[2 * b] = s_r0[x] + 16 * k;
    blk[2 * b + 1] = min(16, s_cnt[x] - 16 * k);
  }
  if (e == 0) {
    counts[0] = tiles;
    counts[1] = blocks;
  }
}

// Gather + re-tile: block b of the table -> MFMA operand order (see pack_x_kernel); rows past the
// block's count are zero.  One workgroup re-tiles 16 consecutive 32-wide steps of one block: each
// wavefront reads 1 KiB of each of four (gathered) rows, the rows meet in an LDS tile and leave
// as 16 contiguous blocks.
__global__ __launch_bounds__(256) void pack_x_grouped_kernel(const uint16_t* __restrict__ x,
                                                             const int32_t* __restrict__ row_map,
                                                             const int32_t* __restrict__ blk,
                                                             const int32_t* __restrict__ counts,
                                                             u32x4* __restrict__ xp, int a_rows, int K, int Q,
                                                             int row_div) {
  __shared__ __attribute__((aligned(16))) unsigned char tile[16 * kPackPitch];
  const int nq = (Q + kPackQ - 1) / kPackQ;           // flat grid: kPackQ steps of one block per workgroup
  const int b = blockIdx.x / nq;
  if (b >= counts[1]) return;
  const int l = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int q0 = (blockIdx.x - b * nq) * kPackQ;
  const int live = blk[2 * b + 1], first = blk[2 * b];
  // Unconditional loads with indices held in range, the surplus zeroed afterwards: a branch around
  // each (map entry, row piece) pair would make the four pairs eight dependent round trips.
  u32x4 v[4];
  unsigned row[4];
  const int k = q0 * 32 + l * 8;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = wave * 4 + i;
    const int pos = first + (r < live ? r : 0);
    row[i] = row_map ? (unsigned)row_map[pos] : (unsigned)pos;
  }
  if (row_map && row_div != 1) {                      // after all four entries have been requested
#pragma unroll
    for (int i = 0; i < 4; ++i) row[i] /= (unsigned)row_div;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bool ok = wave * 4 + i < live && k < K && row[i] < (unsigned)a_rows;
    v[i] = *reinterpret_cast<const u32x4*>(x + (ok ? (size_t)row[i] * K + k : (size_t)0));
    if (!ok) v[i] = u32x4{0u, 0u, 0u, 0u};
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(tile + (wave * 4 + i) * kPackPitch + l * 16) = v[i];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = q0 + wave * 4 + i;
    if (q < Q)
      xp[((size_t)b * Q + q) * 64 + l] =
          *reinterpret_cast<const u32x4*>(tile + (l & 15) * kPackPitch + (wave * 4 + i) * 64 + (l >> 4) * 16);
  }
}

struct TiledMoeLayout {
  long long x_bytes, tile_off, blk_off, cnt_off, total;
  int max_blocks, max_tiles;
};
static inline TiledMoeLayout tiled_moe_layout(int total_rows, int E, int K, int bm) {
  TiledMoeLayout L;
  L.max_blocks = total_rows / 16 + E;
  L.max_tiles = total_rows / bm + E;
  L.x_bytes = (long long)L.max_blocks * 16 * K * 2;
  L.tile_off = (L.x_bytes + 255) & ~255LL;
  L.blk_off = L.tile_off + (((long long)L.max_tiles * 16 + 255) & ~255LL);
  L.cnt_off = L.blk_off + (((long long)L.max_blocks * 8 + 255) & ~255LL);
  L.total = L.cnt_off + 256;
  return L;
}
// Rows per M-tile.  A wavefront skips the 16-row tiles past an expert's last row, so the large tile
// (each weight dequantized once per 256 rows) also serves experts with fewer rows.
constexpr int kMoeBM = 256;

template <class Act, template <class, int> class FMT, bool FUSE>
static int launch_grouped(GemmArgs p, int max_tiles, hipStream_t st) {
  constexpr int BN = 256;
  p.tiles_m = (max_tiles + 7) / 8 * 8;                // whole rounds of the 8 XCDs (surplus workgroups exit)
  p.tiles_n = FUSE ? (p.n_half + BN / 2 - 1) / (BN / 2) : (p.N + BN - 1) / BN;
  using F = FMT<Act, BN>;
  auto kern = gemm_tiled_kernel<Act, F, kMoeBM, BN, true, FUSE>;
  const size_t lds = (size_t)2 * (F::B_CH * 256 / F::CPR) * kPitch * 2;
  static bool raised = false;
  if (lds > 64 * 1024 && !raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) !=
        hipSuccess)
      return MI_ERR_LAUNCH;
    raised = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(256), lds, st, p);
  return launch_status();
}

template <class Act>
static int run_grouped(const GemmArgs& p, bool per_expert, int fuse, int max_tiles, hipStream_t st) {
  if (per_expert)
    return fuse ? launch_grouped<Act, WFp8PlainG, true>(p, max_tiles, st)
                : launch_grouped<Act, WFp8PlainG, false>(p, max_tiles, st);
  return fuse ? launch_grouped<Act, WFp8BlockG, true>(p, max_tiles, st)
              : launch_grouped<Act, WFp8BlockG, false>(p, max_tiles, st);
}

}  // namespace qlin

using namespace qlin;

extern "C" {
int mi_moe_gemm_fp8_tiled_workspace(int total_rows, int E, int K, long long* bytes) {
  if (!bytes) return MI_ERR_ARG;
  if (total_rows < 0 || E < 0 || E > kMapThreads || K <= 0) return MI_ERR_SHAPE;
  const TiledMoeLayout L = tiled_moe_layout(total_rows, E, K, kMoeBM);
  *bytes = L.total;
  // the re-tiled activations are addressed through a 32-bit buffer resource: beyond 2 GiB the tiled
  // route does not apply and the caller stays on the streaming grouped kernel
  if ((uint64_t)L.x_bytes >= (1ull << 31)) return MI_ERR_SHAPE;
  return MI_OK;
}

int mi_moe_gemm_fp8_tiled_ws(const void* a, const int32_t* row_map, int row_map_div, const void* w, const float* w_scale,
                             int scale_per_expert, const int32_t* expert_start, void* out, const int32_t* out_map,
                             const void* row_weight, int a_rows, int total_rows, int E, int N, int K, int fuse_act,
                             int act_dtype, void* workspace, long long workspace_bytes, void* stream) {
  if (!a || !w || !w_scale || !expert_start || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (fuse_act < 0 || fuse_act > 2 || scale_per_expert < 0 || scale_per_expert > 2 || row_map_div < 1) return MI_ERR_ARG;
  if (scale_per_expert == 2 && (N % 2)) return MI_ERR_SHAPE;
  if (E < 0 || E > kMapThreads || N <= 0 || K <= 0 || (K % 128) || a_rows < 0 || total_rows < 0) return MI_ERR_SHAPE;
  if (fuse_act && (N % 2)) return MI_ERR_SHAPE;
  if ((uint64_t)N * (uint64_t)K >= (1ull << 31)) return MI_ERR_SHAPE;
  if (!E || !total_rows) return MI_OK;
  const int bm = kMoeBM;
  const TiledMoeLayout L = tiled_moe_layout(total_rows, E, K, bm);
  if ((uint64_t)L.x_bytes >= (1ull << 31)) return MI_ERR_SHAPE;
  if (!workspace || workspace_bytes < L.total) return MI_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  int32_t* g_tile = (int32_t*)(ws + L.tile_off);
  int32_t* blk = (int32_t*)(ws + L.blk_off);
  int32_t* counts = (int32_t*)(ws + L.cnt_off);
  hipLaunchKernelGGL(moe_tile_map_kernel, dim3(1), dim3(kMapThreads), 0, st, expert_start, E, bm, g_tile, blk, counts);
  const int Q = K / 32;
  hipLaunchKernelGGL(pack_x_grouped_kernel, dim3((unsigned)(((Q + kPackQ - 1) / kPackQ) * L.max_blocks)), dim3(256), 0, st, (const uint16_t*)a,
                     row_map, blk, counts, (u32x4*)ws, a_rows, K, Q, row_map_div);
  GemmArgs p{};
  p.x = ws; p.w = w; p.scale = w_scale; p.out = out; p.M = total_rows; p.N = N; p.K = K;
  p.scale_mode = scale_per_expert == 2 ? 3 : (scale_per_expert ? 1 : 2);
  p.g_tile = g_tile; p.g_count = counts;
  p.g_w_stride = (long long)N * K;
  p.g_s_stride = scale_per_expert ? 4 * scale_per_expert : (long long)((N + 127) / 128) * (K / 128) * 4;
  p.out_map = out_map; p.row_weight = row_weight;
  p.x_blocks = L.max_blocks;
  p.n_half = N / 2; p.gelu = fuse_act == 2;
  p.out_rows = total_rows;
  return act_dtype == DT_F16 ? run_grouped<ActF16>(p, scale_per_expert != 0, fuse_act, L.max_tiles, st)
                             : run_grouped<ActBF16>(p, scale_per_expert != 0, fuse_act, L.max_tiles, st);
}

int mi_moe_mlp_fp8_tiled_workspace(int total_rows, int E, int H, int I, long long* bytes) {
  if (!bytes) return MI_ERR_ARG;
  if (total_rows < 0 || E < 0 || E > kMapThreads || H <= 0 || I <= 0) return MI_ERR_SHAPE;
  const TiledMoeLayout L = tiled_moe_layout(total_rows, E, H, kMoeBM);
  const long long inter = ((long long)L.max_blocks * 16 * I * 2 + 255) & ~255LL;
  *bytes = L.total + inter;
  if ((uint64_t)L.x_bytes >= (1ull << 31) || (uint64_t)inter >= (1ull << 31)) return MI_ERR_SHAPE;
  return MI_OK;
}

int mi_moe_mlp_fp8_tiled_ws(const void* a, const int32_t* row_map, int row_map_div, const void* w13,
                            const float* w13_scale, const void* w2, const float* w2_scale, int scale_per_expert,
                            const int32_t* expert_start, void* out, const int32_t* out_map, const void* row_weight,
                            int a_rows, int total_rows, int E, int H, int I, int fuse_act, int act_dtype,
                            void* workspace, long long workspace_bytes, void* stream) {
  if (!a || !w13 || !w13_scale || !w2 || !w2_scale || !expert_start || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (fuse_act < 1 || fuse_act > 2 || scale_per_expert < 0 || scale_per_expert > 2 || row_map_div < 1) return MI_ERR_ARG;
  if (E < 0 || E > kMapThreads || H <= 0 || I <= 0 || (H % 128) || (I % 128) || a_rows < 0 || total_rows < 0)
    return MI_ERR_SHAPE;
  if ((uint64_t)2 * I * (uint64_t)H >= (1ull << 31)) return MI_ERR_SHAPE;
  if (!E || !total_rows) return MI_OK;
  long long need = 0;
  const int rc = mi_moe_mlp_fp8_tiled_workspace(total_rows, E, H, I, &need);
  if (rc != MI_OK) return rc;
  if (!workspace || workspace_bytes < need) return MI_ERR_ARG;
  const int bm = kMoeBM;
  const TiledMoeLayout L = tiled_moe_layout(total_rows, E, H, bm);
  hipStream_t st = (hipStream_t)stream;
  char* ws = (char*)workspace;
  int32_t* g_tile = (int32_t*)(ws + L.tile_off);
  int32_t* blk = (int32_t*)(ws + L.blk_off);
  int32_t* counts = (int32_t*)(ws + L.cnt_off);
  char* inter = ws + L.total;                          // [blocks][I / 32][1 KiB], operand order
  hipLaunchKernelGGL(moe_tile_map_kernel, dim3(1), dim3(kMapThreads), 0, st, expert_start, E, bm, g_tile, blk, counts);
  const int Q = H / 32;
  hipLaunchKernelGGL(pack_x_grouped_kernel, dim3((unsigned)(((Q + kPackQ - 1) / kPackQ) * L.max_blocks)), dim3(256), 0, st,
                     (const uint16_t*)a, row_map, blk, counts, (u32x4*)ws, a_rows, H, Q, row_map_div);
  GemmArgs p{};
  p.x = ws; p.w = w13; p.scale = w13_scale; p.out = inter; p.M = total_rows; p.N = 2 * I; p.K = H;
  p.scale_mode = scale_per_expert == 2 ? 3 : (scale_per_expert ? 1 : 2);
  p.g_tile = g_tile; p.g_count = counts;
  p.g_w_stride = (long long)2 * I * H;
  p.g_s_stride = scale_per_expert ? 4 * scale_per_expert : (long long)((2 * I + 127) / 128) * (H / 128) * 4;
  p.x_blocks = L.max_blocks;
  p.n_half = I; p.gelu = fuse_act == 2;
  p.out_rows = L.max_blocks * 16; p.out_packed = 1;
  int r = act_dtype == DT_F16 ? run_grouped<ActF16>(p, scale_per_expert != 0, fuse_act, L.max_tiles, st)
                              : run_grouped<ActBF16>(p, scale_per_expert != 0, fuse_act, L.max_tiles, st);
  if (r != MI_OK) return r;
  GemmArgs d{};
  d.x = inter; d.w = w2; d.scale = w2_scale; d.out = out; d.M = total_rows; d.N = H; d.K = I;
  d.scale_mode = scale_per_expert ? 1 : 2;
  d.g_tile = g_tile; d.g_count = counts;
  d.g_w_stride = (long long)H * I;
  d.g_s_stride = scale_per_expert ? 4 : (long long)((H + 127) / 128) * (I / 128) * 4;
  d.out_map = out_map; d.row_weight = row_weight;
  d.x_blocks = L.max_blocks;
  d.n_half = H / 2;
  d.out_rows = total_rows;
  return act_dtype == DT_F16 ? run_grouped<ActF16>(d, scale_per_expert != 0, 0, L.max_tiles, st)
                             : run_grouped<ActBF16>(d, scale_per_expert != 0, 0, L.max_tiles, st);
}

}  // extern "C"
