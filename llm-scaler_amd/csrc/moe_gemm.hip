// Grouped (per-expert) FP8 block-scaled GEMM for MoE, gfx950.
//
// Rows arrive expert-contiguous: expert e owns rows [start[e], start[e+1]) of the
// activation matrix (optionally through a row-gather map).  With top-k routing
// over many experts each expert sees only a few dozen rows, so the op is bound
// by streaming every expert's weights once from HBM, not by the matrix cores:
// one workgroup owns (expert, a few 16-row weight tiles) and all of K and walks
// K in 128-wide granules (= one scale block); its four wavefronts split the
// expert's rows (16 each, up to 64 per pass) and share the weight granule through
// LDS.  Workgroups of experts with no rows exit at once and read nothing.
//
// Two arithmetic modes:
//   A8  : activations pre-quantised to E4M3 per row per 128-k group (scale xs);
//         native v_mfma_f32_16x16x32_fp8_fp8, and the product of the two block
//         scales is applied to each granule's fp32 partial:
//             acc += (A8 . W8)_granule * xs[row, g] * ws[n / 128, g]
//   A16 : fp16 / bf16 activations (w8a16, the reference's mode): weights are
//         converted exactly to 16 bit and ws is applied to the granule partial.
// The weight scale is one value per 128 x 128 block or one per expert.  K may end
// in a partial granule (any multiple of 16): the chunks past K are loaded as zeros
// on both operands.
// Optional fused epilogue: act(gate) * up with act = SiLU or tanh-GELU, where a
// workgroup pairs weight row n (gate) with row n + N/2 (up) and writes N/2 columns.
// Output rows may be scattered through a map (sorted position -> destination row)
// and scaled by a per-destination-row weight.
#include "qlinear_common.hpp"
#include "scratch.hpp"
#include "moe_sort_expert.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

struct MoeGemmArgs {
  const void* a;              // activations: fp8 [rows, K] (A8) or 16-bit [rows, K]
  const float* a_scale;       // A8: [rows, K/128]
  const int32_t* row_map;     // optional: sorted position -> source row of `a` / `a_scale`, times row_div
  int row_div;                // the source row is row_map[position] / row_div (pair index -> token)
  const void* w;              // [E, N, K] e4m3
  const float* w_scale;       // [E, ceil(N/128), ceil(K/128)], or [E]
  const int32_t* start;       // [E+1]
  void* out;                  // [total_rows, N_out]: activation dtype (out_f32 = 0), fp32 (1) or fp16 (2)
  const int32_t* out_map;     // optional: sorted position -> row of `out`
  const void* row_weight;     // optional, activation dtype: factor per row of `out`
  int out_f32;
  int gelu;                   // fused epilogue: tanh-GELU instead of SiLU
  int scale_per_expert;       // 1: w_scale is [E] instead of block scales; 2: [E, 2], first / second half of the N rows
  int E, N, K;                // N = weight rows per expert
  int n_out;                  // output columns (N, or N/2 with the fused SiLU*mul)
  int tiles_per_expert;       // workgroups per expert
  int tpw;                    // tile groups walked by one workgroup
  int a_rows;                 // rows in `a` (bounds the buffer)
  int total_rows;             // rows in `out`
  // SORT kernels: the expert grouping is derived from the routing table inside the launch
  const int32_t* top_ids;     // [P] expert of pair q = token * topk + route
  int32_t* sort_start;        // out [E + 1]
  int32_t* sort_inv;          // out [P]: pair -> expert-sorted position
  int32_t* sort_pairs;        // out [P] or null: expert-sorted position -> pair
  int P, topk, chunk;         // pairs, routes per token, pairs owned by one thread (a multiple of 4)
};

// LDS staging geometry.  Global loads are row-coalesced (8 or 16 consecutive lanes
// read one row's contiguous 128 / 256 bytes of a K granule — loading the MFMA
// operand layout directly, where consecutive lanes hit different rows, halves the
// L1 rate once the activation stream from L2 is added to the weight stream); the
// granule is written to LDS and read back in MFMA layout.  Rows are padded by 16
// bytes so that the 16 lanes of an operand read (row stride 144 / 272 bytes) fall
// into distinct banks.
constexpr int kWPitch = 128 + 16;                    // fp8 weight / activation row of one granule
constexpr long kRoutedMaxPairs = 32 * 256;           // pairs a routed (SORT) launch takes: 32 per thread
constexpr int kA16Pitch = 256 + 16;                  // 16-bit activation row of one granule

// Workgroup = 4 wavefronts.  The workgroup owns RT 16-row weight tiles of one
// expert (per tile group; it walks `tpw` consecutive tile groups) and up to 64 of
// the expert's rows per pass; wavefront w owns activation tile w (rows 16 w ..)
// against ALL of the workgroup's weight tiles, so
//   * a weight granule is fetched once per workgroup, cooperatively (each thread
//     RT/2 16-byte chunks), into a double-buffered shared LDS tile,
//   * every wavefront stages only its own 16 activation rows (private LDS),
//   * outputs of different wavefronts are disjoint: no cross-wave reduction.
// Wavefronts whose tile has no rows still fetch weights and join the barriers.
// D granules are in flight in registers per thread; the loop over (tile group,
// granule) is flattened so the prefetch runs across tile-group boundaries.
// The weights are the MFMA A operand and the activations the B operand, so a lane
// ends up holding ONE activation row (16 w + j) and four consecutive weight rows
// (4 g + v): the per-row activation scale is a single value per lane and granule.
// MT = 16-row activation tiles per wavefront and pass.  Only MT = 1 (up to 64 rows per pass) is
// launched: with 4 the kernel is bound by its LDS traffic and gained nothing for experts with
// hundreds of rows, which run on the tiled matrix-core GEMM instead (moe_gemm_tiled.hip).
// SORT: the launch takes the routing table (expert per (token, route) pair) instead of expert-sorted
// rows.  Every workgroup of expert e finds the expert's pairs itself -- it reads all P ids, the number
// of pairs of lower experts is the expert's first sorted position and a pair's rank is the number of
// earlier pairs of the same expert: the stable counting sort of mi_moe_sort, one round trip to memory,
// overlapped with the resident workgroups that already stream -- gathers its rows by token = pair / topk,
// and the expert's first workgroup writes expert_start / inv / sorted_pairs for the later stages.
template <class Act, bool A8, bool SILU, int RT, int D, bool PE, int MT = 1, bool SORT = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(A8 ? 3 : 2))) void moe_gemm_kernel(const MoeGemmArgs p, const float* __restrict__ w_scale,
                                                        const int32_t* __restrict__ expert_start) {
  static_assert(RT == 2 || RT == 4 || RT == 8, "two, four or eight weight tiles");
  using Elem = typename Act::elem;
  using V8 = typename Act::v8;
  constexpr int WL = RT / 2;                          // weight chunks per thread per granule
  constexpr int NAI = A8 ? 2 : 4;                     // activation chunks per lane per granule
  constexpr int APitch = A8 ? kWPitch : kA16Pitch;
  constexpr uint32_t AGran = A8 ? 128u : 256u;        // activation bytes per row per granule
  constexpr int kWBuf = RT * 16 * kWPitch;
  constexpr int kCols = SILU ? (RT / 2) * 16 : RT * 16;   // output columns per tile group
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];   // 2 * kWBuf + 4 * MT * 16 * APitch

  // The 8 XCDs take workgroups round-robin and each has its own L2: all workgroups of an expert
  // go to XCD (expert % 8), so that the expert's activation rows are fetched into one L2 only.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int e = (slot / p.tiles_per_expert) * 8 + xcd;
  const int wg = slot % p.tiles_per_expert;
  if (e >= p.E) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int r0 = 0, cnt = 0;

  const int j = lane & 15, g = lane >> 4;
  const int K = p.K, N = p.N;
  const int G = (K + 127) >> 7, Kb = G;
  const int ktail = K - ((G - 1) << 7);               // k extent of the last granule (128 = whole)
  const int half = N >> 1;
  const int limit = SILU ? half : N;                  // columns
  const int groups = (limit + kCols - 1) / kCols;     // tile groups per expert
  const int tg0 = wg * p.tpw;
  const int ntg = min(p.tpw, groups - tg0);           // tile groups of this workgroup
  const int col0 = tg0 * kCols;

  // column offset of weight tile t inside a tile group, and its gate/up half
  auto tile_col = [&](int t) { return SILU ? (t >> 1) * 16 : t * 16; };
  auto tile_hi = [&](int t) { return SILU ? (t & 1) * half : 0; };

  // Cooperative weight staging: thread `tid` fetches chunk (tid & 7) of row (tid >> 3) + 32 i of the
  // tile group's RT * 16 rows, i < WL.  32 rows further on is two weight tiles further on, which is
  // the same step in memory for every i (32 rows of the matrix, or 16 rows of the gate and of the up
  // half alike), so one offset register serves all of a thread's chunks and the rest is uniform.
  // Columns at or past `limit` are masked per load (the uniform part of the address travels in the
  // scalar offset, which the buffer bound does not see).
  const int wrow = tid >> 3, wt = wrow >> 4;
  const int wcol = col0 + tile_col(wt) + (wrow & 15);  // output column of chunk 0 in tile group 0
  const int wch = (tid & 7) * 16;                     // first k of the chunk inside the granule
  const uint32_t wvoff = (uint32_t)(tile_hi(wt) + col0 + tile_col(wt) + (wrow & 15)) * (uint32_t)K + (uint32_t)wch;
  const uint32_t wistep = (SILU ? 16u : 32u) * (uint32_t)K;
  unsigned char* const wlds = smem + wrow * kWPitch + wch;
  constexpr int kWldsStep = 32 * kWPitch;
  unsigned char* al = smem + 2 * kWBuf + wave * MT * 16 * APitch;

  const uint8_t* wexp = (const uint8_t*)p.w + (size_t)e * N * K;
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(wexp, (uint32_t)N * (uint32_t)K);
  const uint32_t a_esz = A8 ? 1u : 2u;
  const __amdgpu_buffer_rsrc_t ar = make_rsrc(p.a, (uint32_t)p.a_rows * (uint32_t)K * a_esz);
  const __amdgpu_buffer_rsrc_t xsr = make_rsrc(p.a_scale, A8 ? (uint32_t)p.a_rows * (uint32_t)Kb * 4u : 0u);
  const int Nb = (N + 127) >> 7;
  // read through a restrict kernel argument so the (uniform) scale loads stay on the
  // scalar unit and do not queue behind the vector prefetch
  // PE: one scale per expert (or one per half of its rows: gate / up), read once; otherwise the
  // block scales of this expert
  const bool pe_pair = PE && p.scale_per_expert == 2;
  const float* __restrict__ wsc = PE ? w_scale + (pe_pair ? 2 * e : e) : w_scale + (size_t)e * Nb * Kb;
  const float ws_expert = PE ? wsc[0] : 1.0f;
  const float ws_second = pe_pair ? wsc[1] : ws_expert;
  const uint32_t tg_stride = (uint32_t)kCols * (uint32_t)K;   // weight bytes between tile groups

  struct Regs {                                       // one granule in flight
    u32x4 w[WL];
    u32x4 a[MT][NAI];
    float xs[MT];
  };
  constexpr int kPassRows = 64 * MT;                  // rows of the expert per pass over its weights

  // weight loads of granule gi of tile group tg (dead beyond the last one)
  auto load_weights = [&](Regs& r, int tg, int gi) {
    const uint32_t dead = tg < ntg ? 0u : 0x80000000u;
    const uint32_t wso = (uint32_t)tg * tg_stride + (uint32_t)gi * 128u;
    // quantised activations come in whole 128-groups: no partial granule there
    const int kext = (!A8 && gi == G - 1) ? ktail : 128;   // uniform
    const uint32_t wv = wvoff | dead | ((uint32_t)(wch >= kext) << 31);
    const int wc = wcol + tg * kCols;
#pragma unroll
    for (int i = 0; i < WL; ++i)
      r.w[i] = __builtin_amdgcn_raw_buffer_load_b128(wr, wv | ((uint32_t)(wc + i * 16 * (SILU ? 1 : 2) >= limit) << 31),
                                                     wso + (uint32_t)i * wistep, 2);
  };

  Regs r[D];
  uint32_t smask = 0;                                  // SORT: bit b = pair tid * chunk + b belongs to expert e
  int sbefore = 0;                                     // SORT: rank of this thread's first pair inside the expert
  __shared__ int32_t pass_token[SORT ? 64 * MT : 1];   // SORT: token of each row of the current pass
  // The weights do not depend on the expert's rows: when most experts are in use, the first granules
  // are requested before the workgroup knows its rows, so that its stream already runs while it finds
  // them.  (With few rows per launch most workgroups find none and leave; those request nothing.)
  bool early_w;                                        // the first pass's weight prefetch is already in flight
  u32x4 ids[SORT ? kSortExpertChunkMax / 4 : 1];
  if constexpr (SORT) {
    static_assert(MT == 1, "one activation tile per wavefront");
    expert_ids_load(p.top_ids, p.P, p.chunk, tid, ids);   // ahead of the weights: the sort waits for these only
    early_w = p.P >= 2 * p.E;
  } else {
    early_w = p.total_rows >= 2 * p.E;
  }
  {
    // issued without a branch (a launch that does not prefetch marks the loads dead, and dead loads
    // touch no memory): behind a branch the compiler cannot count the loads in flight and makes the
    // first use of anything loaded earlier wait for all of them
    int etg = early_w ? 0 : ntg, egi = 0;
#pragma unroll
    for (int st = 0; st < D; ++st) {
      load_weights(r[st], etg, egi);
      if (++egi == G) { egi = 0; ++etg; }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if constexpr (SORT) {
    __shared__ int32_t wave_lt[4], wave_eq[4];
    const int E = p.E, q0 = tid * p.chunk;
    int lt, start, count;
    expert_ids_count(ids, p.P, E, e, p.chunk, tid, smask, lt);
    expert_scan<4>(smask, lt, tid, wave_lt, wave_eq, start, count, sbefore);
    r0 = start;
    cnt = count;
    if (wg == 0) {                                     // the expert's first workgroup publishes the grouping
      if (tid == 0) {
        p.sort_start[e] = start;
        if (e == E - 1) p.sort_start[E] = start + count;
      }
      uint32_t m2 = smask;
      int pos = start + sbefore;
      while (m2) {
        const int b = __ffs(m2) - 1;
        m2 &= m2 - 1;
        p.sort_inv[q0 + b] = pos;
        if (p.sort_pairs) p.sort_pairs[pos] = q0 + b;
        ++pos;
      }
    }
  } else {
    r0 = expert_start[e];
    cnt = expert_start[e + 1] - r0;
  }
  if (cnt <= 0) return;

  for (int mc = 0; mc < cnt; mc += kPassRows) {
    const int rows_here = min(kPassRows, cnt - mc);
    const int wrow0 = wave * 16 * MT;                 // first row of this wavefront inside the pass
    if constexpr (SORT) {
      // tokens of the pass's rows, from the threads that own the pairs (the previous pass's readers
      // have passed the barrier that ends a pass)
      uint32_t m2 = smask;
      int rank = sbefore - mc;
      while (m2) {
        const int b = __ffs(m2) - 1;
        m2 &= m2 - 1;
        if (rank >= 0 && rank < kPassRows) pass_token[rank] = (tid * p.chunk + b) / p.topk;
        ++rank;
      }
      __syncthreads();
    }
    // source row (of `a` / `a_scale`) of row m of the expert, m inside this pass
    auto src_row = [&](int m, bool ok) -> uint32_t {
      if constexpr (SORT) return (uint32_t)pass_token[ok ? m - mc : 0];
      const int pos = r0 + (ok ? m : 0);
      return p.row_map ? (uint32_t)p.row_map[pos] / (uint32_t)p.row_div : (uint32_t)pos;
    };
    // source row of this lane's activation row (MFMA layout) and staging slots
    uint32_t xsoff[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mc + wrow0 + mt * 16 + j;
      const bool ok = m < cnt;
      const uint32_t src = src_row(m, ok);
      xsoff[mt] = (src * (uint32_t)Kb * 4u) | ((uint32_t)(!ok) << 31);
    }
    uint32_t aoff[MT][NAI];
    int ach[NAI];
    unsigned char* alds[MT][NAI];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < NAI; ++i) {
        const int row = A8 ? (lane >> 3) + 8 * i : (lane >> 4) + 4 * i;
        const int ch = A8 ? (lane & 7) : (lane & 15);
        const int m = mc + wrow0 + mt * 16 + row;
        const bool ok = m < cnt;
        const uint32_t src = src_row(m, ok);
        aoff[mt][i] = (src * (uint32_t)K * a_esz + (uint32_t)ch * 16u) | ((uint32_t)(!ok) << 31);
        alds[mt][i] = al + (mt * 16 + row) * APitch + ch * 16;
        ach[i] = A8 ? ch * 16 : ch * 8;               // first k of the chunk inside the granule
      }

    // activation loads of granule gi of tile group tg (dead beyond the last one)
    auto load_acts = [&](Regs& r, int tg, int gi) {
      const uint32_t dead = tg < ntg ? 0u : 0x80000000u;
      const int kext = (!A8 && gi == G - 1) ? ktail : 128;   // uniform
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int i = 0; i < NAI; ++i)
          r.a[mt][i] = __builtin_amdgcn_raw_buffer_load_b128(ar, aoff[mt][i] | dead | ((uint32_t)(ach[i] >= kext) << 31),
                                                             (uint32_t)gi * AGran, 0);
        if constexpr (A8)
          r.xs[mt] = __builtin_bit_cast(float,
                                        __builtin_amdgcn_raw_buffer_load_b32(xsr, xsoff[mt] | dead, (uint32_t)gi * 4u, 0));
      }
    };
    auto load_granule = [&](Regs& r, int tg, int gi) {
      load_weights(r, tg, gi);
      load_acts(r, tg, gi);
    };

    // destination row and routing weight of this lane's activation row: fetched once per pass, ahead
    // of the weight stream (a load issued inside the loop would wait for every prefetch before it:
    // the counter of outstanding loads retires in order)
    int dst_row[MT];
    float dst_w[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mc + wrow0 + mt * 16 + j;
      int dst = m < cnt ? (p.out_map ? p.out_map[r0 + m] : r0 + m) : -1;
      if ((unsigned)dst >= (unsigned)p.total_rows) dst = -1;    // a mapped row outside the output is dropped
      dst_row[mt] = dst;
      dst_w[mt] = (p.row_weight && dst >= 0) ? Act::to_f32(((const Elem*)p.row_weight)[dst]) : 1.0f;
    }
    // the same for the row-contiguous store layout of the epilogue: lane l stores 16 bytes of rows
    // (l >> 3) and (l >> 3) + 8 of the wavefront's tile
    int dst_line[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int m = mc + wrow0 + mt * 16 + (lane >> 3) + 8 * h;
        int dst = m < cnt ? (p.out_map ? p.out_map[r0 + m] : r0 + m) : -1;
        if ((unsigned)dst >= (unsigned)p.total_rows) dst = -1;
        dst_line[mt][h] = dst;
      }

    // The (tile group, granule) steps of this workgroup form one linear sequence; D of them are in
    // flight in a register ring.  Steps past the end (the sequence is walked in multiples of D) load
    // nothing and compute nothing.
    const int total = ntg * G;
    int ptg = 0, pgi = 0;                             // position of the next step to fetch
#pragma unroll
    for (int s = 0; s < D; ++s) {
      if (early_w && mc == 0) load_acts(r[s], ptg, pgi);
      else load_granule(r[s], ptg, pgi);
      if (++pgi == G) { pgi = 0; ++ptg; }
      // keep the stages' loads in issue order: the counter of outstanding loads
      // retires in order, and the loop waits for "all but the younger stages"
      __builtin_amdgcn_sched_barrier(0);
    }

    f32x4 acc[MT][RT];
    int tg = 0, gi = 0, par = 0;
    for (int q0 = 0; q0 < total; q0 += D) {
#pragma unroll
      for (int s = 0; s < D; ++s) {
        const bool live = q0 + s < total;             // uniform
        if (gi == 0) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int t = 0; t < RT; ++t) acc[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        // the shared weight tile alternates between two buffers
        unsigned char* wbuf = smem + par * kWBuf;
        // granule -> LDS
#pragma unroll
        for (int i = 0; i < WL; ++i) *reinterpret_cast<u32x4*>(wlds + par * kWBuf + i * kWldsStep) = r[s].w[i];
        // (a wavefront without rows in this pass stages nothing: the LDS write port is the scarcest
        // resource of the step)
        if (wrow0 < rows_here) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < NAI; ++i) *reinterpret_cast<u32x4*>(alds[mt][i]) = r[s].a[mt][i];
        }
        // The activation scale is taken out of the ring slot before the slot is reloaded
        // below.  Left to the scheduler, the multiply sinks under the reload, old and new
        // value overlap, and the loop latch gets a register copy of the NEW value, i.e. a
        // wait for every load in flight on each turn.
        float xs_now[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          xs_now[mt] = A8 ? r[s].xs[mt] : 1.0f;
          asm volatile("" : "+v"(xs_now[mt]));
        }
        float wsv[RT];
#pragma unroll
        for (int t = 0; t < RT; ++t) {
          const int row_t = tile_hi(t) + col0 + tg * kCols + tile_col(t);
          wsv[t] = PE ? (row_t >= half ? ws_second : ws_expert)
                      : wsc[(size_t)min(row_t >> 7, Nb - 1) * Kb + (live ? gi : 0)];
        }
        // prefetch D steps ahead, across the tile-group boundary
        load_granule(r[s], ptg, pgi);
        if (++pgi == G) { pgi = 0; ++ptg; }
        __syncthreads();
        if (live && wrow0 < rows_here) {             // wave-uniform: this wavefront has rows in the pass
          // One weight tile at a time, its fragments read while the previous tile is multiplied: all
          // eight tiles' fragments and partial sums live at once cost 90 registers, which is a
          // workgroup per CU less and with it a third of the bytes in flight.
          auto read_tile = [&](int t, u32x4 (&f)[2]) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
              f[i] = *reinterpret_cast<const u32x4*>(wbuf + (t * 16 + j) * kWPitch + g * 32 + i * 16);
          };
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            if (MT > 1 && wrow0 + mt * 16 >= rows_here) continue;    // wave-uniform
            const unsigned char* am = al + (mt * 16 + j) * APitch;
            u32x4 wf[2][2];
            read_tile(0, wf[0]);
            if constexpr (A8) {
              const u32x4 x0 = *reinterpret_cast<const u32x4*>(am + g * 32);
              const u32x4 x1 = *reinterpret_cast<const u32x4*>(am + g * 32 + 16);
              const long xa = (long)(((uint64_t)x0[1] << 32) | x0[0]);
              const long xb = (long)(((uint64_t)x0[3] << 32) | x0[2]);
              const long xc = (long)(((uint64_t)x1[1] << 32) | x1[0]);
              const long xd = (long)(((uint64_t)x1[3] << 32) | x1[2]);
              // the scaled sum of tile t - 1 follows the matrix instructions of tile t, so that only two
              // tiles' partial sums are live
              f32x4 tt[2];
#pragma unroll
              for (int t = 0; t < RT; ++t) {
                if (t + 1 < RT) read_tile(t + 1, wf[(t + 1) & 1]);
                const u32x4(&f)[2] = wf[t & 1];
                const long w0 = (long)(((uint64_t)f[0][1] << 32) | f[0][0]);
                const long w1 = (long)(((uint64_t)f[0][3] << 32) | f[0][2]);
                const long w2 = (long)(((uint64_t)f[1][1] << 32) | f[1][0]);
                const long w3 = (long)(((uint64_t)f[1][3] << 32) | f[1][2]);
                f32x4 c = f32x4{0.f, 0.f, 0.f, 0.f};
                c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w0, xa, c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w1, xb, c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w2, xc, c, 0, 0, 0);
                c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w3, xd, c, 0, 0, 0);
                tt[t & 1] = c;
                if (t > 0) acc[mt][t - 1] += tt[(t - 1) & 1] * (xs_now[mt] * wsv[t - 1]);
                __builtin_amdgcn_sched_barrier(0);
              }
              acc[mt][RT - 1] += tt[(RT - 1) & 1] * (xs_now[mt] * wsv[RT - 1]);
            } else {
              V8 xf[4];
#pragma unroll
              for (int i = 0; i < 4; ++i) xf[i] = *reinterpret_cast<const V8*>(am + g * 64 + i * 16);
              f32x4 tt[2];
#pragma unroll
              for (int t = 0; t < RT; ++t) {
                if (t + 1 < RT) read_tile(t + 1, wf[(t + 1) & 1]);
                const u32x4(&f)[2] = wf[t & 1];
                f32x4 c = f32x4{0.f, 0.f, 0.f, 0.f};
                c = Act::mfma(fp8x8_to_act<Act>(f[0][0], f[0][1]), xf[0], c);
                c = Act::mfma(fp8x8_to_act<Act>(f[0][2], f[0][3]), xf[1], c);
                c = Act::mfma(fp8x8_to_act<Act>(f[1][0], f[1][1]), xf[2], c);
                c = Act::mfma(fp8x8_to_act<Act>(f[1][2], f[1][3]), xf[3], c);
                tt[t & 1] = c;
                if (t > 0) acc[mt][t - 1] += tt[(t - 1) & 1] * wsv[t - 1];
                __builtin_amdgcn_sched_barrier(0);
              }
              acc[mt][RT - 1] += tt[(RT - 1) & 1] * wsv[RT - 1];
            }
          }
        }

        // ---- epilogue of a tile group: lane holds row 16 w + j, weight rows 4 g + v ----
        if (live && gi == G - 1 && wrow0 < rows_here) {
          constexpr int NO = SILU ? RT / 2 : RT;      // 16-column output tiles of the tile group
          const int ncol0 = col0 + tg * kCols;        // first output column of the tile group
          // four results as 16-bit words: the activation type, or fp16 whatever the activation type
          // (out_f32 = 2; held to the fp16 range, so an overflow is a large number and not an infinity)
          auto to_f16_sat = [](float f) -> _Float16 { return (_Float16)fminf(fmaxf(f, -65504.0f), 65504.0f); };
          auto pack4 = [&](float a0, float a1, float a2, float a3) -> uint64_t {
            if (p.out_f32 == 2) {
              _Float16 h4[4] = {to_f16_sat(a0), to_f16_sat(a1), to_f16_sat(a2), to_f16_sat(a3)};
              return *reinterpret_cast<const uint64_t*>(h4);
            }
            Elem o4[4] = {Act::from_f32(a0), Act::from_f32(a1), Act::from_f32(a2), Act::from_f32(a3)};
            return *reinterpret_cast<const uint64_t*>(o4);
          };
          auto value = [&](int mt, int o, int v, float rw) -> float {
            const int t = SILU ? 2 * o : o;
            if constexpr (SILU) {
              const float gate = acc[mt][t][v], up = acc[mt][t + 1][v];
              if (p.gelu) {
                // 0.5 g (1 + tanh z), tanh through exp(2z) with 2z held in [-30, 30]
                float two_z = 2.0f * (0.7978845608f * (gate + 0.044715f * (gate * gate * gate)));
                two_z = fminf(fmaxf(two_z, -30.0f), 30.0f);
                const float ex = __expf(two_z);
                return 0.5f * gate * (1.0f + (ex - 1.0f) / (ex + 1.0f)) * up * rw;
              }
              return gate / (1.0f + __expf(-gate)) * up * rw;
            } else {
              return acc[mt][t][v] * rw;
            }
          };
          // Whole 128-byte lines: the cost of a store is per cache line it touches, not per byte, and in
          // accumulator layout an instruction puts 32 or 64 bytes into each of 16 rows.  The tile goes
          // through the wavefront's own activation tile in LDS (free until the next step stages into
          // it; a wavefront's LDS operations complete in order, so no barrier) and leaves as 8 rows x
          // 128 contiguous bytes per instruction.  Needs the tile group inside the matrix and rows
          // that start on 16 bytes; anything else takes the element-wise path below.
          const uint32_t esz = p.out_f32 == 1 ? 4u : 2u;
          const bool lines = ncol0 + kCols <= limit && (((uint32_t)p.n_out * esz) & 15u) == 0;
          if (lines) {
            constexpr int kOPitch = 128 + 16;
            static_assert(kOPitch <= APitch, "the output tile is staged in the activation tile");
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              if (MT > 1 && wrow0 + mt * 16 >= rows_here) continue;    // wave-uniform
              unsigned char* ol = al + mt * 16 * APitch;
              const float rw = dst_w[mt];
              if (p.out_f32 == 1) {
                constexpr int TPR = 2;                 // tiles per 128-byte row piece
#pragma unroll
                for (int rd = 0; rd < NO / TPR; ++rd) {
#pragma unroll
                  for (int ot = 0; ot < TPR; ++ot) {
                    const int o = rd * TPR + ot;
                    *reinterpret_cast<f32x4*>(ol + j * kOPitch + (ot * 16 + g * 4) * 4) =
                        f32x4{value(mt, o, 0, rw), value(mt, o, 1, rw), value(mt, o, 2, rw), value(mt, o, 3, rw)};
                  }
#pragma unroll
                  for (int h = 0; h < 2; ++h) {
                    const u32x4 d = *reinterpret_cast<const u32x4*>(ol + ((lane >> 3) + 8 * h) * kOPitch + (lane & 7) * 16);
                    const int dst = dst_line[mt][h];
                    if (dst >= 0) {
                      u32x4* q = reinterpret_cast<u32x4*>((unsigned char*)p.out + ((size_t)dst * p.n_out + ncol0 + rd * 32) * 4 +
                                                (lane & 7) * 16);
                      *q = d;
                    }
                  }
                }
              } else {
                constexpr int TPR = NO < 4 ? NO : 4;
#pragma unroll
                for (int rd = 0; rd < NO / TPR; ++rd) {
#pragma unroll
                  for (int ot = 0; ot < TPR; ++ot) {
                    const int o = rd * TPR + ot;
                    *reinterpret_cast<uint64_t*>(ol + j * kOPitch + (ot * 16 + g * 4) * 2) =
                        pack4(value(mt, o, 0, rw), value(mt, o, 1, rw), value(mt, o, 2, rw), value(mt, o, 3, rw));
                  }
                  constexpr int kChunks = TPR * 2;     // 16-byte chunks per row piece (TPR * 16 columns * 2 bytes)
#pragma unroll
                  for (int h = 0; h < 2; ++h) {
                    const u32x4 d = *reinterpret_cast<const u32x4*>(ol + ((lane >> 3) + 8 * h) * kOPitch + (lane & 7) * 16);
                    const int dst = dst_line[mt][h];
                    if (dst >= 0 && (lane & 7) < kChunks) {
                      u32x4* q = reinterpret_cast<u32x4*>((unsigned char*)p.out + ((size_t)dst * p.n_out + ncol0 + rd * TPR * 16) * 2 +
                                                (lane & 7) * 16);
                      *q = d;
                    }
                  }
                }
              }
            }
          } else {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const int dst = dst_row[mt];
            if (dst >= 0) {
              Elem* out = (Elem*)p.out;
              float* out32 = (float*)p.out;
              const size_t orow = (size_t)dst * p.n_out;
              const float rw = dst_w[mt];
#pragma unroll
              for (int o = 0; o < NO; ++o) {
                const int t = SILU ? 2 * o : o;
                const int n = ncol0 + tile_col(t) + g * 4;   // first of 4 output columns
                float v4[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) v4[v] = value(mt, o, v, rw);
                if (n + 3 < limit && (p.n_out & 3) == 0) {
                  if (p.out_f32 == 1) {
                    *reinterpret_cast<f32x4*>(out32 + orow + n) = f32x4{v4[0], v4[1], v4[2], v4[3]};
                  } else {
                    *reinterpret_cast<uint64_t*>(out + orow + n) = pack4(v4[0], v4[1], v4[2], v4[3]);
                  }
                } else {
#pragma unroll
                  for (int v = 0; v < 4; ++v)
                    if (n + v < limit) {
                      if (p.out_f32 == 1) out32[orow + n + v] = v4[v];
                      else if (p.out_f32 == 2) ((_Float16*)p.out)[orow + n + v] = to_f16_sat(v4[v]);
                      else out[orow + n + v] = Act::from_f32(v4[v]);
                    }
                }
              }
            }
          }
          }
        }
        par ^= 1;
        if (++gi == G) { gi = 0; ++tg; }
      }
    }
    // Nothing is in flight past this point (the last steps' loads are dead ones).  Said explicitly:
    // otherwise the top of the pass loop has to assume the loop's loads pending and waits for the
    // first pass's early weight request before it touches any register they might target.
    __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0)
    __syncthreads();                                  // LDS is rewritten by the next pass
  }
}

template <class K>
static void launch_moe_kernel(K kern, size_t lds, long wgs, const MoeGemmArgs& p, hipStream_t st, bool& raised) {
  if (lds > 64 * 1024 && !raised) {                   // opt in to more than 64 KiB of dynamic LDS, once per kernel
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised = true;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(256), lds, st, p, p.w_scale, p.start);
}

template <class Act, bool A8, bool SILU, int RT, int D, int MT = 1, bool SORT = false>
static int launch_moe(MoeGemmArgs p, int tpw, hipStream_t st) {
  // quantised activations only come with block scales (the per-expert form is the reference's w8a16 mode)
  constexpr bool kHasPE = !A8 && !SORT;
  const int cols = SILU ? p.N / 2 : p.N;
  const int cols_per_group = SILU ? (RT / 2) * 16 : RT * 16;
  const int groups = (cols + cols_per_group - 1) / cols_per_group;
  p.tpw = tpw;
  p.tiles_per_expert = (groups + tpw - 1) / tpw;
  p.n_out = cols;
  const long wgs = (long)((p.E + 7) / 8) * 8 * p.tiles_per_expert;   // whole rounds of the 8 XCDs
  if (wgs <= 0) return MI_OK;
  const size_t lds = (size_t)2 * RT * 16 * kWPitch + (size_t)4 * MT * 16 * (A8 ? kWPitch : kA16Pitch);
  static bool raised_pe = false, raised_block = false; // per instantiation of this function = per kernel
  if constexpr (kHasPE) {
    if (p.scale_per_expert) {
      launch_moe_kernel(moe_gemm_kernel<Act, A8, SILU, RT, D, true, MT>, lds, wgs, p, st, raised_pe);
      return launch_status();
    }
  }
  launch_moe_kernel(moe_gemm_kernel<Act, A8, SILU, RT, D, false, MT, SORT>, lds, wgs, p, st, raised_block);
  return launch_status();
}

template <class Act, bool A8, bool SILU, bool SORT = false>
static int dispatch_moe2(const MoeGemmArgs& p, hipStream_t st) {
  const int G = (p.K + 127) / 128;
  const int cols = SILU ? p.N / 2 : p.N;
  // Wide workgroups (8 weight tiles) re-read the expert's activation rows least
  // often; narrower ones keep the device filled when there are few tiles.
  auto wgs_with = [&](int rt) { return (long)p.E * ((cols + (SILU ? rt / 2 : rt) * 16 - 1) / ((SILU ? rt / 2 : rt) * 16)); };
  const int rt = wgs_with(8) >= 1024 ? 8 : (wgs_with(4) >= 1024 ? 4 : 2);
  // short K: walk two tile groups per workgroup so the prefetch pipeline stays filled
  const int tpw = (G < 16 && wgs_with(rt) >= 2048) ? 2 : 1;
  // two granules in flight per thread (more do not pay: the register ring then costs a resident
  // workgroup); a single granule has nothing to prefetch
  const bool d2 = G >= 2;
  if constexpr (SORT) {
    // the routed launch is instantiated for the shapes that have several granules (K >= 256)
    if (!d2) return MI_ERR_SHAPE;
    if (rt == 8) return launch_moe<Act, A8, SILU, 8, 2, 1, true>(p, tpw, st);
    if (rt == 4) return launch_moe<Act, A8, SILU, 4, 2, 1, true>(p, tpw, st);
    return launch_moe<Act, A8, SILU, 2, 2, 1, true>(p, tpw, st);
  } else {
    if (rt == 8) return d2 ? launch_moe<Act, A8, SILU, 8, 2>(p, tpw, st) : launch_moe<Act, A8, SILU, 8, 1>(p, tpw, st);
    if (rt == 4) return d2 ? launch_moe<Act, A8, SILU, 4, 2>(p, tpw, st) : launch_moe<Act, A8, SILU, 4, 1>(p, tpw, st);
    return d2 ? launch_moe<Act, A8, SILU, 2, 2>(p, tpw, st) : launch_moe<Act, A8, SILU, 2, 1>(p, tpw, st);
  }
}

template <class Act, bool A8>
static int dispatch_moe(const MoeGemmArgs& p, int fuse_silu, hipStream_t st) {
  return fuse_silu ? dispatch_moe2<Act, A8, true>(p, st) : dispatch_moe2<Act, A8, false>(p, st);
}

}  // namespace qlin

using namespace qlin;

extern "C" {

int mi_moe_gemm_fp8_grouped(const void* a, const float* a_scale, const int32_t* row_map, int row_map_div, const void* w,
                            const float* w_scale, int scale_per_expert, const int32_t* expert_start, void* out,
                            const int32_t* out_map, const void* row_weight, int a_rows, int total_rows, int E,
                            int N, int K, int fuse_act, int act_dtype, int out_f32, void* stream) {
  if (!a || !w || !w_scale || !expert_start || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (fuse_act < 0 || fuse_act > 2 || out_f32 < 0 || out_f32 > 2) return MI_ERR_ARG;
  if (E < 0 || N <= 0 || K <= 0 || (K % 16) || a_rows < 0 || total_rows < 0) return MI_ERR_SHAPE;
  if (a_scale && (K % 128)) return MI_ERR_SHAPE;      // quantised activations carry whole 128-groups
  if (fuse_act && (N % 2)) return MI_ERR_SHAPE;
  if (scale_per_expert < 0 || scale_per_expert > 2 || row_map_div < 1) return MI_ERR_ARG;
  if (scale_per_expert == 2 && (N % 2 || (!fuse_act && (N / 2) % 16))) return MI_ERR_SHAPE;   // halves of whole 16-row tiles
  // block scales with the fused epilogue: a 16-row tile of the up half must not straddle two 128-row blocks
  if (!scale_per_expert && fuse_act && (N / 2) % 16) return MI_ERR_SHAPE;
  if ((uint64_t)N * (uint64_t)K >= (1ull << 31) || (uint64_t)a_rows * (uint64_t)K * 2 >= (1ull << 31))
    return MI_ERR_SHAPE;
  if (!E || !total_rows) return MI_OK;
  // prefill (experts averaging 96 rows or more, 16-bit activations and output): the tiled matrix-core GEMM
  if (!a_scale && out_f32 == 0 && (K % 128) == 0 && E <= 1024 && (long)total_rows >= 96L * E) {
    long long bytes = 0;
    // MI_ERR_SHAPE here means the re-tiled activations would pass 2 GiB: the streaming kernel below,
    // which only bounds a_rows * K, takes such a launch
    if (mi_moe_gemm_fp8_tiled_workspace(total_rows, E, K, &bytes) == MI_OK) {
      void* ws = scratch_get((hipStream_t)stream, (size_t)bytes);
      if (!ws) return MI_ERR_LAUNCH;
      return mi_moe_gemm_fp8_tiled_ws(a, row_map, row_map_div, w, w_scale, scale_per_expert, expert_start, out, out_map, row_weight,
                                      a_rows, total_rows, E, N, K, fuse_act, act_dtype, ws, bytes, stream);
    }
  }
  MoeGemmArgs p{};
  p.a = a; p.a_scale = a_scale; p.row_map = row_map; p.row_div = row_map_div; p.w = w; p.w_scale = w_scale;
  p.start = expert_start; p.out = out; p.E = E; p.N = N; p.K = K; p.a_rows = a_rows;
  p.total_rows = total_rows;
  p.out_map = out_map; p.row_weight = row_weight;
  p.out_f32 = out_f32;
  p.gelu = fuse_act == 2;
  if (a_scale && scale_per_expert) return MI_ERR_ARG;
  p.scale_per_expert = scale_per_expert;
  hipStream_t st = (hipStream_t)stream;
  if (a_scale) {
    return act_dtype == DT_F16 ? dispatch_moe<ActF16, true>(p, fuse_act, st)
                               : dispatch_moe<ActBF16, true>(p, fuse_act, st);
  }
  return act_dtype == DT_F16 ? dispatch_moe<ActF16, false>(p, fuse_act, st)
                             : dispatch_moe<ActBF16, false>(p, fuse_act, st);
}

int mi_moe_gate_up_fp8_routed(const void* a, const float* a_scale, const int32_t* top_ids, int T, int topk,
                              const void* w, const float* w_scale, int32_t* expert_start, int32_t* inv,
                              int32_t* sorted_pairs, void* out, int E, int N, int K, int act_dtype, void* stream) {
  if (!a || !a_scale || !top_ids || !w || !w_scale || !expert_start || !inv || !out) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (T < 0 || topk < 1 || E < 1 || E > 1024 || N <= 0 || K < 256 || (K % 128) || (N % 2) || (N / 2) % 16)
    return MI_ERR_SHAPE;
  const long P = (long)T * topk;
  if (P > kRoutedMaxPairs) return MI_ERR_SHAPE;       // 32 pairs per thread of a 256-thread workgroup
  if ((uint64_t)N * (uint64_t)K >= (1ull << 31) || (uint64_t)T * (uint64_t)K * 2 >= (1ull << 31)) return MI_ERR_SHAPE;
  MoeGemmArgs p{};
  p.a = a; p.a_scale = a_scale; p.row_div = 1; p.w = w; p.w_scale = w_scale; p.out = out;
  p.E = E; p.N = N; p.K = K; p.a_rows = T; p.total_rows = (int)P;
  p.top_ids = top_ids; p.sort_start = expert_start; p.sort_inv = inv; p.sort_pairs = sorted_pairs;
  p.P = (int)P; p.topk = topk;
  p.chunk = ((int)((P + 255) / 256) + 3) & ~3;        // whole 16-byte words of ids per thread
  hipStream_t st = (hipStream_t)stream;
  return act_dtype == DT_F16 ? dispatch_moe2<ActF16, true, true, true>(p, st)
                             : dispatch_moe2<ActBF16, true, true, true>(p, st);
}

int mi_moe_gemm_fp8_block(const void* a, const float* a_scale, const int32_t* row_map, const void* w,
                          const float* w_scale, const int32_t* expert_start, void* out, int a_rows,
                          int total_rows, int E, int N, int K, int fuse_silu_mul, int act_dtype,
                          int out_f32, void* stream) {
  return mi_moe_gemm_fp8_grouped(a, a_scale, row_map, 1, w, w_scale, 0, expert_start, out, nullptr, nullptr, a_rows,
                                 total_rows, E, N, K, fuse_silu_mul ? 1 : 0, act_dtype, out_f32, stream);
}

}  // extern "C"
