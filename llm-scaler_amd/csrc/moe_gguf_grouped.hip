// Grouped GGUF MoE GEMMs over chunks of expert-sorted rows: every chunk {expert, first row, rows}
// is a small-M GEMM against that expert's repacked K-quant matrix.  The weight-streaming skinny
// kernel runs them all in one launch (grid = row blocks x chunks): a workgroup owns 64 weight rows
// of the chunk's expert and all of K, and multiplies them with up to 64 (or 16) rows of x, which it
// gathers itself through the token list.  All workgroups of a chunk run on one XCD.
#include "skinny_kernel.hpp"
#include "../../include/mi355x_qlinear.h"

using namespace qlin;

namespace {

template <int FMT, int MT, int UN, bool SL, int RT = 4, int NW = 8>
void launch_grouped_one(SkinnyArgs a, hipStream_t st) {
  a.rpw = RT * 16;
  a.tiles_total = 0;
  for (int i = 0; i < a.nmat; ++i) {
    a.tiles[i] = (a.N[i] + a.rpw - 1) / a.rpw;
    a.tiles_total += a.tiles[i];
  }
  constexpr int MTL = MT ? MT : 4;                    // tiles of x the LDS is sized for
  constexpr int kStage = NW * RT * 16 * (64 + 16) + (MTL >= kSkinnyXLdsFrom ? NW * 16 * (256 + 16) : 0);
  constexpr int kRed = NW * RT * MTL * 1024;
  static_assert((kStage > kRed ? kStage : kRed) <= 160 * 1024, "staging tiles exceed the 160 KiB of LDS per workgroup");
  const int with_tables = kStage + (SL ? skinny_table_bytes<FMT, RT>(a.K) : 0);
  const int lds = with_tables > kRed ? with_tables : kRed;
  // MT = 0: the workgroups choose 1..4 tiles of x themselves (LDS sized for four)
  void (*kern)(const SkinnyArgs);
  if constexpr (MT == 0) kern = skinny_grouped_kernel<ActF16, FMT, RT, NW, SL>;
  else kern = skinny_kernel<ActF16, FMT, 0, MT, RT, NW, UN, SL, true>;
  if (lds > 64 * 1024) {
    static int raised = 0;                            // opt in to > 64 KiB of dynamic LDS (grows with K)
    if (raised < lds) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      raised = lds;
    }
  }
  const long long wgs = (long long)((a.num_chunks + 8 * a.cgroup - 1) / (8 * a.cgroup)) * 8 * a.cgroup * a.tiles_total;
  hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(NW * 64), lds, st, a);
}

template <int FMT, int MT, int UN, int RT = 4, int NW = 8>
void launch_grouped(const SkinnyArgs& a, hipStream_t st) {
  if constexpr (FMT == 2 || FMT == 7) {               // the formats with per-32 scale and min tables
    if (skinny_tables_fit<FMT, MT ? MT : 4, RT, NW>(a.K)) return launch_grouped_one<FMT, MT, UN, true, RT, NW>(a, st);
  }
  launch_grouped_one<FMT, MT, UN, false, RT, NW>(a, st);
}

}  // namespace

extern "C" {

int mi_moe_gguf_grouped(int fmt, const void* x, int x_rows, const int32_t* tok_ids, int nmat, const void* const* ql,
                        const void* const* qh, const void* const* scale, const void* const* qmin, void* out,
                        long long out_stride, int out_rows, const int32_t* chunks, int num_chunks, int num_experts,
                        int N, int K, int rows16, void* stream) {
  if (!x || !ql || !scale || !out || !chunks) return MI_ERR_ARG;
  if (fmt != RF_Q4K && fmt != RF_Q5K && fmt != RF_Q6K) return MI_ERR_ARG;
  if (nmat < 1 || nmat > 2 || num_experts < 1) return MI_ERR_ARG;
  if (x_rows < 0 || out_rows < 0 || num_chunks < 0 || N < 0 || K <= 0 || (K % 32)) return MI_ERR_SHAPE;
  if (out_stride < (long long)nmat * N) return MI_ERR_SHAPE;
  if ((uint64_t)N * (uint64_t)K >= (1ull << 31) || (uint64_t)x_rows * (uint64_t)K * 2ull >= (1ull << 31)) return MI_ERR_SHAPE;
  if (!num_chunks || !N || !out_rows || !x_rows) return MI_OK;
  SkinnyArgs a{};
  a.x = x; a.nmat = nmat; a.K = K; a.M = 0; a.rpw = 64;
  a.chunks = chunks; a.tok_ids = tok_ids; a.num_chunks = num_chunks; a.num_experts = num_experts;
  a.x_rows = x_rows; a.out_rows = out_rows; a.out_stride = out_stride;
  const long long nk = (long long)N * K;
  a.w_stride = nk / 2;
  a.s_stride = fmt == RF_Q6K ? nk / 16 * 2 : nk / 32 * 2;
  a.z_stride = nk / 32 * 2;
  a.h_stride = fmt == RF_Q5K ? nk / 8 : nk / 4;
  for (int i = 0; i < nmat; ++i) {
    if (!ql[i] || !scale[i]) return MI_ERR_ARG;
    if (fmt != RF_Q6K && (!qmin || !qmin[i])) return MI_ERR_ARG;
    if (fmt != RF_Q4K && (!qh || !qh[i])) return MI_ERR_ARG;
    a.w[i] = ql[i]; a.s[i] = scale[i];
    a.z[i] = fmt != RF_Q6K ? qmin[i] : nullptr;
    a.h[i] = fmt != RF_Q4K ? qh[i] : nullptr;
    a.out[i] = (char*)out + (size_t)i * N * 2;
    a.N[i] = N;
    a.tiles[i] = (N + 63) / 64;
    a.tiles_total += a.tiles[i];
  }
  // chunks of one expert follow each other in the caller's list: with about g chunks of 64 rows per expert,
  // groups of g consecutive chunks share an XCD, so an expert's row block is fetched into one L2 once
  const long long per_expert = (long long)out_rows / ((long long)64 * num_experts);
  a.cgroup = rows16 ? 1 : (int)(per_expert < 1 ? 1 : (per_expert > 8 ? 8 : per_expert));
  if ((long long)((num_chunks + 8 * a.cgroup - 1) / (8 * a.cgroup)) * 8 * a.cgroup * a.tiles_total >= (1ll << 31)) return MI_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  // 7 / 8: Q5_K / Q6_K with the high bits in element order.  Small workgroups (two or four wavefronts splitting
  // K, one granule in flight each) so that several share a CU and overlap their load -> LDS -> MFMA chains:
  // T=2048, top 8 of 128 experts, H=2048, I=768: Q4_K up 364 -> 273 us, Q6_K down 345 -> 196 us against eight
  // wavefronts; 16 tokens: up 61 -> 50 us, down 122 -> 46 us.
  if (fmt == RF_Q4K) {
    if (rows16) launch_grouped<RF_Q4K, 1, 2, 4, 4>(a, st);
    else launch_grouped<RF_Q4K, 0, 1, 4, 2>(a, st);
  } else if (fmt == RF_Q5K) {
    if (rows16) launch_grouped<7, 1, 1, 4, 2>(a, st);
    else launch_grouped<7, 0, 1, 4, 2>(a, st);
  } else {
    if (rows16) launch_grouped<8, 1, 1, 4, 2>(a, st);
    else launch_grouped<8, 0, 1, 4, 2>(a, st);
  }
  return launch_status();
}

}  // extern "C"
