// The dispatcher behind the weight-streaming entry points (FP8, INT4, Q4_K): which kernel runs a
// given M, K, N.  Shared by the translation units that hold the entry points, one per weight
// family, so that they compile side by side.
#pragma once
#include "skinny_kernel.hpp"
#include "kslice_kernel.hpp"
#include "scratch.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

// Runs M in chunks of 64 rows (the skinny kernel's limit); each chunk streams
// the weight once, so this is meant for decode-sized M.
template <int FMT, int SC>
static int run(SkinnyArgs a, int act_dtype, hipStream_t st) {
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (FMT == 2 && act_dtype != DT_F16) return MI_ERR_ARG;
  if (a.M < 0 || a.K <= 0) return MI_ERR_SHAPE;
  if (FMT == 0 && (a.K % 32)) return MI_ERR_SHAPE;
  if (FMT == 1 && (a.K % 128)) return MI_ERR_SHAPE;
  if (FMT == 2 && (a.K % 32)) return MI_ERR_SHAPE;
  for (int i = 0; i < a.nmat; ++i) {
    if (a.N[i] < 0 || !a.w[i] || !a.out[i]) return MI_ERR_ARG;
    if (FMT == 1 && (a.z[i] != nullptr) != (a.z[0] != nullptr)) return MI_ERR_ARG;   // zero-points for all or none
    if ((uint64_t)a.N[i] * (uint64_t)a.K >= (1ull << 31)) return MI_ERR_SHAPE;
    a.tiles[i] = (a.N[i] + 15) / 16;
  }
  if (!a.x) return MI_ERR_ARG;
  if (a.M == 0) return MI_OK;
  // decode regime: one wavefront per weight row, activations staged in LDS
  // 3 or 4 rows: the MFMA kernels are ahead of the row kernel's LDS-staged activations (N=14336,
  // K=4096: INT4 fp16 11.0 against 15.8 us, FP8 13.5 against 15.8 us, block-scaled 12.9 against
  // 16.3 us; Q4_K K=N=5120 11.1 against 11.7 us), except FP8 with at most 16 weight rows per CU and
  // long rows (N=4096, K=4096: 7.1 against 6.7 us)
  int rows_max_m = 2;
  if constexpr (FMT == 0) {
    long ntot = 0;
    for (int i = 0; i < a.nmat; ++i) ntot += a.N[i];
    if (!(ntot > 16L * device_cu_count() || a.K <= 2048)) rows_max_m = 4;
  }
  if (a.M <= rows_max_m && rows_lds_bytes(FMT, a.M == 3 ? 4 : a.M, a.K) <= 64 * 1024 && (FMT != 0 || a.K % 16 == 0)) {
    RowsArgs r{};
    r.x = a.x; r.nmat = a.nmat; r.M = a.M; r.K = a.K; r.scale_f16 = a.scale_f16;
    for (int i = 0; i < a.nmat; ++i) {
      r.w[i] = a.w[i]; r.s[i] = a.s[i]; r.z[i] = a.z[i]; r.out[i] = a.out[i]; r.N[i] = a.N[i];
    }
    if constexpr (FMT == 1) {                          // int4: the zero-point load is a template choice
      if (a.z[0]) {
        if (act_dtype == DT_F16) launch_rows_m<ActF16, RF_INT4, RS_ZP>(r, st);
        else launch_rows_m<ActBF16, RF_INT4, RS_ZP>(r, st);
      } else {
        if (act_dtype == DT_F16) launch_rows_m<ActF16, RF_INT4, RS_PERN>(r, st);
        else launch_rows_m<ActBF16, RF_INT4, RS_PERN>(r, st);
      }
    } else if (FMT == 2 || act_dtype == DT_F16)
      launch_rows_m<ActF16, FMT, SC>(r, st);
    else
      launch_rows_m<ActBF16, FMT, SC>(r, st);
    return launch_status();
  }
  // few rows whose slice of x fits the register file: activations resident, weights streamed
  if constexpr (FMT == 0) {
    long ntot = 0;
    for (int i = 0; i < a.nmat; ++i) ntot += a.N[i];
    // measured against the granule-interleaved kernel (M = 5 .. 32): ahead by 5-35 % when a workgroup
    // owns at least two 16-row tiles or rows are short, behind by 10-25 % for one tile of long rows
    const long cus = device_cu_count();
    // 33 .. 64 rows (K <= 2048): between 16 and 32 weight rows per CU the row-split launch of the
    // granule-interleaved kernel is ahead (M=64 K=2048: N=4096 7.4 against 8.5 us, block-scaled
    // N=8192 8.8 against 9.7 us; N=12288 14.1 against 11.8 us, N=2048 8.7 against 8.2 us)
    const bool pays = a.M > 32 ? (ntot > 32 * cus || ntot < 16 * cus) : (ntot > 16 * cus || a.K <= 2048);
    if (const int nq = pays ? kslice_loads(a.M, a.K) : 0)
      return act_dtype == DT_F16 ? kslice_launch<ActF16>(a, SC, nq, st) : kslice_launch<ActBF16>(a, SC, nq, st);
  }
  if constexpr (FMT == 1) {
    // INT4: the same kernel, nibbles decoded with their group's scale; ahead of the granule-interleaved
    // kernel at every N measured (K = 4096, fp16: N = 14336 M=8 13.2 -> 11.6 us, M=32 16.8 -> 14.6 us;
    // N = 4096 7.2 -> 6.5 and 9.7 -> 8.7 us; N = 2048 M=16 8.2 -> 6.3 us; K = 2048 M=64 N = 12288
    // 15.1 -> 11.0 us)
    if (const int nq = kslice_loads(a.M, a.K, 1))
      return act_dtype == DT_F16 ? kslice_launch<ActF16, 1>(a, 0, nq, st) : kslice_launch<ActBF16, 1>(a, 0, nq, st);
  }
  if constexpr (FMT == 2) {
    // Q4_K on the same kernel (fp16; up to 16 rows for K <= 5120, 32 for K <= 3072, 64 for K <= 2048):
    // K = N = 5120 M=8 12.6 -> 11.2 us, M=16 14.0 -> 11.5 us; K=2048 N=8192 M=32 8.6 -> 7.6 us
    if (const int nq = kslice_loads(a.M, a.K, 2)) return kslice_launch<ActF16, 2>(a, 0, nq, st);
  }
  // prefill: the tiled matrix-core GEMM reads the weight once per 256 rows instead of once per 64
  if constexpr (FMT == 0 || FMT == 2) {
    if (a.M > 64 && a.K % 128 == 0) {
      long long bytes = 0;
      if (mi_gemm_tiled_workspace(a.M, a.K, &bytes) != MI_OK) return MI_ERR_SHAPE;
      void* ws = scratch_get(st, (size_t)bytes);
      if (!ws) return MI_ERR_LAUNCH;
      for (int i = 0; i < a.nmat; ++i) {
        const int rc = FMT == 0 ? mi_gemm_fp8_tiled_ws(a.x, a.w[i], a.s[i], SC, a.scale_f16, a.out[i], ws, bytes, a.M,
                                                       a.N[i], a.K, act_dtype, st)
                                : mi_gemm_q4k_tiled_ws(a.x, a.w[i], a.s[i], a.z[i], a.out[i], ws, bytes, a.M, a.N[i],
                                                       a.K, st);
        if (rc != MI_OK) return rc;
      }
      return MI_OK;
    }
  }
  const int M = a.M;
  const size_t esz = 2;
  for (int m0 = 0; m0 < M; m0 += 64) {
    SkinnyArgs c = a;
    c.M = (M - m0) < 64 ? (M - m0) : 64;
    c.x = (const char*)a.x + (size_t)m0 * a.K * esz;
    for (int i = 0; i < a.nmat; ++i) c.out[i] = (char*)a.out[i] + (size_t)m0 * a.N[i] * esz;
    int rc;
    if (FMT == 2)
      rc = launch_mt<ActF16, FMT, SC>(c, st);
    else
      rc = act_dtype == DT_F16 ? launch_mt<ActF16, FMT, SC>(c, st) : launch_mt<ActBF16, FMT, SC>(c, st);
    if (rc != MI_OK) return rc;
  }
  return MI_OK;
}

}  // namespace qlin
