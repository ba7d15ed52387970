// The per-expert step of the stable counting sort of (token, route) pairs by expert, shared by
// moe_sort_expert_kernel and the routed grouped GEMM: a workgroup that serves expert e reads all P
// expert ids itself, thread t owning the contiguous pairs [t * chunk, (t + 1) * chunk).  The pairs of
// lower experts, counted over the workgroup, give the expert's first sorted position; a pair's rank
// inside the expert is the number of earlier pairs of the same expert: an exclusive scan over the
// threads plus a popcount inside the thread's own mask.
#pragma once
#include "qlinear_common.hpp"

namespace qlin {

constexpr int kSortExpertChunkMax = 32;               // pairs per thread: one 32-bit mask

// Thread `tid` owns the pairs [tid * chunk, (tid + 1) * chunk), chunk a multiple of 4, at most 32.  Their
// ids are read with eight unconditional 16-byte buffer loads, all in flight together (words past the
// chunk or past P read nothing; a branch per load would make each wait for the one before).
__device__ __forceinline__ void expert_ids_load(const int32_t* __restrict__ top_ids, int P, int chunk, int tid,
                                                u32x4 (&v)[kSortExpertChunkMax / 4]) {
  const __amdgpu_buffer_rsrc_t ir = make_rsrc(top_ids, (uint32_t)P * 4u);
  const int q0 = tid * chunk;
#pragma unroll
  for (int b4 = 0; b4 < kSortExpertChunkMax / 4; ++b4)
    v[b4] = __builtin_amdgcn_raw_buffer_load_b128(ir, ((uint32_t)(q0 + 4 * b4) * 4u) | (4 * b4 < chunk ? 0u : kOOB), 0, 0);
}

// From the loaded ids: `mask` bit b = pair tid * chunk + b belongs to expert e, `lt` = how many of the
// thread's pairs belong to lower experts.  Ids outside [0, E) are held into the range.
__device__ __forceinline__ void expert_ids_count(const u32x4 (&v)[kSortExpertChunkMax / 4], int P, int E, int e,
                                                 int chunk, int tid, uint32_t& mask, int& lt) {
  const int q0 = tid * chunk;
  mask = 0;
  lt = 0;
#pragma unroll
  for (int b4 = 0; b4 < kSortExpertChunkMax / 4; ++b4)
#pragma unroll
    for (int z = 0; z < 4; ++z) {
      const int b = 4 * b4 + z;
      const int raw = (int)v[b4][z];
      const int id = raw < 0 ? 0 : (raw >= E ? E - 1 : raw);
      const bool mine = b < chunk && q0 + b < P;
      lt += mine && id < e;
      mask |= (uint32_t)(mine && id == e) << b;
    }
}

__device__ __forceinline__ void expert_pairs_of_thread(const int32_t* __restrict__ top_ids, int P, int E, int e,
                                                       int chunk, int tid, uint32_t& mask, int& lt) {
  u32x4 v[kSortExpertChunkMax / 4];
  expert_ids_load(top_ids, P, chunk, tid, v);
  expert_ids_count(v, P, E, e, chunk, tid, mask, lt);
}

// Workgroup-wide sums of one (mask, lt) per thread: the expert's first sorted position, its number of
// pairs, and the rank inside the expert of this thread's first pair.  NWV wavefronts; contains a barrier.
template <int NWV>
__device__ __forceinline__ void expert_scan(uint32_t mask, int lt, int tid, int32_t* wave_lt, int32_t* wave_eq,
                                            int& start, int& count, int& before) {
  const int lane = tid & 63, wave = tid >> 6;
  const int eq = __popc(mask);
  int incl = eq, lsum = lt;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int o = __shfl_up(incl, off, 64);
    if (lane >= off) incl += o;
    lsum += __shfl_xor(lsum, off, 64);
  }
  if (lane == 63) { wave_eq[wave] = incl; wave_lt[wave] = lsum; }
  __syncthreads();
  start = 0;
  count = 0;
  before = incl - eq;
#pragma unroll
  for (int w = 0; w < NWV; ++w) {
    start += wave_lt[w];
    count += wave_eq[w];
    if (w < wave) before += wave_eq[w];
  }
}

}  // namespace qlin
