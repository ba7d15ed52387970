// MoE auxiliary kernels: routing (softmax + top-k), the expert-sorted token
// permutation, dynamic activation quantisation, SiLU*mul, row scatter and the
// weighted top-k combine.  All are small, HBM- or latency-bound integer / byte /
// elementwise kernels; none of them is reshaped into a GEMM.
#include <type_traits>

#include "qlinear_common.hpp"
#include "moe_sort_expert.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

// ---------------------------------------------------------------- top-k
// One wavefront per token.  Expert e lives in lane e % 64, slot e / 64.  The
// selection runs on the logits (softmax is monotone): K rounds of wave-wide
// argmax where the LOWEST index wins ties, then the selected probabilities are
// renormalised.  The logits are 16-bit values, so a round is one 32-bit wave
// maximum over keys (order-preserving 16 logit bits << 16 | 0xFFFF - index),
// reduced with DPP inside rows of 16 lanes and v_readlane across the four rows;
// the winner's logit is recovered from the key itself.
constexpr int kTopkSlots = 16;                       // up to 1024 experts

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v) {
  const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
  return o > v ? o : v;
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = dpp_max_u32<0xB1>(v);
  v = dpp_max_u32<0x4E>(v);
  v = dpp_max_u32<0x141>(v);
  v = dpp_max_u32<0x140>(v);
  uint32_t r = 0;
#pragma unroll
  for (int row = 0; row < 4; ++row) {
    const uint32_t o = (uint32_t)__builtin_amdgcn_readlane((int)v, row * 16);
    r = o > r ? o : r;
  }
  return r;
}
// 16-bit float pattern (fp16 or bf16) -> unsigned, monotone, and back; the smallest key, 0, is kept for
// "no value" (it would be the pattern of the negative NaN with every bit set)
// -0 is ordered as +0: a float compare calls them equal, and then the lowest index wins the tie
__device__ __forceinline__ uint32_t f16_order(uint32_t b) {
  b = b == 0x8000u ? 0u : b;
  return (b & 0x8000u) ? (~b & 0xFFFFu) : (b | 0x8000u);
}
__device__ __forceinline__ uint32_t f16_unorder(uint32_t u) { return (u & 0x8000u) ? (u & 0x7FFFu) : (~u & 0xFFFFu); }
template <class Act, int SLOTS>
__device__ __forceinline__ void moe_topk_body(const typename Act::elem* __restrict__ logits,
                                              typename Act::elem* __restrict__ top_w,
                                              int32_t* __restrict__ top_ids, int T, int E,
                                              int K, int renorm,
                                              const float* __restrict__ expert_scale,
                                              const typename Act::v8* __restrict__ gate_x,
                                              const typename Act::v8* __restrict__ gate_w,
                                              float* __restrict__ gate_out, int H8, int block) {
  const int lane = threadIdx.x & 63;
  const int t = block * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  // optional second result of the same wavefront: gate_out[t] = sigmoid(gate_x[t, :] . gate_w[:]) (the
  // shared expert's gate of the fused decode ops); its loads are in flight while the selection runs
  float gate_acc = 0.f;
  if (gate_out) {
    // four steps' loads are requested together (indices held inside the row, the surplus is not added)
    for (int c0 = lane; c0 < H8; c0 += 256) {
      typename Act::v8 a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = min(c0 + 64 * u, H8 - 1);
        a[u] = gate_x[(size_t)t * H8 + c];
        b[u] = gate_w[c];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (c0 + 64 * u < H8) {
#pragma unroll
          for (int e = 0; e < 8; ++e) gate_acc += Act::to_f32(a[u][e]) * Act::to_f32(b[u][e]);
        }
      }
    }
  }
  const typename Act::elem* row = logits + (size_t)t * E;
  float v[SLOTS];
  uint32_t key[SLOTS];                               // selection keys; 0 = taken or past E
  float mx = -INFINITY;
  // unconditional loads (index held inside the row): with a branch per slot every load waits for the
  // one before
  typename Act::elem raws[SLOTS];
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) raws[s] = row[min(s * 64 + lane, E - 1)];
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) {
    const int e = s * 64 + lane;
    const typename Act::elem raw = raws[s];
    v[s] = e < E ? Act::to_f32(raw) : -INFINITY;
    key[s] = e < E ? (f16_order((uint32_t)__builtin_bit_cast(uint16_t, raw)) << 16) | (0xFFFFu - (uint32_t)e) : 0u;
    mx = fmaxf(mx, v[s]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) sum += (s * 64 + lane < E) ? __expf(v[s] - mx) : 0.f;
  sum = wave_sum(sum);

  float my_w = 0.f;                                  // lane r keeps the r-th pick
  int my_id = 0;
  float sel_sum = 0.f;
  for (int r = 0; r < K; ++r) {
    uint32_t best = 0;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) best = key[s] > best ? key[s] : best;
    best = wave_max_u32(best);
    const int cand = (int)(0xFFFFu - (best & 0xFFFFu));
    const float wbest = Act::to_f32(__builtin_bit_cast(typename Act::elem, (uint16_t)f16_unorder(best >> 16)));
    // remove the winner from its owner lane
#pragma unroll
    for (int s = 0; s < SLOTS; ++s)
      if (s * 64 + lane == cand) key[s] = 0u;
    const float p = __expf(wbest - mx) / sum;
    sel_sum += p;
    if (lane == r) { my_w = p; my_id = cand; }
  }
  if (lane < K) {
    const float w = renorm ? my_w / sel_sum : my_w;
    typename Act::elem w16 = Act::from_f32(w);
    // optional factor per selected expert, applied to the rounded weight and rounded again
    if (expert_scale) w16 = Act::from_f32(Act::to_f32(w16) * expert_scale[my_id]);
    top_w[(size_t)t * K + lane] = w16;
    top_ids[(size_t)t * K + lane] = my_id;
  }
  if (gate_out) {
    gate_acc = wave_sum(gate_acc);
    if (lane == 0) gate_out[t] = 1.0f / (1.0f + __expf(-gate_acc));
  }
}

template <class Act, int SLOTS>
__global__ __launch_bounds__(256) void moe_topk_kernel(const typename Act::elem* __restrict__ logits,
                                                       typename Act::elem* __restrict__ top_w,
                                                       int32_t* __restrict__ top_ids, int T, int E,
                                                       int K, int renorm,
                                                       const float* __restrict__ expert_scale,
                                                       const typename Act::v8* __restrict__ gate_x,
                                                       const typename Act::v8* __restrict__ gate_w,
                                                       float* __restrict__ gate_out, int H8) {
  moe_topk_body<Act, SLOTS>(logits, top_w, top_ids, T, E, K, renorm, expert_scale, gate_x, gate_w, gate_out, H8,
                            (int)blockIdx.x);
}

// ---------------------------------------------------------------- sort
// Stable counting sort of the flattened (token, route) pairs by expert, in one
// workgroup, deterministic.  Inside an expert the pairs keep their pair-index
// order.  Precondition (what a top-k selection produces): a token's K expert ids
// are distinct and lie in [0, E).  Ids outside the range are held into it, and a
// repeated id within a token makes its pairs share one position; in both cases
// the token's result is unspecified, but every index written stays valid (the
// positions no pair claimed hold pair 0 / token 0), so nothing downstream reads
// out of bounds.  Because a token's K experts are distinct, the rank of pair (t, j) in
// expert e equals the number of tokens t' < t that selected e: a per-expert
// bitmap over tokens (built with order-independent LDS atomic ORs) plus popcounts
// gives the rank without any ordered atomics.
//
// When all tokens fit the LDS bitmap (the serving case) a single exclusive scan
// of the popcounts over the expert-major words yields, for every word, the final
// output position of its first pair — expert offsets included — so the kernel is
// clear, OR, scan, write.  Longer inputs run the chunked path: count, prefix,
// then one bitmap pass per chunk of tokens.
constexpr int kSortThreads = 1024;
constexpr int kSortWords = 4096;                     // bitmap words in LDS

// Expert id of pair q, held into [0, E): an id outside the range would index the LDS tables out of bounds.
__device__ __forceinline__ int sort_expert(const int32_t* __restrict__ top_ids, int q, int E) {
  const int e = top_ids[q];
  return e < 0 ? 0 : (e >= E ? E - 1 : e);
}

// inclusive scan of one value per thread over the 1024-thread workgroup
__device__ __forceinline__ uint32_t block_scan_1024(uint32_t v, uint32_t* wave_tot, int tid) {
  const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t o = __shfl_up(v, off, 64);
    if (lane >= off) v += o;
  }
  if (lane == 63) wave_tot[wave] = v;
  __syncthreads();
  if (tid < 64) {
    uint32_t w = tid < 16 ? wave_tot[tid] : 0;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
      const uint32_t o = __shfl_up(w, off, 64);
      if (tid >= off) w += o;
    }
    if (tid < 16) wave_tot[tid] = w;                  // inclusive totals of waves 0..tid
  }
  __syncthreads();
  return v + (wave ? wave_tot[wave - 1] : 0u);
}

struct SortSmem {
  uint32_t bitmap[kSortWords];
  uint32_t wordpre[kSortWords + 4];
  int32_t count[1024];
  int32_t start[1025];
  int32_t base[1024];
  int32_t own[1024];
  uint32_t wave_tot[16];
  int32_t mx;
};

__device__ __forceinline__ void moe_sort_body(
    const int32_t* __restrict__ top_ids, int32_t* __restrict__ sorted_pairs,
    int32_t* __restrict__ expert_start, int32_t* __restrict__ inv, int32_t* __restrict__ sorted_token,
    int32_t* __restrict__ max_count, int T, int K, int E, SortSmem& sm) {
  uint32_t (&bitmap)[kSortWords] = sm.bitmap;
  uint32_t (&wordpre)[kSortWords + 4] = sm.wordpre;
  int32_t (&count)[1024] = sm.count;
  int32_t (&start)[1025] = sm.start;
  int32_t (&base)[1024] = sm.base;
  uint32_t (&wave_tot)[16] = sm.wave_tot;
  int32_t& mx = sm.mx;
  const int tid = threadIdx.x;
  const int P = T * K;
  const int wpe = kSortWords / E;                     // words per expert in one chunk
  const int Tc = wpe * 32;                            // tokens per chunk

  if (T <= Tc) {
    // ---- single pass ----
    constexpr int WPT = kSortWords / kSortThreads;    // consecutive words per thread
#pragma unroll
    for (int i = 0; i < WPT; ++i) bitmap[tid + i * kSortThreads] = 0;
    if (tid == 0) mx = 0;
    constexpr int kCache = 8;                         // pairs per thread kept in registers
    int ecache[kCache];
#pragma unroll
    for (int i = 0; i < kCache; ++i) {
      const int q = tid + i * kSortThreads;
      ecache[i] = q < P ? sort_expert(top_ids, q, E) : -1;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kCache; ++i) {
      const int q = tid + i * kSortThreads;
      if (q < P) { const int tl = q / K; atomicOr(&bitmap[ecache[i] * wpe + (tl >> 5)], 1u << (tl & 31)); }
    }
    for (int q = tid + kCache * kSortThreads; q < P; q += kSortThreads) {
      const int tl = q / K;
      atomicOr(&bitmap[sort_expert(top_ids, q, E) * wpe + (tl >> 5)], 1u << (tl & 31));
    }
    __syncthreads();
    uint32_t pc[WPT], tot = 0;
#pragma unroll
    for (int i = 0; i < WPT; ++i) { pc[i] = __popc(bitmap[tid * WPT + i]); tot += pc[i]; }
    const uint32_t incl = block_scan_1024(tot, wave_tot, tid);
    uint32_t run = incl - tot;
#pragma unroll
    for (int i = 0; i < WPT; ++i) { wordpre[tid * WPT + i] = run; run += pc[i]; }
    if (tid == kSortThreads - 1) wordpre[kSortWords] = run;
    __syncthreads();
    // words of expert e: [e * wpe, (e + 1) * wpe); words past E * wpe are empty
    for (int e = tid; e <= E; e += kSortThreads) {
      const int s0 = (int)wordpre[min(e * wpe, kSortWords)];
      expert_start[e] = s0;
      if (max_count && e < E) atomicMax(&mx, (int)wordpre[min((e + 1) * wpe, kSortWords)] - s0);
    }
    auto place = [&](int q, int e) {
      const int tl = q / K;
      const int wi = e * wpe + (tl >> 5);
      const int pos = (int)wordpre[wi] + __popc(bitmap[wi] & ((1u << (tl & 31)) - 1u));
      sorted_pairs[pos] = q;
      inv[q] = pos;
      if (sorted_token) sorted_token[pos] = tl;
    };
#pragma unroll
    for (int i = 0; i < kCache; ++i) {
      const int q = tid + i * kSortThreads;
      if (q < P) place(q, ecache[i]);
    }
    for (int q = tid + kCache * kSortThreads; q < P; q += kSortThreads) place(q, sort_expert(top_ids, q, E));
    // positions no pair claimed (only with repeated ids inside a token): valid indices
    for (int pos = (int)wordpre[kSortWords] + tid; pos < P; pos += kSortThreads) {
      sorted_pairs[pos] = 0;
      if (sorted_token) sorted_token[pos] = 0;
    }
    if (max_count) {
      __syncthreads();
      if (tid == 0) max_count[0] = mx;
    }
    return;
  }

  // ---- chunked path ----
  if (tid < E) { count[tid] = 0; base[tid] = 0; }
  // every position starts as a valid index: with repeated ids inside a token some positions of
  // an expert's range are claimed by no pair (ordered before the placement by the barriers below)
  for (int pos = tid; pos < P; pos += kSortThreads) {
    sorted_pairs[pos] = 0;
    if (sorted_token) sorted_token[pos] = 0;
  }
  __syncthreads();
  for (int p = tid; p < P; p += kSortThreads) atomicAdd(&count[sort_expert(top_ids, p, E)], 1);
  __syncthreads();
  // exclusive prefix over experts (Hillis-Steele on up to 1024 entries)
  if (tid < E) start[tid + 1] = count[tid];
  if (tid == 0) start[0] = 0;
  __syncthreads();
  for (int off = 1; off < E; off <<= 1) {
    int add = 0;
    if (tid < E && tid >= off) add = start[tid + 1 - off];
    __syncthreads();
    if (tid < E) start[tid + 1] += add;
    __syncthreads();
  }
  for (int i = tid; i <= E; i += kSortThreads) expert_start[i] = start[i];
  if (max_count) {
    if (tid == 0) mx = 0;
    __syncthreads();
    if (tid < E) atomicMax(&mx, count[tid]);
    __syncthreads();
    if (tid == 0) max_count[0] = mx;
  }

  for (int t0 = 0; t0 < T; t0 += Tc) {
    const int tn = min(Tc, T - t0);
    for (int i = tid; i < E * wpe; i += kSortThreads) bitmap[i] = 0;
    __syncthreads();
    for (int q = tid; q < tn * K; q += kSortThreads) {
      const int tl = q / K;
      const int e = sort_expert(top_ids, t0 * K + q, E);
      atomicOr(&bitmap[e * wpe + (tl >> 5)], 1u << (tl & 31));
    }
    __syncthreads();
    if (tid < E) {
      uint32_t run = 0;
      for (int w = 0; w < wpe; ++w) {
        wordpre[tid * wpe + w] = run;
        run += __popc(bitmap[tid * wpe + w]);
      }
      count[tid] = (int32_t)run;                      // pairs of this expert in the chunk
    }
    __syncthreads();
    for (int q = tid; q < tn * K; q += kSortThreads) {
      const int tl = q / K;
      const int p = t0 * K + q;
      const int e = sort_expert(top_ids, p, E);
      const uint32_t word = bitmap[e * wpe + (tl >> 5)];
      const int rank = base[e] + (int)wordpre[e * wpe + (tl >> 5)] +
                       __popc(word & ((1u << (tl & 31)) - 1u));
      const int pos = start[e] + rank;
      sorted_pairs[pos] = p;
      inv[p] = pos;
      if (sorted_token) sorted_token[pos] = t0 + tl;
    }
    __syncthreads();
    if (tid < E) base[tid] += count[tid];
    __syncthreads();
  }
}

// The same sort spread over several workgroups, for thousands of tokens: workgroup c owns the S
// tokens from c * S on (S * E <= 32 * kSortWords, so that its pairs fit one bitmap).  Every
// workgroup counts all pairs per expert (total, and those of earlier tokens than its own) — ids
// are 4 bytes a pair and come out of L2 — derives the experts' first positions and its own first
// position inside each expert from that, and places its own pairs by their rank in the bitmap.
// Nothing passes between the workgroups.  Ids a top-k never produces: as in moe_sort_body (a
// position that no pair claims lies at the end of the owning workgroup's part of an expert's range
// and is filled by that workgroup).
__device__ __forceinline__ void moe_sort_wide_body(
    const int32_t* __restrict__ top_ids, int32_t* __restrict__ sorted_pairs,
    int32_t* __restrict__ expert_start, int32_t* __restrict__ inv, int32_t* __restrict__ sorted_token,
    int32_t* __restrict__ max_count, int T, int K, int E, int S, int c, SortSmem& sm) {
  const int tid = threadIdx.x;
  const int P = T * K;
  const int wpe = kSortWords / E;
  const int lo = c * S, hi = min(T, lo + S);
  const int p_lo = lo * K, p_hi = hi * K;
  constexpr int WPT = kSortWords / kSortThreads;
#pragma unroll
  for (int i = 0; i < WPT; ++i) sm.bitmap[tid + i * kSortThreads] = 0;
  sm.count[tid] = 0;                                  // pairs per expert, all tokens
  sm.base[tid] = 0;                                   // ... of tokens before lo
  sm.own[tid] = 0;                                    // ... of this workgroup's tokens
  if (tid == 0) sm.mx = 0;
  __syncthreads();
  for (int p = tid; p < P; p += kSortThreads) {
    const int e = sort_expert(top_ids, p, E);
    atomicAdd(&sm.count[e], 1);
    if (p < p_lo) {
      atomicAdd(&sm.base[e], 1);
    } else if (p < p_hi) {
      const int tl = p / K - lo;
      atomicAdd(&sm.own[e], 1);
      atomicOr(&sm.bitmap[e * wpe + (tl >> 5)], 1u << (tl & 31));
    }
  }
  __syncthreads();
  const uint32_t mine = tid < E ? (uint32_t)sm.count[tid] : 0u;
  const uint32_t incl = block_scan_1024(mine, sm.wave_tot, tid);
  if (tid < E) sm.start[tid + 1] = (int32_t)incl;
  if (tid == 0) sm.start[0] = 0;
  int claimed = 0;
  if (tid < E) {
    for (int w = 0; w < wpe; ++w) {
      sm.wordpre[tid * wpe + w] = (uint32_t)claimed;
      claimed += __popc(sm.bitmap[tid * wpe + w]);
    }
    if (c == 0 && max_count) atomicMax(&sm.mx, (int)mine);
  }
  __syncthreads();
  if (c == 0) {
    for (int e = tid; e <= E; e += kSortThreads) expert_start[e] = sm.start[e];
    if (max_count && tid == 0) max_count[0] = sm.mx;
  }
  for (int q = p_lo + tid; q < p_hi; q += kSortThreads) {
    const int e = sort_expert(top_ids, q, E);
    const int t = q / K, tl = t - lo;
    const int wi = e * wpe + (tl >> 5);
    const int pos = sm.start[e] + sm.base[e] + (int)sm.wordpre[wi] + __popc(sm.bitmap[wi] & ((1u << (tl & 31)) - 1u));
    sorted_pairs[pos] = q;
    inv[q] = pos;
    if (sorted_token) sorted_token[pos] = t;
  }
  if (tid < E) {
    const int first = sm.start[tid] + sm.base[tid];
    for (int pos = first + claimed; pos < first + sm.own[tid]; ++pos) {
      sorted_pairs[pos] = 0;
      if (sorted_token) sorted_token[pos] = 0;
    }
  }
}

// Tokens per workgroup of the spread-out sort, or 0 where one workgroup does it all (few tokens, or
// more than 256 workgroups' worth).
static inline int sort_wide_span(int T, int E) {
  const int cap = (kSortWords / E) * 32;              // tokens whose pairs fit one bitmap
  if (T <= cap && T < 2048) return 0;
  int S = (T + 63) / 64;
  S = (S + 31) & ~31;
  if (S < 128) S = 128;
  if (S > cap) S = cap;
  return (T + S - 1) / S <= 256 ? S : 0;
}

__global__ __launch_bounds__(kSortThreads) void moe_sort_kernel(
    const int32_t* __restrict__ top_ids, int32_t* __restrict__ sorted_pairs,
    int32_t* __restrict__ expert_start, int32_t* __restrict__ inv, int32_t* __restrict__ sorted_token,
    int32_t* __restrict__ max_count, int T, int K, int E, int S) {
  __shared__ SortSmem sm;
  if (S) moe_sort_wide_body(top_ids, sorted_pairs, expert_start, inv, sorted_token, max_count, T, K, E, S, blockIdx.x, sm);
  else moe_sort_body(top_ids, sorted_pairs, expert_start, inv, sorted_token, max_count, T, K, E, sm);
}

// The same stable sort with one workgroup per EXPERT, for the serving sizes (a few thousand pairs):
// workgroup e reads all P ids itself (P * 4 bytes from L2) and needs nothing from the others -- the
// number of pairs of lower experts is its first position, and a pair's rank among the expert's own is
// the number of earlier pairs with the same id.  Thread t owns the contiguous pairs
// [t * chunk, (t + 1) * chunk), chunk <= 32, so ranks follow from an exclusive scan over the threads
// plus a popcount inside the thread's own mask.  One dependent round trip to memory instead of the
// single workgroup's clear / mark / scan / place sequence.  Ids outside [0, E) are held into the
// range like in the other paths; every pair gets a position of its own.
constexpr int kSortExpertMaxPairs = 32 * 1024;       // 32 pairs per thread, at most 1024 threads

template <int THREADS>
__global__ __launch_bounds__(THREADS) void moe_sort_expert_kernel(
    const int32_t* __restrict__ top_ids, int32_t* __restrict__ sorted_pairs,
    int32_t* __restrict__ expert_start, int32_t* __restrict__ inv, int32_t* __restrict__ sorted_token,
    int P, int K, int E, int chunk) {
  constexpr int NWV = THREADS / 64;
  __shared__ int32_t wave_lt[NWV], wave_eq[NWV];
  const int e = blockIdx.x, tid = threadIdx.x;
  const int q0 = tid * chunk;
  uint32_t mask;
  int lt, start, count, before;                       // `before`: pairs of this expert in earlier threads
  expert_pairs_of_thread(top_ids, P, E, e, chunk, tid, mask, lt);
  expert_scan<NWV>(mask, lt, tid, wave_lt, wave_eq, start, count, before);
  if (tid == 0) {
    expert_start[e] = start;
    if (e == E - 1) expert_start[E] = start + count;
  }
  int pos = start + before;
  while (mask) {
    const int b = __ffs(mask) - 1;
    mask &= mask - 1;
    const int q = q0 + b;
    sorted_pairs[pos] = q;
    inv[q] = pos;
    if (sorted_token) sorted_token[pos] = q / K;
    ++pos;
  }
}

// ---------------------------------------------------------------- activation quant
// Per row, per 128-wide group: s = max|x| / 448 (clamped at 1e-12), q = e4m3(x / s).
// 16 lanes own one group (8 elements each); the group maximum is a DPP butterfly
// inside the 16-lane row.
template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
  return fmaxf(v, __builtin_bit_cast(float, moved));
}

template <class Act>
__device__ __forceinline__ void act_quant_body(const typename Act::v8* __restrict__ x, u32x2* __restrict__ q,
                                               float* __restrict__ s, size_t groups16, size_t i) {
  // one lane = 8 elements, lane index i
  const bool live = (i >> 4) < groups16;
  typename Act::v8 v;
  if (live) v = x[i];
  float f[8];
  float amax = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    f[e] = live ? Act::to_f32(v[e]) : 0.f;
    amax = fmaxf(amax, fabsf(f[e]));
  }
  amax = dpp_max<0xB1>(amax);
  amax = dpp_max<0x4E>(amax);
  amax = dpp_max<0x141>(amax);
  amax = dpp_max<0x140>(amax);
  const float scale = fmaxf(amax, 1e-12f) / 448.0f;
  int lo = 0, hi = 0;
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0] / scale, f[1] / scale, lo, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2] / scale, f[3] / scale, lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4] / scale, f[5] / scale, hi, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6] / scale, f[7] / scale, hi, true);
  if (live) {
    q[i] = u32x2{(uint32_t)lo, (uint32_t)hi};
    if ((threadIdx.x & 15) == 0) s[i >> 4] = scale;
  }
}

template <class Act>
__global__ __launch_bounds__(256) void act_quant_kernel(const typename Act::v8* __restrict__ x,
                                                        u32x2* __restrict__ q, float* __restrict__ s,
                                                        size_t groups16) {   // 16-lane groups in total
  act_quant_body<Act>(x, q, s, groups16, (size_t)blockIdx.x * 256 + threadIdx.x);
}

// The routing (top-k) and the quantisation of the token activations read different inputs and
// neither waits for the other: one launch, the first `ntopk` workgroups select, the others quantise
// 256 lanes' worth each.  The expert sort, which needs every token's selection, follows alone.
template <class Act, int SLOTS>
__global__ __launch_bounds__(256) void moe_topk_quant_kernel(const typename Act::elem* __restrict__ logits,
                                                             typename Act::elem* __restrict__ top_w,
                                                             int32_t* __restrict__ top_ids, int T, int E, int K,
                                                             int renorm, const typename Act::v8* __restrict__ x,
                                                             u32x2* __restrict__ q, float* __restrict__ s,
                                                             size_t groups16, int ntopk) {
  if ((int)blockIdx.x < ntopk)
    moe_topk_body<Act, SLOTS>(logits, top_w, top_ids, T, E, K, renorm, nullptr, nullptr, nullptr, nullptr, 0,
                              (int)blockIdx.x);
  else
    act_quant_body<Act>(x, q, s, groups16, (size_t)(blockIdx.x - ntopk) * 256 + threadIdx.x);
}

// The expert sort (latency-bound) and the quantisation of the token activations (independent of
// the routing) in one launch: the first workgroup(s) sort, the others quantise 1024 lanes' worth
// each.
template <class Act>
__global__ __launch_bounds__(kSortThreads) void moe_sort_quant_kernel(
    const int32_t* __restrict__ top_ids, int32_t* __restrict__ sorted_pairs,
    int32_t* __restrict__ expert_start, int32_t* __restrict__ inv, int32_t* __restrict__ sorted_token,
    int32_t* __restrict__ max_count, int T, int K, int E, const typename Act::v8* __restrict__ x,
    u32x2* __restrict__ q, float* __restrict__ s, size_t groups16, int S, int nsort) {
  __shared__ SortSmem sm;
  if ((int)blockIdx.x >= nsort)
    act_quant_body<Act>(x, q, s, groups16, (size_t)(blockIdx.x - nsort) * kSortThreads + threadIdx.x);
  else if (S)
    moe_sort_wide_body(top_ids, sorted_pairs, expert_start, inv, sorted_token, max_count, T, K, E, S, blockIdx.x, sm);
  else
    moe_sort_body(top_ids, sorted_pairs, expert_start, inv, sorted_token, max_count, T, K, E, sm);
}

// ---------------------------------------------------------------- elementwise
// out[r, c] = act(gate) * up with act = SiLU, or (GELU) the tanh form of GELU:
// 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))), tanh through exp(2z) with 2z held in
// [-30, 30] so that large gates saturate instead of producing inf / inf.
// One element of act(gate) * up: computed in fp32 and THEN rounded to the activation type, as the reference's
// torch expression does.  The result passes through an opaque copy: left to the compiler, the last multiply and
// the fp16 conversion become one v_fma_mixlo_f16 in one kernel and stay two instructions in the other, and the
// two round differently when the fp32 product sits next to the midpoint of two fp16 values.
template <bool GELU>
__device__ __forceinline__ float act_mul_one(float g, float u) {
  float r;
  if constexpr (GELU) {
    float two_z = 2.0f * (0.7978845608f * (g + 0.044715f * (g * g * g)));
    two_z = two_z > 30.0f ? 30.0f : (two_z < -30.0f ? -30.0f : two_z);
    const float e = expf(two_z);
    r = 0.5f * g * (1.0f + (e - 1.0f) / (e + 1.0f)) * u;
  } else {
    r = g / (1.0f + expf(-g)) * u;
  }
  asm volatile("" : "+v"(r));
  return r;
}

template <class Act, bool GELU>
__global__ __launch_bounds__(256) void silu_mul_kernel(const typename Act::elem* __restrict__ in,
                                                       typename Act::elem* __restrict__ out, int n_gate_up,
                                                       int n_half, int rows) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)rows * n_half) return;
  const int r = (int)(i / n_half), c = (int)(i % n_half);
  const float g = Act::to_f32(in[(size_t)r * n_gate_up + c]);
  const float u = Act::to_f32(in[(size_t)r * n_gate_up + n_half + c]);
  out[i] = Act::from_f32(act_mul_one<GELU>(g, u));
}

// The same values, eight columns per thread with 16-byte loads and stores (n_half a multiple of 8, 16-byte
// aligned operands): a thread of the element-wise kernel moves 6 bytes, and large inputs (prefill: tens of
// megabytes) then run at under half the memory rate.
template <class Act, bool GELU>
__global__ __launch_bounds__(256) void silu_mul_vec_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out,
                                                           int half8, size_t total8) {
  using V8 = typename Act::v8;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total8) return;
  const size_t r = i / (size_t)half8;
  const int c = (int)(i - r * (size_t)half8);
  const V8 gv = as_v8<V8>(in[r * (size_t)(2 * half8) + c]);
  const V8 uv = as_v8<V8>(in[r * (size_t)(2 * half8) + half8 + c]);
  V8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    o[e] = Act::from_f32(act_mul_one<GELU>(Act::to_f32(gv[e]), Act::to_f32(uv[e])));
  }
  out[i] = __builtin_bit_cast(u32x4, o);
}

// scattered[pos] = hidden[pair / topk], weights[pos] = top_w[pair]   (pos -> pair = sorted_pairs[pos])
__global__ __launch_bounds__(256) void scatter_rows_kernel(const u32x4* __restrict__ hidden,
                                                           const uint16_t* __restrict__ top_w,
                                                           const int32_t* __restrict__ sorted_pairs,
                                                           u32x4* __restrict__ scattered,
                                                           uint16_t* __restrict__ weights, int K8, int topk,
                                                           int total) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)total * K8) return;
  const int pos = (int)(i / K8), c = (int)(i % K8);
  const int pair = sorted_pairs[pos];
  scattered[i] = hidden[(size_t)(pair / topk) * K8 + c];
  if (c == 0 && weights) weights[pos] = top_w[pair];
}

// Row permutation of 16-byte chunks: dst[i] = src[map[i]] (gather) or
// dst[map[i]] = src[i] (scatter); map is a permutation of 0 .. rows-1.
__global__ __launch_bounds__(256) void permute_rows_kernel(const u32x4* __restrict__ src,
                                                           const int32_t* __restrict__ map,
                                                           u32x4* __restrict__ dst, int C, int rows,
                                                           int scatter) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)rows * C) return;
  const int r = (int)(i / C), c = (int)(i % C);
  const int m = map[r];
  if (scatter) dst[(size_t)m * C + c] = src[i];
  else dst[i] = src[(size_t)m * C + c];
}

// final[t] = sum_j w_j * y[pos(t, j)]; weights either per sorted position
// (by_pos = 1, the reference's scattered_weights) or per pair (top_w).
// With a shared expert: + gate[t] * shared[t], added in fp32 before the one rounding.
// A thread owns 4 columns of fp32 rows (one 16-byte load per row, so a wavefront reads 1 KiB in a
// row) or 8 columns of 16-bit rows.  The positions, weights and row pieces of up to 8 routes are
// requested before any is used: walked one route at a time, every route is a dependent pair of
// round trips (position, then row), and eight of those in sequence were the whole run time.
template <class Act, int YK>                        // rows of y: 0 activation type, 1 fp32, 2 fp16
__global__ __launch_bounds__(256) void combine_kernel(const void* __restrict__ yv,
                                                      const int32_t* __restrict__ inv,
                                                      const typename Act::elem* __restrict__ w,
                                                      void* __restrict__ outv, int HC, int topk,
                                                      int T, int by_pos,
                                                      const void* __restrict__ sharedv,
                                                      const float* __restrict__ gate) {
  using Elem = typename Act::elem;
  constexpr bool Y32 = YK == 1;
  using YAct = typename std::conditional<YK == 2, ActF16, Act>::type;   // element type of 16-bit rows
  constexpr int CW = Y32 ? 4 : 8;                     // columns per thread
  constexpr int kBatch = 8;                           // routes in flight
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)T * HC) return;
  const int t = (int)(i / HC), c = (int)(i % HC);
  float acc[CW];
#pragma unroll
  for (int e = 0; e < CW; ++e) acc[e] = 0.f;
  for (int j0 = 0; j0 < topk; j0 += kBatch) {
    int pos[kBatch];
    float wj[kBatch];
    // The weights are fetched as raw bits in ONE uniform branch and converted after the rows have
    // been requested: a branch and a conversion per weight make every load wait for the one before
    // (eight dependent round trips).
    uint32_t wraw[kBatch];
    const uint16_t* w16 = reinterpret_cast<const uint16_t*>(w);
#pragma unroll
    for (int b = 0; b < kBatch; ++b) wraw[b] = 0;
    if (w && !by_pos) {                                 // indexed by pair: independent of the positions
#pragma unroll
      for (int b = 0; b < kBatch; ++b) wraw[b] = w16[(size_t)t * topk + (j0 + b < topk ? j0 + b : topk - 1)];
    }
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int j = j0 + b < topk ? j0 + b : topk - 1;
      pos[b] = inv ? inv[(size_t)t * topk + j] : t * topk + j;       // no map: y is in pair order
    }
    if (w && by_pos) {
#pragma unroll
      for (int b = 0; b < kBatch; ++b) wraw[b] = w16[pos[b]];
    }
    auto weights = [&]() {
#pragma unroll
      for (int b = 0; b < kBatch; ++b)   // no weights: plain sum
        wj[b] = w ? Act::to_f32(__builtin_bit_cast(Elem, (uint16_t)wraw[b])) : 1.0f;
    };
    if constexpr (Y32) {
      f32x4 v[kBatch];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) v[b] = ((const f32x4*)yv)[(size_t)pos[b] * HC + c];
      weights();
#pragma unroll
      for (int b = 0; b < kBatch; ++b)
        if (j0 + b < topk) {
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[e] += wj[b] * v[b][e];
        }
    } else {
      typename YAct::v8 v[kBatch];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) v[b] = ((const typename YAct::v8*)yv)[(size_t)pos[b] * HC + c];
      weights();
#pragma unroll
      for (int b = 0; b < kBatch; ++b)
        if (j0 + b < topk) {
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] += wj[b] * YAct::to_f32(v[b][e]);
        }
    }
  }
  if (sharedv) {
    const float gt = gate ? gate[t] : 1.0f;
    const Elem* sv = (const Elem*)sharedv + i * CW;
#pragma unroll
    for (int e = 0; e < CW; ++e) acc[e] += gt * Act::to_f32(sv[e]);
  }
  Elem o[CW];
#pragma unroll
  for (int e = 0; e < CW; ++e) o[e] = Act::from_f32(acc[e]);
  if constexpr (Y32) *reinterpret_cast<uint64_t*>((Elem*)outv + i * CW) = *reinterpret_cast<const uint64_t*>(o);
  else *reinterpret_cast<u32x4*>((Elem*)outv + i * CW) = *reinterpret_cast<const u32x4*>(o);
}

// gate[t] = sigmoid(x[t, :] . gw[:]) in fp32, one wavefront per token.
template <class Act>
__global__ __launch_bounds__(256) void shared_gate_kernel(const typename Act::v8* __restrict__ x,
                                                          const typename Act::v8* __restrict__ gw,
                                                          float* __restrict__ gate, int T, int H8) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  float acc = 0.f;
  for (int c = lane; c < H8; c += 64) {
    const typename Act::v8 a = x[(size_t)t * H8 + c], b = gw[c];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc += Act::to_f32(a[e]) * Act::to_f32(b[e]);
  }
  acc = wave_sum(acc);
  if (lane == 0) gate[t] = 1.0f / (1.0f + __expf(-acc));
}

// ---------------------------------------------------------------- RMS norm (+ residual add, + SiLU gate)
// One workgroup per row of length L:  a = x (+ residual, which is then updated in
// place with the rounded sum);  out = a * rsqrt(mean(a^2) + eps) * weight[i % wlen]
// (* silu(gate)), fp32 throughout, one rounding at the store; x and out may be one buffer
// (every element is read and written by the same thread).  With a residual the sum is
// multiplied by res_scale first (1 for the plain residual add).
template <class Act>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const typename Act::elem* x,
                                                      typename Act::elem* residual,
                                                      const typename Act::elem* __restrict__ gate,
                                                      const typename Act::elem* __restrict__ weight,
                                                      typename Act::elem* out, int L, int wlen,
                                                      float eps, float res_scale) {
  __shared__ float wsum[4];
  const size_t base = (size_t)blockIdx.x * L;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float ss = 0.f;
  for (int i = threadIdx.x; i < L; i += 256) {
    float a = Act::to_f32(x[base + i]);
    if (residual) a = (a + Act::to_f32(residual[base + i])) * res_scale;
    ss += a * a;
  }
  ss = wave_sum(ss);
  if (lane == 0) wsum[wave] = ss;
  __syncthreads();
  const float tot = (wsum[0] + wsum[1]) + (wsum[2] + wsum[3]);
  const float inv = rsqrtf(tot / (float)L + eps);
  for (int i = threadIdx.x; i < L; i += 256) {
    float a = Act::to_f32(x[base + i]);
    if (residual) {
      a = (a + Act::to_f32(residual[base + i])) * res_scale;
      residual[base + i] = Act::from_f32(a);
    }
    float v = a * inv * Act::to_f32(weight[i % wlen]);
    if (gate) {
      const float z = Act::to_f32(gate[base + i]);
      v *= z / (1.0f + __expf(-z));
    }
    out[base + i] = Act::from_f32(v);
  }
}

// h2 = sum of `nsum` consecutive rows of src (fp32; nsum = 1: the row itself);
// h1 <- h2 * rsqrt(mean(h2^2) + eps1) * w1 + h1 (stored rounded, its fp32 value feeds the
// second mean); out = round(h1_stored * rsqrt(mean(h1_new^2) + eps2) * w2).  One workgroup per
// token; each thread re-reads only elements it wrote itself.
template <class Act>
__global__ __launch_bounds__(256) void norm_add_norm_kernel(const typename Act::elem* __restrict__ src, int nsum,
                                                            typename Act::elem* h1,
                                                            const typename Act::elem* __restrict__ w1,
                                                            const typename Act::elem* __restrict__ w2,
                                                            typename Act::elem* out, int K, float eps1, float eps2) {
  __shared__ float wsum[2][4];
  const size_t sbase = (size_t)blockIdx.x * nsum * K;
  const size_t base = (size_t)blockIdx.x * K;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  auto h2_at = [&](int i) {
    float v = 0.f;
    for (int r = 0; r < nsum; ++r) v += Act::to_f32(src[sbase + (size_t)r * K + i]);
    return v;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < K; i += 256) {
    const float v = h2_at(i);
    ss += v * v;
  }
  ss = wave_sum(ss);
  if (lane == 0) wsum[0][wave] = ss;
  __syncthreads();
  const float inv1 = rsqrtf(((wsum[0][0] + wsum[0][1]) + (wsum[0][2] + wsum[0][3])) / (float)K + eps1);
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < K; i += 256) {
    const float v = h2_at(i) * inv1 * Act::to_f32(w1[i]) + Act::to_f32(h1[base + i]);
    h1[base + i] = Act::from_f32(v);
    ss2 += v * v;
  }
  ss2 = wave_sum(ss2);
  if (lane == 0) wsum[1][wave] = ss2;
  __syncthreads();
  const float inv2 = rsqrtf(((wsum[1][0] + wsum[1][1]) + (wsum[1][2] + wsum[1][3])) / (float)K + eps2);
  for (int i = threadIdx.x; i < K; i += 256)
    out[base + i] = Act::from_f32(Act::to_f32(h1[base + i]) * inv2 * Act::to_f32(w2[i]));
}

static inline dim3 grid1d(size_t n, int bs = 256) { return dim3((unsigned)((n + bs - 1) / bs)); }

}  // namespace qlin

using namespace qlin;

extern "C" {

int mi_moe_topk(const void* logits, void* top_w, int32_t* top_ids, int T, int E, int K, int renorm,
                const float* expert_scale, const void* gate_x, const void* gate_weight, float* gate_out, int H,
                int act_dtype, void* stream) {
  if (!logits || !top_w || !top_ids) return MI_ERR_ARG;
  if (gate_out && (!gate_x || !gate_weight)) return MI_ERR_ARG;
  if (gate_out && (H <= 0 || (H % 8))) return MI_ERR_SHAPE;
  const int H8 = gate_out ? H / 8 : 0;
  if (T < 0 || E < 1 || E > 64 * kTopkSlots || K < 1 || K > 64 || K > E) return MI_ERR_SHAPE;
  if (!T) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  const dim3 grid((T + 3) / 4), block(256);
#define QLIN_TOPK(SLOTS)                                                                            \
  do {                                                                                              \
    if (act_dtype == DT_F16)                                                                        \
      hipLaunchKernelGGL((moe_topk_kernel<ActF16, SLOTS>), grid, block, 0, st, (const _Float16*)logits, \
                         (_Float16*)top_w, top_ids, T, E, K, renorm, expert_scale, (const f16x8*)gate_x,        \
                         (const f16x8*)gate_weight, gate_out, H8);                               \
    else                                                                                            \
      hipLaunchKernelGGL((moe_topk_kernel<ActBF16, SLOTS>), grid, block, 0, st, (const __bf16*)logits,  \
                         (__bf16*)top_w, top_ids, T, E, K, renorm, expert_scale, (const bf16x8*)gate_x,         \
                         (const bf16x8*)gate_weight, gate_out, H8);                                 \
  } while (0)
  if (E <= 128) QLIN_TOPK(2);
  else if (E <= 256) QLIN_TOPK(4);
  else if (E <= 512) QLIN_TOPK(8);
  else QLIN_TOPK(16);
#undef QLIN_TOPK
  return launch_status();
}

int mi_moe_topk_quant(const void* logits, void* top_w, int32_t* top_ids, int T, int E, int K, int renorm,
                      const void* x, void* q, float* scale, int H, int act_dtype, void* stream) {
  if (!logits || !top_w || !top_ids || !x || !q || !scale) return MI_ERR_ARG;
  if (T < 0 || E < 1 || E > 64 * kTopkSlots || K < 1 || K > 64 || K > E) return MI_ERR_SHAPE;
  if (H <= 0 || (H % 128)) return MI_ERR_SHAPE;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (!T) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  const size_t groups16 = (size_t)T * (H / 128);
  const int ntopk = (T + 3) / 4;
  const dim3 grid((unsigned)ntopk + (unsigned)((groups16 * 16 + 255) / 256)), block(256);
#define QLIN_TOPKQ(SLOTS)                                                                                   \
  do {                                                                                                      \
    if (act_dtype == DT_F16)                                                                                \
      hipLaunchKernelGGL((moe_topk_quant_kernel<ActF16, SLOTS>), grid, block, 0, st, (const _Float16*)logits, \
                         (_Float16*)top_w, top_ids, T, E, K, renorm, (const f16x8*)x, (u32x2*)q, scale, groups16, ntopk); \
    else                                                                                                    \
      hipLaunchKernelGGL((moe_topk_quant_kernel<ActBF16, SLOTS>), grid, block, 0, st, (const __bf16*)logits,  \
                         (__bf16*)top_w, top_ids, T, E, K, renorm, (const bf16x8*)x, (u32x2*)q, scale, groups16, ntopk); \
  } while (0)
  if (E <= 128) QLIN_TOPKQ(2);
  else if (E <= 256) QLIN_TOPKQ(4);
  else if (E <= 512) QLIN_TOPKQ(8);
  else QLIN_TOPKQ(16);
#undef QLIN_TOPKQ
  return launch_status();
}

int mi_moe_sort(const int32_t* top_ids, int32_t* sorted_pairs, int32_t* expert_start, int32_t* inv,
                int32_t* sorted_token, int32_t* max_count, int T, int K, int E, void* stream) {
  if (!expert_start) return MI_ERR_ARG;
  if (T < 0 || K < 1 || E < 1 || E > 1024) return MI_ERR_SHAPE;
  if (T > 0 && (!top_ids || !sorted_pairs || !inv)) return MI_ERR_ARG;   // T == 0 only fills expert_start
  const long P = (long)T * K;
  if (!max_count && P > 0 && P <= kSortExpertMaxPairs && (long)P * E <= (4l << 20)) {
    // one workgroup per expert; each reads all ids (at most 16 MiB from L2 over the whole launch)
    hipStream_t st = (hipStream_t)stream;
    const int threads = P <= 32 * 256 ? 256 : 1024;
    const int chunk = ((int)((P + threads - 1) / threads) + 3) & ~3;     // whole 16-byte words of ids per thread
    if (threads == 256)
      hipLaunchKernelGGL(moe_sort_expert_kernel<256>, dim3((unsigned)E), dim3(256), 0, st, top_ids, sorted_pairs,
                         expert_start, inv, sorted_token, (int)P, K, E, chunk);
    else
      hipLaunchKernelGGL(moe_sort_expert_kernel<1024>, dim3((unsigned)E), dim3(1024), 0, st, top_ids, sorted_pairs,
                         expert_start, inv, sorted_token, (int)P, K, E, chunk);
    return launch_status();
  }
  const int S = sort_wide_span(T, E);
  hipLaunchKernelGGL(moe_sort_kernel, dim3(S ? (unsigned)((T + S - 1) / S) : 1u), dim3(kSortThreads), 0,
                     (hipStream_t)stream, top_ids, sorted_pairs, expert_start, inv, sorted_token, max_count, T, K, E, S);
  return launch_status();
}

int mi_moe_sort_quant(const int32_t* top_ids, int32_t* sorted_pairs, int32_t* expert_start, int32_t* inv,
                      int32_t* sorted_token, int32_t* max_count, int T, int K, int E, const void* x, void* q,
                      float* scale, long long rows, int H, int act_dtype, void* stream) {
  if (!expert_start || !x || !q || !scale) return MI_ERR_ARG;
  if (T < 0 || K < 1 || E < 1 || E > 1024) return MI_ERR_SHAPE;
  if (T > 0 && (!top_ids || !sorted_pairs || !inv)) return MI_ERR_ARG;
  if (rows < 0 || H <= 0 || (H % 128)) return MI_ERR_SHAPE;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  const size_t groups16 = (size_t)rows * (H / 128);
  const int S = sort_wide_span(T, E);
  const int nsort = S ? (T + S - 1) / S : 1;
  const unsigned grid = (unsigned)nsort + (unsigned)((groups16 * 16 + kSortThreads - 1) / kSortThreads);
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == DT_F16)
    hipLaunchKernelGGL(moe_sort_quant_kernel<ActF16>, dim3(grid), dim3(kSortThreads), 0, st, top_ids, sorted_pairs,
                       expert_start, inv, sorted_token, max_count, T, K, E, (const f16x8*)x, (u32x2*)q, scale,
                       groups16, S, nsort);
  else
    hipLaunchKernelGGL(moe_sort_quant_kernel<ActBF16>, dim3(grid), dim3(kSortThreads), 0, st, top_ids, sorted_pairs,
                       expert_start, inv, sorted_token, max_count, T, K, E, (const bf16x8*)x, (u32x2*)q, scale,
                       groups16, S, nsort);
  return launch_status();
}

int mi_act_quant_fp8(const void* x, void* q, float* scale, long long rows, int K, int act_dtype,
                     void* stream) {
  if (!x || !q || !scale) return MI_ERR_ARG;
  if (rows < 0 || K <= 0 || (K % 128)) return MI_ERR_SHAPE;
  const size_t groups16 = (size_t)rows * (K / 128);
  if (!groups16) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid = grid1d(groups16 * 16);
  if (act_dtype == DT_F16)
    hipLaunchKernelGGL(act_quant_kernel<ActF16>, grid, dim3(256), 0, st, (const f16x8*)x, (u32x2*)q, scale,
                       groups16);
  else if (act_dtype == DT_BF16)
    hipLaunchKernelGGL(act_quant_kernel<ActBF16>, grid, dim3(256), 0, st, (const bf16x8*)x, (u32x2*)q, scale,
                       groups16);
  else
    return MI_ERR_ARG;
  return launch_status();
}

static int act_mul_launch(const void* in, void* out, int n_gate_up, int n_half, int rows, int act_dtype,
                          bool gelu, void* stream) {
  if (!in || !out) return MI_ERR_ARG;
  if (rows < 0 || n_half <= 0 || n_gate_up != 2 * n_half) return MI_ERR_SHAPE;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (!rows) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  if (n_half % 8 == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
    const size_t total8 = (size_t)rows * (n_half / 8);
    const dim3 g8 = grid1d(total8);
#define QLIN_ACT_MUL8(ACT, G) \
  hipLaunchKernelGGL((silu_mul_vec_kernel<ACT, G>), g8, dim3(256), 0, st, (const u32x4*)in, (u32x4*)out, n_half / 8, total8)
    if (act_dtype == DT_F16) { if (gelu) QLIN_ACT_MUL8(ActF16, true); else QLIN_ACT_MUL8(ActF16, false); }
    else { if (gelu) QLIN_ACT_MUL8(ActBF16, true); else QLIN_ACT_MUL8(ActBF16, false); }
#undef QLIN_ACT_MUL8
    return launch_status();
  }
  const dim3 grid = grid1d((size_t)rows * n_half);
#define QLIN_ACT_MUL(ACT, ELEM, G) \
  hipLaunchKernelGGL((silu_mul_kernel<ACT, G>), grid, dim3(256), 0, st, (const ELEM*)in, (ELEM*)out, n_gate_up, n_half, rows)
  if (act_dtype == DT_F16) { if (gelu) QLIN_ACT_MUL(ActF16, _Float16, true); else QLIN_ACT_MUL(ActF16, _Float16, false); }
  else { if (gelu) QLIN_ACT_MUL(ActBF16, __bf16, true); else QLIN_ACT_MUL(ActBF16, __bf16, false); }
#undef QLIN_ACT_MUL
  return launch_status();
}

int mi_moe_silu_mul(const void* in, void* out, int n_gate_up, int n_half, int rows, int act_dtype,
                    void* stream) {
  return act_mul_launch(in, out, n_gate_up, n_half, rows, act_dtype, false, stream);
}

int mi_moe_gelu_tanh_mul(const void* in, void* out, int n_gate_up, int n_half, int rows, int act_dtype,
                         void* stream) {
  return act_mul_launch(in, out, n_gate_up, n_half, rows, act_dtype, true, stream);
}

int mi_moe_scatter(const void* hidden, const void* top_w, const int32_t* sorted_pairs, void* scattered,
                   void* scattered_w, int K, int topk, int total, void* stream) {
  if (!hidden || !sorted_pairs || !scattered) return MI_ERR_ARG;
  if (K <= 0 || (K % 8) || topk < 1 || total < 0) return MI_ERR_SHAPE;
  if (scattered_w && !top_w) return MI_ERR_ARG;
  if (!total) return MI_OK;
  hipLaunchKernelGGL(scatter_rows_kernel, grid1d((size_t)total * (K / 8)), dim3(256), 0, (hipStream_t)stream,
                     (const u32x4*)hidden, (const uint16_t*)top_w, sorted_pairs, (u32x4*)scattered,
                     (uint16_t*)scattered_w, K / 8, topk, total);
  return launch_status();
}

int mi_moe_combine_shared(const void* y, const int32_t* inv, const void* w, void* out, const void* shared,
                          const float* gate, int H, int topk, int T, int weights_by_position, int act_dtype,
                          int y_f32, void* stream) {
  if (!y || !out) return MI_ERR_ARG;
  if (gate && !shared) return MI_ERR_ARG;
  if (H <= 0 || (H % 8) || topk < 1 || T < 0) return MI_ERR_SHAPE;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (!T) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  if (y_f32 < 0 || y_f32 > 2) return MI_ERR_ARG;
  const int HC = y_f32 == 1 ? H / 4 : H / 8;          // column groups per row: 4 columns of fp32, 8 of 16 bit
  const dim3 grid = grid1d((size_t)T * HC);
#define QLIN_COMBINE(ACT, YK, WT)                                                                          \
  hipLaunchKernelGGL((combine_kernel<ACT, YK>), grid, dim3(256), 0, st, y, inv, (const WT*)w, out, HC, topk, T, \
                     weights_by_position, shared, gate)
  if (act_dtype == DT_F16) {
    if (y_f32 == 1) QLIN_COMBINE(ActF16, 1, _Float16); else QLIN_COMBINE(ActF16, 0, _Float16);
  } else {
    if (y_f32 == 1) QLIN_COMBINE(ActBF16, 1, __bf16);
    else if (y_f32 == 2) QLIN_COMBINE(ActBF16, 2, __bf16);
    else QLIN_COMBINE(ActBF16, 0, __bf16);
  }
#undef QLIN_COMBINE
  return launch_status();
}

int mi_moe_combine(const void* y, const int32_t* inv, const void* w, void* out, int H, int topk, int T,
                   int weights_by_position, int act_dtype, int y_f32, void* stream) {
  return mi_moe_combine_shared(y, inv, w, out, nullptr, nullptr, H, topk, T, weights_by_position, act_dtype,
                               y_f32, stream);
}

int mi_permute_rows(const void* src, const int32_t* map, void* dst, int rows, long long row_bytes, int scatter,
                    void* stream) {
  if (!src || !map || !dst) return MI_ERR_ARG;
  if (rows < 0 || row_bytes <= 0 || (row_bytes % 16) || row_bytes / 16 > 0x7fffffff) return MI_ERR_SHAPE;
  if (!rows) return MI_OK;
  const int C = (int)(row_bytes / 16);
  hipLaunchKernelGGL(permute_rows_kernel, grid1d((size_t)rows * C), dim3(256), 0, (hipStream_t)stream,
                     (const u32x4*)src, map, (u32x4*)dst, C, rows, scatter);
  return launch_status();
}

int mi_rmsnorm(const void* x, void* residual, const void* gate, const void* weight, void* out, int rows, int L,
               int weight_len, float eps, int act_dtype, float residual_scale,
               void* stream) {
  if (!x || !weight || !out) return MI_ERR_ARG;
  if (rows < 0 || L <= 0 || weight_len <= 0 || (L % weight_len)) return MI_ERR_SHAPE;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (!rows) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == DT_F16)
    hipLaunchKernelGGL(rmsnorm_kernel<ActF16>, dim3(rows), dim3(256), 0, st, (const _Float16*)x, (_Float16*)residual,
                       (const _Float16*)gate, (const _Float16*)weight, (_Float16*)out, L, weight_len, eps, residual_scale);
  else
    hipLaunchKernelGGL(rmsnorm_kernel<ActBF16>, dim3(rows), dim3(256), 0, st, (const __bf16*)x, (__bf16*)residual,
                       (const __bf16*)gate, (const __bf16*)weight, (__bf16*)out, L, weight_len, eps, residual_scale);
  return launch_status();
}

int mi_norm_add_norm(const void* src, int rows_per_token, void* h1, const void* w1, const void* w2, void* out,
                     int T, int K, float eps1, float eps2, int act_dtype, void* stream) {
  if (!src || !h1 || !w1 || !w2 || !out) return MI_ERR_ARG;
  if (T < 0 || K <= 0 || rows_per_token < 1) return MI_ERR_SHAPE;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (!T) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == DT_F16)
    hipLaunchKernelGGL(norm_add_norm_kernel<ActF16>, dim3(T), dim3(256), 0, st, (const _Float16*)src, rows_per_token,
                       (_Float16*)h1, (const _Float16*)w1, (const _Float16*)w2, (_Float16*)out, K, eps1, eps2);
  else
    hipLaunchKernelGGL(norm_add_norm_kernel<ActBF16>, dim3(T), dim3(256), 0, st, (const __bf16*)src, rows_per_token,
                       (__bf16*)h1, (const __bf16*)w1, (const __bf16*)w2, (__bf16*)out, K, eps1, eps2);
  return launch_status();
}

int mi_moe_shared_gate(const void* x, const void* gate_weight, float* gate, int T, int H, int act_dtype,
                       void* stream) {
  if (!x || !gate_weight || !gate) return MI_ERR_ARG;
  if (H <= 0 || (H % 8) || T < 0) return MI_ERR_SHAPE;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (!T) return MI_OK;
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == DT_F16)
    hipLaunchKernelGGL(shared_gate_kernel<ActF16>, dim3((T + 3) / 4), dim3(256), 0, st, (const f16x8*)x,
                       (const f16x8*)gate_weight, gate, T, H / 8);
  else
    hipLaunchKernelGGL(shared_gate_kernel<ActBF16>, dim3((T + 3) / 4), dim3(256), 0, st, (const bf16x8*)x,
                       (const bf16x8*)gate_weight, gate, T, H / 8);
  return launch_status();
}

}  // extern "C"
