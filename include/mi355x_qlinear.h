/* C ABI of libmi355x_qlinear.so — the gfx950 quantized-linear kernels.
 *
 * One function per operator of the reference's custom-kernel packages
 * (vllm/custom-esimd-kernels-vllm = V/, sglang/custom-esimd-kernels = S/).  The
 * reference binds its kernels to torch.ops with ATen tensors; the functions here
 * take what those launchers extract from the tensors: raw device pointers,
 * sizes, and the stream to enqueue on.  Conventions shared by all of them:
 *
 *   - every pointer is device memory; outputs are pre-allocated by the caller;
 *   - the call enqueues on `stream` (a hipStream_t, 0 = the null stream) and
 *     returns without synchronising; nothing is allocated or freed, except by the
 *     entries that say so: a grow-only scratch buffer per (device, stream), allocated with
 *     hipMalloc on first use or growth (not possible under stream capture), is used by
 *     mi_gemm_int4, by mi_gemm_fp8_{pern,pert,blockscale}[_multi] and mi_gemv_q4k for M > 64,
 *     and by mi_moe_gemm_fp8_grouped / _block when the experts average 96 rows or more;
 *     mi_norm_gemv[_scaled] takes a 2 KiB counter block per device and stream on first use.
 *     Callers that capture or must not allocate use the *_ws variants with
 *     mi_gemm_tiled_workspace / mi_moe_gemm_fp8_tiled_workspace bytes of their own memory
 *     (what the torch ops do), and mi_norm_gemv_static;
 *   - tensors are dense row-major;
 *   - act_dtype: 0 = fp16, 1 = bf16 (inputs and outputs share it);
 *   - return value: 0 on success, MI_ERR_ARG (-1) for a null pointer or bad
 *     enum, MI_ERR_SHAPE (-2) for a shape the kernels do not cover,
 *     MI_ERR_LAUNCH (-3) if the launch itself failed, MI_ERR_LIMIT (-4) for a size
 *     beyond the fixed capacity of an entry point that allocates nothing,
 *     MI_ERR_BUSY (-5) when that entry point's static scratch belongs to another stream.
 */
#ifndef MI355X_QLINEAR_H_
#define MI355X_QLINEAR_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI_DT_F16 0
#define MI_DT_BF16 1

/* ---- FP8 (E4M3) weight-only, per-output-channel scale ---------------------
 * out[M,N] = (x[M,K] @ e4m3(w[N,K])^T) * scale[n].   K % 32 == 0.
 * Replaces esimd_gemv_fp8_pern (V/csrc/xpu/esimd_kernel.sycl:39-48,
 * V/csrc/xpu/esimd_kernels/fp8_GEMV_v2.h:123-162), extended to any M and to
 * fp32 scales (scale_is_f16 = 0).  E4M3 decode is exact (no subnormal flush).
 * The _multi form runs up to 3 weight matrices that share x in one launch and
 * replaces esimd_gemv_fp8_pern_fused2/3 (V/csrc/xpu/torch_extension.cc:13-25). */
int mi_gemm_fp8_pern(const void* x, const void* w, const void* scale, void* out, int M, int N, int K,
                     int act_dtype, int scale_is_f16, void* stream);
int mi_gemm_fp8_pern_multi(const void* x, int nmat, const void* const* w, const void* const* scale,
                           void* const* out, const int* N, int M, int K, int act_dtype,
                           int scale_is_f16, void* stream);

/* ---- FP8 weight-only, per-tensor scale (fp32 scalar read from device memory)
 * Replaces esimd_gemv_fp8_pert / _bmg / _fused2/3 and esimd_gemm_fp8_pert
 * (V/csrc/xpu/esimd_kernel.sycl:88-98, :654-670; esimd_kernel_gemm.sycl:32-49). */
int mi_gemm_fp8_pert(const void* x, const void* w, const float* scale, void* out, int M, int N, int K,
                     int act_dtype, void* stream);
int mi_gemm_fp8_pert_multi(const void* x, int nmat, const void* const* w, const float* const* scale,
                           void* const* out, const int* N, int M, int K, int act_dtype, void* stream);

/* ---- FP8 weight-only, 128x128 block scale (w8a16) --------------------------
 * out = x @ (e4m3(w) * S[n/128, k/128])^T, S fp32 [ceil(N/128), K/128], K % 128 == 0.
 * Replaces esimd_gemm_fp8_blockscale and esimd_gemv_fp8_blockscale_fused2
 * (V/csrc/xpu/esimd_kernel_gemm.sycl:97-139,
 * V/csrc/xpu/esimd_kernels/fp8_GEMM_blockscale.h:197-223). */
int mi_gemm_fp8_blockscale(const void* x, const void* w, const float* scale, void* out, int M, int N,
                           int K, int act_dtype, void* stream);
int mi_gemm_fp8_blockscale_multi(const void* x, int nmat, const void* const* w,
                                 const float* const* scale, void* const* out, const int* N, int M,
                                 int K, int act_dtype, void* stream);

/* ---- INT4, group 128, weight-streaming (decode) ----------------------------
 * w [N, K/2] uint8 (== [N, K/8] int32), low nibble = even k, stored value =
 * signed + 8; scale [N, K/128] fp16; zp [N, K/128] uint8 in 0..15 or NULL for
 * the implicit zero-point 8.  out = x @ ((nib - zp) * scale)^T.  K % 128 == 0.
 * Replaces esimd_gemv_int4 / esimd_gemv_int4_fused2
 * (V/csrc/xpu/esimd_kernel.sycl:200-230,
 * V/csrc/xpu/esimd_kernels/int4_GEMV.h:267-304, :414-462) and, for M <= 64,
 * esimd_gemm_int4_pgrp (esimd_kernel_gemm.sycl:55-91).  The zero-point operand
 * has no counterpart in the reference's kernels. */
int mi_gemv_int4(const void* x, const void* w, const void* scale, const void* zp, void* out, int M,
                 int N, int K, int act_dtype, void* stream);
int mi_gemv_int4_multi(const void* x, int nmat, const void* const* w, const void* const* scale,
                       const void* const* zp, void* const* out, const int* N, int M, int K,
                       int act_dtype, void* stream);

/* ---- INT4 group-128 GEMM, any M (prefill) --------------------------------------
 * Same operands as mi_gemv_int4.  M <= 64 runs the weight-streaming kernel; larger
 * M runs the MFMA GEMM (weights dequantized to the activation dtype while they are
 * staged into LDS; activations re-tiled into MFMA operand order by a pre-pass and
 * read straight into registers).  Replaces esimd_gemm_int4_pgrp
 * (V/csrc/xpu/esimd_kernel_gemm.sycl:55-91, V/csrc/xpu/esimd_kernels/int4_GEMM.h:291-320),
 * without its 64-row limit; the zero-point operand (cfg2's asymmetric weights) has
 * no counterpart in the reference's kernels.
 * mi_gemm_int4 keeps its scratch for the re-tiled activations in a grow-only
 * buffer per (device, stream), the convention of the reference's launchers
 * (V/csrc/xpu/esimd_kernel_moe.sycl:45-67): the first call of a size allocates
 * (not possible while the stream is being captured), later calls reuse it;
 * mi_gemm_int4_ws uses a caller-provided workspace of at least
 * mi_gemm_int4_workspace() bytes (0 when no workspace is needed), 16-byte aligned,
 * which must stay untouched until the stream has passed the call. */
int mi_gemm_int4(const void* x, const void* w, const void* scale, const void* zp, void* out, int M, int N,
                 int K, int act_dtype, void* stream);
int mi_gemm_int4_workspace(int M, int N, int K, long long* bytes);
int mi_gemm_int4_ws(const void* x, const void* w, const void* scale, const void* zp, void* out,
                    void* workspace, long long workspace_bytes, int M, int N, int K, int act_dtype,
                    void* stream);

/* ---- GPTQ / AWQ style operands of the reference's asymmetric W4A16 linear -----------
 * The reference calls a third-party op for these weights,
 * int4_gemm_w4a16(x, qweight[K/8, N] int32, bias, scales[K/g, N], qzeros, g, g_idx)
 * (vllm/patches/vllm_for_multi_arc.patch:5492-5500, AWQ :5002-5010, GPTQ :5080-5088; the op's
 * source is not part of the reference tree, so its zero-point packing is restated here from
 * the published GPTQ layout).  mi_w4a16_kmajor_prepare turns those operands into the ones
 * mi_gemm_int4 / mi_gemv_int4 read, bit for bit, on the device:
 *   w_out [N, K/8] int32  = qweight transposed (nibble z of a word = element 8i + z on both
 *                           sides); pass qweight = w_out = NULL when the caller's [K/8, N]
 *                           tensor already has strides (1, K/8), i.e. the same bytes;
 *   s_out [N, K/128] fp16 = scales [K/128, N] transposed;
 *   zp_out[N, K/128] u8   = zero_scalar ? qzeros[0]
 *                         : ((qzeros[g][n / 8] >> 4 (n % 8)) & 15) + zero_bias, qzeros [K/128, N/8]
 *                           int32 (zero_bias 1 for checkpoints that store zero - 1); NULL for none.
 * Group size 128 only; N % 8 == 0 with packed zero-points.  mi_add_bias adds bias[N] to every
 * row of out[M, N] in place (fp32 sum, one rounding), the op's optional bias argument. */
int mi_w4a16_kmajor_prepare(const int32_t* qweight, const void* scales, const int32_t* qzeros, int zero_scalar,
                            int zero_bias, void* w_out, void* s_out, uint8_t* zp_out, int N, int K, void* stream);
int mi_add_bias(void* out, const void* bias, int M, int N, int act_dtype, void* stream);

/* ---- GGUF Q4_K on the repacked representation, fp16 -------------------------
 * ql [N, K/2] uint8 interleaved nibbles, scale/qmin [N, K/32] fp16;
 * w = fp16(fp16(nib * scale) - qmin);  out = x @ w^T.  K % 32 == 0.
 * Replaces esimd_gemv_q4_k (S/csrc/xpu/esimd_kernel.sycl:224-239,
 * S/csrc/xpu/esimd_kernels/q4_k_GEMV.h:110-132), extended to any M. */
int mi_gemv_q4k(const void* x, const void* ql, const void* scale, const void* qmin, void* out, int M,
                int N, int K, void* stream);

/* ---- dequant-only entries (bit-exactness checks, load-time dense copies) ----
 * They share the in-register dequant routines of the fused kernels.
 * mi_dequant_int4: out [N,K] fp16/bf16 = rne((nib - zp) * scale), the value
 *   V/tests/test_gemv_int4.py:172-212 defines (int4_dequantize_ref).
 * mi_dequant_fp8: out [N,K] fp32 = e4m3(w) * scale; scale_mode 0 = per-channel
 *   fp32 [N], 1 = per-channel fp16 [N], 2 = per-tensor fp32 [1], 3 = 128x128
 *   block fp32 (V/tests/test_fp8_blockscale_gemm.py:31-36, dequant_weight).
 * mi_decode_e4m3: count codes (multiple of 8) -> fp16/bf16, exact for all 254
 *   finite codes (V/csrc/xpu/esimd_kernels/fp8_GEMM_blockscale.h:40-49).
 * mi_dequant_q4k: repacked Q4_K -> dense fp16, two fp16 roundings
 *   (_xpu_dequant_q4_k, sglang/patches/sglang_for_multi_arc.patch:2576-2587).
 * mi_q4k_repack: raw GGUF block_q4_K rows [N, K/256*144] -> ql [N,K/2] u8,
 *   scale/qmin [N,K/32] fp16 (_xpu_repack_q4_k, same patch :2527-2573). */
int mi_dequant_int4(const void* w, const void* scale, const void* zp, void* out, int N, int K,
                    int out_dtype, void* stream);
int mi_dequant_fp8(const void* w, const void* scale, int scale_mode, float* out, int N, int K,
                   void* stream);
int mi_decode_e4m3(const void* codes, void* out, long long count, int out_dtype, void* stream);
int mi_dequant_q4k(const void* ql, const void* scale, const void* qmin, void* out, int N, int K,
                   void* stream);
int mi_q4k_repack(const void* raw, void* ql, void* scale, void* qmin, int N, int K, void* stream);

/* ---- other GGUF formats: weight preparation, dequant, decode GEMV (fp16) ------
 * Resident representations (what the reference's ops read):
 *   Q4_0: packed [N,K/2] u8 interleaved nibbles (byte j = elem 2j | elem 2j+1 << 4),
 *         scale [N,K/32] fp16; w = (nib - 8) * scale.
 *   Q8_0: qs [N,K] int8, scale [N,K/32] fp16; w = qs * scale.
 *   Q5_K: ql [N,K/2] interleaved low nibbles, qh [N,K/8] (per 512-k tile, bit b of
 *         byte t = fifth bit of element b*64+t), scale/qmin [N,K/32] fp16;
 *         w = fp16(fp16(v5 * scale) - qmin).
 *   Q6_K: ql [N,K/2], qh [N,K/4] (per 512-k tile, 2-bit field p of byte t = top
 *         bits of element p*128+t), scale [N,K/16] fp16; w = (v6 - 32) * scale.
 * mi_q4_0_repack / mi_q8_0_repack / mi_q5k_repack / mi_q6k_repack: raw GGML rows
 *   ([N, K/32*18], [N, K/32*34], [N, K/256*176], [N, K/256*210] bytes) -> resident
 *   (_xpu_repack_q4_0, _xpu_repack_q8_0, _xpu_repack_q5_k, _xpu_repack_q6_k,
 *   sglang/patches/sglang_for_multi_arc.patch:2173-2193, 3031-3044, 2725-2740,
 *   2996-3008).  K % 32 == 0; K % 512 == 0 for the K-quants (whole shuffle tiles).
 * mi_dequant_*: resident -> dense fp16 [N,K] with the fp16 roundings of
 *   _xpu_dequant_q4_0_packed / _q8_0 / _q5_k / _q6_k (same patch :2196-2213,
 *   3047-3054, 2952-2970, 3011-3026), the reference's route for M > 1.
 * mi_gemv_*: out [M,N] fp16 = x [M,K] fp16 @ w^T, fp32 accumulation.  Replace
 *   esimd_gemv_q4_0, esimd_gemm_q4_0, esimd_gemv_q8_0(_m), esimd_gemv_q5_k,
 *   esimd_gemv_q6_k(_m) (S/csrc/xpu/torch_extension.cc:48-106), for any M (up to 4 rows: one
 *   wavefront per weight row; more rows: the MFMA kernels, 64 rows per pass).
 * mi_q4_0_quantize: x [rows,K] fp16/bf16 -> qweight [rows,K/8] int32 (nibble i of
 *   word w = element 8w+i, value + 8) + scale [rows,K/128] fp16 = max/-8, the
 *   layout mi_gemv_int4 reads.  GGML's quantize_row_q4_0 rule on 128-wide blocks;
 *   replaces q4_0_quantize (V/csrc/xpu/torch_extension_q4_0.cc:27-75,
 *   V/csrc/xpu/q4_0_quant.sycl:30-120).  K % 128 == 0. */
/* Routed decode GEMVs of a GGUF MoE layer, one launch over all routes r = t * top_k + j:
 *   out[i][r, :] = route_weight[r] * (x[r / x_div, :] @ dequant(W_i[route_expert[r]])^T), i < nmat <= 2,
 * W_i = the per-expert stack [E, N, ...] of the repacked representation
 * (fmt 2 = Q4_K: ql, scale, qmin; 5 = Q5_K: + qh; 6 = Q6_K: ql, qh, scale), fp16, rows of out
 * out_stride elements apart, route_weight (fp16) optional, expert ids clamped into [0, E).
 * The high bits of the Q5_K / Q6_K stacks are in ELEMENT order, not tile-shuffled as for the
 * dense GEMVs: Q5_K qh [E,N,K/8], bit b of byte j = fifth bit of element 8j+b; Q6_K qh
 * [E,N,K/4], 2-bit field p of byte j = top bits of element 4j+p (moe_kquant_GEMV.h:109-116,
 * 159-166; built by _xpu_repack_q5_k_plain / _q6_k_plain, sglang_for_multi_arc.patch:2736-2765,
 * here mi_q5k_repack_plain / mi_q6k_repack_plain).  K % 32 == 0 for every format.
 * One kernel launch per matrix.
 * Replaces the launches of esimd_moe_up_q4k (two matrices: gate and up halves of one buffer,
 * x_div = top_k; SiLU * up follows as mi_moe_silu_mul) and esimd_moe_down_q5k / _q6k
 * (x = the intermediate in route order, x_div = 1, route_weight = topk_w)
 * (S/csrc/xpu/torch_extension.cc:86-101, S/csrc/xpu/esimd_kernels/moe_kquant_GEMV.h). */
int mi_moe_gguf_gemv(int fmt, const void* x, int x_div, int nmat, const void* const* ql, const void* const* qh,
                     const void* const* scale, const void* const* qmin, void* const* out, long long out_stride,
                     const int32_t* route_expert, const void* route_weight, int routes, int num_experts, int N,
                     int K, void* stream);
/* Grouped form over chunks of expert-sorted rows (MoE prefill and multi-token verify):
 * chunks [num_chunks, 3] int32 = {expert, first row t0, rows nt}; for every chunk and matrix i
 *   out[t0 + m, i N + n] = sum_k x[row(t0 + m), k] W_i[expert][n, k],   m < min(nt, 64)   (16 when rows16)
 * with row(p) = tok_ids[p] when tok_ids is given (the expert-sort permutation, out_rows entries; the
 * gather of x happens inside the load) and p otherwise.  x [x_rows, K] fp16, out [out_rows, out_stride]
 * fp16 with out_stride >= nmat N; stacks as for mi_moe_gguf_gemv ([E, N, K/2] nibbles, [E, N, K/32] fp16
 * scales and mins).  Chunks with nt <= 0, an expert outside [0, E) or rows outside the output are
 * skipped; rows of a chunk past the 64 (16) are not computed, as in the reference kernel; token ids
 * outside [0, x_rows) read as zero rows.  Weights are dequantized as fp16(fp16(nibble * scale) - min)
 * and accumulated in fp32.  fmt = 2 (Q4_K), 5 (Q5_K: fp16(fp16(v5 * scale) - min)) or 6 (Q6_K:
 * fp16((v6 - 32) * scale), scales [E, N, K/16]); the high bits of 5 / 6 in ELEMENT order as for
 * mi_moe_gguf_gemv.  nmat <= 2, K % 32 == 0; one kernel launch.
 * Replaces moe_up_q4k_ggemv / moe_up_q4k_ggemv_smallm (S/csrc/moe_grouped/moe_q4k_ggemv.h:47-201, 311-321),
 * moe_down_q5k_ggemv / _smallm (moe_q5k_down_ggemv.h:26-191) and moe_down_q6k_ggemv / _smallm
 * (moe_q6k_down_ggemv.h) with x = the intermediate in sorted order and no token list; ATen entries
 * S/csrc/moe_grouped/moe_grouped_entry.sycl:24-106; callers sglang_for_multi_arc.patch:2899-2924. */
int mi_moe_gguf_grouped(int fmt, const void* x, int x_rows, const int32_t* tok_ids, int nmat, const void* const* ql,
                        const void* const* qh, const void* const* scale, const void* const* qmin, void* out,
                        long long out_stride, int out_rows, const int32_t* chunks, int num_chunks, int num_experts,
                        int N, int K, int rows16, void* stream);
int mi_q4_0_repack(const void* raw, void* packed, void* scale, int N, int K, void* stream);
int mi_q8_0_repack(const void* raw, void* qs, void* scale, int N, int K, void* stream);
int mi_q5k_repack(const void* raw, void* ql, void* qh, void* scale, void* qmin, int N, int K,
                  void* stream);
int mi_q6k_repack(const void* raw, void* ql, void* qh, void* scale, int N, int K, void* stream);
/* The same with qh in element order (the MoE down stacks, see mi_moe_gguf_gemv); K % 256 == 0.
 * Replace _xpu_repack_q5_k_plain / _xpu_repack_q6_k_plain (sglang_for_multi_arc.patch:2736-2765). */
int mi_q5k_repack_plain(const void* raw, void* ql, void* qh, void* scale, void* qmin, int N, int K,
                        void* stream);
int mi_q6k_repack_plain(const void* raw, void* ql, void* qh, void* scale, int N, int K, void* stream);
int mi_dequant_q4_0(const void* packed, const void* scale, void* out, int N, int K, void* stream);
int mi_dequant_q8_0(const void* qs, const void* scale, void* out, int N, int K, void* stream);
int mi_dequant_q5k(const void* ql, const void* qh, const void* scale, const void* qmin, void* out,
                   int N, int K, void* stream);
int mi_dequant_q6k(const void* ql, const void* qh, const void* scale, void* out, int N, int K,
                   void* stream);
int mi_gemv_q4_0(const void* x, const void* packed, const void* scale, void* out, int M, int N, int K,
                 void* stream);
int mi_gemv_q8_0(const void* x, const void* qs, const void* scale, void* out, int M, int N, int K,
                 void* stream);
int mi_gemv_q5k(const void* x, const void* ql, const void* qh, const void* scale, const void* qmin,
                void* out, int M, int N, int K, void* stream);
int mi_gemv_q6k(const void* x, const void* ql, const void* qh, const void* scale, void* out, int M,
                int N, int K, void* stream);
int mi_q4_0_quantize(const void* x, void* qweight, void* scale, int rows, int K, int in_dtype,
                     void* stream);

/* ---- MoE routing and permutation --------------------------------------------
 * mi_moe_topk: fp32 softmax over E experts -> top-K (lowest index wins ties,
 *   descending probability) -> optional renormalisation; top_w in the activation
 *   dtype, top_ids int32.  E <= 1024, K <= 64.  expert_scale (optional, fp32 [E]): the rounded
 *   weight of a selected expert is multiplied by its entry and rounded again (MoeFoldExpertScale,
 *   V/csrc/moe_batch/moe_decode_gemv.h:146-158).  gate_out (optional, fp32 [T], with gate_x [T, H]
 *   and gate_weight [H] in the activation type, H % 8 == 0): the same launch also writes
 *   sigmoid(gate_x[t] . gate_weight), the shared expert's gate of the fused decode ops (what
 *   mi_moe_shared_gate computes on its own).  Replaces esimd_moe_topk /
 *   moe_ops::moe_topk (V/csrc/xpu/esimd_kernels/moe_ops.h:106-231,
 *   V/csrc/xpu/esimd_kernel_moe.sycl:71-84).
 * mi_moe_sort: stable counting sort of the T*K (token, route) pairs by expert:
 *   sorted_pairs[pos] = t*K + j, expert_start[E+1] (exclusive prefix of counts),
 *   inv[t*K + j] = pos, optional sorted_token[pos] = t and max_count[0] = largest
 *   expert load.  Deterministic; the K experts of a token must be distinct.
 *   Same result as build_sorted_token_ids / build_topk_ids
 *   (V/csrc/xpu/esimd_kernels/moe_ops.h:238-271); replaces the scatter
 *   init/prefix kernels (:437-520) and moe_prefill_gather_forward_kernel_fp8
 *   (S/csrc/moe_prefill/moe_prefill_fp8.sycl:105-161), whose in-expert order is
 *   atomic-arrival order. */
int mi_moe_topk(const void* logits, void* top_w, int32_t* top_ids, int T, int E, int K, int renorm,
                const float* expert_scale, const void* gate_x, const void* gate_weight, float* gate_out, int H,
                int act_dtype, void* stream);
int mi_moe_sort(const int32_t* top_ids, int32_t* sorted_pairs, int32_t* expert_start, int32_t* inv,
                int32_t* sorted_token, int32_t* max_count, int T, int K, int E, void* stream);

/* ---- MoE elementwise helpers -------------------------------------------------
 * mi_act_quant_fp8: per row, per 128-wide K group: s = max|x|/448 (>= 1e-12/448),
 *   q = e4m3(x / s).  No counterpart in the reference's kernels (they are w8a16,
 *   V/csrc/xpu/esimd_kernels/fp8_moe_gemm_blockscale.h:5-7).
 * mi_moe_silu_mul: out[r, c] = silu(in[r, c]) * in[r, n_half + c]
 *   (esimd_moe_silu_mul, V/csrc/xpu/esimd_kernels/moe_ops.h:576-621).
 * mi_moe_gelu_tanh_mul: the same with the tanh form of GELU on the gate half
 *   (esimd_moe_gelu_tanh_mul, moe_ops.h:680-728; exp argument held in [-30, 30]).
 * mi_moe_scatter: scattered[pos] = hidden[sorted_pairs[pos] / topk], optional
 *   scattered_w[pos] = top_w[sorted_pairs[pos]]   (esimd_moe_scatter, moe_ops.h:522-569).
 * mi_moe_combine: out[t] = sum_j w * y[inv[t*topk + j]], weights indexed by sorted
 *   position (weights_by_position = 1, esimd_moe_gather, moe_ops.h:627-676) or by
 *   pair; y is in the activation dtype (y_f32 = 0), fp32 (1) or fp16 beside any activation
 *   dtype (2).  w may be null: the rows are
 *   summed unweighted (moe_accumulate, V/csrc/moe_batch/moe.sycl:1177-1230).
 *   inv may be null: y is then already in pair order (row t*topk + j), as
 *   moe_prefill_accumulate_forward_fp8 takes it
 *   (S/csrc/moe_prefill/moe_prefill_fp8.sycl:413-436).
 * mi_permute_rows: dst[i] = src[map[i]] (scatter = 0) or dst[map[i]] = src[i]
 *   (scatter = 1) on rows of row_bytes (multiple of 16) bytes; moves grouped-GEMM
 *   rows between expert-sorted and pair order (the reference's up/down prefill
 *   kernels scatter to pair order themselves, moe_prefill_fp8.sycl:280-300, :385-411).
 * mi_moe_shared_gate: gate[t] = sigmoid(x[t, :] . gate_weight[:]) in fp32
 *   (moe_down_gate_precompute_kernel, V/csrc/moe_batch/moe.sycl:978-1010).
 * mi_moe_combine_shared: mi_moe_combine + gate[t] * shared[t, :] (shared expert's
 *   output, activation dtype; gate may be null = 1), summed in fp32 and rounded once
 *   (the finalize step of moe_down_finalize_fp8_block_batched_kernel,
 *   V/csrc/moe_batch/moe.sycl:1570-1663). */
/* mi_moe_sort and mi_act_quant_fp8 of the token activations x [rows, H] in one launch
 * (the two are independent; the sort is a single latency-bound workgroup).  No counterpart
 * in the reference: its MoE path keeps 16-bit activations. */
int mi_moe_sort_quant(const int32_t* top_ids, int32_t* sorted_pairs, int32_t* expert_start, int32_t* inv,
                      int32_t* sorted_token, int32_t* max_count, int T, int K, int E, const void* x,
                      void* q, float* scale, long long rows, int H, int act_dtype, void* stream);
/* mi_moe_topk (without the expert factors and the shared gate) and mi_act_quant_fp8 of the token
 * activations x [T, H] in one launch: the routing reads the logits, the quantisation reads x, and
 * neither waits for the other, while the expert sort needs every token's selection and follows
 * alone (mi_moe_sort).  Same results as the two separate calls, bit for bit.  No counterpart in the
 * reference: its MoE path keeps 16-bit activations. */
int mi_moe_topk_quant(const void* logits, void* top_w, int32_t* top_ids, int T, int E, int K, int renorm,
                      const void* x, void* q, float* scale, int H, int act_dtype, void* stream);
int mi_act_quant_fp8(const void* x, void* q, float* scale, long long rows, int K, int act_dtype,
                     void* stream);
int mi_moe_silu_mul(const void* in, void* out, int n_gate_up, int n_half, int rows, int act_dtype,
                    void* stream);
int mi_moe_gelu_tanh_mul(const void* in, void* out, int n_gate_up, int n_half, int rows, int act_dtype,
                         void* stream);
int mi_moe_scatter(const void* hidden, const void* top_w, const int32_t* sorted_pairs, void* scattered,
                   void* scattered_w, int K, int topk, int total, void* stream);
int mi_moe_combine(const void* y, const int32_t* inv, const void* w, void* out, int H, int topk, int T,
                   int weights_by_position, int act_dtype, int y_f32, void* stream);
int mi_permute_rows(const void* src, const int32_t* map, void* dst, int rows, long long row_bytes, int scatter,
                    void* stream);
int mi_moe_shared_gate(const void* x, const void* gate_weight, float* gate, int T, int H, int act_dtype,
                       void* stream);
int mi_moe_combine_shared(const void* y, const int32_t* inv, const void* w, void* out, const void* shared,
                          const float* gate, int H, int topk, int T, int weights_by_position, int act_dtype,
                          int y_f32, void* stream);

/* ---- RMS norm in front of a GEMV -------------------------------------------------
 * Per row of length L:  a = x (+ residual; residual is then overwritten with the
 * rounded sum);  out = a * rsqrt(mean(a^2) + eps) * weight[i % weight_len]
 * (* silu(gate[i]) when gate is given), fp32 arithmetic, one rounding.  residual and
 * gate may be null.  This is the normalisation half of the reference's fused
 * decode ops — esimd_resadd_norm_gemv_{int4,fp8}_pert
 * (V/csrc/xpu/esimd_kernels/resadd_norm_gemv_int4.h:56-100), esimd_norm_gemv_*_pert
 * (per-head gated norm, norm_gemv_int4.h), esimd_rms_norm (esimd_kernel.sycl:488-502);
 * the ops run it and then the GEMV entry point on its output.  With a residual the sum is
 * multiplied by residual_scale before it is stored and normalised (1 for the plain add;
 * esimd_fused_scaled_add_rms_norm, V/csrc/xpu/torch_extension.cc:145-148).  x and out may be
 * the same buffer (esimd_fused_add_rms_norm writes the normalised row over hidden_states). */
int mi_rmsnorm(const void* x, void* residual, const void* gate, const void* weight, void* out, int rows, int L,
               int weight_len, float eps, int act_dtype,
               float residual_scale, void* stream);

/* Two chained norms around a residual add, per token:
 *   h2 = sum of rows_per_token consecutive rows of src (fp32; 1: the row itself),
 *   h1 <- h2 * rsqrt(mean(h2^2) + eps1) * w1 + h1 (in place),
 *   out = h1 * rsqrt(mean(h1^2) + eps2) * w2, the second mean over the unrounded h1.
 * Replaces esimd_norm_add_norm (rows_per_token = 1) and esimd_accum_norm_add_norm
 * (rows_per_token = top_k) (V/csrc/xpu/torch_extension.cc:168-175,
 * esimd_kernels/norm_add_norm.h:46-86, accum_norm_add_norm.h). */
int mi_norm_add_norm(const void* src, int rows_per_token, void* h1, const void* w1, const void* w2, void* out,
                     int T, int K, float eps1, float eps2, int act_dtype, void* stream);

/* The same normalisation fused into the decode GEMV (one launch, M == 1):
 *   x' = rmsnorm(x (+ residual)) (* silu(gate)) per head of norm_len elements
 *   (norm_len == K: the whole row), out[i] = x' @ dequant(w[i])^T for nmat <= 3
 *   matrices.  fmt 0 = FP8 per-tensor scale (scale[i] -> fp32 [1]), 1 = FP8 128x128
 *   block scale, 2 = INT4 group 128 (scale[i] fp16 [N, K/128]).  residual (in place),
 *   gate and normed_out may be null.  Every workgroup normalises its own copy of the
 *   row; the in-place residual and normed_out are written by the workgroup that
 *   arrives last at a per-stream device counter (2 KiB, from a pool of 64 blocks that the
 *   first call on a device allocates and zeroes: that one call must not run under stream
 *   capture; later streams take a block without allocating), after all others have read
 *   their inputs.  Rows longer than 16384 fall back to mi_rmsnorm + the GEMV (normed_out
 *   is then required).  Replaces the launch of esimd_resadd_norm_gemv_{int4,fp8}_pert,
 *   esimd_resadd_norm_gemv2_fp8_pert, esimd_norm_gemv_{int4,fp8}_pert and
 *   esimd_norm_gemv_fp8_blockscale (V/csrc/xpu/torch_extension.cc:103-133,
 *   V/csrc/xpu/esimd_kernels/resadd_norm_gemv_fused.h:1-24, norm_gemv_fused.h). */
int mi_norm_gemv(const void* x, void* residual, const void* gate, const void* norm_weight,
                 void* normed_out, int norm_len, float eps, int fmt, int nmat, const void* const* w,
                 const void* const* scale, void* const* out, const int* N, int K, int act_dtype,
                 void* stream);
/* The same with x + residual multiplied by residual_scale before it is stored and normalised
 * (unrounded into the norm, as the reference does): replaces esimd_scaled_resadd_norm_gemv_fp8_pert
 * (V/csrc/xpu/torch_extension.cc:163-166, esimd_kernels/scaled_resadd_norm_gemv_fp8.h:70-100). */
int mi_norm_gemv_scaled(const void* x, void* residual, const void* gate, const void* norm_weight,
                        void* normed_out, int norm_len, float eps, float residual_scale, int fmt, int nmat,
                        const void* const* w, const void* const* scale, void* const* out, const int* N, int K,
                        int act_dtype, void* stream);
/* mi_norm_gemv_scaled for callers that cannot allocate: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same
 * arguments and results; the arrival counters live in a 2 KiB static device array inside the
 * library (one copy per GPU, held until the process ends) instead of a per-stream hipMalloc,
 * and the call allocates and frees nothing.  Only the fused single launch is covered: rows
 * beyond its limit (K > 16384, or K whose staged row exceeds 64 KiB of LDS) return
 * MI_ERR_LIMIT (-4) instead of taking the two-kernel route.  All calls on one GPU share the
 * counters: the kernel leaves them at zero when it ends, so back-to-back calls on one stream
 * are fine, while calls that overlap on one GPU (different streams) would race.  Therefore the
 * first call after a set-up claims the array for its stream, and a call on any other stream of
 * that GPU returns MI_ERR_BUSY (-5) without launching.
 * mi_static_scratch_setup resolves the array's address on the current device (the first call
 * of mi_norm_gemv_static on a device does the same), clears the counters with a blocking
 * hipMemset and releases the claim: call it once per device before capturing; call it again,
 * with no mi_norm_gemv_static work in flight on that GPU, to hand the array to another stream
 * or to recover after a kernel that ended abnormally and left counters non-zero. */
int mi_static_scratch_setup(void);
int mi_norm_gemv_static(const void* x, void* residual, const void* gate, const void* norm_weight,
                        void* normed_out, int norm_len, float eps, float residual_scale, int fmt, int nmat,
                        const void* const* w, const void* const* scale, void* const* out, const int* N, int K,
                        int act_dtype, void* stream);

/* ---- MoE prefill: grouped FP8 GEMM on the tiled matrix-core kernel ---------------
 * mi_moe_gemm_fp8_grouped in w8a16 mode (no a_scale, output in the activation type) for experts
 * with hundreds of rows: a device-built table of M-tiles per expert, activations gathered and
 * re-tiled per 16-row block, then the 256 x 256 tiled GEMM with one weight matrix per expert, so
 * that an expert's weights are read once per 256 of its rows (a wavefront skips the 16-row tiles
 * past an expert's last row).  Same arguments and
 * results; K % 128 == 0, E <= 1024.  workspace: mi_moe_gemm_fp8_tiled_workspace bytes; that call
 * returns MI_ERR_SHAPE (with *bytes still set) when the re-tiled activations,
 * (total_rows / 16 + E) * 16 * K * 2 bytes, would reach 2 GiB: such a launch belongs to the
 * streaming kernel.  mi_moe_gemm_fp8_grouped takes this route itself (per-stream scratch) when the
 * experts average 96 rows or more and the workspace call succeeds, and streams otherwise.  Reference: the 64-row expert tiles with a device-built tile map of
 * V/csrc/xpu/esimd_kernels/fp8_moe_gemm_blockscale.h:83-120, 187-302 and the per-expert M-tiled
 * GEMMs of S/csrc/moe_prefill/moe_prefill_fp8.sycl:167-410. */
int mi_moe_gemm_fp8_tiled_workspace(int total_rows, int E, int K, long long* bytes);
int mi_moe_gemm_fp8_tiled_ws(const void* a, const int32_t* row_map, int row_map_div, const void* w,
                             const float* w_scale, int scale_per_expert, const int32_t* expert_start, void* out,
                             const int32_t* out_map, const void* row_weight, int a_rows, int total_rows,
                             int E, int N, int K, int fuse_act, int act_dtype, void* workspace,
                             long long workspace_bytes, void* stream);
/* The expert MLP of that regime as one call: out = (act(a W13_gate^T) * (a W13_up^T)) W2^T per expert,
 * w13 [E, 2 I, H] and w2 [E, H, I] E4M3, block scales [E, 2I/128, H/128] / [E, H/128, I/128]
 * (scale_per_expert 0), one fp32 per expert and matrix (1), or gate / up scalars for w13 and one
 * for w2 (2); fuse_act 1 = SiLU, 2 = tanh-GELU.  row_map / row_map_div gather the rows of `a`;
 * out_map / row_weight apply to `out` [rows, H] as in mi_moe_gemm_fp8_tiled_ws.  Bit-identical to
 * two mi_moe_gemm_fp8_tiled_ws calls with a row-major intermediate between them; the tile table
 * is built once, and the first GEMM writes the intermediate in the operand order the second
 * reads, so it is neither stored row-major nor re-tiled.  H % 128 == 0, I % 128 == 0.  Reference:
 * the gate_up, SiLU x up, down sequence of the fused forward (V/csrc/xpu/moe.sycl:1509-1663) on
 * the grouped prefill GEMM (V/csrc/xpu/esimd_kernels/fp8_moe_gemm_blockscale.h:304-357). */
int mi_moe_mlp_fp8_tiled_workspace(int total_rows, int E, int H, int I, long long* bytes);
int mi_moe_mlp_fp8_tiled_ws(const void* a, const int32_t* row_map, int row_map_div, const void* w13,
                            const float* w13_scale, const void* w2, const float* w2_scale, int scale_per_expert,
                            const int32_t* expert_start, void* out, const int32_t* out_map, const void* row_weight,
                            int a_rows, int total_rows, int E, int H, int I, int fuse_act, int act_dtype,
                            void* workspace, long long workspace_bytes, void* stream);

/* ---- prefill (M > 64) on FP8 and Q4_K weights: the tiled matrix-core GEMM ---------
 * The same results as mi_gemm_fp8_pern / _pert / _blockscale and mi_gemv_q4k, computed by the
 * 256 x 256 (224, 128) tiled GEMM that also serves mi_gemm_int4, so that a weight byte is read
 * once per 256 activation rows.  scale_mode 0 = per output channel (fp32, or fp16 with
 * scale_is_f16), 1 = per tensor (fp32 [1]), 2 = 128 x 128 blocks (fp32 [ceil(N/128), K/128],
 * folded into the weight before its rounding to the activation type).  K % 128 == 0.
 * workspace: mi_gemm_tiled_workspace(M, K) bytes for the re-tiled activations.  The entry points
 * above take this route themselves for M > 64 (with the per-stream scratch buffer); the torch
 * ops pass a workspace from the caching allocator.  Reference: the M > 64 dispatch of
 * GEMM_fp8_pert_dispatch (V/csrc/xpu/esimd_kernels/fp8_GEMM_pert.h:4030-4075), the M >= 16 torch
 * route of the block-scaled linear (vllm/patches/vllm_for_multi_arc.patch:2671-2691) and the
 * M > 1 dense route of Q4_K (sglang/patches/sglang_for_multi_arc.patch:3211-3213). */
int mi_gemm_tiled_workspace(int M, int K, long long* bytes);
int mi_gemm_fp8_tiled_ws(const void* x, const void* w, const void* scale, int scale_mode, int scale_is_f16,
                         void* out, void* workspace, long long workspace_bytes, int M, int N, int K,
                         int act_dtype, void* stream);
int mi_gemm_q4k_tiled_ws(const void* x, const void* ql, const void* scale, const void* qmin, void* out,
                         void* workspace, long long workspace_bytes, int M, int N, int K, void* stream);

/* ---- MoE grouped FP8 block-scaled GEMM ----------------------------------------
 * out[r, :] = a[src(r), :] @ dequant(w[e])^T for the rows r of expert e,
 * expert_start[e] <= r < expert_start[e+1]; src(r) = row_map[r] if row_map else r.
 * w [E, N, K] e4m3, w_scale [E, ceil(N/128), K/128] fp32, K % 128 == 0.
 * a_scale == NULL: a is fp16/bf16 (w8a16) — replaces esimd_moe_gemm_fp8_blockscale
 *   (V/csrc/xpu/esimd_kernel_moe.sycl:201-269,
 *   V/csrc/xpu/esimd_kernels/fp8_moe_gemm_blockscale.h:123-334).
 * a_scale != NULL: a is e4m3 with per-row per-128 scales [a_rows, K/128]; native
 *   fp8 MFMA.  fuse_silu_mul: weight rows [0, N/2) are gate, [N/2, N) up; out is
 *   [total_rows, N/2] = silu(gate) * up.  Both have no reference counterpart.
 * out is in the activation dtype (out_f32 = 0), fp32 (1), or fp16 whatever the activation dtype (2:
 * values beyond the fp16 range saturate at +-65504). */
int mi_moe_gemm_fp8_block(const void* a, const float* a_scale, const int32_t* row_map, const void* w,
                          const float* w_scale, const int32_t* expert_start, void* out, int a_rows,
                          int total_rows, int E, int N, int K, int fuse_silu_mul, int act_dtype,
                          int out_f32, void* stream);
/* mi_moe_sort and the gate_up mi_moe_gemm_fp8_block (quantised activations, fused silu(gate) * up) in
 * one launch, for up to 8192 (token, route) pairs: every workgroup of an expert finds the expert's
 * pairs in top_ids [T, topk] itself (the same stable counting sort: lower experts' pairs first, pair
 * order inside an expert; ids outside [0, E) are held into the range) and gathers its rows of
 * a [T, K] e4m3 / a_scale [T, K/128] by token = pair / topk; out [T*topk, N/2] is in expert-sorted
 * order, and expert_start [E+1], inv [T*topk] and (optional) sorted_pairs [T*topk] are written as
 * mi_moe_sort writes them, for the stages that follow.  K % 128 == 0, K >= 256, (N/2) % 16 == 0;
 * MI_ERR_SHAPE beyond 8192 pairs (sort and GEMM are then two calls).  Takes the place of the
 * reference's scatter + grouped up GEMM sequence (V/csrc/xpu/esimd_kernels/moe_ops.h:437-569,
 * V/csrc/xpu/esimd_kernels/fp8_moe_gemm_blockscale.h:123-334). */
int mi_moe_gate_up_fp8_routed(const void* a, const float* a_scale, const int32_t* top_ids, int T, int topk,
                              const void* w, const float* w_scale, int32_t* expert_start, int32_t* inv,
                              int32_t* sorted_pairs, void* out, int E, int N, int K, int act_dtype,
                              void* stream);

/* Decode form of the same product for a handful of (token, expert) routes: one GEMV per route,
 * out[r, :] = (act(x[r / x_div, :]) @ dequant(w[e_r])^T) * route_weight[r], e_r = route_expert[r] (held
 * into [0, num_experts)); all routes in ONE launch of the row GEMV (a wavefront per weight row, routes
 * as the grid's second dimension), so each expert's weights stream at the full rate instead of
 * through the few workgroups a grouped launch has work for.  x [rows, K] and out [routes +
 * shared_rows, out_stride] in the activation type, w [E, N, K] e4m3 with 128 x 128 block scales
 * w_scale [E, ceil(N/128), K/128], route_weight (optional) in the activation type.
 * x_silu = 1: a row of x is 2 K wide, gate then up, and act(row) = silu(gate) * up rounded to the
 *   activation type (mi_moe_silu_mul fused into the staging of the row); 0: act is the identity.
 * shared_w / shared_scale (optional, one matrix [N, K] with its block scales): shared_rows further
 *   rows r = routes + i run against it -- the layer's shared expert in the same launch -- with
 *   activation row shared_x_first + i and no route weight.
 * K % 128 == 0; at most 65535 rows.  The small-batch form of moe_forward_full_fp8_block's expert loop
 * (V/csrc/moe_batch/moe.sycl:1509-1663: one work-item row per (token, route), the shared expert
 * beside them). */
int mi_moe_gemv_fp8_block_routed(const void* x, int x_div, int x_silu, const void* w, const float* w_scale,
                                 void* out, long long out_stride, const int32_t* route_expert,
                                 const void* route_weight, int routes, int num_experts, const void* shared_w,
                                 const float* shared_scale, int shared_rows, int shared_x_first, int N, int K,
                                 int act_dtype, void* stream);

/* The same GEMM with the per-expert-scalar scale of the reference's per-tensor MoE
 * kernels and their epilogues:
 *   scale_per_expert = 1: w_scale is [E] fp32 (one factor per expert); K may then be
 *     any multiple of 16 (the chunks of the last 128-granule past K read as zeros).
 *     scale_per_expert = 2: w_scale is [E, 2] fp32, the first factor for weight rows [0, N/2)
 *     and the second for rows [N/2, N) (the gate / up scales of the sglang prefill kernels,
 *     S/csrc/moe_prefill/moe_prefill_fp8.sycl:480-530); without fuse_act N/2 must be a multiple of 16.
 *     scale_per_expert = 0: block scales [E, ceil(N/128), ceil(K/128)] as above; with fuse_act
 *     N/2 must then be a multiple of 16 (a 16-row tile of the up half stays inside one block).
 *   row_map_div (>= 1): the source row of sorted position r is row_map[r] / row_map_div, so that a
 *     map of pair indices (token * top_k + slot) gathers token rows with row_map_div = top_k.
 *   fuse_act: 0 none, 1 silu(gate) * up, 2 gelu_tanh(gate) * up (exp argument held in
 *     [-30, 30]); gate = weight rows [0, N/2), up = rows [N/2, N); N/2 need not be a
 *     multiple of 128.
 *   out_map (optional, [total_rows] int32): the row of expert-sorted position r is
 *     written to out[out_map[r]] (the reference's kernels write pair order themselves);
 *   row_weight (optional, activation dtype, indexed by destination row): the row is
 *     multiplied by it before rounding (routing weight of the down projection).
 * Replaces moe_up_fp8_grouped_gelu_tanh_kernel / moe_down_fp8_grouped_kernel
 * (V/csrc/moe_batch/moe_fp8_grouped.h:98-245, :247-341), moe_up_routed_e4m3_gelu_tanh_kernel
 * / moe_down_routed_e4m3_vllm_layout_kernel (V/csrc/moe_batch/moe.sycl:458-558, :870-924)
 * and the scatter at the end of the sglang prefill kernels
 * (S/csrc/moe_prefill/moe_prefill_fp8.sycl:280-300, :385-411). */
int mi_moe_gemm_fp8_grouped(const void* a, const float* a_scale, const int32_t* row_map, int row_map_div,
                            const void* w, const float* w_scale, int scale_per_expert, const int32_t* expert_start, void* out,
                            const int32_t* out_map, const void* row_weight, int a_rows, int total_rows, int E,
                            int N, int K, int fuse_act, int act_dtype, int out_f32, void* stream);

/* ---- Decode MoE on K-major per-tensor FP8 expert weights --------------------------
 * The routed experts of the reference's per-tensor FP8 MoE decode op keep the reduction
 * index outermost: gate_up [E, H, 2I], down [E, I, H] e4m3, one fp32 scale per expert
 * (moe_forward_full, V/csrc/moe_batch/moe.sycl:1855-1940; kernels moe_up_routed_e4m3_kernel
 * :371-456, moe_down_routed_e4m3_kernel :815-868, moe_down_finalize_e4m3_kernel :1386-1421).
 * route r = t * top_k + j uses expert route_expert[r] and token t.
 * mi_moe_kmajor_up:   partial[r][s][:] = sum over split s's rows k of x[t][k] * W13[e][k][:]
 *                     (fp32 [routes, splits, 2I], unscaled); 2I % 32 == 0.
 * mi_moe_kmajor_down: inter[i] = act(s13[e] gate[i]) * (s13[e] up[i]) with gate / up summed over
 *                     the up partials in split order and the product rounded to the activation
 *                     type; partial[r][s][:] = sum over split s's rows i of inter[i] * W2[e][i][:]
 *                     (fp32 [routes, splits, H], unscaled); gelu = 0: SiLU, 1: tanh-GELU; H % 16 == 0.
 * mi_moe_kmajor_act:  inter[r][i] (activation type, [routes, I]) = the same act(..) * (..) product,
 *                     written out for a caller whose down projection is N-major
 *                     (moe_forward_full_silu_routed, S/csrc/moe_batch/moe.sycl:2022-2077: K-major
 *                     gate_up, [E, H, I] down).
 * mi_moe_kmajor_finalize: out[t][:] = sum_j top_w[t][j] * s2[e] * sum_s partial[r][s][:]
 *                     + gate[t] * shared[t][:] (shared / gate optional), rounded once.
 * `splits` (K split over workgroups, rows per split = ceil(K / splits) rounded up to 8, at most
 * 1024) is the caller's choice; a route whose expert id is outside [0, num_experts) contributes zeros: about two workgroups per compute unit over
 * routes * ceil(N / 1024) column blocks fills the device. */
int mi_moe_kmajor_up(const void* x, const void* w, const int32_t* route_expert, float* partial, int routes,
                     int top_k, int num_experts, int H, int two_i, int splits, int act_dtype, void* stream);
int mi_moe_kmajor_down(const float* up_partial, int up_splits, const float* up_scale, const void* w2,
                       const int32_t* route_expert, float* partial, int routes, int num_experts, int I, int H,
                       int splits, int gelu, int act_dtype, void* stream);
int mi_moe_kmajor_act(const float* up_partial, int up_splits, const float* up_scale, const int32_t* route_expert,
                      void* inter, int routes, int num_experts, int I, int gelu, int act_dtype, void* stream);
int mi_moe_kmajor_finalize(const float* partial, int splits, const float* down_scale, const int32_t* route_expert,
                           const void* top_w, const void* shared, const float* gate, void* out, int T, int top_k,
                           int num_experts, int H, int act_dtype, void* stream);

/* ---- 16-bit (unquantized) weight GEMV for the small projections beside the quantized ones
 * out[M, N] = x[M, K] @ w[N, K]^T, w in the activation type; K % 8 == 0.  gelu_mul = 1: w is
 * [2N, K] (gate rows first) and out = gelu_tanh(x @ gate^T) * (x @ up^T).
 * Replaces esimd_gemv_fp16 and esimd_gemv_fp16_gelu_mul (V/csrc/xpu/torch_extension.cc:27-34)
 * and the fp16 half of esimd_gemv_fp8_blockscale_fp16_fused2 (torch_extension_gemm.cc:37-41,
 * V/csrc/xpu/esimd_kernels/fp8_GEMM_blockscale.h:228-446). */
int mi_gemv_w16(const void* x, const void* w, void* out, int M, int N, int K, int gelu_mul, int act_dtype,
                void* stream);

/* ---- measurement yardstick -------------------------------------------------------------
 * No counterpart in the reference.  mi_stream_read fetches `bytes` (a multiple of 16, src 16-byte
 * aligned) from HBM with non-temporal 16-byte loads and keeps nothing: the time a kernel that
 * must read that many bytes cannot beat on this device, which the benchmark reports beside each
 * memory-bound configuration.  The fastest launch shape depends on the size, so the shapes are
 * numbered `variant`s in [0, mi_stream_read_variants()); the floor is the minimum over them.
 * `sink` must hold the number of 32-bit words mi_stream_read_sink_words returns (it is written
 * only if a lane's XOR hits one magic value). */
int mi_stream_read_variants(void);
int mi_stream_read_sink_words(long long* words);
int mi_stream_read(const void* src, long long bytes, unsigned int* sink, int variant, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_QLINEAR_H_ */
