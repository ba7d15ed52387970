// RMS norm (+ residual add, + SiLU gate) fused into the decode GEMV.
//
// One launch: every workgroup of the one-wavefront-per-row GEMV normalises the
// activation row itself while it stages it in LDS (the row is a few KiB and sits
// in L2), so the GEMV does not wait for a separate norm kernel.  The in-place
// residual update and the normalised row are written by the workgroup that
// arrives last at a device-wide counter: by then every workgroup holds its copy
// of the inputs in registers, so no workgroup can read a half-updated residual.
// Rows too long for the staging registers take the two-kernel route.
#include "gemv_rows.hpp"
#include "scratch.hpp"
#include "../../include/mi355x_qlinear.h"

#include <mutex>

using namespace qlin;

// ---- arrival counters that live in the library image ---------------------------
// mi_norm_gemv_static counts arriving workgroups in this array instead of a buffer
// from hipMalloc.  Every GPU the library runs on holds its own copy at its own
// address; host code never uses the name below as an address, only the per-device
// pointer that hipGetSymbolAddress returns.  The loader zero-fills it and the kernel
// leaves every counter at zero when it ends, so one call finds what the previous one
// left: zeros.  Calls that overlap on one GPU (two streams) would share the counters
// and race; calls on one stream are ordered by the stream.  So one stream per GPU owns the
// array: the first call after a set-up claims it for its stream, and a call on another
// stream is refused with MI_ERR_BUSY until mi_static_scratch_setup releases the claim.
constexpr int kStaticCounterWords = 512;                       // 2 KiB, the size the kernel indexes into
static __device__ __align__(256) unsigned int scratch[kStaticCounterWords];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_static_mu;
unsigned int* g_static_ptr[kMaxDevices];                       // per device, resolved once
hipStream_t g_static_owner[kMaxDevices];                       // the stream that claimed the array
bool g_static_owned[kMaxDevices];

// MI_OK and *out = the current device's copy of `scratch`; *dev_out = the device
int static_counters_locked(unsigned int** out, int* dev_out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) { (void)hipGetLastError(); return MI_ERR_LAUNCH; }
  if (!g_static_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) { (void)hipGetLastError(); return MI_ERR_LAUNCH; }
    g_static_ptr[dev] = static_cast<unsigned int*>(p);
  }
  *out = g_static_ptr[dev];
  *dev_out = dev;
  return MI_OK;
}

// Shared body.  counters == nullptr: take the per-stream counters (allocated on first use) and
// fall back to two kernels for rows the fused staging cannot hold; otherwise use `counters` and
// refuse those rows.
int norm_gemv_run(const void* x, void* residual, const void* gate, const void* norm_weight, void* normed_out,
                  int norm_len, float eps, float residual_scale, int fmt, int nmat, const void* const* w,
                  const void* const* scale, void* const* out, const int* N, int K, int act_dtype, void* stream,
                  unsigned int* counters);
}  // namespace

extern "C" {

int mi_static_scratch_setup(void) {
  unsigned int* p = nullptr;
  int dev = -1;
  std::lock_guard<std::mutex> lock(g_static_mu);
  const int rc = static_counters_locked(&p, &dev);
  if (rc != MI_OK) return rc;
  // back to the state the loader left: all counters zero (a kernel that ended abnormally may have
  // left some non-zero), nobody owns the array.  A blocking clear: not for use under capture.
  if (hipMemset(p, 0, sizeof(unsigned int) * kStaticCounterWords) != hipSuccess) { (void)hipGetLastError(); return MI_ERR_LAUNCH; }
  g_static_owned[dev] = false;
  return MI_OK;
}

int mi_norm_gemv_static(const void* x, void* residual, const void* gate, const void* norm_weight, void* normed_out,
                        int norm_len, float eps, float residual_scale, int fmt, int nmat, const void* const* w,
                        const void* const* scale, void* const* out, const int* N, int K, int act_dtype,
                        void* stream) {
  unsigned int* counters = nullptr;
  {
    int dev = -1;
    std::lock_guard<std::mutex> lock(g_static_mu);
    const int rc = static_counters_locked(&counters, &dev);
    if (rc != MI_OK) return rc;
    if (!g_static_owned[dev]) {
      g_static_owned[dev] = true;
      g_static_owner[dev] = (hipStream_t)stream;
    } else if (g_static_owner[dev] != (hipStream_t)stream) {
      return MI_ERR_BUSY;                  // another stream's calls could overlap with this one
    }
  }
  return norm_gemv_run(x, residual, gate, norm_weight, normed_out, norm_len, eps, residual_scale, fmt, nmat, w, scale,
                       out, N, K, act_dtype, stream, counters);
}

int mi_norm_gemv(const void* x, void* residual, const void* gate, const void* norm_weight, void* normed_out,
                 int norm_len, float eps, int fmt, int nmat, const void* const* w, const void* const* scale,
                 void* const* out, const int* N, int K, int act_dtype, void* stream) {
  return mi_norm_gemv_scaled(x, residual, gate, norm_weight, normed_out, norm_len, eps, 1.0f, fmt, nmat, w, scale, out,
                             N, K, act_dtype, stream);
}

int mi_norm_gemv_scaled(const void* x, void* residual, const void* gate, const void* norm_weight, void* normed_out,
                        int norm_len, float eps, float residual_scale, int fmt, int nmat, const void* const* w,
                        const void* const* scale, void* const* out, const int* N, int K, int act_dtype,
                        void* stream) {
  return norm_gemv_run(x, residual, gate, norm_weight, normed_out, norm_len, eps, residual_scale, fmt, nmat, w, scale,
                       out, N, K, act_dtype, stream, nullptr);
}

}  // extern "C"

namespace {

int norm_gemv_run(const void* x, void* residual, const void* gate, const void* norm_weight, void* normed_out,
                  int norm_len, float eps, float residual_scale, int fmt, int nmat, const void* const* w,
                  const void* const* scale, void* const* out, const int* N, int K, int act_dtype, void* stream,
                  unsigned int* counters) {
  if (!x || !norm_weight || !w || !scale || !out || !N) return MI_ERR_ARG;
  if (nmat < 1 || nmat > kRowsMaxMat) return MI_ERR_ARG;
  if (act_dtype != DT_F16 && act_dtype != DT_BF16) return MI_ERR_ARG;
  if (fmt < 0 || fmt > 2) return MI_ERR_ARG;
  if (K <= 0 || norm_len <= 0 || (norm_len % 8) || (K % norm_len)) return MI_ERR_SHAPE;
  if (fmt == 0 ? (K % 16) : (K % 128)) return MI_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  RowsArgs r{};
  r.x = x; r.nmat = nmat; r.M = 1; r.K = K; r.scale_f16 = 0;
  for (int i = 0; i < nmat; ++i) {
    if (!w[i] || !scale[i] || !out[i] || N[i] < 0) return MI_ERR_ARG;
    if ((uint64_t)N[i] * (uint64_t)K >= (1ull << 31)) return MI_ERR_SHAPE;
    r.w[i] = w[i]; r.s[i] = scale[i]; r.out[i] = out[i]; r.N[i] = N[i];
  }
  const int rfmt = fmt == 2 ? RF_INT4 : RF_FP8;
  const bool fused = K <= kRowsNormMaxK && rows_lds_bytes(rfmt, 1, K) + rows_norm_lds_bytes(K) <= 64 * 1024;
  if (!fused && counters) return MI_ERR_LIMIT;          // the no-allocation entry covers the fused launch only
  if (!fused) {
    // two kernels: the norm writes the row (into normed_out, or over x's scratch copy), then the GEMV
    if (!normed_out) return MI_ERR_ARG;
    const int rc = mi_rmsnorm(x, residual, gate, norm_weight, normed_out, K / norm_len, norm_len, norm_len, eps,
                              act_dtype, residual_scale, stream);
    if (rc != MI_OK) return rc;
    const float* const* fs = reinterpret_cast<const float* const*>(scale);
    if (fmt == 0) return mi_gemm_fp8_pert_multi(normed_out, nmat, w, fs, out, N, 1, K, act_dtype, stream);
    if (fmt == 1) return mi_gemm_fp8_blockscale_multi(normed_out, nmat, w, fs, out, N, 1, K, act_dtype, stream);
    return mi_gemv_int4_multi(normed_out, nmat, w, scale, nullptr, out, N, 1, K, act_dtype, stream);
  }
  r.n_res = residual; r.n_gate = gate; r.n_weight = norm_weight; r.n_out = normed_out;
  r.n_len = norm_len; r.n_eps = eps; r.n_rscale = residual_scale;
  r.n_arrive = counters ? counters : arrival_counter_get(st);
  if (!r.n_arrive) return MI_ERR_LAUNCH;
  const bool f16 = act_dtype == DT_F16;
  if (fmt == 0) {
    if (f16) launch_rows_norm<ActF16, RF_FP8, RS_PERT>(r, st); else launch_rows_norm<ActBF16, RF_FP8, RS_PERT>(r, st);
  } else if (fmt == 1) {
    if (f16) launch_rows_norm<ActF16, RF_FP8, RS_BLOCK>(r, st); else launch_rows_norm<ActBF16, RF_FP8, RS_BLOCK>(r, st);
  } else {
    if (f16) launch_rows_norm<ActF16, RF_INT4, RS_PERN>(r, st); else launch_rows_norm<ActBF16, RF_INT4, RS_PERN>(r, st);
  }
  return launch_status();
}

}  // namespace
