#include "gguf_skinny.hpp"
#include "skinny_kernel.hpp"
#include "kslice_kernel.hpp"
#include "../../include/mi355x_qlinear.h"

namespace qlin {

template <int FMT>
static int gguf_skinny_fmt(SkinnyArgs a, hipStream_t st) {
  const int M = a.M;
  for (int m0 = 0; m0 < M; m0 += 64) {
    SkinnyArgs c = a;
    c.M = (M - m0) < 64 ? (M - m0) : 64;
    c.x = (const char*)a.x + (size_t)m0 * a.K * 2;
    c.out[0] = (char*)a.out[0] + (size_t)m0 * a.N[0] * 2;
    int rc;
    int nq = 0;
    if constexpr (FMT == 3 || FMT == 4) nq = kslice_loads(c.M, c.K, FMT);   // few rows: x resident in registers
    if constexpr (FMT == 3 || FMT == 4) rc = nq ? kslice_launch<ActF16, FMT>(c, 0, nq, st) : launch_mt<ActF16, FMT, 0>(c, st);
    else rc = launch_mt<ActF16, FMT, 0>(c, st);
    if (rc != MI_OK) return rc;
  }
  return MI_OK;
}

bool gguf_skinny_resident(int fmt, int M, int K) { return (fmt == 3 || fmt == 4) && kslice_loads(M, K, fmt) != 0; }

int gguf_skinny(int fmt, const void* x, const void* w, const void* h, const void* s, const void* z, void* out,
                int M, int N, int K, hipStream_t st) {
  SkinnyArgs a{};
  a.x = x; a.w[0] = w; a.h[0] = h; a.s[0] = s; a.z[0] = z; a.out[0] = out; a.N[0] = N; a.nmat = 1; a.M = M; a.K = K;
  a.tiles[0] = (N + 15) / 16;
  switch (fmt) {
    case 3: return gguf_skinny_fmt<3>(a, st);
    case 4: return gguf_skinny_fmt<4>(a, st);
    case 5: return gguf_skinny_fmt<5>(a, st);
    case 6: return gguf_skinny_fmt<6>(a, st);
    default: return MI_ERR_ARG;
  }
}

}  // namespace qlin
