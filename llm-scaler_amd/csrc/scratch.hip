#include "scratch.hpp"

#include <map>
#include <mutex>
#include <utility>

namespace qlin {

namespace {
struct Buf {
  void* p = nullptr;
  size_t bytes = 0;
};
std::mutex g_mu;
std::map<std::pair<int, hipStream_t>, Buf> g_bufs;
std::map<std::pair<int, hipStream_t>, unsigned int*> g_counters;
}  // namespace

void* scratch_get(hipStream_t stream, size_t bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  std::lock_guard<std::mutex> lock(g_mu);
  Buf& b = g_bufs[{dev, stream}];
  if (b.bytes >= bytes && b.p) return b.p;
  size_t want = 1u << 20;                             // at least 1 MiB, then powers of two
  while (want < bytes) want <<= 1;
  void* p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  // the old buffer stays allocated: kernels already queued may still use it
  b.p = p;
  b.bytes = want;
  return p;
}

unsigned int* arrival_counter_get(hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  std::lock_guard<std::mutex> lock(g_mu);
  unsigned int*& c = g_counters[{dev, stream}];
  if (c) return c;
  void* p = nullptr;
  if (hipMalloc(&p, 2048) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  if (hipMemset(p, 0, 2048) != hipSuccess) { (void)hipGetLastError(); (void)hipFree(p); return nullptr; }
  c = static_cast<unsigned int*>(p);
  return c;
}

}  // namespace qlin
