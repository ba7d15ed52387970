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

// One pool of counter blocks per device, handed out to streams in order: only the first call on a
// device allocates (and clears) anything, so a stream first seen while it is being captured still
// gets its block without an allocation.
namespace {
constexpr int kCounterBlockBytes = 2048;
constexpr int kCounterBlocksPerPool = 64;
struct CounterPool {
  unsigned char* base = nullptr;
  int used = 0;
};
std::map<int, CounterPool> g_pools;
}  // namespace

unsigned int* arrival_counter_get(hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
  std::lock_guard<std::mutex> lock(g_mu);
  unsigned int*& c = g_counters[{dev, stream}];
  if (c) return c;
  CounterPool& pool = g_pools[dev];
  if (!pool.base || pool.used == kCounterBlocksPerPool) {
    // a fresh pool (the exhausted one stays allocated: its blocks are in use)
    void* p = nullptr;
    const size_t bytes = (size_t)kCounterBlockBytes * kCounterBlocksPerPool;
    if (hipMalloc(&p, bytes) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    if (hipMemset(p, 0, bytes) != hipSuccess) { (void)hipGetLastError(); (void)hipFree(p); return nullptr; }
    pool.base = static_cast<unsigned char*>(p);
    pool.used = 0;
  }
  c = reinterpret_cast<unsigned int*>(pool.base + (size_t)kCounterBlockBytes * pool.used++);
  return c;
}

}  // namespace qlin
