// Grow-only device scratch, one buffer per (device, stream).
//
// Some entry points need a little device memory beyond their operands (the
// activations re-tiled into MFMA operand order).  The reference's launchers keep
// such scratch in thread-local, only-growing buffers keyed per (device, queue) so
// that addresses baked into a captured graph stay valid
// (V/csrc/xpu/esimd_kernel_moe.sycl:45-67, V/csrc/moe_batch/moe.sycl:1460-1498);
// this is the same convention.  A buffer that has become too small is replaced by
// a larger one and kept allocated until the process ends: work already queued on
// the stream may still read it, and a graph captured earlier has its address baked
// in, so no later point is safe for freeing it.  Sizes grow in powers of two, so
// the replaced buffers of a stream add up to less than the one in use.  Growing calls hipMalloc, which is not allowed
// while the stream is being captured: run a call of the same size once before
// capturing, as graph users do anyway.  Calls on different streams never share a
// buffer; calls on one stream are ordered by the stream.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace qlin {

// nullptr when the allocation fails (e.g. under stream capture)
void* scratch_get(hipStream_t stream, size_t bytes);

// A zero-initialised block of 512 32-bit counters per (device, stream) for kernels that
// count arriving workgroups and leave the counters at zero again when they finish.  The
// blocks come from a pool of 64 that the first call on a device allocates and clears (not
// possible under stream capture); later streams take the next block without allocating.
// nullptr on failure.
unsigned int* arrival_counter_get(hipStream_t stream);

}  // namespace qlin
