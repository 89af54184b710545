// A small pool of host threads for the CPU side of the host-buffer path: copies between the caller's
// (pageable) buffers and the library's pinned staging buffers, and the change detection of the C++ layer.
// One pool per process, created at first use; the calling thread always takes a share of the work itself.
#pragma once
#include <stddef.h>

#include <functional>

namespace pimdl {

class HostPool {
public:
    // number of pieces a job is cut into (worker threads + the caller)
    virtual int width() const = 0;
    // runs fn(piece) for piece = 0 .. pieces-1 on the pool and the calling thread; returns when all are done.
    // One job at a time: concurrent callers take turns.
    virtual void run(int pieces, const std::function<void(int)>& fn) = 0;
    virtual ~HostPool() {}
};

// The process-wide pool.  PIMDL_COPY_THREADS sets its width (default 8, at most the hardware's concurrency: measured
// over several hosts, four threads are within 5 % of the best on some and 30 % behind on others, eight within 5 %
// everywhere, sixteen on a 16-CPU share much slower).
HostPool& host_pool();

// memcpy cut into cache-line aligned pieces over the pool, with streaming stores (PIMDL_COPY_MODE: 0 plain memcpy,
// 1 SSE2 streaming stores -- the default --, 2 AVX2); small copies stay on the calling thread
void parallel_copy(void* dst, const void* src, size_t bytes);

}  // namespace pimdl
