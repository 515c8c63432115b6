// Staging for the host-pointer entry points (the nt_matmult<T> drop-in seam: the caller's matrices live in ordinary
// pageable host memory, nt/functional/cpu/matmult_cpu.cpp:118, :150, :740, :851).
//
// One HostSession per call.  It leases the process-wide staging state of the current device:
//   * a device arena that only grows (no hipMalloc / hipFree per call once it has reached the working-set size),
//   * a ring of pinned staging buffers (hipHostMalloc) and a private stream: a transfer is cut into chunks, the CPU
//     copies chunk i + 1 between the caller's memory and a pinned buffer (several threads: one core moves ~30 GB/s,
//     the link ~57 GB/s) while the DMA engine moves chunk i,
//   * a few helper threads for those CPU copies.
// Concurrent callers are serialised on the lease (the reference's kernel layer is not re-entrant per dtype at all:
// static pack buffers, nt/functional/cpu/matmult/nt_matmult_blocks.h:12-16).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace ntg {

class HostSession {
public:
    HostSession();
    ~HostSession();                       // waits for the stream if work may still be in flight, then releases the lease
    HostSession(const HostSession&) = delete;
    HostSession& operator=(const HostSession&) = delete;

    // device arena of at least `bytes` bytes, 256-byte aligned; contents are undefined
    hipError_t reserve(size_t bytes);
    char* at(size_t off) const { return arena_ + off; }
    hipStream_t stream() const { return stream_; }

    // host -> arena.  On return the caller's bytes have been read (they may change); the device copy is ordered on stream().
    hipError_t upload(size_t dev_off, const void* src, size_t bytes);
    // arena -> host, after everything enqueued on stream() so far.  On return dst holds the bytes.
    hipError_t download(void* dst, size_t dev_off, size_t bytes);
    hipError_t sync();

    // frees the arena, the pinned buffers and the stream of every device (helper threads stay); for tests and for
    // callers that want the memory back
    static void release_all();

    struct State;

private:
    State* st_;
    char* arena_;
    hipStream_t stream_;
    bool dirty_;
};

}  // namespace ntg
