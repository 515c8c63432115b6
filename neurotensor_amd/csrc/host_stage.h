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

    // ---- pipelined form, for calls whose operands cross the link in panels (uploads, products and downloads overlapping) ----
    // begin_uploads: every range of the call, in the order in which they are needed, each tagged with the panel it belongs
    // to (tags ascending).  Helper threads stage them slice by slice -- each takes the next slice, copies it into a pinned
    // buffer of its own and enqueues the device copy on stream() -- while the caller goes on; no thread waits for another.
    // uploaded_through(tag): returns once every slice of the panels up to `tag` has been enqueued, and makes
    // compute_stream() wait for them.  end_uploads(): all helpers done; reports the first error.
    struct Range { size_t dev_off; const void* src; size_t bytes; int tag; };
    hipError_t begin_uploads(const Range* ranges, size_t count, int tags);
    hipError_t uploaded_through(int tag);
    hipError_t end_uploads();
    // the stream for the panels' products, so that a panel's kernel does not hold up the next panel's uploads on stream()
    hipStream_t compute_stream() const { return compute_; }
    // download: arena -> host after everything enqueued on `after` so far (nullptr: stream()), carried out by a helper
    // thread on a third stream with pinned buffers and copy threads of its own, while the caller goes on (the link is
    // full duplex).  dst holds the bytes once finish_downloads() has returned, which also reports the first error.
    hipError_t download_async(void* dst, size_t dev_off, size_t bytes, hipStream_t after = nullptr);
    hipError_t finish_downloads();

    // true when the `bytes` bytes at p are all zero (several threads; stops at the first non-zero word)
    static bool all_zero(const void* p, size_t bytes);

    // frees the arena, the pinned buffers and the stream of every device (helper threads stay); for tests and for
    // callers that want the memory back
    static void release_all();

    struct State;

private:
    struct Downloader;
    struct Uploader;
    State* st_;
    char* arena_;
    hipStream_t stream_;
    bool dirty_;
    Downloader* dl_;
    Uploader* ul_;
    int device_;
    hipStream_t compute_;
    size_t events_used_;
};

}  // namespace ntg
