// Staging of the host-pointer entry points: grow-only device arena, pinned chunk ring, private stream, copy threads.
#include "host_stage.h"

#include <algorithm>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <map>
#include <mutex>
#include <thread>
#include <vector>

namespace ntg {

namespace {

// CPU copies between pageable and pinned memory on a few threads.  One copy at a time (the lease serialises callers).
class CopyPool {
public:
    static CopyPool& get() {
        static CopyPool* pool = new CopyPool();      // never destroyed: its threads sleep until the process ends
        return *pool;
    }
    void copy(void* dst, const void* src, size_t n) {
        if (n < (size_t)(1 << 20) || helpers_ == 0) { std::memcpy(dst, src, n); return; }
        const int parts = helpers_ + 1;
        const size_t slice = ((n + parts - 1) / parts + 4095) / 4096 * 4096;
        {
            std::lock_guard<std::mutex> l(m_);
            for (int i = 0; i < helpers_; ++i) {
                const size_t b = std::min(n, slice * (size_t)(i + 1)), e = std::min(n, slice * (size_t)(i + 2));
                jobs_[i] = Job{static_cast<char*>(dst) + b, static_cast<const char*>(src) + b, e - b};
            }
            pending_ = helpers_;
            ++generation_;
        }
        cv_work_.notify_all();
        std::memcpy(dst, src, std::min(n, slice));
        std::unique_lock<std::mutex> l(m_);
        cv_done_.wait(l, [&] { return pending_ == 0; });
    }

private:
    struct Job { char* d; const char* s; size_t n; };
    CopyPool() {
        const unsigned hw = std::thread::hardware_concurrency();
        helpers_ = hw >= 8 ? 3 : hw >= 4 ? 2 : hw >= 2 ? 1 : 0;
        jobs_.resize((size_t)helpers_);
        for (int i = 0; i < helpers_; ++i) std::thread([this, i] { run(i); }).detach();
    }
    void run(int idx) {
        unsigned seen = 0;
        for (;;) {
            Job j;
            {
                std::unique_lock<std::mutex> l(m_);
                cv_work_.wait(l, [&] { return generation_ != seen; });
                seen = generation_;
                j = jobs_[(size_t)idx];
            }
            if (j.n) std::memcpy(j.d, j.s, j.n);
            std::lock_guard<std::mutex> l(m_);
            if (--pending_ == 0) cv_done_.notify_one();
        }
    }
    std::mutex m_;
    std::condition_variable cv_work_, cv_done_;
    std::vector<Job> jobs_;
    unsigned generation_ = 0;
    int pending_ = 0, helpers_ = 0;
};

constexpr int kBuffers = 4;
constexpr size_t kChunk = (size_t)8 << 20;

std::mutex g_lease;

}  // namespace

struct HostSession::State {
    char* arena = nullptr;
    size_t arena_cap = 0;
    hipStream_t stream = nullptr;
    char* pin[kBuffers] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t ev[kBuffers] = {nullptr, nullptr, nullptr, nullptr};
    bool busy[kBuffers] = {false, false, false, false};
    int next = 0;

    hipError_t ready() {
        if (!stream) {
            hipError_t e = hipStreamCreateWithFlags(&stream, hipStreamNonBlocking);
            if (e != hipSuccess) { stream = nullptr; return e; }
        }
        for (int b = 0; b < kBuffers; ++b) {
            if (!pin[b]) {
                hipError_t e = hipHostMalloc(reinterpret_cast<void**>(&pin[b]), kChunk, hipHostMallocDefault);
                if (e != hipSuccess) { pin[b] = nullptr; return e; }
            }
            if (!ev[b]) {
                hipError_t e = hipEventCreateWithFlags(&ev[b], hipEventDisableTiming);
                if (e != hipSuccess) { ev[b] = nullptr; return e; }
            }
        }
        return hipSuccess;
    }
    // the next staging buffer, free of earlier transfers
    hipError_t acquire(int& b) {
        b = next;
        next = (next + 1) % kBuffers;
        if (busy[b]) {
            hipError_t e = hipEventSynchronize(ev[b]);
            if (e != hipSuccess) return e;
            busy[b] = false;
        }
        return hipSuccess;
    }
    void free_all() {
        if (stream) (void)hipStreamSynchronize(stream);
        if (arena) (void)hipFree(arena);
        arena = nullptr;
        arena_cap = 0;
        for (int b = 0; b < kBuffers; ++b) {
            if (pin[b]) (void)hipHostFree(pin[b]);
            if (ev[b]) (void)hipEventDestroy(ev[b]);
            pin[b] = nullptr; ev[b] = nullptr; busy[b] = false;
        }
        if (stream) (void)hipStreamDestroy(stream);
        stream = nullptr;
    }
};

namespace {
std::map<int, HostSession::State*>& states() {
    static std::map<int, HostSession::State*>* m = new std::map<int, HostSession::State*>();
    return *m;
}
}  // namespace

HostSession::HostSession() : st_(nullptr), arena_(nullptr), stream_(nullptr), dirty_(false) {
    g_lease.lock();
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0) return;         // reserve() reports the failure
    State*& s = states()[dev];
    if (!s) s = new State();
    st_ = s;
}

HostSession::~HostSession() {
    if (st_ && dirty_ && st_->stream) {
        (void)hipStreamSynchronize(st_->stream);
        for (int b = 0; b < kBuffers; ++b) st_->busy[b] = false;
    }
    g_lease.unlock();
}

hipError_t HostSession::reserve(size_t bytes) {
    if (!st_) {
        int n = 0;
        const hipError_t e = hipGetDeviceCount(&n);
        return e != hipSuccess ? e : hipErrorNoDevice;
    }
    hipError_t e = st_->ready();
    if (e != hipSuccess) return e;
    if (bytes > st_->arena_cap) {
        if (st_->arena) {
            e = hipStreamSynchronize(st_->stream);
            if (e != hipSuccess) return e;
            (void)hipFree(st_->arena);
            st_->arena = nullptr;
            st_->arena_cap = 0;
        }
        const size_t want = (bytes + ((size_t)1 << 20) - 1) >> 20 << 20;      // whole MiB
        void* p = nullptr;
        e = hipMalloc(&p, want);
        if (e != hipSuccess) return e;
        st_->arena = static_cast<char*>(p);
        st_->arena_cap = want;
    }
    arena_ = st_->arena;
    stream_ = st_->stream;
    return hipSuccess;
}

hipError_t HostSession::upload(size_t dev_off, const void* src, size_t bytes) {
    if (!st_ || !arena_) return hipErrorNotInitialized;
    const char* s = static_cast<const char*>(src);
    for (size_t off = 0; off < bytes; off += kChunk) {
        const size_t len = std::min(kChunk, bytes - off);
        int b;
        hipError_t e = st_->acquire(b);
        if (e != hipSuccess) return e;
        CopyPool::get().copy(st_->pin[b], s + off, len);
        dirty_ = true;
        e = hipMemcpyAsync(arena_ + dev_off + off, st_->pin[b], len, hipMemcpyHostToDevice, stream_);
        if (e != hipSuccess) return e;
        e = hipEventRecord(st_->ev[b], stream_);
        if (e != hipSuccess) return e;
        st_->busy[b] = true;
    }
    return hipSuccess;
}

hipError_t HostSession::download(void* dst, size_t dev_off, size_t bytes) {
    if (!st_ || !arena_) return hipErrorNotInitialized;
    struct Piece { int b; size_t off, len; };
    std::deque<Piece> flight;
    char* d = static_cast<char*>(dst);
    auto drain = [&]() -> hipError_t {
        const Piece p = flight.front();
        flight.pop_front();
        const hipError_t e = hipEventSynchronize(st_->ev[p.b]);
        if (e != hipSuccess) return e;
        st_->busy[p.b] = false;
        CopyPool::get().copy(d + p.off, st_->pin[p.b], p.len);
        return hipSuccess;
    };
    for (size_t off = 0; off < bytes; off += kChunk) {
        const size_t len = std::min(kChunk, bytes - off);
        while ((int)flight.size() >= kBuffers - 1) {              // the ring's next buffer is never one in flight here
            const hipError_t e = drain();
            if (e != hipSuccess) return e;
        }
        int b;
        hipError_t e = st_->acquire(b);
        if (e != hipSuccess) return e;
        dirty_ = true;
        e = hipMemcpyAsync(st_->pin[b], arena_ + dev_off + off, len, hipMemcpyDeviceToHost, stream_);
        if (e != hipSuccess) return e;
        e = hipEventRecord(st_->ev[b], stream_);
        if (e != hipSuccess) return e;
        st_->busy[b] = true;
        flight.push_back(Piece{b, off, len});
    }
    while (!flight.empty()) {
        const hipError_t e = drain();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t HostSession::sync() {
    if (!st_ || !st_->stream) return hipSuccess;
    const hipError_t e = hipStreamSynchronize(st_->stream);
    if (e == hipSuccess) {
        for (int b = 0; b < kBuffers; ++b) st_->busy[b] = false;
        dirty_ = false;
    }
    return e;
}

void HostSession::release_all() {
    std::lock_guard<std::mutex> l(g_lease);
    for (auto& kv : states()) {
        int cur = -1;
        (void)hipGetDevice(&cur);
        if (cur != kv.first) (void)hipSetDevice(kv.first);
        kv.second->free_all();
        if (cur != kv.first && cur >= 0) (void)hipSetDevice(cur);
    }
}

}  // namespace ntg
