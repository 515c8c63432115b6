// Staging of the host-pointer entry points: grow-only device arena, pinned chunk ring, private stream, copy threads.
#include "host_stage.h"

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <functional>
#include <map>
#include <mutex>
#include <thread>
#include <vector>

namespace ntg {

namespace {

// CPU copies between pageable and pinned memory on a few threads.  One copy at a time (the lease serialises callers).
// all bytes zero?  (8 bytes at a time, leaves at the first non-zero word or when another thread has found one)
static bool span_is_zero(const char* p, size_t n, const std::atomic<bool>* found) {
    size_t i = 0;
    for (; i < n && (reinterpret_cast<uintptr_t>(p + i) & 7) != 0; ++i)
        if (p[i]) return false;
    const uint64_t* w = reinterpret_cast<const uint64_t*>(p + i);
    const size_t words = (n - i) / 8;
    for (size_t j = 0; j < words; j += 512) {
        uint64_t acc = 0;
        const size_t e = std::min(words, j + 512);
        for (size_t q = j; q < e; ++q) acc |= w[q];
        if (acc) return false;
        if (found && found->load(std::memory_order_relaxed)) return false;
    }
    for (i += words * 8; i < n; ++i)
        if (p[i]) return false;
    return true;
}

// Threads that run one function each and sleep between jobs: the stagers of a pipelined call's uploads.
class WorkerSet {
public:
    static WorkerSet& stagers() {
        static WorkerSet* w = new WorkerSet();       // never destroyed
        return *w;
    }
    int size() const { return n_; }
    void start(const std::function<void(int)>* fn) {
        {
            std::lock_guard<std::mutex> l(m_);
            fn_ = fn;
            pending_ = n_;
            ++generation_;
        }
        cv_work_.notify_all();
    }
    void join() {
        std::unique_lock<std::mutex> l(m_);
        cv_done_.wait(l, [&] { return pending_ == 0; });
        fn_ = nullptr;
    }

private:
    WorkerSet() {
        const unsigned hw = std::thread::hardware_concurrency();
        n_ = hw >= 16 ? 5 : hw >= 8 ? 3 : hw >= 4 ? 2 : 1;
        for (int i = 0; i < n_; ++i) std::thread([this, i] { loop(i); }).detach();
    }
    void loop(int idx) {
        unsigned seen = 0;
        for (;;) {
            const std::function<void(int)>* fn;
            {
                std::unique_lock<std::mutex> l(m_);
                cv_work_.wait(l, [&] { return generation_ != seen; });
                seen = generation_;
                fn = fn_;
            }
            (*fn)(idx);
            std::lock_guard<std::mutex> l(m_);
            if (--pending_ == 0) cv_done_.notify_all();
        }
    }
    std::mutex m_;
    std::condition_variable cv_work_, cv_done_;
    const std::function<void(int)>* fn_ = nullptr;
    unsigned generation_ = 0;
    int pending_ = 0, n_ = 0;
};

class CopyPool {
public:
    static CopyPool& get() {
        static CopyPool* pool = new CopyPool();      // never destroyed: its threads sleep until the process ends
        return *pool;
    }
    static CopyPool& down() {                         // the downloader thread's helpers
        static CopyPool* pool = new CopyPool();
        return *pool;
    }
    bool all_zero(const void* p, size_t n) {
        nonzero_.store(false);
        scan_ = true;
        copy(nullptr, p, n);
        scan_ = false;
        return !nonzero_.load();
    }
    void copy(void* dst, const void* src, size_t n) {
        if (n < (size_t)(1 << 20) || helpers_ == 0) { work(static_cast<char*>(dst), static_cast<const char*>(src), n); return; }
        const int parts = helpers_ + 1;
        const size_t slice = ((n + parts - 1) / parts + 4095) / 4096 * 4096;
        {
            std::lock_guard<std::mutex> l(m_);
            for (int i = 0; i < helpers_; ++i) {
                const size_t b = std::min(n, slice * (size_t)(i + 1)), e = std::min(n, slice * (size_t)(i + 2));
                jobs_[i] = Job{dst ? static_cast<char*>(dst) + b : nullptr, static_cast<const char*>(src) + b, e - b};
            }
            pending_ = helpers_;
            ++generation_;
        }
        cv_work_.notify_all();
        work(static_cast<char*>(dst), static_cast<const char*>(src), std::min(n, slice));
        std::unique_lock<std::mutex> l(m_);
        cv_done_.wait(l, [&] { return pending_ == 0; });
    }

private:
    struct Job { char* d; const char* s; size_t n; };
    // (scan mode: no copy, the bytes at s are tested for zero)
    void work(char* d, const char* s, size_t n) {
        if (!n) return;
        if (!scan_) std::memcpy(d, s, n);
        else if (!span_is_zero(s, n, &nonzero_)) nonzero_.store(true);
    }
    std::atomic<bool> nonzero_{false};
    bool scan_ = false;
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
            work(j.d, j.s, j.n);
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
constexpr int kSegBufs = 4;
constexpr size_t kSegment = (size_t)16 << 20;    // pipelined uploads: bytes per device copy (one pinned buffer) ...
constexpr size_t kSlice = (size_t)1 << 20;       // ... and what one stager copies into it at a time

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
    // pipelined calls: pinned buffers and events of the stagers; the downloads' stream, buffers and events; the stream of
    // the panels' products; events that order the three streams
    char* spin[kSegBufs] = {};
    hipEvent_t sev[kSegBufs] = {};
    std::atomic<int> sbusy[kSegBufs] = {};           // a device copy out of the buffer has been enqueued since the stream was last waited for
    hipStream_t down_stream = nullptr, compute_stream = nullptr;
    char* dpin[kBuffers] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t dev_[kBuffers] = {nullptr, nullptr, nullptr, nullptr};
    std::vector<hipEvent_t> order_events;

    hipError_t ready_pipeline(int stagers) {
        for (hipStream_t* sp : {&down_stream, &compute_stream})
            if (!*sp) {
                hipError_t e = hipStreamCreateWithFlags(sp, hipStreamNonBlocking);
                if (e != hipSuccess) { *sp = nullptr; return e; }
            }
        for (int b = 0; b < kBuffers; ++b) {
            if (!dpin[b]) {
                hipError_t e = hipHostMalloc(reinterpret_cast<void**>(&dpin[b]), kChunk, hipHostMallocDefault);
                if (e != hipSuccess) { dpin[b] = nullptr; return e; }
            }
            if (!dev_[b]) {
                hipError_t e = hipEventCreateWithFlags(&dev_[b], hipEventDisableTiming);
                if (e != hipSuccess) { dev_[b] = nullptr; return e; }
            }
        }
        for (int b = 0; b < kSegBufs && stagers > 0; ++b) {
            if (!spin[b]) {
                hipError_t e = hipHostMalloc(reinterpret_cast<void**>(&spin[b]), kSegment, hipHostMallocDefault);
                if (e != hipSuccess) { spin[b] = nullptr; return e; }
            }
            if (!sev[b]) {
                hipError_t e = hipEventCreateWithFlags(&sev[b], hipEventDisableTiming);
                if (e != hipSuccess) { sev[b] = nullptr; return e; }
            }
        }
        return hipSuccess;
    }
    hipError_t order_event(size_t i, hipEvent_t& out) {
        while (order_events.size() <= i) {
            hipEvent_t ev = nullptr;
            hipError_t e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
            if (e != hipSuccess) return e;
            order_events.push_back(ev);
        }
        out = order_events[i];
        return hipSuccess;
    }

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
        for (hipStream_t* sp : {&down_stream, &compute_stream})
            if (*sp) { (void)hipStreamSynchronize(*sp); (void)hipStreamDestroy(*sp); *sp = nullptr; }
        for (int b = 0; b < kBuffers; ++b) {
            if (dpin[b]) (void)hipHostFree(dpin[b]);
            if (dev_[b]) (void)hipEventDestroy(dev_[b]);
            dpin[b] = nullptr; dev_[b] = nullptr;
        }
        for (int b = 0; b < kSegBufs; ++b) {
            if (spin[b]) (void)hipHostFree(spin[b]);
            if (sev[b]) (void)hipEventDestroy(sev[b]);
            spin[b] = nullptr; sev[b] = nullptr; sbusy[b].store(0);
        }
        for (hipEvent_t ev : order_events) (void)hipEventDestroy(ev);
        order_events.clear();
    }
};

// The uploads of a pipelined call.  The DMA engine wants large pieces (192 MiB in 2 MiB copies: 22 - 40 GB/s, in 8 MiB
// copies 53, in one 57), a CPU thread copies about 30 GB/s: so the ranges are cut into segments of up to kSegment bytes, each
// staged into one pinned buffer by all stagers together -- they take its 1 MiB slices through one counter -- and whoever
// copies a segment's last slice enqueues its one device copy.  Nobody waits for a segment to finish: the stagers are
// already on the next one (a ring of kSegBufs buffers; a buffer is reused once the event behind its device copy has come).
struct HostSession::Uploader {
    struct Segment { char* dst; const char* src; size_t len; int tag; size_t first_slice; std::atomic<int> left{0}, ready{0}, enqueued{0}; };
    std::deque<Segment> segments;                  // (deque: atomics do not move)
    std::vector<size_t> slice_segment;             // slice -> segment
    std::vector<std::atomic<int>> left;            // per tag: segments not yet enqueued
    std::atomic<size_t> next{0};
    std::atomic<int> error{(int)hipSuccess};
    State* st;
    hipStream_t stream;
    int device;
    std::function<void(int)> fn;

    Uploader(State* s, hipStream_t str, int dev, int tags) : left((size_t)tags), st(s), stream(str), device(dev) {
        for (auto& l : left) l.store(0);
        fn = [this](int) { stage(); };
    }
    void add(char* dst, const char* src, size_t bytes, int tag) {
        for (size_t off = 0; off < bytes; off += kSegment) {
            const size_t len = std::min(kSegment, bytes - off), g = segments.size();
            segments.emplace_back();
            Segment& sg = segments.back();
            sg.dst = dst + off; sg.src = src + off; sg.len = len; sg.tag = tag; sg.first_slice = slice_segment.size();
            const size_t n = (len + kSlice - 1) / kSlice;
            sg.left.store((int)n);
            for (size_t i = 0; i < n; ++i) slice_segment.push_back(g);
            left[(size_t)tag].fetch_add(1);
        }
    }
    void stage() {
        if (hipSetDevice(device) != hipSuccess) error.store((int)hipErrorInvalidDevice);
        for (;;) {
            const size_t i = next.fetch_add(1);
            if (i >= slice_segment.size()) return;
            const size_t g = slice_segment[i];
            Segment& sg = segments[g];
            const int buf = (int)(g % kSegBufs);
            if (i == sg.first_slice) {
                // the segment's first slice: its buffer must be free of its previous user -- the segment kSegBufs segments ago
                // (whose slices may still be under way in other stagers: wait until its device copy has been enqueued), or
                // an earlier upload of this call -- and that user's device copy must have read it
                bool used = st->sbusy[buf].load(std::memory_order_acquire) != 0;
                if (g >= (size_t)kSegBufs) {
                    while (!segments[g - kSegBufs].enqueued.load(std::memory_order_acquire)) __builtin_ia32_pause();
                    used = true;
                }
                if (used && error.load() == (int)hipSuccess) {
                    const hipError_t e = hipEventSynchronize(st->sev[buf]);
                    if (e != hipSuccess) error.store((int)e);
                }
                sg.ready.store(1, std::memory_order_release);
            } else {
                while (!sg.ready.load(std::memory_order_acquire)) __builtin_ia32_pause();
            }
            const size_t off = (i - sg.first_slice) * kSlice, len = std::min(kSlice, sg.len - off);
            std::memcpy(st->spin[buf] + off, sg.src + off, len);
            if (sg.left.fetch_sub(1, std::memory_order_acq_rel) == 1) {
                hipError_t e = (hipError_t)error.load();
                if (e == hipSuccess) e = hipMemcpyAsync(sg.dst, st->spin[buf], sg.len, hipMemcpyHostToDevice, stream);
                if (e == hipSuccess) e = hipEventRecord(st->sev[buf], stream);
                if (e != hipSuccess) error.store((int)e);
                else st->sbusy[buf].store(1, std::memory_order_release);
                sg.enqueued.store(1, std::memory_order_release);
                left[(size_t)sg.tag].fetch_sub(1, std::memory_order_release);       // (also after an error: nobody waits forever)
            }
        }
    }
};

// The thread that carries out the queued downloads of one session: for each, the download stream waits for the event that
// marks the download's place on the producing stream, then the bytes come over chunk by chunk through the download side's
// pinned buffers and are copied out to the caller's memory.
struct HostSession::Downloader {
    struct Job { hipEvent_t after; char* dst; const char* src; size_t bytes; };
    State* st;
    int device;
    std::mutex m;
    std::condition_variable cv;
    std::deque<Job> jobs;
    bool closing = false;
    hipError_t error = hipSuccess;
    std::thread thread;

    Downloader(State* s, int dev) : st(s), device(dev), thread([this] { run(); }) {}
    void push(const Job& j) {
        { std::lock_guard<std::mutex> l(m); jobs.push_back(j); }
        cv.notify_one();
    }
    hipError_t close() {
        { std::lock_guard<std::mutex> l(m); closing = true; }
        cv.notify_one();
        thread.join();
        return error;
    }
    // One pipeline across the jobs: while the bytes of one chunk are copied out to the caller's memory, the device copies of
    // the next chunks -- of the same job or the following ones -- are under way (at most kBuffers - 1 in flight).
    void run() {
        if (hipSetDevice(device) != hipSuccess) error = hipErrorInvalidDevice;
        struct Piece { int b; char* dst; size_t len; };
        std::deque<Piece> flight;
        int nextbuf = 0;
        bool have = false;
        Job cur{};
        size_t cur_off = 0;
        for (;;) {
            if (!have) {
                std::unique_lock<std::mutex> l(m);
                if (flight.empty()) cv.wait(l, [&] { return closing || !jobs.empty(); });
                if (!jobs.empty()) {
                    cur = jobs.front();
                    jobs.pop_front();
                    have = true;
                    cur_off = 0;
                } else if (flight.empty()) {
                    return;                                  // closing, nothing queued, nothing in flight
                }
            }
            if (have && error == hipSuccess && (int)flight.size() < kBuffers - 1) {
                hipError_t e = hipSuccess;
                if (cur_off == 0) e = hipStreamWaitEvent(st->down_stream, cur.after, 0);
                const size_t len = std::min(kChunk, cur.bytes - cur_off);
                const int b = nextbuf;
                nextbuf = (nextbuf + 1) % kBuffers;
                if (e == hipSuccess) e = hipMemcpyAsync(st->dpin[b], cur.src + cur_off, len, hipMemcpyDeviceToHost, st->down_stream);
                if (e == hipSuccess) e = hipEventRecord(st->dev_[b], st->down_stream);
                if (e != hipSuccess) { error = e; have = false; continue; }
                flight.push_back(Piece{b, cur.dst + cur_off, len});
                cur_off += len;
                if (cur_off >= cur.bytes) have = false;
                continue;
            }
            if (have && error != hipSuccess) { have = false; continue; }          // (the queue is drained without working)
            if (!flight.empty()) {
                const Piece p = flight.front();
                flight.pop_front();
                const hipError_t e = hipEventSynchronize(st->dev_[p.b]);
                if (e != hipSuccess) { if (error == hipSuccess) error = e; continue; }
                CopyPool::down().copy(p.dst, st->dpin[p.b], p.len);
            }
        }
    }
};

namespace {
std::map<int, HostSession::State*>& states() {
    static std::map<int, HostSession::State*>* m = new std::map<int, HostSession::State*>();
    return *m;
}
}  // namespace

HostSession::HostSession()
    : st_(nullptr), arena_(nullptr), stream_(nullptr), dirty_(false), dl_(nullptr), ul_(nullptr), device_(-1), compute_(nullptr), events_used_(0) {
    g_lease.lock();
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0) return;         // reserve() reports the failure
    State*& s = states()[dev];
    if (!s) s = new State();
    st_ = s;
    device_ = dev;
}

HostSession::~HostSession() {
    (void)end_uploads();
    (void)finish_downloads();
    if (st_ && compute_ && dirty_) (void)hipStreamSynchronize(compute_);
    if (st_ && dirty_ && st_->stream) {
        (void)hipStreamSynchronize(st_->stream);
        for (int b = 0; b < kBuffers; ++b) st_->busy[b] = false;
        for (int b = 0; b < kSegBufs; ++b) st_->sbusy[b].store(0);
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

hipError_t HostSession::begin_uploads(const Range* ranges, size_t count, int tags) {
    if (!st_ || !arena_ || ul_) return hipErrorNotInitialized;
    WorkerSet& ws = WorkerSet::stagers();
    hipError_t e = st_->ready_pipeline(ws.size());
    if (e != hipSuccess) return e;
    compute_ = st_->compute_stream;
    ul_ = new Uploader(st_, stream_, device_, tags);
    for (size_t r = 0; r < count; ++r)
        ul_->add(arena_ + ranges[r].dev_off, static_cast<const char*>(ranges[r].src), ranges[r].bytes, ranges[r].tag);
    dirty_ = true;
    ws.start(&ul_->fn);
    return hipSuccess;
}

hipError_t HostSession::uploaded_through(int tag) {
    if (!ul_) return hipErrorNotInitialized;
    for (int t = 0; t <= tag && t < (int)ul_->left.size(); ++t)
        while (ul_->left[(size_t)t].load(std::memory_order_acquire) > 0) __builtin_ia32_pause();
    if (ul_->error.load() != (int)hipSuccess) return (hipError_t)ul_->error.load();
    hipEvent_t ev = nullptr;
    hipError_t e = st_->order_event(events_used_, ev);
    if (e != hipSuccess) return e;
    ++events_used_;
    e = hipEventRecord(ev, stream_);
    if (e != hipSuccess) return e;
    return hipStreamWaitEvent(compute_, ev, 0);
}

hipError_t HostSession::end_uploads() {
    if (!ul_) return hipSuccess;
    WorkerSet::stagers().join();
    const hipError_t e = (hipError_t)ul_->error.load();
    delete ul_;
    ul_ = nullptr;
    return e;
}

hipError_t HostSession::download_async(void* dst, size_t dev_off, size_t bytes, hipStream_t after_stream) {
    if (!st_ || !arena_) return hipErrorNotInitialized;
    if (bytes == 0) return hipSuccess;
    hipError_t e = st_->ready_pipeline(0);
    if (e != hipSuccess) return e;
    if (!dl_) dl_ = new Downloader(st_, device_);
    hipEvent_t after = nullptr;
    e = st_->order_event(events_used_, after);
    if (e != hipSuccess) return e;
    ++events_used_;
    e = hipEventRecord(after, after_stream ? after_stream : stream_);
    if (e != hipSuccess) return e;
    dirty_ = true;
    dl_->push(Downloader::Job{after, static_cast<char*>(dst), arena_ + dev_off, bytes});
    return hipSuccess;
}

hipError_t HostSession::finish_downloads() {
    if (!dl_) return hipSuccess;
    const hipError_t e = dl_->close();
    delete dl_;
    dl_ = nullptr;
    return e;
}

bool HostSession::all_zero(const void* p, size_t bytes) { return CopyPool::get().all_zero(p, bytes); }

hipError_t HostSession::sync() {
    if (!st_ || !st_->stream) return hipSuccess;
    const hipError_t e = hipStreamSynchronize(st_->stream);
    if (e == hipSuccess) {
        for (int b = 0; b < kBuffers; ++b) st_->busy[b] = false;
        for (int b = 0; b < kSegBufs; ++b) st_->sbusy[b].store(0);
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
