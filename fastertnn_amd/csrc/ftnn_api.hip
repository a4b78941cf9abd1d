// C ABI of libftnn_hip.so: argument checking, the device-memory entry points, and
// the reference's host-memory entry points built on top of them.
#include <stdarg.h>
#include <stdio.h>

#include <sched.h>
#include <malloc.h>
#include <stdlib.h>
#include <sys/mman.h>
#include <time.h>
#include <string.h>

#include <algorithm>
#include <condition_variable>
#include <functional>
#include <mutex>
#include <system_error>
#include <thread>
#include <vector>

#include "../../include/ftnn.h"
#include "ftnn_internal.h"
#include "host_hash.h"

namespace ftnn {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

static int hip_fail(hipError_t e, const char* what) {
    return fail(FTNN_EHIP, "%s: %s", what, hipGetErrorString(e));
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// words per operand row (one plane) that every engine's 32-bit sums and offsets hold
constexpr int kMaxRowWords = (1 << 24) - 4;
// the fp4 GEMM sums lanes of {0, 0.5, 1}: products are multiples of 1/4, exact in fp32 while 4 * 64 * Kw <= 2^24
constexpr int kMaxF4GemmWords = 1 << 16;

// whether rows of ceil(C/64) * KH * KW words are within what 32-bit sums and offsets hold; no intermediate product
// overflows whatever the (positive) arguments are
static bool row_fits(int C, int KH, int KW) {
    int64_t k;
    if (C > (1 << 30) || __builtin_mul_overflow((int64_t)KH, (int64_t)KW, &k) ||
        __builtin_mul_overflow(k, ((int64_t)C + 63) / 64, &k))
        return false;
    return k <= kMaxRowWords;
}

// common conv-shape validation; fills OH/OW
int check_conv_shape(int N, int C, int H, int W, int H_pad, int W_pad, int kH, int kW,
                            int H_stride, int W_stride, int* OH, int* OW) {
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || kH <= 0 || kW <= 0 || H_stride <= 0 ||
        W_stride <= 0 || H_pad < 0 || W_pad < 0)
        return fail(FTNN_EINVAL, "non-positive dimension or negative padding");
    const int64_t Hp = (int64_t)H + 2 * (int64_t)H_pad, Wp = (int64_t)W + 2 * (int64_t)W_pad;
    if (Hp < kH || Wp < kW)
        return fail(FTNN_EINVAL, "kernel %dx%d larger than padded input %lldx%lld", kH, kW, (long long)Hp,
                    (long long)Wp);
    if (N > 65535) return fail(FTNN_EINVAL, "batch %d above the supported 65535", N);
    // pixel indices within one image plane are 32-bit in the kernels (27 of them in one store offset)
    if (Hp > 0x3ffffffLL || Wp > 0x3ffffffLL || Hp * Wp > 0x3ffffffLL)
        return fail(FTNN_EINVAL, "padded image plane above the supported 2^26 pixels");
    // 32-bit accumulators count up to 128 per word of a row
    if (!row_fits(C, kH, kW))
        return fail(FTNN_EINVAL, "more than %d words per im2row row", kMaxRowWords);
    *OH = out_dim(H, H_pad, kH, H_stride);
    *OW = out_dim(W, W_pad, kW, W_stride);
    return FTNN_OK;
}

// ---- lazily created state behind the host-memory entry points ----
// grow-only device buffers of the host entry points, one per kind of operand
enum { SLOT_X = 0, SLOT_THR, SLOT_W, SLOT_ROWS, SLOT_SCRATCH, SLOT_Y, SLOT_PREP, SLOT_COUNT };
struct HostCtx {
    hipStream_t stream = nullptr;
    void* buf[SLOT_COUNT] = {};
    size_t cap[SLOT_COUNT] = {};
};
static HostCtx g_ctx;
// The reference's entry points are called from one thread (its drivers are single-threaded); the
// workspace is nevertheless guarded so that concurrent callers serialise instead of racing.
static std::mutex g_ctx_mutex;

[[noreturn]] static void die(const char* what) {
    // the reference reports failure by abort() (src/timing_layers.c:156-159)
    fprintf(stderr, "libftnn_hip: %s: %s\n", what, g_err);
    abort();
}

static void hip_or_die(hipError_t e, const char* what) {
    if (e != hipSuccess) {
        hip_fail(e, what);
        die("HIP failure");
    }
}

// Every host entry point returns a buffer that the caller free()s, call after call, layer after layer.  With the
// allocator's defaults such buffers are cut from the top of the heap and given back to the system as soon as 2 x the
// largest of them is free there, or are mappings of their own beyond 32 MiB: a good part of the results then lands in
// memory that has to be faulted in again, page by page, by the copy (ResNet-152 through the reference's e2e driver:
// five results of 25 MB per pass at 4.4 ms instead of 0.6 ms each).  With FTNN_HOST_KEEP_HEAP=1 in the environment the
// host entry points tell the allocator on their first call to keep freed memory (blocks up to 32 MiB from the heap,
// the heap's top trimmed only beyond 512 MiB): 163 -> 155 ms on that network, 24 -> 21 ms on VGG-16.  Off by default:
// it changes the allocator of the whole process.
static void keep_heap_once() {
    static const bool done = []() {
        const char* e = getenv("FTNN_HOST_KEEP_HEAP");
        if (!e || atoi(e) == 0) return true;
        mallopt(M_MMAP_THRESHOLD, 32 << 20);
        mallopt(M_TRIM_THRESHOLD, 512 << 20);
        if (atoi(e) >= 2) {
            mallopt(M_MMAP_MAX, 0);                    // no mappings at all: results beyond 32 MiB come from the heap too
            mallopt(M_TRIM_THRESHOLD, 1 << 30);
        }
        return true;
    }();
    (void)done;
}

static hipStream_t host_stream() {
    if (!g_ctx.stream) {
        keep_heap_once();
        hip_or_die(hipStreamCreate(&g_ctx.stream), "hipStreamCreate");
    }
    return g_ctx.stream;
}

// grow-only device buffer number `slot`
static void* dev_buf(int slot, size_t bytes) {
    if (bytes == 0) bytes = 16;
    if (g_ctx.cap[slot] < bytes) {
        if (g_ctx.buf[slot]) {
            hip_or_die(hipStreamSynchronize(host_stream()), "hipStreamSynchronize");
            hip_or_die(hipFree(g_ctx.buf[slot]), "hipFree");
        }
        g_ctx.buf[slot] = nullptr;
        g_ctx.cap[slot] = 0;
        hip_or_die(hipMalloc(&g_ctx.buf[slot], bytes), "hipMalloc");
        g_ctx.cap[slot] = bytes;
    }
    return g_ctx.buf[slot];
}

// ---- large host <-> device copies of the host-memory entry points ----
// The reference's callers pass ordinary (pageable) memory and free() what they get back.  The runtime copies such
// memory through its own staging at about 29 GB/s up and 18 GB/s down, and at 4 GB/s down into memory that was
// never touched (a large result is a fresh mapping: every page faults on the one copying thread).  From 4 MiB on
// the copies here go through a small ring of pinned chunks instead: the DMA engine moves a chunk (57 GB/s) while
// a few threads copy the neighbouring chunk between the ring and the caller's memory, where the page faults of a
// fresh result spread over those threads.
constexpr size_t kStageChunk = 4u << 20;   // bytes per chunk (2, 8 and 16 MiB measured no faster)
constexpr int kStageSlots = 4;
constexpr size_t kStageFrom = 4u << 20;    // smaller copies take the plain path (the ring's event waits cost more)

// A fixed set of worker threads that work on page-aligned slices of one buffer -- slices of one memcpy, or of one
// content hash; created on first use and never joined (the object is leaked on purpose: at exit the workers are blocked
// on its condition variable).
class CopyPool {
public:
    static CopyPool& get() {
        static CopyPool* pool = new CopyPool;
        return *pool;
    }
    // with one thread the runtime's own pageable copy is the faster one (29 GB/s up against a single memcpy into the ring)
    bool parallel() const { return workers_ > 0; }
    // slices a job is cut into: one per worker and one for the caller
    int parts() const { return workers_ + 1; }
    typedef std::function<void(int part, size_t lo, size_t hi)> Job;
    // fn(part, lo, hi) for every slice [lo, hi) of [0, bytes), each on a thread of its own; returns when all are done
    void run_slices(size_t bytes, const Job& fn) {
        if (workers_ == 0) {
            fn(0, 0, bytes);
            return;
        }
        std::unique_lock<std::mutex> lock(m_);
        job_ = &fn;
        bytes_ = bytes;
        pending_ = workers_;
        generation_++;
        wake_.notify_all();
        lock.unlock();
        slice(workers_);   // the calling thread takes the last slice
        lock.lock();
        done_.wait(lock, [this] { return pending_ == 0; });
    }
    void copy(void* dst, const void* src, size_t bytes) {
        if (workers_ == 0 || bytes < (256u << 10)) {
            memcpy(dst, src, bytes);
            return;
        }
        char* d = static_cast<char*>(dst);
        const char* s = static_cast<const char*>(src);
        run_slices(bytes, [d, s](int, size_t lo, size_t hi) { memcpy(d + lo, s + lo, hi - lo); });
    }

private:
    CopyPool() {
        cpu_set_t set;
        int cores = 1;
        if (sched_getaffinity(0, sizeof(set), &set) == 0) cores = CPU_COUNT(&set);
        int threads = std::min(cores, 4);   // measured: eight threads are no faster on 25 MB and slower on 3 MB (wake-ups)
        if (const char* env = getenv("FTNN_HOST_COPY_THREADS")) threads = std::max(1, std::min(atoi(env), 16));   // tuning aid
        const int wanted = threads - 1;   // a caller pinned to one core (the reference's Makefile) copies alone
        // workers_ is final before the first worker runs: a slice's bounds depend on it
        std::vector<std::thread> started;
        try {
            for (int t = 0; t < wanted; t++) started.emplace_back([this, t] { run(t); });
        } catch (const std::system_error&) {   // no more threads to be had: go on with those that started
        }
        std::unique_lock<std::mutex> lock(m_);
        workers_ = (int)started.size();
        lock.unlock();
        for (std::thread& th : started) th.detach();
    }
    void slice(int t) {
        const size_t parts = (size_t)workers_ + 1;
        const size_t per = (bytes_ / parts + 4095) & ~(size_t)4095;   // whole pages per thread
        const size_t lo = std::min(bytes_, per * (size_t)t), hi = std::min(bytes_, lo + per);
        const size_t end = t == workers_ ? bytes_ : hi;
        (*job_)(t, lo, std::max(lo, end));   // an empty slice is still reported: a job may keep a result per part
    }
    void run(int t) {
        uint64_t seen = 0;
        for (;;) {
            std::unique_lock<std::mutex> lock(m_);
            wake_.wait(lock, [&] { return generation_ != seen; });
            seen = generation_;
            lock.unlock();
            slice(t);
            lock.lock();
            if (--pending_ == 0) done_.notify_one();
        }
    }
    std::mutex m_;
    std::condition_variable wake_, done_;
    const Job* job_ = nullptr;
    size_t bytes_ = 0;
    int workers_ = 0, pending_ = 0;
    uint64_t generation_ = 0;
};

struct StageRing {
    char* pin = nullptr;   // kStageSlots chunks of pinned host memory
    hipEvent_t ev[kStageSlots] = {};
};
static StageRing g_ring;

static StageRing& stage_ring() {
    if (!g_ring.pin) {
        hip_or_die(hipHostMalloc((void**)&g_ring.pin, kStageChunk * kStageSlots, hipHostMallocDefault), "hipHostMalloc");
        for (int i = 0; i < kStageSlots; i++)
            hip_or_die(hipEventCreateWithFlags(&g_ring.ev[i], hipEventDisableTiming), "hipEventCreate");
    }
    return g_ring;
}

// host -> device, ordered on the host stream; returns when the last chunk has been queued
static void staged_upload(void* dev, const void* host, size_t bytes) {
    StageRing& r = stage_ring();
    CopyPool& pool = CopyPool::get();
    hipStream_t st = host_stream();
    const size_t chunks = (bytes + kStageChunk - 1) / kStageChunk;
    for (size_t c = 0; c < chunks; c++) {
        const int slot = (int)(c % kStageSlots);
        const size_t off = c * kStageChunk, len = std::min(kStageChunk, bytes - off);
        if (c >= (size_t)kStageSlots) hip_or_die(hipEventSynchronize(r.ev[slot]), "hipEventSynchronize");   // chunk free again
        pool.copy(r.pin + (size_t)slot * kStageChunk, static_cast<const char*>(host) + off, len);
        hip_or_die(hipMemcpyAsync(static_cast<char*>(dev) + off, r.pin + (size_t)slot * kStageChunk, len,
                                  hipMemcpyHostToDevice, st), "H2D copy");
        hip_or_die(hipEventRecord(r.ev[slot], st), "hipEventRecord");
    }
    // the ring is reused by the next copy: its chunks must have left
    hip_or_die(hipStreamSynchronize(st), "hipStreamSynchronize");
}

// device -> host after everything queued on the host stream; returns when `host` is complete
static void staged_download(void* host, const void* dev, size_t bytes) {
    StageRing& r = stage_ring();
    CopyPool& pool = CopyPool::get();
    hipStream_t st = host_stream();
    const size_t chunks = (bytes + kStageChunk - 1) / kStageChunk;
    auto fetch = [&](size_t c) {
        const int slot = (int)(c % kStageSlots);
        const size_t off = c * kStageChunk, len = std::min(kStageChunk, bytes - off);
        hip_or_die(hipMemcpyAsync(r.pin + (size_t)slot * kStageChunk, static_cast<const char*>(dev) + off, len,
                                  hipMemcpyDeviceToHost, st), "D2H copy");
        hip_or_die(hipEventRecord(r.ev[slot], st), "hipEventRecord");
    };
    for (size_t c = 0; c < std::min(chunks, (size_t)kStageSlots); c++) fetch(c);
    for (size_t c = 0; c < chunks; c++) {
        const int slot = (int)(c % kStageSlots);
        const size_t off = c * kStageChunk, len = std::min(kStageChunk, bytes - off);
        hip_or_die(hipEventSynchronize(r.ev[slot]), "hipEventSynchronize");
        pool.copy(static_cast<char*>(host) + off, r.pin + (size_t)slot * kStageChunk, len);
        if (c + kStageSlots < chunks) fetch(c + kStageSlots);
    }
}

// ---- copies below kStageFrom ----
// Layer-sized tensors (a few MB) are where the reference's drivers spend their calls.  The runtime moves such
// pageable memory at 118 us up and 195 us down for 3.2 MB, and takes 33 / 112 us for 64 / 256 KiB; the DMA engine on
// pinned memory needs 65 us for the same 3.2 MB and 9 us for 64 KiB.  So these copies pass through pinned areas of
// their own, one per kind of operand, each as large as the largest copy that takes this path: a chunk is copied
// into (out of) the area while the DMA engine moves its neighbour.  An area is written again only by a later call,
// and every host entry point returns after a download that has waited for the stream.
constexpr size_t kSmallChunk = 1u << 20;
constexpr size_t kSmallArea = kStageFrom;          // activations / rows, weights, results
constexpr size_t kSmallThrArea = 256u << 10;       // thresholds: at most 65535 floats
enum { AREA_ACT = 0, AREA_W, AREA_THR, AREA_DOWN, AREA_COUNT };

struct SmallStage {
    char* area[AREA_COUNT] = {};
    hipEvent_t ev[kSmallArea / kSmallChunk] = {};
};
static SmallStage g_small;

static SmallStage& small_stage() {
    if (!g_small.area[0]) {
        char* base = nullptr;
        hip_or_die(hipHostMalloc((void**)&base, 3 * kSmallArea + kSmallThrArea, hipHostMallocDefault), "hipHostMalloc");
        g_small.area[AREA_ACT] = base;
        g_small.area[AREA_W] = base + kSmallArea;
        g_small.area[AREA_DOWN] = base + 2 * kSmallArea;
        g_small.area[AREA_THR] = base + 3 * kSmallArea;
        for (hipEvent_t& e : g_small.ev) hip_or_die(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate");
    }
    return g_small;
}

// host -> device through pinned area `area`; queued on the host stream, not waited for
static void small_upload(void* dev, const void* host, size_t bytes, int area) {
    char* pin = small_stage().area[area];
    CopyPool& pool = CopyPool::get();
    for (size_t off = 0; off < bytes; off += kSmallChunk) {
        const size_t len = std::min(kSmallChunk, bytes - off);
        pool.copy(pin + off, static_cast<const char*>(host) + off, len);
        hip_or_die(hipMemcpyAsync(static_cast<char*>(dev) + off, pin + off, len, hipMemcpyHostToDevice, host_stream()), "H2D copy");
    }
}

// device -> host after everything queued on the host stream; returns when `host` is complete
static void small_download(void* host, const void* dev, size_t bytes) {
    SmallStage& s = small_stage();
    char* pin = s.area[AREA_DOWN];
    CopyPool& pool = CopyPool::get();
    hipStream_t st = host_stream();
    int c = 0;
    for (size_t off = 0; off < bytes; off += kSmallChunk, c++) {
        const size_t len = std::min(kSmallChunk, bytes - off);
        hip_or_die(hipMemcpyAsync(pin + off, static_cast<const char*>(dev) + off, len, hipMemcpyDeviceToHost, st), "D2H copy");
        hip_or_die(hipEventRecord(s.ev[c], st), "hipEventRecord");
    }
    if (bytes == 0) hip_or_die(hipStreamSynchronize(st), "hipStreamSynchronize");
    c = 0;
    for (size_t off = 0; off < bytes; off += kSmallChunk, c++) {
        const size_t len = std::min(kSmallChunk, bytes - off);
        hip_or_die(hipEventSynchronize(s.ev[c]), "hipEventSynchronize");
        pool.copy(static_cast<char*>(host) + off, pin + off, len);
    }
}

static int area_of_slot(int slot);

static void* upload(int slot, const void* host, size_t bytes) {
    void* d = dev_buf(slot, bytes);
    const int area = area_of_slot(slot);
    if (bytes >= kStageFrom) {
        if (CopyPool::get().parallel()) {
            staged_upload(d, host, bytes);
            return d;
        }
    } else if (area >= 0 && bytes <= (area == AREA_THR ? kSmallThrArea : kSmallArea)) {
        small_upload(d, host, bytes, area);
        return d;
    }
    hip_or_die(hipMemcpyAsync(d, host, bytes, hipMemcpyHostToDevice, host_stream()), "H2D copy");
    return d;
}

static void download(void* host, const void* dev, size_t bytes) {
    if (bytes >= kStageFrom) {
        if (CopyPool::get().parallel()) {
            staged_download(host, dev, bytes);
            return;
        }
    } else {
        small_download(host, dev, bytes);
        return;
    }
    hip_or_die(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, host_stream()), "D2H copy");
    hip_or_die(hipStreamSynchronize(host_stream()), "hipStreamSynchronize");
}

// heap memory for a result of kStageFrom bytes or more, as the caller will free() it
static void* large_alloc(size_t bytes, bool aligned32) {
    // A large result is often memory the process has not touched yet (a fresh mapping, or new heap), and the copy
    // into it then pays a page fault per 4 KiB (25 MB: 2.6 ms on one thread, 1.1 ms on eight).  Its 2 MiB-aligned
    // interior is therefore marked for transparent huge pages: 13 faults instead of 6300 (0.5 ms on one thread)
    // where the memory is fresh, nothing where the allocator hands out memory that is mapped already.  Still
    // plain heap memory that the caller free()s; where huge pages are unavailable the hint is ignored.
    constexpr size_t kHuge = 2u << 20;
    void* p = aligned32 ? aligned_alloc(32, (bytes + 31) / 32 * 32) : malloc(bytes);
    static const bool no_thp = getenv("FTNN_HOST_NO_THP") != nullptr;   // tuning aid
    if (p && !no_thp) {
        const uintptr_t lo = (reinterpret_cast<uintptr_t>(p) + kHuge - 1) / kHuge * kHuge;
        const uintptr_t hi = (reinterpret_cast<uintptr_t>(p) + bytes) / kHuge * kHuge;
        if (hi > lo) (void)madvise(reinterpret_cast<void*>(lo), hi - lo, MADV_HUGEPAGE);
    }
    return p;
}

// Even with huge pages a fresh result costs the copy the time the kernel needs to zero it: the reference's e2e driver
// on ResNet-152 spends 27 of its 162 ms per pass there (results of 25 and 100 MB, each a new mapping: the allocator
// returns blocks of that size to the system at once).  A caller that walks the same layers again and again asks for
// the same sizes again and again, so from the second request for a size on, a thread of its own allocates the next
// buffer of that size ahead of time and touches its pages; host_alloc hands that one out if it is ready.  The spare
// is ordinary malloc memory like any other result.  At most kSpareCap bytes wait as spares; a caller confined to
// fewer than four cores gets none (the thread would take the time from the caller).
class SparePool {
public:
    static SparePool& get() {
        static SparePool* pool = new SparePool;   // leaked on purpose, like the copy pool
        return *pool;
    }
    // frees every spare that is ready (those being prepared arrive later and age out)
    void release() {
        if (!running_) return;
        std::lock_guard<std::mutex> lock(m_);
        for (const Spare& r : ready_) free(r.p);
        ready_.clear();
        held_ = 0;
        seen_.clear();
    }
    // a ready buffer of exactly this kind, or nullptr
    void* take(size_t bytes, bool aligned32) {
        if (!running_) return nullptr;
        std::lock_guard<std::mutex> lock(m_);
        for (size_t i = 0; i < ready_.size(); i++)
            if (ready_[i].bytes == bytes && ready_[i].aligned32 == aligned32) {
                void* p = ready_[i].p;
                ready_.erase(ready_.begin() + (long)i);
                held_ -= bytes;
                return p;
            }
        return nullptr;
    }
    // a buffer of this kind was just handed out: prepare the next one if the size has been seen before
    void handed_out(size_t bytes, bool aligned32) {
        if (!running_) return;
        std::lock_guard<std::mutex> lock(m_);
        // a spare that kSpareMaxAge large results have passed by belongs to a caller that has moved on: free it
        clock_++;
        for (size_t i = 0; i < ready_.size();) {
            if (clock_ - ready_[i].born > kSpareMaxAge) {
                free(ready_[i].p);
                held_ -= ready_[i].bytes;
                ready_.erase(ready_.begin() + (long)i);
            } else {
                i++;
            }
        }
        bool seen = false;
        for (const Key& k : seen_) seen = seen || (k.bytes == bytes && k.aligned32 == aligned32);
        if (!seen) {
            if (seen_.size() < 64) seen_.push_back(Key{bytes, aligned32});
            return;
        }
        for (const Spare& r : ready_)
            if (r.bytes == bytes && r.aligned32 == aligned32) return;
        for (const Key& k : wanted_)
            if (k.bytes == bytes && k.aligned32 == aligned32) return;
        if (held_ + queued_ + bytes > kSpareCap) return;
        wanted_.push_back(Key{bytes, aligned32});
        queued_ += bytes;
        wake_.notify_one();
    }

private:
    static constexpr size_t kSpareCap = 512u << 20;
    static constexpr uint64_t kSpareMaxAge = 256;
    struct Key {
        size_t bytes;
        bool aligned32;
    };
    struct Spare {
        void* p;
        size_t bytes;
        bool aligned32;
        uint64_t born;   // clock_ when it became ready
    };
    SparePool() {
        cpu_set_t set;
        int cores = 1;
        if (sched_getaffinity(0, sizeof(set), &set) == 0) cores = CPU_COUNT(&set);
        if (cores < 4 || getenv("FTNN_HOST_NO_SPARES")) return;   // (the variable: tuning aid)
        try {
            std::thread([this] { run(); }).detach();
            running_ = true;
        } catch (const std::system_error&) {
        }
    }
    void run() {
        for (;;) {
            std::unique_lock<std::mutex> lock(m_);
            wake_.wait(lock, [this] { return !wanted_.empty(); });
            const Key k = wanted_.front();
            wanted_.erase(wanted_.begin());
            lock.unlock();
            unsigned char* p = static_cast<unsigned char*>(large_alloc(k.bytes, k.aligned32));
            if (p)
                for (size_t i = 0; i < k.bytes; i += 4096) p[i] = 0;   // maps the page (a huge page where there is one)
            lock.lock();
            queued_ -= k.bytes;
            if (p) {
                ready_.push_back(Spare{p, k.bytes, k.aligned32, clock_});
                held_ += k.bytes;
            }
        }
    }
    std::mutex m_;
    std::condition_variable wake_;
    std::vector<Key> seen_, wanted_;
    std::vector<Spare> ready_;
    size_t held_ = 0, queued_ = 0;
    uint64_t clock_ = 0;
    bool running_ = false;
};

static void* host_alloc(size_t bytes, bool aligned32) {
    void* p;
    if (bytes >= kStageFrom) {
        p = SparePool::get().take(bytes, aligned32);
        if (!p) p = large_alloc(bytes, aligned32);
        if (p) SparePool::get().handed_out(bytes, aligned32);
    } else if (aligned32) {
        // aligned_alloc(32, ...) as src/tnns/ternarize2row_avx2.c:735
        p = aligned_alloc(32, (bytes + 31) / 32 * 32);
    } else {
        p = malloc(bytes ? bytes : 1);
    }
    if (!p) {
        fail(FTNN_ENOMEM, "host allocation of %zu bytes failed", bytes);
        die("out of memory");
    }
    return p;
}

// the pinned area an operand below kStageFrom is staged through: the activation-side operand, the weight-side
// operand and the thresholds of one call each have their own
static int area_of_slot(int slot) {
    switch (slot) {
        case SLOT_X:
        case SLOT_ROWS: return AREA_ACT;
        case SLOT_W: return AREA_W;
        case SLOT_THR: return AREA_THR;
        default: return -1;
    }
}

// ---- weights of tnns_conv, kept in engine form across calls ----
// The reference's layer functions read the packed weights where they lie; here they must reach the device and, for
// the matrix-core engine, be re-arranged into fragments: an upload, a launch and their latencies on every call for
// data that a network never changes.  tnns_conv therefore keeps the prepared weights of the layers it has seen,
// found again by byte count, layer shape and a 128-bit hash of the CONTENTS, recomputed on every call: rows that are
// rewritten in place, or another layer's rows packed into memory that malloc hands out again, give another hash and
// a fresh upload; the same rows packed again at another address are found.  The host address is not part of the
// identity.  The hash must cost less than the upload it saves: it runs on AES rounds where the CPU has them (limited
// by memory bandwidth: 35 GB/s on one thread of the GPU box's host against 15 GB/s for multiply-rotate lanes) and rows
// of 1 MiB and more are hashed in slices on the copy threads (64 MiB in 0.36 ms, against 1.6 ms for their upload).
// Entries are dropped least recently used first beyond 512 entries or the byte cap (1 GiB of device memory;
// FTNN_HOST_WEIGHT_CACHE_MB = n sets it, FTNN_HOST_NO_WEIGHT_CACHE = 1 or a cap of 0 switches the cache off; a layer
// whose prepared weights alone exceed the cap is uploaded and prepared on every call); ftnn_host_forget_weights()
// drops them all.
struct PreparedWeights {
    size_t bytes;
    Hash128 hash;
    int type, C, KN, KH, KW;
    void* dev;
    size_t dev_bytes;
    uint64_t last_use;
};
static std::vector<PreparedWeights> g_weights;
static uint64_t g_weights_clock = 0;
static size_t g_weights_bytes = 0;
constexpr size_t kWeightCacheEntries = 512;
constexpr size_t kParallelHashFrom = (size_t)1 << 20;

static size_t weight_cache_cap() {
    static const size_t cap = []() -> size_t {
        if (const char* off = getenv("FTNN_HOST_NO_WEIGHT_CACHE"))
            if (atoi(off) != 0) return 0;
        if (const char* mb = getenv("FTNN_HOST_WEIGHT_CACHE_MB")) return (size_t)std::max(0LL, atoll(mb)) << 20;
        return (size_t)1 << 30;
    }();
    return cap;
}

// 128-bit hash of the packed rows; from kParallelHashFrom bytes on, the slices of the copy threads are hashed side by
// side and their hashes hashed in order (the number of slices is fixed per process, so the result is stable)
static Hash128 content_hash(const void* data, size_t bytes) {
    CopyPool& pool = CopyPool::get();
    if (bytes < kParallelHashFrom || !pool.parallel()) return hash128(data, bytes, 0);
    Hash128 part[32] = {};
    const char* base = static_cast<const char*>(data);
    pool.run_slices(bytes, [&part, base](int t, size_t lo, size_t hi) { part[t & 31] = hash128(base + lo, hi - lo, (uint64_t)t + 1); });
    return hash128(part, sizeof(Hash128) * (size_t)std::min(pool.parts(), 32), bytes);
}

static void drop_weight_entry(size_t i) {
    hip_or_die(hipStreamSynchronize(host_stream()), "hipStreamSynchronize");
    hip_or_die(hipFree(g_weights[i].dev), "hipFree");
    g_weights_bytes -= g_weights[i].dev_bytes;
    g_weights.erase(g_weights.begin() + (long)i);
}

// device pointer of the prepared weights of this layer (uploading and preparing them on a miss)
static const void* prepared_weights(int type, const int64_t* host, size_t bytes, int C, int KN, int KH, int KW) {
    const size_t dev_bytes = (size_t)ftnn_conv_weights_bytes(type, C, KN, KH, KW);
    const size_t cap = weight_cache_cap();
    if (cap == 0 || dev_bytes > cap) {
        // not kept: uploaded and prepared into a work buffer on every call
        void* d_prep = dev_buf(SLOT_PREP, dev_bytes);
        int64_t* d_rows = (int64_t*)upload(SLOT_W, host, bytes);
        if (ftnn_conv_prepare_weights(type, d_rows, C, KN, KH, KW, d_prep, host_stream()) != FTNN_OK) die("tnns_conv");
        return d_prep;
    }
    const Hash128 hash = content_hash(host, bytes);
    g_weights_clock++;
    for (PreparedWeights& e : g_weights)
        if (e.bytes == bytes && e.hash == hash && e.type == type && e.C == C && e.KN == KN && e.KH == KH && e.KW == KW) {
            e.last_use = g_weights_clock;
            return e.dev;
        }
    PreparedWeights e = {bytes, hash, type, C, KN, KH, KW, nullptr, dev_bytes, g_weights_clock};
    while (!g_weights.empty() && (g_weights.size() >= kWeightCacheEntries || g_weights_bytes + e.dev_bytes > cap)) {
        size_t oldest = 0;
        for (size_t i = 1; i < g_weights.size(); i++)
            if (g_weights[i].last_use < g_weights[oldest].last_use) oldest = i;
        drop_weight_entry(oldest);
    }
    hip_or_die(hipMalloc(&e.dev, e.dev_bytes ? e.dev_bytes : 16), "hipMalloc");
    int64_t* d_rows = (int64_t*)upload(SLOT_W, host, bytes);
    if (ftnn_conv_prepare_weights(type, d_rows, C, KN, KH, KW, e.dev, host_stream()) != FTNN_OK) die("tnns_conv");
    g_weights_bytes += e.dev_bytes;
    g_weights.push_back(e);
    return e.dev;
}

static int64_t* host_quantize_im2row(bool ternary, float* x, float* thr, int N, int C, int H, int W,
                                     int H_pad, int W_pad, int kH, int kW, int H_stride,
                                     int W_stride) {
    std::lock_guard<std::mutex> lock(g_ctx_mutex);
    int OH, OW;
    if (check_conv_shape(N, C, H, W, H_pad, W_pad, kH, kW, H_stride, W_stride, &OH, &OW) != FTNN_OK)
        die(ternary ? "t2r_p2_opt" : "b2r");
    const size_t out_bytes =
        (size_t)N * OH * OW * (size_t)ftnn_row_words(C, kH, kW, ternary) * sizeof(int64_t);
    float* d_x = (float*)upload(SLOT_X, x, (size_t)N * C * H * W * sizeof(float));
    float* d_thr = (float*)upload(SLOT_THR, thr, (size_t)N * sizeof(float));
    int64_t* d_rows = (int64_t*)dev_buf(SLOT_ROWS, out_bytes);
    void* d_scr = dev_buf(SLOT_SCRATCH, (size_t)ftnn_pack_scratch_bytes(N, C, H, W, ternary));
    if (ftnn_quantize_im2row(ternary, d_x, d_thr, N, C, H, W, H_pad, W_pad, kH, kW, H_stride,
                             W_stride, d_rows, d_scr, host_stream()) != FTNN_OK)
        die(ternary ? "t2r_p2_opt" : "b2r");
    int64_t* out = (int64_t*)host_alloc(out_bytes, true);
    download(out, d_rows, out_bytes);
    return out;
}

// the reference's weight packers (src/utils.c:468-521, 634-675) on host pointers: fp32 (KN, C, KH, KW) up, the device
// packer, Packing-2 rows down into aligned_alloc(32, ...) memory as the reference returns it
static int64_t* host_pack_weights(bool ternary, float* w, float* thr, int KN, int C, int KH, int KW) {
    std::lock_guard<std::mutex> lock(g_ctx_mutex);
    const char* who = ternary ? "ternarize_opt_avx2" : "binarize_opt_avx2";
    if (KN <= 0 || C <= 0 || KH <= 0 || KW <= 0 || !row_fits(C, KH, KW) || !w || !thr) {
        fail(FTNN_EINVAL, "non-positive dimension, null pointer or more than %d words per row", kMaxRowWords);
        die(who);
    }
    const size_t out_bytes = (size_t)KN * (size_t)ftnn_row_words(C, KH, KW, ternary) * sizeof(int64_t);
    float* d_w = (float*)upload(SLOT_X, w, (size_t)KN * C * KH * KW * sizeof(float));
    float* d_thr = (float*)upload(SLOT_THR, thr, (size_t)KN * sizeof(float));
    int64_t* d_rows = (int64_t*)dev_buf(SLOT_ROWS, out_bytes);
    if (ftnn_pack_weights(ternary, d_w, d_thr, KN, C, KH, KW, d_rows, host_stream()) != FTNN_OK) die(who);
    int64_t* out = (int64_t*)host_alloc(out_bytes, true);
    download(out, d_rows, out_bytes);
    return out;
}

// bitpacking2 (src/utils.c:257-291) on host pointers
static int64_t* host_pack_gemm_operand(float* x, int I, int J) {
    std::lock_guard<std::mutex> lock(g_ctx_mutex);
    if (I <= 0 || J <= 0 || J % 256 != 0 || !x) {   // the reference asserts J % 256 == 0 (src/utils.c:258)
        fail(FTNN_EINVAL, "bitpacking2: I = %d, J = %d (J must be a positive multiple of 256)", I, J);
        die("bitpacking2");
    }
    const size_t out_bytes = (size_t)I * J / 32 * sizeof(int64_t);
    float* d_x = (float*)upload(SLOT_X, x, (size_t)I * J * sizeof(float));
    int64_t* d_rows = (int64_t*)dev_buf(SLOT_ROWS, out_bytes);
    if (ftnn_pack_gemm_operand(d_x, I, J, d_rows, host_stream()) != FTNN_OK) die("bitpacking2");
    int64_t* out = (int64_t*)host_alloc(out_bytes, true);
    download(out, d_rows, out_bytes);
    return out;
}

static float* host_mm(int type, int64_t* a, int64_t* b, int N, int OH, int OW, int KN, int K,
                      int K_unpack, float alpha) {
    std::lock_guard<std::mutex> lock(g_ctx_mutex);
    if (N <= 0 || OH <= 0 || OW <= 0 || KN <= 0 || K <= 0 || K > kMaxRowWords) {
        fail(FTNN_EINVAL, "GEMM dimension non-positive or K above %d words", kMaxRowWords);
        die("mm");
    }
    const size_t M = (size_t)N * OH * OW;
    const size_t kw = (size_t)round4(K);
    const size_t a_words = kw * ((type == kTNN || type == kTBN) ? 2 : 1);
    const size_t b_words = kw * ((type == kTNN || type == kBTN) ? 2 : 1);
    int64_t* d_a = (int64_t*)upload(SLOT_ROWS, a, M * a_words * sizeof(int64_t));
    int64_t* d_b = (int64_t*)upload(SLOT_W, b, (size_t)KN * b_words * sizeof(int64_t));
    const size_t y_bytes = M * KN * sizeof(float);
    float* d_y = (float*)dev_buf(SLOT_Y, y_bytes);
    const int64_t scr = ftnn_mm_scratch_bytes(FTNN_ENGINE_AUTO, type, N, OH, OW, KN, K);
    void* d_scr = scr > 0 ? dev_buf(SLOT_SCRATCH, (size_t)scr) : nullptr;
    if (ftnn_mm_engine(FTNN_ENGINE_AUTO, type, d_a, d_b, N, OH, OW, KN, K, K_unpack, alpha, d_y, d_scr, scr,
                       host_stream()) != FTNN_OK)
        die("mm");
    float* y = (float*)host_alloc(y_bytes, false);
    download(y, d_y, y_bytes);
    return y;
}

// bytes of the two regions of the matrix-core layer path: P4 (32 bytes per pixel and 64 channels),
// then the fp4 fragments of the weights
int64_t conv_f4_p4_bytes(int N, int C, int H, int W) {
    return ((int64_t)N * H * W * cpack_of(C) * 32 + 255) / 256 * 256;
}

// the same region for a few-channel layer on the dense fp4 path: nibble pixels, then the dense rows
int64_t conv_f4_dense_bytes(int N, int C, int H, int W, int KH, int KW, int OH, int OW) {
    int T, Kd;
    dense_applies(C, KH, KW, &T, &Kd);
    return dense_f4_pq_bytes(N, H, W) + ((int64_t)N * OH * OW * Kd * 32 + 255) / 256 * 256;
}

// Large layers with an fp32 result run as quantise + im2row + expansion + the GEMM kernel with LDS-staged 128 / 256
// tiles: from about 12 GMAC, with tiles for every compute unit, the layer kernel's wavefronts, each fetching its own
// fragments through the L1, fall behind it (the reference's 1024-channel 56 x 56 layer at batch 8, 59 GMAC: 139 us
// against 80 us; 15 GMAC layers with 100-200 tiles are a tie).
bool conv_f4_gemm_route(int64_t M, int KN, int K) {
    static const bool off = getenv("FTNN_CONV_NO_GEMM_ROUTE") != nullptr;   // tuning aid
    // enough 128 x 128 tiles for every compute unit, and enough work to pay for the three extra passes
    const int64_t tiles = ((M + 127) / 128) * ((KN + 127) / 128);
    return !off && tiles >= 256 && M <= 0x7fffffffLL && (double)M * KN * 64.0 * K >= 1.2e10;
}

// its buffers: channel-packed planes, Packing-2 rows, the rows as matrix-core fragments (each 256-byte aligned)
static int64_t gemm_route_plane_bytes(int N, int C, int H, int W) {
    return (ftnn_pack_scratch_bytes(N, C, H, W, 1) + 255) / 256 * 256;
}
static int64_t gemm_route_row_bytes(int64_t M, int Kw) { return (M * Kw * 16 + 255) / 256 * 256; }

// operand region of the fp4 layer for this shape, whichever form it takes
int64_t conv_f4_operand_bytes(int N, int C, int H, int W, int KH, int KW, int OH, int OW, int KN, int W_stride) {
    if (dense_f4_applies(C, KH, KW)) return conv_f4_dense_bytes(N, C, H, W, KH, KW, OH, OW);
    int64_t bytes = conv_f4_p4_bytes(N, C, H, W);
    const int64_t M = (int64_t)N * OH * OW;
    // the tile kernel's layout of the same input: a little larger where the width is no multiple of the stride
    const int64_t t4 = quantize_f4_tiled_bytes(N, C, H, W, W_stride);
    if (conv_f4_tile_route(M, KN, cpack_of(C), KH * KW, t4, 0, W_stride)) bytes = std::max(bytes, (t4 + 255) / 256 * 256);
    if (conv_f4_gemm_route(M, KN, cpack_of(C) * KH * KW)) {
        const int Kw = conv_f4_weight_words(C, KH, KW);
        const int64_t route = gemm_route_plane_bytes(N, C, H, W) + gemm_route_row_bytes(M, Kw) +
                              (mfma_fragment_bytes(true, M, Kw) + 255) / 256 * 256;
        if (route > bytes) bytes = route;
    }
    return bytes;
}

// words per expanded weight row on the fp4 layer path
int conv_f4_weight_words(int C, int KH, int KW) {
    int T, Kd;
    if (dense_f4_applies(C, KH, KW)) {
        dense_applies(C, KH, KW, &T, &Kd);
        return round4(Kd);
    }
    return round4(cpack_of(C) * KH * KW);
}

// the matrix-core layer with the weights already expanded (d_wf); d_p4 takes the quantised input
int conv_f4_expanded(int type, const float* d_x, const float* d_thr, const void* d_wf, int N, int C, int H,
                           int W, int KN, int KH, int KW, int H_pad, int W_pad, int H_stride, int W_stride,
                           float prelu_alpha, void* d_p4, float* d_y, hipStream_t st, const QuantOut& qo) {
    const int OH = out_dim(H, H_pad, KH, H_stride), OW = out_dim(W, W_pad, KW, W_stride);
    const bool act_ternary = (type == kTNN || type == kTBN);
    hipError_t e = hipSuccess;
    if (dense_f4_applies(C, KH, KW)) {
        // few channels: several taps per 64-lane word, materialised per output pixel; the layer is then a 1x1
        // layer with Kd words per pixel over the OH x OW output pixels
        if (!d_x) return fail(FTNN_EINVAL, "a few-channel layer takes fp32 input");
        static const bool fused_off = getenv("FTNN_NO_FUSED_STEM") != nullptr;   // tuning aid: the two-kernel form
        if (stem_f4_lds_bytes(C, KH, KW, H_stride, W_stride) > 0 && !fused_off) {
            e = launch_stem_f4(type, d_x, d_thr, d_wf, N, C, H, W, KN, KH, KW, H_pad, W_pad, H_stride, W_stride,
                               prelu_alpha, d_y, st, qo);
            return e == hipSuccess ? FTNN_OK : hip_fail(e, "fp4 first-layer launch");
        }
        int T, Kd;
        dense_applies(C, KH, KW, &T, &Kd);
        void* d_a4 = static_cast<char*>(d_p4) + dense_f4_pq_bytes(N, H, W);
        e = launch_dense_rows_f4(act_ternary, d_x, d_thr, N, C, H, W, H_pad, W_pad, KH, KW, H_stride, W_stride, d_p4,
                                 d_a4, st);
        if (e != hipSuccess) return hip_fail(e, "fp4 dense rows launch");
        const ConvGeom cg = {OH, OW, Kd, OH, OW, 1, Kd, 0, 0, 1, 1,
                             make_fastdiv((uint32_t)OW), make_fastdiv((uint32_t)Kd), make_fastdiv(1u)};
        e = launch_conv_f4(type, d_a4, d_wf, cg, N, KN, C * KH * KW, prelu_alpha, d_y, st, qo);
        return e == hipSuccess ? FTNN_OK : hip_fail(e, "fp4 conv launch");
    }
    const int64_t M = (int64_t)N * OH * OW;
    const bool tiles = d_x && qo.mode == 0 && conv_f4_tile_route(M, KN, cpack_of(C), KH * KW, quantize_f4_tiled_bytes(N, C, H, W, W_stride), W_pad, W_stride);
    if (d_x && qo.mode == 0 && !tiles && conv_f4_gemm_route(M, KN, cpack_of(C) * KH * KW)) {
        const int Kw = conv_f4_weight_words(C, KH, KW);
        char* base = static_cast<char*>(d_p4);
        int64_t* d_rows = reinterpret_cast<int64_t*>(base + gemm_route_plane_bytes(N, C, H, W));
        void* d_af = reinterpret_cast<char*>(d_rows) + gemm_route_row_bytes(M, Kw);
        e = launch_quantize_im2row(act_ternary, d_x, d_thr, N, C, H, W, H_pad, W_pad, KH, KW, H_stride, W_stride, d_rows,
                                   base, st);
        if (e != hipSuccess) return hip_fail(e, "quantise + im2row launch");
        e = launch_mfma_expand(true, act_ternary, d_rows, (int)M, Kw, d_af, st);
        if (e != hipSuccess) return hip_fail(e, "row expansion launch");
        e = launch_mfma_gemm(true, type, d_af, d_wf, M, OH * OW, KN, Kw, C * KH * KW, prelu_alpha, d_y, st);
        return e == hipSuccess ? FTNN_OK : hip_fail(e, "matrix-core GEMM launch");
    }
    const ConvGeom cg = {H, W, cpack_of(C), OH, OW, KW, cpack_of(C) * KH * KW, H_pad, W_pad, H_stride, W_stride,
                         make_fastdiv((uint32_t)OW), make_fastdiv((uint32_t)cpack_of(C)), make_fastdiv((uint32_t)KW)};
    // many tiles, fp32 input and result: workgroup tiles staged through LDS, gathered from the quantised input in the
    // tile kernel's own layout
    if (tiles) {
        e = launch_quantize_f4_tiled(act_ternary, d_x, d_thr, N, C, H, W, W_stride, d_p4, st);
        if (e != hipSuccess) return hip_fail(e, "fp4 quantize launch");
        e = launch_conv_f4_tiles(type, d_p4, d_wf, cg, N, KN, C * KH * KW, prelu_alpha, d_y, st);
        return e == hipSuccess ? FTNN_OK : hip_fail(e, "fp4 conv tile launch");
    }
    if (d_x) e = launch_quantize_f4(act_ternary, d_x, d_thr, N, C, H, W, d_p4, st);   // else d_p4 is ready
    if (e != hipSuccess) return hip_fail(e, "fp4 quantize launch");
    e = launch_conv_f4(type, d_p4, d_wf, cg, N, KN, C * KH * KW, prelu_alpha, d_y, st, qo);
    return e == hipSuccess ? FTNN_OK : hip_fail(e, "fp4 conv launch");
}

// the vector-ALU layer: quantise to bit planes, then the implicit-im2row GEMM (or, for few channels, the dense
// re-packing and the plain GEMM)
int conv_valu(int type, const float* d_x, const float* d_thr, const int64_t* d_qw, int N, int C, int H, int W,
              int KN, int KH, int KW, int H_pad, int W_pad, int H_stride, int W_stride, float prelu_alpha,
              void* d_scratch, float* d_y, hipStream_t st, const QuantOut& qo, bool weights_prepared) {
    const int OH = out_dim(H, H_pad, KH, H_stride), OW = out_dim(W, W_pad, KW, W_stride);
    const bool act_ternary = (type == kTNN || type == kTBN);
    const bool w_ternary = (type == kTNN || type == kBTN);
    hipError_t e = launch_quantize(act_ternary, d_x, d_thr, N, C, H, W, d_scratch, st);
    if (e != hipSuccess) return hip_fail(e, "quantize launch");
    int T, Kd;
    if (dense_applies(C, KH, KW, &T, &Kd)) {
        // few channels: re-pack both operands with several taps per word and run the plain GEMM
        char* base = static_cast<char*>(d_scratch);
        const int64_t p_bytes = (ftnn_pack_scratch_bytes(N, C, H, W, act_ternary) + 255) / 256 * 256;
        const int64_t rows_bytes =
            ((int64_t)N * OH * OW * round4(Kd) * (act_ternary ? 16 : 8) + 255) / 256 * 256;
        int64_t* d_rows = reinterpret_cast<int64_t*>(base + p_bytes);
        const int64_t* d_wd = d_qw;   // prepared weights are the re-packed rows already
        e = launch_dense_rows(act_ternary, d_scratch, N, C, H, W, H_pad, W_pad, KH, KW, H_stride, W_stride,
                              d_rows, st);
        if (e != hipSuccess) return hip_fail(e, "dense rows launch");
        if (!weights_prepared) {
            int64_t* d_tmp = reinterpret_cast<int64_t*>(base + p_bytes + rows_bytes);
            e = launch_dense_weights(w_ternary, d_qw, KN, C, KH, KW, d_tmp, st);
            if (e != hipSuccess) return hip_fail(e, "dense weights launch");
            d_wd = d_tmp;
        }
        e = launch_mm(type, d_rows, d_wd, (int64_t)N * OH * OW, OH * OW, KN, round4(Kd), C * KH * KW,
                      prelu_alpha, d_y, st, qo);
        return e == hipSuccess ? FTNN_OK : hip_fail(e, "mm launch");
    }
    const ConvGeom cg = {H, W, cpack_of(C), OH, OW, KW, cpack_of(C) * KH * KW, H_pad, W_pad, H_stride, W_stride,
                         make_fastdiv((uint32_t)OW), make_fastdiv((uint32_t)cpack_of(C)), make_fastdiv((uint32_t)KW)};
    e = launch_mm_implicit(type, d_scratch, d_qw, cg, N, KN, C * KH * KW, prelu_alpha, d_y, st, qo);
    return e == hipSuccess ? FTNN_OK : hip_fail(e, "implicit-im2row mm launch");
}

// ---- the scratch memory of ftnn_conv_static ----
// Device memory that exists from the moment the code object is loaded until the process ends, one copy per GPU,
// so that a caller who may not allocate (a stream under graph capture, a serving loop, a harness that forbids
// hipMalloc) still has somewhere to put a layer's quantised input and weight fragments.  `scratch` is the
// host-side handle of that array, not a device address: the address of each GPU's copy comes from
// hipGetSymbolAddress, once per device, and is what every launch below is given.
constexpr int64_t kStaticScratchBytes = FTNN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void* g_static_scratch[kMaxDevices] = {};
static std::mutex g_static_scratch_mutex;

// address of the current device's copy of `scratch`; nullptr (and the error text set) on failure
static void* static_scratch_of_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        hip_fail(e, "hipGetDevice");
        return nullptr;
    }
    if (dev < 0 || dev >= kMaxDevices) {
        fail(FTNN_EINVAL, "device ordinal %d beyond the %d this library keeps scratch for", dev, kMaxDevices);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (!g_static_scratch[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            hip_fail(e, "hipGetSymbolAddress(scratch)");
            return nullptr;
        }
        g_static_scratch[dev] = ptr;
    }
    return g_static_scratch[dev];
}

}  // namespace ftnn

using namespace ftnn;

extern "C" {

const char* ftnn_last_error(void) { return g_err; }

const char* ftnn_version(void) { return "ftnn-hip 0.1 gfx950"; }

int ftnn_out_dim(int in, int pad, int k, int stride) { return out_dim(in, pad, k, stride); }

int64_t ftnn_row_words(int C, int KH, int KW, int ternary) {
    if (C <= 0 || KH <= 0 || KW <= 0) return 0;
    int64_t k;   // the window alone can exceed 64 bits: KH * KW up to 2^62 times 2^25 channel words
    if (__builtin_mul_overflow((int64_t)KH, (int64_t)KW, &k) || __builtin_mul_overflow(k, ((int64_t)C + 63) / 64, &k)) return 0;
    if (k > kMaxRowWords) return 0;
    const int64_t kw = (k + 3) / 4 * 4;
    return ternary ? 2 * kw : kw;
}

int64_t ftnn_pack_scratch_bytes(int N, int C, int H, int W, int ternary) {
    if (N <= 0 || C <= 0 || H <= 0 || W <= 0) return 0;
    int64_t bytes;   // 0 for a tensor whose packed copy does not fit 63 bits (no such tensor passes the shape checks)
    if (__builtin_mul_overflow((int64_t)N * cpack_of(C), (int64_t)H * W, &bytes) ||
        __builtin_mul_overflow(bytes, (int64_t)(ternary ? 16 : 8), &bytes))
        return 0;
    return bytes;
}

// Layer engine by shape, from measurements on MI355X: the fp4 matrix-core kernel wins wherever it
// applies.
static int select_conv_engine(int type, int N, int C, int H, int W, int KN, int KH, int KW, int OH, int OW) {
    (void)type; (void)N; (void)H; (void)W; (void)KN; (void)OH; (void)OW;
    int T, Kd;
    // few channels: the dense re-packing feeds the matrix cores for C <= 8, the vector ALU beyond
    if (dense_applies(C, KH, KW, &T, &Kd)) return C <= 8 ? FTNN_ENGINE_MFMA_F4 : FTNN_ENGINE_VALU;
    if (64LL * cpack_of(C) * KH * KW >= (1LL << 24)) return FTNN_ENGINE_VALU;   // fp32 accumulation must stay exact
    return FTNN_ENGINE_MFMA_F4;
}

int ftnn_select_conv_engine(int type, int N, int C, int H, int W, int KN, int KH, int KW, int H_pad, int W_pad,
                            int H_stride, int W_stride) {
    int OH, OW;
    if (check_conv_shape(N, C, H, W, H_pad, W_pad, KH, KW, H_stride, W_stride, &OH, &OW) != FTNN_OK || KN <= 0)
        return FTNN_ENGINE_VALU;
    return select_conv_engine(type, N, C, H, W, KN, KH, KW, OH, OW);
}

int64_t ftnn_conv_scratch_bytes(int type, int N, int C, int H, int W, int KN, int KH, int KW, int H_pad,
                                int W_pad, int H_stride, int W_stride) {
    int OH, OW;
    if (check_conv_shape(N, C, H, W, H_pad, W_pad, KH, KW, H_stride, W_stride, &OH, &OW) != FTNN_OK || KN <= 0)
        return 0;
    const bool at = (type == kTNN || type == kTBN), wt = (type == kTNN || type == kBTN);
    int64_t bytes = ftnn_pack_scratch_bytes(N, C, H, W, at);
    int T, Kd;
    if (dense_applies(C, KH, KW, &T, &Kd)) {
        bytes = (bytes + 255) / 256 * 256;
        bytes += ((int64_t)N * OH * OW * round4(Kd) * (at ? 16 : 8) + 255) / 256 * 256;
        bytes += (int64_t)KN * round4(Kd) * (wt ? 16 : 8);
    }
    // enough for either engine, so that one buffer serves ftnn_conv and ftnn_conv_engine
    // fp4: operand region, fragments of the weights and, on the dense path, the re-packed weight rows
    int64_t f4 = conv_f4_operand_bytes(N, C, H, W, KH, KW, OH, OW, KN, W_stride) +
                 (mfma_fragment_bytes(true, KN, conv_f4_weight_words(C, KH, KW)) + 255) / 256 * 256;
    if (dense_f4_applies(C, KH, KW)) f4 += (int64_t)KN * conv_f4_weight_words(C, KH, KW) * (wt ? 16 : 8);
    return bytes > f4 ? bytes : f4;
}

int ftnn_quantize_im2row(int ternary, const float* d_x, const float* d_thr, int N, int C, int H,
                         int W, int H_pad, int W_pad, int kH, int kW, int H_stride, int W_stride,
                         int64_t* d_out, void* d_scratch, void* stream) {
    int OH, OW;
    int rc = check_conv_shape(N, C, H, W, H_pad, W_pad, kH, kW, H_stride, W_stride, &OH, &OW);
    if (rc != FTNN_OK) return rc;
    if (!d_x || !d_thr || !d_out || !d_scratch) return fail(FTNN_EINVAL, "null device pointer");
    if (!aligned16(d_out) || !aligned16(d_scratch))
        return fail(FTNN_EINVAL, "d_out and d_scratch must be 16-byte aligned");
    hipError_t e = launch_quantize_im2row(ternary != 0, d_x, d_thr, N, C, H, W, H_pad, W_pad, kH,
                                          kW, H_stride, W_stride, d_out, d_scratch,
                                          (hipStream_t)stream);
    return e == hipSuccess ? FTNN_OK : hip_fail(e, "quantize_im2row launch");
}

int ftnn_mm(int type, const int64_t* d_a, const int64_t* d_b, int N, int OH, int OW, int KN, int K,
            int K_unpack, float prelu_alpha, float* d_y, void* stream) {
    if (type < kTNN || type > kBNN) return fail(FTNN_EINVAL, "unknown network type %d", type);
    if (N <= 0 || OH <= 0 || OW <= 0 || KN <= 0 || K <= 0)
        return fail(FTNN_EINVAL, "non-positive GEMM dimension");
    if (K > kMaxRowWords) return fail(FTNN_EINVAL, "K = %d words above the supported %d", K, kMaxRowWords);
    if (!d_a || !d_b || !d_y) return fail(FTNN_EINVAL, "null device pointer");
    if (!aligned16(d_a) || !aligned16(d_b))
        return fail(FTNN_EINVAL, "GEMM operands must be 16-byte aligned");
    const int64_t M = (int64_t)N * OH * OW;
    if (M > 0x7fffffffLL || (int64_t)OH * OW > 0x7fffffffLL)
        return fail(FTNN_EINVAL, "more than 2^31-1 output rows");
    hipError_t e = launch_mm(type, d_a, d_b, M, OH * OW, KN, round4(K), K_unpack, prelu_alpha, d_y,
                             (hipStream_t)stream);
    return e == hipSuccess ? FTNN_OK : hip_fail(e, "mm launch");
}

// Engine choice by shape, from measurements on MI355X (m x m x 8m, whole calls from packed rows, device time): the
// matrix-core path pays one launch that expands both operands and works on tiles of 64 x 64, 128 x 128 or 256 x 256 by
// tile count; the vector-ALU kernel is one launch near 0.3 PMAC/s.  m = 512 (1.1e9 lane-MACs): 12.0 us on the vector
// ALU against 13.3 us on fp4; 576 (1.5e9): 13.9 against 13.0; 640 (2.1e9): 17.8 against 13.3; 768: 23.8 against 15.1;
// other shapes with 1.6e9 - 1.9e9 lane-MACs are ties within 1 us either way, hence fp4 from 2e9 on.
static int select_engine(int type, int64_t M, int KN, int Kw) {
    (void)type;
    const double lane_macs = (double)M * KN * 64.0 * Kw;
    if (lane_macs >= 2e9 && KN >= 128 && Kw <= kMaxF4GemmWords) return FTNN_ENGINE_MFMA_F4;
    return FTNN_ENGINE_VALU;
}

int ftnn_select_engine(int type, int N, int OH, int OW, int KN, int K) {
    if (N <= 0 || OH <= 0 || OW <= 0 || KN <= 0 || K <= 0 || K > kMaxRowWords) return FTNN_ENGINE_VALU;
    return select_engine(type, (int64_t)N * OH * OW, KN, round4(K));
}

int64_t ftnn_mm_scratch_bytes(int engine, int type, int N, int OH, int OW, int KN, int K) {
    if (N <= 0 || OH <= 0 || OW <= 0 || KN <= 0 || K <= 0 || K > kMaxRowWords) return 0;
    const int64_t M = (int64_t)N * OH * OW;
    const int Kw = round4(K);
    if (engine == FTNN_ENGINE_AUTO) engine = select_engine(type, M, KN, Kw);
    if (engine != FTNN_ENGINE_MFMA_I8 && engine != FTNN_ENGINE_MFMA_F4) return 0;
    if (engine == FTNN_ENGINE_MFMA_F4) return mfma_f4_mm_scratch_bytes(M, KN, Kw);
    return mfma_fragment_bytes(false, M, Kw) + mfma_fragment_bytes(false, KN, Kw);
}

static int check_mfma_engine(int engine, int Kw) {
    if (engine != FTNN_ENGINE_MFMA_I8 && engine != FTNN_ENGINE_MFMA_F4)
        return fail(FTNN_EINVAL, "engine %d is not a matrix-core engine", engine);
    if (engine == FTNN_ENGINE_MFMA_F4 && Kw > kMaxF4GemmWords)
        return fail(FTNN_EINVAL, "K too long for exact fp32 accumulation; use the int8 engine");
    return FTNN_OK;
}

int64_t ftnn_expand_bytes(int engine, int rows, int K) {
    if (rows <= 0 || K <= 0 || K > kMaxRowWords || (engine != FTNN_ENGINE_MFMA_I8 && engine != FTNN_ENGINE_MFMA_F4)) return 0;
    return engine == FTNN_ENGINE_MFMA_F4 ? mfma_packed4_bytes(rows, round4(K)) : mfma_fragment_bytes(false, rows, round4(K));
}

int ftnn_expand_rows(int engine, int ternary, const int64_t* d_rows, int rows, int K, void* d_out,
                     void* stream) {
    if (rows <= 0 || K <= 0 || K > kMaxRowWords) return fail(FTNN_EINVAL, "dimension non-positive or K too long");
    int rc = check_mfma_engine(engine, round4(K));
    if (rc != FTNN_OK) return rc;
    if (!d_rows || !d_out || !aligned16(d_rows) || !aligned16(d_out))
        return fail(FTNN_EINVAL, "null or misaligned device pointer");
    hipError_t e = engine == FTNN_ENGINE_MFMA_F4
                       ? launch_mfma_pack4(ternary != 0, d_rows, rows, round4(K), d_out, (hipStream_t)stream)
                       : launch_mfma_expand(false, ternary != 0, d_rows, rows, round4(K), d_out, (hipStream_t)stream);
    return e == hipSuccess ? FTNN_OK : hip_fail(e, "expand launch");
}

int ftnn_mm_expanded(int engine, int type, const void* d_a_exp, const void* d_b_exp, int N, int OH, int OW,
                     int KN, int K, int K_unpack, float prelu_alpha, float* d_y, void* stream) {
    if (type < kTNN || type > kBNN) return fail(FTNN_EINVAL, "unknown network type %d", type);
    if (N <= 0 || OH <= 0 || OW <= 0 || KN <= 0 || K <= 0)
        return fail(FTNN_EINVAL, "non-positive GEMM dimension");
    if (K > kMaxRowWords) return fail(FTNN_EINVAL, "K = %d words above the supported %d", K, kMaxRowWords);
    int rc = check_mfma_engine(engine, round4(K));
    if (rc != FTNN_OK) return rc;
    const int64_t M = (int64_t)N * OH * OW;
    if (M > 0x7fffffffLL) return fail(FTNN_EINVAL, "more than 2^31-1 output rows");
    if (!d_a_exp || !d_b_exp || !d_y || !aligned16(d_a_exp) || !aligned16(d_b_exp))
        return fail(FTNN_EINVAL, "null or misaligned device pointer");
    hipError_t e = engine == FTNN_ENGINE_MFMA_F4
                       ? launch_mfma_gemm_packed4(type, d_a_exp, d_b_exp, M, OH * OW, KN, round4(K), K_unpack, prelu_alpha, d_y,
                                                  (hipStream_t)stream)
                       : launch_mfma_gemm(false, type, d_a_exp, d_b_exp, M, OH * OW, KN, round4(K), K_unpack, prelu_alpha, d_y,
                                          (hipStream_t)stream);
    return e == hipSuccess ? FTNN_OK : hip_fail(e, "mfma gemm launch");
}

int ftnn_mm_engine(int engine, int type, const int64_t* d_a, const int64_t* d_b, int N, int OH, int OW,
                   int KN, int K, int K_unpack, float prelu_alpha, float* d_y, void* d_scratch,
                   int64_t scratch_bytes, void* stream) {
    if (engine < FTNN_ENGINE_AUTO || engine > FTNN_ENGINE_MFMA_F4)
        return fail(FTNN_EINVAL, "unknown engine %d", engine);
    if (type < kTNN || type > kBNN) return fail(FTNN_EINVAL, "unknown network type %d", type);
    if (N <= 0 || OH <= 0 || OW <= 0 || KN <= 0 || K <= 0)
        return fail(FTNN_EINVAL, "non-positive GEMM dimension");
    if (K > kMaxRowWords) return fail(FTNN_EINVAL, "K = %d words above the supported %d", K, kMaxRowWords);
    const int64_t M = (int64_t)N * OH * OW;
    const int Kw = round4(K);
    if (engine == FTNN_ENGINE_AUTO) {
        engine = select_engine(type, M, KN, Kw);
        // AUTO never fails for lack of scratch: it falls back to the engine that needs none
        if (engine != FTNN_ENGINE_VALU &&
            (!d_scratch || scratch_bytes < ftnn_mm_scratch_bytes(engine, type, N, OH, OW, KN, K)))
            engine = FTNN_ENGINE_VALU;
    }
    if (engine == FTNN_ENGINE_VALU)
        return ftnn_mm(type, d_a, d_b, N, OH, OW, KN, K, K_unpack, prelu_alpha, d_y, stream);
    if (!d_a || !d_b || !d_y) return fail(FTNN_EINVAL, "null device pointer");
    if (!aligned16(d_a) || !aligned16(d_b)) return fail(FTNN_EINVAL, "GEMM operands must be 16-byte aligned");
    if (M > 0x7fffffffLL) return fail(FTNN_EINVAL, "more than 2^31-1 output rows");
    const bool f4 = engine == FTNN_ENGINE_MFMA_F4;
    if (f4 && Kw > kMaxF4GemmWords)
        return fail(FTNN_EINVAL, "K too long for exact fp32 accumulation; use the int8 engine");
    const int64_t need = ftnn_mm_scratch_bytes(engine, type, N, OH, OW, KN, K);
    if (!d_scratch || !aligned16(d_scratch) || scratch_bytes < need)
        return fail(FTNN_EINVAL, "engine %d needs %lld bytes of 16-byte aligned scratch", engine, (long long)need);
    hipError_t e = launch_mm_mfma(f4, type, d_a, d_b, M, OH * OW, KN, Kw, K_unpack, prelu_alpha, d_y,
                                  d_scratch, (hipStream_t)stream);
    return e == hipSuccess ? FTNN_OK : hip_fail(e, "mfma mm launch");
}

int ftnn_conv_engine(int engine, int type, const float* d_x, const float* d_thr, const int64_t* d_qw, int N,
                     int C, int H, int W, int KN, int KH, int KW, int H_pad, int W_pad, int H_stride,
                     int W_stride, float prelu_alpha, void* d_scratch, float* d_y, void* stream) {
    if (type < kTNN || type > kBNN) return fail(FTNN_EINVAL, "unknown network type %d", type);
    int OH, OW;
    int rc = check_conv_shape(N, C, H, W, H_pad, W_pad, KH, KW, H_stride, W_stride, &OH, &OW);
    if (rc != FTNN_OK) return rc;
    if (KN <= 0) return fail(FTNN_EINVAL, "non-positive kernel count");
    if (!d_x || !d_thr || !d_qw || !d_scratch || !d_y) return fail(FTNN_EINVAL, "null device pointer");
    if (!aligned16(d_scratch) || !aligned16(d_qw))
        return fail(FTNN_EINVAL, "d_scratch and d_qw must be 16-byte aligned");
    if ((int64_t)N * OH * OW > 0x7fffffffLL) return fail(FTNN_EINVAL, "more than 2^31-1 output rows");
    const bool fits_f4 = (int64_t)N * H * W * cpack_of(C) <= 0x7fffffffLL &&
                         (int64_t)N * OH * OW * conv_f4_weight_words(C, KH, KW) <= 0x7fffffffLL;
    if (engine == FTNN_ENGINE_AUTO)   // a layer beyond the fp4 kernel's 32-bit pixel indices goes to the vector ALU
        engine = fits_f4 ? select_conv_engine(type, N, C, H, W, KN, KH, KW, OH, OW) : FTNN_ENGINE_VALU;
    const bool w_ternary = (type == kTNN || type == kBTN);
    if (engine == FTNN_ENGINE_MFMA_F4) {
        const int Kw = conv_f4_weight_words(C, KH, KW);
        if (64LL * Kw >= (1LL << 24))
            return fail(FTNN_EINVAL, "K too long for exact fp32 accumulation; use the vector-ALU engine");
        if (!fits_f4) return fail(FTNN_EINVAL, "more than 2^31-1 input pixel words: use the vector-ALU engine");
        char* d_wf = static_cast<char*>(d_scratch) + conv_f4_operand_bytes(N, C, H, W, KH, KW, OH, OW, KN, W_stride);
        const int64_t* rows = d_qw;
        hipError_t e;
        if (dense_f4_applies(C, KH, KW)) {   // the weights take the same re-packing first
            int64_t* d_wd = reinterpret_cast<int64_t*>(d_wf + (mfma_fragment_bytes(true, KN, Kw) + 255) / 256 * 256);
            e = launch_dense_weights(w_ternary, d_qw, KN, C, KH, KW, d_wd, (hipStream_t)stream);
            if (e != hipSuccess) return hip_fail(e, "dense weights launch");
            rows = d_wd;
        }
        e = launch_mfma_expand(true, w_ternary, rows, KN, Kw, d_wf, (hipStream_t)stream);
        if (e != hipSuccess) return hip_fail(e, "weight expansion launch");
        return conv_f4_expanded(type, d_x, d_thr, d_wf, N, C, H, W, KN, KH, KW, H_pad, W_pad, H_stride, W_stride,
                                prelu_alpha, d_scratch, d_y, (hipStream_t)stream, QuantOut());
    }
    if (engine != FTNN_ENGINE_VALU) return fail(FTNN_EINVAL, "layer engine %d (vector ALU and fp4 only)", engine);
    return conv_valu(type, d_x, d_thr, d_qw, N, C, H, W, KN, KH, KW, H_pad, W_pad, H_stride, W_stride, prelu_alpha,
                     d_scratch, d_y, (hipStream_t)stream, QuantOut(), false);
}

// Weights in the form the layer's engine reads them, made once per layer instead of once per call.
static int64_t prepared_bytes(int type, int C, int KN, int KH, int KW, int64_t* tmp_off) {
    const bool wt = (type == kTNN || type == kBTN);
    const int engine = select_conv_engine(type, 1, C, KH, KW, KN, KH, KW, 1, 1);
    int T, Kd;
    const bool dense = dense_applies(C, KH, KW, &T, &Kd);
    if (tmp_off) *tmp_off = 0;
    if (engine == FTNN_ENGINE_MFMA_F4) {
        const int64_t frag = (mfma_fragment_bytes(true, KN, conv_f4_weight_words(C, KH, KW)) + 255) / 256 * 256;
        if (tmp_off) *tmp_off = frag;
        // the dense path expands the re-packed rows, which need a place of their own
        return frag + (dense_f4_applies(C, KH, KW) ? (int64_t)KN * round4(Kd) * (wt ? 16 : 8) : 0);
    }
    return (int64_t)KN * (dense ? round4(Kd) : round4(cpack_of(C) * KH * KW)) * (wt ? 16 : 8);
}

int64_t ftnn_conv_weights_bytes(int type, int C, int KN, int KH, int KW) {
    if (type < kTNN || type > kBNN || C <= 0 || KN <= 0 || KH <= 0 || KW <= 0) return 0;
    if (!row_fits(C, KH, KW)) return 0;
    return prepared_bytes(type, C, KN, KH, KW, nullptr);
}

int ftnn_conv_prepare_weights(int type, const int64_t* d_qw, int C, int KN, int KH, int KW, void* d_prepared,
                              void* stream) {
    if (type < kTNN || type > kBNN) return fail(FTNN_EINVAL, "unknown network type %d", type);
    if (C <= 0 || KN <= 0 || KH <= 0 || KW <= 0) return fail(FTNN_EINVAL, "non-positive dimension");
    if (!row_fits(C, KH, KW))
        return fail(FTNN_EINVAL, "more than %d words per weight row", kMaxRowWords);
    if (!d_qw || !d_prepared || !aligned16(d_qw) || !aligned16(d_prepared))
        return fail(FTNN_EINVAL, "null or misaligned device pointer");
    const bool wt = (type == kTNN || type == kBTN);
    hipStream_t st = (hipStream_t)stream;
    int64_t tmp_off;
    const int64_t bytes = prepared_bytes(type, C, KN, KH, KW, &tmp_off);
    const int engine = select_conv_engine(type, 1, C, KH, KW, KN, KH, KW, 1, 1);
    int T, Kd;
    const bool dense = dense_applies(C, KH, KW, &T, &Kd);
    hipError_t e;
    if (engine == FTNN_ENGINE_MFMA_F4) {
        const int64_t* rows = d_qw;
        if (dense_f4_applies(C, KH, KW)) {
            int64_t* d_wd = reinterpret_cast<int64_t*>(static_cast<char*>(d_prepared) + tmp_off);
            e = launch_dense_weights(wt, d_qw, KN, C, KH, KW, d_wd, st);
            if (e != hipSuccess) return hip_fail(e, "dense weights launch");
            rows = d_wd;
        }
        e = launch_mfma_expand(true, wt, rows, KN, conv_f4_weight_words(C, KH, KW), d_prepared, st);
        return e == hipSuccess ? FTNN_OK : hip_fail(e, "weight expansion launch");
    }
    if (dense) {
        e = launch_dense_weights(wt, d_qw, KN, C, KH, KW, static_cast<int64_t*>(d_prepared), st);
        return e == hipSuccess ? FTNN_OK : hip_fail(e, "dense weights launch");
    }
    e = hipMemcpyAsync(d_prepared, d_qw, (size_t)bytes, hipMemcpyDeviceToDevice, st);
    return e == hipSuccess ? FTNN_OK : hip_fail(e, "weight copy");
}

int ftnn_conv_prepared(int type, const float* d_x, const float* d_thr, const void* d_prepared, int N, int C, int H,
                       int W, int KN, int KH, int KW, int H_pad, int W_pad, int H_stride, int W_stride,
                       float prelu_alpha, void* d_scratch, float* d_y, void* stream) {
    if (type < kTNN || type > kBNN) return fail(FTNN_EINVAL, "unknown network type %d", type);
    int OH, OW;
    int rc = check_conv_shape(N, C, H, W, H_pad, W_pad, KH, KW, H_stride, W_stride, &OH, &OW);
    if (rc != FTNN_OK) return rc;
    if (KN <= 0) return fail(FTNN_EINVAL, "non-positive kernel count");
    if (!d_x || !d_thr || !d_prepared || !d_scratch || !d_y) return fail(FTNN_EINVAL, "null device pointer");
    if (!aligned16(d_scratch) || !aligned16(d_prepared))
        return fail(FTNN_EINVAL, "d_scratch and d_prepared must be 16-byte aligned");
    if ((int64_t)N * OH * OW > 0x7fffffffLL) return fail(FTNN_EINVAL, "more than 2^31-1 output rows");
    if (select_conv_engine(type, N, C, H, W, KN, KH, KW, OH, OW) == FTNN_ENGINE_MFMA_F4) {
        if ((int64_t)N * H * W * cpack_of(C) > 0x7fffffffLL ||
            (int64_t)N * OH * OW * conv_f4_weight_words(C, KH, KW) > 0x7fffffffLL)
            return fail(FTNN_EINVAL, "more than 2^31-1 input pixel words");
        return conv_f4_expanded(type, d_x, d_thr, d_prepared, N, C, H, W, KN, KH, KW, H_pad, W_pad, H_stride,
                                W_stride, prelu_alpha, d_scratch, d_y, (hipStream_t)stream, QuantOut());
    }
    return conv_valu(type, d_x, d_thr, static_cast<const int64_t*>(d_prepared), N, C, H, W, KN, KH, KW, H_pad, W_pad,
                     H_stride, W_stride, prelu_alpha, d_scratch, d_y, (hipStream_t)stream, QuantOut(), true);
}

int ftnn_conv(int type, const float* d_x, const float* d_thr, const int64_t* d_qw, int N, int C,
              int H, int W, int KN, int KH, int KW, int H_pad, int W_pad, int H_stride, int W_stride,
              float prelu_alpha, void* d_scratch, float* d_y, void* stream) {
    return ftnn_conv_engine(FTNN_ENGINE_AUTO, type, d_x, d_thr, d_qw, N, C, H, W, KN, KH, KW, H_pad, W_pad,
                            H_stride, W_stride, prelu_alpha, d_scratch, d_y, stream);
}

int ftnn_conv_static(int type, const float* d_x, const float* d_thr, const int64_t* d_qw, int N, int C, int H, int W,
                     int KN, int KH, int KW, int H_pad, int W_pad, int H_stride, int W_stride, float prelu_alpha,
                     float* d_y, void* stream) {
    if (type < kTNN || type > kBNN) return fail(FTNN_EINVAL, "unknown network type %d", type);
    int OH, OW;
    int rc = check_conv_shape(N, C, H, W, H_pad, W_pad, KH, KW, H_stride, W_stride, &OH, &OW);
    if (rc != FTNN_OK) return rc;
    if (KN <= 0) return fail(FTNN_EINVAL, "non-positive kernel count");
    const int64_t need = ftnn_conv_scratch_bytes(type, N, C, H, W, KN, KH, KW, H_pad, W_pad, H_stride, W_stride);
    if (need <= 0 || need > kStaticScratchBytes)
        return fail(FTNN_EINVAL, "layer needs %lld bytes of scratch, ftnn_conv_static holds %lld: use ftnn_conv with "
                    "a buffer of the caller's", (long long)need, (long long)kStaticScratchBytes);
    void* d_scr = static_scratch_of_current_device();
    if (!d_scr) return FTNN_EHIP;
    return ftnn_conv_engine(FTNN_ENGINE_AUTO, type, d_x, d_thr, d_qw, N, C, H, W, KN, KH, KW, H_pad, W_pad, H_stride,
                            W_stride, prelu_alpha, d_scr, d_y, stream);
}

int ftnn_pack_weights(int ternary, const float* d_w, const float* d_thr, int KN, int C, int KH,
                      int KW, int64_t* d_out, void* stream) {
    if (KN <= 0 || C <= 0 || KH <= 0 || KW <= 0) return fail(FTNN_EINVAL, "non-positive dimension");
    if (!row_fits(C, KH, KW))
        return fail(FTNN_EINVAL, "more than %d words per weight row", kMaxRowWords);
    if (!d_w || !d_thr || !d_out) return fail(FTNN_EINVAL, "null device pointer");
    hipError_t e = launch_pack_weights(ternary != 0, d_w, d_thr, KN, C, KH, KW, d_out,
                                       (hipStream_t)stream);
    return e == hipSuccess ? FTNN_OK : hip_fail(e, "pack_weights launch");
}

int ftnn_pack_gemm_operand(const float* d_x, int I, int J, int64_t* d_out, void* stream) {
    if (I <= 0 || J <= 0) return fail(FTNN_EINVAL, "non-positive dimension");
    // the reference asserts the same (src/utils.c:258)
    if (J % 256 != 0) return fail(FTNN_EINVAL, "J = %d is not a multiple of 256", J);
    if (J / 64 / 4 > 65535) return fail(FTNN_EINVAL, "J = %d too large", J);
    if (!d_x || !d_out) return fail(FTNN_EINVAL, "null device pointer");
    hipError_t e = launch_pack_gemm_operand(d_x, I, J, d_out, (hipStream_t)stream);
    return e == hipSuccess ? FTNN_OK : hip_fail(e, "pack_gemm_operand launch");
}

// ------------------------------------------------- reference entry points

int64_t* t2r_p2_opt(float* x, float* q_thresholds, int N, int C, int H, int W, int H_pad, int W_pad,
                    int kH, int kW, int H_stride, int W_stride) {
    return host_quantize_im2row(true, x, q_thresholds, N, C, H, W, H_pad, W_pad, kH, kW, H_stride,
                                W_stride);
}

int64_t* b2r(float* x, float* q_thresholds, int N, int C, int H, int W, int H_pad, int W_pad, int kH,
             int kW, int H_stride, int W_stride) {
    return host_quantize_im2row(false, x, q_thresholds, N, C, H, W, H_pad, W_pad, kH, kW, H_stride,
                                W_stride);
}

float* mm_tnn(int64_t* a, int64_t* b, int N, int OH, int OW, int KN, int K, float prelu_alpha) {
    return host_mm(kTNN, a, b, N, OH, OW, KN, K, 0, prelu_alpha);
}
float* mm_tbn(int64_t* a, int64_t* b, int N, int OH, int OW, int KN, int K, float prelu_alpha) {
    return host_mm(kTBN, a, b, N, OH, OW, KN, K, 0, prelu_alpha);
}
float* mm_btn(int64_t* a, int64_t* b, int N, int OH, int OW, int KN, int K, float prelu_alpha) {
    return host_mm(kBTN, a, b, N, OH, OW, KN, K, 0, prelu_alpha);
}
float* mm_bnn(int64_t* a, int64_t* b, int N, int OH, int OW, int KN, int K, int K_unpack,
              float prelu_alpha) {
    return host_mm(kBNN, a, b, N, OH, OW, KN, K, K_unpack, prelu_alpha);
}

void tnns_conv(testcase_t* t) {
    std::lock_guard<std::mutex> lock(g_ctx_mutex);
    const int type = (int)t->type;
    const int N = t->batchcount, C = t->channelcount, H = t->inputH, W = t->inputW;
    const int KN = t->kernelcount, KH = t->kernelH, KW = t->kernelW;
    int OH, OW;
    if (type < kTNN || type > kBNN) {
        fail(FTNN_EINVAL, "unknown network type %d", type);
        die("tnns_conv");
    }
    if (check_conv_shape(N, C, H, W, t->paddingH, t->paddingW, KH, KW, t->strideH, t->strideW, &OH,
                         &OW) != FTNN_OK || KN <= 0)
        die("tnns_conv");
    const int w_tern = (type == kTNN || type == kBTN);
    const size_t rows = (size_t)N * OH * OW;
    if (rows > 0x7fffffffull) {
        fail(FTNN_EINVAL, "more than 2^31-1 output rows");
        die("tnns_conv");
    }
    const size_t y_bytes = rows * KN * sizeof(float);
    static const bool trace = getenv("FTNN_HOST_TRACE") != nullptr;   // tuning aid: phase times of every call on stderr
    auto nowus = []() {
        struct timespec ts;
        clock_gettime(CLOCK_MONOTONIC, &ts);
        return ts.tv_sec * 1e6 + ts.tv_nsec * 1e-3;
    };
    const double T0 = nowus();
    float* y = (float*)host_alloc(y_bytes, false);
    const double T1 = nowus();
    float* d_x = (float*)upload(SLOT_X, t->input, (size_t)N * C * H * W * sizeof(float));
    float* d_thr = (float*)upload(SLOT_THR, t->input_thresholds, (size_t)N * sizeof(float));
    const size_t w_bytes = (size_t)KN * ftnn_row_words(C, KH, KW, w_tern) * sizeof(int64_t);
    void* d_scr = dev_buf(SLOT_SCRATCH, (size_t)ftnn_conv_scratch_bytes(type, N, C, H, W, KN, KH, KW, t->paddingH,
                                                                  t->paddingW, t->strideH, t->strideW));
    float* d_y = (float*)dev_buf(SLOT_Y, y_bytes);
    const double T2 = nowus();
    // a layer within the fp4 engine's 32-bit pixel indices (or on the vector ALU) takes its weights prepared
    const bool prepared_ok =
        select_conv_engine(type, N, C, H, W, KN, KH, KW, OH, OW) != FTNN_ENGINE_MFMA_F4 ||
        ((int64_t)N * H * W * cpack_of(C) <= 0x7fffffffLL && (int64_t)rows * conv_f4_weight_words(C, KH, KW) <= 0x7fffffffLL);
    int rc;
    if (prepared_ok) {
        const void* d_prep = prepared_weights(type, t->quantized_kernel_packing2, w_bytes, C, KN, KH, KW);
        rc = ftnn_conv_prepared(type, d_x, d_thr, d_prep, N, C, H, W, KN, KH, KW, t->paddingH, t->paddingW, t->strideH,
                                t->strideW, t->preluAlpha, d_scr, d_y, host_stream());
    } else {
        int64_t* d_w = (int64_t*)upload(SLOT_W, t->quantized_kernel_packing2, w_bytes);
        rc = ftnn_conv(type, d_x, d_thr, d_w, N, C, H, W, KN, KH, KW, t->paddingH, t->paddingW, t->strideH, t->strideW,
                       t->preluAlpha, d_scr, d_y, host_stream());
    }
    if (rc != FTNN_OK) die("tnns_conv");
    const double T3 = nowus();
    if (trace) hip_or_die(hipStreamSynchronize(host_stream()), "hipStreamSynchronize");   // separates kernels from download
    const double T4 = nowus();
    download(y, d_y, y_bytes);
    const double T5 = nowus();
    if (trace)
        fprintf(stderr, "tnns_conv: alloc %.0f, upload %.0f, weights + launch %.0f, kernels %.0f, download %.0f, total %.0f us\n",
                T1 - T0, T2 - T1, T3 - T2, T4 - T3, T5 - T4, T5 - T0);
    t->output = y;  // src/tnns/tnns_cpu_mm_p2.c:119
}

int64_t* ternarize_opt_avx2(float* x, float* q_thresholds, int N, int C, int H, int W) {
    return host_pack_weights(true, x, q_thresholds, N, C, H, W);
}

int64_t* binarize_opt_avx2(float* x, float* q_thresholds, int N, int C, int H, int W) {
    return host_pack_weights(false, x, q_thresholds, N, C, H, W);
}

int64_t* bitpacking2(float* x, int I, int J) { return host_pack_gemm_operand(x, I, J); }

void ftnn_host_forget_weights(void) {
    std::lock_guard<std::mutex> lock(g_ctx_mutex);
    while (!g_weights.empty()) drop_weight_entry(g_weights.size() - 1);
}

void ftnn_host_release_spares(void) { SparePool::get().release(); }

int ftnn_host_hash_uses_aes(void) { return hash128_uses_aes() ? 1 : 0; }

void ftnn_host_hash128(const void* data, int64_t bytes, int portable, uint64_t out[2]) {
    const Hash128 h = portable ? hash128_portable(data, (size_t)bytes, 0) : content_hash(data, (size_t)bytes);
    out[0] = h.lo;
    out[1] = h.hi;
}

int64_t ftnn_host_cached_weight_bytes(void) {
    std::lock_guard<std::mutex> lock(g_ctx_mutex);
    return (int64_t)g_weights_bytes;
}

int64_t ftnn_static_scratch_bytes(void) { return kStaticScratchBytes; }

void tnns_gemm(testcase_tnns_gemm_t* t) {
    // alpha is fixed to 1 (src/tnns/tnns_cpu_mm_p2.c:123)
    float* result = mm_tnn(t->x_packing2, t->w_packing2, t->m, 1, 1, t->n, t->p_packed, 1.0f);
    if (t->output) {
        memcpy(t->output, result, (size_t)t->m * t->n * sizeof(float));
        free(result);
    } else {
        t->output = result;
    }
}

}  // extern "C"
