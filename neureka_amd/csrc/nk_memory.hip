// Device memory and host transfers: the buffer pool behind nk_alloc / nk_free and the pinned staging ring behind
// nk_h2d / nk_d2h.
//
// The reference creates and releases an OpenCL buffer per tensor (J/devices/opencl/OpenCLDevice.java:465,954-966) and
// every operation allocates its output (J/backend/main/algorithms/Broadcast.java:89-92,
// J/backend/main/algorithms/MatMulAlgorithm.java:74-85).  On this device an allocation from the driver costs tens of
// microseconds to milliseconds and a release waits for the stream to drain, so both would cost more than most of
// the kernels between them.  Blocks therefore rest in a pool by size class and change owners without a wait: the
// device's one in-order stream already orders the work of the old owner before the work of the new one.
#include "nk_internal.h"
#include <atomic>
#include <condition_variable>
#include <cstring>
#include <thread>

namespace nk {

// ---- size classes ------------------------------------------------------------------------------------
// Multiples of 256 bytes up to 4 KiB, then eight classes per power of two: at most an eighth of a block is unused.
static uint64_t size_class(uint64_t bytes) {
    if (bytes <= 256) return 256;
    if (bytes <= 4096) return (bytes + 255) & ~(uint64_t)255;
    const int p = 63 - __builtin_clzll(bytes - 1);          // 2^p <= bytes - 1 < 2^(p + 1)
    const uint64_t step = (uint64_t)1 << (p - 3);
    return (bytes + step - 1) & ~(step - 1);
}

static int release_pool(Device* dev) {
    if (dev->pool_bytes == 0) return NK_OK;
    NK_HIP(hipStreamSynchronize(dev->stream));              // queued work may still use a block at rest
    for (auto& cls : dev->pool)
        for (void* p : cls.second) (void)hipFree(p);
    dev->pool.clear();
    dev->pool_bytes = 0;
    return NK_OK;
}

// Makes room for `incoming` more bytes at rest: blocks of the largest classes go back to the driver first.
static int evict_for(Device* dev, uint64_t incoming) {
    bool synced = false;
    while (dev->pool_bytes + incoming > dev->pool_limit && !dev->pool.empty()) {
        auto last = std::prev(dev->pool.end());
        if (last->second.empty()) { dev->pool.erase(last); continue; }
        if (!synced) { NK_HIP(hipStreamSynchronize(dev->stream)); synced = true; }
        (void)hipFree(last->second.back());
        last->second.pop_back();
        dev->pool_bytes -= last->first;
    }
    return NK_OK;
}

// ---- host copies on several threads --------------------------------------------------------------------
// One thread copies 10 to 15 GB/s between pageable memory and a pinned chunk, a PCIe 5 x16 link moves 50 to 60:
// the copies into and out of the staging chunks are cut into slices and shared among a crew of threads.  The crew
// is created with the first large transfer and is never destroyed (its threads are detached and the object is
// leaked on purpose, so nothing of it is torn down under a thread at process exit).
class CopyCrew {
public:
    static CopyCrew& get() {
        static CopyCrew* crew = new CopyCrew();
        return *crew;
    }
    static constexpr uint64_t PARALLEL_FROM = 512 << 10;

    void copy(void* dst, const void* src, uint64_t n) {
        if (n < PARALLEL_FROM || workers_ == 0) { memcpy(dst, src, n); return; }
        std::lock_guard<std::mutex> one_job(job_mu_);
        uint64_t slice = (n / (2 * (uint64_t)(workers_ + 1)) + 4095) & ~(uint64_t)4095;
        if (slice < (64 << 10)) slice = 64 << 10;
        if (slice > (1 << 20)) slice = 1 << 20;
        uint64_t parts = (n + slice - 1) / slice;
        if (parts > 0xFFFF) { slice = ((n / 0xFFFF) + 4096) & ~(uint64_t)4095; parts = (n + slice - 1) / slice; }
        job_ = {(char*)dst, (const char*)src, n, slice};
        done_.store(0, std::memory_order_relaxed);
        const uint64_t gen = (ticket_.load(std::memory_order_relaxed) >> 32) + 1;
        ticket_.store(gen << 32 | parts << 16, std::memory_order_release);
        if (sleepers_.load(std::memory_order_acquire) > 0) {
            { std::lock_guard<std::mutex> l(sleep_mu_); }
            sleep_cv_.notify_all();
        }
        work(gen);
        while (done_.load(std::memory_order_acquire) != parts) __builtin_ia32_pause();
    }

private:
    struct Job { char* dst; const char* src; uint64_t n, slice; };
    Job job_{};
    int workers_ = 0;
    std::mutex job_mu_, sleep_mu_;
    std::condition_variable sleep_cv_;
    std::atomic<uint64_t> ticket_{0};      // generation << 32 | parts << 16 | next part
    std::atomic<uint64_t> done_{0};
    std::atomic<int> sleepers_{0};

    CopyCrew() {
        unsigned hw = std::thread::hardware_concurrency();
        int want = hw >= 16 ? 7 : hw >= 8 ? 3 : hw >= 4 ? 1 : 0;     // the calling thread is the crew's last member
        for (int i = 0; i < want; i++) {
            try { std::thread([this] { run(); }).detach(); workers_++; } catch (...) { break; }
        }
    }

    // Takes parts of generation `gen` until none is left.  A part is taken by a compare-and-swap on the whole ticket, so a
    // thread that still looks at an older generation can never take a part of a newer job with the older job's pointers.
    void work(uint64_t gen) {
        for (;;) {
            uint64_t t = ticket_.load(std::memory_order_acquire);
            if (t >> 32 != gen) return;
            const uint64_t parts = (t >> 16) & 0xFFFF, next = t & 0xFFFF;
            if (next >= parts) return;
            if (!ticket_.compare_exchange_weak(t, t + 1, std::memory_order_acq_rel)) continue;
            const Job j = job_;             // the job of `gen` stays in place until this part is reported done
            const uint64_t lo = next * j.slice, hi = lo + j.slice < j.n ? lo + j.slice : j.n;
            memcpy(j.dst + lo, j.src + lo, hi - lo);
            done_.fetch_add(1, std::memory_order_release);
        }
    }

    void run() {
        uint64_t seen = 0;
        for (;;) {
            uint64_t gen = ticket_.load(std::memory_order_acquire) >> 32;
            if (gen == seen) {
                // a transfer is a train of jobs some tens of microseconds apart: stay awake for about a millisecond after
                // the last one (waking a sleeper costs more than the copy of a piece)
                const uint64_t until = __builtin_ia32_rdtsc() + 3000000;
                while (gen == seen && __builtin_ia32_rdtsc() < until) {
                    __builtin_ia32_pause();
                    gen = ticket_.load(std::memory_order_acquire) >> 32;
                }
                if (gen == seen) {
                    std::unique_lock<std::mutex> l(sleep_mu_);
                    sleepers_.fetch_add(1, std::memory_order_acq_rel);
                    sleep_cv_.wait(l, [&] { return ticket_.load(std::memory_order_acquire) >> 32 != seen; });
                    sleepers_.fetch_sub(1, std::memory_order_acq_rel);
                    continue;
                }
            }
            seen = gen;
            work(gen);
        }
    }
};

// ---- the staging ring ------------------------------------------------------------------------------------
// CHUNKS pinned chunks per device, each with a copy stream of its own ("lane"); a transfer is cut into pieces that go
// through them in turn, so that the copy between pageable memory and one chunk runs while the DMA engine moves
// another.  The host waits for a piece with hipStreamSynchronize on its lane.  Measured on 256 MiB with 4 MiB pieces:
// 53.7 GB/s in both directions this way, 45.7 (up) and 47.2 (down) with all pieces on the device's own stream and an
// event per chunk; the DMA engine alone moves 57.  The lanes start behind the work already queued on the device's
// stream (an event it records, which they wait for on the device), and a transfer returns when its last piece has
// arrived, so the next launch on the device's stream comes after it.
struct Staging {
    static constexpr int CHUNKS = 4;
    static constexpr uint64_t CHUNK_BYTES = 4 << 20;
    void* chunk[CHUNKS] = {};
    hipStream_t lane[CHUNKS] = {};
    hipEvent_t queued = nullptr;
};

static void staging_destroy(Staging* s) {
    for (int k = 0; k < Staging::CHUNKS; k++) {
        if (s->chunk[k]) (void)hipHostFree(s->chunk[k]);
        if (s->lane[k]) (void)hipStreamDestroy(s->lane[k]);
    }
    if (s->queued) (void)hipEventDestroy(s->queued);
    delete s;
}

static int staging_of(Device* dev, Staging** out) {
    if (!dev->staging) {
        auto* s = new Staging();
        hipError_t e = hipEventCreateWithFlags(&s->queued, hipEventDisableTiming);
        for (int i = 0; i < Staging::CHUNKS && e == hipSuccess; i++) {
            e = hipHostMalloc(&s->chunk[i], Staging::CHUNK_BYTES, hipHostMallocDefault);
            if (e == hipSuccess) e = hipStreamCreateWithFlags(&s->lane[i], hipStreamNonBlocking);
        }
        if (e != hipSuccess) {
            staging_destroy(s);
            return set_error((int)e, "pinned staging memory for host transfers: %s", hipGetErrorString(e));
        }
        dev->staging = s;
    }
    *out = dev->staging;
    return NK_OK;
}

// Pieces of a transfer: small transfers are cut finer, so that they too overlap copy and DMA.
static uint64_t piece_bytes(uint64_t bytes) {
    uint64_t piece = (bytes / 8 + 65535) & ~(uint64_t)65535;
    if (piece < (256 << 10)) piece = 256 << 10;
    if (piece > Staging::CHUNK_BYTES) piece = Staging::CHUNK_BYTES;
    return piece;
}

// The first `lanes` lanes wait, on the device, for everything queued on the device's stream so far.
static int lanes_follow_stream(Device* dev, Staging* s, uint64_t lanes) {
    NK_HIP(hipEventRecord(s->queued, dev->stream));
    for (uint64_t k = 0; k < lanes && k < (uint64_t)Staging::CHUNKS; k++) NK_HIP(hipStreamWaitEvent(s->lane[k], s->queued, 0));
    return NK_OK;
}

int memory_release_all(Device* dev) {
    for (auto& kv : dev->live) (void)hipFree((void*)kv.first);
    dev->live.clear();
    dev->capacity.clear();
    dev->live_bytes = 0;
    for (auto& cls : dev->pool)
        for (void* p : cls.second) (void)hipFree(p);
    dev->pool.clear();
    dev->pool_bytes = 0;
    if (dev->staging) {
        staging_destroy(dev->staging);
        dev->staging = nullptr;
    }
    return NK_OK;
}

}  // namespace nk

using namespace nk;

extern "C" {

int nk_device_stats(nk_dev h, uint64_t* live_buffers, uint64_t* live_bytes) {
    NK_DEVICE(dev, h);
    std::lock_guard<std::mutex> lock(dev->mu);
    if (live_buffers) *live_buffers = dev->live.size();
    if (live_bytes) *live_bytes = dev->live_bytes;
    return NK_OK;
}

int nk_alloc(nk_dev h, uint64_t bytes, nk_buf* buf) {
    NK_DEVICE(dev, h);
    NK_REQUIRE(buf != nullptr, "nk_alloc: null output");
    NK_REQUIRE(bytes < ((uint64_t)1 << 48), "nk_alloc: %llu bytes", (unsigned long long)bytes);
    const uint64_t cls = size_class(bytes);
    void* p = nullptr;
    auto rest = dev->pool.find(cls);
    if (rest != dev->pool.end() && !rest->second.empty()) {
        p = rest->second.back();
        rest->second.pop_back();
        dev->pool_bytes -= cls;
        dev->pool_reuses++;
    } else {
        hipError_t e = hipMalloc(&p, cls);
        if (e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation) {
            (void)hipGetLastError();
            if (int r = release_pool(dev)) return r;         // the blocks at rest may be what is in the way
            e = hipMalloc(&p, cls);
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return set_error((int)e, "nk_alloc: hipMalloc of %llu bytes failed: %s", (unsigned long long)cls, hipGetErrorString(e));
        }
        dev->driver_allocs++;
    }
    {
        std::lock_guard<std::mutex> lock(dev->mu);
        dev->live[(uint64_t)p] = bytes;
        dev->capacity[(uint64_t)p] = cls;
        dev->live_bytes += bytes;
    }
    if (dev->poison) {
        launch_fill_bytes(dev, p, cls, ~(uint64_t)0);
        NK_HIP(hipGetLastError());
    }
    *buf = (uint64_t)p;
    return NK_OK;
}

int nk_free(nk_dev h, nk_buf buf) {
    NK_DEVICE(dev, h);
    uint64_t cls = 0;
    {
        std::lock_guard<std::mutex> lock(dev->mu);
        auto it = dev->live.find(buf);
        if (it == dev->live.end())
            return set_error(NK_ERR_HANDLE, "nk_free: 0x%llx is not a live buffer of this device (double free?)",
                             (unsigned long long)buf);
        dev->live_bytes -= it->second;
        dev->live.erase(it);
        auto cap = dev->capacity.find(buf);
        cls = cap->second;
        dev->capacity.erase(cap);
    }
    if (cls > dev->pool_limit) {
        // kernels still in flight on the device stream may use the buffer
        NK_HIP(hipStreamSynchronize(dev->stream));
        NK_HIP(hipFree((void*)buf));
        return NK_OK;
    }
    if (int e = evict_for(dev, cls)) return e;
    dev->pool[cls].push_back((void*)buf);
    dev->pool_bytes += cls;
    return NK_OK;
}

int nk_pool_trim(nk_dev h) {
    NK_DEVICE(dev, h);
    return release_pool(dev);
}

int nk_pool_stats(nk_dev h, uint64_t* resting_blocks, uint64_t* resting_bytes, uint64_t* driver_allocations, uint64_t* reuses) {
    NK_DEVICE(dev, h);
    if (resting_blocks) {
        uint64_t n = 0;
        for (auto& cls : dev->pool) n += cls.second.size();
        *resting_blocks = n;
    }
    if (resting_bytes) *resting_bytes = dev->pool_bytes;
    if (driver_allocations) *driver_allocations = dev->driver_allocs;
    if (reuses) *reuses = dev->pool_reuses;
    return NK_OK;
}

int nk_pool_config(nk_dev h, uint64_t max_resting_bytes, int poison) {
    NK_DEVICE(dev, h);
    dev->pool_limit = max_resting_bytes;
    dev->poison = poison != 0;
    return evict_for(dev, 0);
}

int nk_h2d(nk_dev h, nk_buf dst, uint64_t off, const void* host, uint64_t bytes) {
    NK_DEVICE(dev, h);
    if (bytes == 0) return NK_OK;
    NK_REQUIRE(host != nullptr, "nk_h2d: null host pointer");
    if (int e = check_range(dev, "nk_h2d", dst, off, bytes)) return e;
    Staging* s = nullptr;
    if (int e = staging_of(dev, &s)) return e;
    CopyCrew& crew = CopyCrew::get();
    const uint64_t piece = piece_bytes(bytes);
    const uint64_t pieces = (bytes + piece - 1) / piece;
    if (int e = lanes_follow_stream(dev, s, pieces)) return e;
    char* to = (char*)dst + off;
    const char* from = (const char*)host;
    for (uint64_t k = 0; k < pieces; k++) {
        const int slot = (int)(k % Staging::CHUNKS);
        const uint64_t len = k + 1 < pieces ? piece : bytes - k * piece;
        if (k >= (uint64_t)Staging::CHUNKS) NK_HIP(hipStreamSynchronize(s->lane[slot]));     // the chunk's last piece has left it
        crew.copy(s->chunk[slot], from + k * piece, len);
        NK_HIP(hipMemcpyAsync(to + k * piece, s->chunk[slot], len, hipMemcpyHostToDevice, s->lane[slot]));
    }
    for (uint64_t k = 0; k < pieces && k < (uint64_t)Staging::CHUNKS; k++) NK_HIP(hipStreamSynchronize(s->lane[k]));
    return NK_OK;
}

int nk_d2h(nk_dev h, void* host, nk_buf src, uint64_t off, uint64_t bytes) {
    NK_DEVICE(dev, h);
    if (bytes == 0) return NK_OK;
    NK_REQUIRE(host != nullptr, "nk_d2h: null host pointer");
    if (int e = check_range(dev, "nk_d2h", src, off, bytes)) return e;
    Staging* s = nullptr;
    if (int e = staging_of(dev, &s)) return e;
    CopyCrew& crew = CopyCrew::get();
    const uint64_t piece = piece_bytes(bytes);
    const uint64_t pieces = (bytes + piece - 1) / piece;
    if (int e = lanes_follow_stream(dev, s, pieces)) return e;
    const char* from = (const char*)src + off;
    char* to = (char*)host;
    auto length = [&](uint64_t k) { return k + 1 < pieces ? piece : bytes - k * piece; };
    auto fetch = [&](uint64_t k) {
        const int slot = (int)(k % Staging::CHUNKS);
        return hipMemcpyAsync(s->chunk[slot], from + k * piece, length(k), hipMemcpyDeviceToHost, s->lane[slot]);
    };
    for (uint64_t k = 0; k < pieces && k < (uint64_t)Staging::CHUNKS; k++) NK_HIP(fetch(k));
    for (uint64_t k = 0; k < pieces; k++) {
        const int slot = (int)(k % Staging::CHUNKS);
        NK_HIP(hipStreamSynchronize(s->lane[slot]));
        crew.copy(to + k * piece, s->chunk[slot], length(k));
        if (k + Staging::CHUNKS < pieces) NK_HIP(fetch(k + Staging::CHUNKS));
    }
    return NK_OK;
}

}  // extern "C"
