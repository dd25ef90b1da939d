/*
 * Staged copies between pageable host memory and the device: see host_copy.h.
 */
#include "host_copy.h"
#include "hip_common.h"

#include <algorithm>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

namespace {

constexpr size_t CHUNK = 16u << 20;         /* one DMA: 0.29 ms at 57 GB/s */
constexpr int RING = 4;                     /* pinned chunks in flight */
constexpr size_t DIRECT_BELOW = 1u << 20;   /* smaller copies go straight to the runtime */
constexpr size_t MIN_PER_THREAD = 256u << 10;

/* A fixed set of parked threads that split one memcpy. The object is created on
 * first use and never destroyed: the threads are detached and sleep on its
 * condition variable until the process ends, so no destructor can meet a
 * running thread at exit. */
class CopyGang {
public:
    explicit CopyGang(int helpers) : helpers_(helpers) {
        for (int i = 0; i < helpers_; i++) std::thread([this, i] { work(i); }).detach();
    }
    int helpers() const { return helpers_; }

    /* memcpy(dst, src, n) split over the caller and up to `helpers` threads */
    void copy(char* dst, const char* src, size_t n) {
        int parts = (int)std::min<size_t>((size_t)helpers_ + 1, std::max<size_t>(1, n / MIN_PER_THREAD));
        if (parts <= 1) { memcpy(dst, src, n); return; }
        const size_t per = ((n / (size_t)parts) + 4095) & ~(size_t)4095;
        {
            std::lock_guard<std::mutex> l(m_);
            dst_ = dst; src_ = src; n_ = n; per_ = per;
            active_ = parts - 1; pending_ = parts - 1;
            gen_++;
        }
        wake_.notify_all();
        /* the caller takes the last slice */
        const size_t off = per * (size_t)(parts - 1);
        if (off < n) memcpy(dst + off, src + off, n - off);
        std::unique_lock<std::mutex> l(m_);
        done_.wait(l, [this] { return pending_ == 0; });
    }

private:
    void work(int idx) {
        unsigned long seen = 0;
        for (;;) {
            char* d; const char* s; size_t n, per; bool mine;
            {
                std::unique_lock<std::mutex> l(m_);
                wake_.wait(l, [&] { return gen_ != seen; });
                seen = gen_;
                mine = idx < active_;
                d = dst_; s = src_; n = n_; per = per_;
            }
            if (!mine) continue;
            const size_t off = per * (size_t)idx;
            if (off < n) memcpy(d + off, s + off, std::min(per, n - off));
            {
                std::lock_guard<std::mutex> l(m_);
                pending_--;
            }
            done_.notify_one();
        }
    }

    const int helpers_;
    std::mutex m_;
    std::condition_variable wake_, done_;
    unsigned long gen_ = 0;
    char* dst_ = nullptr; const char* src_ = nullptr;
    size_t n_ = 0, per_ = 0;
    int active_ = 0, pending_ = 0;
};

CopyGang* g_gang = nullptr;
int g_threads = -1;          /* total copying threads (caller included); 0 = staging off */

char* g_pin[RING] = {};
hipEvent_t g_ev[RING] = {};
bool g_busy[RING] = {};
bool g_ring_ok = false;

int copy_threads(void) {
    if (g_threads >= 0) return g_threads;
    int t = 8;                                   /* memcpy rate peaks near eight threads */
    const unsigned hw = std::thread::hardware_concurrency();
    if (hw) t = (int)std::min<unsigned>(8u, std::max(1u, hw / 2));
    if (const char* e = getenv("ESHKOL_GPU_COPY_THREADS")) {
        char* end = nullptr;
        const long v = strtol(e, &end, 10);
        if (end != e && v >= 0) {
            t = (int)std::min<long>(v, 32);
            if (v > 32) fprintf(stderr, "[GPU] ESHKOL_GPU_COPY_THREADS=%ld clamped to 32\n", v);
        }
    }
    g_threads = t;
    return t;
}

bool ensure_ring(void) {
    if (g_ring_ok) return true;
    if (copy_threads() == 0) return false;
    for (int i = 0; i < RING; i++) {
        if (!g_pin[i] && !ESHKOL_HIP_OK(hipHostMalloc((void**)&g_pin[i], CHUNK, hipHostMallocDefault))) {
            (void)hipGetLastError();
            g_pin[i] = nullptr;
            return false;
        }
        if (!g_ev[i] && !ESHKOL_HIP_OK(hipEventCreateWithFlags(&g_ev[i], hipEventDisableTiming))) {
            (void)hipGetLastError();
            g_ev[i] = nullptr;
            return false;
        }
    }
    if (!g_gang) g_gang = new CopyGang(copy_threads() - 1);
    g_ring_ok = true;
    return true;
}

/* waits until the DMA that last used the slot has finished */
bool slot_free(int s) {
    if (!g_busy[s]) return true;
    if (!ESHKOL_HIP_OK(hipEventSynchronize(g_ev[s]))) return false;
    g_busy[s] = false;
    return true;
}

}  // namespace

int eshkol_hip_upload(void* dev, const void* host, size_t bytes, hipStream_t st) {
    if (bytes == 0) return 0;
    if (!dev || !host) return -1;
    if (bytes < DIRECT_BELOW || !ensure_ring()) {
        /* pageable source: the runtime stages it; wait so that the source is free on return */
        return (ESHKOL_HIP_OK(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, st)) &&
                ESHKOL_HIP_OK(hipStreamSynchronize(st))) ? 0 : -1;
    }
    const char* src = (const char*)host;
    char* dst = (char*)dev;
    int s = 0;
    for (size_t off = 0; off < bytes; off += CHUNK, s = (s + 1) % RING) {
        const size_t n = std::min(CHUNK, bytes - off);
        if (!slot_free(s)) return -1;
        g_gang->copy(g_pin[s], src + off, n);
        if (!ESHKOL_HIP_OK(hipMemcpyAsync(dst + off, g_pin[s], n, hipMemcpyHostToDevice, st)) ||
            !ESHKOL_HIP_OK(hipEventRecord(g_ev[s], st))) return -1;
        g_busy[s] = true;
    }
    return 0;
}

int eshkol_hip_download(void* host, const void* dev, size_t bytes, hipStream_t st) {
    if (bytes == 0) return 0;
    if (!dev || !host) return -1;
    if (bytes < DIRECT_BELOW || !ensure_ring()) {
        return (ESHKOL_HIP_OK(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, st)) &&
                ESHKOL_HIP_OK(hipStreamSynchronize(st))) ? 0 : -1;
    }
    char* dst = (char*)host;
    const char* src = (const char*)dev;
    const size_t chunks = (bytes + CHUNK - 1) / CHUNK;
    auto request = [&](size_t c) -> bool {
        const int s = (int)(c % RING);
        const size_t off = c * CHUNK, n = std::min(CHUNK, bytes - off);
        if (!slot_free(s)) return false;
        if (!ESHKOL_HIP_OK(hipMemcpyAsync(g_pin[s], src + off, n, hipMemcpyDeviceToHost, st)) ||
            !ESHKOL_HIP_OK(hipEventRecord(g_ev[s], st))) return false;
        g_busy[s] = true;
        return true;
    };
    for (size_t c = 0; c < chunks && c < (size_t)RING; c++) if (!request(c)) return -1;
    for (size_t c = 0; c < chunks; c++) {
        const int s = (int)(c % RING);
        const size_t off = c * CHUNK, n = std::min(CHUNK, bytes - off);
        if (!slot_free(s)) return -1;                 /* chunk c has arrived in its slot */
        g_gang->copy(dst + off, g_pin[s], n);
        if (c + RING < chunks && !request(c + RING)) return -1;
    }
    return 0;
}

void eshkol_hip_copy_release(void) {
    for (int i = 0; i < RING; i++) {
        if (g_busy[i] && g_ev[i]) (void)hipEventSynchronize(g_ev[i]);
        g_busy[i] = false;
        if (g_pin[i]) { (void)hipHostFree(g_pin[i]); g_pin[i] = nullptr; }
        if (g_ev[i]) { (void)hipEventDestroy(g_ev[i]); g_ev[i] = nullptr; }
    }
    g_ring_ok = false;
    g_threads = -1;          /* the environment is read again after a re-init */
}
