// SPDX-License-Identifier: Apache-2.0
//
// TEST INFRASTRUCTURE.  In-memory stand-in for the GPU runtime seam
// (fstx_dev, fastsafetensors_amd/csrc/fstx_internal.h) so that the copy
// pipeline's host code -- threads, ring slots, request bookkeeping, error
// paths -- runs under sanitizers on a machine without a GPU.  "Device memory"
// is ordinary host memory.  Streams are real threads that execute their work
// in order and late (each copy sleeps a little first), so a ring slot that is
// refilled before its copy has run shows up as wrong bytes.
// Never linked into libfstx.so.

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <mutex>
#include <thread>

#include "fstx.h"
#include "fstx_internal.h"

namespace {

struct SimEvent {
    std::mutex m;
    std::condition_variable cv;
    uint64_t recorded = 0, completed = 0;
};

struct SimStream {
    std::mutex m;
    std::condition_variable cv;
    std::deque<std::function<void()>> q;
    bool stop = false;
    uint64_t submitted = 0, finished = 0;
    std::thread th;
    SimStream() : th([this] { run(); }) {}
    void run() {
        for (;;) {
            std::function<void()> f;
            {
                std::unique_lock<std::mutex> lk(m);
                cv.wait(lk, [&] { return stop || !q.empty(); });
                if (q.empty()) return;
                f = std::move(q.front());
                q.pop_front();
            }
            f();
            {
                std::lock_guard<std::mutex> lk(m);
                ++finished;
            }
            cv.notify_all();
        }
    }
    void push(std::function<void()> f) {
        {
            std::lock_guard<std::mutex> lk(m);
            q.push_back(std::move(f));
            ++submitted;
        }
        cv.notify_all();
    }
    void sync() {
        std::unique_lock<std::mutex> lk(m);
        uint64_t target = submitted;
        cv.wait(lk, [&] { return finished >= target; });
    }
    ~SimStream() {
        {
            std::lock_guard<std::mutex> lk(m);
            stop = true;
        }
        cv.notify_all();
        th.join();
    }
};

// Storage model behind the O_DIRECT reads of the pipeline (fstx_test_after_direct_read): up to
// `parallel` requests are served at once, each at bandwidth / parallel, after a fixed latency.
struct StorageModel {
    std::mutex m;
    std::condition_variable cv;
    int lat_us = 0, parallel = 0, busy = 0;
    double bytes_per_us = 0; // of one channel
};
StorageModel g_storage;

std::atomic<int> g_copy_delay_us{50};
std::atomic<int64_t> g_fail_copy_after{-1};
std::atomic<int64_t> g_pinned_live{0};
std::atomic<int> g_host_alloc_delay_us{0};
std::atomic<int> g_host_alloc_failures{0};

} // namespace

extern "C" {
// knobs for the tests
void fstx_sim_set_copy_delay_us(int us) { g_copy_delay_us.store(us); }
// parallel = 0 switches the model off
void fstx_sim_set_storage(int lat_us, double bandwidth_MBps, int parallel) {
    std::lock_guard<std::mutex> lk(g_storage.m);
    g_storage.lat_us = lat_us;
    g_storage.parallel = parallel;
    g_storage.bytes_per_us = parallel > 0 ? bandwidth_MBps / parallel : 0; // MB/s = bytes/us
}
// the pipeline calls this after every O_DIRECT pread (a weak symbol there, defined only here)
void fstx_test_after_direct_read(uint64_t bytes) {
    std::unique_lock<std::mutex> lk(g_storage.m);
    if (g_storage.parallel <= 0) return;
    g_storage.cv.wait(lk, [] { return g_storage.busy < g_storage.parallel; });
    ++g_storage.busy;
    const double us = g_storage.lat_us + (g_storage.bytes_per_us > 0 ? bytes / g_storage.bytes_per_us : 0);
    lk.unlock();
    std::this_thread::sleep_for(std::chrono::microseconds((long long)us));
    lk.lock();
    --g_storage.busy;
    lk.unlock();
    g_storage.cv.notify_one();
}
void fstx_sim_fail_copy_after(int64_t n) { g_fail_copy_after.store(n); }
// the pinned allocation takes this long (a slow context build), and the next `n` of them fail
void fstx_sim_set_host_alloc_delay_us(int us) { g_host_alloc_delay_us.store(us); }
void fstx_sim_fail_host_allocs(int n) { g_host_alloc_failures.store(n); }
int64_t fstx_sim_pinned_live(void) { return g_pinned_live.load(); }
// a caller-side stream: created here, handed to fstx_ctx_order_after as its `stream`
void *fstx_sim_stream_create(void) { return new SimStream; }
void fstx_sim_stream_destroy(void *s) { delete static_cast<SimStream *>(s); }
// queue a task that sleeps and then writes `value` to *flag
void fstx_sim_stream_sleep_then_set(void *s, int us, volatile int *flag, int value) {
    static_cast<SimStream *>(s)->push([=] {
        std::this_thread::sleep_for(std::chrono::microseconds(us));
        *flag = value;
    });
}
}

namespace fstx_dev {

int device_count() { return std::getenv("FSTX_SIM_NO_DEVICE") ? -FSTX_E_NO_DEVICE : 1; }
int set_device(int device_id) { return device_id == 0 ? 0 : -FSTX_E_HIP; }
int pci_bus_id(int, char *out, int len) {
    if (len > 0) out[0] = 0;
    return 0;
}
int host_alloc(void **out, size_t bytes) {
    if (int us = g_host_alloc_delay_us.load()) std::this_thread::sleep_for(std::chrono::microseconds(us));
    if (g_host_alloc_failures.load() > 0 && g_host_alloc_failures.fetch_sub(1) > 0) return -FSTX_E_HIP;
    if (posix_memalign(out, 4096, bytes ? bytes : 1) != 0) return -FSTX_E_HIP;
    g_pinned_live.fetch_add(1);
    return 0;
}
int host_free(void *p) {
    std::free(p);
    g_pinned_live.fetch_sub(1);
    return 0;
}
int stream_create(stream_t *out) {
    *out = new SimStream;
    return 0;
}
int stream_destroy(stream_t s) {
    delete static_cast<SimStream *>(s);
    return 0;
}
int stream_sync(stream_t s) {
    static_cast<SimStream *>(s)->sync();
    return 0;
}
int event_create(event_t *out) {
    *out = new SimEvent;
    return 0;
}
int event_destroy(event_t e) {
    delete static_cast<SimEvent *>(e);
    return 0;
}
int event_record(event_t e, stream_t s) {
    SimEvent *ev = static_cast<SimEvent *>(e);
    uint64_t gen;
    {
        std::lock_guard<std::mutex> lk(ev->m);
        gen = ++ev->recorded;
    }
    static_cast<SimStream *>(s)->push([ev, gen] {
        {
            std::lock_guard<std::mutex> lk(ev->m);
            if (ev->completed < gen) ev->completed = gen;
        }
        ev->cv.notify_all();
    });
    return 0;
}
int event_ready(event_t e) {
    SimEvent *ev = static_cast<SimEvent *>(e);
    std::lock_guard<std::mutex> lk(ev->m);
    return ev->completed >= ev->recorded ? 1 : 0;
}
int event_sync(event_t e) {
    SimEvent *ev = static_cast<SimEvent *>(e);
    std::unique_lock<std::mutex> lk(ev->m);
    uint64_t target = ev->recorded;
    ev->cv.wait(lk, [&] { return ev->completed >= target; });
    return 0;
}
int stream_idle(stream_t s) {
    SimStream *st = static_cast<SimStream *>(s);
    std::lock_guard<std::mutex> lk(st->m);
    return st->finished >= st->submitted ? 1 : 0;
}
int stream_wait_event(stream_t s, event_t e) {
    // the waiting stream stalls until the record that is the event's latest right now has run
    SimEvent *ev = static_cast<SimEvent *>(e);
    uint64_t gen;
    {
        std::lock_guard<std::mutex> lk(ev->m);
        gen = ev->recorded;
    }
    static_cast<SimStream *>(s)->push([ev, gen] {
        std::unique_lock<std::mutex> lk(ev->m);
        ev->cv.wait(lk, [&] { return ev->completed >= gen; });
    });
    return 0;
}
int copy_to_device_async(void *dev_dst, const void *host_src, size_t bytes, stream_t s) {
    int64_t left = g_fail_copy_after.load();
    if (left >= 0 && g_fail_copy_after.fetch_sub(1) == 0) return -FSTX_E_HIP;
    static_cast<SimStream *>(s)->push([=] {
        int us = g_copy_delay_us.load();
        if (us > 0) std::this_thread::sleep_for(std::chrono::microseconds(us));
        std::memcpy(dev_dst, host_src, bytes);
    });
    return 0;
}

} // namespace fstx_dev

namespace fstx_internal {
int check_launch(const char *) { return 0; }
int gather_mode() { return 1; }
} // namespace fstx_internal
