// SPDX-License-Identifier: Apache-2.0
//
// File -> pinned ring -> HBM copy pipeline.
//
// What it replaces: nogds_file_reader of the reference (cpp/ext.cpp:648-806,
// cpp/ext.hpp:155-185), which starts one thread per request and, inside it,
// alternates a page-cache pread with a synchronous host-to-device memcpy.
//
// Shape of this one:
//   * a fixed pool of worker threads, pinned to the GPU's NUMA node;
//   * every request is cut into blocks of `block_bytes` on 4 KiB file
//     boundaries; workers pull blocks from one FIFO, so a single large file
//     is read by all workers at once;
//   * each worker cycles through its own slots of a pinned ring that is
//     allocated once per context (by a short-lived thread bound to the node, so
//     the creating thread's affinity and memory policy are never touched);
//     after the read it enqueues an asynchronous
//     host-to-device copy and an event on one of the shared copy streams and
//     moves on to its next slot, so the copy of block k overlaps the read of
//     block k+1 (the event is waited only when the slot comes round again);
//   * a block is read either from the page cache straight into the ring, or
//     with O_DIRECT -- one large pread covering a run of consecutive blocks,
//     issued in ascending file order -- into an ordinary aligned staging block
//     and then moved into the ring block by block.  O_DIRECT cannot target the ring itself: device-visible
//     pinned memory is not backed by pages the block layer can pin, and
//     the read fails with EFAULT.  In AUTO mode the choice is made per block
//     from mincore() residency.
//
// Nothing here touches the GPU runtime directly; see fstx_internal.h.

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include <dlfcn.h>
#include <errno.h>
#include <fcntl.h>
#include <sched.h>
#include <limits.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <sys/sysmacros.h>
#include <sys/syscall.h>
#include <unistd.h>

#include "fstx.h"
#include "fstx_internal.h"

namespace {

constexpr uint64_t kPage = 4096;
constexpr uint64_t kDefaultBlock = 4ull << 20;
constexpr uint64_t kSmallRequestBlock = 1ull << 20;  // block size for requests under kSmallRequest
constexpr uint64_t kSmallRequest = 2ull << 30;
constexpr double kResidentEnough = 0.95;

inline uint64_t align_down(uint64_t v, uint64_t a) { return v - v % a; }
inline uint64_t align_up(uint64_t v, uint64_t a) { return align_down(v + a - 1, a); }
inline uint64_t now_ns() {
    return (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(
               std::chrono::steady_clock::now().time_since_epoch())
        .count();
}

std::atomic<int> g_debug{0};
std::atomic<int64_t> g_bounce_bytes{0};
std::atomic<uint32_t> g_depth_hint{2}; // O_DIRECT depth the last adaptive context settled on

// ---- NUMA and storage facts from sysfs --------------------------------------------

// "/sys" unless FSTX_SYSFS_ROOT names another tree (tests lay one out with the nodes and
// block devices they want the library to see)
std::string sysfs_root() {
    const char *e = std::getenv("FSTX_SYSFS_ROOT");
    return e && *e ? std::string(e) : std::string("/sys");
}

// first line of a sysfs attribute, without the newline; false when unreadable
bool read_sysfs_line(const std::string &path, std::string &out) {
    FILE *f = std::fopen(path.c_str(), "r");
    if (!f) return false;
    char buf[4096];
    const bool ok = std::fgets(buf, sizeof buf, f) != nullptr;
    std::fclose(f);
    if (!ok) return false;
    out.assign(buf);
    while (!out.empty() && (out.back() == '\n' || out.back() == ' ')) out.pop_back();
    return true;
}

// "0-3,8,10-11" -> 0 1 2 3 8 10 11 (the kernel's cpulist format); stops at the first thing it
// cannot read and returns what it had
std::vector<int> parse_cpulist(const char *text) {
    std::vector<int> cpus;
    const char *p = text;
    while (*p && *p != '\n') {
        char *end;
        long a = std::strtol(p, &end, 10);
        if (end == p || a < 0) break;
        long b = a;
        p = end;
        if (*p == '-') {
            b = std::strtol(p + 1, &end, 10);
            if (end == p + 1) break;
            p = end;
        }
        for (long c = a; c <= b && c < CPU_SETSIZE; ++c) cpus.push_back((int)c);
        if (*p == ',') ++p;
        else break;
    }
    return cpus;
}

// CPUs of a node; empty when the node is unknown
std::vector<int> node_cpus(int node) {
    std::string line;
    if (node < 0 || !read_sysfs_line(sysfs_root() + "/devices/system/node/node" + std::to_string(node) + "/cpulist", line))
        return {};
    return parse_cpulist(line.c_str());
}

constexpr int kMaxNode = 1024;

// Restrict the calling thread to the node's CPUs and prefer the node's memory
// (MPOL_PREFERRED: allocate there while it has room).  0, or the first failure as -errno;
// -ENODEV for a node without CPUs.
int bind_thread_to_node(int node) {
    if (node < 0) return 0;
    std::vector<int> cpus = node_cpus(node);
    if (cpus.empty()) return -ENODEV;
    cpu_set_t set;
    CPU_ZERO(&set);
    for (int c : cpus) CPU_SET(c, &set);
    if (sched_setaffinity(0, sizeof set, &set) != 0) return -errno;
    if (node >= kMaxNode) return -EINVAL;
#ifdef SYS_set_mempolicy
    unsigned long mask[kMaxNode / (8 * sizeof(unsigned long))] = {0};
    mask[node / (8 * sizeof(unsigned long))] = 1ul << (node % (8 * sizeof(unsigned long)));
    if (syscall(SYS_set_mempolicy, 1 /* MPOL_PREFERRED */, mask, (unsigned long)kMaxNode + 1) != 0) return -errno;
#endif
    return 0;
}

// whether the calling thread may run on CPUs of `node` only (and on at least one of them)
bool thread_sits_on_node(int node) {
    std::vector<int> cpus = node_cpus(node);
    cpu_set_t have;
    CPU_ZERO(&have);
    if (cpus.empty() || sched_getaffinity(0, sizeof have, &have) != 0 || CPU_COUNT(&have) == 0) return false;
    cpu_set_t of_node;
    CPU_ZERO(&of_node);
    for (int c : cpus) CPU_SET(c, &of_node);
    for (int c = 0; c < CPU_SETSIZE; ++c)
        if (CPU_ISSET(c, &have) && !CPU_ISSET(c, &of_node)) return false;
    return true;
}

// node that holds the page at `addr` (which must have been touched), or -1 when the kernel
// does not say (memory that is mapped from a device driver has no struct page to ask about)
int node_of_address(const void *addr) {
#ifdef SYS_get_mempolicy
    int node = -1;
    if (syscall(SYS_get_mempolicy, &node, nullptr, 0ul, addr, 3ul /* MPOL_F_NODE | MPOL_F_ADDR */) == 0) return node;
#endif
#ifdef SYS_move_pages
    void *pages[1] = {const_cast<void *>(addr)};
    int status[1] = {-1};
    if (syscall(SYS_move_pages, 0, 1ul, pages, nullptr, status, 0) == 0 && status[0] >= 0) return status[0];
#endif
    return -1;
}

// What the block layer says about the device under a file: how many requests its queue
// holds, how large one request may be, whether it seeks, whether it is a paravirtual disk.
struct StorageFacts {
    bool known = false;
    uint64_t nr_requests = 0, max_sectors_kb = 0;
    bool rotational = false, virtio = false;
    std::string name;
};

StorageFacts storage_facts(dev_t dev) {
    StorageFacts out;
    const std::string base = sysfs_root() + "/dev/block/" + std::to_string(major(dev)) + ":" + std::to_string(minor(dev));
    // a partition has no queue of its own: its parent directory is the whole device
    std::string dir = base, line;
    if (!read_sysfs_line(dir + "/queue/nr_requests", line)) {
        dir = base + "/..";
        if (!read_sysfs_line(dir + "/queue/nr_requests", line)) return out;
    }
    out.nr_requests = std::strtoull(line.c_str(), nullptr, 10);
    if (read_sysfs_line(dir + "/queue/max_sectors_kb", line)) out.max_sectors_kb = std::strtoull(line.c_str(), nullptr, 10);
    if (read_sysfs_line(dir + "/queue/rotational", line)) out.rotational = line == "1";
    char resolved[PATH_MAX];
    if (realpath(dir.c_str(), resolved)) {
        out.name = resolved;
        const size_t cut = out.name.rfind('/');
        if (cut != std::string::npos) out.name = out.name.substr(cut + 1);
        // virtio-blk disks are named vdX and hang off a virtioN device
        out.virtio = out.name.rfind("vd", 0) == 0 || std::strstr(resolved, "/virtio") != nullptr;
    }
    out.known = out.nr_requests > 0 && out.max_sectors_kb > 0;
    return out;
}

// MemAvailable of /proc/meminfo (of $FSTX_PROCFS_ROOT/meminfo in tests); 0 when unknown
uint64_t mem_available_bytes() {
    const char *e = std::getenv("FSTX_PROCFS_ROOT");
    const std::string path = std::string(e && *e ? e : "/proc") + "/meminfo";
    FILE *f = std::fopen(path.c_str(), "r");
    if (!f) return 0;
    char line[256];
    uint64_t kb = 0;
    while (std::fgets(line, sizeof line, f))
        if (std::sscanf(line, "MemAvailable: %llu kB", (unsigned long long *)&kb) == 1) break;
    std::fclose(f);
    return kb * 1024;
}

// ---- data model ------------------------------------------------------------

struct FileEntry {
    int fd_buffered = -1;
    int fd_direct = -1; // -1: the filesystem refused O_DIRECT
    int mode = FSTX_READ_AUTO;
    uint64_t size = 0;
    void *map = nullptr; // read-only mapping, used only for mincore()
    std::atomic<bool> direct_ok{true};
    std::atomic<int64_t> open_requests{0};
};

struct Request {
    int64_t id = 0;
    std::shared_ptr<FileEntry> file;
    uint64_t length = 0;
    bool small = false; // under kSmallRequest: short blocks, few slots
    std::atomic<uint64_t> blocks_left{0};
    std::atomic<int64_t> error{0};      // first negative status seen by a worker
    std::atomic<uint64_t> stream_mask{0}; // copy streams that carry blocks of this request
};

struct Block {
    std::shared_ptr<Request> req;
    uint64_t file_off; // first payload byte in the file
    uint64_t len;      // payload bytes
    char *dev;         // device address of the first payload byte
};

// A staging buffer on loan: goes back to its context's pool when the last block that
// still has bytes in it has been copied to the ring.
struct StageLoan {
    fstx_ctx *ctx;
    char *stage;
    StageLoan(fstx_ctx *c, char *s) : ctx(c), stage(s) {}
    ~StageLoan();
};

// One block whose bytes an O_DIRECT read left in a staging buffer; any worker may
// move it into the ring and on to the device.
struct Staged {
    Block block;
    const char *bytes = nullptr;
    std::shared_ptr<StageLoan> loan;
};

struct Slot {
    char *host = nullptr;
    fstx_dev::event_t ev = nullptr;
    bool pending = false; // an async copy out of this slot may still be running
    bool used = false;    // a read has written to it: its first pages are mapped
};

// Bounds the O_DIRECT preads in flight.  Storage differs a lot in the queue depth
// it wants (a virtio disk peaks at 1 or 2, an NVMe array at 16 or more); a steered gate
// finds it while reading.  Completed reads are counted in windows; a window yields a rate.
// From a measured base the gate tries one read more: a gain of 8 % keeps the step and tries
// the next one, anything less takes it back.  Then it tries one read fewer, and keeps that
// when the rate holds (within 3 %): of two depths that read equally fast the smaller one
// needs fewer staging buffers and keeps the requests in order.  After a step in each
// direction has failed the depth rests for a few windows before the next round.
class Gate {
  public:
    Gate(uint32_t start, uint32_t hi, bool adaptive) { configure(start, hi, adaptive); }
    // (re)set depth, ceiling and steering; reads in flight keep their tokens
    void configure(uint32_t start, uint32_t hi, bool adaptive) {
        std::lock_guard<std::mutex> lk(m_);
        hi_ = std::max(1u, hi);
        limit_ = std::max(1u, std::min(start, hi_));
        adaptive_ = adaptive;
        phase_ = kBase;
        win_blocks_ = 0;
    }
    // take a token if one is free; callers that must start their reads in file
    // order call this while they hold the block queue's lock
    bool try_enter() {
        std::lock_guard<std::mutex> lk(m_);
        if (busy_ >= limit_) return false;
        ++busy_;
        return true;
    }
    void leave(uint64_t bytes) {
        std::lock_guard<std::mutex> lk(m_);
        --busy_;
        if (adaptive_) steer(bytes);
    }
    uint32_t limit() {
        std::lock_guard<std::mutex> lk(m_);
        return limit_;
    }
    // the depth that was last found good: a step that is still being tried does not count
    uint32_t settled() {
        std::lock_guard<std::mutex> lk(m_);
        if (phase_ == kTryUp && limit_ > 1) return limit_ - 1;
        if (phase_ == kTryDown && limit_ < hi_) return limit_ + 1;
        return limit_;
    }

  private:
    enum Phase { kBase, kTryUp, kTryDown, kRest };

    void steer(uint64_t bytes) {
        const uint64_t now = now_ns();
        const bool paused = last_done_ != 0 && now - last_done_ > 50'000'000ull;
        last_done_ = now;
        if (paused) { // what was measured before the pause is stale: take a trial step back, start over
            if (phase_ == kTryUp && limit_ > 1) --limit_;
            if (phase_ == kTryDown && limit_ < hi_) ++limit_;
            phase_ = kBase;
            went_up_ = false;
            win_blocks_ = 0;
        }
        if (win_blocks_ == 0) { // this read opens a window: its own bytes came before the clock started
            win_t0_ = now;
            win_bytes_ = 0;
            win_blocks_ = 1;
            return;
        }
        win_bytes_ += bytes;
        // a window: at least 8 reads, four per read in flight, and 20 ms (short windows of small reads measure the scheduler)
        if (++win_blocks_ <= std::max(8u, 4 * limit_) || now - win_t0_ < 20'000'000ull) return;
        const double rate = (double)win_bytes_ / (double)(now - win_t0_);
        win_blocks_ = 0;
        fstx_internal::debug("gate: depth %u phase %d rate %.3f GB/s base %.3f", limit_, (int)phase_, rate, base_rate_);
        auto rest = [&] { phase_ = kRest, rest_ = kRestWindows; };
        switch (phase_) {
        case kBase:
            base_rate_ = rate;
            went_up_ = false;
            if (limit_ < hi_) ++limit_, phase_ = kTryUp;
            else if (limit_ > 1) --limit_, phase_ = kTryDown;
            break;
        case kTryUp:
            if (rate >= 1.08 * base_rate_) { // worth it: keep the step and try the next one
                base_rate_ = rate;
                went_up_ = true;
                if (limit_ < hi_) ++limit_;
                else rest();
            } else {
                --limit_;
                // a round that gained nothing upwards looks downwards next
                if (!went_up_ && limit_ > 1) --limit_, phase_ = kTryDown;
                else rest();
            }
            break;
        case kTryDown:
            if (rate >= 0.97 * base_rate_) { // no worse with one read fewer: keep
                base_rate_ = std::max(base_rate_, rate);
                if (limit_ > 1) --limit_;
                else rest();
            } else {
                ++limit_;
                rest();
            }
            break;
        case kRest:
            if (--rest_ == 0) phase_ = kBase;
            break;
        }
    }

    static constexpr uint32_t kRestWindows = 6;
    std::mutex m_;
    uint32_t limit_ = 1, hi_ = 1, busy_ = 0;
    bool adaptive_ = false;
    Phase phase_ = kBase;
    bool went_up_ = false; // the last round of upward steps kept at least one: no downward try after it
    uint32_t rest_ = 0;
    double base_rate_ = 0;
    uint64_t win_t0_ = 0, win_bytes_ = 0, last_done_ = 0;
    uint32_t win_blocks_ = 0;
};

struct Counters {
    std::atomic<uint64_t> bytes_read{0}, bytes_copied{0}, blocks_buffered{0}, blocks_direct{0},
        read_ns{0}, stage_ns{0}, slot_wait_ns{0}, direct_fallbacks{0}, direct_reads{0}, workers_on_node{0},
        bind_errors{0}, pretouched_bytes{0};
    std::atomic<int64_t> first_bind_error{0};
};

} // namespace

struct fstx_ctx {
    fstx_config cfg{};
    uint64_t ring_bytes = 0;
    uint64_t slot_bytes = 0;
    char *ring = nullptr;
    std::vector<fstx_dev::stream_t> streams;
    std::vector<std::vector<Slot>> slots; // [thread][slot]
    std::vector<std::thread> workers;
    std::unique_ptr<Gate> direct_gate;

    std::mutex q_mutex;
    std::condition_variable q_cv;
    std::deque<Block> queue;
    std::deque<Staged> staged; // read by O_DIRECT, waiting for a worker to ship them (q_mutex)
    uint64_t queue_bytes = 0;              // payload bytes of the blocks in `queue` (q_mutex)
    uint32_t burst_runs = 0;               // O_DIRECT runs started since `queue` was last empty (q_mutex)
    uint64_t ramp_bytes = 0;               // size of the first run of a burst
    uint64_t queue_pops = 0;               // blocks taken off `queue` so far (q_mutex)
    uint64_t head_verdict_for = ~0ull;     // value of queue_pops the cached verdict belongs to
    bool head_wants_direct = false;        // whether the block at the head of `queue` is to be read with O_DIRECT
    bool extending = false;                // a worker asks the page cache how far its run may reach: `queue` is its alone meanwhile
    bool closing = false;
    // Workers that take work (q_mutex).  A small request on an idle context wakes only half of
    // them: every slot that is used for the first time costs its first touch, and eight workers
    // keep the link as busy as sixteen; anything larger, or more work behind it, wakes all.
    uint32_t active_workers = 0;
    std::atomic<bool> work_seen{false};    // something was queued at least once: the workers stop touching their idle slots

    std::mutex done_mutex;
    std::condition_variable done_cv;

    // start-up handshake (ready_mutex): the workers are started first and make their events while
    // the ring is allocated and the streams are created; `parts_ready` releases them, and every
    // worker reports once its slots exist.  `built` closes the build; a failed one leaves its
    // status in `build_status` and in `failed` (q_mutex), the workers count off whatever is queued.
    std::mutex ready_mutex;
    std::condition_variable ready_cv;
    uint32_t ready = 0;
    int ready_status = 0;
    bool ring_ready = false;      // the ring's fate is known (it exists, or parts_status says why not)
    bool parts_ready = false;
    std::unique_ptr<std::atomic<uint8_t>[]> head_mapped; // per ring slot: its owner has mapped the head already
    std::atomic<bool> parts_seen{false}; // parts_ready, for the workers that map their slots meanwhile
    int parts_status = 0;
    bool built = false;
    int build_status = 0;
    std::thread builder;          // FSTX_CREATE_ASYNC: runs build_context() behind fstx_ctx_create's back
    uint64_t create_t0 = 0;
    uint64_t small_block = 0;     // block size for small requests (see fstx_submit_read) on a ring whose pages are yet to be mapped
    uint64_t small_block_mapped = 0; // ... and on a ring that an earlier context has used
    uint64_t burst_bytes = 0;     // bytes submitted since a submit last found nothing queued (q_mutex)
    uint64_t small_burst = 0;     // requests are small while burst_bytes stays under this
    uint32_t small_workers = 0;   // workers such a request wakes on an idle context
    uint32_t small_slots = 1;     // slots of each worker such a request goes through
    int64_t failed = 0;           // build failure, reported by every submit from then on (q_mutex)

    // fstx_ctx_order_after: one event, recorded on the caller's stream, awaited by the copy streams
    std::mutex order_mutex;
    fstx_dev::event_t order_event = nullptr;
    uint64_t create_ns = 0;
    bool no_copy = false, no_read = false; // FSTX_PROBE_*

    std::mutex table_mutex;
    std::map<int64_t, std::shared_ptr<FileEntry>> files;
    std::map<int64_t, std::shared_ptr<Request>> requests;
    std::vector<fstx_dev::event_t> event_pool; // markers of finished waits, for the next ones (table_mutex)
    int64_t next_file = 1;
    int64_t next_request = 1;

    Counters ctr;
    // Shape of the O_DIRECT reads: what the configuration fixes, and for what it leaves at 0 the
    // figures of the block device under the first file that is opened for O_DIRECT (q_mutex)
    bool shape_settled = false;
    StorageFacts storage;
    int ring_node = -1;        // node of the ring's first page, where the kernel says (ready_mutex)
    bool ring_reused = false;  // the ring is the one an earlier context of this process left behind
    bool ring_cache = true;    // take over a parked ring, and leave this one parked (the environment, read when the context is created)
    uint64_t direct_bytes = 0; // bytes one O_DIRECT pread may cover
    // ordinary page-backed blocks that O_DIRECT reads land in; handed out together
    // with the read token (under q_mutex), returned after the last byte left for the ring
    std::vector<char *> stage_free;
    uint32_t stage_made = 0, stage_max = 0;
    bool adaptive_depth = false;
    std::atomic<int64_t> fault_after{-1}; // test hook: fail the n-th block read with EIO
};

namespace {

StageLoan::~StageLoan() {
    {
        std::lock_guard<std::mutex> lk(ctx->q_mutex);
        ctx->stage_free.push_back(stage);
    }
    ctx->q_cv.notify_all();
}

// ---- reading one block -------------------------------------------------------

} // namespace
// Test seam: a host-only test build may define this to put a storage model (latency, bandwidth,
// parallelism) behind every O_DIRECT read; the shipped library leaves it undefined.
extern "C" __attribute__((weak)) void fstx_test_after_direct_read(uint64_t bytes);
namespace {

// pread until `want` bytes arrived, EOF or error; returns bytes or -errno
int64_t pread_full(int fd, char *buf, uint64_t want, uint64_t off) {
    uint64_t got = 0;
    while (got < want) {
        ssize_t c = pread(fd, buf + got, want - got, (off_t)(off + got));
        if (c < 0) {
            if (errno == EINTR) continue;
            return -(int64_t)errno;
        }
        if (c == 0) break;
        got += (uint64_t)c;
    }
    return (int64_t)got;
}

bool block_is_cached(const FileEntry &f, uint64_t lo, uint64_t hi) {
    if (!f.map) return false;
    lo = align_down(lo, kPage);
    hi = std::min(align_up(hi, kPage), align_up(f.size, kPage));
    if (hi <= lo) return true;
    const size_t pages = (size_t)((hi - lo) / kPage);
    unsigned char stack_vec[2048];
    std::vector<unsigned char> heap_vec;
    unsigned char *vec = stack_vec;
    if (pages > sizeof stack_vec) {
        heap_vec.resize(pages);
        vec = heap_vec.data();
    }
    if (mincore(static_cast<char *>(f.map) + lo, hi - lo, vec) != 0) return false;
    size_t in = 0;
    for (size_t i = 0; i < pages; ++i) in += vec[i] & 1;
    return (double)in >= kResidentEnough * (double)pages;
}

// Page-cache residency of one stretch of a file, asked once (mincore) and then queried per block.
struct Residency {
    std::vector<unsigned char> vec;
    uint64_t lo = 0, hi = 0;
    void probe(const FileEntry &f, uint64_t from, uint64_t to) {
        if (!f.map) return;
        lo = align_down(from, kPage);
        hi = std::min(align_up(to, kPage), align_up(f.size, kPage));
        if (hi <= lo) { hi = lo; return; }
        vec.resize((size_t)((hi - lo) / kPage));
        if (mincore(static_cast<char *>(f.map) + lo, hi - lo, vec.data()) != 0) vec.clear(), hi = lo;
    }
    // whether [a, b) lies in the probed stretch and is (nearly) all resident
    bool cached(uint64_t a, uint64_t b) const {
        a = align_down(a, kPage);
        b = std::min(align_up(b, kPage), hi);
        if (vec.empty() || a < lo || b <= a) return false;
        size_t in = 0;
        const size_t first = (size_t)((a - lo) / kPage), n = (size_t)((b - a) / kPage);
        for (size_t i = 0; i < n; ++i) in += vec[first + i] & 1;
        return (double)in >= kResidentEnough * (double)n;
    }
};

struct Worker {
    fstx_ctx *ctx;
    uint32_t index;
    char *stage = nullptr; // staging block borrowed from the context for one O_DIRECT read
    std::vector<Slot> *mine = nullptr;
    size_t turn = 0;
    uint32_t stream_ix = 0;
    fstx_dev::stream_t stream = nullptr;

    bool wants_direct(const Block &b) {
        FileEntry &f = *b.req->file;
        if (f.fd_direct >= 0 && f.direct_ok.load(std::memory_order_relaxed)) {
            if (f.mode == FSTX_READ_DIRECT) return true;
            if (f.mode == FSTX_READ_AUTO) return !block_is_cached(f, b.file_off, b.file_off + b.len);
        } else if (f.mode == FSTX_READ_DIRECT) {
            ctx->ctr.direct_fallbacks.fetch_add(1, std::memory_order_relaxed);
        }
        return false;
    }

    bool fault_hook() {
        int64_t hook = ctx->fault_after.load(std::memory_order_relaxed);
        return hook >= 0 && ctx->fault_after.fetch_sub(1) == 0;
    }

    // next ring slot of this worker, its previous copy finished.  A small request stays within
    // the first few slots: every slot it uses has pages to be mapped first, and a worker whose
    // one copy is in flight is covered by the other workers' reads.
    int64_t take_slot(Slot **out, bool small) {
        const uint32_t n = small ? std::min<uint32_t>(ctx->small_slots, (uint32_t)mine->size()) : (uint32_t)mine->size();
        if (turn >= n) turn = 0;
        Slot &slot = (*mine)[turn];
        turn = (turn + 1) % n;
        slot.used = true;
        int64_t status = 0;
        if (slot.pending) {
            if (fstx_dev::event_ready(slot.ev) != 1) {
                uint64_t t0 = now_ns();
                status = fstx_dev::event_sync(slot.ev);
                ctx->ctr.slot_wait_ns.fetch_add(now_ns() - t0, std::memory_order_relaxed);
            }
            slot.pending = false;
        }
        *out = &slot;
        return status;
    }

    // enqueue slot -> device for block b; payload sits at slot.host + at
    int64_t ship(const Block &b, Slot &slot, uint64_t at) {
        ctx->ctr.bytes_read.fetch_add(b.len, std::memory_order_relaxed);
        if (ctx->no_copy) return 0; // measuring the reads alone
        int64_t status = fstx_dev::copy_to_device_async(b.dev, slot.host + at, b.len, stream);
        if (status < 0) return status;
        slot.pending = true;
        status = fstx_dev::event_record(slot.ev, stream);
        b.req->stream_mask.fetch_or(1ull << stream_ix, std::memory_order_relaxed);
        ctx->ctr.bytes_copied.fetch_add(b.len, std::memory_order_relaxed);
        return status;
    }

    void finish(const Block &b, int64_t status) {
        if (status < 0) {
            int64_t none = 0;
            b.req->error.compare_exchange_strong(none, status);
        }
        if (b.req->blocks_left.fetch_sub(1, std::memory_order_acq_rel) == 1) {
            std::lock_guard<std::mutex> lk(ctx->done_mutex);
            ctx->done_cv.notify_all();
        }
    }

    // page-cache read straight into a ring slot
    int64_t do_buffered(const Block &b) {
        if (fault_hook()) return -EIO;
        Slot *slot = nullptr;
        int64_t status = take_slot(&slot, b.req->small);
        if (status < 0) return status;
        const uint64_t at = b.file_off % kPage;
        uint64_t t0 = now_ns();
        int64_t got = ctx->no_read ? (int64_t)b.len
                                   : pread_full(b.req->file->fd_buffered, slot->host + at, b.len, b.file_off);
        ctx->ctr.read_ns.fetch_add(now_ns() - t0, std::memory_order_relaxed);
        if (got < 0) return got;
        if ((uint64_t)got < b.len) return -FSTX_E_SHORT_READ;
        ctx->ctr.blocks_buffered.fetch_add(1, std::memory_order_relaxed);
        return ship(b, *slot, at);
    }

    // hand the O_DIRECT token back and wake a worker that waits for it
    void release_token(uint64_t bytes) {
        ctx->direct_gate->leave(bytes);
        {
            std::lock_guard<std::mutex> lk(ctx->q_mutex);
        }
        ctx->q_cv.notify_all();
    }

    // One O_DIRECT pread covers a run of consecutive blocks of one request: the storage
    // serves one very large sequential request faster than the same bytes in pieces
    // (measured on a virtio disk: 5.2 GB/s with 64 MiB requests, 7.0 GB/s with 1 GiB).
    // The bytes land in a staging buffer; the blocks are then put on the `staged` queue,
    // where every idle worker helps to move them through the ring, so the copy of a
    // large run is spread over all threads and the next read starts at once.  Returns
    // false when the file turned out not to support O_DIRECT and the run has to be read
    // buffered.  Blocks that failed are reported in `status`; staged ones are marked 1.
    bool do_direct(std::vector<Block> &run, std::vector<int64_t> &status) {
        FileEntry &f = *run.front().req->file;
        const uint64_t window = align_down(run.front().file_off, kPage);
        const uint64_t end = run.back().file_off + run.back().len;
        const uint64_t want = align_up(end, kPage) - window;
        if (!stage) {
            release_token(0);
            status.assign(run.size(), -ENOMEM);
            return true;
        }
        if (fault_hook()) {
            release_token(0);
            return_stage();
            status.assign(run.size(), -EIO);
            return true;
        }
        fstx_internal::Range range("fstx O_DIRECT read: %llu MiB at %llu, %zu blocks", (unsigned long long)(want >> 20),
                                   (unsigned long long)window, run.size());
        uint64_t t0 = now_ns();
        int64_t got = ctx->no_read ? (int64_t)std::min(want, align_up(f.size, kPage) - window)
                                   : pread_full(f.fd_direct, stage, want, window);
        if (fstx_test_after_direct_read && got > 0) fstx_test_after_direct_read((uint64_t)got);
        uint64_t t1 = now_ns();
        ctx->ctr.direct_reads.fetch_add(1, std::memory_order_relaxed);
        release_token(got > 0 ? (uint64_t)got : 0);
        if (got == -EINVAL || got == -EFAULT || got == -EOPNOTSUPP) {
            f.direct_ok.store(false, std::memory_order_relaxed);
            ctx->ctr.direct_fallbacks.fetch_add(run.size(), std::memory_order_relaxed);
            return_stage();
            return false;
        }
        ctx->ctr.read_ns.fetch_add(t1 - t0, std::memory_order_relaxed);
        std::shared_ptr<StageLoan> loan = std::make_shared<StageLoan>(ctx, stage);
        stage = nullptr; // the loan returns it
        std::vector<Staged> ready;
        ready.reserve(run.size());
        for (size_t i = 0; i < run.size(); ++i) {
            const Block &b = run[i];
            if (got < 0) { status[i] = got; continue; }
            if (window + (uint64_t)got < b.file_off + b.len) { status[i] = -FSTX_E_SHORT_READ; continue; }
            status[i] = 1;
            ready.push_back(Staged{b, loan->stage + (b.file_off - window), loan});
        }
        if (!ready.empty()) {
            {
                std::lock_guard<std::mutex> lk(ctx->q_mutex);
                for (Staged &st : ready) ctx->staged.push_back(std::move(st));
            }
            ctx->q_cv.notify_all();
        }
        return true; // `loan` drops here; the staged blocks keep the buffer alive
    }

    // staging buffer -> ring slot -> device, for one block another read left behind
    void ship_staged(Staged &st) {
        const Block &b = st.block;
        int64_t status = b.req->error.load(std::memory_order_relaxed);
        Slot *slot = nullptr;
        if (status == 0 && ctx->no_copy) { // measuring the reads alone: the bytes stay where the read left them
            ctx->ctr.blocks_direct.fetch_add(1, std::memory_order_relaxed);
            ctx->ctr.bytes_read.fetch_add(b.len, std::memory_order_relaxed);
        } else if (status == 0 && (status = take_slot(&slot, b.req->small)) == 0) {
            uint64_t t0 = now_ns();
            std::memcpy(slot->host, st.bytes, b.len);
            ctx->ctr.stage_ns.fetch_add(now_ns() - t0, std::memory_order_relaxed);
            ctx->ctr.blocks_direct.fetch_add(1, std::memory_order_relaxed);
            status = ship(b, *slot, 0);
        }
        st.loan.reset(); // outside q_mutex: the last one hands the buffer back
        finish(b, status < 0 ? status : 0);
    }

    // called with q_mutex held: borrow a staging block, making one if the pool may still grow
    bool borrow_stage() {
        if (!ctx->stage_free.empty()) {
            stage = ctx->stage_free.back();
            ctx->stage_free.pop_back();
            return true;
        }
        if (ctx->stage_made >= ctx->stage_max) return false;
        // address space only: pages become resident as reads touch them, in huge pages where
        // the system allows (a read into fresh 4 KiB pages spends most of its time faulting)
        void *p = nullptr;
        const uint64_t bytes = ctx->direct_bytes + 2 * kPage;
        if (posix_memalign(&p, bytes >= (4u << 20) ? (2u << 20) : kPage, bytes) != 0) p = nullptr;
#ifdef MADV_HUGEPAGE
        if (p && bytes >= (4u << 20)) (void)madvise(p, bytes, MADV_HUGEPAGE);
#endif
        stage = static_cast<char *>(p); // nullptr: the read reports ENOMEM
        if (p) ++ctx->stage_made;
        return true;
    }

    // called with q_mutex held: bytes the next O_DIRECT pread may cover.  The first read after
    // the queue was empty is small, so that copies start early, and the following ones grow
    // fourfold up to the full size; towards the end of what is queued the reads halve again,
    // because the copy of the last read is the one stretch during which the storage idles.
    uint64_t run_limit() const {
        uint64_t limit = ctx->direct_bytes;
        const uint64_t ramp = ctx->ramp_bytes;
        if (ramp < limit) {
            const uint32_t k = std::min(ctx->burst_runs, 16u);
            const uint64_t up = ramp << (2 * k);
            if ((up >> (2 * k)) == ramp && up < limit) limit = up;
            const uint64_t down = std::max(ramp, ctx->queue_bytes / 2);
            if (down < limit) limit = down;
        }
        const uint64_t bb = ctx->cfg.block_bytes;
        return std::max(bb, align_down(limit, bb));
    }

    void return_stage() {
        if (!stage) return;
        {
            std::lock_guard<std::mutex> lk(ctx->q_mutex);
            ctx->stage_free.push_back(stage);
        }
        stage = nullptr;
        ctx->q_cv.notify_all();
    }

    // the events that guard this worker's slots (the ring itself may not exist yet)
    int make_slots() {
        for (uint32_t k = 0; k < ctx->cfg.slots_per_thread; ++k) {
            Slot s;
            int rc = fstx_dev::event_create(&s.ev);
            if (rc < 0) return rc;
            mine->push_back(s);
        }
        return 0;
    }

    // the worker's share of the ring
    void place_slots() {
        for (uint32_t k = 0; k < mine->size(); ++k)
            (*mine)[k].host = ctx->ring + ((uint64_t)index * ctx->cfg.slots_per_thread + k) * ctx->slot_bytes;
    }

    // Map the ring's pages into the process before the first block needs them: pinned memory
    // is mapped page by page at its first touch, and that costs more per byte than copying it
    // to the device (measured: 0.34 ms per MiB on one thread, 0.06 with eight or more, i.e.
    // 18 GB/s at best against a 57 GB/s link).  A few of the workers do it -- more gain nothing,
    // and the creating thread and its caller must still find a free CPU -- by READING one byte
    // per page, which is harmless to a slot that is already in use.  The part of every slot that
    // the blocks of small requests use comes first.  Runs while the creating thread builds the
    // rest of the context and its caller parses file headers, and stops as soon as anything is
    // queued: from then on the reads touch what is left as they go.
    void pretouch(uint32_t helpers) {
        const uint64_t slots = (uint64_t)ctx->cfg.n_threads * ctx->cfg.slots_per_thread;
        const uint64_t head = std::min(ctx->slot_bytes, ctx->small_block + kPage);
        uint64_t done = 0;
        char sink = 0;
        const uint32_t per = ctx->cfg.slots_per_thread, few = std::min(ctx->small_slots, per);
        auto touch = [&](uint64_t s, uint64_t from, uint64_t to) { // false: work has arrived
            const char *base = ctx->ring + s * ctx->slot_bytes;
            for (uint64_t at = from; at < to; at += kPage) {
                if ((at & (16 * kPage - 1)) == 0 && ctx->work_seen.load(std::memory_order_acquire)) return false;
                sink ^= *(const volatile char *)(base + at);
                done += kPage;
            }
            return true;
        };
        bool go_on = true;
        // first the heads of the slots a small request goes through, dealt out evenly ...
        for (uint64_t i = index; go_on && i < (uint64_t)ctx->cfg.n_threads * few; i += helpers) {
            const uint64_t s = i / few * per + i % few;
            if (ctx->head_mapped[s].exchange(1, std::memory_order_relaxed)) continue; // somebody has been there, or is
            go_on = touch(s, 0, head);
        }
        // ... then all the rest
        for (uint64_t s = index; go_on && s < slots; s += helpers) go_on = touch(s, s % per < few ? head : 0, ctx->slot_bytes);
        (void)sink;
        ctx->ctr.pretouched_bytes.fetch_add(done, std::memory_order_relaxed);
    }

    // The same for this worker's own slots, while the context is still being built: the part of
    // each slot that the blocks of a small request use.  Stops once the streams exist and work
    // is queued -- from then on a page is mapped when a read first writes to it.
    void pretouch_own() {
        const uint64_t head = std::min(ctx->slot_bytes, ctx->small_block + kPage);
        uint64_t done = 0;
        char sink = 0;
        for (uint32_t k = 0; k < mine->size() && k < ctx->small_slots; ++k) {
            // whoever gets to a slot's head first maps it (another worker may be going through the whole ring)
            if (ctx->head_mapped[(uint64_t)index * ctx->cfg.slots_per_thread + k].exchange(1, std::memory_order_relaxed)) continue;
            const char *base = (*mine)[k].host;
            for (uint64_t at = 0; at < head; at += kPage) {
                if ((at & (16 * kPage - 1)) == 0 && ctx->parts_seen.load(std::memory_order_acquire) &&
                    ctx->work_seen.load(std::memory_order_acquire))
                    goto out;
                sink ^= *(const volatile char *)(base + at);
                done += kPage;
            }
        }
    out:
        (void)sink;
        ctx->ctr.pretouched_bytes.fetch_add(done, std::memory_order_relaxed);
    }

    void run() {
        const int node = ctx->cfg.numa_node;
        if (node >= 0) {
            const int bound = bind_thread_to_node(node);
            if (bound < 0) {
                ctx->ctr.bind_errors.fetch_add(1, std::memory_order_relaxed);
                int64_t none = 0;
                ctx->ctr.first_bind_error.compare_exchange_strong(none, bound);
            }
            if (thread_sits_on_node(node)) ctx->ctr.workers_on_node.fetch_add(1, std::memory_order_relaxed);
        }
        int64_t dev_rc = fstx_dev::set_device(ctx->cfg.device_id);
        mine = &ctx->slots[index];
        if (dev_rc == 0) dev_rc = make_slots();
        {
            // the ring is allocated by another thread meanwhile
            std::unique_lock<std::mutex> lk(ctx->ready_mutex);
            ctx->ready_cv.wait(lk, [&] { return ctx->ring_ready || ctx->parts_ready; });
            if (dev_rc == 0 && !ctx->ring) dev_rc = ctx->parts_status ? ctx->parts_status : -FSTX_E_HIP;
        }
        if (dev_rc == 0) {
            place_slots();
            // until the streams exist there is nothing else to do: map what a small request will use
            if (!ctx->no_read && !(ctx->cfg.flags & FSTX_NO_PRETOUCH) && index < ctx->small_workers) pretouch_own();
        }
        {
            std::unique_lock<std::mutex> lk(ctx->ready_mutex);
            ctx->ready_cv.wait(lk, [&] { return ctx->parts_ready; });
            if (dev_rc == 0) dev_rc = ctx->parts_status;
            if (dev_rc == 0) {
                stream_ix = index % (uint32_t)ctx->streams.size();
                stream = ctx->streams[stream_ix];
            }
            ++ctx->ready;
            if (dev_rc < 0 && ctx->ready_status == 0) ctx->ready_status = (int)dev_rc;
        }
        ctx->ready_cv.notify_all();
        if (dev_rc == 0 && !ctx->no_read && !(ctx->cfg.flags & FSTX_NO_PRETOUCH)) {
            const uint32_t helpers = std::min(std::min(ctx->cfg.n_threads, 8u), std::max(1u, std::thread::hardware_concurrency() / 2));
            if (index < helpers) pretouch(helpers);
        }
        std::vector<Block> run;
        std::vector<int64_t> status;
        for (;;) {
            run.clear();
            bool direct = false;
            Staged todo;
            bool have_staged = false, woke_others = false;
            {
                // Blocks leave the queue in file order.  A block that needs O_DIRECT is
                // taken together with its token, under this lock, so that the reads reach
                // the storage in ascending order too (storage that detects sequential
                // streams serves them about twice as fast as the same requests shuffled).
                // Blocks that a read has already staged come first: they hold a staging buffer.
                std::unique_lock<std::mutex> lk(ctx->q_mutex);
                auto take_staged = [&] {
                    todo = std::move(ctx->staged.front());
                    ctx->staged.pop_front();
                    have_staged = true;
                };
                for (;;) {
                    // (while another worker extends its run, the queue is that worker's alone)
                    ctx->q_cv.wait(lk, [&] {
                        if (index >= ctx->active_workers && !ctx->closing) return false; // not needed for what is queued
                        return !ctx->staged.empty() || (!ctx->extending && (ctx->closing || !ctx->queue.empty()));
                    });
                    if (ctx->extending || ctx->queue.empty()) {
                        if (!ctx->staged.empty()) take_staged();
                        break; // with nothing taken: closing and drained
                    }
                    // The storage comes first: whenever a token and a staging buffer are free the
                    // next read starts, even while staged blocks wait -- they are what the other
                    // workers do meanwhile.  The verdict on the head block (one mincore call) is
                    // kept until that block leaves the queue.
                    if (ctx->head_verdict_for != ctx->queue_pops) {
                        const Block &head = ctx->queue.front();
                        ctx->head_wants_direct = dev_rc == 0 && head.req->error.load(std::memory_order_relaxed) == 0 &&
                                                 wants_direct(head);
                        ctx->head_verdict_for = ctx->queue_pops;
                        // O_DIRECT reads want everybody: each one in flight holds a worker, and what
                        // they stage is copied out by all the others
                        if (ctx->head_wants_direct && ctx->active_workers < ctx->cfg.n_threads) {
                            ctx->active_workers = ctx->cfg.n_threads;
                            woke_others = true;
                        }
                    }
                    direct = ctx->head_wants_direct;
                    if (!direct) break; // a page-cache block: read it now
                    if ((!ctx->stage_free.empty() || ctx->stage_made < ctx->stage_max) &&
                        ctx->direct_gate->try_enter()) {
                        borrow_stage();
                        break;
                    }
                    direct = false;
                    if (!ctx->staged.empty()) {
                        take_staged();
                        break;
                    }
                    // tokens or staging buffers are all out and nothing is staged: wait for either
                    ctx->q_cv.wait(lk);
                }
                if (!have_staged) {
                    if (ctx->queue.empty()) break;
                    const uint64_t limit = direct ? run_limit() : 0;
                    auto pop = [&] {
                        ctx->queue_bytes -= ctx->queue.front().len;
                        run.push_back(std::move(ctx->queue.front()));
                        ctx->queue.pop_front();
                        ++ctx->queue_pops;
                    };
                    pop();
                    if (direct) {
                        // extend the run with the blocks that follow it in the file; in AUTO mode
                        // only as far as the file is not in the page cache.  That is one mincore
                        // call over the stretch the run may cover (262,144 pages for 1 GiB), made
                        // with the lock released: `extending` keeps the queue for this worker
                        // while the others go on shipping staged blocks.
                        ++ctx->burst_runs;
                        FileEntry &f = *run[0].req->file;
                        Residency seen;
                        if (f.mode == FSTX_READ_AUTO && !ctx->queue.empty()) {
                            const uint64_t from = run[0].file_off + run[0].len, to = run[0].file_off + limit;
                            ctx->extending = true;
                            lk.unlock();
                            seen.probe(f, from, to);
                            lk.lock();
                            ctx->extending = false;
                            woke_others = true;
                        }
                        uint64_t bytes = run[0].len + run[0].file_off % kPage;
                        while (!ctx->queue.empty()) {
                            const Block &nx = ctx->queue.front();
                            const Block &last = run.back();
                            if (nx.req != last.req || nx.file_off != last.file_off + last.len || bytes + nx.len > limit ||
                                seen.cached(nx.file_off, nx.file_off + nx.len))
                                break;
                            bytes += nx.len;
                            pop();
                        }
                    }
                    if (ctx->queue.empty()) ctx->burst_runs = 0; // the next read starts a new burst
                }
            }
            if (woke_others) ctx->q_cv.notify_all(); // the queue is everybody's again
            if (have_staged) {
                ship_staged(todo);
                continue;
            }
            // once a request has failed, its remaining blocks are only counted off
            if (dev_rc < 0 || run[0].req->error.load(std::memory_order_relaxed) != 0) {
                if (direct) {
                    release_token(0);
                    return_stage();
                }
                for (Block &b : run) finish(b, dev_rc);
                continue;
            }
            if (direct) {
                status.assign(run.size(), 0);
                if (do_direct(run, status)) {
                    for (size_t i = 0; i < run.size(); ++i)
                        if (status[i] <= 0) finish(run[i], status[i]); // 1: staged, finished by whoever ships it
                    continue;
                }
            }
            for (Block &b : run) finish(b, do_buffered(b));
        }
        // leave no copy in flight that still reads this worker's slots
        for (Slot &s : *mine)
            if (s.pending) {
                fstx_dev::event_sync(s.ev);
                s.pending = false;
            }
    }
};

void release_file(FileEntry &f) {
    if (f.map) munmap(f.map, f.size);
    if (f.fd_direct >= 0) close(f.fd_direct);
    if (f.fd_buffered >= 0) close(f.fd_buffered);
    f.map = nullptr;
    f.fd_direct = f.fd_buffered = -1;
}

} // namespace

// ---- library-wide helpers ----------------------------------------------------

namespace fstx_internal {
bool debug_enabled() { return g_debug.load(std::memory_order_relaxed) != 0; }
void debug(const char *fmt, ...) {
    if (!debug_enabled()) return;
    va_list ap;
    va_start(ap, fmt);
    std::fputs("[fstx] ", stderr);
    std::vfprintf(stderr, fmt, ap);
    std::fputc('\n', stderr);
    va_end(ap);
}
void note_bounce_bytes(int64_t delta) { g_bounce_bytes.fetch_add(delta); }

namespace {
typedef int (*roctx_push_t)(const char *);
typedef int (*roctx_pop_t)(void);
std::atomic<int> g_roctx_state{0}; // 0 not looked yet, 1 on, -1 off
roctx_push_t g_roctx_push = nullptr;
roctx_pop_t g_roctx_pop = nullptr;
std::once_flag g_roctx_once;

bool roctx_on() {
    const int st = g_roctx_state.load(std::memory_order_acquire);
    if (st) return st > 0;
    std::call_once(g_roctx_once, [] {
        int found = -1;
        const char *want = std::getenv("FSTX_ROCTX");
        if (want && want[0] == '1') {
            const char *named = std::getenv("FSTX_ROCTX_LIB");
            // rocprofv3 records the ranges of its own roctx library; the older one serves the older tools
            const char *names[] = {named && *named ? named : "librocprofiler-sdk-roctx.so", "librocprofiler-sdk-roctx.so.1",
                                   "libroctx64.so", "libroctx64.so.4"};
            for (const char *n : names) {
                void *h = dlopen(n, RTLD_NOW | RTLD_GLOBAL);
                if (!h) continue;
                g_roctx_push = reinterpret_cast<roctx_push_t>(dlsym(h, "roctxRangePushA"));
                g_roctx_pop = reinterpret_cast<roctx_pop_t>(dlsym(h, "roctxRangePop"));
                if (g_roctx_push && g_roctx_pop) {
                    found = 1;
                    break;
                }
            }
            if (found < 0) debug("FSTX_ROCTX=1 but no roctx library could be loaded: no ranges");
        }
        g_roctx_state.store(found, std::memory_order_release);
    });
    return g_roctx_state.load(std::memory_order_acquire) > 0;
}
} // namespace

Range::Range(const char *fmt, ...) {
    if (!roctx_on()) return;
    char text[160];
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(text, sizeof text, fmt, ap);
    va_end(ap);
    g_roctx_push(text);
    open_ = true;
}
Range::~Range() {
    if (open_) g_roctx_pop();
}
} // namespace fstx_internal

extern "C" {

int fstx_abi_version(void) { return FSTX_ABI_VERSION; }
int fstx_device_count(void) { return fstx_dev::device_count(); }
int fstx_get_alignment_size(void) { return (int)kPage; }
void fstx_set_debug_log(int enabled) { g_debug.store(enabled ? 1 : 0); }
uint64_t fstx_bounce_buffer_bytes(void) { return (uint64_t)g_bounce_bytes.load(); }

int fstx_get_device_pci_bus(int device_id, char *out, int len) {
    if (!out || len < 13) return -FSTX_E_INVAL;
    out[0] = 0;
    return fstx_dev::pci_bus_id(device_id, out, len);
}

int fstx_set_numa_node(int numa_node) { return bind_thread_to_node(numa_node); }

int fstx_node_cpus(int numa_node, int *cpus, int capacity) {
    if (numa_node < 0 || capacity < 0 || (capacity && !cpus)) return -FSTX_E_INVAL;
    const std::vector<int> found = node_cpus(numa_node);
    if (found.empty()) return -ENODEV;
    for (size_t i = 0; i < found.size() && i < (size_t)capacity; ++i) cpus[i] = found[i];
    return (int)found.size();
}

void *fstx_host_alloc(uint64_t length) {
    void *p = nullptr;
    if (posix_memalign(&p, kPage, length ? length : 1) != 0) return nullptr;
    return p;
}
void fstx_host_free(void *p) { std::free(p); }

const char *fstx_strerror(int64_t code) {
    if (code >= 0) return "ok";
    int64_t c = -code;
    switch (c) {
    case FSTX_E_INVAL: return "fstx: invalid argument";
    case FSTX_E_HIP: return "fstx: HIP runtime call failed";
    case FSTX_E_RANGE: return "fstx: range exceeds the device buffer";
    case FSTX_E_SHORT_READ: return "fstx: file ended before the requested range";
    case FSTX_E_NO_REQ: return "fstx: unknown request or file handle";
    case FSTX_E_CLOSED: return "fstx: context is shutting down";
    case FSTX_E_NO_DEVICE: return "fstx: no HIP device visible";
    case FSTX_E_TOO_MANY: return "fstx: batch exceeds FSTX_BATCH_MAX";
    default: break;
    }
    if (c < FSTX_E_BASE) return std::strerror((int)c);
    return "fstx: unknown error";
}

// ---- context -----------------------------------------------------------------

namespace {

// defaults filled in, limits checked; 0 or a negative status
int normalize(fstx_config &cfg) {
    if (cfg.n_threads == 0) cfg.n_threads = 8;
    if (cfg.n_streams == 0) cfg.n_streams = 4;
    if (cfg.block_bytes == 0) cfg.block_bytes = kDefaultBlock;
    if (cfg.slots_per_thread == 0) cfg.slots_per_thread = 2;
    // max_direct_reads and direct_read_bytes stay 0 when the caller leaves them open: they are
    // settled from the block device under the first file that is opened for O_DIRECT
    if (cfg.block_bytes % kPage || cfg.n_threads > 1024 || cfg.n_streams > 64 || cfg.slots_per_thread > 64 ||
        (cfg.flags & ~(FSTX_ADAPTIVE_DEPTH | FSTX_PROBE_NO_COPY | FSTX_PROBE_NO_READ | FSTX_NO_PRETOUCH | FSTX_CREATE_ASYNC)))
        return -FSTX_E_INVAL;
    if (cfg.direct_read_bytes)
        cfg.direct_read_bytes = std::max(cfg.block_bytes, align_down(cfg.direct_read_bytes, cfg.block_bytes));
    if (cfg.direct_ramp_kb == 0) cfg.direct_ramp_kb = 64 * 1024;
    cfg.n_streams = std::min(cfg.n_streams, cfg.n_threads);
    cfg.struct_size = sizeof(fstx_config);
    return 0;
}

// The ring of the context that was destroyed last stays allocated for the next context of the
// same device, node and size in this process: a fresh ring costs its allocation (0.2 to 0.5 ms)
// and, far more, the mapping of every page at its first touch (1 ms per 12 MiB with twelve
// threads at it), which is a tenth of the time a 0.5 GB file takes to load.  One ring at most;
// fstx_trim_cache frees it, FSTX_RING_CACHE=0 keeps the library from parking any.
struct ParkedRing {
    void *p = nullptr;
    uint64_t bytes = 0, slot_bytes = 0;
    int device = -1, node = -1, ring_node = -1;
    std::vector<uint8_t> head_mapped; // per slot: its first pages have been touched
};
std::mutex g_park_mutex;
ParkedRing g_parked;

bool ring_cache_on() {
    const char *e = std::getenv("FSTX_RING_CACHE");
    return !(e && e[0] == '0');
}

// the parked ring, if it fits; the caller owns it from here on
bool take_parked(int device, int node, uint64_t bytes, ParkedRing &out) {
    std::lock_guard<std::mutex> lk(g_park_mutex);
    if (!g_parked.p || g_parked.device != device || g_parked.node != node || g_parked.bytes != bytes) return false;
    out = std::move(g_parked);
    g_parked = ParkedRing{};
    return true;
}

// leaves the ring of a context behind for the next one (replacing what is parked), or frees it
void park_or_free_ring(fstx_ctx *ctx) {
    ParkedRing old;
    if (ctx->ring_cache && ctx->build_status == 0 && !ctx->failed) {
        ParkedRing mine;
        mine.p = ctx->ring;
        mine.bytes = ctx->ring_bytes;
        mine.slot_bytes = ctx->slot_bytes;
        mine.device = ctx->cfg.device_id;
        mine.node = ctx->cfg.numa_node;
        mine.ring_node = ctx->ring_node;
        const uint32_t per = ctx->cfg.slots_per_thread;
        mine.head_mapped.resize((size_t)ctx->cfg.n_threads * per);
        for (uint32_t w = 0; w < ctx->cfg.n_threads; ++w)
            for (uint32_t k = 0; k < per; ++k)
                mine.head_mapped[(size_t)w * per + k] =
                    ctx->head_mapped[(size_t)w * per + k].load() || (k < ctx->slots[w].size() && ctx->slots[w][k].used);
        std::lock_guard<std::mutex> lk(g_park_mutex);
        old = std::move(g_parked);
        g_parked = std::move(mine);
    } else {
        old.p = ctx->ring;
    }
    if (old.p) fstx_dev::host_free(old.p);
}

void free_parts(fstx_ctx *ctx) {
    const uint64_t t0 = now_ns();
    for (auto &per : ctx->slots)
        for (Slot &s : per)
            if (s.ev) fstx_dev::event_destroy(s.ev);
    if (ctx->order_event) fstx_dev::event_destroy(ctx->order_event);
    for (auto e : ctx->event_pool) fstx_dev::event_destroy(e);
    const uint64_t t1 = now_ns();
    for (auto s : ctx->streams) fstx_dev::stream_destroy(s);
    const uint64_t t2 = now_ns();
    if (ctx->ring) {
        park_or_free_ring(ctx);
        fstx_internal::note_bounce_bytes(-(int64_t)ctx->ring_bytes); // a parked ring is nobody's bounce buffer
    }
    fstx_internal::debug("free_parts: events %.2f ms, streams %.2f ms, ring %.2f ms", (t1 - t0) / 1e6, (t2 - t1) / 1e6,
                         (now_ns() - t2) / 1e6);
}

void stop_workers(fstx_ctx *ctx) {
    {
        std::lock_guard<std::mutex> lk(ctx->q_mutex);
        ctx->closing = true;
    }
    ctx->q_cv.notify_all();
    for (std::thread &t : ctx->workers) t.join(); // workers drain the queue first
}

// contexts handed out by fstx_ctx_acquire
struct Shared {
    fstx_config cfg;
    fstx_ctx *ctx;
    uint64_t users;
};
std::mutex g_shared_mutex;
std::vector<Shared> g_shared;

bool same_config(const fstx_config &a, const fstx_config &b) {
    return a.device_id == b.device_id && a.numa_node == b.numa_node && a.n_threads == b.n_threads &&
           a.n_streams == b.n_streams && a.block_bytes == b.block_bytes && a.slots_per_thread == b.slots_per_thread &&
           a.max_direct_reads == b.max_direct_reads && a.direct_read_bytes == b.direct_read_bytes &&
           // how the context came to be is not part of what it is
           (a.flags & ~FSTX_CREATE_ASYNC) == (b.flags & ~FSTX_CREATE_ASYNC) &&
           a.direct_ramp_kb == b.direct_ramp_kb;
}

// Depth and size of the O_DIRECT reads (call with q_mutex held, or before the workers exist).
// What the configuration names is kept.  What it leaves at 0 follows the device: one request
// queue's worth of bytes (nr_requests x max_sectors_kb, between 64 MiB and 1 GiB) is the budget.
//   * a paravirtual or rotating disk, or one the block layer tells nothing about, is read with
//     ONE request in flight that carries the whole budget (measured on a virtio disk: two
//     readers, or the same bytes in smaller requests, lose up to half the rate);
//   * anything else (NVMe, SCSI SSDs, md / dm arrays of them) wants several requests in flight:
//     reads of a quarter of the budget, depth 2 to begin with, steered while reading.
// The staging buffers those reads land in are ordinary memory: their number times their size
// stays under 1/16 of MemAvailable (at least 128 MiB).
void settle_direct_shape(fstx_ctx *ctx, const StorageFacts &facts) {
    const fstx_config &cfg = ctx->cfg;
    const bool asked_adaptive = (cfg.flags & FSTX_ADAPTIVE_DEPTH) != 0;
    uint64_t budget = 1ull << 30;
    if (facts.known) budget = std::min<uint64_t>(1ull << 30, std::max<uint64_t>(64ull << 20, facts.nr_requests * facts.max_sectors_kb * 1024));
    const bool serial = !facts.known || facts.virtio || facts.rotational;
    const bool adaptive = asked_adaptive || (cfg.max_direct_reads == 0 && !serial);
    uint32_t depth = cfg.max_direct_reads;
    if (depth == 0) depth = adaptive ? g_depth_hint.load() : 1; // the hint: where the last steered context ended, 2 at first
    const uint32_t hi = std::min(cfg.n_threads, 32u);
    uint64_t bytes = cfg.direct_read_bytes;
    if (bytes == 0) bytes = adaptive ? std::max<uint64_t>(64ull << 20, budget / 4) : budget;
    bytes = std::max(cfg.block_bytes, align_down(bytes, cfg.block_bytes));
    // one staging buffer per read in flight plus one that is being emptied into the ring meanwhile
    uint32_t stages = (adaptive ? std::min(hi, 16u) : std::min(depth, cfg.n_threads)) + 1;
    if (cfg.direct_read_bytes == 0) {
        const uint64_t avail = mem_available_bytes();
        const uint64_t cap = std::max<uint64_t>(128ull << 20, (avail ? avail : (64ull << 30)) / 16);
        const uint32_t fewest = adaptive ? 3 : 2;
        while (stages > fewest && stages * bytes > cap) --stages;
        if (stages * bytes > cap) bytes = std::max(cfg.block_bytes, align_down(cap / stages, cfg.block_bytes));
    }
    ctx->storage = facts;
    ctx->direct_bytes = bytes;
    ctx->ramp_bytes = std::max(cfg.block_bytes, align_down((uint64_t)cfg.direct_ramp_kb * 1024, cfg.block_bytes));
    ctx->stage_max = stages;
    ctx->adaptive_depth = adaptive;
    ctx->direct_gate->configure(depth, hi, adaptive);
    ctx->shape_settled = true;
    fstx_internal::debug("direct reads: device %s (nr_requests %llu, max_sectors_kb %llu%s%s) -> %llu bytes per read, depth %u%s, %u staging buffers",
                         facts.known ? facts.name.c_str() : "unknown", (unsigned long long)facts.nr_requests,
                         (unsigned long long)facts.max_sectors_kb, facts.rotational ? ", rotational" : "",
                         facts.virtio ? ", virtio" : "", (unsigned long long)bytes, depth, adaptive ? " (steered)" : "", stages);
}

} // namespace

namespace {

// Ring, streams, events and workers of a context whose configuration has been checked.
// The workers start first and make their events while a thread of its own allocates the ring
// (bound to the node, so that the ring is placed there and the caller's affinity and memory
// policy stay as they are; one allocation: sixteen small ones take ten times as long) and
// this thread creates the streams: the build takes as long as its slowest part.  Returns 0 or
// the first failure; the workers exist and run either way (after a failure they count off
// every block with that status), so that tearing down is the same in both cases.
int build_context(fstx_ctx *ctx) {
    const fstx_config &cfg = ctx->cfg;
    fstx_internal::Range range("fstx build reader: %u threads, %u streams, ring %llu MiB", cfg.n_threads, cfg.n_streams,
                               (unsigned long long)(ctx->ring_bytes >> 20));
    void *p = nullptr;
    int ring_rc = 0, bound = 0, ring_node = -1;
    bool reused = false;
    uint64_t t_ring = 0;
    auto place_ring = [&](bool own_thread) {
        if (own_thread) bound = bind_thread_to_node(cfg.numa_node); // never the caller's own affinity and policy
        ring_rc = fstx_dev::set_device(cfg.device_id);
        ParkedRing parked;
        if (ring_rc == 0 && ctx->ring_cache && take_parked(cfg.device_id, cfg.numa_node, ctx->ring_bytes, parked)) {
            // the ring an earlier context left behind: allocated, placed, and mapped where it was used
            p = parked.p;
            ring_node = parked.ring_node;
            reused = true;
            // (a ring of the same size cut into other slots says nothing about these)
            if (parked.head_mapped.size() == (size_t)cfg.n_threads * cfg.slots_per_thread && parked.slot_bytes == ctx->slot_bytes)
                for (size_t i = 0; i < parked.head_mapped.size(); ++i)
                    if (parked.head_mapped[i]) ctx->head_mapped[i].store(1, std::memory_order_relaxed);
        }
        if (ring_rc == 0 && !p) ring_rc = fstx_dev::host_alloc(&p, ctx->ring_bytes);
        if (ring_rc == 0 && p && !reused && cfg.numa_node >= 0) {
            *static_cast<volatile char *>(p) = 0; // the page exists from here on, on the node the policy names
            ring_node = node_of_address(p);
        }
        t_ring = now_ns();
        {
            // the workers take their slots and begin to map them while the streams are still being made
            std::lock_guard<std::mutex> lk(ctx->ready_mutex);
            if (p) {
                ctx->ring = static_cast<char *>(p);
                fstx_internal::note_bounce_bytes((int64_t)ctx->ring_bytes);
            } else {
                ctx->parts_status = ring_rc ? ring_rc : -FSTX_E_HIP;
            }
            ctx->ring_node = ring_node;
            ctx->ring_reused = reused;
            ctx->ring_ready = true;
        }
        ctx->ready_cv.notify_all();
    };
    std::thread placer;
    try {
        placer = std::thread(place_ring, true);
    } catch (const std::system_error &) {
        place_ring(false); // no thread to be had: here, unbound
    }
    int spawn_rc = 0;
    try {
        for (uint32_t t = 0; t < cfg.n_threads; ++t) {
            ctx->workers.emplace_back([ctx, t] {
                Worker w{ctx, t};
                w.run();
            });
        }
    } catch (const std::system_error &) {
        spawn_rc = -EAGAIN;
    }
    const uint64_t t_spawned = now_ns();
    int rc = fstx_dev::set_device(cfg.device_id);
    for (uint32_t i = 0; i < cfg.n_streams && rc == 0; ++i) {
        fstx_dev::stream_t s = nullptr;
        if ((rc = fstx_dev::stream_create(&s)) == 0) ctx->streams.push_back(s);
    }
    if (rc == 0) rc = fstx_dev::event_create(&ctx->order_event);
    const uint64_t t_streams = now_ns();
    if (placer.joinable()) placer.join();
    if (rc == 0) rc = ring_rc;
    if (rc == 0) rc = spawn_rc;
    if (bound < 0) {
        ctx->ctr.bind_errors.fetch_add(1);
        int64_t none = 0;
        ctx->ctr.first_bind_error.compare_exchange_strong(none, bound);
    }
    {
        std::unique_lock<std::mutex> lk(ctx->ready_mutex);
        ctx->parts_status = rc;
        ctx->parts_ready = true;
        ctx->parts_seen.store(true, std::memory_order_release);
        ctx->ready_cv.notify_all();
        // a context exists once every worker has its slots
        const uint32_t started = (uint32_t)ctx->workers.size();
        ctx->ready_cv.wait(lk, [&] { return ctx->ready == started; });
        if (rc == 0) rc = ctx->ready_status;
    }
    if (rc < 0) {
        // submits fail from here on; what is queued already is counted off by the workers, and by
        // this thread when not one of them could be started
        std::deque<Block> orphans;
        {
            std::lock_guard<std::mutex> lk(ctx->q_mutex);
            ctx->failed = rc;
            if (ctx->workers.empty()) {
                orphans.swap(ctx->queue);
                ctx->queue_bytes = 0;
            }
        }
        for (Block &b : orphans) {
            int64_t none = 0;
            b.req->error.compare_exchange_strong(none, rc);
            if (b.req->blocks_left.fetch_sub(1, std::memory_order_acq_rel) == 1) {
                std::lock_guard<std::mutex> lk(ctx->done_mutex);
                ctx->done_cv.notify_all();
            }
        }
    }
    ctx->create_ns = now_ns() - ctx->create_t0;
    fstx_internal::debug("ctx_create: device=%d threads=%u streams=%u block=%llu ring=%llu in %.2f ms (workers started %.2f, streams %.2f, ring %.2f)%s; "
                         "node %d: %llu of %u workers on it, ring on node %d, %llu failed bindings (first: %lld); status %d",
                         cfg.device_id, cfg.n_threads, cfg.n_streams, (unsigned long long)cfg.block_bytes,
                         (unsigned long long)ctx->ring_bytes, ctx->create_ns / 1e6, (t_spawned - ctx->create_t0) / 1e6,
                         (t_streams - ctx->create_t0) / 1e6, (t_ring - ctx->create_t0) / 1e6,
                         (cfg.flags & FSTX_CREATE_ASYNC) ? ", behind the caller's back" : "", cfg.numa_node,
                         (unsigned long long)ctx->ctr.workers_on_node.load(), cfg.n_threads, ctx->ring_node,
                         (unsigned long long)ctx->ctr.bind_errors.load(), (long long)ctx->ctr.first_bind_error.load(), rc);
    {
        std::lock_guard<std::mutex> lk(ctx->ready_mutex);
        ctx->build_status = rc;
        ctx->built = true;
    }
    ctx->ready_cv.notify_all();
    return rc;
}

// the build's status, once it is over (at once for a context that was built by its creator)
int wait_built(fstx_ctx *ctx) {
    std::unique_lock<std::mutex> lk(ctx->ready_mutex);
    ctx->ready_cv.wait(lk, [&] { return ctx->built; });
    return ctx->build_status;
}

void teardown(fstx_ctx *ctx) {
    if (ctx->builder.joinable()) ctx->builder.join();
    stop_workers(ctx);
    fstx_dev::set_device(ctx->cfg.device_id);
    for (auto s : ctx->streams) fstx_dev::stream_sync(s);
    for (auto &kv : ctx->files) release_file(*kv.second);
    for (char *p : ctx->stage_free) std::free(p);
    free_parts(ctx);
    delete ctx;
}

} // namespace

uint64_t fstx_cached_ring_bytes(void) {
    std::lock_guard<std::mutex> lk(g_park_mutex);
    return g_parked.p ? g_parked.bytes : 0;
}

uint64_t fstx_trim_cache(void) {
    ParkedRing old;
    {
        std::lock_guard<std::mutex> lk(g_park_mutex);
        old = std::move(g_parked);
        g_parked = ParkedRing{};
    }
    if (!old.p) return 0;
    fstx_dev::host_free(old.p);
    return old.bytes;
}

int fstx_ctx_create(const fstx_config *cfg_in, fstx_ctx **out) {
    if (!cfg_in || !out || cfg_in->struct_size < sizeof(fstx_config)) return -FSTX_E_INVAL;
    *out = nullptr;
    const uint64_t t_start = now_ns();
    fstx_config cfg = *cfg_in;
    int rc = normalize(cfg);
    if (rc < 0) return rc;

    int n_dev = fstx_dev::device_count();
    if (n_dev < 0) return n_dev;
    if (cfg.device_id < 0 || cfg.device_id >= n_dev) return -FSTX_E_INVAL;

    std::unique_ptr<fstx_ctx> ctx(new fstx_ctx);
    ctx->cfg = cfg;
    ctx->create_t0 = t_start;
    ctx->no_copy = (cfg.flags & FSTX_PROBE_NO_COPY) != 0;
    ctx->no_read = (cfg.flags & FSTX_PROBE_NO_READ) != 0;
    ctx->direct_gate.reset(new Gate(1, 1, false));
    // a configuration that names both depth and size needs no device to settle on
    if (cfg.max_direct_reads && cfg.direct_read_bytes) settle_direct_shape(ctx.get(), StorageFacts{});
    if (const char *e = std::getenv("FSTX_FAULT_READ_AFTER")) ctx->fault_after.store(std::atoll(e));
    ctx->small_block = kSmallRequestBlock;
    ctx->small_block_mapped = 2 * kSmallRequestBlock;
    if (const char *e = std::getenv("FSTX_SMALL_BLOCK_KB")) {
        const uint64_t kb = std::strtoull(e, nullptr, 10);
        if (kb >= 64 && kb % 4 == 0) ctx->small_block = ctx->small_block_mapped = kb * 1024;
    }

    // measured on 0.5 and 0.7 GB files in the page cache: twelve workers with one slot each beat
    // eight with two by 4 to 6 % (12 MiB of pinned memory to map before the link runs, not 16)
    ctx->ring_cache = ring_cache_on();
    ctx->small_burst = kSmallRequest;
    if (const char *e = std::getenv("FSTX_SMALL_BURST_MB")) {
        const uint64_t mb = std::strtoull(e, nullptr, 10);
        if (mb >= 1) ctx->small_burst = mb << 20;
    }
    ctx->small_workers = std::min(cfg.n_threads, std::max(4u, cfg.n_threads * 3 / 4));
    if (const char *e = std::getenv("FSTX_SMALL_WORKERS")) {
        const uint64_t n = std::strtoull(e, nullptr, 10);
        if (n >= 1) ctx->small_workers = (uint32_t)std::min<uint64_t>(n, cfg.n_threads);
    }
    if (const char *e = std::getenv("FSTX_SMALL_SLOTS")) {
        const uint64_t n = std::strtoull(e, nullptr, 10);
        if (n >= 1) ctx->small_slots = (uint32_t)std::min<uint64_t>(n, cfg.slots_per_thread);
    }
    // each slot holds one block plus the 4 KiB lead-in of an unaligned start
    ctx->slot_bytes = cfg.block_bytes + kPage;
    ctx->ring_bytes = ctx->slot_bytes * cfg.n_threads * cfg.slots_per_thread;
    ctx->slots.resize(cfg.n_threads);
    ctx->head_mapped.reset(new std::atomic<uint8_t>[(size_t)cfg.n_threads * cfg.slots_per_thread]);
    for (uint64_t i = 0; i < (uint64_t)cfg.n_threads * cfg.slots_per_thread; ++i) ctx->head_mapped[i].store(0);
    fstx_ctx *raw = ctx.release();
    if (cfg.flags & FSTX_CREATE_ASYNC) {
        // the caller goes on (headers to parse, files to open, reads to queue); whatever needs the
        // streams or the outcome of the build waits for it
        try {
            raw->builder = std::thread([raw] { build_context(raw); });
            *out = raw;
            return 0;
        } catch (const std::system_error &) {
            // no thread to be had: build it here
        }
    }
    rc = build_context(raw);
    if (rc < 0) {
        teardown(raw);
        return rc;
    }
    *out = raw;
    return 0;
}

int fstx_ctx_destroy(fstx_ctx *ctx) {
    if (!ctx) return -FSTX_E_INVAL;
    const uint64_t t0 = now_ns();
    if (ctx->builder.joinable()) ctx->builder.join();
    stop_workers(ctx);
    const uint64_t t1 = now_ns();
    if (ctx->adaptive_depth && ctx->ctr.blocks_direct.load() > 64) g_depth_hint.store(ctx->direct_gate->settled());
    fstx_dev::set_device(ctx->cfg.device_id);
    for (auto s : ctx->streams) fstx_dev::stream_sync(s);
    for (auto &kv : ctx->files) release_file(*kv.second);
    for (char *p : ctx->stage_free) std::free(p);
    const uint64_t t2 = now_ns();
    free_parts(ctx);
    delete ctx;
    fstx_internal::debug("ctx_destroy: workers joined in %.2f ms, streams idle and files closed in %.2f ms, ring, events and streams freed in %.2f ms",
                         (t1 - t0) / 1e6, (t2 - t1) / 1e6, (now_ns() - t2) / 1e6);
    return 0;
}

int fstx_ctx_acquire(const fstx_config *cfg_in, fstx_ctx **out) {
    if (!cfg_in || !out || cfg_in->struct_size < sizeof(fstx_config)) return -FSTX_E_INVAL;
    *out = nullptr;
    fstx_config cfg = *cfg_in;
    int rc = normalize(cfg);
    if (rc < 0) return rc;
    std::lock_guard<std::mutex> lk(g_shared_mutex);
    for (Shared &s : g_shared)
        if (same_config(s.cfg, cfg)) {
            ++s.users;
            *out = s.ctx;
            return 0;
        }
    fstx_ctx *ctx = nullptr;
    if ((rc = fstx_ctx_create(&cfg, &ctx)) < 0) return rc;
    g_shared.push_back(Shared{cfg, ctx, 1});
    *out = ctx;
    return 0;
}

int fstx_ctx_release(fstx_ctx *ctx) {
    if (!ctx) return -FSTX_E_INVAL;
    {
        std::lock_guard<std::mutex> lk(g_shared_mutex);
        for (size_t i = 0; i < g_shared.size(); ++i)
            if (g_shared[i].ctx == ctx) {
                if (--g_shared[i].users > 0) return 0;
                g_shared.erase(g_shared.begin() + (long)i);
                break;
            }
    }
    return fstx_ctx_destroy(ctx); // the last user, or a private context
}

int fstx_ctx_order_after(fstx_ctx *ctx, void *stream) {
    if (!ctx) return -FSTX_E_INVAL;
    std::lock_guard<std::mutex> lk(ctx->order_mutex);
    int rc = fstx_dev::set_device(ctx->cfg.device_id);
    if (rc < 0) return rc;
    // Nothing running on the caller's stream: nothing to wait for.  (Worth asking: an event on
    // an idle stream can still complete late, when that stream shares a hardware queue with a
    // busy one.)
    if (fstx_dev::stream_idle(stream) == 1) return 0;
    if ((rc = wait_built(ctx)) < 0) return rc; // the copy streams are needed from here on
    rc = fstx_dev::event_record(ctx->order_event, stream);
    for (size_t i = 0; i < ctx->streams.size() && rc == 0; ++i) rc = fstx_dev::stream_wait_event(ctx->streams[i], ctx->order_event);
    return rc;
}

// ---- files ---------------------------------------------------------------------

int64_t fstx_file_open(fstx_ctx *ctx, const char *path, int mode) {
    if (!ctx || !path || mode < FSTX_READ_AUTO || mode > FSTX_READ_DIRECT) return -FSTX_E_INVAL;
    auto f = std::make_shared<FileEntry>();
    f->mode = mode;
    f->fd_buffered = open(path, O_RDONLY | O_CLOEXEC);
    if (f->fd_buffered < 0) return -(int64_t)errno;
    struct stat st;
    if (fstat(f->fd_buffered, &st) != 0) {
        int64_t e = -(int64_t)errno;
        release_file(*f);
        return e;
    }
    f->size = (uint64_t)st.st_size;
    if (mode != FSTX_READ_BUFFERED) {
        f->fd_direct = open(path, O_RDONLY | O_CLOEXEC | O_DIRECT); // EINVAL on some filesystems
        if (f->fd_direct < 0) fstx_internal::debug("file_open: no O_DIRECT for %s (%s)", path, std::strerror(errno));
    }
    if (mode == FSTX_READ_AUTO && f->fd_direct >= 0 && f->size > 0) {
        void *m = mmap(nullptr, f->size, PROT_READ, MAP_SHARED, f->fd_buffered, 0);
        if (m != MAP_FAILED) f->map = m;
    }
    if (f->fd_direct >= 0) {
        // the first file that can be read with O_DIRECT names the device the reads are shaped for
        bool open_shape;
        {
            std::lock_guard<std::mutex> lk(ctx->q_mutex);
            open_shape = !ctx->shape_settled;
        }
        if (open_shape) {
            const StorageFacts facts = storage_facts(st.st_dev); // sysfs reads: outside the lock
            std::lock_guard<std::mutex> lk(ctx->q_mutex);
            if (!ctx->shape_settled) settle_direct_shape(ctx, facts);
        }
    }
    std::lock_guard<std::mutex> lk(ctx->table_mutex);
    int64_t id = ctx->next_file++;
    ctx->files[id] = f;
    return id;
}

int fstx_file_close(fstx_ctx *ctx, int64_t file) {
    if (!ctx) return -FSTX_E_INVAL;
    std::shared_ptr<FileEntry> f;
    bool idle = false;
    {
        std::lock_guard<std::mutex> lk(ctx->table_mutex);
        auto it = ctx->files.find(file);
        if (it == ctx->files.end()) return -FSTX_E_NO_REQ;
        if (it->second->open_requests.load() != 0) return -EBUSY;
        f = it->second;
        ctx->files.erase(it);
        idle = ctx->files.empty();
    }
    release_file(*f);
    if (idle) {
        // nothing is open any more: the staging buffers of the O_DIRECT reads (up to
        // direct_read_bytes each) that are not on loan go back to the system until the next cold read
        std::vector<char *> spare;
        {
            std::lock_guard<std::mutex> lq(ctx->q_mutex);
            spare.swap(ctx->stage_free);
            ctx->stage_made -= (uint32_t)spare.size();
        }
        for (char *p : spare) std::free(p);
    }
    return 0;
}

// ---- requests ------------------------------------------------------------------

int64_t fstx_submit_read(fstx_ctx *ctx, int64_t file, uint64_t file_off, uint64_t length,
                         void *dev_base, uint64_t dev_capacity, uint64_t dst_off) {
    if (!ctx || (!dev_base && length)) return -FSTX_E_INVAL;
    if (dst_off > dev_capacity || length > dev_capacity - dst_off) return -FSTX_E_RANGE;
    fstx_internal::Range range("fstx submit_read file %lld: %llu bytes at %llu", (long long)file, (unsigned long long)length,
                               (unsigned long long)file_off);
    auto req = std::make_shared<Request>();
    {
        std::lock_guard<std::mutex> lk(ctx->table_mutex);
        auto it = ctx->files.find(file);
        if (it == ctx->files.end()) return -FSTX_E_NO_REQ;
        req->file = it->second;
        req->id = ctx->next_request++;
        ctx->requests[req->id] = req;
        req->file->open_requests.fetch_add(1);
    }
    req->length = length;
    {
        // A request is small while less than 2 GiB have been submitted since a submit last found
        // nothing queued: a single file of that size, or the first files of a checkpoint made of
        // many.  (Eight files of 1.9 GB each, all cut into 1 MiB blocks, load at 53.8 GB/s; with
        // only the first of them treated so, at 56.)
        std::lock_guard<std::mutex> lk(ctx->q_mutex);
        if (ctx->queue.empty() && ctx->staged.empty()) ctx->burst_bytes = 0;
        ctx->burst_bytes += length;
        req->small = ctx->burst_bytes < ctx->small_burst;
    }
    if (file_off > req->file->size || length > req->file->size - file_off)
        req->error.store(-FSTX_E_SHORT_READ); // reported by wait_read, like a failed read

    // Cut on multiples of block_bytes counted from the 4 KiB boundary below the
    // first byte, so that every block's O_DIRECT window fits one slot.
    std::vector<Block> blocks;
    if (length && req->error.load() == 0) {
        // Small requests are cut into blocks of 1 MiB: a slot's pages are mapped at their
        // first touch, at 18 GB/s at best, so a load moves at that rate until the part of the ring
        // it uses has been touched once -- 2.5 ms for 32 slots of 2 MiB, which is a sixth of a
        // 0.7 GB load.  1 MiB blocks still run the link at 54 of its 57 GB/s.  On a ring that an
        // earlier context has left behind there is little or nothing to map: 2 MiB blocks, which
        // run the link at 56 (0.5 and 0.7 GB files: 10.0 and 14.1 ms against 10.5 and 15.1).
        uint64_t bb = ctx->cfg.block_bytes;
        if (req->small) {
            bool mapped;
            {
                std::lock_guard<std::mutex> lk(ctx->ready_mutex);
                mapped = ctx->ring_ready && ctx->ring_reused; // (a ring that is still being allocated is a fresh one)
            }
            // (likewise the ring of a context that has served requests before: a reader that is held)
            mapped = mapped || ctx->ctr.bytes_read.load(std::memory_order_relaxed) > 0;
            bb = std::min(bb, mapped ? ctx->small_block_mapped : ctx->small_block);
        }
        const uint64_t origin = align_down(file_off, kPage);
        const uint64_t end = file_off + length;
        for (uint64_t lo = origin; lo < end; lo += bb) {
            uint64_t a = std::max(lo, file_off), z = std::min(lo + bb, end);
            blocks.push_back(Block{req, a, z - a, static_cast<char *>(dev_base) + dst_off + (a - file_off)});
        }
    }
    req->blocks_left.store(blocks.size());
    if (!blocks.empty()) {
        {
            std::lock_guard<std::mutex> lk(ctx->q_mutex);
            if (ctx->closing || ctx->failed) {
                std::lock_guard<std::mutex> lk2(ctx->table_mutex);
                ctx->requests.erase(req->id);
                req->file->open_requests.fetch_sub(1);
                return ctx->failed ? ctx->failed : -FSTX_E_CLOSED;
            }
            const bool idle = ctx->queue.empty() && ctx->staged.empty();
            const uint32_t all = ctx->cfg.n_threads;
            // (and no more of them than there are blocks: the others would wake to find nothing)
            ctx->active_workers = idle && req->small ? (uint32_t)std::min<uint64_t>(ctx->small_workers, blocks.size()) : all;
            for (Block &b : blocks) {
                ctx->queue_bytes += b.len;
                ctx->queue.push_back(std::move(b));
            }
            ctx->work_seen.store(true, std::memory_order_release);
        }
        ctx->q_cv.notify_all();
    }
    return req->id;
}

int64_t fstx_wait_read(fstx_ctx *ctx, int64_t request) {
    if (!ctx) return -FSTX_E_INVAL;
    fstx_internal::Range range("fstx wait_read request %lld", (long long)request);
    std::shared_ptr<Request> req;
    {
        std::lock_guard<std::mutex> lk(ctx->table_mutex);
        auto it = ctx->requests.find(request);
        if (it == ctx->requests.end()) return -FSTX_E_NO_REQ;
        req = it->second;
        ctx->requests.erase(it);
    }
    {
        std::unique_lock<std::mutex> lk(ctx->done_mutex);
        ctx->done_cv.wait(lk, [&] { return req->blocks_left.load(std::memory_order_acquire) == 0; });
    }
    bool alone; // no other request submitted and not yet waited for
    {
        std::lock_guard<std::mutex> lk(ctx->table_mutex);
        alone = ctx->requests.empty();
    }
    // Every block is enqueued on its stream by now; wait for the copies themselves.  With nothing
    // queued behind them the streams are synchronized (which also lets the runtime retire their
    // finished commands while this thread has to wait anyway; left to pile up until the streams
    // are destroyed, they cost milliseconds there).  A caller that queues the next files before
    // waiting for these keeps the streams busy, and a synchronize of a stream that is being fed
    // returned 8 ms after these copies were done: then a marker is put behind them on each stream
    // and waited for instead.
    int64_t status = req->error.load();
    const uint64_t mask = req->stream_mask.load();
    if (mask == 0) { // nothing went to a stream: an empty request, a failed one, or a context that could not be built
        req->file->open_requests.fetch_sub(1);
        return status < 0 ? status : (int64_t)req->length;
    }
    fstx_dev::set_device(ctx->cfg.device_id);
    if (alone) {
        for (size_t i = 0; i < ctx->streams.size(); ++i)
            if (mask >> i & 1) {
                int rc = fstx_dev::stream_sync(ctx->streams[i]);
                if (rc < 0 && status == 0) status = rc;
            }
        req->file->open_requests.fetch_sub(1);
        return status < 0 ? status : (int64_t)req->length;
    }
    std::vector<fstx_dev::event_t> marks;
    {
        std::lock_guard<std::mutex> lk(ctx->table_mutex);
        for (size_t i = 0; i < ctx->streams.size(); ++i)
            if ((mask >> i & 1) && !ctx->event_pool.empty()) {
                marks.push_back(ctx->event_pool.back());
                ctx->event_pool.pop_back();
            }
    }
    size_t m = 0;
    std::vector<fstx_dev::event_t> used;
    for (size_t i = 0; i < ctx->streams.size(); ++i) {
        if (!(mask >> i & 1)) continue;
        fstx_dev::event_t ev = nullptr;
        if (m < marks.size()) ev = marks[m++];
        int rc = ev ? 0 : fstx_dev::event_create(&ev);
        if (rc == 0) {
            used.push_back(ev);
            rc = fstx_dev::event_record(ev, ctx->streams[i]);
        }
        if (rc < 0) { // no marker to be had: the stream itself
            int rs = fstx_dev::stream_sync(ctx->streams[i]);
            if (rs < 0 && status == 0) status = rs;
        }
    }
    for (fstx_dev::event_t ev : used) {
        int rc = fstx_dev::event_sync(ev);
        if (rc < 0 && status == 0) status = rc;
    }
    {
        std::lock_guard<std::mutex> lk(ctx->table_mutex);
        ctx->event_pool.insert(ctx->event_pool.end(), used.begin(), used.end());
    }
    req->file->open_requests.fetch_sub(1);
    return status < 0 ? status : (int64_t)req->length;
}

int fstx_get_metrics(fstx_ctx *ctx, fstx_metrics *out) {
    // the caller says how large its struct is; a caller built against an older header gets the
    // fields it knows and nothing is written behind them
    if (!ctx || !out || out->struct_size < 2 * sizeof(uint64_t)) return -FSTX_E_INVAL;
    (void)wait_built(ctx); // where the workers and the ring ended up is part of the answer
    const Counters &c = ctx->ctr;
    fstx_metrics m{};
    m.struct_size = std::min<uint64_t>(out->struct_size, sizeof(fstx_metrics));
    m.bounce_buffer_bytes = ctx->ring_bytes;
    m.bytes_read = c.bytes_read.load();
    m.bytes_copied = c.bytes_copied.load();
    m.blocks_buffered = c.blocks_buffered.load();
    m.blocks_direct = c.blocks_direct.load();
    m.read_ns = c.read_ns.load();
    m.stage_ns = c.stage_ns.load();
    m.slot_wait_ns = c.slot_wait_ns.load();
    m.direct_fallbacks = c.direct_fallbacks.load();
    m.direct_depth = ctx->direct_gate->settled();
    m.direct_reads = c.direct_reads.load();
    m.create_ns = ctx->create_ns;
    m.numa_node = ctx->cfg.numa_node;
    m.workers_on_node = c.workers_on_node.load();
    m.ring_node = ctx->ring_node;
    m.bind_errors = c.bind_errors.load();
    m.first_bind_error = c.first_bind_error.load();
    m.pretouched_bytes = c.pretouched_bytes.load();
    m.ring_reused = ctx->ring_reused ? 1 : 0;
    {
        std::lock_guard<std::mutex> lk(ctx->q_mutex);
        m.direct_read_bytes = ctx->shape_settled ? ctx->direct_bytes : 0;
        m.direct_steered = ctx->shape_settled && ctx->adaptive_depth;
        m.staging_buffers_max = ctx->shape_settled ? ctx->stage_max : 0;
        m.storage_nr_requests = ctx->storage.nr_requests;
        m.storage_max_sectors_kb = ctx->storage.max_sectors_kb;
        m.storage_flags = (ctx->storage.known ? FSTX_STORAGE_KNOWN : 0) | (ctx->storage.rotational ? FSTX_STORAGE_ROTATIONAL : 0) |
                          (ctx->storage.virtio ? FSTX_STORAGE_VIRTIO : 0);
    }
    std::memcpy(out, &m, (size_t)m.struct_size);
    return 0;
}

} // extern "C"
