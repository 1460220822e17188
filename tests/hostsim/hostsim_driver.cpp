// SPDX-License-Identifier: Apache-2.0
//
// TEST INFRASTRUCTURE.  Drives the copy pipeline (built against the in-memory
// device stand-in) from several caller threads at once; meant to be built with
// -fsanitize=thread or -fsanitize=address.  Exit status 0 = every byte matched.
//
//   hostsim_driver <file> [rounds]

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <thread>
#include <vector>

#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include "fstx.h"

extern "C" void fstx_sim_set_copy_delay_us(int us);
extern "C" void *fstx_sim_stream_create(void);
extern "C" void fstx_sim_stream_destroy(void *s);
extern "C" void fstx_sim_stream_sleep_then_set(void *s, int us, volatile int *flag, int value);

int main(int argc, char **argv) {
    if (argc < 2) return 2;
    const char *path = argv[1];
    int rounds = argc > 2 ? std::atoi(argv[2]) : 3;
    struct stat st;
    if (stat(path, &st) != 0) return 2;
    const uint64_t size = (uint64_t)st.st_size;
    std::vector<char> truth(size);
    {
        int fd = open(path, O_RDONLY);
        uint64_t got = 0;
        while (got < size) {
            ssize_t c = pread(fd, truth.data() + got, size - got, (off_t)got);
            if (c <= 0) return 2;
            got += (uint64_t)c;
        }
        close(fd);
    }
    fstx_sim_set_copy_delay_us(20);
    const char *cache_env = std::getenv("FSTX_RING_CACHE");
    const bool ring_cache_expected = !(cache_env && cache_env[0] == '0');
    std::atomic<int> bad{0};
    for (int turn = 0; turn < 2 * rounds; ++turn) {
        const int round = turn / 2; // every shape twice in a row: the second context takes over the ring the first left parked
        fstx_config cfg{};
        cfg.struct_size = sizeof cfg;
        cfg.device_id = 0;
        cfg.numa_node = round == 1 ? 0 : -1; // one round with the workers bound to a node and the ring placed on it
        cfg.n_threads = 2 + round * 3;
        cfg.n_streams = 1 + round;
        cfg.block_bytes = 4096u << (round * 2);
        cfg.slots_per_thread = 1 + round % 2;
        cfg.direct_read_bytes = round == 1 ? 0 : cfg.block_bytes * 3;
        // rounds 0 and 1: the context is built behind the callers' backs while they open files and queue reads
        cfg.flags = round == 2 ? FSTX_ADAPTIVE_DEPTH : FSTX_CREATE_ASYNC;
        cfg.direct_ramp_kb = round == 0 ? 4 : 0;
        fstx_ctx *ctx = nullptr, *again = nullptr;
        // odd rounds go through the shared table: two users of one context
        if (round % 2) {
            if (fstx_ctx_acquire(&cfg, &ctx) != 0 || fstx_ctx_acquire(&cfg, &again) != 0 || again != ctx) return 3;
        } else if (fstx_ctx_create(&cfg, &ctx) != 0) {
            return 3;
        }
        void *foreign = fstx_sim_stream_create();
        volatile int flag = 0;
        std::vector<std::thread> callers;
        for (int c = 0; c < 3; ++c) {
            callers.emplace_back([&, c] {
                std::mt19937_64 rng(round * 100 + c);
                int64_t file = fstx_file_open(ctx, path, c % 3);
                if (file < 0) { bad++; return; }
                std::vector<char> dev(size + 64, 0x5a);
                std::vector<int64_t> reqs;
                std::vector<std::pair<uint64_t, uint64_t>> spans;
                uint64_t at = 0;
                while (at < size) {
                    uint64_t len = 1 + rng() % (size / 5 + 1);
                    if (at + len > size) len = size - at;
                    if (rng() % 4 == 0) {
                        fstx_sim_stream_sleep_then_set(foreign, 50, &flag, c);
                        if (fstx_ctx_order_after(ctx, foreign) != 0) bad++;
                    }
                    int64_t r = fstx_submit_read(ctx, file, at, len, dev.data(), dev.size(), at + 7);
                    if (r < 0) { bad++; break; }
                    reqs.push_back(r);
                    spans.push_back({at, len});
                    at += len;
                }
                for (size_t i = 0; i < reqs.size(); ++i)
                    if (fstx_wait_read(ctx, reqs[i]) != (int64_t)spans[i].second) bad++;
                if (std::memcmp(dev.data() + 7, truth.data(), size) != 0) bad++;
                if (fstx_file_close(ctx, file) != 0) bad++;
            });
        }
        for (auto &t : callers) t.join();
        fstx_metrics m{};
        m.struct_size = sizeof m;
        fstx_get_metrics(ctx, &m);
        if (m.bytes_copied != 3 * size) bad++;
        if (ring_cache_expected && m.ring_reused != (uint64_t)(turn % 2)) bad++;
        fstx_sim_stream_destroy(foreign); // drains it: the stand-in's events must outlive their records
        if (again && fstx_ctx_release(again) != 0) bad++;
        if ((again ? fstx_ctx_release(ctx) : fstx_ctx_destroy(ctx)) != 0) bad++;
    }
    fstx_trim_cache(); // the ring the last context left parked
    if (fstx_bounce_buffer_bytes() != 0 || fstx_cached_ring_bytes() != 0) bad++;
    std::printf("hostsim_driver: %s\n", bad.load() ? "MISMATCH" : "ok");
    return bad.load() ? 1 : 0;
}
