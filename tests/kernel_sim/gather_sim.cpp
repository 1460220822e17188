// SPDX-License-Identifier: Apache-2.0
//
// TEST INFRASTRUCTURE.  Runs the gather kernel's lane logic (fstx_gather_core.h, the same
// source the GPU kernel is built from) lane by lane on the CPU over caller-provided buffers,
// with every memory access checked: a load must lie inside one source's block (first byte of
// its first segment to last byte of its last), a store must hit payload bytes of the destination, and every payload byte must be
// written exactly once.  Lets the index arithmetic be swept over odd shapes and alignments
// without a GPU.  Not part of the shipped library.
#include <cstdint>
#include <cstring>
#include <vector>

#include "fstx_gather_core.h"

using namespace fstx_gather;

namespace {

struct SimMem {
    const Job *job;
    const Src *srcs;
    std::vector<uint8_t> *written; // per destination position: times written
    char *dst_lo;                  // allocation bounds of the destination
    char *dst_hi;
    int64_t errors = 0;

    Vec16 load16_stream(const char *p) { return load16(p); }
    // a table entry read by a lane of its own: inside the job's part of the launch's table
    Src table(const Src *more, uint32_t index) {
        if (index < job->more0 || index >= (uint32_t)job->more0 + job->nsrc) {
            ++errors;
            return Src{nullptr, 0, 0, 0, 0};
        }
        return more[index];
    }
    // a load must lie inside one source's block: from the first byte of its first segment to the
    // last byte of its last segment (what the caller guarantees to be readable)
    Vec16 load16(const char *p) {
        bool ok = false;
        for (uint32_t k = 0; k < job->nsrc && !ok; ++k) {
            const Src &s = srcs[k];
            ok = p >= s.src && p + kVec <= s.src + (uint64_t)(job->rows - 1) * s.pitch + s.seg;
        }
        Vec16 v = {{0, 0, 0, 0}};
        if (!ok) {
            ++errors;
            return v;
        }
        std::memcpy(&v, p, kVec);
        return v;
    }
    void note(char *p) {
        if (p < job->dst || p >= dst_hi) {
            ++errors;
            return;
        }
        const uint64_t pos = (uint64_t)(p - job->dst);
        const uint64_t row = pos / job->dst_pitch, c = pos % job->dst_pitch;
        if (row >= job->rows || c >= job->row_bytes || (*written)[pos] == 255) {
            ++errors;
            return;
        }
        ++(*written)[pos];
    }
    void store16(char *p, Vec16 v) {
        if (((uintptr_t)p & 15) || p < dst_lo || p + kVec > dst_hi) {
            ++errors;
            return;
        }
        for (uint32_t i = 0; i < kVec; ++i) note(p + i);
        std::memcpy(p, &v, kVec);
    }
    // sixteen bytes at any address; the bytes a neighbouring vector has written already must not change
    void store16_any(char *p, Vec16 v) {
        if (p < dst_lo || p + kVec > dst_hi) {
            ++errors;
            return;
        }
        const char *bytes = reinterpret_cast<const char *>(&v);
        for (uint32_t i = 0; i < kVec; ++i) {
            const uint64_t pos = (uint64_t)(p + i - job->dst);
            if (p + i >= job->dst && pos < written->size() && (*written)[pos] && p[i] != bytes[i]) ++errors;
            note(p + i);
        }
        std::memcpy(p, &v, kVec);
    }
    void store8(char *p, unsigned char b) {
        note(p);
        if (p >= dst_lo && p < dst_hi) *p = (char)b;
    }
};

uint32_t g_dies_log2 = 3;

} // namespace

// dies the simulated launch deals its tiles out to: 1 << log2, log2 in 0..3
extern "C" void fstx_sim_set_dies_log2(uint32_t log2) { g_dies_log2 = log2 > kMaxDiesLog2 ? kMaxDiesLog2 : log2; }

// Runs one job: `n` sources (src[i], seg[i], pitch[i]) into dst rows `dst_pitch` apart.
// Returns 0 when every access was legal and every payload byte was written exactly once,
// -1 when the shape is outside the kernel's domain, else the number of violations.
extern "C" int64_t fstx_gather_sim(char *dst, uint64_t dst_capacity_before, uint64_t dst_capacity_after, uint64_t dst_pitch,
                                   uint64_t rows, const char *const *src, const uint64_t *seg, const uint64_t *pitch,
                                   uint32_t n, int general) {
    std::vector<Src> srcs(n);
    uint64_t col = 0, min_seg = ~0ull, equal = n ? seg[0] : 0;
    for (uint32_t i = 0; i < n; ++i) {
        srcs[i] = Src{src[i], pitch[i], (uint32_t)seg[i], (uint32_t)col, 0};
        col += seg[i];
        if (seg[i] < min_seg) min_seg = seg[i];
        if (seg[i] != equal) equal = 0;
    }
    if (dst_pitch == 0) dst_pitch = col;
    if (!shape_ok(dst_pitch, col, min_seg) || rows == 0 || rows > rows_per_job(dst_pitch, col)) return -1;
    // the sources of a job with several sit in the launch's table; one source travels in the job
    const uint32_t more0 = 3; // somewhere inside a larger table
    std::vector<Src> more(more0 + n);
    for (uint32_t i = 0; i < n; ++i) more[more0 + i] = srcs[i];
    const Job jb = make_job(dst, dst_pitch, col, rows, srcs[0], more0, n, n > 1 ? equal : 0, min_seg);
    std::vector<uint8_t> written((rows - 1) * dst_pitch + col, 0);
    SimMem mem{&jb, srcs.data(), &written, dst - dst_capacity_before, dst + dst_capacity_after};
    const uint64_t tiles = tiles_of(jb);
    // the leanest variant the job allows, as the library picks it (general = 1 forces the full one)
    const bool multi = n > 1 || general, pitched = dst_pitch != col || general;
    // workgroup by workgroup in the order the kernel deals tiles out to the dies; a tile that is
    // skipped or visited twice shows up as payload bytes written never or twice
    const uint64_t dies = 1ull << g_dies_log2;
    for (uint64_t lb = 0; lb < (tiles + dies - 1) / dies * dies; ++lb) {
        uint32_t t;
        if (!tile_for_die((uint32_t)lb, (uint32_t)tiles, g_dies_log2, t)) continue;
        for (uint32_t lane = 0; lane < kLanes; ++lane) {
            if (multi && pitched) gather_lane<true, true>(jb, more.data(), (uint32_t)t, lane, mem);
            else if (multi) gather_lane<true, false>(jb, more.data(), (uint32_t)t, lane, mem);
            else if (pitched) gather_lane<false, true>(jb, more.data(), (uint32_t)t, lane, mem);
            else gather_lane<false, false>(jb, more.data(), (uint32_t)t, lane, mem);
        }
    }
    int64_t bad = mem.errors;
    for (uint64_t r = 0; r < rows; ++r)
        for (uint64_t c = 0; c < col; ++c)
            if (written[r * dst_pitch + c] != 1 && !((jb.flags & kLooseRows) && written[r * dst_pitch + c] == 2)) ++bad;
    return bad;
}

// The tile a workgroup takes (tile_for_die), for all workgroups of a job of n_tiles tiles:
// out[lb] = tile, or 0xffffffff for an idle workgroup.  Returns the number of workgroups.
extern "C" uint64_t fstx_tile_order_sim(uint32_t n_tiles, uint32_t *out) {
    const uint64_t dies = 1ull << g_dies_log2;
    const uint64_t groups = ((uint64_t)n_tiles + dies - 1) / dies * dies;
    for (uint64_t lb = 0; lb < groups; ++lb) {
        uint32_t t = 0;
        out[lb] = tile_for_die((uint32_t)lb, n_tiles, g_dies_log2, t) ? t : 0xffffffffu;
    }
    return groups;
}

// floor(n / d) by the kernel's multiply-high division, for the tests
extern "C" uint32_t fstx_div_magic_sim(uint32_t n, uint64_t d) { return div_magic(n, magic_of(d)); }
