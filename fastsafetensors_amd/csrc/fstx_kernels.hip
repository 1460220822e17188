// SPDX-License-Identifier: Apache-2.0
//
// HBM kernels of the load path, written for gfx950 (CDNA4): 64-wide wavefronts,
// 16-byte global loads/stores per lane, no MFMA (data movement and element-wise
// rounding only; the bound is HBM bandwidth).
//
//   realign copy   : dst[0:n) = src[0:n) for any byte alignment of src and dst.
//                    Stands in for gds_device_buffer::memmove of the reference
//                    (cpp/ext.cpp:606-645: two cudaMemcpy through a temporary).
//   slice extract  : dense copy of `outer` segments read at a fixed pitch.
//                    Stands in for t[slices].contiguous() per rank in
//                    LazyTensorFactory.shuffle (tensor_factory.py:168-175), and, with
//                    several sources side by side, for that plus torch.cat in
//                    shuffle_multi_cols (tensor_factory.py:194-259).  The gather kernel
//                    serves every shape and alignment with 16-byte loads at the data's own
//                    byte address; a 16-byte-unit kernel serves cuts that are aligned
//                    throughout, a small-unit kernel segments shorter than 16 bytes.
//   down-cast      : element type conversion towards a narrower type with torch's
//                    rounding (SafeTensorsMetadata.get_tensors with a dtype,
//                    common.py:355-375).
//
// Every kernel takes a table of jobs as a by-value kernel argument (up to
// FSTX_BATCH_MAX), so that the many small tensors of a checkpoint file cost one
// launch.  A workgroup is one wavefront and owns 64 consecutive 16-byte vectors
// of one job's destination; consecutive lanes touch consecutive vectors, so each
// wavefront reads and writes contiguous spans.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <atomic>
#include <mutex>

#include "fstx.h"
#include "fstx_gather_core.h"
#include "fstx_internal.h"

namespace {

typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef v4u v4u_anywhere __attribute__((aligned(1))); // sixteen bytes at any address

// Every pointer a job carries is device memory.  Saying so (address space 1) lets the
// compiler emit global_load/global_store instead of flat accesses, which would have to
// allow for LDS and scratch apertures and cannot be issued wide at odd alignments.
#define FSTX_GLOBAL __attribute__((address_space(1)))
template <typename T> __device__ __forceinline__ T ld_stream(const T *p) {
    return __builtin_nontemporal_load((const FSTX_GLOBAL T *)p);
}
template <typename T> __device__ __forceinline__ void st_stream(T v, T *p) {
    __builtin_nontemporal_store(v, (FSTX_GLOBAL T *)p);
}
template <typename T> __device__ __forceinline__ T ld_global(const T *p) { return *(const FSTX_GLOBAL T *)p; }
template <typename T> __device__ __forceinline__ void st_global(T v, T *p) { *(FSTX_GLOBAL T *)p = v; }

// One wavefront per workgroup measured fastest for a streaming copy on MI355X
// (6.5 TB/s against 6.3 TB/s with 128..512 lanes): the dispatcher then spreads
// single waves evenly and none waits for a sibling to retire.
#ifndef FSTX_BLOCK
#define FSTX_BLOCK 64
#endif
constexpr int kBlock = FSTX_BLOCK; // lanes per workgroup
constexpr int kVecBytes = 16;      // bytes moved per lane per step

// ---------------------------------------------------------------- job tables

struct alignas(32) RealignJob {
    char *dst;
    const char *src;
    uint64_t nbytes;
    uint64_t pad;
};

// 32 bytes, so that a workgroup fetches its job with one wide scalar load
struct alignas(32) SliceJob {
    char *dst;
    const char *src;
    uint64_t pitch_unit;  // bytes between segment starts in src (< 2^56) | log2(unit bytes) << 56
    uint32_t seg_units;   // units per segment
    uint32_t total_units; // outer * seg_units  (< 2^32 by construction)
};

// Workgroup -> job in O(1).  The grid is cut into granules of 2^granule_log2
// workgroups; every job starts on a granule boundary (its last granule may hold a
// few idle workgroups) and owner[] names the job of each granule.  The host picks
// the smallest granule for which the launch fits kOwnerSlots granules, so a
// workgroup finds its job with one table lookup instead of a search.
constexpr uint32_t kOwnerSlots = 2048;

typedef uint32_t v8u __attribute__((ext_vector_type(8)));
typedef uint32_t v16u __attribute__((ext_vector_type(16)));

// Kernel arguments are limited to 4 KiB: 48 jobs of 32 bytes or 24 jobs of 64 bytes fit
// next to the two lookup tables.
template <typename Job, uint32_t kJobsN = (sizeof(Job) == 32 ? FSTX_BATCH_MAX : FSTX_BATCH_MAX / 2),
          uint32_t kSlotsN = kOwnerSlots>
struct JobTable {
    static_assert(sizeof(Job) == 32 || sizeof(Job) == 64, "jobs are fetched as eight or sixteen dwords");
    static constexpr uint32_t kJobs = kJobsN;
    static constexpr uint32_t kSlots = kSlotsN;
    Job job[kJobs];
    uint32_t first_block[kJobs]; // first workgroup of each job (granule aligned)
    uint32_t owner[kSlots / 4];  // one byte per granule: index into job[]

    // the whole job in one scalar load
    __device__ __forceinline__ Job fetch(uint32_t ji) const {
        Job out;
        if constexpr (sizeof(Job) == 32) {
            const v8u raw = *reinterpret_cast<const v8u *>(&job[ji]);
            __builtin_memcpy(&out, &raw, sizeof out);
        } else {
            const v16u raw = *reinterpret_cast<const v16u *>(&job[ji]);
            __builtin_memcpy(&out, &raw, sizeof out);
        }
        return out;
    }
};

template <typename Table>
__device__ __forceinline__ uint32_t find_job(const Table &t, uint32_t granule_log2, uint32_t b) {
    const uint32_t g = b >> granule_log2;
    return (t.owner[g >> 2] >> ((g & 3) * 8)) & 0xffu;
}

// Dies the current device deals workgroups out to, as log2: its compute units / 32 (a die of an
// MI355X has 32 of them active, so a whole device gives 8 and its partitions 4, 2 or 1), 8 when
// the runtime does not say; FSTX_DIES overrides it (1, 2, 4 or 8; measurements and tests).  Any
// value gives the right bytes -- the tile order is a permutation for each -- the right one keeps
// neighbouring tiles on one die.
inline uint32_t dies_log2() {
    static std::atomic<int> cache[64];
    static std::once_flag once;
    std::call_once(once, [] {
        for (auto &c : cache) c.store(-1);
    });
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fstx_gather::kMaxDiesLog2;
    int got = cache[dev].load(std::memory_order_relaxed);
    if (got >= 0) return (uint32_t)got;
    uint32_t dies = 8;
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0) dies = (uint32_t)cus / 32;
    if (const char *e = getenv("FSTX_DIES")) dies = (uint32_t)strtoul(e, nullptr, 10);
    uint32_t log2 = 0;
    while (log2 < fstx_gather::kMaxDiesLog2 && (2u << log2) <= dies) ++log2;
    cache[dev].store((int)log2, std::memory_order_relaxed);
    return log2;
}
inline uint64_t pad_to_dies(uint64_t workgroups) {
    const uint64_t d = 1ull << dies_log2();
    return (workgroups + d - 1) / d * d;
}

// Host side: lays the jobs' workgroup counts out on granules; returns the grid size and the
// kernels' leading argument (granule_log2 | dies_log2 << 8).
template <typename Table>
inline uint64_t plan_grid(Table &t, const uint64_t *blocks_of, uint32_t n, uint32_t *launch_word) {
    uint32_t gl = 0;
    for (;; ++gl) {
        uint64_t need = 0;
        for (uint32_t i = 0; i < n; ++i) need += (blocks_of[i] + (1ull << gl) - 1) >> gl;
        if (need <= Table::kSlots) break;
    }
    uint64_t granule = 0;
    uint8_t *owner = reinterpret_cast<uint8_t *>(t.owner);
    for (uint32_t i = 0; i < n; ++i) {
        t.first_block[i] = (uint32_t)(granule << gl);
        const uint64_t span = (blocks_of[i] + (1ull << gl) - 1) >> gl;
        for (uint64_t k = 0; k < span; ++k) owner[granule + k] = (uint8_t)i;
        granule += span;
    }
    *launch_word = gl | dies_log2() << 8;
    return granule << gl;
}

using fstx_gather::tile_for_die;

// ------------------------------------------------------------- realign copy

// bytes [4*Q + r, 4*Q + r + 16) of the 32-byte pair (lo, hi); r in 0..3
template <int Q>
__device__ __forceinline__ v4u funnel(v4u lo, v4u hi, uint32_t r) {
    const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    v4u out;
    out.x = __builtin_amdgcn_alignbyte(w[Q + 1], w[Q + 0], r);
    out.y = __builtin_amdgcn_alignbyte(w[Q + 2], w[Q + 1], r);
    out.z = __builtin_amdgcn_alignbyte(w[Q + 3], w[Q + 2], r);
    out.w = __builtin_amdgcn_alignbyte(w[Q + 4], w[Q + 3], r);
    return out;
}

// value of `v` in the next lane of the wavefront (lane 63 gets an unspecified value)
__device__ __forceinline__ uint32_t from_next_lane(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x130 /* wave_shl:1 */, 0xf, 0xf, false);
}

__global__ __launch_bounds__(kBlock) void realign_kernel(const uint32_t launch_word,
                                                          const JobTable<RealignJob> t) {
    const uint32_t b = blockIdx.x;
    const uint32_t granule_log2 = launch_word & 0xffu, dies_log2 = launch_word >> 8;
    const uint32_t ji = find_job(t, granule_log2, b);
    const RealignJob job = t.fetch(ji);
    const uint32_t lb = b - t.first_block[ji];

    // split into head bytes (until dst is 16-aligned), whole vectors, tail bytes
    uint64_t head = (uint64_t)(-(intptr_t)job.dst) & (kVecBytes - 1);
    if (head > job.nbytes) head = job.nbytes;
    const uint64_t nvec = (job.nbytes - head) / kVecBytes;
    const uint64_t tail_at = head + nvec * kVecBytes;

    if (lb == 0) {
        // at most 15 + 15 edge bytes, one per lane
        const uint64_t edge = head + (job.nbytes - tail_at);
        const uint64_t e = threadIdx.x;
        if (e < edge) {
            const uint64_t at = e < head ? e : tail_at + (e - head);
            st_global(ld_global(job.src + at), job.dst + at);
        }
    }

    v4u *dstv = reinterpret_cast<v4u *>(job.dst + head);
    const char *s = job.src + head;
    const uint32_t m = (uint32_t)(uintptr_t)s & (kVecBytes - 1);
    // The 1 KiB spans of neighbouring wavefronts share a cache line (source or destination not
    // on a 128-byte boundary) or a source vector (source shifted): neighbours run on the same
    // die, in the tile order of tile_for_die (which also measured faster than dispatch order
    // when nothing is shared).
    uint32_t tile;
    const bool tile_live = tile_for_die(lb, (uint32_t)((nvec + kBlock - 1) / kBlock), dies_log2, tile);
    const uint64_t j = (uint64_t)tile * kBlock + threadIdx.x;
    if (m == 0) {
        // source vectors are aligned: a plain streaming copy
        const v4u *srcv = reinterpret_cast<const v4u *>(s);
        if (tile_live && j < nvec) st_stream(ld_stream(srcv + j), dstv + j);
        return;
    }
    const bool live = tile_live && j < nvec; // idle workgroups pad a job to a multiple of eight and to granules
    // Source vectors are loaded at their natural 16-byte alignment; output vector j
    // is bytes [m, m+16) of aligned vectors j and j+1.  Every lane loads vector j
    // once and takes vector j+1 from its right-hand neighbour in the wavefront;
    // only the last lane of a wavefront (and the lane that ends the job) loads
    // j+1 itself.  Vector j+1 always overlaps a source byte of this job, so it
    // never leaves the 16-byte granule that holds the last valid byte.
    const v4u *srcv = reinterpret_cast<const v4u *>(s - m);
    const bool edge = live && ((threadIdx.x & 63) == 63 || j + 1 == nvec);
    v4u lo = {0, 0, 0, 0}, own_hi = {0, 0, 0, 0};
    if (live) lo = ld_stream(srcv + j);
    if (edge) own_hi = ld_stream(srcv + j + 1); // issued before lo is waited for
    v4u hi;
    hi.x = from_next_lane(lo.x);
    hi.y = from_next_lane(lo.y);
    hi.z = from_next_lane(lo.z);
    hi.w = from_next_lane(lo.w);
    if (!live) return;
    if (edge) hi = own_hi;
    const uint32_t r = m & 3;
    v4u out;
    switch (m >> 2) { // uniform across the workgroup
    case 0: out = funnel<0>(lo, hi, r); break;
    case 1: out = funnel<1>(lo, hi, r); break;
    case 2: out = funnel<2>(lo, hi, r); break;
    default: out = funnel<3>(lo, hi, r); break;
    }
    st_stream(out, dstv + j);
}

// ------------------------------------------------------------ slice extract

template <typename Unit>
__device__ __forceinline__ void slice_units(const SliceJob &job, uint32_t u) {
    const uint32_t row = u / job.seg_units;
    const uint32_t col = u - row * job.seg_units;
    const uint64_t pitch = job.pitch_unit & 0x00ffffffffffffffull;
    const Unit *src = reinterpret_cast<const Unit *>(job.src + (uint64_t)row * pitch) + col;
    Unit *dst = reinterpret_cast<Unit *>(job.dst) + u;
    st_stream(ld_stream(src), dst);
}

// Units under 16 bytes into a 16-byte-aligned dense destination: a lane gathers the 16 / sizeof(Unit)
// units of one destination vector -- as many loads, issued together -- and writes them with one
// 16-byte store, so a wavefront still writes 1 KiB of contiguous memory (one unit per lane is
// 64 to 512 bytes per wavefront).  `g` is the index of the destination vector.
template <typename Unit>
__device__ __forceinline__ void slice_units_packed(const SliceJob &job, uint32_t g) {
    constexpr uint32_t kPer = kVecBytes / sizeof(Unit);
    const uint32_t u0 = g * kPer; // < total_units + kPer, which the host keeps below 2^32
    if (u0 >= job.total_units) return;
    const uint64_t pitch = job.pitch_unit & 0x00ffffffffffffffull;
    uint32_t row = u0 / job.seg_units;
    uint32_t col = u0 - row * job.seg_units;
    const uint32_t live = job.total_units - u0 < kPer ? job.total_units - u0 : kPer;
    Unit part[kPer];
#pragma unroll
    for (uint32_t k = 0; k < kPer; ++k) {
        part[k] = Unit{};
        if (k < live) part[k] = ld_global(reinterpret_cast<const Unit *>(job.src + (uint64_t)row * pitch) + col);
        if (++col == job.seg_units) {
            col = 0;
            ++row;
        }
    }
    Unit *dst = reinterpret_cast<Unit *>(job.dst) + u0;
    if (live == kPer) {
        v4u whole;
        __builtin_memcpy(&whole, part, sizeof whole);
        st_stream(whole, reinterpret_cast<v4u *>(dst));
    } else {
#pragma unroll
        for (uint32_t k = 0; k < kPer; ++k)
            if (k < live) st_global(part[k], dst + k);
    }
}

constexpr uint32_t kPackedUnits = 0x80; // in the unit byte of SliceJob::pitch_unit: slice_units_packed

__global__ __launch_bounds__(kBlock) void slice_kernel(const uint32_t launch_word,
                                                        const JobTable<SliceJob> t) {
    const uint32_t b = blockIdx.x;
    const uint32_t granule_log2 = launch_word & 0xffu, dies_log2 = launch_word >> 8;
    const uint32_t ji = find_job(t, granule_log2, b);
    const SliceJob job = t.fetch(ji);
    const uint32_t lb = b - t.first_block[ji];
    const uint32_t mode = (uint32_t)(job.pitch_unit >> 56);
    // items: units, or (packed) destination vectors of 16 >> unit_log2 units
    const uint32_t per_log2 = mode & kPackedUnits ? 4 - (mode & 7) : 0;
    const uint32_t items = (uint32_t)(((uint64_t)job.total_units + (1u << per_log2) - 1) >> per_log2);
    // neighbouring workgroups on the same die, in the tile order of tile_for_die
    uint32_t tile;
    if (!tile_for_die(lb, (items + kBlock - 1) / kBlock, dies_log2, tile)) return;
    const uint64_t u64 = (uint64_t)tile * kBlock + threadIdx.x;
    if (u64 >= items) return; // also retires the idle workgroups of a job's last granule
    const uint32_t u = (uint32_t)u64;
    switch (mode) { // uniform across the workgroup
    case 4: slice_units<v4u>(job, u); break;
    case 3: slice_units<uint64_t>(job, u); break;
    case 2: slice_units<uint32_t>(job, u); break;
    case 1: slice_units<uint16_t>(job, u); break;
    case 0: slice_units<uint8_t>(job, u); break;
    case kPackedUnits | 3: slice_units_packed<uint64_t>(job, u); break;
    case kPackedUnits | 2: slice_units_packed<uint32_t>(job, u); break;
    case kPackedUnits | 1: slice_units_packed<uint16_t>(job, u); break;
    default: slice_units_packed<uint8_t>(job, u); break;
    }
}

// Segments under 16 bytes whose rows lie close together (a [N, 4] tensor cut in four: two bytes of
// every eight): the rows that feed one tile of the destination span a few KiB of source, which the
// wavefront copies into LDS with whole 16-byte loads -- every line of the source is requested once --
// and then picks apart: a lane reads the 16 / unit units of its destination vector out of LDS and
// writes them with one 16-byte store.  One unit per global load, as the other unit paths do it,
// asks the memory pipeline for each line many times over.
constexpr uint32_t kStageBytes = 8192;

template <typename Unit>
__device__ __forceinline__ void units_from_stage(const SliceJob &job, const unsigned char *stage, uint32_t pitch, uint32_t r0,
                                                 uint32_t q, uint32_t total) {
    constexpr uint32_t kPer = kVecBytes / sizeof(Unit);
    const uint32_t seg = job.seg_units * (uint32_t)sizeof(Unit);
    uint32_t row = q / seg;
    uint32_t cu = (q - row * seg) / (uint32_t)sizeof(Unit);
    const uint32_t left = (total - q) / (uint32_t)sizeof(Unit);
    const uint32_t live = left < kPer ? left : kPer;
    Unit part[kPer];
#pragma unroll
    for (uint32_t k = 0; k < kPer; ++k) {
        part[k] = Unit{};
        if (k < live) part[k] = *reinterpret_cast<const Unit *>(stage + (row - r0) * pitch + cu * (uint32_t)sizeof(Unit));
        if (++cu == job.seg_units) {
            cu = 0;
            ++row;
        }
    }
    char *dst = job.dst + q;
    if (live == kPer) {
        v4u whole;
        __builtin_memcpy(&whole, part, sizeof whole);
        st_stream(whole, reinterpret_cast<v4u *>(dst));
    } else {
#pragma unroll
        for (uint32_t k = 0; k < kPer; ++k)
            if (k < live) st_global(part[k], reinterpret_cast<Unit *>(dst) + k);
    }
}

__global__ __launch_bounds__(kBlock) void stage_kernel(const uint32_t launch_word, const JobTable<SliceJob> t) {
    extern __shared__ __attribute__((aligned(16))) unsigned char stage[]; // as many bytes as the launch's widest window (<= kStageBytes)
    const uint32_t b = blockIdx.x;
    const uint32_t granule_log2 = launch_word & 0xffu, dies_log2 = launch_word >> 8;
    const uint32_t ji = find_job(t, granule_log2, b);
    const SliceJob job = t.fetch(ji);
    const uint32_t lb = b - t.first_block[ji];
    const uint32_t ul = (uint32_t)(job.pitch_unit >> 56) & 7u;
    const uint32_t pitch = (uint32_t)job.pitch_unit; // a few KiB at most (the host checks)
    const uint32_t seg = job.seg_units << ul;
    const uint32_t total = job.total_units << ul;    // destination bytes, below 2^32 (the host cuts jobs accordingly)
    constexpr uint32_t kTileBytes = kBlock * kVecBytes;
    uint32_t tile;
    if (!tile_for_die(lb, (total + kTileBytes - 1) / kTileBytes, dies_log2, tile)) return;
    const uint32_t d0 = tile * kTileBytes;
    const uint32_t d1 = total - d0 < kTileBytes ? total : d0 + kTileBytes;
    const uint32_t r0 = d0 / seg, r1 = (d1 - 1) / seg; // rows that feed this tile
    const char *win = job.src + (uint64_t)r0 * pitch;
    const uint32_t window = (r1 - r0) * pitch + seg;   // <= kStageBytes; ends with the last row's segment, inside the block
    for (uint32_t at = kVecBytes * threadIdx.x; at < window; at += kTileBytes) {
        if (at + kVecBytes <= window) {
            *reinterpret_cast<v4u *>(stage + at) = *(const FSTX_GLOBAL v4u_anywhere *)(win + at);
        } else { // the window's ragged end: byte by byte, never past the last segment
            for (uint32_t i = at; i < window; ++i) stage[i] = (unsigned char)ld_global(win + i);
        }
    }
    __syncthreads();
    const uint32_t q = d0 + kVecBytes * threadIdx.x;
    if (q >= total) return;
    switch (ul) { // uniform across the workgroup
    case 3: units_from_stage<uint64_t>(job, stage, pitch, r0, q, total); break;
    case 2: units_from_stage<uint32_t>(job, stage, pitch, r0, q, total); break;
    case 1: units_from_stage<uint16_t>(job, stage, pitch, r0, q, total); break;
    default: units_from_stage<uint8_t>(job, stage, pitch, r0, q, total); break;
    }
}

// The same gather with a strided destination: segment `row` is written to
// dst + row * dst_pitch.  Used to cut the blocks of several tensors straight into one
// joined tensor along an inner dimension.
struct alignas(64) Slice2dJob {
    char *dst;
    const char *src;
    uint64_t src_pitch, dst_pitch;
    uint32_t seg_units, total_units, unit_log2, pad0;
    uint64_t pad1, pad2;
};

template <typename Unit>
__device__ __forceinline__ void slice2d_units(const Slice2dJob &job, uint32_t u) {
    const uint32_t row = u / job.seg_units;
    const uint32_t col = u - row * job.seg_units;
    const Unit *src = reinterpret_cast<const Unit *>(job.src + (uint64_t)row * job.src_pitch) + col;
    Unit *dst = reinterpret_cast<Unit *>(job.dst + (uint64_t)row * job.dst_pitch) + col;
    st_stream(ld_stream(src), dst);
}

__global__ __launch_bounds__(kBlock) void slice2d_kernel(const uint32_t launch_word,
                                                          const JobTable<Slice2dJob> t) {
    const uint32_t b = blockIdx.x;
    const uint32_t granule_log2 = launch_word & 0xffu, dies_log2 = launch_word >> 8;
    const uint32_t ji = find_job(t, granule_log2, b);
    const Slice2dJob job = t.fetch(ji);
    const uint32_t lb = b - t.first_block[ji];
    uint32_t tile;
    if (!tile_for_die(lb, (job.total_units + kBlock - 1) / kBlock, dies_log2, tile)) return;
    const uint64_t u64 = (uint64_t)tile * kBlock + threadIdx.x;
    if (u64 >= job.total_units) return;
    const uint32_t u = (uint32_t)u64;
    switch (job.unit_log2) { // uniform across the workgroup
    case 4: slice2d_units<v4u>(job, u); break;
    case 3: slice2d_units<uint64_t>(job, u); break;
    case 2: slice2d_units<uint32_t>(job, u); break;
    case 1: slice2d_units<uint16_t>(job, u); break;
    default: slice2d_units<uint8_t>(job, u); break;
    }
}

// ----------------------------------------------------------------- gather
//
// Slice extract and fused slice + join for any shape and alignment: the lane logic is in
// fstx_gather_core.h (it also runs on the CPU under the bounds-checking simulator of the
// tests).  One 16-byte load at the data's own byte address, one aligned 16-byte store; a
// launch carries up to FSTX_BATCH_MAX jobs and FSTX_BATCH_MAX sources in its arguments.


// kKeep: the launch holds a job with segments shorter than kShortSeg.  A cache line then holds
// parts of several segments, which neighbouring lanes and tiles fetch one after the other, and
// the bulk loads are plain ones that leave the line in the caches (+14 % on a join of 254-byte
// segments; on segments of 2 KB and more streaming loads are 1-5 % faster).
constexpr uint64_t kShortSeg = fstx_gather::kShortSeg;
template <bool kKeep> struct GatherMem {
    // one entry of the launch's source table, for a lane of its own (the table sits in the kernel
    // arguments; two 16-byte loads that hit the same few lines in every wavefront)
    __device__ __forceinline__ fstx_gather::Src table(const fstx_gather::Src *more, uint32_t index) {
        const v4u a = *(const FSTX_GLOBAL v4u *)(&more[index]);
        const v4u b = *((const FSTX_GLOBAL v4u *)(&more[index]) + 1);
        fstx_gather::Src out;
        const uint32_t raw[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        __builtin_memcpy(&out, raw, sizeof out);
        return out;
    }
    // the bulk: streaming loads (every byte of a checkpoint is cut once)
    __device__ __forceinline__ fstx_gather::Vec16 load16_stream(const char *p) {
        const v4u v = kKeep ? *(const FSTX_GLOBAL v4u_anywhere *)p : __builtin_nontemporal_load((const FSTX_GLOBAL v4u_anywhere *)p);
        return fstx_gather::Vec16{{v.x, v.y, v.z, v.w}};
    }
    // the seams: plain loads, their cache lines are about to be used by the neighbouring lanes
    __device__ __forceinline__ fstx_gather::Vec16 load16(const char *p) {
        const v4u v = *(const FSTX_GLOBAL v4u_anywhere *)p;
        return fstx_gather::Vec16{{v.x, v.y, v.z, v.w}};
    }
    __device__ __forceinline__ void store16(char *p, fstx_gather::Vec16 v) {
        st_stream(v4u{v.w[0], v.w[1], v.w[2], v.w[3]}, reinterpret_cast<v4u *>(p));
    }
    // sixteen bytes at any address
    __device__ __forceinline__ void store16_any(char *p, fstx_gather::Vec16 v) {
        __builtin_nontemporal_store(v4u{v.w[0], v.w[1], v.w[2], v.w[3]}, (FSTX_GLOBAL v4u_anywhere *)p);
    }
    __device__ __forceinline__ void store8(char *p, unsigned char b) { st_global(b, reinterpret_cast<unsigned char *>(p)); }
};

// per launch: 32 jobs (one with a single source carries it), 24 sources of joins, 1,024 granules
constexpr uint32_t kGatherJobs = 32;
constexpr uint32_t kGatherMore = FSTX_JOIN_MAX;
struct GatherTable : JobTable<fstx_gather::Job, kGatherJobs, 1024> {
    fstx_gather::Src more[kGatherMore];
};
static_assert(sizeof(GatherTable) + 32 <= 4096, "kernel arguments are limited to 4 KiB");

template <bool kMulti, bool kPitched, bool kKeep>
__global__ __launch_bounds__(64) void gather_kernel(const uint32_t launch_word, const GatherTable t) {
    const uint32_t b = blockIdx.x;
    const uint32_t granule_log2 = launch_word & 0xffu, dies_log2 = launch_word >> 8;
    const uint32_t ji = find_job(t, granule_log2, b);
    const fstx_gather::Job job = t.fetch(ji);
    const uint32_t lb = b - t.first_block[ji];
    // neighbouring tiles share the cache lines their common border cuts through: neighbours on
    // the same die (tile_for_die)
    const uint32_t n_tiles = (job.nvec + fstx_gather::kLanes - 1) / fstx_gather::kLanes;
    uint32_t tile;
    if (!tile_for_die(lb, n_tiles, dies_log2, tile)) return; // idle padding of the job's grid
    GatherMem<kKeep> mem;
    fstx_gather::gather_lane<kMulti, kPitched>(job, t.more, tile, threadIdx.x, mem);
}

// ------------------------------------------------- down-cast while loading
//
// copy_files_to_device(dtype=...) of the reference converts every tensor with
// torch's Tensor.to() and copies the result back over the start of the tensor's
// bytes (common.py:355-375).  Here one batched launch converts the tensors of a
// file out of place into a smaller arena.  Rounding follows torch's own
// conversions bit for bit: round to nearest even everywhere, bf16 NaNs become
// 0x7fc0, fp8 e4m3fn has no infinity (everything from 480 up, and NaN, becomes
// 0x7f), fp8 e5m2 overflows to infinity; double goes through float first.

#ifndef FSTX_HW_FP8
#define FSTX_HW_FP8 1
#endif
enum : uint32_t { kF64 = 0, kF32 = 1, kF16 = 2, kBF16 = 3, kF8E4M3 = 4, kF8E5M2 = 5 };

struct alignas(32) ConvertJob {
    char *dst;
    const char *src;
    uint64_t n_elems;
    uint32_t src_type, dst_type;
};

__device__ __forceinline__ uint32_t f32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }

template <uint32_t T> struct Elem;
template <> struct Elem<kF64> {
    typedef double type;
    static __device__ __forceinline__ float to_f32(double v) {
        // torch rounds double -> float -> target (two roundings).  The empty asm keeps the
        // compiler from merging the two steps into one correctly rounded double -> half.
        float f = (float)v;
        asm volatile("" : "+v"(f));
        return f;
    }
};
template <> struct Elem<kF32> {
    typedef float type;
    static __device__ __forceinline__ float to_f32(float v) { return v; }
    static __device__ __forceinline__ float from_f32(float f) { return f; }
};
template <> struct Elem<kF16> {
    typedef _Float16 type;
    static __device__ __forceinline__ float to_f32(_Float16 v) { return (float)v; }
    static __device__ __forceinline__ _Float16 from_f32(float f) { return (_Float16)f; } // v_cvt_f16_f32: RNE
};
template <> struct Elem<kBF16> {
    typedef uint16_t type;
    static __device__ __forceinline__ float to_f32(uint16_t v) { return bits_f32((uint32_t)v << 16); }
    static __device__ __forceinline__ uint16_t from_f32(float f) {
        const uint32_t u = f32_bits(f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0; // NaN
        return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
    }
};
template <> struct Elem<kF8E4M3> {
    typedef uint8_t type;
    static __device__ __forceinline__ uint8_t from_f32(float f) {
        uint32_t u = f32_bits(f);
        const uint32_t sign = u & 0x80000000u;
        u ^= sign;
        uint8_t r;
        if (u >= (1087u << 20)) {
            r = 0x7f; // 480 and above, infinities and NaN
        } else if (u < (121u << 23)) {
            // below 2^-6, the smallest normal: let a float addition do the denormal rounding
            const uint32_t magic = 141u << 23;
            r = (uint8_t)(f32_bits(bits_f32(u) + bits_f32(magic)) - magic);
        } else {
            const uint32_t odd = (u >> 20) & 1u;
            u += ((uint32_t)(7 - 127) << 23) + 0x7ffffu + odd;
            r = (uint8_t)(u >> 20);
        }
        return r | (uint8_t)(sign >> 24);
    }
};
template <> struct Elem<kF8E5M2> {
    typedef uint8_t type;
    static __device__ __forceinline__ uint8_t from_f32(float f) {
        uint32_t u = f32_bits(f);
        const uint32_t sign = u & 0x80000000u;
        u ^= sign;
        uint8_t r;
        if (u >= (143u << 23)) {
            r = u > (255u << 23) ? 0x7f : 0x7c; // NaN : infinity (65536 and above overflow)
        } else if (u < (113u << 23)) {
            const uint32_t magic = 134u << 23;
            r = (uint8_t)(f32_bits(bits_f32(u) + bits_f32(magic)) - magic);
        } else {
            const uint32_t odd = (u >> 21) & 1u;
            u += ((uint32_t)(15 - 127) << 23) + 0xfffffu + odd;
            r = (uint8_t)(u >> 21);
        }
        return r | (uint8_t)(sign >> 24);
    }
};

// a 16-byte vector that is only aligned like one element of N bytes
template <int N> struct LooseVec;
template <> struct LooseVec<2> { typedef v4u type __attribute__((aligned(2))); };
template <> struct LooseVec<4> { typedef v4u type __attribute__((aligned(4))); };
template <> struct LooseVec<8> { typedef v4u type __attribute__((aligned(8))); };

template <int N> struct WordOf;
template <> struct WordOf<2> { typedef uint16_t type; };
template <> struct WordOf<4> { typedef uint32_t type; };
template <> struct WordOf<8> { typedef uint64_t type; };
template <> struct WordOf<16> { typedef v4u type; };

// One 16-byte load per lane (16 / sizeof(src) elements), one narrower store per lane.
template <uint32_t S, uint32_t D>
__device__ __forceinline__ void convert_span(const ConvertJob &job, uint32_t lb) {
    typedef typename Elem<S>::type src_t;
    typedef typename Elem<D>::type dst_t;
    constexpr uint32_t kPer = 16 / sizeof(src_t); // elements per lane
    typedef typename WordOf<kPer * sizeof(dst_t)>::type out_t;
    // the 16-byte load is only as aligned as one element: global loads of any width take
    // element-aligned addresses on this hardware
    typedef typename LooseVec<sizeof(src_t)>::type in_t;
    const src_t *src = reinterpret_cast<const src_t *>(job.src);
    dst_t *dst = reinterpret_cast<dst_t *>(job.dst);
    const uint64_t first = ((uint64_t)lb * kBlock + threadIdx.x) * kPer;
    if (first >= job.n_elems) return;
    if (first + kPer <= job.n_elems) {
        const v4u raw = *(const FSTX_GLOBAL in_t *)(src + first);
        src_t in[kPer];
        dst_t out[kPer];
        __builtin_memcpy(in, &raw, 16);
#if FSTX_HW_FP8
        if constexpr (D == kF8E4M3 || D == kF8E5M2) {
            // the hardware's own packed conversion: two values per instruction, nearest-even, overflow
            // to NaN (e4m3fn) or infinity (e5m2) like torch's.  Only its NaNs are encoded differently
            // (torch: 0x7f with the sign of the input): those bytes are put right afterwards.
            uint32_t words[(kPer + 3) / 4] = {};
#pragma unroll
            for (uint32_t k = 0; k < kPer; k += 2) {
                const float a = Elem<S>::to_f32(in[k]), b = Elem<S>::to_f32(in[k + 1]);
                const int old = (int)words[k / 4];
                if constexpr (D == kF8E4M3) {
                    words[k / 4] = (uint32_t)((k / 2) & 1 ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, false));
                } else {
                    words[k / 4] = (uint32_t)((k / 2) & 1 ? __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, false));
                }
                const uint32_t at = 8 * (k & 3);
                if (a != a) words[k / 4] = (words[k / 4] & ~(0xffu << at)) | ((0x7fu | (f32_bits(a) >> 31) << 7) << at);
                if (b != b) words[k / 4] = (words[k / 4] & ~(0xff00u << at)) | ((0x7f00u | (f32_bits(b) >> 31) << 15) << at);
            }
            __builtin_memcpy(out, words, sizeof out);
        } else
#endif
        {
#pragma unroll
            for (uint32_t k = 0; k < kPer; ++k) out[k] = Elem<D>::from_f32(Elem<S>::to_f32(in[k]));
        }
        if (((uintptr_t)job.dst & (sizeof(out_t) - 1)) == 0) { // uniform: one store at its natural alignment
            out_t packed;
            __builtin_memcpy(&packed, out, sizeof packed);
            st_global(packed, reinterpret_cast<out_t *>(dst + first));
        } else { // a destination that is only element-aligned: one store per element
#pragma unroll
            for (uint32_t k = 0; k < kPer; ++k) st_global(out[k], dst + first + k);
        }
    } else { // the ragged end: element by element
        for (uint32_t k = 0; k < kPer && first + k < job.n_elems; ++k)
            st_global(Elem<D>::from_f32(Elem<S>::to_f32(ld_global(src + first + k))), dst + first + k);
    }
}

__global__ __launch_bounds__(kBlock) void convert_kernel(const uint32_t launch_word,
                                                          const JobTable<ConvertJob> t) {
    const uint32_t b = blockIdx.x;
    const uint32_t granule_log2 = launch_word & 0xffu, dies_log2 = launch_word >> 8;
    const uint32_t ji = find_job(t, granule_log2, b);
    const ConvertJob job = t.fetch(ji);
    uint32_t lb = b - t.first_block[ji];
    { // neighbouring workgroups on the same die, in the tile order of tile_for_die, as in the copy kernels
        const uint32_t per_block_log2 = 7 + (job.src_type < 2 ? job.src_type : 2); // 64 lanes x 16 bytes of f64 / f32 / 16-bit
        const uint32_t n_tiles = (uint32_t)((job.n_elems + (1ull << per_block_log2) - 1) >> per_block_log2);
        uint32_t tile;
        if (!tile_for_die(lb, n_tiles, dies_log2, tile)) return;
        lb = tile;
    }
#define FSTX_CONVERT(S, D) \
    case (S) * 8 + (D): convert_span<S, D>(job, lb); break;
    switch (job.src_type * 8 + job.dst_type) { // uniform across the workgroup
        FSTX_CONVERT(kF64, kF32) FSTX_CONVERT(kF64, kF16) FSTX_CONVERT(kF64, kBF16)
        FSTX_CONVERT(kF64, kF8E4M3) FSTX_CONVERT(kF64, kF8E5M2)
        FSTX_CONVERT(kF32, kF16) FSTX_CONVERT(kF32, kBF16) FSTX_CONVERT(kF32, kF8E4M3) FSTX_CONVERT(kF32, kF8E5M2)
        FSTX_CONVERT(kF16, kBF16) FSTX_CONVERT(kF16, kF8E4M3) FSTX_CONVERT(kF16, kF8E5M2)
        FSTX_CONVERT(kBF16, kF16) FSTX_CONVERT(kBF16, kF8E4M3) FSTX_CONVERT(kBF16, kF8E5M2)
    default: break; // rejected on the host
    }
#undef FSTX_CONVERT
}

// --------------------------------------------------------------- host side

inline uint32_t blocks_for(uint64_t items) {
    uint64_t nb = (items + kBlock - 1) / kBlock;
    return nb == 0 ? 1u : (uint32_t)nb;
}

inline uint32_t common_unit_log2(uint64_t bits) {
    // largest power of two <= 16 dividing every value OR-ed into `bits`
    uint32_t l = 0;
    while (l < 4 && ((bits >> l) & 1) == 0) ++l;
    return l;
}

// The size of a launch is counted in work-items with 32 bits: at most 2^32 - 1 lanes, 67.1 M
// workgroups of 64.  Launches are planned up to 56 M workgroups, which leaves room for the
// idle workgroups that pad jobs to granules and eighths; one job takes at most 48 M.
struct Limits {
    uint64_t launch; // workgroups one launch is planned up to
    uint64_t job;    // workgroups one job may take
    uint64_t units() const { return job * kBlock; } // 3.2 G at most: unit indices stay in 32 bits
};
// FSTX_MAX_BLOCKS_PER_LAUNCH shrinks the limits so that tests reach the cutting logic with small tensors.
inline Limits limits() {
    if (const char *e = getenv("FSTX_MAX_BLOCKS_PER_LAUNCH")) {
        const uint64_t v = strtoull(e, nullptr, 10);
        if (v >= 64 && v <= (56ull << 20)) return Limits{v, v - v / 8};
    }
    return Limits{56ull << 20, 48ull << 20};
}
inline bool grid_fits(uint64_t workgroups) { return workgroups * kBlock <= 0xffffffffull; }

// Collects gather jobs and their sources for launches of gather_kernel.
struct GatherBatch {
    GatherTable t;
    uint64_t tiles_of[kGatherJobs];
    uint64_t tiles = 0;
    uint32_t nj = 0, ns = 0;
    bool multi = false, pitched = false, short_segs = false; // what the jobs collected so far ask of the kernel
    hipStream_t stream;
    Limits lim;

    explicit GatherBatch(void *s) : stream(static_cast<hipStream_t>(s)), lim(limits()) {}

    int flush() {
        if (nj == 0) return 0;
        uint32_t gl = 0;
        const uint64_t grid = plan_grid(t, tiles_of, nj, &gl);
        if (!grid_fits(grid)) return -FSTX_E_RANGE;
        fstx_internal::Range range("fstx gather_kernel: %u jobs, %u sources, %llu tiles%s%s%s", nj, ns, (unsigned long long)tiles,
                                   multi ? ", joins" : "", pitched ? ", pitched" : "", short_segs ? ", short segments" : "");
        // the leanest variant that serves every job of the launch
        const dim3 g((uint32_t)grid), w(64);
#define FSTX_GATHER(M, P)                                                                       \
    do {                                                                                        \
        if (short_segs) hipLaunchKernelGGL((gather_kernel<M, P, true>), g, w, 0, stream, gl, t); \
        else hipLaunchKernelGGL((gather_kernel<M, P, false>), g, w, 0, stream, gl, t);           \
    } while (0)
        if (multi && pitched) FSTX_GATHER(true, true);
        else if (multi) FSTX_GATHER(true, false);
        else if (pitched) FSTX_GATHER(false, true);
        else FSTX_GATHER(false, false);
#undef FSTX_GATHER
        nj = ns = 0;
        tiles = 0;
        multi = pitched = short_segs = false;
        return fstx_internal::check_launch("gather_kernel");
    }

    // whether the kernel takes this shape (every segment at least 16 bytes, rows that fit 32-bit positions)
    static bool takes(uint64_t dst_pitch, uint64_t rows, const fstx_join_src *srcs, uint32_t n) {
        uint64_t row_bytes = 0, min_seg = ~0ull;
        uint32_t live = 0;
        for (uint32_t i = 0; i < n; ++i) {
            if (srcs[i].seg_bytes == 0) continue;
            row_bytes += srcs[i].seg_bytes;
            if (srcs[i].seg_bytes < min_seg) min_seg = srcs[i].seg_bytes;
            if (rows > 1 && srcs[i].src_pitch >> 56) return false;
            ++live;
        }
        if (live == 0 || live > kGatherMore) return false;
        return fstx_gather::shape_ok(dst_pitch ? dst_pitch : row_bytes, row_bytes, min_seg);
    }

    // rows x (segments of the n sources side by side) into dst, rows dst_pitch apart (0: dense)
    int add(void *dst, uint64_t dst_pitch, uint64_t rows, const fstx_join_src *srcs, uint32_t n) {
        fstx_join_src live[kGatherMore];
        uint32_t m = 0;
        uint64_t row_bytes = 0, equal = 0, min_seg = ~0ull;
        for (uint32_t i = 0; i < n; ++i) {
            if (srcs[i].seg_bytes == 0) continue;
            if (m == 0) equal = srcs[i].seg_bytes;
            if (srcs[i].seg_bytes != equal) equal = 0;
            if (srcs[i].seg_bytes < min_seg) min_seg = srcs[i].seg_bytes;
            live[m++] = srcs[i];
            row_bytes += srcs[i].seg_bytes;
        }
        if (dst_pitch == 0) dst_pitch = row_bytes;
        // rows per job: 32-bit positions, and no more tiles than one job may take
        uint64_t per_job = fstx_gather::rows_per_job(dst_pitch, row_bytes);
        const uint64_t by_tiles = lim.job * fstx_gather::kTile / dst_pitch;
        if (by_tiles < per_job) per_job = by_tiles;
        if (per_job == 0) return -FSTX_E_RANGE; // one row is more than a job holds
        for (uint64_t row = 0; row < rows; row += per_job) {
            const uint64_t part = rows - row < per_job ? rows - row : per_job;
            auto source = [&](uint32_t i, uint64_t col) {
                return fstx_gather::Src{static_cast<const char *>(live[i].src) + row * live[i].src_pitch, live[i].src_pitch,
                                        (uint32_t)live[i].seg_bytes, (uint32_t)col, 0};
            };
            fstx_gather::Job job = fstx_gather::make_job(static_cast<char *>(dst) + row * dst_pitch, dst_pitch, row_bytes,
                                                         part, source(0, 0), 0, m, m > 1 ? equal : 0, min_seg);
            const uint64_t need = pad_to_dies(fstx_gather::tiles_of(job));
            if (nj == kGatherJobs || (m > 1 && ns + m > kGatherMore) || tiles + need > lim.launch) {
                int rc = flush();
                if (rc < 0) return rc;
            }
            job.more0 = (uint16_t)ns;
            uint64_t col = 0;
            for (uint32_t i = 0; m > 1 && i < m; ++i) { // one source travels in the job itself
                t.more[ns++] = source(i, col);
                col += live[i].seg_bytes;
            }
            t.job[nj] = job;
            tiles_of[nj] = need;
            tiles += need;
            ++nj;
            multi |= m > 1;
            pitched |= dst_pitch != row_bytes;
            short_segs |= min_seg < kShortSeg;
        }
        return 0;
    }
};

} // namespace

extern "C" int fstx_realign_copy_batch(const fstx_copy_desc *descs, uint32_t n, void *stream) {
    if (n == 0) return 0;
    if (!descs) return -FSTX_E_INVAL;
    if (n > FSTX_BATCH_MAX) return -FSTX_E_TOO_MANY;
    JobTable<RealignJob> t;
    uint64_t blocks_of[FSTX_BATCH_MAX];
    uint64_t sum = 0;
    uint32_t k = 0;
    auto flush = [&]() -> int {
        if (k == 0) return 0;
        uint32_t gl = 0;
        const uint64_t blocks = plan_grid(t, blocks_of, k, &gl);
        if (!grid_fits(blocks)) return -FSTX_E_RANGE;
        fstx_internal::Range range("fstx realign_kernel: %u jobs, %llu workgroups", k, (unsigned long long)blocks);
        hipLaunchKernelGGL(realign_kernel, dim3((uint32_t)blocks), dim3(kBlock), 0,
                           static_cast<hipStream_t>(stream), gl, t);
        k = 0;
        sum = 0;
        return fstx_internal::check_launch("realign_kernel");
    };
    // a span larger than one job may be is cut into pieces (any multiple of 16 bytes keeps
    // the relative alignment of source and destination)
    const Limits lim = limits();
    const uint64_t piece = lim.job * (uint64_t)kBlock * kVecBytes;
    for (uint32_t i = 0; i < n; ++i) {
        const fstx_copy_desc &d = descs[i];
        if (d.nbytes == 0) continue;
        if (!d.dst || !d.src) return -FSTX_E_INVAL;
        const char *s = static_cast<const char *>(d.src);
        char *o = static_cast<char *>(d.dst);
        if ((s < o + d.nbytes) && (o < s + d.nbytes)) return -FSTX_E_INVAL; // overlap
        for (uint64_t done = 0; done < d.nbytes; done += piece) {
            const uint64_t len = d.nbytes - done < piece ? d.nbytes - done : piece;
            const uint64_t need = pad_to_dies(blocks_for(len / kVecBytes));
            if (k == FSTX_BATCH_MAX || sum + need > lim.launch) {
                int rc = flush();
                if (rc < 0) return rc;
            }
            t.job[k] = RealignJob{o + done, s + done, len, 0};
            blocks_of[k] = need;
            sum += need;
            ++k;
        }
    }
    return flush();
}

extern "C" int fstx_realign_copy(void *dst, const void *src, uint64_t nbytes, void *stream) {
    fstx_copy_desc d{dst, src, nbytes};
    return fstx_realign_copy_batch(&d, 1, stream);
}

// Where a strided cut goes.  Contiguous spans never get here (they go to the realign copy).
//   gather_kernel   every shape with segments of at least 16 bytes: dense and pitched
//                   destinations, one source or several, any alignment of anything;
//   slice_kernel    dense cuts in which every address, segment and pitch is a multiple of 16
//                   bytes: nothing to realign, 3 % faster than the gather on such shapes;
//   slice2d_kernel  what is left: segments shorter than 16 bytes (and FSTX_GATHER_MODE=0, for
//                   measurements), moved in the largest unit of 1..16 bytes that divides everything.
extern "C" int fstx_slice_copy_batch(const fstx_slice_desc *descs, uint32_t n, void *stream) {
    if (n == 0) return 0;
    if (!descs) return -FSTX_E_INVAL;
    if (n > FSTX_BATCH_MAX) return -FSTX_E_TOO_MANY;
    JobTable<SliceJob> t;
    uint64_t blocks_of[FSTX_BATCH_MAX];
    uint64_t blocks = 0;
    uint32_t k = 0;
    auto flush = [&]() -> int {
        if (k == 0) return 0;
        uint32_t gl = 0;
        const uint64_t grid = plan_grid(t, blocks_of, k, &gl);
        if (!grid_fits(grid)) return -FSTX_E_RANGE;
        fstx_internal::Range range("fstx slice_kernel: %u jobs, %llu workgroups", k, (unsigned long long)grid);
        hipLaunchKernelGGL(slice_kernel, dim3((uint32_t)grid), dim3(kBlock), 0,
                           static_cast<hipStream_t>(stream), gl, t);
        k = 0;
        blocks = 0;
        return fstx_internal::check_launch("slice_kernel");
    };
    // the same for cuts that go through LDS (stage_kernel)
    JobTable<SliceJob> ts;
    uint64_t blocks_of_s[FSTX_BATCH_MAX];
    uint64_t blocks_s = 0, stage_bytes = 0;
    uint32_t ks = 0;
    auto flush_staged = [&]() -> int {
        if (ks == 0) return 0;
        uint32_t gl = 0;
        const uint64_t grid = plan_grid(ts, blocks_of_s, ks, &gl);
        if (!grid_fits(grid)) return -FSTX_E_RANGE;
        fstx_internal::Range range("fstx stage_kernel: %u jobs, %llu workgroups", ks, (unsigned long long)grid);
        // the less LDS a wavefront holds, the more of them a compute unit runs at once
        hipLaunchKernelGGL(stage_kernel, dim3((uint32_t)grid), dim3(kBlock), (uint32_t)stage_bytes, static_cast<hipStream_t>(stream), gl, ts);
        ks = 0;
        blocks_s = stage_bytes = 0;
        return fstx_internal::check_launch("stage_kernel");
    };
    fstx_copy_desc spans[FSTX_BATCH_MAX];
    uint32_t n_spans = 0;
    const Limits lim = limits();
    const int mode = fstx_internal::gather_mode();
    GatherBatch gather(stream);
    for (uint32_t i = 0; i < n; ++i) {
        const fstx_slice_desc &d = descs[i];
        if (d.outer == 0 || d.seg_bytes == 0) continue;
        if (!d.dst || !d.src) return -FSTX_E_INVAL;
        if (d.outer > 1 && (d.src_pitch < d.seg_bytes || d.src_pitch >> 56)) return -FSTX_E_INVAL;
        if (d.outer == 1 || d.src_pitch == d.seg_bytes) {
            // one contiguous span (a block of rows, or a cut that takes whole rows):
            // the realign copy moves it at full width whatever its alignment
            spans[n_spans++] = fstx_copy_desc{d.dst, d.src, d.outer * d.seg_bytes};
            continue;
        }
        uint64_t outer = d.outer, seg = d.seg_bytes, pitch = d.src_pitch;
        const uint32_t ul = common_unit_log2((uint64_t)(uintptr_t)d.dst | (uint64_t)(uintptr_t)d.src |
                                             seg | pitch | 16u);
        const fstx_join_src one{d.src, seg, pitch};
        if ((mode == 2 || (mode == 1 && ul < 4)) && GatherBatch::takes(0, outer, &one, 1)) {
            int rc = gather.add(d.dst, 0, outer, &one, 1);
            if (rc < 0) return rc;
            continue;
        }
        const uint64_t seg_units = seg >> ul;
        // Short segments in rows that lie close together, into an aligned destination: through LDS, when
        // the rows that feed one tile of the destination fit the staging buffer.
        constexpr uint64_t kTileBytes = (uint64_t)kBlock * kVecBytes;
        const uint64_t window_max = ((kTileBytes / seg + 2) * pitch + seg + kVecBytes - 1) / kVecBytes * kVecBytes;
        if (ul < 4 && seg < 64 && ((uintptr_t)d.dst & (kVecBytes - 1)) == 0 && window_max <= kStageBytes) {
            const uint64_t per_job = ((1ull << 32) - 2 * kTileBytes) / seg / 16 * 16; // destination bytes below 2^32; whole vectors per job
            for (uint64_t row = 0; row < outer; row += per_job) {
                const uint64_t rows = outer - row < per_job ? outer - row : per_job;
                const uint64_t need = pad_to_dies(blocks_for(rows * seg / kVecBytes + 1));
                if (ks == FSTX_BATCH_MAX || blocks_s + need > lim.launch) {
                    int rc = flush_staged();
                    if (rc < 0) return rc;
                }
                ts.job[ks] = SliceJob{static_cast<char *>(d.dst) + row * seg, static_cast<const char *>(d.src) + row * pitch,
                                      pitch | ((uint64_t)ul << 56), (uint32_t)seg_units, (uint32_t)(rows * seg_units)};
                blocks_of_s[ks] = need;
                blocks_s += need;
                if (window_max > stage_bytes) stage_bytes = window_max;
                ++ks;
            }
            continue;
        }
        // rows per job so that the unit index fits 32 bits
        uint64_t rows_per_job = lim.units() / seg_units;
        if (rows_per_job == 0) return -FSTX_E_RANGE; // a single segment of 3 Gi units or more
        for (uint64_t row = 0; row < outer; row += rows_per_job) {
            uint64_t rows = outer - row < rows_per_job ? outer - row : rows_per_job;
            uint64_t units = rows * seg_units;
            if (k == FSTX_BATCH_MAX || blocks + blocks_for(units) + 8 > lim.launch) { // (an upper bound when packed)
                int rc = flush();
                if (rc < 0) return rc;
            }
            // units under 16 bytes are packed into whole destination vectors when those are aligned
            char *job_dst = static_cast<char *>(d.dst) + row * seg;
            const bool packed = ul < 4 && ((uintptr_t)job_dst & (kVecBytes - 1)) == 0;
            const uint64_t items = packed ? (units + (16u >> ul) - 1) / (16u >> ul) : units;
            t.job[k] = SliceJob{job_dst, static_cast<const char *>(d.src) + row * pitch,
                                pitch | ((uint64_t)(ul | (packed ? kPackedUnits : 0u)) << 56), (uint32_t)seg_units, (uint32_t)units};
            blocks_of[k] = pad_to_dies(blocks_for(items));
            blocks += blocks_of[k];
            ++k;
        }
    }
    int rc = flush();
    if (rc < 0) return rc;
    if ((rc = flush_staged()) < 0) return rc;
    if ((rc = gather.flush()) < 0) return rc;
    return n_spans ? fstx_realign_copy_batch(spans, n_spans, stream) : 0;
}

extern "C" int fstx_slice_copy(void *dst, const void *src, uint64_t outer, uint64_t seg_bytes,
                               uint64_t src_pitch, void *stream) {
    fstx_slice_desc d{dst, src, outer, seg_bytes, src_pitch};
    return fstx_slice_copy_batch(&d, 1, stream);
}

extern "C" int fstx_slice_copy2d_batch(const fstx_slice2d_desc *descs, uint32_t n, void *stream) {
    if (n == 0) return 0;
    if (!descs) return -FSTX_E_INVAL;
    if (n > FSTX_BATCH_MAX) return -FSTX_E_TOO_MANY;
    JobTable<Slice2dJob> t;
    constexpr uint32_t kJobs = JobTable<Slice2dJob>::kJobs;
    uint64_t blocks_of[kJobs];
    uint64_t blocks = 0;
    uint32_t k = 0;
    auto flush = [&]() -> int {
        if (k == 0) return 0;
        uint32_t gl = 0;
        const uint64_t grid = plan_grid(t, blocks_of, k, &gl);
        if (!grid_fits(grid)) return -FSTX_E_RANGE;
        fstx_internal::Range range("fstx slice2d_kernel: %u jobs, %llu workgroups", k, (unsigned long long)grid);
        hipLaunchKernelGGL(slice2d_kernel, dim3((uint32_t)grid), dim3(kBlock), 0,
                           static_cast<hipStream_t>(stream), gl, t);
        k = 0;
        blocks = 0;
        return fstx_internal::check_launch("slice2d_kernel");
    };
    fstx_slice_desc dense[FSTX_BATCH_MAX];
    uint32_t n_dense = 0;
    const Limits lim = limits();
    const int mode = fstx_internal::gather_mode();
    GatherBatch gather(stream);
    for (uint32_t i = 0; i < n; ++i) {
        const fstx_slice2d_desc &d = descs[i];
        if (d.outer == 0 || d.seg_bytes == 0) continue;
        if (!d.dst || !d.src) return -FSTX_E_INVAL;
        if (d.outer > 1 && (d.src_pitch < d.seg_bytes || d.dst_pitch < d.seg_bytes)) return -FSTX_E_INVAL;
        if (d.outer == 1 || d.dst_pitch == d.seg_bytes) {
            // a dense destination: the plain slice extract (and its span form) serves it
            dense[n_dense++] = fstx_slice_desc{d.dst, d.src, d.outer, d.seg_bytes, d.src_pitch};
            continue;
        }
        const fstx_join_src one{d.src, d.seg_bytes, d.src_pitch};
        const uint32_t ul = common_unit_log2((uint64_t)(uintptr_t)d.dst | (uint64_t)(uintptr_t)d.src | d.seg_bytes |
                                             d.src_pitch | d.dst_pitch | 16u);
        if (mode != 0 && GatherBatch::takes(d.dst_pitch, d.outer, &one, 1)) {
            int rc = gather.add(d.dst, d.dst_pitch, d.outer, &one, 1);
            if (rc < 0) return rc;
            continue;
        }
        const uint64_t seg_units = d.seg_bytes >> ul;
        uint64_t rows_per_job = lim.units() / seg_units;
        if (rows_per_job == 0) return -FSTX_E_RANGE; // a single segment of 3 Gi units or more
        for (uint64_t row = 0; row < d.outer; row += rows_per_job) {
            const uint64_t rows = d.outer - row < rows_per_job ? d.outer - row : rows_per_job;
            const uint64_t units = rows * seg_units;
            if (k == kJobs || blocks + blocks_for(units) + 8 > lim.launch) {
                int rc = flush();
                if (rc < 0) return rc;
            }
            t.job[k] = Slice2dJob{static_cast<char *>(d.dst) + row * d.dst_pitch,
                                  static_cast<const char *>(d.src) + row * d.src_pitch,
                                  d.src_pitch, d.dst_pitch, (uint32_t)seg_units, (uint32_t)units, ul, 0, 0, 0};
            blocks_of[k] = pad_to_dies(blocks_for(units));
            blocks += blocks_of[k];
            ++k;
        }
    }
    int rc = flush();
    if (rc < 0) return rc;
    if ((rc = gather.flush()) < 0) return rc;
    return n_dense ? fstx_slice_copy_batch(dense, n_dense, stream) : 0;
}

namespace {

// one join into `gather`, or, when some block is narrower than the gather kernel takes, every
// block on its own into its columns of the joined rows (small-unit kernel)
int add_join(GatherBatch &gather, void *dst, uint64_t dst_pitch, uint64_t rows, const fstx_join_src *srcs, uint32_t n,
             void *stream) {
    if (n == 0 || rows == 0) return 0;
    if (!dst || !srcs) return -FSTX_E_INVAL;
    if (n > FSTX_JOIN_MAX) return -FSTX_E_TOO_MANY;
    uint64_t row_bytes = 0;
    for (uint32_t i = 0; i < n; ++i) {
        const fstx_join_src &s = srcs[i];
        if (s.seg_bytes == 0) continue;
        if (!s.src || (rows > 1 && s.src_pitch < s.seg_bytes) || s.seg_bytes >> 32) return -FSTX_E_INVAL;
        row_bytes += s.seg_bytes;
    }
    if (row_bytes == 0) return 0;
    if (dst_pitch == 0) dst_pitch = row_bytes;
    if (dst_pitch < row_bytes) return -FSTX_E_INVAL;
    if (fstx_internal::gather_mode() != 0 && GatherBatch::takes(dst_pitch, rows, srcs, n))
        return gather.add(dst, dst_pitch, rows, srcs, n);
    fstx_slice2d_desc each[FSTX_JOIN_MAX];
    uint32_t m = 0;
    uint64_t col = 0;
    for (uint32_t i = 0; i < n; ++i) {
        const fstx_join_src &s = srcs[i];
        if (s.seg_bytes == 0) continue;
        each[m++] = fstx_slice2d_desc{static_cast<char *>(dst) + col, s.src, rows, s.seg_bytes, s.src_pitch, dst_pitch};
        col += s.seg_bytes;
    }
    return fstx_slice_copy2d_batch(each, m, stream);
}

} // namespace

extern "C" int fstx_join_copy(void *dst, uint64_t dst_pitch, uint64_t rows, const fstx_join_src *srcs, uint32_t n,
                              void *stream) {
    GatherBatch gather(stream);
    int rc = add_join(gather, dst, dst_pitch, rows, srcs, n, stream);
    return rc < 0 ? rc : gather.flush();
}

extern "C" int fstx_join_copy_batch(const fstx_join_desc *joins, uint32_t n, void *stream) {
    if (n == 0) return 0;
    if (!joins) return -FSTX_E_INVAL;
    GatherBatch gather(stream);
    for (uint32_t i = 0; i < n; ++i) {
        int rc = add_join(gather, joins[i].dst, joins[i].dst_pitch, joins[i].rows, joins[i].srcs, joins[i].n_srcs, stream);
        if (rc < 0) return rc;
    }
    return gather.flush();
}

extern "C" int fstx_convert_batch(const fstx_convert_desc *descs, uint32_t n, void *stream) {
    if (n == 0) return 0;
    if (!descs) return -FSTX_E_INVAL;
    if (n > FSTX_BATCH_MAX) return -FSTX_E_TOO_MANY;
    static const uint32_t size_of[6] = {8, 4, 2, 2, 1, 1};
    const Limits lim = limits();
    JobTable<ConvertJob> t;
    uint64_t blocks_of[FSTX_BATCH_MAX];
    uint64_t sum = 0;
    uint32_t k = 0;
    auto flush = [&]() -> int {
        if (k == 0) return 0;
        uint32_t gl = 0;
        const uint64_t grid = plan_grid(t, blocks_of, k, &gl);
        if (!grid_fits(grid)) return -FSTX_E_RANGE;
        fstx_internal::Range range("fstx convert_kernel: %u jobs, %llu workgroups", k, (unsigned long long)grid);
        hipLaunchKernelGGL(convert_kernel, dim3((uint32_t)grid), dim3(kBlock), 0, static_cast<hipStream_t>(stream),
                           gl, t);
        k = 0;
        sum = 0;
        return fstx_internal::check_launch("convert_kernel");
    };
    for (uint32_t i = 0; i < n; ++i) {
        const fstx_convert_desc &d = descs[i];
        if (d.n_elems == 0) continue;
        if (!d.dst || !d.src || d.src_type > FSTX_F8_E5M2 || d.dst_type > FSTX_F8_E5M2) return -FSTX_E_INVAL;
        const uint32_t ss = size_of[d.src_type], ds = size_of[d.dst_type];
        // only towards a type that is not wider, never from fp8, never onto the same type
        if (ds > ss || d.src_type >= FSTX_F8_E4M3 || d.src_type == d.dst_type || d.dst_type == FSTX_F64) return -FSTX_E_INVAL;
        if (((uintptr_t)d.src % ss) || ((uintptr_t)d.dst % ds)) return -FSTX_E_INVAL;
        const char *sb = static_cast<const char *>(d.src);
        char *db = static_cast<char *>(d.dst);
        if (sb < db + d.n_elems * ds && db < sb + d.n_elems * ss) return -FSTX_E_INVAL; // overlap
        const uint64_t per_block = (uint64_t)kBlock * (16 / ss);
        const uint64_t piece = lim.job * per_block; // elements one job may take
        for (uint64_t done = 0; done < d.n_elems; done += piece) {
            const uint64_t len = d.n_elems - done < piece ? d.n_elems - done : piece;
            const uint64_t need = pad_to_dies((len + per_block - 1) / per_block);
            if (k == FSTX_BATCH_MAX || sum + need > lim.launch) {
                int rc = flush();
                if (rc < 0) return rc;
            }
            t.job[k] = ConvertJob{db + done * ds, sb + done * ss, len, d.src_type, d.dst_type};
            blocks_of[k] = need;
            sum += need;
            ++k;
        }
    }
    return flush();
}
