// SPDX-License-Identifier: Apache-2.0
//
// HBM data-movement kernels of the load path, written for gfx950 (CDNA4):
// 64-wide wavefronts, 16-byte global loads/stores per lane, no MFMA (there is
// no arithmetic here; the bound is HBM bandwidth).
//
//   realign copy  : dst[0:n) = src[0:n) for any byte alignment of src and dst.
//                   Stands in for gds_device_buffer::memmove of the reference
//                   (cpp/ext.cpp:606-645: two cudaMemcpy through a temporary).
//   slice extract : dense copy of `outer` segments read at a fixed pitch.
//                   Stands in for t[slices].contiguous() per rank in
//                   LazyTensorFactory.shuffle (tensor_factory.py:168-175).
//
// Both kernels take a table of up to FSTX_BATCH_MAX jobs as a by-value kernel
// argument, so that the many small tensors of a checkpoint file cost one
// launch.  A workgroup of 256 lanes owns 256 consecutive 16-byte vectors of
// one job's destination; consecutive lanes touch consecutive vectors, so each
// wavefront reads and writes 1 KiB contiguous spans.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fstx.h"
#include "fstx_internal.h"

namespace {

typedef unsigned int v4u __attribute__((ext_vector_type(4)));

constexpr int kBlock = 256;        // lanes per workgroup (4 wavefronts)
constexpr int kVecBytes = 16;      // bytes moved per lane per step

// ---------------------------------------------------------------- job tables

struct RealignJob {
    char *dst;
    const char *src;
    uint64_t nbytes;
};

struct SliceJob {
    char *dst;
    const char *src;
    uint64_t src_pitch;   // bytes between segment starts in src
    uint32_t seg_units;   // units per segment
    uint32_t total_units; // outer * seg_units  (< 2^32 by construction)
    uint32_t unit_log2;   // log2 of the unit size in bytes: 0..4
    uint32_t pad;
};

template <typename Job>
struct JobTable {
    Job job[FSTX_BATCH_MAX];
    uint32_t first_block[FSTX_BATCH_MAX + 1]; // prefix sum of blocks per job
    uint32_t n;
};

// index of the job that owns workgroup `b` (first_block is ascending)
template <typename Job>
__device__ __forceinline__ uint32_t find_job(const JobTable<Job> &t, uint32_t b) {
    uint32_t lo = 0, hi = t.n; // invariant: first_block[lo] <= b < first_block[hi]
    while (hi - lo > 1) {
        uint32_t mid = (lo + hi) >> 1;
        if (t.first_block[mid] <= b) lo = mid; else hi = mid;
    }
    return lo;
}

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

template <int Q>
__device__ __forceinline__ void shifted_vec(v4u *dstv, const v4u *srcv, uint64_t j, uint32_t r) {
    v4u lo = __builtin_nontemporal_load(srcv + j);
    v4u hi = __builtin_nontemporal_load(srcv + j + 1);
    __builtin_nontemporal_store(funnel<Q>(lo, hi, r), dstv + j);
}

__global__ __launch_bounds__(kBlock) void realign_kernel(const JobTable<RealignJob> t) {
    const uint32_t b = blockIdx.x;
    const uint32_t ji = t.n == 1 ? 0u : find_job(t, b);
    const RealignJob job = t.job[ji];
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
            job.dst[at] = job.src[at];
        }
    }

    const uint64_t j = (uint64_t)lb * kBlock + threadIdx.x;
    if (j >= nvec) return;

    v4u *dstv = reinterpret_cast<v4u *>(job.dst + head);
    const char *s = job.src + head;
    const uint32_t m = (uint32_t)(uintptr_t)s & (kVecBytes - 1);
    if (m == 0) {
        const v4u *srcv = reinterpret_cast<const v4u *>(s);
        __builtin_nontemporal_store(__builtin_nontemporal_load(srcv + j), dstv + j);
        return;
    }
    // Source vectors are loaded at their natural 16-byte alignment; lane j needs
    // aligned vectors j and j+1 and shifts the pair right by m bytes.  Vector
    // j+1 always overlaps a source byte of this job, so it never leaves the
    // 16-byte granule that holds the last valid byte.
    const v4u *srcv = reinterpret_cast<const v4u *>(s - m);
    const uint32_t r = m & 3;
    switch (m >> 2) { // uniform across the workgroup
    case 0: shifted_vec<0>(dstv, srcv, j, r); break;
    case 1: shifted_vec<1>(dstv, srcv, j, r); break;
    case 2: shifted_vec<2>(dstv, srcv, j, r); break;
    default: shifted_vec<3>(dstv, srcv, j, r); break;
    }
}

// ------------------------------------------------------------ slice extract

template <typename Unit>
__device__ __forceinline__ void slice_units(const SliceJob &job, uint32_t u) {
    const uint32_t row = u / job.seg_units;
    const uint32_t col = u - row * job.seg_units;
    const Unit *src = reinterpret_cast<const Unit *>(job.src + (uint64_t)row * job.src_pitch) + col;
    Unit *dst = reinterpret_cast<Unit *>(job.dst) + u;
    __builtin_nontemporal_store(__builtin_nontemporal_load(src), dst);
}

__global__ __launch_bounds__(kBlock) void slice_kernel(const JobTable<SliceJob> t) {
    const uint32_t b = blockIdx.x;
    const uint32_t ji = t.n == 1 ? 0u : find_job(t, b);
    const SliceJob job = t.job[ji];
    const uint32_t lb = b - t.first_block[ji];
    const uint64_t u64 = (uint64_t)lb * kBlock + threadIdx.x;
    if (u64 >= job.total_units) return;
    const uint32_t u = (uint32_t)u64;
    switch (job.unit_log2) { // uniform across the workgroup
    case 4: slice_units<v4u>(job, u); break;
    case 3: slice_units<uint64_t>(job, u); break;
    case 2: slice_units<uint32_t>(job, u); break;
    case 1: slice_units<uint16_t>(job, u); break;
    default: slice_units<uint8_t>(job, u); break;
    }
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

constexpr uint64_t kMaxUnitsPerJob = 0xffffff00ull; // keeps lb * 256 + lane in 32 bits
constexpr uint64_t kMaxBlocksPerLaunch = 0x7fffff00ull;

} // namespace

extern "C" int fstx_realign_copy_batch(const fstx_copy_desc *descs, uint32_t n, void *stream) {
    if (n == 0) return 0;
    if (!descs) return -FSTX_E_INVAL;
    if (n > FSTX_BATCH_MAX) return -FSTX_E_TOO_MANY;
    JobTable<RealignJob> t;
    uint64_t blocks = 0;
    uint32_t k = 0;
    for (uint32_t i = 0; i < n; ++i) {
        const fstx_copy_desc &d = descs[i];
        if (d.nbytes == 0) continue;
        if (!d.dst || !d.src) return -FSTX_E_INVAL;
        const char *s = static_cast<const char *>(d.src);
        char *o = static_cast<char *>(d.dst);
        if ((s < o + d.nbytes) && (o < s + d.nbytes)) return -FSTX_E_INVAL; // overlap
        t.job[k] = RealignJob{o, s, d.nbytes};
        t.first_block[k] = (uint32_t)blocks;
        blocks += blocks_for(d.nbytes / kVecBytes);
        if (blocks > kMaxBlocksPerLaunch) return -FSTX_E_RANGE;
        ++k;
    }
    if (k == 0) return 0;
    t.first_block[k] = (uint32_t)blocks;
    t.n = k;
    hipLaunchKernelGGL(realign_kernel, dim3((uint32_t)blocks), dim3(kBlock), 0,
                       static_cast<hipStream_t>(stream), t);
    return fstx_internal::check_launch("realign_kernel");
}

extern "C" int fstx_realign_copy(void *dst, const void *src, uint64_t nbytes, void *stream) {
    // one launch covers < 2^31 workgroups of 4 KiB; split beyond that
    const uint64_t piece = (kMaxBlocksPerLaunch - 1) * (uint64_t)kBlock * kVecBytes;
    uint64_t done = 0;
    do {
        uint64_t len = nbytes - done < piece ? nbytes - done : piece;
        fstx_copy_desc d{static_cast<char *>(dst) + done, static_cast<const char *>(src) + done, len};
        int rc = fstx_realign_copy_batch(&d, 1, stream);
        if (rc < 0) return rc;
        done += len;
    } while (done < nbytes);
    return 0;
}

extern "C" int fstx_slice_copy_batch(const fstx_slice_desc *descs, uint32_t n, void *stream) {
    if (n == 0) return 0;
    if (!descs) return -FSTX_E_INVAL;
    if (n > FSTX_BATCH_MAX) return -FSTX_E_TOO_MANY;
    JobTable<SliceJob> t;
    uint64_t blocks = 0;
    uint32_t k = 0;
    auto flush = [&]() -> int {
        if (k == 0) return 0;
        t.first_block[k] = (uint32_t)blocks;
        t.n = k;
        hipLaunchKernelGGL(slice_kernel, dim3((uint32_t)blocks), dim3(kBlock), 0,
                           static_cast<hipStream_t>(stream), t);
        k = 0;
        blocks = 0;
        return fstx_internal::check_launch("slice_kernel");
    };
    for (uint32_t i = 0; i < n; ++i) {
        const fstx_slice_desc &d = descs[i];
        if (d.outer == 0 || d.seg_bytes == 0) continue;
        if (!d.dst || !d.src) return -FSTX_E_INVAL;
        if (d.outer > 1 && d.src_pitch < d.seg_bytes) return -FSTX_E_INVAL;
        // a lone segment is one contiguous span; treat it as one long row so
        // that its length need not be a multiple of the unit of the pitch
        uint64_t outer = d.outer, seg = d.seg_bytes, pitch = d.outer > 1 ? d.src_pitch : 0;
        const uint32_t ul = common_unit_log2((uint64_t)(uintptr_t)d.dst | (uint64_t)(uintptr_t)d.src |
                                             seg | pitch | 16u);
        const uint64_t seg_units = seg >> ul;
        // rows per job so that units fit 32 bits; a single huge row is cut along itself
        uint64_t rows_per_job = kMaxUnitsPerJob / seg_units;
        if (rows_per_job == 0) {
            // only reachable with outer == 1 spans >= 4 Gi units; cut into spans
            if (outer != 1) return -FSTX_E_RANGE;
            uint64_t done_units = 0;
            while (done_units < seg_units) {
                uint64_t take = seg_units - done_units < kMaxUnitsPerJob ? seg_units - done_units
                                                                        : kMaxUnitsPerJob;
                if (k == FSTX_BATCH_MAX || blocks + blocks_for(take) > kMaxBlocksPerLaunch) {
                    int rc = flush();
                    if (rc < 0) return rc;
                }
                t.job[k] = SliceJob{static_cast<char *>(d.dst) + (done_units << ul),
                                    static_cast<const char *>(d.src) + (done_units << ul),
                                    0, (uint32_t)take, (uint32_t)take, ul, 0};
                t.first_block[k] = (uint32_t)blocks;
                blocks += blocks_for(take);
                ++k;
                done_units += take;
            }
            continue;
        }
        for (uint64_t row = 0; row < outer; row += rows_per_job) {
            uint64_t rows = outer - row < rows_per_job ? outer - row : rows_per_job;
            uint64_t units = rows * seg_units;
            if (k == FSTX_BATCH_MAX || blocks + blocks_for(units) > kMaxBlocksPerLaunch) {
                int rc = flush();
                if (rc < 0) return rc;
            }
            t.job[k] = SliceJob{static_cast<char *>(d.dst) + row * seg,
                                static_cast<const char *>(d.src) + row * pitch,
                                pitch, (uint32_t)seg_units, (uint32_t)units, ul, 0};
            t.first_block[k] = (uint32_t)blocks;
            blocks += blocks_for(units);
            ++k;
        }
    }
    return flush();
}

extern "C" int fstx_slice_copy(void *dst, const void *src, uint64_t outer, uint64_t seg_bytes,
                               uint64_t src_pitch, void *stream) {
    fstx_slice_desc d{dst, src, outer, seg_bytes, src_pitch};
    return fstx_slice_copy_batch(&d, 1, stream);
}
