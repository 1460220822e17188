/* SPDX-License-Identifier: Apache-2.0
 *
 * fstx: C ABI of the MI355X safetensors load path.
 *
 * One shared library (libfstx.so, HIP, gfx950) holds
 *   - the file -> pinned ring -> HBM copy pipeline, and
 *   - the kernels that post-process tensors in HBM (realign copy, slice
 *     extract into dense, pitched and joined destinations, down-cast).
 * Every entry point takes plain pointers and sizes; there are no C++ or torch
 * types in the signatures, so the library binds from ctypes, cgo, JNI or any
 * other FFI.  Each declaration names the interface of the reference
 * (foundation-model-stack/fastsafetensors 0.3.2, paths relative to its root)
 * that it stands in for.
 *
 * Conventions
 *   - int / int64_t returns: >= 0 success, < 0 is -(fstx_status) or -errno
 *     (errno values are < FSTX_E_BASE in magnitude); never aborts, never
 *     prints unless fstx_set_debug_log(1).
 *   - `stream` is a hipStream_t passed as void*; NULL is the device's null
 *     stream.  Kernel entry points only enqueue work; they do not synchronize.
 *   - Device pointers must belong to the device that is current on the
 *     calling thread (kernels) or to the context's device (reads).
 *   - A strided source (`outer` segments `src_pitch` apart) must be readable from the
 *     first byte of its first segment to the last byte of its last one, bytes between the
 *     segments included: it is a block of a tensor.  The kernels never touch a byte before
 *     or behind that range, and never write a destination byte that is not a segment's.
 */
#ifndef FSTX_H
#define FSTX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FSTX_ABI_VERSION 4

/* status codes beyond errno */
#define FSTX_E_BASE 10000
enum fstx_status {
    FSTX_OK = 0,
    FSTX_E_INVAL = FSTX_E_BASE + 1,     /* bad argument                                 */
    FSTX_E_HIP = FSTX_E_BASE + 2,       /* a HIP runtime call failed                    */
    FSTX_E_RANGE = FSTX_E_BASE + 3,     /* destination range exceeds the device buffer  */
    FSTX_E_SHORT_READ = FSTX_E_BASE + 4,/* file ended before the requested range        */
    FSTX_E_NO_REQ = FSTX_E_BASE + 5,    /* unknown or already-waited request id         */
    FSTX_E_CLOSED = FSTX_E_BASE + 6,    /* context is shutting down                     */
    FSTX_E_NO_DEVICE = FSTX_E_BASE + 7, /* no HIP device visible                        */
    FSTX_E_TOO_MANY = FSTX_E_BASE + 8   /* batch larger than FSTX_BATCH_MAX             */
};

/* read modes of fstx_file_open / fstx_submit_read */
enum fstx_read_mode {
    FSTX_READ_AUTO = 0,     /* per block: buffered when the block is in the page cache, else O_DIRECT */
    FSTX_READ_BUFFERED = 1, /* page-cache pread straight into the pinned ring                         */
    FSTX_READ_DIRECT = 2    /* O_DIRECT pread into an aligned staging block, then into the ring       */
};

typedef struct fstx_ctx fstx_ctx;

typedef struct fstx_config {
    uint32_t struct_size;    /* = sizeof(fstx_config); lets the struct grow                      */
    int32_t device_id;       /* HIP device ordinal                                               */
    int32_t numa_node;       /* node to pin I/O threads and the ring to; < 0 = do not pin        */
    uint32_t n_threads;      /* I/O worker threads (0 = default 8)                               */
    uint32_t n_streams;      /* HIP copy streams shared by the workers (0 = default 4)           */
    uint64_t block_bytes;    /* bytes per read block = per ring slot, multiple of 4096 (0 = 4 MiB)*/
    uint32_t slots_per_thread; /* ring slots each worker cycles through (0 = default 2)          */
    uint32_t max_direct_reads; /* O_DIRECT preads allowed in flight at once; 0 = from the block
                                  device under the first file opened for O_DIRECT: 1 for a
                                  paravirtual, rotating or unknown disk, else 2 and steered while
                                  reading (as with FSTX_ADAPTIVE_DEPTH)                          */
    uint64_t direct_read_bytes; /* bytes one O_DIRECT pread covers: a run of consecutive blocks,
                                   multiple of block_bytes; 0 = from that device: one request
                                   queue's worth (nr_requests x max_sectors_kb, 64 MiB .. 1 GiB)
                                   with one read in flight, a quarter of it with several, and
                                   never more staging memory than 1/16 of MemAvailable           */
    uint32_t flags;          /* FSTX_ADAPTIVE_DEPTH | FSTX_PROBE_* | FSTX_NO_PRETOUCH | FSTX_CREATE_ASYNC */
    uint32_t direct_ramp_kb; /* KiB of the first O_DIRECT pread after the queue was empty; the next
                                ones are 4x, 16x .. as large up to direct_read_bytes, and towards the
                                end of the queued bytes they halve down to this size again, so that
                                the copy of one read overlaps the next read from the start and only a
                                small last read is copied with the storage idle (0 = 64 MiB; a value
                                >= direct_read_bytes / 1024 keeps every read at full size)        */
} fstx_config;

/* fstx_config.flags: steer max_direct_reads while reading (start value = max_direct_reads) */
#define FSTX_ADAPTIVE_DEPTH 1u
/* Measurement contexts: the same threads, queue, request sizes and ring, with one stage left
 * out, so that the rate of the other stage alone can be put next to a load's.  The bytes
 * that arrive in device memory are unspecified with either flag.
 *   NO_COPY  reads run (O_DIRECT runs into staging, page-cache reads into the ring), nothing
 *            is moved to the ring by memcpy or to the device: what the storage delivers to
 *            this engine's request pattern;
 *   NO_READ  no pread: every block's ring slot is sent to the device as it is: what the
 *            ring -> HBM copies deliver with this engine's slots, streams and threads. */
#define FSTX_PROBE_NO_COPY 2u
#define FSTX_PROBE_NO_READ 4u
/* The workers do not map the pages of their ring slots ahead of the first request (they do by
 * default: pinned memory is mapped at its first touch, which is slow); for measurements. */
#define FSTX_NO_PRETOUCH 8u
/* fstx_ctx_create / fstx_ctx_acquire return as soon as the configuration has been checked; a
 * thread of the library builds ring, streams and workers meanwhile (about a millisecond, during
 * which the caller parses headers, opens files and queues reads: none of that waits).  The calls
 * that need the outcome wait for it: fstx_wait_read, fstx_get_metrics, fstx_ctx_order_after on a
 * busy stream, fstx_ctx_destroy.  A build that fails is reported by fstx_wait_read for whatever
 * was queued, and by every fstx_submit_read after it. */
#define FSTX_CREATE_ASYNC 16u

/* fstx_metrics.storage_flags */
#define FSTX_STORAGE_KNOWN 1u      /* the block layer named queue depth and request size          */
#define FSTX_STORAGE_ROTATIONAL 2u
#define FSTX_STORAGE_VIRTIO 4u

typedef struct fstx_metrics {
    uint64_t struct_size;         /* in: sizeof(fstx_metrics) of the caller; out: bytes filled in.
                                     The struct only ever grows at its end.                       */
    uint64_t bounce_buffer_bytes; /* pinned ring bytes currently allocated by this context       */
    uint64_t bytes_read;          /* file bytes delivered into the ring                          */
    uint64_t bytes_copied;        /* bytes enqueued host -> device                               */
    uint64_t blocks_buffered;     /* blocks served by page-cache pread                           */
    uint64_t blocks_direct;       /* blocks served by O_DIRECT                                   */
    uint64_t read_ns;             /* summed over workers: time inside pread                      */
    uint64_t stage_ns;            /* summed over workers: staging memcpy after O_DIRECT          */
    uint64_t slot_wait_ns;        /* summed over workers: waiting for a ring slot's last copy    */
    uint64_t direct_fallbacks;    /* blocks that asked for O_DIRECT but were read buffered       */
    uint64_t direct_depth;        /* O_DIRECT preads allowed in flight (steered: the depth last
                                     found good, not a step that is still being tried)           */
    uint64_t direct_reads;        /* O_DIRECT preads issued (each covers a run of blocks)        */
    uint64_t create_ns;           /* from the call of fstx_ctx_create until threads, ring, streams
                                     and events existed                                           */
    /* where the I/O side runs (fstx_config.numa_node >= 0) */
    int64_t numa_node;            /* the node asked for, -1 = none                               */
    uint64_t workers_on_node;     /* workers whose CPU affinity, read back with sched_getaffinity
                                     after binding, lies inside the node's cpulist               */
    int64_t ring_node;            /* node that holds the ring's first page, -1 where the kernel
                                     does not say (it does not for device-mapped pinned memory)  */
    uint64_t bind_errors;         /* threads (workers + the one that allocates the ring) whose
                                     affinity or memory policy could not be set                  */
    int64_t first_bind_error;     /* the first such failure as -errno, 0 = none                  */
    uint64_t pretouched_bytes;    /* ring bytes the workers mapped before the first request      */
    /* the O_DIRECT reads as settled (0 until a file has been opened for O_DIRECT) */
    uint64_t direct_read_bytes;   /* bytes one read covers                                       */
    uint64_t direct_steered;      /* 1 = direct_depth is steered while reading                   */
    uint64_t staging_buffers_max; /* staging buffers of direct_read_bytes the context may hold   */
    uint64_t storage_nr_requests; /* /sys/dev/block/<dev>/queue/nr_requests of that file's device */
    uint64_t storage_max_sectors_kb;
    uint64_t storage_flags;       /* FSTX_STORAGE_*                                              */
    uint64_t ring_reused;         /* 1 = the ring is the one the last destroyed context left parked */
} fstx_metrics;

/* ---- library-wide helpers ------------------------------------------------ */

/* ABI version of the loaded library (FSTX_ABI_VERSION).  Call it first and compare it with the
 * FSTX_ABI_VERSION the caller was built against: structs passed by pointer carry their size
 * (fstx_config, fstx_metrics), everything else is only guaranteed within one version. */
int fstx_abi_version(void);

/* Number of visible HIP devices, or -FSTX_E_NO_DEVICE.
 * Stands in for load_library_functions + is_hip_found (cpp/ext.cpp:278-410). */
int fstx_device_count(void);

/* Required alignment of O_DIRECT windows: 4096.  get_alignment_size (cpp/ext.cpp:412-415). */
int fstx_get_alignment_size(void);

/* "dddd:bb:dd.f" PCI id of a device into out[len].  get_device_pci_bus (cpp/ext.cpp:508-523). */
int fstx_get_device_pci_bus(int device_id, char *out, int len);

/* Restrict the calling thread (and threads it creates later) to the CPUs of a
 * NUMA node and prefer its memory.  0, or what failed as -errno (-ENODEV: the node has no
 * CPUs or does not exist).  set_numa_node (cpp/ext.cpp:525-533). */
int fstx_set_numa_node(int numa_node);

/* The CPUs of a NUMA node as the library reads them from sysfs
 * (<root>/devices/system/node/node<N>/cpulist, root = /sys or $FSTX_SYSFS_ROOT): up to
 * `capacity` of them into cpus[], ascending; returns how many the node has, or -ENODEV.
 * The I/O workers of a context with numa_node = N are bound to exactly these.  Stands in
 * for libnuma's node-to-CPU lookup behind numa_run_on_node (cpp/ext.cpp:525-533). */
int fstx_node_cpus(int numa_node, int *cpus, int capacity);

/* Toggle debug lines on stderr.  set_debug_log (cpp/ext.cpp:417-420). */
void fstx_set_debug_log(int enabled);

/* Pinned ring bytes of all contexts alive in the process (a parked ring belongs to none).
 * get_cpp_metrics().bounce_buffer_bytes (cpp/ext.cpp:952-954). */
uint64_t fstx_bounce_buffer_bytes(void);

/* The pinned ring of the context that was destroyed last stays allocated ("parked") for the next
 * context of the same device, node and ring size in this process, which thereby skips the
 * allocation and, above all, the page-by-page mapping of fresh pinned memory at its first touch
 * (the reference allocates its bounce buffer per reader, nogds.py:107-116 / ext.cpp:648-672, and
 * pays that every time).  At most one ring is parked; it is not counted by
 * fstx_bounce_buffer_bytes.  fstx_cached_ring_bytes tells its size, fstx_trim_cache frees it
 * (returns the bytes freed); a context created with FSTX_RING_CACHE=0 in the environment neither
 * takes over a parked ring nor leaves its own behind.
 * No counterpart in the reference. */
uint64_t fstx_cached_ring_bytes(void);
uint64_t fstx_trim_cache(void);

/* Text for a negative return value (errno or fstx_status); never NULL. */
const char *fstx_strerror(int64_t code);

/* 4096-aligned host allocation.  cpu_malloc / cpu_free (cpp/ext.cpp:542-557). */
void *fstx_host_alloc(uint64_t length);
void fstx_host_free(void *p);

/* ---- file -> HBM pipeline -------------------------------------------------- */

/* Create the reader: worker threads, copy streams and the pinned ring
 * (allocated once, reused by every file).  Replaces the nogds_file_reader
 * constructor (cpp/ext.hpp:176-180) and its lazy cudaHostAlloc (cpp/ext.cpp:735-751). */
int fstx_ctx_create(const fstx_config *cfg, fstx_ctx **out);

/* Drain outstanding work, join the workers, free ring, streams and events.
 * ~nogds_file_reader (cpp/ext.cpp:778-806). */
int fstx_ctx_destroy(fstx_ctx *ctx);

/* A context shared by everyone in the process who asks for the same configuration: the
 * first call creates it, later calls with an equal fstx_config (after defaults) get the same
 * context and raise its use count; fstx_ctx_release drops the count and destroys the context
 * with the last user, so the pinned ring is gone when nobody holds a reader
 * (fstx_bounce_buffer_bytes() == 0 again).  Loaders that are alive at the same time thereby
 * share one set of threads, one ring and one set of streams, as the files of one loader share
 * one nogds_file_reader in the reference (copier/nogds.py:107-116).  Requests of different
 * users go through one FIFO.  A context from fstx_ctx_create is private; releasing it
 * destroys it. */
int fstx_ctx_acquire(const fstx_config *cfg, fstx_ctx **out);
int fstx_ctx_release(fstx_ctx *ctx);

/* Order the context's copy streams after the work that is queued on `stream` right now:
 * copies of requests submitted after this call start only when that work has finished.  A
 * caller whose allocator hands out device memory that kernels on `stream` may still be
 * using calls this before fstx_submit_read instead of synchronizing the device.  (The
 * reference has no counterpart: its copies are synchronous cudaMemcpy calls on the null
 * stream, cpp/ext.cpp:693-705.) */
int fstx_ctx_order_after(fstx_ctx *ctx, void *stream);

/* Open a file for reading in `mode`; returns a file handle >= 1.
 * The reference's Python opens the fd itself (copier/nogds.py:26-31); here the
 * library owns the descriptors because O_DIRECT needs its own. */
int64_t fstx_file_open(fstx_ctx *ctx, const char *path, int mode);

/* Close a handle; outstanding requests on it must have been waited. */
int fstx_file_close(fstx_ctx *ctx, int64_t file);

/* Enqueue: copy file bytes [file_off, file_off+length) to dev_base + dst_off.
 * dev_capacity is the size of the device buffer at dev_base; the range is
 * checked against it (gds_device_buffer::_get_raw_pointer, cpp/ext.hpp:139-146).
 * Returns a request id >= 1 immediately; I/O proceeds on the workers.
 * nogds_file_reader::submit_read (cpp/ext.cpp:726-763). */
int64_t fstx_submit_read(fstx_ctx *ctx, int64_t file, uint64_t file_off, uint64_t length,
                         void *dev_base, uint64_t dev_capacity, uint64_t dst_off);

/* Block until every byte of the request is in device memory; returns the byte
 * count or a negative error.  The id is consumed.  Requests may be waited for in any
 * order; requests submitted later do not hold the wait up (a caller may queue the next
 * file's reads before waiting for this one's, and the transfer then runs on without a
 * pause between the files).
 * nogds_file_reader::wait_read (cpp/ext.cpp:765-776). */
int64_t fstx_wait_read(fstx_ctx *ctx, int64_t request);

/* Snapshot of the context's counters.  Set out->struct_size = sizeof(fstx_metrics) before the
 * call: the library fills in at most that many bytes and stores the count it filled. */
int fstx_get_metrics(fstx_ctx *ctx, fstx_metrics *out);

/* ---- HBM kernels ----------------------------------------------------------- */

/* dst[0:nbytes) = src[0:nbytes), any byte alignment on either side, ranges
 * must not overlap.  The bulk moves as 16-byte vectors with the source
 * funnel-shifted into place.  Replaces gds_device_buffer::memmove
 * (cpp/ext.cpp:606-645), which the reference drives to shift a file's data
 * section down by header_length % 16 bytes (copier/gds.py:138-159). */
int fstx_realign_copy(void *dst, const void *src, uint64_t nbytes, void *stream);

typedef struct fstx_copy_desc {
    void *dst;
    const void *src;
    uint64_t nbytes;
} fstx_copy_desc;

#define FSTX_BATCH_MAX 48

/* n <= FSTX_BATCH_MAX independent realign copies in one launch. */
int fstx_realign_copy_batch(const fstx_copy_desc *descs, uint32_t n, void *stream);

/* Gather `outer` segments of seg_bytes, the o-th read from src + o*src_pitch,
 * into dst + o*seg_bytes (a dense [outer, seg_bytes] block).  This is one
 * rank's shard of a row-major tensor cut along a dimension: for shape
 * [.., S, ..] cut at dim d into blocks of bs, outer = prod(shape[:d]),
 * src_pitch = S * inner_bytes, seg_bytes = rows_of_this_rank * inner_bytes and
 * src already points at the rank's first row.  Nothing has to be aligned: segments
 * of 16 bytes and more move as 16-byte vectors whatever the addresses, lengths and
 * pitches are.  Replaces the per-rank t[slices].contiguous() of
 * LazyTensorFactory.shuffle (tensor_factory.py:168-175). */
int fstx_slice_copy(void *dst, const void *src, uint64_t outer, uint64_t seg_bytes,
                    uint64_t src_pitch, void *stream);

typedef struct fstx_slice_desc {
    void *dst;
    const void *src;
    uint64_t outer;
    uint64_t seg_bytes;
    uint64_t src_pitch;
} fstx_slice_desc;

/* n <= FSTX_BATCH_MAX slice extractions in one launch (the shards of many
 * tensors for one rank, as FilesBufferOnDevice.as_dict asks for them,
 * file_buffer.py:238-259). */
int fstx_slice_copy_batch(const fstx_slice_desc *descs, uint32_t n, void *stream);

typedef struct fstx_slice2d_desc {
    void *dst;
    const void *src;
    uint64_t outer;
    uint64_t seg_bytes;
    uint64_t src_pitch;
    uint64_t dst_pitch; /* bytes between segment starts in dst, >= seg_bytes */
} fstx_slice2d_desc;

/* As fstx_slice_copy_batch, but the o-th segment is written to dst + o*dst_pitch: the
 * rank's blocks of several tensors land side by side along an inner dimension of one
 * joined tensor (dst_pitch = the joined row, dst = the joined tensor + the bytes of the
 * blocks before this one).  Replaces the per-tensor t[slices].contiguous() followed by
 * torch.cat of LazyTensorFactory.shuffle_multi_cols (tensor_factory.py:194-259) when the
 * join runs along a dimension that is not the outermost.  n <= FSTX_BATCH_MAX. */
int fstx_slice_copy2d_batch(const fstx_slice2d_desc *descs, uint32_t n, void *stream);

typedef struct fstx_join_src {
    const void *src;    /* first byte of this tensor's block in its first row */
    uint64_t seg_bytes; /* bytes of the block per row */
    uint64_t src_pitch; /* bytes between rows of the source tensor */
} fstx_join_src;

#define FSTX_JOIN_MAX 24 /* sources per call */

/* Fused slice + concatenate along an inner dimension: row r of the destination (rows
 * dst_pitch bytes apart; 0 = dense, sum(seg_bytes)) is the r-th segments of the n sources
 * side by side.  Same result as n descriptors of fstx_slice_copy2d_batch, but the
 * destination is written front to back in whole 16-byte vectors -- a vector that holds the
 * end of one block and the beginning of the next is put together in registers -- whatever
 * the widths and alignments of the blocks are.
 * Replaces the contiguous() + torch.cat of LazyTensorFactory.shuffle_multi_cols
 * (tensor_factory.py:194-259).  n <= FSTX_JOIN_MAX. */
int fstx_join_copy(void *dst, uint64_t dst_pitch, uint64_t rows, const fstx_join_src *srcs, uint32_t n,
                   void *stream);

typedef struct fstx_join_desc {
    void *dst;
    uint64_t dst_pitch;        /* 0 = dense */
    uint64_t rows;
    const fstx_join_src *srcs; /* n_srcs <= FSTX_JOIN_MAX sources */
    uint32_t n_srcs;
    uint32_t reserved;
} fstx_join_desc;

/* Several joins at once: as many of them per launch as the kernel's tables hold (the q/k/v and
 * gate/up packing of all layers of a file, as a caller that walks a checkpoint asks for them).
 * Any count.  Same result as one fstx_join_copy per descriptor. */
int fstx_join_copy_batch(const fstx_join_desc *joins, uint32_t n, void *stream);

/* element types of fstx_convert_batch */
enum fstx_elem_type {
    FSTX_F64 = 0,
    FSTX_F32 = 1,
    FSTX_F16 = 2,
    FSTX_BF16 = 3,
    FSTX_F8_E4M3 = 4, /* e4m3fn: no infinity, 0x7f / 0xff are NaN */
    FSTX_F8_E5M2 = 5
};

typedef struct fstx_convert_desc {
    void *dst;
    const void *src;
    uint64_t n_elems;
    uint32_t src_type; /* enum fstx_elem_type */
    uint32_t dst_type;
} fstx_convert_desc;

/* n <= FSTX_BATCH_MAX element-type conversions in one launch, out of place, towards a
 * type that is not wider (f64 -> f32/f16/bf16/fp8, f32 -> f16/bf16/fp8, f16 <-> bf16,
 * f16/bf16 -> fp8), with the rounding of torch's Tensor.to().  Replaces the per-tensor
 * t2.to(dtype) + copy_ of SafeTensorsMetadata.get_tensors when copy_files_to_device is
 * given a dtype (common.py:355-375). */
int fstx_convert_batch(const fstx_convert_desc *descs, uint32_t n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FSTX_H */
