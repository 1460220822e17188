/* SPDX-License-Identifier: Apache-2.0
 *
 * TEST INFRASTRUCTURE -- not part of the shipped load path.
 *
 * Plain-C, CPU-only restatement of the reference's device="cpu", nogds=True
 * read path (foundation-model-stack/fastsafetensors 0.3.2).  It is the checker
 * that the HIP path is compared with and the CPU baseline that is timed beside
 * it; nothing in the package may call it.
 *
 * What follows what (reference paths relative to its root):
 *   reader geometry      fastsafetensors/cpp/ext.hpp:176-180  slot KiB = ceil(bbuf_kb / max_threads)
 *   bounce allocation    fastsafetensors/cpp/ext.cpp:735-751  one 4096-aligned buffer of slot*threads, on first submit
 *                        (cpu_cudaHostAlloc = posix_memalign, ext.cpp:154-159)
 *   submit_read          fastsafetensors/cpp/ext.cpp:726-763  id = next_id++, slot = id % threads, join the slot's old thread
 *   worker loop          fastsafetensors/cpp/ext.cpp:676-710  pread <= slot bytes, then copy to dst + ptr_off + count
 *                        (cpu_cudaMemcpy = memcpy, ext.cpp:143-146); a short pread fails the request (:688-693)
 *   bounds check         fastsafetensors/cpp/ext.hpp:139-146  dst range must fit the buffer
 *   wait_read            fastsafetensors/cpp/ext.cpp:765-776  block on the result, erase it
 *   file split           fastsafetensors/copier/nogds.py:39-56 requests of max_copy_block_size over [header_length, size)
 *   drain                fastsafetensors/copier/nogds.py:58-78 wait every request, then report
 *   memmove via tmp      fastsafetensors/cpp/ext.cpp:606-645  src -> tmp -> dst, two full copies
 *   slice + contiguous   fastsafetensors/tensor_factory.py:168-175  row-major dense copy of t[(:,)*dim + (lo:hi,)]
 *
 * Parity of this file is pinned by tests/test_oracle.py: against file bytes
 * read with Python I/O (closed form: tensor bytes == file[header+s : header+e]),
 * against numpy slicing for the slice copy, and against the reference's own
 * nogds_file_reader compiled into oracle/_ref when that build is present.
 */
#define _GNU_SOURCE
#include <errno.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>
#include <fcntl.h>

#define ORACLE_ALIGN 4096
#define ORACLE_MAX_REQ 65536

typedef struct job {
    struct fst_oracle_reader *r;
    int id;
    int fd;
    char *dst;          /* base of the destination buffer */
    int64_t offset;     /* file offset */
    int64_t length;
    uint64_t ptr_off;   /* offset inside the destination buffer */
} job_t;

typedef struct fst_oracle_reader {
    uint64_t slot_bytes;
    uint64_t max_threads;
    char *bounce;
    int next_id;
    pthread_t *threads;
    char *thread_live;
    job_t **jobs;
    pthread_mutex_t mu;
    pthread_cond_t cv;
    signed char result[ORACLE_MAX_REQ]; /* 0 pending, 1 ok, -1 failed */
} fst_oracle_reader;

fst_oracle_reader *fst_oracle_reader_new(uint64_t bbuf_size_kb, uint64_t max_threads) {
    fst_oracle_reader *r = calloc(1, sizeof *r);
    if (!r || max_threads == 0) { free(r); return NULL; }
    r->slot_bytes = ((bbuf_size_kb + max_threads - 1) / max_threads) * 1024;
    r->max_threads = max_threads;
    r->next_id = 1;
    r->threads = calloc(max_threads, sizeof(pthread_t));
    r->thread_live = calloc(max_threads, 1);
    r->jobs = calloc(max_threads, sizeof(job_t *));
    pthread_mutex_init(&r->mu, NULL);
    pthread_cond_init(&r->cv, NULL);
    return r;
}

uint64_t fst_oracle_bounce_bytes(const fst_oracle_reader *r) {
    return r->bounce ? r->slot_bytes * r->max_threads : 0;
}

static void *worker(void *arg) {
    job_t *j = arg;
    fst_oracle_reader *r = j->r;
    char *buffer = r->bounce + r->slot_bytes * ((uint64_t)j->id % r->max_threads);
    int failed = 0;
    int64_t count = 0;
    while (count < j->length) {
        int64_t l = j->length - count;
        if (l > (int64_t)r->slot_bytes) l = (int64_t)r->slot_bytes;
        int64_t c = pread(j->fd, buffer, (size_t)l, j->offset + count);
        if (c != l) { failed = 1; break; }
        memcpy(j->dst + j->ptr_off + count, buffer, (size_t)c);
        count += c;
    }
    pthread_mutex_lock(&r->mu);
    r->result[j->id % ORACLE_MAX_REQ] = failed ? -1 : 1;
    pthread_cond_broadcast(&r->cv);
    pthread_mutex_unlock(&r->mu);
    return NULL;
}

/* returns the request id (> 0) or -1 */
int fst_oracle_submit_read(fst_oracle_reader *r, int fd, void *dst, uint64_t dst_len,
                           int64_t offset, int64_t length, uint64_t ptr_off) {
    if (ptr_off + (uint64_t)length > dst_len) return -1; /* out of bound access */
    int id = r->next_id++;
    if (!r->bounce) {
        void *p = NULL;
        if (posix_memalign(&p, ORACLE_ALIGN, r->slot_bytes * r->max_threads) != 0) return -1;
        r->bounce = p;
    }
    uint64_t slot = (uint64_t)id % r->max_threads;
    if (r->thread_live[slot]) {
        pthread_join(r->threads[slot], NULL);
        free(r->jobs[slot]);
        r->thread_live[slot] = 0;
    }
    job_t *j = malloc(sizeof *j);
    *j = (job_t){r, id, fd, dst, offset, length, ptr_off};
    pthread_mutex_lock(&r->mu);
    r->result[id % ORACLE_MAX_REQ] = 0;
    pthread_mutex_unlock(&r->mu);
    if (pthread_create(&r->threads[slot], NULL, worker, j) != 0) { free(j); return -1; }
    r->jobs[slot] = j;
    r->thread_live[slot] = 1;
    return id;
}

/* 0 on success, -1 when the request failed */
int fst_oracle_wait_read(fst_oracle_reader *r, int id) {
    pthread_mutex_lock(&r->mu);
    while (r->result[id % ORACLE_MAX_REQ] == 0) pthread_cond_wait(&r->cv, &r->mu);
    int ok = r->result[id % ORACLE_MAX_REQ] == 1;
    r->result[id % ORACLE_MAX_REQ] = 0;
    pthread_mutex_unlock(&r->mu);
    return ok ? 0 : -1;
}

void fst_oracle_reader_free(fst_oracle_reader *r) {
    if (!r) return;
    for (uint64_t i = 0; i < r->max_threads; ++i)
        if (r->thread_live[i]) { pthread_join(r->threads[i], NULL); free(r->jobs[i]); }
    free(r->bounce);
    free(r->threads);
    free(r->thread_live);
    free(r->jobs);
    pthread_mutex_destroy(&r->mu);
    pthread_cond_destroy(&r->cv);
    free(r);
}

/* NoGdsFileCopier.submit_io + wait_io for one file: dst receives the data section
 * [header_length, size_bytes).  Returns bytes loaded or -1. */
int64_t fst_oracle_load_file(fst_oracle_reader *r, const char *path, uint64_t header_length,
                             uint64_t size_bytes, void *dst, uint64_t max_copy_block_size) {
    int fd = open(path, O_RDONLY);
    if (fd < 0) return -1;
    uint64_t total = size_bytes - header_length, count = 0;
    int first = 0, last = 0, failed = 0;
    while (count < total) {
        uint64_t l = total - count;
        if (max_copy_block_size < l) l = max_copy_block_size;
        int id = fst_oracle_submit_read(r, fd, dst, total, (int64_t)(header_length + count), (int64_t)l, count);
        if (id < 0) { failed = 1; break; }
        if (!first) first = id;
        last = id;
        count += l;
    }
    for (int id = first; first && id <= last; ++id)
        if (fst_oracle_wait_read(r, id) < 0) failed = 1;
    close(fd);
    return failed ? -1 : (int64_t)total;
}

void *fst_oracle_alloc(uint64_t length) { /* cpu_malloc, ext.cpp:542-548 */
    void *p = NULL;
    if (posix_memalign(&p, ORACLE_ALIGN, length ? length : 1) != 0) return NULL;
    return p;
}
void fst_oracle_free(void *p) { free(p); }

/* gds_device_buffer::memmove: buf[dst_off : dst_off+n) = buf[src_off : src_off+n) through tmp */
int fst_oracle_memmove(char *buf, uint64_t buf_len, uint64_t dst_off, uint64_t src_off, char *tmp,
                       uint64_t tmp_len, uint64_t n) {
    if (buf_len < dst_off || buf_len < src_off || tmp_len < n) return -1;
    if (n == 0) return 0;
    memcpy(tmp, buf + src_off, n);
    memcpy(buf + dst_off, tmp, n);
    return 0;
}

/* Dense copy of one rank's block: `outer` segments of seg bytes, read `pitch` apart. */
void fst_oracle_slice(char *dst, const char *src, uint64_t outer, uint64_t seg, uint64_t pitch) {
    for (uint64_t o = 0; o < outer; ++o) memcpy(dst + o * seg, src + o * pitch, seg);
}
