/* SPDX-License-Identifier: Apache-2.0
 *
 * TEST PROGRAM: drives libfstx.so from plain C through include/fstx.h only -- no Python,
 * no torch, no C++ types -- the way a cgo / JNI / N-API binding of the reference would.
 * Device memory comes from the HIP runtime's C API.
 *
 *   cabi_check FILE
 *
 * Loads FILE (any bytes) into device memory with the read pipeline in every read mode, through
 * a private and through a shared context, then checks the realign copy, the slice extract
 * (dense, batched, strided destination, joined, joined in a batch) and the fp32 -> bf16
 * conversion against loops on the host, and calls the small entry points.  Every function
 * include/fstx.h declares is called at least once.  Prints "cabi_check: ok".
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "fstx.h"

/* the six HIP runtime entry points this program needs, declared the way an FFI would */
typedef int hipError_t;
enum { hipSuccess = 0, hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2 };
hipError_t hipSetDevice(int device);
hipError_t hipMalloc(void **ptr, size_t size);
hipError_t hipFree(void *ptr);
hipError_t hipMemcpy(void *dst, const void *src, size_t size, int kind);
hipError_t hipMemset(void *dst, int value, size_t size);
hipError_t hipDeviceSynchronize(void);

#define CHECK(cond)                                                              \
    do {                                                                         \
        if (!(cond)) {                                                           \
            fprintf(stderr, "cabi_check: FAILED at line %d: %s\n", __LINE__, #cond); \
            return 1;                                                            \
        }                                                                        \
    } while (0)

static uint16_t bf16_of(float f) { /* round to nearest even; NaN -> 0x7fc0 */
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

int main(int argc, char **argv) {
    if (argc != 2) {
        fprintf(stderr, "usage: %s FILE\n", argv[0]);
        return 2;
    }
    FILE *fp = fopen(argv[1], "rb");
    CHECK(fp != NULL);
    fseek(fp, 0, SEEK_END);
    uint64_t size = (uint64_t)ftell(fp);
    fseek(fp, 0, SEEK_SET);
    CHECK(size >= 4096);
    unsigned char *want = malloc(size), *got = malloc(size), *tmp = malloc(size);
    CHECK(want && got && tmp && fread(want, 1, size, fp) == size);
    fclose(fp);

    CHECK(fstx_abi_version() == FSTX_ABI_VERSION);
    CHECK(fstx_device_count() >= 1);
    CHECK(hipSetDevice(0) == hipSuccess);
    unsigned char *arena = NULL, *out = NULL;
    CHECK(hipMalloc((void **)&arena, size + 256) == hipSuccess);
    CHECK(hipMalloc((void **)&out, size + 256) == hipSuccess);

    /* ---- the read pipeline, every mode, data landing at an odd offset ---- */
    fstx_config cfg;
    memset(&cfg, 0, sizeof cfg);
    cfg.struct_size = sizeof cfg;
    cfg.device_id = 0;
    cfg.numa_node = -1;
    cfg.n_threads = 4;
    cfg.block_bytes = 256 * 1024;
    fstx_ctx *ctx = NULL;
    CHECK(fstx_ctx_create(&cfg, &ctx) == 0);
    const int modes[3] = {FSTX_READ_AUTO, FSTX_READ_BUFFERED, FSTX_READ_DIRECT};
    for (int m = 0; m < 3; ++m) {
        CHECK(hipMemset(arena, 0xee, size + 256) == hipSuccess);
        int64_t file = fstx_file_open(ctx, argv[1], modes[m]);
        CHECK(file > 0);
        const uint64_t skip = 10; /* like a header whose length is not a multiple of 16 */
        int64_t req = fstx_submit_read(ctx, file, skip, size - skip, arena, size + 256, 3);
        CHECK(req > 0);
        CHECK(fstx_wait_read(ctx, req) == (int64_t)(size - skip));
        CHECK(fstx_file_close(ctx, file) == 0);
        CHECK(hipMemcpy(got, arena + 3, size - skip, hipMemcpyDeviceToHost) == hipSuccess);
        CHECK(memcmp(got, want + skip, size - skip) == 0);
        /* a range beyond the buffer is refused at submit */
        file = fstx_file_open(ctx, argv[1], modes[m]);
        CHECK(fstx_submit_read(ctx, file, 0, size, arena, size - 1, 0) < 0);
        CHECK(fstx_file_close(ctx, file) == 0);
    }
    fstx_metrics met;
    memset(&met, 0, sizeof met);
    met.struct_size = sizeof met;
    CHECK(fstx_get_metrics(ctx, &met) == 0 && met.bytes_copied >= 3 * (size - 10) && met.struct_size == sizeof met);
    {
        /* a caller built against a shorter struct: the library fills what fits and not a byte more */
        uint64_t old_caller[8];
        memset(old_caller, 0xEE, sizeof old_caller);
        old_caller[0] = 4 * sizeof(uint64_t);
        CHECK(fstx_get_metrics(ctx, (fstx_metrics *)old_caller) == 0);
        CHECK(old_caller[0] == 4 * sizeof(uint64_t) && old_caller[2] == met.bytes_read && old_caller[4] == 0xEEEEEEEEEEEEEEEEull);
        int cpus[4];
        CHECK(fstx_node_cpus(-1, cpus, 4) < 0);
    }
    const uint64_t ring_of_ctx = met.bounce_buffer_bytes;
    CHECK(fstx_ctx_destroy(ctx) == 0);
    CHECK(fstx_bounce_buffer_bytes() == 0);
    /* the ring stays parked for the next context of this shape, which takes it over; trimming frees it */
    CHECK(fstx_cached_ring_bytes() == ring_of_ctx);
    {
        fstx_ctx *next = NULL;
        CHECK(fstx_ctx_create(&cfg, &next) == 0);
        met.struct_size = sizeof met;
        CHECK(fstx_get_metrics(next, &met) == 0 && met.ring_reused == 1 && fstx_cached_ring_bytes() == 0);
        CHECK(fstx_ctx_destroy(next) == 0 && fstx_cached_ring_bytes() == ring_of_ctx);
        CHECK(fstx_trim_cache() == ring_of_ctx && fstx_cached_ring_bytes() == 0 && fstx_trim_cache() == 0);
    }

    /* ---- a shared context: two users, one ring; ordered after the null stream's work ---- */
    {
        fstx_ctx *a = NULL, *b = NULL;
        /* the first user has it built behind its back; how a context came to be is not part of what it is */
        fstx_config behind = cfg;
        behind.flags = FSTX_CREATE_ASYNC;
        CHECK(fstx_ctx_acquire(&behind, &a) == 0 && fstx_ctx_acquire(&cfg, &b) == 0 && a == b);
        met.struct_size = sizeof met;
        CHECK(fstx_get_metrics(a, &met) == 0 && met.create_ns > 0); /* waits for the build */
        const uint64_t ring = fstx_bounce_buffer_bytes();
        CHECK(ring > 0);
        CHECK(hipMemset(arena, 0x11, size + 256) == hipSuccess); /* queued on the null stream ... */
        CHECK(fstx_ctx_order_after(a, NULL) == 0);               /* ... and the copies come after it */
        int64_t file = fstx_file_open(b, argv[1], FSTX_READ_BUFFERED);
        CHECK(file > 0);
        int64_t first = fstx_submit_read(a, file, 0, size / 2, arena, size + 256, 0);
        int64_t second = fstx_submit_read(b, file, size / 2, size - size / 2, arena, size + 256, size / 2);
        CHECK(first > 0 && second > 0);
        CHECK(fstx_wait_read(a, first) == (int64_t)(size / 2)); /* with the second still in flight */
        CHECK(fstx_wait_read(b, second) == (int64_t)(size - size / 2));
        CHECK(fstx_file_close(a, file) == 0);
        CHECK(hipMemcpy(got, arena, size, hipMemcpyDeviceToHost) == hipSuccess && memcmp(got, want, size) == 0);
        CHECK(fstx_ctx_release(a) == 0 && fstx_bounce_buffer_bytes() == ring); /* one user left */
        CHECK(fstx_ctx_release(b) == 0 && fstx_bounce_buffer_bytes() == 0);
        /* put the bytes back where the kernel checks below expect them */
        CHECK(hipMemcpy(arena + 3, want + 10, size - 10, hipMemcpyHostToDevice) == hipSuccess);
    }

    /* ---- kernels: arena + 3 holds file bytes [10, size) ---- */
    const unsigned char *src = arena + 3;
    const unsigned char *hsrc = want + 10;
    const uint64_t n = size - 10;
    CHECK(fstx_realign_copy(out, src, n, NULL) == 0);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    CHECK(hipMemcpy(got, out, n, hipMemcpyDeviceToHost) == hipSuccess && memcmp(got, hsrc, n) == 0);

    const uint64_t pitch = 1000, seg = 336, outer = n / pitch; /* a [outer, 1000] byte matrix, columns 100..435 */
    CHECK(fstx_slice_copy(out, src + 100, outer, seg, pitch, NULL) == 0);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    CHECK(hipMemcpy(got, out, outer * seg, hipMemcpyDeviceToHost) == hipSuccess);
    for (uint64_t r = 0; r < outer; ++r) CHECK(memcmp(got + r * seg, hsrc + r * pitch + 100, seg) == 0);

    /* the same cut and a whole-row block in one batched call */
    fstx_slice_desc sd[2] = {{out, src + 100, outer, seg, pitch}, {out + outer * seg, src, 7, pitch, pitch}};
    CHECK(hipMemset(out, 0, outer * seg + 7 * pitch) == hipSuccess);
    CHECK(fstx_slice_copy_batch(sd, 2, NULL) == 0);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    CHECK(hipMemcpy(got, out, outer * seg + 7 * pitch, hipMemcpyDeviceToHost) == hipSuccess);
    for (uint64_t r = 0; r < outer; ++r) CHECK(memcmp(got + r * seg, hsrc + r * pitch + 100, seg) == 0);
    CHECK(memcmp(got + outer * seg, hsrc, 7 * pitch) == 0);

    /* two column blocks side by side in one joined matrix, both ways */
    const uint64_t seg2 = 64, joined = seg + seg2;
    fstx_join_src parts[2] = {{src + 100, seg, pitch}, {src + 600, seg2, pitch}};
    CHECK(fstx_join_copy(out, 0, outer, parts, 2, NULL) == 0);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    CHECK(hipMemcpy(got, out, outer * joined, hipMemcpyDeviceToHost) == hipSuccess);
    for (uint64_t r = 0; r < outer; ++r) {
        CHECK(memcmp(got + r * joined, hsrc + r * pitch + 100, seg) == 0);
        CHECK(memcmp(got + r * joined + seg, hsrc + r * pitch + 600, seg2) == 0);
    }
    CHECK(hipMemset(out, 0, outer * joined) == hipSuccess);
    fstx_slice2d_desc d2[2] = {{out, src + 100, outer, seg, pitch, joined}, {out + seg, src + 600, outer, seg2, pitch, joined}};
    CHECK(fstx_slice_copy2d_batch(d2, 2, NULL) == 0);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    CHECK(hipMemcpy(tmp, out, outer * joined, hipMemcpyDeviceToHost) == hipSuccess);
    CHECK(memcmp(tmp, got, outer * joined) == 0);

    /* two joins in one batched call: the same one, and its blocks the other way round */
    {
        fstx_join_src swapped[2] = {parts[1], parts[0]};
        fstx_join_desc jd[2] = {{out, 0, outer, parts, 2, 0}, {out + outer * joined, 0, outer, swapped, 2, 0}};
        CHECK(hipMemset(out, 0, 2 * outer * joined) == hipSuccess);
        CHECK(fstx_join_copy_batch(jd, 2, NULL) == 0);
        CHECK(hipDeviceSynchronize() == hipSuccess);
        CHECK(hipMemcpy(tmp, out, 2 * outer * joined, hipMemcpyDeviceToHost) == hipSuccess);
        CHECK(memcmp(tmp, got, outer * joined) == 0);
        for (uint64_t r = 0; r < outer; ++r) {
            CHECK(memcmp(tmp + (outer + r) * joined, hsrc + r * pitch + 600, seg2) == 0);
            CHECK(memcmp(tmp + (outer + r) * joined + seg2, hsrc + r * pitch + 100, seg) == 0);
        }
    }

    /* fp32 -> bf16 on values of our own */
    enum { NF = 100000 };
    float *hf = malloc(NF * sizeof(float));
    uint16_t *hb = malloc(NF * sizeof(uint16_t));
    CHECK(hf && hb);
    uint32_t lcg = 12345u;
    for (int i = 0; i < NF; ++i) {
        lcg = lcg * 1664525u + 1013904223u;
        uint32_t bits = lcg; /* any bit pattern: normals, denormals, infinities, NaNs */
        memcpy(&hf[i], &bits, 4);
    }
    CHECK(hipMemcpy(arena, hf, NF * sizeof(float), hipMemcpyHostToDevice) == hipSuccess);
    fstx_convert_desc cd = {out, arena, NF, FSTX_F32, FSTX_BF16};
    CHECK(fstx_convert_batch(&cd, 1, NULL) == 0);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    CHECK(hipMemcpy(hb, out, NF * sizeof(uint16_t), hipMemcpyDeviceToHost) == hipSuccess);
    for (int i = 0; i < NF; ++i) CHECK(hb[i] == bf16_of(hf[i]));

    /* the small entry points */
    CHECK(fstx_get_alignment_size() == 4096);
    char pci[32];
    CHECK(fstx_get_device_pci_bus(0, pci, (int)sizeof pci) == 0 && strlen(pci) >= 7 && strchr(pci, ':') != NULL);
    CHECK(fstx_get_device_pci_bus(0, pci, 2) < 0);
    void *host = fstx_host_alloc(5000);
    CHECK(host != NULL && ((uintptr_t)host & 4095) == 0);
    memset(host, 1, 5000);
    fstx_host_free(host);
    fstx_set_debug_log(0);
    (void)fstx_set_numa_node(0); /* a machine without NUMA information answers with an error; nothing to check but that it returns */

    /* error text and argument checks */
    CHECK(strcmp(fstx_strerror(0), "ok") == 0);
    CHECK(fstx_realign_copy_batch(NULL, 3, NULL) == -FSTX_E_INVAL);
    CHECK(fstx_join_copy(out, 8, 4, parts, 2, NULL) == -FSTX_E_INVAL); /* rows would overlap */

    hipFree(arena);
    hipFree(out);
    printf("cabi_check: ok (%llu bytes, 3 read modes, shared context, realign, slice, join, convert)\n", (unsigned long long)size);
    return 0;
}
