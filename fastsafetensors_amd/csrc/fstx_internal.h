// SPDX-License-Identifier: Apache-2.0
//
// Seams inside libfstx: the pipeline (fstx_pipeline.cpp) is plain C++ and
// reaches the GPU runtime only through the few calls declared in fstx_dev.
// The shipped library binds them to HIP (fstx_device_hip.cpp).  The host-side
// unit tests link the same pipeline source against an in-memory stand-in so
// that thread sanitizers can run without a GPU; that stand-in is not part of
// the shipped library.
#ifndef FSTX_INTERNAL_H
#define FSTX_INTERNAL_H

#include <stddef.h>
#include <stdint.h>

namespace fstx_dev {

typedef void *stream_t;
typedef void *event_t;

// every call returns 0 or a negative fstx status
int device_count();
int set_device(int device_id);
int pci_bus_id(int device_id, char *out, int len);
int host_alloc(void **out, size_t bytes);   // pinned, device-visible host memory
int host_free(void *p);
int stream_create(stream_t *out);
int stream_destroy(stream_t s);
int stream_sync(stream_t s);
int event_create(event_t *out);
int event_destroy(event_t e);
int event_record(event_t e, stream_t s);
int event_ready(event_t e);                 // 1 done, 0 still running, <0 error
int event_sync(event_t e);
int stream_idle(stream_t s);                  // 1 nothing queued on s is still running, 0 busy, <0 error
int stream_wait_event(stream_t s, event_t e); // work queued on s after this call waits for e's last record
int copy_to_device_async(void *dev_dst, const void *host_src, size_t bytes, stream_t s);

} // namespace fstx_dev

namespace fstx_internal {

int check_launch(const char *what);  // hipGetLastError -> 0 / -FSTX_E_HIP
// FSTX_GATHER_MODE, for measurements: 0 the gather kernel is never used (unit-sized moves instead),
// 1 (default) it serves every strided shape but dense cuts that are 16-byte aligned throughout,
// 2 those too
int gather_mode();
bool debug_enabled();
void debug(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
void note_bounce_bytes(int64_t delta); // process-wide pinned ring accounting

// Named ranges for a profiler's timeline (roctx: they show up in rocprofv3 --marker-trace and in
// tools that read its output), switched on by FSTX_ROCTX=1: the library then loads
// librocprofiler-sdk-roctx.so, else libroctx64.so (or what FSTX_ROCTX_LIB names) by itself.  Off, or without that library, a range costs one
// relaxed load.  Ranges nest per thread and are closed by the destructor.
struct Range {
    explicit Range(const char *fmt, ...) __attribute__((format(printf, 2, 3)));
    ~Range();
    Range(const Range &) = delete;
    Range &operator=(const Range &) = delete;

  private:
    bool open_ = false;
};

} // namespace fstx_internal

#endif
