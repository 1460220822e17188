// SPDX-License-Identifier: Apache-2.0
//
// HIP binding of the device seam used by the copy pipeline.  Streams are
// created at the default priority; events carry no timing and block the
// waiting thread instead of spinning, because the waiters are the same
// threads that should be inside pread().

#include <hip/hip_runtime.h>

#include <cstdlib>

#include "fstx.h"
#include "fstx_internal.h"

namespace {
inline int rc(hipError_t e, const char *what) {
    if (e == hipSuccess) return 0;
    fstx_internal::debug("%s failed: %s", what, hipGetErrorString(e));
    return -FSTX_E_HIP;
}
} // namespace

namespace fstx_dev {

int device_count() {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return -FSTX_E_NO_DEVICE;
    }
    return n;
}

int set_device(int device_id) { return rc(hipSetDevice(device_id), "hipSetDevice"); }

int pci_bus_id(int device_id, char *out, int len) {
    return rc(hipDeviceGetPCIBusId(out, len, device_id), "hipDeviceGetPCIBusId");
}

int host_alloc(void **out, size_t bytes) {
    return rc(hipHostMalloc(out, bytes, hipHostMallocDefault), "hipHostMalloc");
}

int host_free(void *p) { return rc(hipHostFree(p), "hipHostFree"); }

int stream_create(stream_t *out) {
    hipStream_t s = nullptr;
    int r = rc(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreateWithFlags");
    *out = s;
    return r;
}

int stream_destroy(stream_t s) {
    return rc(hipStreamDestroy(static_cast<hipStream_t>(s)), "hipStreamDestroy");
}

int stream_sync(stream_t s) {
    return rc(hipStreamSynchronize(static_cast<hipStream_t>(s)), "hipStreamSynchronize");
}

int event_create(event_t *out) {
    hipEvent_t e = nullptr;
    int r = rc(hipEventCreateWithFlags(&e, hipEventDisableTiming | hipEventBlockingSync),
               "hipEventCreateWithFlags");
    *out = e;
    return r;
}

int event_destroy(event_t e) {
    return rc(hipEventDestroy(static_cast<hipEvent_t>(e)), "hipEventDestroy");
}

int event_record(event_t e, stream_t s) {
    return rc(hipEventRecord(static_cast<hipEvent_t>(e), static_cast<hipStream_t>(s)),
              "hipEventRecord");
}

int event_ready(event_t e) {
    hipError_t q = hipEventQuery(static_cast<hipEvent_t>(e));
    if (q == hipSuccess) return 1;
    if (q == hipErrorNotReady) {
        (void)hipGetLastError();
        return 0;
    }
    return rc(q, "hipEventQuery");
}

int event_sync(event_t e) {
    return rc(hipEventSynchronize(static_cast<hipEvent_t>(e)), "hipEventSynchronize");
}

int stream_idle(stream_t s) {
    hipError_t q = hipStreamQuery(static_cast<hipStream_t>(s));
    if (q == hipSuccess) return 1;
    if (q == hipErrorNotReady) {
        (void)hipGetLastError();
        return 0;
    }
    return rc(q, "hipStreamQuery");
}

int stream_wait_event(stream_t s, event_t e) {
    return rc(hipStreamWaitEvent(static_cast<hipStream_t>(s), static_cast<hipEvent_t>(e), 0), "hipStreamWaitEvent");
}

int copy_to_device_async(void *dev_dst, const void *host_src, size_t bytes, stream_t s) {
    return rc(hipMemcpyAsync(dev_dst, host_src, bytes, hipMemcpyHostToDevice,
                             static_cast<hipStream_t>(s)),
              "hipMemcpyAsync");
}

} // namespace fstx_dev

namespace fstx_internal {
int check_launch(const char *what) { return rc(hipGetLastError(), what); }
int gather_mode() {
    const char *e = getenv("FSTX_GATHER_MODE"); // read per call so that a benchmark can flip it
    return e && e[0] >= '0' && e[0] <= '2' ? e[0] - '0' : 1;
}
} // namespace fstx_internal
