// Asynchronous upload of small host-built tables (work lists) into a caller's device workspace.
#ifndef ATBMI_UPLOAD_RING_H
#define ATBMI_UPLOAD_RING_H
#include <cstring>
#include <mutex>
#include "atbmi_common.h"

namespace atbmi {

// Pinned staging for hipMemcpyAsync: a slot is reused only after the copy that last read it has finished.
// One ring per process, taken under a lock for the length of an upload.
struct UploadRing {
    static constexpr int RING = 4;
    std::mutex lock;
    void *pinned[RING] = {nullptr, nullptr, nullptr, nullptr};
    size_t cap[RING] = {0, 0, 0, 0};
    hipEvent_t copied[RING] = {nullptr, nullptr, nullptr, nullptr};
    bool inFlight[RING] = {false, false, false, false};
    int pos = 0;
};
inline UploadRing g_uploadRing;

// Copies `bytes` at `src` (pageable host memory, free to change once this returns) to `dst` on `stream`.
inline int UploadTable(const void *src, size_t bytes, void *dst, hipStream_t stream)
{
    UploadRing &r = g_uploadRing;
    std::lock_guard<std::mutex> hold(r.lock);
    const int slot = r.pos;
    r.pos = (r.pos + 1) % UploadRing::RING;
    if (r.inFlight[slot]) {
        ATBMI_HIP_CHECK(hipEventSynchronize(r.copied[slot]));
        r.inFlight[slot] = false;
    }
    if (r.cap[slot] < bytes) {
        if (r.pinned[slot]) {
            ATBMI_HIP_CHECK(hipHostFree(r.pinned[slot]));
            r.pinned[slot] = nullptr;
            r.cap[slot] = 0;
        }
        const size_t cap = (bytes * 2 + 4095) / 4096 * 4096;
        ATBMI_HIP_CHECK(hipHostMalloc(&r.pinned[slot], cap, hipHostMallocDefault));
        r.cap[slot] = cap;
    }
    if (!r.copied[slot]) {
        ATBMI_HIP_CHECK(hipEventCreateWithFlags(&r.copied[slot], hipEventDisableTiming));
    }
    memcpy(r.pinned[slot], src, bytes);
    ATBMI_HIP_CHECK(hipMemcpyAsync(dst, r.pinned[slot], bytes, hipMemcpyHostToDevice, stream));
    ATBMI_HIP_CHECK(hipEventRecord(r.copied[slot], stream));
    r.inFlight[slot] = true;
    return OK;
}

} // namespace atbmi
#endif
