// Host bytes -> device memory through pinned staging.
//
// The loader hands over slices of a memory-mapped model file: pageable
// memory.  A plain hipMemcpy(Async) of such memory is staged by the runtime in
// small pieces and runs well below what the host link carries.  Here the
// library keeps a ring of pinned slots per device: the caller's bytes are
// copied into a slot by a few host threads while the previous slots' DMA
// transfers are in flight, each slot is sent with one hipMemcpyAsync on the
// caller's stream, and an event per slot tells when it may be refilled.  On
// return every byte has left the caller's buffer (it may be unmapped); the
// device copy completes in stream order.
//
// No kernel here: host code only.
#include <algorithm>
#include <cstring>
#include <mutex>
#include <thread>
#include <unordered_map>

#include "rfq_common.hpp"

namespace rfq {
namespace {

constexpr size_t SLOT_BYTES = (size_t)8 << 20;
constexpr int SLOTS = 4;
constexpr int COPY_THREADS = 4;                        // host threads filling one slot
constexpr size_t THREAD_MIN = (size_t)1 << 20;         // below this a slot is filled by the calling thread alone

struct Ring {
    uint8_t *host[SLOTS] = {nullptr, nullptr, nullptr, nullptr};
    hipEvent_t done[SLOTS] = {nullptr, nullptr, nullptr, nullptr};
    bool in_flight[SLOTS] = {false, false, false, false};
    int next = 0;
    bool ready = false;
};
std::mutex ring_mutex;                                  // one upload at a time: the ring is shared
std::unordered_map<int, Ring> rings;                    // per device

int ring_for_current_device(Ring **out)
{
    int device = 0;
    RFQ_HIP(hipGetDevice(&device));
    Ring &r = rings[device];
    if (!r.ready) {
        for (int i = 0; i < SLOTS; i++) {
            // (a call that failed half way leaves what it got; the next one carries on from there)
            if (!r.host[i]) RFQ_HIP(hipHostMalloc(reinterpret_cast<void **>(&r.host[i]), SLOT_BYTES, hipHostMallocDefault));
            if (!r.done[i]) RFQ_HIP(hipEventCreateWithFlags(&r.done[i], hipEventDisableTiming));
        }
        r.ready = true;
    }
    *out = &r;
    return RFQ_OK;
}

void fill_slot(uint8_t *dst, const uint8_t *src, size_t bytes)
{
    if (bytes < 2 * THREAD_MIN) {
        std::memcpy(dst, src, bytes);
        return;
    }
    const int parts = (int)std::min<size_t>(COPY_THREADS, bytes / THREAD_MIN);
    const size_t per = ((bytes / parts) + 4095) & ~(size_t)4095;
    // (no exception may leave through the C ABI: a part whose thread cannot be started is copied here)
    std::thread helpers[COPY_THREADS];
    int started = 0;
    for (int p = 1; p < parts; p++) {
        const size_t at = per * p, len = p == parts - 1 ? bytes - at : per;
        try {
            helpers[started] = std::thread([=] { std::memcpy(dst + at, src + at, len); });
            started++;
        } catch (...) {
            std::memcpy(dst + at, src + at, len);
        }
    }
    std::memcpy(dst, src, per);
    for (int i = 0; i < started; i++) helpers[i].join();
}

} // namespace

int upload_bytes(const void *h_src, size_t bytes, void *d_dst, hipStream_t s)
{
    std::lock_guard<std::mutex> lock(ring_mutex);
    Ring *r = nullptr;
    if (int rc = ring_for_current_device(&r)) return rc;
    const uint8_t *src = static_cast<const uint8_t *>(h_src);
    uint8_t *dst = static_cast<uint8_t *>(d_dst);
    for (size_t at = 0; at < bytes; at += SLOT_BYTES) {
        const size_t len = std::min(SLOT_BYTES, bytes - at);
        const int slot = r->next;
        r->next = (slot + 1) % SLOTS;
        if (r->in_flight[slot]) {                      // (also a slot an earlier call on another stream left in flight)
            RFQ_HIP(hipEventSynchronize(r->done[slot]));
            r->in_flight[slot] = false;
        }
        fill_slot(r->host[slot], src + at, len);
        RFQ_HIP(hipMemcpyAsync(dst + at, r->host[slot], len, hipMemcpyHostToDevice, s));
        RFQ_HIP(hipEventRecord(r->done[slot], s));
        r->in_flight[slot] = true;
    }
    return RFQ_OK;
}

int release_upload_rings()
{
    std::lock_guard<std::mutex> lock(ring_mutex);
    if (rings.empty()) return RFQ_OK;
    int current = 0;
    RFQ_HIP(hipGetDevice(&current));
    hipError_t first = hipSuccess;
    auto note = [&](hipError_t e) { if (first == hipSuccess) first = e; };
    for (auto &entry : rings) {
        Ring &r = entry.second;
        note(hipSetDevice(entry.first));
        for (int i = 0; i < SLOTS; i++) {
            if (r.in_flight[i]) note(hipEventSynchronize(r.done[i]));
            if (r.done[i]) note(hipEventDestroy(r.done[i]));
            if (r.host[i]) note(hipHostFree(r.host[i]));
        }
    }
    rings.clear();
    note(hipSetDevice(current));
    if (first != hipSuccess) return hip_fail(first, "rfq_release_temporaries (staging ring)");
    return RFQ_OK;
}

} // namespace rfq
