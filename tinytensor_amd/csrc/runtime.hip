// runtime.hip — device selection, storage, copies, events and error text of libttamd.
// GPU peer of tinytensor's DeviceMemory<T> (cuda/data_types.cuh:28-101) and launch helper
// (cuda/kernel_launch.cuh:19-29), written for HIP on gfx950 only.
#include "common.h"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <unordered_map>
#include <utility>
#include <vector>

namespace ttamd {

namespace {
thread_local char g_error[512] = "no error";
std::atomic<uint64_t> g_current[kMaxDevices];
std::atomic<uint64_t> g_total[kMaxDevices];

// Caching allocator.  Every backend operation allocates its result, and hipMalloc + hipFree cost 25-70 us per pair
// (hipFree also waits for the device), several times the run time of the small kernels between them.  Freed
// blocks are therefore kept per device, by rounded size, and handed out again; they go back to the driver on
// ttamd_empty_cache, when an allocation fails, and never otherwise.
//
// A cached block may still be read or written by kernels that were enqueued before it was freed.  Each block
// therefore remembers the streams it was used on -- the one it was allocated for and the one it was freed for -- and
// is handed out again
//   * to a request for one of those streams at once (stream order makes that safe; the reference's model, where one
//     stream carries all work of a device, cuda/kernel_launch.cuh:19-29, only ever takes this road),
//   * to a request for another stream only after an event recorded on each of its streams has completed (the event is
//     recorded when the block is first considered for such a request, which is later than the free and so covers it),
//   * to anyone once the whole device has been synchronised after the free (ttamd_device_synchronize,
//     ttamd_empty_cache).
// While the requesting stream is being captured into a graph only the first and the last road are open: no events
// are recorded or queried during a capture.
struct CachedBlock {
    void *ptr = nullptr;
    int n_streams = 0;
    hipStream_t stream[2] = {nullptr, nullptr};
    hipEvent_t event[2] = {nullptr, nullptr};  // recorded lazily, see above
    uint64_t epoch = 0;                        // the device's synchronisation count when the block was freed
};
struct LiveBlock {
    size_t rounded = 0;
    hipStream_t stream = nullptr;  // the stream the block was allocated for
};
// Tag of a live block whose allocation stream has been released (ttamd_stream_release) in the meantime.
const hipStream_t kNoStream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(1));
struct BlockCache {
    std::mutex mu;
    std::multimap<size_t, CachedBlock> free_blocks;  // rounded size -> block
    std::unordered_map<void *, LiveBlock> live;       // block -> rounded size, allocation stream
    uint64_t cached_bytes = 0;
    std::atomic<uint64_t> epoch{0};                   // bumped when a whole-device synchronisation starts
    std::atomic<uint64_t> synced{0};                  // blocks freed at an epoch below this are idle: a synchronisation
                                                      // that started after their free has completed
};
BlockCache g_cache[kMaxDevices];

bool cache_enabled() {
    static const bool on = [] {
        const char *e = std::getenv("TTAMD_ALLOC_CACHE");
        return !(e && e[0] == '0');
    }();
    return on;
}

// Size classes: multiples of 512 bytes up to 4 KiB, then eight classes per power of two (at most 12.5 % slack).
size_t round_block(size_t bytes) {
    if (bytes <= 4096) return (bytes + 511) & ~size_t(511);
    size_t p = 4096;
    while (p < bytes) p <<= 1;       // smallest power of two >= bytes
    const size_t step = p >> 4;      // p/2 < bytes <= p: eight steps of p/16 above p/2
    return (bytes + step - 1) / step * step;
}

void drop_events(CachedBlock &b) {
    for (int i = 0; i < 2; ++i)
        if (b.event[i]) {
            (void)hipEventDestroy(b.event[i]);
            b.event[i] = nullptr;
        }
}

void release_cached(int device) {
    BlockCache &c = g_cache[device];
    for (auto &kv : c.free_blocks) {
        drop_events(kv.second);
        (void)hipFree(kv.second.ptr);
    }
    c.free_blocks.clear();
    c.cached_bytes = 0;
}

bool is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
        (void)hipGetLastError();
        return true;  // an unusable stream handle: take the conservative road
    }
    return status != hipStreamCaptureStatusNone;
}

// May the cached block be handed to a request for `stream` now?  `may_use_events`: the requesting stream is not under
// capture, so events on the block's other streams may be recorded and queried.
bool reusable(CachedBlock &b, hipStream_t stream, uint64_t synced_epoch, bool may_use_events) {
    if (b.epoch < synced_epoch) return true;  // the device has been synchronised since the free
    for (int i = 0; i < b.n_streams; ++i) {
        if (b.stream[i] == stream) continue;  // stream order
        if (!may_use_events) return false;
        if (!b.event[i]) {
            if (is_capturing(b.stream[i])) return false;  // an event recorded there would become a graph node
            hipEvent_t ev = nullptr;
            if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
                (void)hipGetLastError();
                return false;
            }
            if (hipEventRecord(ev, b.stream[i]) != hipSuccess) {  // e.g. the stream has been destroyed since
                (void)hipGetLastError();
                (void)hipEventDestroy(ev);
                return false;  // only a whole-device synchronisation releases this block
            }
            b.event[i] = ev;
        }
        if (hipEventQuery(b.event[i]) != hipSuccess) {
            (void)hipGetLastError();  // hipErrorNotReady: work enqueued before the free may still be running
            return false;
        }
    }
    return true;
}
}  // namespace

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

ttamd_status use_device(int device) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess) {
        (void)hipGetLastError();
        count = 0;
    }
    if (device < 0 || device >= count || device >= kMaxDevices) {
        set_error("Invalid device id %d: %d AMD device(s) visible", device, count);
        return TTAMD_ERR_INVALID_DEVICE;
    }
    TTAMD_HIP_CHECK(hipSetDevice(device));
    return TTAMD_OK;
}

ttamd_status stream_scratch(int device, hipStream_t stream, size_t bytes, void **out) {
    struct Buf {
        void *ptr = nullptr;
        size_t bytes = 0;
    };
    static std::mutex mu;
    static std::map<std::pair<int, hipStream_t>, Buf> bufs;  // lives until the process ends
    static std::vector<void *> retired;                       // outgrown buffers, see below
    std::lock_guard<std::mutex> lock(mu);
    Buf &b = bufs[{device, stream}];
    if (b.bytes < bytes) {
        size_t want = bytes < (size_t(4) << 20) ? (size_t(4) << 20) : bytes;
        if (want < 2 * b.bytes) want = 2 * b.bytes;
        want = (want + 255) & ~size_t(255);
        void *p = nullptr;
        hipError_t e = hipMalloc(&p, want);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            set_error("Unable to allocate %zu bytes of scratch on AMD device %d: %s", want, device, hipGetErrorString(e));
            return TTAMD_ERR_OUT_OF_MEMORY;
        }
        // The old buffer is kept until the process ends: kernels in flight may still use it, and a captured graph has
        // its address baked in and may be replayed at any time.  Growth at least doubles the size, so all retired
        // buffers of a stream together stay below its current one.
        if (b.ptr) retired.push_back(b.ptr);
        b.ptr = p;
        b.bytes = want;
    }
    *out = b.ptr;
    return TTAMD_OK;
}

uint64_t device_sync_started(int device) {
    return device >= 0 && device < kMaxDevices ? g_cache[device].epoch.load() : 0;
}
uint64_t device_sync_completed(int device) {
    return device >= 0 && device < kMaxDevices ? g_cache[device].synced.load() : 0;
}

}  // namespace ttamd

using namespace ttamd;

namespace {
// Zero fill as a kernel rather than a memset node, so that callers may capture it in a HIP graph.
__global__ void __launch_bounds__(256) zero_fill_kernel(uint32_t *dst, size_t n_words, uint8_t *tail, int n_tail) {
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n_words; i += stride) dst[i] = 0u;
    if (blockIdx.x == 0 && static_cast<int>(threadIdx.x) < n_tail) tail[threadIdx.x] = 0;
}
}  // namespace

extern "C" {

ttamd_status ttamd_device_count(int *count) {
    if (!count) {
        set_error("ttamd_device_count: count is NULL");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();  // "no device" is a count of 0, not a failure
        n = 0;
    }
    *count = n;
    return TTAMD_OK;
}

const char *ttamd_last_error_string(void) { return g_error; }

const char *ttamd_target_arch(void) { return "gfx950"; }

ttamd_status ttamd_malloc_on_stream(int device, size_t bytes, void *stream, void **out) {
    if (!out) {
        set_error("ttamd_malloc: out is NULL");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    *out = nullptr;
    if (ttamd_status s = use_device(device)) return s;
    if (bytes == 0) return TTAMD_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    void *p = nullptr;
    const bool cached = cache_enabled();
    const size_t want = cached ? round_block(bytes) : bytes;
    BlockCache &c = g_cache[device];
    if (cached) {
        std::lock_guard<std::mutex> lock(c.mu);
        const auto range = c.free_blocks.equal_range(want);
        if (range.first != range.second) {
            const uint64_t epoch = c.synced.load();
            auto hit = range.second;
            for (auto it = range.first; it != range.second && hit == range.second; ++it)  // stream order or synchronised: no HIP calls
                if (reusable(it->second, st, epoch, false)) hit = it;
            if (hit == range.second && !is_capturing(st))
                for (auto it = range.first; it != range.second && hit == range.second; ++it)
                    if (reusable(it->second, st, epoch, true)) hit = it;
            if (hit != range.second) {
                p = hit->second.ptr;
                drop_events(hit->second);
                c.free_blocks.erase(hit);
                c.cached_bytes -= want;
                c.live[p] = LiveBlock{want, st};
            }
        }
    }
    if (!p) {
        hipError_t e = hipMalloc(&p, want);
        if (e != hipSuccess && cached) {  // give the cached blocks back to the driver and try once more
            (void)hipGetLastError();
            if (hipDeviceSynchronize() == hipSuccess) {  // cached blocks may still be in use by enqueued kernels
                std::lock_guard<std::mutex> lock(c.mu);
                release_cached(device);
            }
            e = hipMalloc(&p, want);
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();
            set_error("Unable to allocate %zu bytes on AMD device %d: %s", bytes, device, hipGetErrorString(e));
            return TTAMD_ERR_OUT_OF_MEMORY;
        }
        if (cached) {
            std::lock_guard<std::mutex> lock(c.mu);
            c.live[p] = LiveBlock{want, st};
        }
    }
    g_current[device] += bytes;
    g_total[device] += bytes;
    *out = p;
    return TTAMD_OK;
}

ttamd_status ttamd_free_on_stream(int device, void *ptr, size_t bytes, void *stream) {
    if (!ptr) return TTAMD_OK;
    if (ttamd_status s = use_device(device)) return s;
    BlockCache &c = g_cache[device];
    bool kept = false;
    {
        std::lock_guard<std::mutex> lock(c.mu);
        auto it = c.live.find(ptr);
        if (it != c.live.end()) {  // a block of the caching allocator: keep it for the next request of its class
            CachedBlock b;
            b.ptr = ptr;
            if (it->second.stream != kNoStream) b.stream[b.n_streams++] = it->second.stream;  // (released since: nothing pending there)
            if (static_cast<hipStream_t>(stream) != it->second.stream) b.stream[b.n_streams++] = static_cast<hipStream_t>(stream);
            b.epoch = c.epoch.load();
            c.cached_bytes += it->second.rounded;
            c.free_blocks.emplace(it->second.rounded, b);
            c.live.erase(it);
            kept = true;
        }
    }
    if (!kept) TTAMD_HIP_CHECK(hipFree(ptr));  // synchronous, like ~DeviceMemory (cuda/data_types.cu:102-116)
    g_current[device] -= bytes;
    return TTAMD_OK;
}

ttamd_status ttamd_stream_release(int device, void *stream) {
    if (ttamd_status s = use_device(device)) return s;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!st) return TTAMD_OK;  // the default stream is never destroyed
    TTAMD_HIP_CHECK(hipStreamSynchronize(st));
    // Nothing of this stream's is pending any more: forget the handle, so that no later request touches it (it is about
    // to be destroyed).  Live blocks allocated for it count as allocated for no stream from here on; cached blocks
    // lose it from their list of streams to wait for.
    BlockCache &c = g_cache[device];
    std::lock_guard<std::mutex> lock(c.mu);
    for (auto &kv : c.live)
        if (kv.second.stream == st) kv.second.stream = kNoStream;
    for (auto &kv : c.free_blocks) {
        CachedBlock &b = kv.second;
        int n = 0;
        for (int i = 0; i < b.n_streams; ++i) {
            if (b.stream[i] == st) {
                if (b.event[i]) (void)hipEventDestroy(b.event[i]);
                continue;
            }
            b.stream[n] = b.stream[i];
            b.event[n] = b.event[i];
            ++n;
        }
        for (int i = n; i < 2; ++i) b.stream[i] = nullptr, b.event[i] = nullptr;
        b.n_streams = n;
    }
    return TTAMD_OK;
}

ttamd_status ttamd_malloc(int device, size_t bytes, void **out) { return ttamd_malloc_on_stream(device, bytes, nullptr, out); }

ttamd_status ttamd_free(int device, void *ptr, size_t bytes) { return ttamd_free_on_stream(device, ptr, bytes, nullptr); }

ttamd_status ttamd_empty_cache(int device) {
    if (ttamd_status s = use_device(device)) return s;
    if (ttamd_status s = ttamd_device_synchronize(device)) return s;  // cached blocks may still be in use by enqueued kernels
    BlockCache &c = g_cache[device];
    std::lock_guard<std::mutex> lock(c.mu);
    release_cached(device);
    return TTAMD_OK;
}

ttamd_status ttamd_memory_cached(int device, uint64_t *cached_bytes) {
    if (ttamd_status s = use_device(device)) return s;
    if (cached_bytes) {
        BlockCache &c = g_cache[device];
        std::lock_guard<std::mutex> lock(c.mu);
        *cached_bytes = c.cached_bytes;
    }
    return TTAMD_OK;
}

ttamd_status ttamd_memory_allocated(int device, uint64_t *current_bytes, uint64_t *total_bytes) {
    if (ttamd_status s = use_device(device)) return s;
    if (current_bytes) *current_bytes = g_current[device].load();
    if (total_bytes) *total_bytes = g_total[device].load();
    return TTAMD_OK;
}

ttamd_status ttamd_memcpy_h2d(int device, void *dst_device, const void *src_host, size_t bytes) {
    if (bytes == 0) return TTAMD_OK;
    if (!dst_device || !src_host) {
        set_error("ttamd_memcpy_h2d: NULL pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    TTAMD_HIP_CHECK(hipMemcpy(dst_device, src_host, bytes, hipMemcpyHostToDevice));
    return TTAMD_OK;
}

ttamd_status ttamd_memcpy_d2h(int device, void *dst_host, const void *src_device, size_t bytes) {
    if (bytes == 0) return TTAMD_OK;
    if (!dst_host || !src_device) {
        set_error("ttamd_memcpy_d2h: NULL pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    TTAMD_HIP_CHECK(hipMemcpy(dst_host, src_device, bytes, hipMemcpyDeviceToHost));
    return TTAMD_OK;
}

ttamd_status ttamd_memset_zero(int device, void *dst_device, size_t bytes, void *stream) {
    if (bytes == 0) return TTAMD_OK;
    if (!dst_device) {
        set_error("ttamd_memset_zero: NULL pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    if (reinterpret_cast<uintptr_t>(dst_device) % 4 != 0) {
        set_error("ttamd_memset_zero: destination must be 4-byte aligned");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const size_t n_words = bytes / 4;
    const int n_tail = static_cast<int>(bytes % 4);
    size_t blocks = (n_words + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (blocks == 0) blocks = 1;
    zero_fill_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<uint32_t *>(dst_device), n_words, static_cast<uint8_t *>(dst_device) + n_words * 4, n_tail);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

ttamd_status ttamd_device_synchronize(int device) {
    if (ttamd_status s = use_device(device)) return s;
    // Blocks freed before this point are idle afterwards, whatever stream used them.  The epoch moves on before the
    // wait, so a block freed while the wait is in progress carries the new epoch and is not released by it.
    BlockCache &c = g_cache[device];
    const uint64_t mine = ++c.epoch;
    TTAMD_HIP_CHECK(hipDeviceSynchronize());
    uint64_t seen = c.synced.load();
    while (seen < mine && !c.synced.compare_exchange_weak(seen, mine)) {
    }
    return TTAMD_OK;
}

ttamd_status ttamd_event_create(int device, void **event) {
    if (!event) {
        set_error("ttamd_event_create: event is NULL");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (ttamd_status s = use_device(device)) return s;
    hipEvent_t e;
    TTAMD_HIP_CHECK(hipEventCreate(&e));
    *event = e;
    return TTAMD_OK;
}

ttamd_status ttamd_event_destroy(void *event) {
    if (!event) return TTAMD_OK;
    TTAMD_HIP_CHECK(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return TTAMD_OK;
}

ttamd_status ttamd_event_record(void *event, void *stream) {
    if (!event) {
        set_error("ttamd_event_record: event is NULL");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    TTAMD_HIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
    return TTAMD_OK;
}

ttamd_status ttamd_event_elapsed_ms(void *start, void *stop, float *ms) {
    if (!start || !stop || !ms) {
        set_error("ttamd_event_elapsed_ms: NULL argument");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    TTAMD_HIP_CHECK(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
    TTAMD_HIP_CHECK(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return TTAMD_OK;
}

}  // extern "C"
