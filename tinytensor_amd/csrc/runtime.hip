// runtime.hip — device selection, storage, copies, events and error text of libttamd.
// GPU peer of tinytensor's DeviceMemory<T> (cuda/data_types.cuh:28-101) and launch helper
// (cuda/kernel_launch.cuh:19-29), written for HIP on gfx950 only.
#include "common.h"

#include <atomic>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>

namespace ttamd {

namespace {
thread_local char g_error[512] = "no error";
constexpr int kMaxDevices = 64;
std::atomic<uint64_t> g_current[kMaxDevices];
std::atomic<uint64_t> g_total[kMaxDevices];
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
    std::lock_guard<std::mutex> lock(mu);
    Buf &b = bufs[{device, stream}];
    if (b.bytes < bytes) {
        size_t want = bytes < (size_t(4) << 20) ? (size_t(4) << 20) : bytes;
        want = (want + 255) & ~size_t(255);
        void *p = nullptr;
        hipError_t e = hipMalloc(&p, want);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            set_error("Unable to allocate %zu bytes of scratch on AMD device %d: %s", want, device, hipGetErrorString(e));
            return TTAMD_ERR_OUT_OF_MEMORY;
        }
        if (b.ptr) TTAMD_HIP_CHECK(hipFree(b.ptr));  // waits for kernels that may still read the old buffer
        b.ptr = p;
        b.bytes = want;
    }
    *out = b.ptr;
    return TTAMD_OK;
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

ttamd_status ttamd_malloc(int device, size_t bytes, void **out) {
    if (!out) {
        set_error("ttamd_malloc: out is NULL");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    *out = nullptr;
    if (ttamd_status s = use_device(device)) return s;
    if (bytes == 0) return TTAMD_OK;
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_error("Unable to allocate %zu bytes on AMD device %d: %s", bytes, device, hipGetErrorString(e));
        return TTAMD_ERR_OUT_OF_MEMORY;
    }
    g_current[device] += bytes;
    g_total[device] += bytes;
    *out = p;
    return TTAMD_OK;
}

ttamd_status ttamd_free(int device, void *ptr, size_t bytes) {
    if (!ptr) return TTAMD_OK;
    if (ttamd_status s = use_device(device)) return s;
    TTAMD_HIP_CHECK(hipFree(ptr));  // synchronous, like ~DeviceMemory (cuda/data_types.cu:102-116)
    g_current[device] -= bytes;
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
    TTAMD_HIP_CHECK(hipDeviceSynchronize());
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
