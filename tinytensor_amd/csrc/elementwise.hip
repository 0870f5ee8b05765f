// elementwise.hip — strided view -> dense copy (the `identity` op behind Tensor::contiguous()/clone(),
// tinytensor/tensor/tensor.cpp:583-596, CPU form tinytensor/tensor/backend/cpu/unary.cpp:26-58 with the
// index map of tinytensor/tensor/backend/common/util.h:18-34).  The GEMM kernels never need it (they
// read views in place); it exists for the callers around them (reshape of a non-dense view, conv's
// grad_output) and moves raw bytes, so one kernel per element size serves every dtype.
#include "common.h"

namespace ttamd {
namespace {

constexpr int kMaxDims = 8;
struct ViewDesc {
    int64_t shape[kMaxDims];
    int64_t stride[kMaxDims];
    int ndim;
};

template <typename W>
__global__ void __launch_bounds__(256) contiguous_kernel(const W *__restrict__ src, W *__restrict__ dst, ViewDesc v,
                                                        int64_t numel) {
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < numel; i += step) {
        int64_t rank = i, flat = 0;
        for (int d = v.ndim - 1; d >= 0; --d) {
            flat += (rank % v.shape[d]) * v.stride[d];
            rank /= v.shape[d];
        }
        dst[i] = src[flat];
    }
}

template <typename W>
ttamd_status launch_contiguous(const void *src, void *dst, const ViewDesc &v, int64_t numel, hipStream_t stream) {
    int64_t blocks = (numel + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    contiguous_kernel<W><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(static_cast<const W *>(src),
                                                                                       static_cast<W *>(dst), v, numel);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

extern "C" ttamd_status ttamd_contiguous(int device, ttamd_dtype dtype, int ndim, const int64_t *shape,
                                         const int64_t *stride, const void *data, int64_t offset, void *out,
                                         void *stream) {
    const size_t esz = dtype_size(dtype);
    if (esz == 0 || dtype < TTAMD_BOOL || dtype > TTAMD_F64) {
        set_error("contiguous: unknown dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    if (ndim < 0 || ndim > kMaxDims || (ndim > 0 && (!shape || !stride)) || offset < 0) {
        set_error("contiguous: ndim must be in [0,%d] with non-NULL shape/stride and offset >= 0", kMaxDims);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    ViewDesc v{};
    v.ndim = ndim;
    int64_t numel = 1;
    for (int d = 0; d < ndim; ++d) {
        if (shape[d] < 0 || stride[d] < 0) {
            set_error("contiguous: negative extent or stride in dimension %d", d);
            return TTAMD_ERR_INVALID_ARGUMENT;
        }
        v.shape[d] = shape[d];
        v.stride[d] = stride[d];
        numel *= shape[d];
    }
    if (ttamd_status s = use_device(device)) return s;
    if (numel == 0) return TTAMD_OK;
    if (!data || !out) {
        set_error("contiguous: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const char *src = static_cast<const char *>(data) + offset * static_cast<int64_t>(esz);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (esz) {
    case 1: return launch_contiguous<uint8_t>(src, out, v, numel, st);
    case 2: return launch_contiguous<uint16_t>(src, out, v, numel, st);
    case 4: return launch_contiguous<uint32_t>(src, out, v, numel, st);
    default: return launch_contiguous<uint64_t>(src, out, v, numel, st);
    }
}
