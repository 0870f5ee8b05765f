// storage_amd.h
// Underlying storage of the AMD (MI355X, gfx950) backend: one device allocation of libttamd.
//
// Peer of the reference's StorageCUDA / DeviceMemory<T> (tinytensor/tensor/backend/cuda/storage_cuda.h,
// cuda/data_types.cuh:28-101), but untyped: a tensor's dtype travels with the Tensor (include/tt/tensor.h:235), and
// every entry point of the C ABI (include/ttamd.h) takes the dtype code next to the pointer.

#ifndef TINYTENSOR_STORAGE_AMD_H_
#define TINYTENSOR_STORAGE_AMD_H_

#include "tensor/storage_base.h"

#include <cstddef>

namespace tinytensor::amd {

class StorageAMD : public StorageBase {
public:
    // Allocates `bytes` on device `device_id` (at least one byte, so that an empty tensor still owns an address);
    // throws TTException when the device id is invalid or the allocation fails.
    StorageAMD(int device_id, std::size_t bytes);
    ~StorageAMD() override;

    StorageAMD(const StorageAMD &) = delete;
    StorageAMD(StorageAMD &&) = delete;
    auto operator=(const StorageAMD &) -> StorageAMD & = delete;
    auto operator=(StorageAMD &&) -> StorageAMD & = delete;

    void *ptr = nullptr;    // device pointer (ttamd_malloc)
    std::size_t bytes = 0;  // size of the allocation
    int device_id = 0;
};

}    // namespace tinytensor::amd

#endif    // TINYTENSOR_STORAGE_AMD_H_
