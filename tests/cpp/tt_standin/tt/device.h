// tt/device.h — TEST-SIDE STAND-IN (see tt/exception.h in this directory): Backend / Device with the `amd` value and
// kAMD that tinytensor_amd/host/adapter/patches/device.h.patch adds to the reference's include/tt/device.h.
#ifndef TT_STANDIN_DEVICE_H_
#define TT_STANDIN_DEVICE_H_

namespace tinytensor {

enum class Backend { cpu, amd };

struct Device {
    constexpr static auto AMD(int dev_id) -> Device { return {Backend::amd, dev_id}; }
    constexpr auto operator==(const Device &other) const -> bool { return backend == other.backend && id == other.id; }
    Backend backend;
    int id;
};

constexpr Device kCPU = Device{Backend::cpu, 0};
constexpr Device kAMD = Device{Backend::amd, 0};

}    // namespace tinytensor

#endif    // TT_STANDIN_DEVICE_H_
