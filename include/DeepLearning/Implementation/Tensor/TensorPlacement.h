// Where a tensor's memory lives: host memory or the HBM of GPU `deviceNum`
// (reference: DeepLearning/Implementation/Tensor/TensorPlacement.h:9-38).
#pragma once

#include "DeepLearning/Implementation/ThorError.h"

#include <string>

namespace ThorImplementation {

class TensorPlacement {
   public:
    enum class MemDevices { INVALID = 0, CPU, GPU };

    TensorPlacement() = default;
    explicit TensorPlacement(MemDevices device, int deviceNum = 0) : memDevice(device), deviceNum(deviceNum) {
        THOR_THROW_IF_FALSE(device == MemDevices::CPU || device == MemDevices::GPU);
        THOR_THROW_IF_FALSE(device == MemDevices::GPU || deviceNum == 0);
    }

    MemDevices getMemDevice() const { return memDevice; }
    int getDeviceNum() const { return deviceNum; }

    bool operator==(const TensorPlacement& other) const { return memDevice == other.memDevice && deviceNum == other.deviceNum; }
    bool operator!=(const TensorPlacement& other) const { return !(*this == other); }

    std::string toString() const {
        THOR_THROW_IF_FALSE(memDevice != MemDevices::INVALID);
        return memDevice == MemDevices::CPU ? std::string("CPU") : "GPU:" + std::to_string(deviceNum);
    }

   private:
    MemDevices memDevice = MemDevices::INVALID;
    int deviceNum = 0;
};

}  // namespace ThorImplementation
