// dtype + dimensions of a dense row-major array (reference: DeepLearning/Implementation/Tensor/TensorDescriptor.h:21-60).
#pragma once

#include "DeepLearning/Implementation/Tensor/DataType.h"
#include "DeepLearning/Implementation/ThorError.h"

#include <cstdint>
#include <string>
#include <vector>

namespace ThorImplementation {

class TensorDescriptor {
   public:
    TensorDescriptor() = default;
    TensorDescriptor(DataType dataType, const std::vector<uint64_t>& dimensions) : dataType(dataType), dimensions(dimensions) {
        THOR_THROW_IF_FALSE(!dimensions.empty());
        totalNumElements = 1;
        for (uint64_t d : dimensions) {
            THOR_THROW_IF_FALSE(d != 0);
            totalNumElements *= d;
        }
    }

    DataType getDataType() const { return dataType; }
    const std::vector<uint64_t>& getDimensions() const { return dimensions; }
    uint32_t getNumDimensions() const { return static_cast<uint32_t>(dimensions.size()); }
    uint64_t getTotalNumElements() const { return totalNumElements; }
    uint64_t getArraySizeInBytes() const { return totalNumElements * dataTypeSizeInBytes(dataType); }
    static uint64_t getArraySizeInBytes(uint64_t numElements, DataType dataType) { return numElements * dataTypeSizeInBytes(dataType); }
    static uint32_t getElementSizeInBytes(DataType dataType) { return dataTypeSizeInBytes(dataType); }
    static std::string getElementTypeName(DataType dataType) { return dataTypeName(dataType); }
    std::string getElementTypeName() const { return dataTypeName(dataType); }

    void reshape(const std::vector<uint64_t>& newDimensions) {
        uint64_t n = 1;
        for (uint64_t d : newDimensions) n *= d;
        THOR_THROW_IF_FALSE(!newDimensions.empty() && n == totalNumElements);
        dimensions = newDimensions;
    }

    bool operator==(const TensorDescriptor& other) const { return dataType == other.dataType && dimensions == other.dimensions; }
    bool operator!=(const TensorDescriptor& other) const { return !(*this == other); }

    std::string toString() const {
        std::string s = std::string(dataTypeName(dataType)) + "[";
        for (size_t i = 0; i < dimensions.size(); ++i) s += (i ? "," : "") + std::to_string(dimensions[i]);
        return s + "]";
    }

   private:
    DataType dataType = DataType::FP32;
    std::vector<uint64_t> dimensions;
    uint64_t totalNumElements = 0;
};

}  // namespace ThorImplementation
