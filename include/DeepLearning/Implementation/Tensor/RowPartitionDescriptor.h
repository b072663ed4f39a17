// Static description of a ragged batch's row partition: B rows packed into at most maxTotalValues value rows, delimited by
// B + 1 non-decreasing offsets held in a UINT32 (default) or UINT64 tensor (reference:
// DeepLearning/Implementation/Tensor/RowPartitionDescriptor.h:13-52, Utilities/TensorOperations/Ragged/RowPartitionDTypePolicy.h).
#pragma once

#include "DeepLearning/Implementation/Tensor/DataType.h"
#include "DeepLearning/Implementation/Tensor/TensorDescriptor.h"

#include <cstdint>
#include <limits>
#include <stdexcept>
#include <string>

namespace ThorImplementation {

inline constexpr DataType kDefaultRowPartitionOffsetDataType = DataType::UINT32;

inline constexpr bool isCanonicalRowPartitionOffsetDataType(DataType dtype) { return dtype == DataType::UINT32 || dtype == DataType::UINT64; }

inline constexpr bool canonicalRowPartitionOffsetCanRepresent(DataType dtype, uint64_t value) {
    return dtype == DataType::UINT64 || (dtype == DataType::UINT32 && value <= std::numeric_limits<uint32_t>::max());
}

class RowPartitionDescriptor {
   public:
    RowPartitionDescriptor() = default;
    RowPartitionDescriptor(uint64_t batchSize, uint64_t maxTotalValues, DataType offsetsDataType = kDefaultRowPartitionOffsetDataType)
        : batchSize(batchSize), maxTotalValues(maxTotalValues), offsetsDataType(offsetsDataType) {
        if (!isValidOffsetsDataType(offsetsDataType)) throw std::invalid_argument("Row partition offsets must use UINT32 or UINT64.");
        if (maxTotalValues == 0) throw std::invalid_argument("Row partition needs a non-zero value capacity.");
        if (!canonicalRowPartitionOffsetCanRepresent(offsetsDataType, maxTotalValues)) {
            throw std::invalid_argument("Row partition offsets dtype cannot represent the value capacity.");
        }
        if (batchSize + 1 <= batchSize) throw std::invalid_argument("Row partition batch size overflows the offsets element count.");
    }

    static bool isValidOffsetsDataType(DataType dataType) { return isCanonicalRowPartitionOffsetDataType(dataType); }

    uint64_t getBatchSize() const { return batchSize; }
    uint64_t getMaxTotalValues() const { return maxTotalValues; }
    DataType getOffsetsDataType() const { return offsetsDataType; }
    TensorDescriptor getOffsetsDescriptor() const { return TensorDescriptor(offsetsDataType, {batchSize + 1}); }

    bool operator==(const RowPartitionDescriptor& rhs) const {
        return batchSize == rhs.batchSize && maxTotalValues == rhs.maxTotalValues && offsetsDataType == rhs.offsetsDataType;
    }
    bool operator!=(const RowPartitionDescriptor& rhs) const { return !(*this == rhs); }

    std::string toString() const {
        return "RowPartitionDescriptor(batch_size=" + std::to_string(batchSize) + ", max_total_values=" + std::to_string(maxTotalValues) +
               ", offsets_data_type=" + dataTypeName(offsetsDataType) + ")";
    }

   private:
    uint64_t batchSize = 0;
    uint64_t maxTotalValues = 0;
    DataType offsetsDataType = kDefaultRowPartitionOffsetDataType;
};

}  // namespace ThorImplementation
