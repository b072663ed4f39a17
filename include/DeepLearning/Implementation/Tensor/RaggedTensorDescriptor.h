// A ragged batch = packed values [maxTotalValues, D...] plus a row partition (reference:
// DeepLearning/Implementation/Tensor/RaggedTensorDescriptor.h:14-87).  Only ragged rank 1 exists.
#pragma once

#include "DeepLearning/Implementation/Tensor/RowPartitionDescriptor.h"

#include <vector>

namespace ThorImplementation {

class RaggedTensorDescriptor {
   public:
    RaggedTensorDescriptor() = default;
    RaggedTensorDescriptor(TensorDescriptor valuesDescriptor, RowPartitionDescriptor rowPartition, uint32_t raggedRank = 1)
        : valuesDescriptor(std::move(valuesDescriptor)), rowPartition(rowPartition), raggedRank(raggedRank) {
        validate();
    }
    RaggedTensorDescriptor(DataType valuesDataType, const std::vector<uint64_t>& trailingDimensions, uint64_t batchSize, uint64_t maxTotalValues,
                           DataType offsetsDataType = kDefaultRowPartitionOffsetDataType, uint32_t raggedRank = 1)
        : valuesDescriptor(valuesDataType, packedDimensions(maxTotalValues, trailingDimensions)),
          rowPartition(batchSize, maxTotalValues, offsetsDataType),
          raggedRank(raggedRank) {
        validate();
    }

    TensorDescriptor getValuesDescriptor() const { return valuesDescriptor; }
    TensorDescriptor getOffsetsDescriptor() const { return rowPartition.getOffsetsDescriptor(); }
    RowPartitionDescriptor getRowPartition() const { return rowPartition; }
    DataType getValuesDataType() const { return valuesDescriptor.getDataType(); }
    DataType getOffsetsDataType() const { return rowPartition.getOffsetsDataType(); }
    uint64_t getBatchSize() const { return rowPartition.getBatchSize(); }
    uint64_t getMaxTotalValues() const { return rowPartition.getMaxTotalValues(); }
    uint32_t getRaggedRank() const { return raggedRank; }
    std::vector<uint64_t> getValuesDimensions() const { return valuesDescriptor.getDimensions(); }
    std::vector<uint64_t> getTrailingDimensions() const {
        const std::vector<uint64_t> dims = valuesDescriptor.getDimensions();
        return std::vector<uint64_t>(dims.begin() + 1, dims.end());
    }

    bool operator==(const RaggedTensorDescriptor& rhs) const {
        return valuesDescriptor == rhs.valuesDescriptor && rowPartition == rhs.rowPartition && raggedRank == rhs.raggedRank;
    }
    bool operator!=(const RaggedTensorDescriptor& rhs) const { return !(*this == rhs); }

    std::string toString() const {
        return "RaggedTensorDescriptor(values=" + valuesDescriptor.toString() + ", " + rowPartition.toString() + ")";
    }

   private:
    static std::vector<uint64_t> packedDimensions(uint64_t maxTotalValues, const std::vector<uint64_t>& trailing) {
        if (maxTotalValues == 0) throw std::invalid_argument("Ragged values need a non-zero row capacity.");
        std::vector<uint64_t> dims{maxTotalValues};
        for (uint64_t d : trailing) {
            if (d == 0) throw std::invalid_argument("Ragged trailing dimensions must be non-zero.");
            dims.push_back(d);
        }
        return dims;
    }
    void validate() const {
        if (raggedRank != 1) throw std::invalid_argument("Only ragged rank 1 is supported.");
        const std::vector<uint64_t> dims = valuesDescriptor.getDimensions();
        if (dims.empty() || dims[0] != rowPartition.getMaxTotalValues()) {
            throw std::invalid_argument("Ragged values must have the row partition's capacity as their first dimension.");
        }
    }

    TensorDescriptor valuesDescriptor;
    RowPartitionDescriptor rowPartition;
    uint32_t raggedRank = 1;
};

}  // namespace ThorImplementation
