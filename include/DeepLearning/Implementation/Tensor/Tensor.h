// Tensor: a shared-ownership handle of a dense (or strided-view) array in host memory or GPU HBM
// (reference: DeepLearning/Implementation/Tensor/Tensor.h:54-264, Tensor.cpp:221-299,617-660,731-866).
//
// Copies of a handle share one allocation; view metadata (descriptor, element offset, custom strides) belongs to the
// handle.  Every allocation carries 128 spare bytes after the payload, as the reference's does, although no kernel of
// this backend reads or writes past the last element.
#pragma once

#include "DeepLearning/Implementation/Tensor/TensorDescriptor.h"
#include "DeepLearning/Implementation/Tensor/TensorPlacement.h"
#include "Utilities/Common/Stream.h"

#include <atomic>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

namespace ThorImplementation {

class Tensor {
   public:
    Tensor() = default;
    Tensor(TensorPlacement placement, TensorDescriptor descriptor, uint32_t alignmentBytes = 0);
    virtual ~Tensor() = default;

    bool isInitialized() const { return backingMemory != nullptr; }

    Tensor clone() const { return isInitialized() ? Tensor(placement, descriptor) : Tensor(); }
    Tensor clone(TensorPlacement newPlacement) const { return isInitialized() ? Tensor(newPlacement, descriptor) : Tensor(); }
    Tensor clone(DataType newDataType) const {
        return isInitialized() ? Tensor(placement, TensorDescriptor(newDataType, descriptor.getDimensions())) : Tensor();
    }
    Tensor clone(TensorPlacement newPlacement, DataType newDataType) const {
        return isInitialized() ? Tensor(newPlacement, TensorDescriptor(newDataType, descriptor.getDimensions())) : Tensor();
    }
    Tensor clone(std::vector<uint64_t> newDimensions) const {
        return isInitialized() ? Tensor(placement, TensorDescriptor(getDataType(), newDimensions)) : Tensor();
    }

    TensorPlacement getPlacement() const { return placement; }
    TensorDescriptor getDescriptor() const { return descriptor; }
    uint64_t getTensorId() const { return isInitialized() ? instanceId : 0; }

    // Address of the view's first element (the storage offset is already applied).
    template <typename ElementDataType = void>
    ElementDataType* getMemPtr() {
        return static_cast<ElementDataType*>(viewPointer());
    }
    template <typename ElementDataType = void>
    const ElementDataType* getMemPtr() const {
        return static_cast<const ElementDataType*>(viewPointer());
    }

    // Copies (and converts, when the dtypes differ) `source` into this tensor at the back of `stream`.  Both tensors
    // must be dense; host<->device, device<->device on one GPU and host<->host are supported.
    void copyFromAsync(Tensor source, Stream stream);

    static Tensor zeros(TensorPlacement placement, TensorDescriptor descriptor, Stream stream);

    void memset(int8_t value, uint64_t numElements = 0);
    void memsetAsync(Stream stream, int8_t value, uint64_t numElements = 0);
    void fillZero(Stream stream) { memsetAsync(stream, 0); }
    void dropReference() { *this = Tensor(); }

    void reshape(std::vector<uint64_t> dimensions);
    [[nodiscard]] Tensor aliasView(std::vector<uint64_t> dimensions, std::vector<uint64_t> strides_elements,
                                   uint64_t element_offset = 0) const;
    [[nodiscard]] bool hasCustomStrides() const { return !customStridesElements.empty(); }
    [[nodiscard]] bool isDenseContiguous() const;
    [[nodiscard]] uint64_t getStorageElementOffset() const { return storageElementOffset; }
    [[nodiscard]] std::vector<uint64_t> getStridesElements() const;

    bool operator==(const Tensor& other) const { return instanceId == other.instanceId; }
    bool operator!=(const Tensor& other) const { return instanceId != other.instanceId; }
    bool operator<(const Tensor& other) const { return instanceId < other.instanceId; }

    DataType getDataType() const {
        THOR_THROW_IF_FALSE(isInitialized());
        return descriptor.getDataType();
    }
    std::vector<uint64_t> getDimensions() const {
        THOR_THROW_IF_FALSE(isInitialized());
        return descriptor.getDimensions();
    }
    uint32_t getNumDimensions() const {
        THOR_THROW_IF_FALSE(isInitialized());
        return descriptor.getNumDimensions();
    }
    uint64_t getTotalNumElements() const {
        THOR_THROW_IF_FALSE(isInitialized());
        return descriptor.getTotalNumElements();
    }
    uint64_t getArraySizeInBytes() const {
        THOR_THROW_IF_FALSE(isInitialized());
        return descriptor.getArraySizeInBytes();
    }
    std::string dimensionsToString() const { return descriptor.toString(); }

    static constexpr uint64_t kTailPadBytes = 128;

   private:
    struct BackingMemory {
        TensorPlacement placement;
        void* mem = nullptr;
        bool pinned = false;
        ~BackingMemory();
    };

    void* viewPointer() const;

    TensorPlacement placement;
    TensorDescriptor descriptor;
    std::shared_ptr<BackingMemory> backingMemory;
    uint64_t storageElementOffset = 0;
    uint64_t storageNumElements = 0;
    std::vector<uint64_t> customStridesElements;
    uint64_t instanceId = 0;

    static std::atomic<uint64_t> nextInstanceId;
};

}  // namespace ThorImplementation
