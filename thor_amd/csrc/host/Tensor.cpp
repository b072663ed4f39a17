#include "DeepLearning/Implementation/Tensor/Tensor.h"

#include "Utilities/Common/ScopedGpu.h"
#include "Utilities/TensorOperations/DataTypeConversions/TypeConverter.h"

#include <cstdlib>
#include <cstring>

namespace ThorImplementation {

std::atomic<uint64_t> Tensor::nextInstanceId{1};

namespace {
bool gpuAvailable() {
    static const bool available = [] {
        int n = 0;
        return thorhip_device_count(&n) == 0 && n > 0;
    }();
    return available;
}
}  // namespace

Tensor::BackingMemory::~BackingMemory() {
    if (mem == nullptr) return;
    if (placement.getMemDevice() == TensorPlacement::MemDevices::GPU) {
        int previous = 0;
        const bool known = thorhip_get_device(&previous) == 0;
        if (known && previous != placement.getDeviceNum()) (void)thorhip_set_device(placement.getDeviceNum());
        (void)thorhip_free(mem);
        if (known && previous != placement.getDeviceNum()) (void)thorhip_set_device(previous);
    } else if (pinned) {
        (void)thorhip_host_free(mem);
    } else {
        std::free(mem);
    }
}

Tensor::Tensor(TensorPlacement placement, TensorDescriptor descriptor, uint32_t alignmentBytes)
    : placement(placement), descriptor(descriptor) {
    THOR_THROW_IF_FALSE(placement.getMemDevice() != TensorPlacement::MemDevices::INVALID);
    THOR_THROW_IF_FALSE(descriptor.getTotalNumElements() > 0);
    Stream::drainFinishedHostCalls();  // release what finished copies kept alive before asking for more memory
    auto memory = std::make_shared<BackingMemory>();
    memory->placement = placement;
    const size_t bytes = descriptor.getArraySizeInBytes() + kTailPadBytes;
    if (placement.getMemDevice() == TensorPlacement::MemDevices::GPU) {
        ScopedGpu scoped(placement.getDeviceNum());
        const int rc = thorhip_malloc(&memory->mem, bytes);
        if (rc != 0) {
            throw std::runtime_error("Tensor allocation of " + descriptor.toString() + " on " + this->placement.toString() +
                                     " failed: " + thorhip_last_error());
        }
    } else if (gpuAvailable()) {
        THOR_HIP_CHECK(thorhip_host_malloc(&memory->mem, bytes));
        memory->pinned = true;
    } else {
        const size_t align = alignmentBytes > 256 ? alignmentBytes : 256;
        if (posix_memalign(&memory->mem, align, bytes) != 0) throw std::bad_alloc();
    }
    backingMemory = std::move(memory);
    storageNumElements = descriptor.getTotalNumElements();
    instanceId = nextInstanceId.fetch_add(1);
}

void* Tensor::viewPointer() const {
    THOR_THROW_IF_FALSE(isInitialized());
    return static_cast<char*>(backingMemory->mem) + storageElementOffset * dataTypeSizeInBytes(descriptor.getDataType());
}

std::vector<uint64_t> Tensor::getStridesElements() const {
    THOR_THROW_IF_FALSE(isInitialized());
    if (!customStridesElements.empty()) return customStridesElements;
    const std::vector<uint64_t>& dims = descriptor.getDimensions();
    std::vector<uint64_t> strides(dims.size(), 1);
    for (size_t i = dims.size(); i-- > 1;) strides[i - 1] = strides[i] * dims[i];
    return strides;
}

bool Tensor::isDenseContiguous() const {
    if (customStridesElements.empty()) return true;
    const std::vector<uint64_t>& dims = descriptor.getDimensions();
    uint64_t expected = 1;
    for (size_t i = dims.size(); i-- > 0;) {
        if (dims[i] != 1 && customStridesElements[i] != expected) return false;
        expected *= dims[i];
    }
    return true;
}

void Tensor::reshape(std::vector<uint64_t> dimensions) {
    THOR_THROW_IF_FALSE(isInitialized());
    THOR_THROW_IF_FALSE(isDenseContiguous());
    descriptor.reshape(dimensions);
    customStridesElements.clear();
}

Tensor Tensor::aliasView(std::vector<uint64_t> dimensions, std::vector<uint64_t> strides_elements, uint64_t element_offset) const {
    THOR_THROW_IF_FALSE(isInitialized());
    if (dimensions.empty() || dimensions.size() != strides_elements.size()) {
        throw std::invalid_argument("Tensor::aliasView requires one stride per dimension.");
    }
    // the last element the view reaches, every product and sum checked: strides that wrap around 2^64 must not slip past the
    // bounds test
    const char* outside = "Tensor::aliasView addresses elements outside the backing allocation.";
    uint64_t last = element_offset;
    for (size_t i = 0; i < dimensions.size(); ++i) {
        if (dimensions[i] == 0) throw std::invalid_argument("Tensor::aliasView does not support zero-sized dimensions.");
        uint64_t reach = 0;
        if (__builtin_mul_overflow(dimensions[i] - 1, strides_elements[i], &reach) || __builtin_add_overflow(last, reach, &last)) {
            throw std::invalid_argument(outside);
        }
    }
    uint64_t lastInStorage = 0;
    if (__builtin_add_overflow(storageElementOffset, last, &lastInStorage)) throw std::invalid_argument(outside);
    // storageNumElements is the element count of the whole allocation; views inherit it unchanged
    if (lastInStorage >= storageNumElements) {
        throw std::invalid_argument("Tensor::aliasView addresses elements outside the backing allocation.");
    }
    Tensor view = *this;
    view.descriptor = TensorDescriptor(getDataType(), dimensions);
    view.storageElementOffset = storageElementOffset + element_offset;
    view.customStridesElements = std::move(strides_elements);
    view.instanceId = nextInstanceId.fetch_add(1);
    if (view.isDenseContiguous()) view.customStridesElements.clear();
    return view;
}

void Tensor::memsetAsync(Stream stream, int8_t value, uint64_t numElements) {
    THOR_THROW_IF_FALSE(isInitialized() && isDenseContiguous());
    const uint64_t n = numElements == 0 ? getTotalNumElements() : numElements;
    THOR_THROW_IF_FALSE(n <= getTotalNumElements());
    const size_t bytes = n * dataTypeSizeInBytes(getDataType());
    if (placement.getMemDevice() == TensorPlacement::MemDevices::GPU) {
        THOR_HIP_CHECK(thorhip_memset_async(getMemPtr(), value, bytes, stream.getStream()));
    } else {
        stream.synchronize();
        std::memset(getMemPtr(), value, bytes);
    }
}

void Tensor::memset(int8_t value, uint64_t numElements) {
    THOR_THROW_IF_FALSE(isInitialized() && isDenseContiguous());
    const uint64_t n = numElements == 0 ? getTotalNumElements() : numElements;
    THOR_THROW_IF_FALSE(n <= getTotalNumElements());
    const size_t bytes = n * dataTypeSizeInBytes(getDataType());
    if (placement.getMemDevice() == TensorPlacement::MemDevices::GPU) {
        ScopedGpu scoped(placement.getDeviceNum());
        THOR_HIP_CHECK(thorhip_memset_async(getMemPtr(), value, bytes, nullptr));
        THOR_HIP_CHECK(thorhip_stream_synchronize(nullptr));
    } else {
        std::memset(getMemPtr(), value, bytes);
    }
}

Tensor Tensor::zeros(TensorPlacement placement, TensorDescriptor descriptor, Stream stream) {
    Tensor t(placement, descriptor);
    t.memsetAsync(stream, 0);
    return t;
}

namespace {
struct KeepAlive : HostFunctionArgsBase {
    std::vector<Tensor> tensors;
};
void releaseKeepAlive(void*) {}
}  // namespace

void Tensor::copyFromAsync(Tensor source, Stream stream) {
    THOR_THROW_IF_FALSE(isInitialized() && source.isInitialized());
    if (getTotalNumElements() != source.getTotalNumElements()) {
        throw std::invalid_argument("Tensor::copyFromAsync: element counts differ (" + source.dimensionsToString() + " -> " +
                                    dimensionsToString() + ").");
    }
    if (!isDenseContiguous() || !source.isDenseContiguous()) {
        throw std::invalid_argument("Tensor::copyFromAsync requires dense tensors.");
    }
    const bool srcGpu = source.placement.getMemDevice() == TensorPlacement::MemDevices::GPU;
    const bool dstGpu = placement.getMemDevice() == TensorPlacement::MemDevices::GPU;
    if (srcGpu && dstGpu && source.placement.getDeviceNum() != placement.getDeviceNum()) {
        throw std::invalid_argument("Tensor::copyFromAsync between two GPUs is outside this single-GPU backend.");
    }
    const long n = static_cast<long>(getTotalNumElements());
    const DataType srcType = source.getDataType(), dstType = getDataType();
    const size_t srcBytes = source.getArraySizeInBytes();

    if (srcType == dstType) {
        if (!srcGpu && !dstGpu) {
            stream.synchronize();
            std::memcpy(getMemPtr(), source.getMemPtr(), srcBytes);
            return;
        }
        const int kind = srcGpu ? (dstGpu ? THORHIP_D2D : THORHIP_D2H) : THORHIP_H2D;
        ScopedGpu scoped(stream.getGpuNum());
        THOR_HIP_CHECK(thorhip_memcpy_async(getMemPtr(), source.getMemPtr(), srcBytes, kind, stream.getStream()));
        return;
    }

    if (srcGpu && dstGpu) {
        TypeConverter::convertType(source.getMemPtr(), getMemPtr(), srcType, dstType, n, stream, placement.getDeviceNum());
        return;
    }
    if (!srcGpu && !dstGpu) {
        TypeConverter::convertType(source, *this, srcType, dstType, n, stream);
        return;
    }
    // One side on the GPU: move the raw bytes first, convert on the GPU, and keep the staging tensor alive until the
    // stream has passed the conversion.
    const int gpu = srcGpu ? source.placement.getDeviceNum() : placement.getDeviceNum();
    ScopedGpu scoped(gpu);
    auto keep = std::make_unique<KeepAlive>();
    if (!srcGpu) {
        Tensor staged(placement, TensorDescriptor(srcType, source.getDimensions()));
        THOR_HIP_CHECK(thorhip_memcpy_async(staged.getMemPtr(), source.getMemPtr(), srcBytes, THORHIP_H2D, stream.getStream()));
        TypeConverter::convertType(staged.getMemPtr(), getMemPtr(), srcType, dstType, n, stream, gpu);
        keep->tensors = {staged, source, *this};
    } else {
        Tensor staged(source.placement, TensorDescriptor(dstType, getDimensions()));
        TypeConverter::convertType(source.getMemPtr(), staged.getMemPtr(), srcType, dstType, n, stream, gpu);
        THOR_HIP_CHECK(thorhip_memcpy_async(getMemPtr(), staged.getMemPtr(), getArraySizeInBytes(), THORHIP_D2H, stream.getStream()));
        keep->tensors = {staged, source, *this};
    }
    stream.enqueueHostFunction(&releaseKeepAlive, std::move(keep));
}

}  // namespace ThorImplementation
