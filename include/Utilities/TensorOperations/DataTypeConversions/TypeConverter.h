// Storage dtype conversion between any two of the 15 tensor dtypes, on the host or on a GPU, in place or out of place
// (reference: Utilities/TensorOperations/DataTypeConversions/TypeConverter.h:20-46).
#pragma once

#include "DeepLearning/Implementation/Tensor/DataType.h"
#include "Utilities/Common/Stream.h"

namespace ThorImplementation {

class Tensor;

class TypeConverter {
   public:
    // Schedules dest[i] = static_cast<destDataType>(source[i]) at the back of `stream`.
    // deviceNum == -1: both pointers are host memory and the conversion runs inside a stream host callback (OpenMP,
    // numProcs = max(min(cores, numElements / 500000), 1)); the caller keeps the memory alive until the stream reaches
    // the callback.  deviceNum >= 0: both pointers are HBM of that GPU and `stream` must belong to it.
    // The two dtypes must differ.  source == dest converts in place; any other overlap is an error.
    static void convertType(void* source, void* dest, DataType sourceDataType, DataType destDataType, long numElements,
                            Stream stream, int deviceNum);

    // Host-tensor form: the callback keeps both tensors alive until it has run.
    static void convertType(const Tensor& source, const Tensor& dest, DataType sourceDataType, DataType destDataType,
                            long numElements, Stream stream);

    // Synchronous host conversion used by the callback above (exposed for host-side tests).
    static void cpuConvertNow(const void* source, void* dest, DataType sourceDataType, DataType destDataType, long numElements);

    static constexpr int THREADS_PER_UNSYNCED_BLOCK = 256;
};

}  // namespace ThorImplementation
