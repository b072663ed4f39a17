// Storage / compute dtype tokens.  The numeric values are part of the contract with callers and serialized graphs
// (reference: DeepLearning/Implementation/Tensor/DataType.h:7-27); the same values cross the C ABI as thorhip_dtype.
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>

namespace ThorImplementation {

enum class DataType : int {
    FP16 = 10,
    FP32 = 11,
    FP64 = 12,
    INT8 = 13,
    INT16 = 14,
    INT32 = 15,
    INT64 = 16,
    UINT8 = 17,
    UINT16 = 18,
    UINT32 = 19,
    UINT64 = 20,
    BOOLEAN = 21,
    FP8_E4M3 = 22,
    FP8_E5M2 = 23,
    BF16 = 24,
    TF32 = 25,  // compute-only token of the reference's GEMM path; never a storage dtype here
};

inline uint32_t dataTypeSizeInBytes(DataType dt) {
    switch (dt) {
        case DataType::FP8_E4M3:
        case DataType::FP8_E5M2:
        case DataType::INT8:
        case DataType::UINT8:
        case DataType::BOOLEAN:
            return 1;
        case DataType::FP16:
        case DataType::BF16:
        case DataType::INT16:
        case DataType::UINT16:
            return 2;
        case DataType::FP32:
        case DataType::INT32:
        case DataType::UINT32:
            return 4;
        case DataType::FP64:
        case DataType::INT64:
        case DataType::UINT64:
            return 8;
        default:
            throw std::invalid_argument("dataTypeSizeInBytes: not a storage dtype: " + std::to_string(static_cast<int>(dt)));
    }
}

inline const char* dataTypeName(DataType dt) {
    switch (dt) {
        case DataType::FP16: return "fp16";
        case DataType::FP32: return "fp32";
        case DataType::FP64: return "fp64";
        case DataType::INT8: return "int8";
        case DataType::INT16: return "int16";
        case DataType::INT32: return "int32";
        case DataType::INT64: return "int64";
        case DataType::UINT8: return "uint8";
        case DataType::UINT16: return "uint16";
        case DataType::UINT32: return "uint32";
        case DataType::UINT64: return "uint64";
        case DataType::BOOLEAN: return "boolean";
        case DataType::FP8_E4M3: return "fp8_e4m3";
        case DataType::FP8_E5M2: return "fp8_e5m2";
        case DataType::BF16: return "bf16";
        case DataType::TF32: return "tf32";
    }
    return "<invalid dtype>";
}

}  // namespace ThorImplementation
