// Host half of the TypeConverter: argument checks, the stream-ordered host path and the hand-off to the GPU kernels
// through the C ABI (reference: Utilities/TensorOperations/DataTypeConversions/TypeConverter.cpp:58-101,899-942).
#include "Utilities/TensorOperations/DataTypeConversions/TypeConverter.h"

#include "DeepLearning/Implementation/Tensor/Tensor.h"
#include "Utilities/Common/ScopedGpu.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <type_traits>
#include <vector>

namespace ThorImplementation {

namespace {

// ---- software codecs for the storage types the host has no native type for ----------------------------------------
// Narrowing is one round-to-nearest-even step from a double that holds the source value exactly (every source type but
// 64-bit integers above 2^53 fits; those are far outside every narrow format's finite range, where only the
// saturate / overflow decision matters).
struct Format {
    int exponentBits, mantissaBits, bias;
    bool saturate;       // true: no infinities are produced, overflow clamps to maxFiniteCode
    uint32_t maxFiniteCode, nanCode;
};
constexpr Format kHalf{5, 10, 15, false, 0x7bff, 0x7fff};
constexpr Format kBrain{8, 7, 127, false, 0x7f7f, 0x7fff};
constexpr Format kE4m3{4, 3, 7, true, 0x7e, 0x7f};
constexpr Format kE5m2{5, 2, 15, true, 0x7b, 0x7f};

uint32_t encode(double value, const Format& f) {
    const uint32_t signBit = 1u << (f.exponentBits + f.mantissaBits);
    const uint32_t sign = std::signbit(value) ? signBit : 0u;
    if (std::isnan(value)) return f.saturate ? (sign | f.nanCode) : f.nanCode;
    const uint32_t infCode = ((1u << f.exponentBits) - 1u) << f.mantissaBits;
    const uint32_t overflowCode = f.saturate ? f.maxFiniteCode : infCode;
    double mag = std::fabs(value);
    if (std::isinf(mag)) return sign | overflowCode;
    if (mag == 0.0) return sign;
    int exponent = 0;
    (void)std::frexp(mag, &exponent);  // mag = m * 2^exponent, m in [0.5, 1)
    int unbiased = exponent - 1;       // mag in [2^unbiased, 2^(unbiased+1))
    const int minNormal = 1 - f.bias;
    // quantum = spacing of representable values around mag
    const int quantumExponent = (unbiased < minNormal ? minNormal : unbiased) - f.mantissaBits;
    const double scaled = std::ldexp(mag, -quantumExponent);  // exact: power-of-two scaling
    // nearbyint under the default rounding mode is round-half-to-even
    const double steps = std::nearbyint(scaled);
    if (steps == 0.0) return sign;
    uint64_t q = static_cast<uint64_t>(steps);
    uint64_t code;
    if (unbiased < minNormal) {
        code = q;  // subnormal (a carry into the first normal lands on the right code by construction)
    } else {
        code = (static_cast<uint64_t>(unbiased + f.bias - 1) << f.mantissaBits) + q;
    }
    if (code > f.maxFiniteCode) return sign | overflowCode;
    return sign | static_cast<uint32_t>(code);
}

double decode(uint32_t bits, const Format& f) {
    const uint32_t signBit = 1u << (f.exponentBits + f.mantissaBits);
    const bool negative = (bits & signBit) != 0;
    const uint32_t mag = bits & (signBit - 1u);
    const uint32_t e = mag >> f.mantissaBits, m = mag & ((1u << f.mantissaBits) - 1u);
    double v;
    if (f.saturate && f.exponentBits == 4) {
        if (mag == 0x7f) return negative ? -NAN : NAN;
    } else if (e == (1u << f.exponentBits) - 1u) {
        v = m ? NAN : INFINITY;
        return negative ? -v : v;
    }
    if (e == 0) {
        v = std::ldexp(static_cast<double>(m), 1 - f.bias - f.mantissaBits);
    } else {
        v = std::ldexp(static_cast<double>(m | (1u << f.mantissaBits)), static_cast<int>(e) - f.bias - f.mantissaBits);
    }
    return negative ? -v : v;
}

struct Fp16 { uint16_t bits; };
struct Bf16 { uint16_t bits; };
struct E4m3 { uint8_t bits; };
struct E5m2 { uint8_t bits; };
struct Bool8 { uint8_t bits; };

template <typename T> struct IsSoftFloat : std::false_type {};
template <> struct IsSoftFloat<Fp16> : std::true_type {};
template <> struct IsSoftFloat<Bf16> : std::true_type {};
template <> struct IsSoftFloat<E4m3> : std::true_type {};
template <> struct IsSoftFloat<E5m2> : std::true_type {};

template <typename T> const Format& formatOf();
template <> const Format& formatOf<Fp16>() { return kHalf; }
template <> const Format& formatOf<Bf16>() { return kBrain; }
template <> const Format& formatOf<E4m3>() { return kE4m3; }
template <> const Format& formatOf<E5m2>() { return kE5m2; }

// 64-bit integers beyond 2^53 are not exact in double; nudge the double so that it is never *on* a rounding boundary
// it did not start on (round-to-odd), which keeps the single narrow rounding step correct.
template <typename I>
double integerToStickyDouble(I v) {
    const double d = static_cast<double>(v);
    if constexpr (sizeof(I) < 8) {
        return d;
    } else {
        if (std::fabs(d) < 9007199254740992.0) return d;
        const long double exact = static_cast<long double>(v);
        if (static_cast<long double>(d) == exact) return d;
        uint64_t bits;
        std::memcpy(&bits, &d, 8);
        if (std::fabs(static_cast<long double>(d)) > std::fabs(exact)) bits -= 1;
        bits |= 1;
        double r;
        std::memcpy(&r, &bits, 8);
        return r;
    }
}

template <typename From>
double widenToDouble(From v) {
    if constexpr (IsSoftFloat<From>::value) {
        return decode(v.bits, formatOf<From>());
    } else if constexpr (std::is_same_v<From, Bool8>) {
        return v.bits ? 1.0 : 0.0;
    } else if constexpr (std::is_integral_v<From>) {
        return integerToStickyDouble(v);
    } else {
        return static_cast<double>(v);
    }
}

template <typename From, typename To>
To convertOne(From v) {
    if constexpr (IsSoftFloat<To>::value) {
        To out;
        out.bits = static_cast<decltype(out.bits)>(encode(widenToDouble(v), formatOf<To>()));
        return out;
    } else if constexpr (std::is_same_v<To, Bool8>) {
        Bool8 out;
        if constexpr (std::is_integral_v<From>) {
            out.bits = v != 0;
        } else {
            const double d = widenToDouble(v);
            out.bits = (d != 0.0) ? 1 : 0;
        }
        return out;
    } else if constexpr (std::is_integral_v<To>) {
        if constexpr (std::is_integral_v<From>) {
            return static_cast<To>(v);
        } else if constexpr (std::is_same_v<From, Bool8>) {
            return static_cast<To>(v.bits ? 1 : 0);
        } else {
            const double d = widenToDouble(v);  // C++ float -> integer: truncation toward zero
            if (std::isnan(d)) return To(0);
            if constexpr (std::is_signed_v<To>) {
                return static_cast<To>(static_cast<int64_t>(d));
            } else {
                return d < 0 ? static_cast<To>(static_cast<int64_t>(d)) : static_cast<To>(static_cast<uint64_t>(d));
            }
        }
    } else {  // float / double destination
        if constexpr (IsSoftFloat<From>::value) {
            if constexpr (std::is_same_v<From, Fp16>) {
                // fp16 NaN widens to the canonical quiet NaN
                if ((v.bits & 0x7fffu) > 0x7c00u) {
                    if constexpr (std::is_same_v<To, float>) {
                        const uint32_t q = 0x7fffffffu;
                        float r;
                        std::memcpy(&r, &q, 4);
                        return r;
                    }
                }
            }
            if constexpr (std::is_same_v<From, Bf16> && std::is_same_v<To, float>) {
                const uint32_t b = static_cast<uint32_t>(v.bits) << 16;
                float r;
                std::memcpy(&r, &b, 4);
                return r;
            }
            return static_cast<To>(decode(v.bits, formatOf<From>()));
        } else if constexpr (std::is_same_v<From, Bool8>) {
            return static_cast<To>(v.bits ? 1 : 0);
        } else {
            return static_cast<To>(v);
        }
    }
}

template <typename From, typename To>
void convertSpan(const From* source, To* dest, long begin, long end, bool backward) {
    if (!backward) {
        for (long i = begin; i < end; ++i) dest[i] = convertOne<From, To>(source[i]);
    } else {
        for (long i = end - 1; i >= begin; --i) dest[i] = convertOne<From, To>(source[i]);
    }
}

// cpuConvertTypeImpl (TypeConverter.cpp:899-942): out of place or same-size in place -> static partition over
// numProcs = max(min(cores, n / 500000), 1) threads; in-place narrowing walks forward, in-place widening backward.
template <typename From, typename To>
void convertArray(const void* sourceV, void* destV, long n) {
    const From* source = static_cast<const From*>(sourceV);
    To* dest = static_cast<To*>(destV);
    const bool inPlace = sourceV == destV;
    if (!inPlace) {
        const char* sb = static_cast<const char*>(sourceV);
        const char* db = static_cast<const char*>(destV);
        if (sb < db + n * (long)sizeof(To) && db < sb + n * (long)sizeof(From)) {
            throw std::invalid_argument("TypeConverter: source and destination overlap without being the same buffer.");
        }
    }
    if (!inPlace || sizeof(From) == sizeof(To)) {
        const long cores = std::max(1u, std::thread::hardware_concurrency());
        const long procs = std::max(std::min(cores, n / 500000), 1L);
        if (procs > 1) {
            const long per = (n + procs - 1) / procs;
            std::vector<std::thread> workers;
            workers.reserve(procs);
            for (long t = 0; t < procs; ++t) {
                const long b = t * per, e = std::min(n, b + per);
                if (b < e) workers.emplace_back([=] { convertSpan<From, To>(source, dest, b, e, false); });
            }
            for (std::thread& w : workers) w.join();
        } else {
            convertSpan<From, To>(source, dest, 0, n, false);
        }
    } else {
        convertSpan<From, To>(source, dest, 0, n, sizeof(To) > sizeof(From));
    }
}

template <typename From>
void dispatchDest(const void* s, void* d, DataType to, long n) {
    switch (to) {
        case DataType::FP16: return convertArray<From, Fp16>(s, d, n);
        case DataType::BF16: return convertArray<From, Bf16>(s, d, n);
        case DataType::FP8_E4M3: return convertArray<From, E4m3>(s, d, n);
        case DataType::FP8_E5M2: return convertArray<From, E5m2>(s, d, n);
        case DataType::FP32: return convertArray<From, float>(s, d, n);
        case DataType::FP64: return convertArray<From, double>(s, d, n);
        case DataType::INT8: return convertArray<From, int8_t>(s, d, n);
        case DataType::INT16: return convertArray<From, int16_t>(s, d, n);
        case DataType::INT32: return convertArray<From, int32_t>(s, d, n);
        case DataType::INT64: return convertArray<From, int64_t>(s, d, n);
        case DataType::UINT8: return convertArray<From, uint8_t>(s, d, n);
        case DataType::UINT16: return convertArray<From, uint16_t>(s, d, n);
        case DataType::UINT32: return convertArray<From, uint32_t>(s, d, n);
        case DataType::UINT64: return convertArray<From, uint64_t>(s, d, n);
        case DataType::BOOLEAN: return convertArray<From, Bool8>(s, d, n);
        default: break;
    }
    throw std::invalid_argument(std::string("TypeConverter: unsupported destination dtype ") + dataTypeName(to));
}

struct RawArgs : HostFunctionArgsBase {
    const void* source;
    void* dest;
    DataType from, to;
    long n;
    Tensor keepSource, keepDest;
};

void hostCallback(void* raw) {
    RawArgs* a = static_cast<RawArgs*>(raw);
    TypeConverter::cpuConvertNow(a->source, a->dest, a->from, a->to, a->n);
}

}  // namespace

void TypeConverter::cpuConvertNow(const void* s, void* d, DataType from, DataType to, long n) {
    THOR_THROW_IF_FALSE(from != to);
    THOR_THROW_IF_FALSE(n >= 0);
    if (n == 0) return;
    switch (from) {
        case DataType::FP16: return dispatchDest<Fp16>(s, d, to, n);
        case DataType::BF16: return dispatchDest<Bf16>(s, d, to, n);
        case DataType::FP8_E4M3: return dispatchDest<E4m3>(s, d, to, n);
        case DataType::FP8_E5M2: return dispatchDest<E5m2>(s, d, to, n);
        case DataType::FP32: return dispatchDest<float>(s, d, to, n);
        case DataType::FP64: return dispatchDest<double>(s, d, to, n);
        case DataType::INT8: return dispatchDest<int8_t>(s, d, to, n);
        case DataType::INT16: return dispatchDest<int16_t>(s, d, to, n);
        case DataType::INT32: return dispatchDest<int32_t>(s, d, to, n);
        case DataType::INT64: return dispatchDest<int64_t>(s, d, to, n);
        case DataType::UINT8: return dispatchDest<uint8_t>(s, d, to, n);
        case DataType::UINT16: return dispatchDest<uint16_t>(s, d, to, n);
        case DataType::UINT32: return dispatchDest<uint32_t>(s, d, to, n);
        case DataType::UINT64: return dispatchDest<uint64_t>(s, d, to, n);
        case DataType::BOOLEAN: return dispatchDest<Bool8>(s, d, to, n);
        default: break;
    }
    throw std::invalid_argument(std::string("TypeConverter: unsupported source dtype ") + dataTypeName(from));
}

void TypeConverter::convertType(void* source, void* dest, DataType sourceDataType, DataType destDataType, long numElements,
                                Stream stream, int deviceNum) {
    THOR_THROW_IF_FALSE(sourceDataType != destDataType);
    THOR_THROW_IF_FALSE(numElements >= 0);
    if (numElements == 0) return;
    if (deviceNum == -1) {
        auto args = std::make_unique<RawArgs>();
        args->source = source;
        args->dest = dest;
        args->from = sourceDataType;
        args->to = destDataType;
        args->n = numElements;
        stream.enqueueHostFunction(&hostCallback, std::move(args));
        return;
    }
    THOR_THROW_IF_FALSE(stream.getGpuNum() == deviceNum);
    ScopedGpu scoped(deviceNum);
    THOR_HIP_CHECK(thorhip_convert(source, dest, static_cast<int>(sourceDataType), static_cast<int>(destDataType), numElements,
                                   stream.getStream()));
}

void TypeConverter::convertType(const Tensor& source, const Tensor& dest, DataType sourceDataType, DataType destDataType,
                                long numElements, Stream stream) {
    THOR_THROW_IF_FALSE(sourceDataType != destDataType);
    THOR_THROW_IF_FALSE(source.isInitialized() && dest.isInitialized());
    THOR_THROW_IF_FALSE(source.getPlacement().getMemDevice() == TensorPlacement::MemDevices::CPU);
    THOR_THROW_IF_FALSE(dest.getPlacement().getMemDevice() == TensorPlacement::MemDevices::CPU);
    THOR_THROW_IF_FALSE(numElements >= 0);
    if (numElements == 0) return;
    auto args = std::make_unique<RawArgs>();
    args->source = source.getMemPtr();
    args->dest = const_cast<Tensor&>(dest).getMemPtr();
    args->from = sourceDataType;
    args->to = destDataType;
    args->n = numElements;
    args->keepSource = source;
    args->keepDest = dest;
    stream.enqueueHostFunction(&hostCallback, std::move(args));
}

}  // namespace ThorImplementation
