// Internal-consistency checks.  A failed THOR_THROW_IF_FALSE raises std::logic_error with the source location, which
// is the error type the reference uses for "impossible" states (DeepLearning/Implementation/ThorError.h:11-48).
#pragma once

#include <stdexcept>
#include <string>

namespace ThorImplementation {

[[noreturn]] inline void throwLogicError(const char* condition, const char* file, int line) {
    throw std::logic_error(std::string("Thor check failed: ") + condition + " at " + file + ":" + std::to_string(line));
}

}  // namespace ThorImplementation

#define THOR_THROW_IF_FALSE(condition)                                                   \
    do {                                                                                 \
        if (!(condition)) ::ThorImplementation::throwLogicError(#condition, __FILE__, __LINE__); \
    } while (0)

#define THOR_UNREACHABLE() ::ThorImplementation::throwLogicError("unreachable code", __FILE__, __LINE__)
