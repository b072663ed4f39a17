// Internal: the kernel behind Expression::rotaryPositionEmbedding.
#pragma once

#include "Utilities/Expression/Expression.h"
#include "Utilities/Expression/StampedEquation.h"

#include <cstdint>
#include <memory>
#include <optional>

namespace ThorImplementation {

// output = values with every pair of the rotary part of the head dimension turned by position * frequency(pair); the rest of
// the head dimension is copied.  `node` carries the ROPE parameters.  positionIds (any numeric dtype, one element per
// element of the sequence axis) replace coordinate + offset; effectiveLength (one element) replaces the extent of the sequence
// axis in the Dynamic-NTK and LongRoPE rules.  All tensors dense.  Kernel arguments: values, [ids], [length], output.
std::shared_ptr<StampedEquation> stampRotaryEmbedding(const Tensor& values, const std::optional<Tensor>& positionIds,
                                                      const std::optional<Tensor>& effectiveLength, const Tensor& output, const ExprNode& node,
                                                      int deviceNum);

// Elementwise work around the rotation that runs inside its kernel (reference: RoPE is one more operation of a fused kernel there,
// Utilities/Expression/CudaSourceEmitter.cpp:3538-3697): a prologue computes the rotated operand from tensors of its shape, an
// epilogue computes the stored element from the rotated value and further tensors of that shape.  Statements are the
// `const T tN = ...;` lines of a BodyEmitter; "@P<i>@" / "@E<i>@" stand for the loaded storage element of prologue / epilogue
// tensor i and "@R@" for the rotated value (held in the C type of `rotatedDType`, rounded to it as a separate kernel would have
// stored it).  Runtime scalars are kernel arguments `float s<slot>`.
struct RopeFusion {
    struct Piece {
        std::vector<Tensor> tensors;
        std::string statements;
        std::string value;      // prologue: fp32 expression of the operand as the rotation reads it; epilogue: the storage element to write
        bool contract = false;  // all-fp32 arithmetic: mul+add may fuse, as in the elementwise kernel that would have run it
    };
    std::optional<Piece> prologue, epilogue;
    std::vector<uint32_t> scalarSlots;
    std::vector<std::string> scalarNames;
    DataType operandDType = DataType::FP32;  // dtype the operand would have been stored in (with a prologue)
    DataType rotatedDType = DataType::FP32;  // dtype the rotation would have stored
    uint64_t extraFlopsPerElement = 0;
};
// `values` gives the shape (and, without a prologue, the data); `output` has the dtype the epilogue stores.
// Kernel arguments: prologue tensors (or values), [ids], [length], epilogue tensors, runtime scalars, output.
std::shared_ptr<StampedEquation> stampRotaryEmbedding(const Tensor& values, const std::optional<Tensor>& positionIds,
                                                      const std::optional<Tensor>& effectiveLength, const Tensor& output, const ExprNode& node,
                                                      int deviceNum, const RopeFusion& fusion);

}  // namespace ThorImplementation
