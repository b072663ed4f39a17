// Expressions over a ragged batch: packed values [maxTotalValues, D...] plus one offsets expression [B + 1] that every derived
// expression shares (reference: Utilities/Expression/RaggedExpression.h:16-119).  Valuewise operations compose on the packed
// values and stay fusable; getValues() wraps the result in a runtime-extent marker, so the kernel that produces it computes
// the first offsets[B] rows only and leaves the unused capacity of its output untouched.  Per-segment reductions return dense
// [B, D...] expressions.
//
// Differences from the reference on this backend: segment_softmax / segment_log_softmax use the segment maximum and sum
// broadcast back over the rows for scalar values too (the reference runs segmented scans there; the values agree to fp32
// rounding); RaggedExpressionRuntimeExtent carries no activeValueCount expression (the kernels read offsets[B] themselves).
#pragma once

#include "DeepLearning/Implementation/Tensor/RaggedTensorDescriptor.h"
#include "Utilities/Expression/Expression.h"

#include <cstdint>
#include <functional>
#include <set>
#include <string>
#include <vector>

namespace ThorImplementation {

struct RaggedExpressionRuntimeExtent {
    uint64_t maxActiveValues = 0;
    uint64_t elementsPerValue = 1;
    bool isInitialized() const { return maxActiveValues != 0 && elementsPerValue != 0; }
    uint64_t maxLaunchElements() const;
};

class RaggedExpression {
   public:
    RaggedExpression() = default;
    RaggedExpression(Expression values, Expression offsets, RaggedTensorDescriptor descriptor);

    // inputs "<name>.values" and "<name>.offsets"
    static RaggedExpression input(const std::string& logical_name, const RaggedTensorDescriptor& descriptor);
    static RaggedExpression input(const std::string& values_name, const std::string& offsets_name, const RaggedTensorDescriptor& descriptor);

    bool isInitialized() const { return initialized; }
    const Expression& getValues() const;   // with the runtime-extent marker: what to name as an output
    const Expression& getOffsets() const;
    const RaggedTensorDescriptor& getDescriptor() const;
    const RaggedExpressionRuntimeExtent& getRuntimeExtent() const;

    DataType getValuesDataType() const { return getDescriptor().getValuesDataType(); }
    DataType getOffsetsDataType() const { return getDescriptor().getOffsetsDataType(); }
    uint64_t getBatchSize() const { return getDescriptor().getBatchSize(); }
    uint64_t getMaxTotalValues() const { return getDescriptor().getMaxTotalValues(); }
    std::vector<uint64_t> getValuesDimensions() const { return getDescriptor().getValuesDimensions(); }
    std::vector<uint64_t> getTrailingDimensions() const { return getDescriptor().getTrailingDimensions(); }

    std::set<std::string> getInputNames() const;
    std::set<std::string> getMetadataInputNames() const;
    std::set<std::string> getDifferentiableInputNames() const;

    // new values over the same row partition (the descriptor may change dtype and trailing shape)
    RaggedExpression withValues(Expression new_values, RaggedTensorDescriptor new_descriptor) const;
    // any shape-preserving function of the unwrapped packed values
    RaggedExpression mapValues(const std::function<Expression(const Expression&)>& mapper) const;
    // [start, start + length) of one trailing axis, as a strided view of the packed values: consecutive slices compose into
    // one view of the original storage (reference: RaggedExpression.cpp:143-203 there).  The values have to resolve to a
    // dense tensor (an input or a stored value).
    RaggedExpression sliceTrailingDimension(uint64_t trailing_axis, uint64_t start, uint64_t length) const;
    RaggedExpression sliceLastDimension(uint64_t start, uint64_t length) const;
    RaggedExpression cast(DataType output_dtype) const;

    RaggedExpression operator+(const RaggedExpression& other) const;
    RaggedExpression operator-(const RaggedExpression& other) const;
    RaggedExpression operator*(const RaggedExpression& other) const;
    RaggedExpression operator/(const RaggedExpression& other) const;
    RaggedExpression equal(const RaggedExpression& other) const;
    RaggedExpression notEqual(const RaggedExpression& other) const;
    RaggedExpression lessThan(const RaggedExpression& other) const;
    RaggedExpression lessEqual(const RaggedExpression& other) const;
    RaggedExpression greaterThan(const RaggedExpression& other) const;
    RaggedExpression greaterEqual(const RaggedExpression& other) const;

    RaggedExpression abs() const;
    RaggedExpression exp() const;
    RaggedExpression ln() const;
    RaggedExpression log() const { return ln(); }
    RaggedExpression relu() const;

    RaggedExpression softmax() const { return segment_softmax(); }
    Expression reduce_sum() const { return segment_sum(); }
    Expression segment_sum() const;
    Expression segment_min() const;
    Expression segment_max() const;
    Expression segment_mean() const;
    RaggedExpression segment_softmax() const;
    RaggedExpression segment_log_softmax() const;

   private:
    enum class Comparison { Equal, NotEqual, Less, LessEqual, Greater, GreaterEqual };
    void requireInitialized(const char* caller) const;
    void requireCompatible(const RaggedExpression& other, const char* caller) const;
    uint64_t elementsPerValue() const;
    Expression segmentReduction(ExprOp op) const;
    Expression overRows(const Expression& per_segment_values, bool normalize_by_segment_length) const;
    RaggedExpression compare(const RaggedExpression& other, Comparison which, const char* caller) const;
    RaggedExpression shiftedExponentials(Expression& shifted) const;

    // a slice remembers the storage it views, so that the next slice re-views that storage with composed strides
    struct SliceOrigin {
        Expression source = Expression::constantScalar(0.0);
        std::vector<uint64_t> strides;
        uint64_t offset = 0;
        bool valid = false;
    };
    SliceOrigin sliceOrigin;

    Expression values = Expression::constantScalar(0.0);           // what ragged operations compose on
    Expression executionValues = Expression::constantScalar(0.0);  // values under the runtime-extent marker
    Expression offsets = Expression::constantScalar(0.0);
    RaggedTensorDescriptor descriptor;
    RaggedExpressionRuntimeExtent runtimeExtent;
    bool initialized = false;
};

RaggedExpression cast(const RaggedExpression& input, DataType output_dtype);
RaggedExpression abs(const RaggedExpression& input);
RaggedExpression exp(const RaggedExpression& input);
RaggedExpression log(const RaggedExpression& input);
RaggedExpression relu(const RaggedExpression& input);
Expression segment_sum(const RaggedExpression& input);
Expression segment_min(const RaggedExpression& input);
Expression segment_max(const RaggedExpression& input);
Expression segment_mean(const RaggedExpression& input);
RaggedExpression segment_softmax(const RaggedExpression& input);
RaggedExpression segment_log_softmax(const RaggedExpression& input);

}  // namespace ThorImplementation
