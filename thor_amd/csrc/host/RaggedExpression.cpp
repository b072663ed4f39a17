#include "Utilities/Expression/RaggedExpression.h"

#include <limits>
#include <stdexcept>

namespace ThorImplementation {

namespace {

std::string prefix(const char* caller) { return std::string("RaggedExpression::") + caller + ": "; }

RaggedTensorDescriptor withValuesDataType(const RaggedTensorDescriptor& d, DataType dtype) {
    return RaggedTensorDescriptor(TensorDescriptor(dtype, d.getValuesDimensions()), d.getRowPartition(), d.getRaggedRank());
}

}  // namespace

uint64_t RaggedExpressionRuntimeExtent::maxLaunchElements() const {
    if (!isInitialized()) throw std::runtime_error("RaggedExpressionRuntimeExtent is not initialized.");
    if (elementsPerValue > std::numeric_limits<uint64_t>::max() / maxActiveValues) {
        throw std::invalid_argument("ragged expression runtime extent max launch elements overflows uint64_t.");
    }
    return maxActiveValues * elementsPerValue;
}

RaggedExpression::RaggedExpression(Expression values, Expression offsets, RaggedTensorDescriptor descriptor)
    : values(std::move(values)), offsets(std::move(offsets)), descriptor(std::move(descriptor)) {
    initialized = true;
    runtimeExtent.maxActiveValues = this->descriptor.getMaxTotalValues();
    runtimeExtent.elementsPerValue = elementsPerValue();
    executionValues = this->values.withRaggedRuntimeExtent(this->offsets, this->descriptor.getBatchSize(), runtimeExtent.maxActiveValues,
                                                           runtimeExtent.elementsPerValue);
}

RaggedExpression RaggedExpression::input(const std::string& logical_name, const RaggedTensorDescriptor& descriptor) {
    if (logical_name.empty()) throw std::invalid_argument("RaggedExpression::input requires a non-empty logical input name.");
    return input(logical_name + ".values", logical_name + ".offsets", descriptor);
}

RaggedExpression RaggedExpression::input(const std::string& values_name, const std::string& offsets_name, const RaggedTensorDescriptor& descriptor) {
    if (values_name.empty() || offsets_name.empty()) {
        throw std::invalid_argument("RaggedExpression::input requires non-empty values and offsets input names.");
    }
    return RaggedExpression(Expression::input(values_name, std::nullopt, descriptor.getValuesDataType()),
                            Expression::input(offsets_name, std::nullopt, descriptor.getOffsetsDataType()), descriptor);
}

void RaggedExpression::requireInitialized(const char* caller) const {
    if (!initialized) throw std::runtime_error(prefix(caller) + "ragged expression is not initialized.");
}

const Expression& RaggedExpression::getValues() const {
    requireInitialized("getValues");
    return executionValues;
}
const Expression& RaggedExpression::getOffsets() const {
    requireInitialized("getOffsets");
    return offsets;
}
const RaggedTensorDescriptor& RaggedExpression::getDescriptor() const {
    requireInitialized("getDescriptor");
    return descriptor;
}
const RaggedExpressionRuntimeExtent& RaggedExpression::getRuntimeExtent() const {
    requireInitialized("getRuntimeExtent");
    return runtimeExtent;
}

uint64_t RaggedExpression::elementsPerValue() const {
    uint64_t elements = 1;
    for (uint64_t d : descriptor.getTrailingDimensions()) {
        if (d != 0 && elements > std::numeric_limits<uint64_t>::max() / d) {
            throw std::invalid_argument("ragged expression elementsPerValue overflows uint64_t.");
        }
        elements *= d;
    }
    return elements;
}

std::set<std::string> RaggedExpression::getMetadataInputNames() const {
    requireInitialized("getMetadataInputNames");
    return offsets.getInputNames();
}

std::set<std::string> RaggedExpression::getInputNames() const {
    requireInitialized("getInputNames");
    std::set<std::string> names = executionValues.getInputNames();
    for (const std::string& n : getMetadataInputNames()) names.insert(n);
    return names;
}

std::set<std::string> RaggedExpression::getDifferentiableInputNames() const {
    requireInitialized("getDifferentiableInputNames");
    std::set<std::string> names = values.getInputNames();
    for (const std::string& n : getMetadataInputNames()) names.erase(n);
    return names;
}

RaggedExpression RaggedExpression::withValues(Expression new_values, RaggedTensorDescriptor new_descriptor) const {
    requireInitialized("withValues");
    if (new_descriptor.getRowPartition() != descriptor.getRowPartition()) {
        throw std::invalid_argument("RaggedExpression::withValues requires the row partition to be preserved.");
    }
    return RaggedExpression(std::move(new_values), offsets, std::move(new_descriptor));
}

RaggedExpression RaggedExpression::mapValues(const std::function<Expression(const Expression&)>& mapper) const {
    requireInitialized("mapValues");
    if (!mapper) throw std::invalid_argument("RaggedExpression::mapValues requires a valid mapper.");
    return withValues(mapper(values), descriptor);
}

RaggedExpression RaggedExpression::sliceTrailingDimension(uint64_t trailing_axis, uint64_t start, uint64_t length) const {
    requireInitialized("sliceTrailingDimension");
    const std::vector<uint64_t> trailing = descriptor.getTrailingDimensions();
    if (trailing_axis >= trailing.size()) throw std::invalid_argument("RaggedExpression::sliceTrailingDimension trailing axis is out of range.");
    if (length == 0) throw std::invalid_argument("RaggedExpression::sliceTrailingDimension requires a non-zero slice length.");
    if (start >= trailing[trailing_axis] || length > trailing[trailing_axis] - start) {
        throw std::invalid_argument("RaggedExpression::sliceTrailingDimension slice exceeds the source trailing dimension.");
    }
    std::vector<uint64_t> dims = descriptor.getValuesDimensions();
    // strides address storage, not the index space of an earlier view: a slice of a slice re-views the first slice's source
    SliceOrigin origin = sliceOrigin;
    if (!origin.valid) {
        origin.source = values;
        origin.strides.assign(dims.size(), 1);
        for (size_t a = dims.size() - 1; a-- > 0;) origin.strides[a] = origin.strides[a + 1] * dims[a + 1];
        origin.offset = 0;
        origin.valid = true;
    }
    origin.offset += start * origin.strides[trailing_axis + 1];
    dims[trailing_axis + 1] = length;
    RaggedExpression out = withValues(origin.source.stridedView(dims, origin.strides, origin.offset),
                                      RaggedTensorDescriptor(TensorDescriptor(descriptor.getValuesDataType(), dims), descriptor.getRowPartition(),
                                                             descriptor.getRaggedRank()));
    out.sliceOrigin = origin;
    return out;
}

RaggedExpression RaggedExpression::sliceLastDimension(uint64_t start, uint64_t length) const {
    requireInitialized("sliceLastDimension");
    const size_t rank = descriptor.getTrailingDimensions().size();
    if (rank == 0) throw std::invalid_argument("RaggedExpression::sliceLastDimension requires at least one trailing value dimension.");
    return sliceTrailingDimension(rank - 1, start, length);
}

RaggedExpression RaggedExpression::cast(DataType output_dtype) const {
    requireInitialized("cast");
    return withValues(values.cast(output_dtype), withValuesDataType(descriptor, output_dtype));
}

void RaggedExpression::requireCompatible(const RaggedExpression& other, const char* caller) const {
    requireInitialized(caller);
    other.requireInitialized(caller);
    if (!offsets.isSameLogicalNode(other.offsets)) {
        throw std::invalid_argument(prefix(caller) + "binary ragged valuewise ops require the exact same offsets expression object.");
    }
    if (descriptor.getRowPartition() != other.descriptor.getRowPartition()) throw std::invalid_argument(prefix(caller) + "ragged row partitions differ.");
    if (descriptor.getValuesDimensions() != other.descriptor.getValuesDimensions()) throw std::invalid_argument(prefix(caller) + "ragged values shapes differ.");
    if (descriptor.getValuesDataType() != other.descriptor.getValuesDataType()) throw std::invalid_argument(prefix(caller) + "ragged values dtypes differ.");
}

RaggedExpression RaggedExpression::operator+(const RaggedExpression& other) const {
    requireCompatible(other, "operator+");
    return withValues(values + other.values, descriptor);
}
RaggedExpression RaggedExpression::operator-(const RaggedExpression& other) const {
    requireCompatible(other, "operator-");
    return withValues(values - other.values, descriptor);
}
RaggedExpression RaggedExpression::operator*(const RaggedExpression& other) const {
    requireCompatible(other, "operator*");
    return withValues(values * other.values, descriptor);
}
RaggedExpression RaggedExpression::operator/(const RaggedExpression& other) const {
    requireCompatible(other, "operator/");
    return withValues(values / other.values, descriptor);
}

RaggedExpression RaggedExpression::compare(const RaggedExpression& other, Comparison which, const char* caller) const {
    requireCompatible(other, caller);
    Expression result = values;
    switch (which) {
        case Comparison::Equal: result = values.equal(other.values); break;
        case Comparison::NotEqual: result = values.notEqual(other.values); break;
        case Comparison::Less: result = values.lessThan(other.values); break;
        case Comparison::LessEqual: result = values.lessEqual(other.values); break;
        case Comparison::Greater: result = values.greaterThan(other.values); break;
        case Comparison::GreaterEqual: result = values.greaterEqual(other.values); break;
    }
    return withValues(result, withValuesDataType(descriptor, DataType::BOOLEAN));
}
RaggedExpression RaggedExpression::equal(const RaggedExpression& o) const { return compare(o, Comparison::Equal, "equal"); }
RaggedExpression RaggedExpression::notEqual(const RaggedExpression& o) const { return compare(o, Comparison::NotEqual, "notEqual"); }
RaggedExpression RaggedExpression::lessThan(const RaggedExpression& o) const { return compare(o, Comparison::Less, "lessThan"); }
RaggedExpression RaggedExpression::lessEqual(const RaggedExpression& o) const { return compare(o, Comparison::LessEqual, "lessEqual"); }
RaggedExpression RaggedExpression::greaterThan(const RaggedExpression& o) const { return compare(o, Comparison::Greater, "greaterThan"); }
RaggedExpression RaggedExpression::greaterEqual(const RaggedExpression& o) const { return compare(o, Comparison::GreaterEqual, "greaterEqual"); }

RaggedExpression RaggedExpression::abs() const {
    requireInitialized("abs");
    return withValues(values.abs(), descriptor);
}
RaggedExpression RaggedExpression::exp() const {
    requireInitialized("exp");
    return withValues(values.exp(), descriptor);
}
RaggedExpression RaggedExpression::ln() const {
    requireInitialized("ln");
    return withValues(values.ln(), descriptor);
}
RaggedExpression RaggedExpression::relu() const {
    requireInitialized("relu");
    return withValues(values.max(Expression::constantScalar(0.0)), descriptor);
}

Expression RaggedExpression::segmentReduction(ExprOp op) const {
    return Expression::segmentedReduceWithRaggedMetadata(values, offsets, op, descriptor.getBatchSize(), descriptor.getMaxTotalValues(),
                                                         elementsPerValue());
}
Expression RaggedExpression::segment_sum() const {
    requireInitialized("segment_sum");
    return segmentReduction(ExprOp::SEGMENTED_REDUCE_SUM);
}
Expression RaggedExpression::segment_min() const {
    requireInitialized("segment_min");
    return segmentReduction(ExprOp::SEGMENTED_REDUCE_MIN);
}
Expression RaggedExpression::segment_max() const {
    requireInitialized("segment_max");
    return segmentReduction(ExprOp::SEGMENTED_REDUCE_MAX);
}
Expression RaggedExpression::segment_mean() const {
    requireInitialized("segment_mean");
    switch (descriptor.getValuesDataType()) {
        case DataType::FP8_E4M3:
        case DataType::FP8_E5M2:
        case DataType::FP16:
        case DataType::BF16:
        case DataType::FP32:
            break;
        default:
            throw std::invalid_argument("RaggedExpression::segment_mean requires floating-point ragged values.");
    }
    return segmentReduction(ExprOp::SEGMENTED_REDUCE_MEAN);
}

Expression RaggedExpression::overRows(const Expression& per_segment_values, bool normalize_by_segment_length) const {
    return Expression::segmentedBroadcast(per_segment_values, offsets, descriptor.getBatchSize(), descriptor.getMaxTotalValues(), elementsPerValue(),
                                          normalize_by_segment_length);
}

// exp(x - max of x's segment) as a ragged expression; `shifted` receives x - max
RaggedExpression RaggedExpression::shiftedExponentials(Expression& shifted) const {
    shifted = values - overRows(segment_max(), false);
    return withValues(shifted.exp(), descriptor);
}

RaggedExpression RaggedExpression::segment_softmax() const {
    requireInitialized("segment_softmax");
    Expression shifted = values;
    const RaggedExpression exponentials = shiftedExponentials(shifted);
    return withValues(exponentials.values / overRows(exponentials.segment_sum(), false), descriptor);
}

RaggedExpression RaggedExpression::segment_log_softmax() const {
    requireInitialized("segment_log_softmax");
    Expression shifted = values;
    const RaggedExpression exponentials = shiftedExponentials(shifted);
    return withValues(shifted - overRows(exponentials.segment_sum(), false).ln(), descriptor);
}

RaggedExpression cast(const RaggedExpression& input, DataType output_dtype) { return input.cast(output_dtype); }
RaggedExpression abs(const RaggedExpression& input) { return input.abs(); }
RaggedExpression exp(const RaggedExpression& input) { return input.exp(); }
RaggedExpression log(const RaggedExpression& input) { return input.log(); }
RaggedExpression relu(const RaggedExpression& input) { return input.relu(); }
Expression segment_sum(const RaggedExpression& input) { return input.segment_sum(); }
Expression segment_min(const RaggedExpression& input) { return input.segment_min(); }
Expression segment_max(const RaggedExpression& input) { return input.segment_max(); }
Expression segment_mean(const RaggedExpression& input) { return input.segment_mean(); }
RaggedExpression segment_softmax(const RaggedExpression& input) { return input.segment_softmax(); }
RaggedExpression segment_log_softmax(const RaggedExpression& input) { return input.segment_log_softmax(); }

}  // namespace ThorImplementation
