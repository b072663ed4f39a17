#include "Utilities/Expression/ExpressionDTypeResolution.h"

#include <stdexcept>

namespace ThorImplementation {

namespace {

bool isComparison(ExprOp op) { return op >= ExprOp::EQUAL && op <= ExprOp::GREATER_EQUAL; }
bool isLogical(ExprOp op) { return op == ExprOp::LOGICAL_AND || op == ExprOp::LOGICAL_OR || op == ExprOp::LOGICAL_NOT; }
bool isShapeOnly(ExprOp op) { return op == ExprOp::RESHAPE || op == ExprOp::UNSQUEEZE || op == ExprOp::SQUEEZE || isStorageViewOp(op); }
bool isScalarLeaf(ExprOp op) { return op == ExprOp::SCALAR_FP || op == ExprOp::RUNTIME_SCALAR || op == ExprOp::TENSOR_RUNTIME_SCALAR; }

bool isBindableInputDType(DataType dtype) {
    switch (dtype) {
        case DataType::BOOLEAN:
        case DataType::UINT8:
        case DataType::INT8:
        case DataType::UINT16:
        case DataType::INT16:
        case DataType::UINT32:
        case DataType::INT32:
        case DataType::UINT64:
        case DataType::INT64:
            return true;
        default:
            return isSupportedFusionFloatingType(dtype);
    }
}

void rejectUnsupportedOp(ExprOp op) {
    if (isRaggedOp(op) || isStorageViewOp(op) || isWinnerRoutingOp(op) || op == ExprOp::TAKE_ALONG_AXIS || op == ExprOp::ROPE || isScatterRoutingOp(op) || isScanOp(op)) return;
    if (Expression::isLeafOp(op) || Expression::isUnaryOp(op) || Expression::isBinaryOp(op) || Expression::isTernaryOp(op)) return;
    throw std::runtime_error("Expression op '" + opName(op) + "' is outside the elementwise / reduction / cast path of this backend.");
}

std::vector<DataType> tensorParentDTypes(const ExprNode& node, const std::vector<ExprNode>& nodes, const std::vector<DataType>& resolved) {
    std::vector<DataType> out;
    if (isRaggedOp(node.op)) return {resolved.at(node.lhs)};  // the offsets are structure, not a value
    if (isWinnerRoutingOp(node.op) || node.op == ExprOp::TAKE_ALONG_AXIS || node.op == ExprOp::ROPE || isScatterRoutingOp(node.op) || isScanOp(node.op)) return {resolved.at(node.lhs)};
    auto add = [&](uint32_t parent) {
        if (parent >= nodes.size()) throw std::runtime_error("Parent node index out of range during dtype resolution.");
        if (!isScalarLeaf(nodes[parent].op)) out.push_back(resolved[parent]);
    };
    if (!Expression::isLeafOp(node.op)) add(node.lhs);
    if (Expression::isBinaryOp(node.op) || Expression::isTernaryOp(node.op)) add(node.rhs);
    if (Expression::isTernaryOp(node.op)) add(node.aux);
    return out;
}

DataType promoteWhereBranches(const std::vector<DataType>& dtypes) {
    if (dtypes.empty()) return DataType::FP32;
    bool same = true, floating = true;
    for (DataType d : dtypes) {
        same = same && d == dtypes.front();
        floating = floating && isSupportedFusionFloatingType(d);
    }
    if (same) return dtypes.front();
    if (floating) return promoteTensorValueDTypes(dtypes);
    throw std::runtime_error("Where branch dtypes must either match exactly or be supported floating dtypes.");
}

const char* raggedOpLabel(ExprOp op) {
    if (op == ExprOp::SEGMENTED_BROADCAST) return "segmented-broadcast";
    if (op == ExprOp::RAGGED_VALUEWISE_EXTENT) return "ragged valuewise extent";
    return "segmented-reduction";
}

// Reference rules (Utilities/Expression/ExpressionDTypeResolution.cpp:635-646,705-733 there): offsets are UINT32 / UINT64, the
// result has the values' dtype, and segmented reductions / broadcasts take floating-point values only.
DataType raggedOutputDType(const ExprNode& node, const std::vector<DataType>& resolved) {
    const DataType offsets = resolved.at(node.rhs);
    if (offsets != DataType::UINT32 && offsets != DataType::UINT64) {
        throw std::runtime_error(std::string(raggedOpLabel(node.op)) + " offsets must have UINT32 or UINT64 dtype, received: " + dataTypeName(offsets));
    }
    const DataType values = resolved.at(node.lhs);
    if (node.op == ExprOp::RAGGED_VALUEWISE_EXTENT) return node.output_dtype.value_or(values);
    if (!isSupportedFusionFloatingType(values)) {
        throw std::runtime_error(std::string("Unsupported ") + raggedOpLabel(node.op) + " dtype: " + dataTypeName(values));
    }
    if (node.output_dtype.has_value() && node.output_dtype.value() != values) {
        throw std::runtime_error(std::string("Expression ") + (node.op == ExprOp::SEGMENTED_BROADCAST ? "segmented broadcast" : "segmented reduction") +
                                 " currently requires output dtype to match input dtype.");
    }
    return values;
}

DataType nodeOutputDType(const ExprNode& node, const std::vector<ExprNode>& nodes, const std::vector<DataType>& resolved) {
    if (isRaggedOp(node.op)) return raggedOutputDType(node, resolved);
    if (isScanOp(node.op)) {
        // values keep their dtype, arg scans return flattened UINT32 indices; offsets are structure
        const DataType in = resolved[node.lhs];
        if (in != DataType::UINT32 && in != DataType::FP16 && in != DataType::BF16 && in != DataType::FP32) {
            throw std::runtime_error(std::string("Expression scan requires UINT32, FP16, BF16 or FP32 values, received: ") + dataTypeName(in));
        }
        if (node.op == ExprOp::SEGMENTED_SCAN && resolved[node.rhs] != DataType::UINT32 && resolved[node.rhs] != DataType::UINT64) {
            throw std::runtime_error(std::string("Expression segmented-scan offsets must have UINT32 or UINT64 dtype, received: ") +
                                     dataTypeName(resolved[node.rhs]));
        }
        const DataType out = isArgScanOp(node.scan_op) ? DataType::UINT32 : in;
        if (node.output_dtype.has_value() && node.output_dtype.value() != out) {
            throw std::runtime_error("Expression scan output dtype is fixed by its input (UINT32 for arg scans).");
        }
        return out;
    }
    if (node.op == ExprOp::TAKE_ALONG_AXIS) {
        const DataType indexType = resolved[node.rhs];
        if (indexType != DataType::UINT32 && indexType != DataType::UINT64) {
            throw std::runtime_error(std::string("take_along_axis indices must have UINT32 or UINT64 dtype, received: ") + dataTypeName(indexType));
        }
        return node.output_dtype.value_or(resolved[node.lhs]);
    }
    if (node.op == ExprOp::STRIDED_VIEW_BACKWARD) {
        if (resolved[node.lhs] != DataType::FP32) throw std::runtime_error("Strided view backward requires an FP32 gradient.");
        if (node.output_dtype.has_value() && node.output_dtype.value() != DataType::FP32) throw std::runtime_error("Strided view backward produces FP32.");
        return DataType::FP32;
    }
    if (isSegmentWinnerRoutingOp(node.op)) {
        if (!isSupportedFusionFloatingType(resolved[node.lhs])) throw std::runtime_error("Segmented min/max backward requires floating-point values.");
        if (resolved[node.rhs] != DataType::FP32) throw std::runtime_error("Segmented min/max backward requires an FP32 gradient.");
        if (node.output_dtype.has_value() && node.output_dtype.value() != DataType::FP32) throw std::runtime_error("Segmented min/max backward produces FP32.");
        return DataType::FP32;
    }
    if (isScanBackwardOp(node.op)) {
        const DataType in = resolved[node.lhs];
        if (in != DataType::UINT32 && in != DataType::FP16 && in != DataType::BF16 && in != DataType::FP32) {
            throw std::runtime_error(std::string("Expression scan requires UINT32, FP16, BF16 or FP32 values, received: ") + dataTypeName(in));
        }
        if (resolved[node.rhs] != DataType::FP32) throw std::runtime_error("Scan min/max backward requires an FP32 gradient.");
        if (node.output_dtype.has_value() && node.output_dtype.value() != DataType::FP32) {
            throw std::runtime_error("Scan min/max backward produces FP32.");
        }
        return DataType::FP32;
    }
    if (node.op == ExprOp::ROPE) {
        // fp32 arithmetic on stored values; the result keeps the operand's dtype unless the node names another
        const DataType out = node.output_dtype.value_or(resolved[node.lhs]);
        if (!isSupportedFusionFloatingType(resolved[node.lhs]) || !isSupportedFusionFloatingType(out)) {
            throw std::runtime_error("RoPE requires floating-point input and output dtypes.");
        }
        return out;
    }
    if (isWinnerRoutingOp(node.op)) {
        // the gradient of the reduced operand, in the operand's dtype unless the node names another
        const DataType out = node.output_dtype.value_or(resolved[node.lhs]);
        if (!isSupportedFusionFloatingType(out) || !isSupportedFusionFloatingType(resolved[node.rhs])) {
            throw std::runtime_error("Min/max reduction backward requires floating-point operand and gradient dtypes.");
        }
        return out;
    }
    if (isArgReductionOp(node.op)) return DataType::UINT32;
    if (isValueReductionOp(node.op)) {
        // fp32 accumulate and finalise, then one conversion to the requested storage dtype (fp32 unless overridden)
        const DataType out = node.output_dtype.value_or(DataType::FP32);
        if (!isSupportedFusionFloatingType(out)) {
            throw std::runtime_error(std::string("Dense floating-point reduction requested unsupported output dtype: ") + dataTypeName(out));
        }
        return out;
    }
    if (isComparison(node.op) || isLogical(node.op)) return node.output_dtype.value_or(DataType::BOOLEAN);
    if (node.op == ExprOp::SOFTMAX) {
        // the input's dtype, fp8 widened to fp16 (the reference's toSupportedInputDType for its softmax stage,
        // Utilities/Expression/ExpressionDTypeResolution.cpp:259-272)
        const DataType in = resolved[node.lhs];
        if (!isSupportedFusionFloatingType(in)) throw std::runtime_error("Softmax requires a floating-point input.");
        return node.output_dtype.value_or(isFp8Type(in) ? DataType::FP16 : in);
    }
    if (node.op == ExprOp::WHERE) {
        if (resolved[node.lhs] != DataType::BOOLEAN) {
            throw std::runtime_error(std::string("Where condition must have BOOLEAN dtype, received: ") + dataTypeName(resolved[node.lhs]));
        }
        std::vector<DataType> branches;
        if (!isScalarLeaf(nodes[node.rhs].op)) branches.push_back(resolved[node.rhs]);
        if (!isScalarLeaf(nodes[node.aux].op)) branches.push_back(resolved[node.aux]);
        return node.output_dtype.value_or(promoteWhereBranches(branches));
    }
    const std::vector<DataType> parents = tensorParentDTypes(node, nodes, resolved);
    const DataType fallback = parents.empty() ? DataType::FP32 : promoteTensorValueDTypes(parents);
    return node.output_dtype.value_or(fallback);
}

DataType nodeLogicalInputDType(const ExprNode& node, const std::vector<ExprNode>& nodes, const std::vector<DataType>& resolved) {
    if (node.op == ExprOp::SCALAR_FP || node.op == ExprOp::FILL) return node.output_dtype.value_or(DataType::FP32);
    if (node.op == ExprOp::CAST) return resolved[node.lhs];
    if (node.op == ExprOp::WHERE) {
        std::vector<DataType> branches;
        if (!isScalarLeaf(nodes[node.rhs].op)) branches.push_back(resolved[node.rhs]);
        if (!isScalarLeaf(nodes[node.aux].op)) branches.push_back(resolved[node.aux]);
        return promoteWhereBranches(branches);
    }
    const std::vector<DataType> parents = tensorParentDTypes(node, nodes, resolved);
    if (parents.empty()) return DataType::FP32;
    bool allFloating = true;
    for (DataType d : parents) allFloating = allFloating && isSupportedFusionFloatingType(d);
    if (allFloating) return promoteTensorValueDTypes(parents);
    // integer / boolean operands: identical dtypes stay, anything mixed is handled as fp32 arithmetic
    for (DataType d : parents)
        if (d != parents.front()) return DataType::FP32;
    return parents.front();
}

DataType widenRequiredCompute(ExprOp op, DataType current, DataType propagated) {
    if (op == ExprOp::CAST) return toSupportedComputeDType(op, current);
    if (isComparison(op) || isLogical(op) || op == ExprOp::WHERE) {
        if (isSupportedFusionFloatingType(current) && isSupportedFusionFloatingType(propagated)) {
            return toSupportedComputeDType(op, promoteTensorValueDTypes(current, propagated));
        }
        if (isSupportedFusionFloatingType(propagated)) return toSupportedComputeDType(op, propagated);
        return toSupportedComputeDType(op, current);
    }
    if (!isSupportedFusionFloatingType(current)) return current;
    return toSupportedComputeDType(op, promoteTensorValueDTypes(current, propagated));
}

void seed(std::optional<DataType>& slot, DataType dtype) {
    if (!isSupportedFusionFloatingType(dtype)) return;
    slot = slot.has_value() ? promoteTensorValueDTypes(*slot, dtype) : dtype;
}

// A materialised value's storage dtype flows upward as a lower bound on the compute dtype of what feeds it.
void propagateMaterialisedDTypes(PhysicalExpression& expr, const std::vector<uint32_t>& outputs, const std::vector<uint8_t>& explicitCompute) {
    std::vector<std::optional<DataType>> required(expr.nodes.size());
    for (uint32_t out : outputs) {
        const ExprNode& n = expr.nodes.at(out);
        if (n.compute_dtype) {
            seed(required[out], *n.compute_dtype);
        } else if (n.output_dtype) {
            seed(required[out], *n.output_dtype);
        }
    }
    for (uint32_t idx = static_cast<uint32_t>(expr.nodes.size()); idx-- > 0;) {
        if (!required[idx]) continue;
        ExprNode& node = expr.nodes[idx];
        DataType flowing = *required[idx];
        if (!Expression::isLeafOp(node.op) && node.compute_dtype) {
            if (!explicitCompute[idx]) node.compute_dtype = widenRequiredCompute(node.op, *node.compute_dtype, flowing);
            flowing = *node.compute_dtype;
        }
        auto toParent = [&](uint32_t p) { seed(required.at(p), flowing); };
        if (node.op == ExprOp::CAST) {
            // an explicit conversion boundary: the source keeps its own compute dtype
        } else if (node.op == ExprOp::RAGGED_VALUEWISE_EXTENT || node.op == ExprOp::SEGMENTED_BROADCAST) {
            toParent(node.lhs);  // never into the offsets
        } else if (isWinnerRoutingOp(node.op) || node.op == ExprOp::TAKE_ALONG_AXIS || node.op == ExprOp::ROPE || isScatterRoutingOp(node.op) || isScanOp(node.op)) {
            // the operands are read as stored tensors: nothing to widen
        } else if (isReductionOp(node.op) || node.op == ExprOp::SOFTMAX || isSegmentedReduceOp(node.op)) {
            // the reduction's mandatory fp32 stays inside the reduction; its producer keeps its own policy
            const ExprNode& producer = expr.nodes.at(node.lhs);
            if (producer.compute_dtype) {
                seed(required[node.lhs], *producer.compute_dtype);
            } else if (producer.output_dtype) {
                seed(required[node.lhs], *producer.output_dtype);
            }
        } else if (node.op == ExprOp::WHERE) {
            for (uint32_t p : {node.rhs, node.aux}) {
                const ExprNode& parent = expr.nodes.at(p);
                if (parent.output_dtype && isSupportedFusionFloatingType(*parent.output_dtype)) toParent(p);
            }
        } else {
            if (!Expression::isLeafOp(node.op)) toParent(node.lhs);
            if (Expression::isBinaryOp(node.op) || Expression::isTernaryOp(node.op)) toParent(node.rhs);
            if (Expression::isTernaryOp(node.op)) toParent(node.aux);
        }
    }
}

void resolveInPlace(PhysicalExpression& expr, const std::vector<DataType>& rootDTypes, const std::vector<uint32_t>& outputs) {
    std::vector<DataType> resolved(expr.nodes.size(), DataType::FP32);
    std::vector<uint8_t> explicitCompute(expr.nodes.size(), 0);
    for (size_t i = 0; i < expr.nodes.size(); ++i) explicitCompute[i] = expr.nodes[i].compute_dtype.has_value();

    for (uint32_t idx = 0; idx < expr.nodes.size(); ++idx) {
        ExprNode& node = expr.nodes[idx];
        rejectUnsupportedOp(node.op);
        if (node.op == ExprOp::INPUT || node.op == ExprOp::RUNTIME_SCALAR || node.op == ExprOp::TENSOR_RUNTIME_SCALAR) {
            if (node.input_slot >= rootDTypes.size()) throw std::runtime_error("Input slot out of range during dtype resolution.");
            const DataType actual = rootDTypes[node.input_slot];
            if (!isBindableInputDType(actual)) {
                throw std::runtime_error(std::string("Unsupported input dtype for a fused expression: ") + dataTypeName(actual));
            }
            node.input_tensor_dtype = actual;
            const DataType out = node.output_dtype.value_or(actual);
            DataType compute = out;
            if (isSupportedFusionFloatingType(actual) && isSupportedFusionFloatingType(out)) {
                compute = toSupportedComputeDType(node.op, node.compute_dtype.value_or(defaultComputeDType(actual, out)));
            } else if (node.compute_dtype) {
                compute = *node.compute_dtype;
            }
            node.output_dtype = out;
            node.compute_dtype = compute;
            resolved[idx] = out;
            continue;
        }
        const DataType out = nodeOutputDType(node, expr.nodes, resolved);
        const DataType logicalIn = nodeLogicalInputDType(node, expr.nodes, resolved);
        DataType requested;
        if (node.op == ExprOp::CAST || isShapeOnly(node.op) || node.op == ExprOp::RAGGED_VALUEWISE_EXTENT || node.op == ExprOp::SEGMENTED_BROADCAST ||
            isWinnerRoutingOp(node.op) || node.op == ExprOp::TAKE_ALONG_AXIS || node.op == ExprOp::ROPE || isScatterRoutingOp(node.op) || isScanOp(node.op)) {
            requested = out;  // values pass through unchanged (a normalised broadcast divides in fp32 and rounds once)
        } else if (isSegmentedReduceOp(node.op)) {
            requested = DataType::FP32;
        } else if (node.op == ExprOp::SOFTMAX) {
            requested = DataType::FP32;  // fp32 arithmetic whatever the storage
        } else if (node.op == ExprOp::SUB && (logicalIn == DataType::UINT32 || logicalIn == DataType::UINT64) && logicalIn == out) {
            requested = logicalIn;  // exact unsigned differences stay in the integer domain
        } else if (isComparison(node.op)) {
            if (node.compute_dtype) {
                requested = *node.compute_dtype;
            } else if (logicalIn == DataType::BOOLEAN || logicalIn == DataType::UINT8) {
                requested = DataType::BOOLEAN;
            } else if (isSupportedFusionFloatingType(logicalIn)) {
                requested = defaultComputeDType(logicalIn);
            } else {
                requested = DataType::FP32;
            }
        } else if (isLogical(node.op) || node.op == ExprOp::WHERE) {
            requested = node.compute_dtype.value_or(logicalIn);
            if (!isSupportedFusionFloatingType(requested) && requested != DataType::BOOLEAN && requested != DataType::UINT8) {
                requested = DataType::FP32;
            }
        } else if (node.compute_dtype) {
            requested = *node.compute_dtype;
        } else if (isSupportedFusionFloatingType(logicalIn) && isSupportedFusionFloatingType(out)) {
            requested = defaultComputeDType(logicalIn, out);
        } else {
            requested = DataType::FP32;  // integer-valued operands of float arithmetic are read as fp32
        }
        node.output_dtype = out;
        node.compute_dtype = toSupportedComputeDType(node.op, requested);
        resolved[idx] = out;
    }
    propagateMaterialisedDTypes(expr, outputs, explicitCompute);
}

}  // namespace

bool isSupportedFusionFloatingType(DataType dtype) {
    return dtype == DataType::FP8_E4M3 || dtype == DataType::FP8_E5M2 || dtype == DataType::FP16 || dtype == DataType::BF16 ||
           dtype == DataType::FP32;
}

bool isFp8Type(DataType dtype) { return dtype == DataType::FP8_E4M3 || dtype == DataType::FP8_E5M2; }

DataType promoteTensorValueDTypes(DataType a, DataType b) {
    if (a == b) return a;
    if (!isSupportedFusionFloatingType(a) || !isSupportedFusionFloatingType(b)) {
        throw std::runtime_error("Unsupported dtype in promoteTensorValueDTypes.");
    }
    if (a == DataType::FP32 || b == DataType::FP32) return DataType::FP32;
    const bool hasHalf = a == DataType::FP16 || b == DataType::FP16;
    const bool hasBrain = a == DataType::BF16 || b == DataType::BF16;
    if (hasHalf && hasBrain) return DataType::FP32;
    if (hasBrain) return DataType::BF16;
    return DataType::FP16;  // fp16 with fp8, or the two fp8 flavours together
}

DataType promoteTensorValueDTypes(const std::vector<DataType>& dtypes) {
    if (dtypes.empty()) throw std::runtime_error("promoteTensorValueDTypes requires at least one dtype.");
    DataType out = dtypes.front();
    for (size_t i = 1; i < dtypes.size(); ++i) out = promoteTensorValueDTypes(out, dtypes[i]);
    return out;
}

DataType defaultComputeDType(DataType value_dtype) {
    if (isFp8Type(value_dtype)) return DataType::FP16;
    if (value_dtype == DataType::FP16 || value_dtype == DataType::BF16 || value_dtype == DataType::FP32) return value_dtype;
    throw std::runtime_error("Unsupported dtype in defaultComputeDType.");
}

DataType defaultComputeDType(DataType input_dtype, DataType output_dtype) {
    if (!isSupportedFusionFloatingType(input_dtype) || !isSupportedFusionFloatingType(output_dtype)) {
        throw std::runtime_error("Unsupported dtype in defaultComputeDType(input_dtype, output_dtype).");
    }
    return promoteTensorValueDTypes(input_dtype, output_dtype);
}

DataType toSupportedComputeDType(ExprOp op, DataType requested) {
    if (isComparison(op) || isLogical(op) || op == ExprOp::WHERE) {
        if (requested == DataType::BOOLEAN || requested == DataType::UINT8) return DataType::BOOLEAN;
        if (isSupportedFusionFloatingType(requested)) return toSupportedComputeDType(ExprOp::ADD, requested);
        throw std::runtime_error("Unsupported boolean/comparison/where dtype in toSupportedComputeDType.");
    }
    if (op == ExprOp::CAST || isShapeOnly(op) || op == ExprOp::RAGGED_VALUEWISE_EXTENT || op == ExprOp::SEGMENTED_BROADCAST || isWinnerRoutingOp(op) ||
        op == ExprOp::TAKE_ALONG_AXIS || op == ExprOp::ROPE || isScatterRoutingOp(op) || isScanOp(op)) {
        if (isBindableInputDType(requested)) return requested;
        throw std::runtime_error("Unsupported passthrough dtype in toSupportedComputeDType.");
    }
    if (op == ExprOp::SUB && (requested == DataType::UINT32 || requested == DataType::UINT64)) return requested;
    if (!isSupportedFusionFloatingType(requested)) throw std::runtime_error("Unsupported dtype in toSupportedComputeDType.");
    if (isReductionOp(op) || op == ExprOp::SOFTMAX || isSegmentedReduceOp(op)) return DataType::FP32;
    if (isFp8Type(requested) || requested == DataType::FP16) return DataType::FP16;
    return requested;  // bf16 or fp32
}

void resolveExpressionDTypesInPlace(PhysicalExpression& expr, const std::vector<DataType>& root_input_dtypes) {
    if (expr.output_node >= expr.nodes.size()) throw std::runtime_error("resolveExpressionDTypesInPlace requires a valid output_node.");
    resolveInPlace(expr, root_input_dtypes, {expr.output_node});
}

void resolveOutputsDTypesInPlace(PhysicalOutputs& outputs, const std::vector<DataType>& root_input_dtypes) {
    if (!outputs.expr) throw std::runtime_error("resolveOutputsDTypesInPlace requires non-null outputs.expr.");
    std::vector<uint32_t> nodes;
    for (const NamedOutput& o : outputs.outputs) nodes.push_back(o.node_idx);
    resolveInPlace(*outputs.expr, root_input_dtypes, nodes);
}

}  // namespace ThorImplementation
