// Per-node dtype policy of the Expression compiler: which dtype each node's value has (output dtype) and which dtype
// its arithmetic runs in (compute dtype), given the dtypes of the tensors bound to the inputs
// (reference: Utilities/Expression/ExpressionDTypeResolution.cpp:95-307,777-790,885-1137).
#pragma once

#include "Utilities/Expression/Expression.h"

#include <vector>

namespace ThorImplementation {

bool isSupportedFusionFloatingType(DataType dtype);  // fp8 e4m3/e5m2, fp16, bf16, fp32
bool isFp8Type(DataType dtype);

// fp16 (+) bf16 -> fp32; anything (+) fp32 -> fp32; bf16 beats fp8; fp16 beats fp8; e4m3 (+) e5m2 -> fp16
DataType promoteTensorValueDTypes(DataType a, DataType b);
DataType promoteTensorValueDTypes(const std::vector<DataType>& dtypes);

// fp8 and fp16 values compute in fp16, bf16 in bf16, fp32 in fp32
DataType defaultComputeDType(DataType value_dtype);
DataType defaultComputeDType(DataType input_dtype, DataType output_dtype);
DataType toSupportedComputeDType(ExprOp op, DataType requested_compute_dtype);

// Fills input_tensor_dtype / output_dtype / compute_dtype of every node in place.  `root_input_dtypes` is indexed by
// input slot.  The listed output nodes are the values that get materialised; their storage dtype widens the compute
// dtype of the nodes feeding them (never narrows it, never crosses a CAST, never leaks a reduction's fp32 policy).
void resolveExpressionDTypesInPlace(PhysicalExpression& expr, const std::vector<DataType>& root_input_dtypes);
void resolveOutputsDTypesInPlace(PhysicalOutputs& outputs, const std::vector<DataType>& root_input_dtypes);

}  // namespace ThorImplementation
