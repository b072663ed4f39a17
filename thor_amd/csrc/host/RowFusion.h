// Internal: recognises groups of stages that all work on the rows of one [rows, R] tensor -- last-axis reductions and
// the elementwise work between them -- and emits them as ONE kernel that loads each row once, keeps it in registers,
// folds it with wave64 shuffles / LDS, and writes the final values (softmax: 6 B/element instead of ~20 B/element for
// the staged max -> exp -> sum -> divide plan; mean/variance normalisation: 8 B/element).
#pragma once

#include "Utilities/Expression/Expression.h"
#include "Utilities/Expression/StampedEquation.h"

#include <functional>
#include <vector>

namespace ThorImplementation {

struct RowFusionContext {
    enum Role : uint8_t { Inline = 0, InputSource = 1, Materialized = 2, View = 3 };
    const PhysicalExpression& expr;
    const std::vector<NamedOutput>& outputs;
    const std::vector<NamedInput>& rootInputs;
    const std::vector<uint8_t>& role;
    const std::vector<std::vector<uint64_t>>& dims;
    std::vector<Tensor>& tensorOf;
    std::vector<char>& done;
    std::vector<StampedExecutionStage>& stages;
    std::vector<int>& stageOfNode;
    std::function<Tensor(uint32_t)> allocateFor;
    int deviceNum;
    Stream stream;  // the stream of the stamp call (workspaces are prepared on it)
};

// Appends FusedRowKernel stages for every group it recognises and marks the nodes they produce as done.
void tryRowFusion(RowFusionContext& ctx);

// Groups the remaining value reductions that run over the same shape and axes and whose inputs are tensors that already
// exist (or elementwise functions of such tensors that nothing else needs) into FusedReduction stages: one pass over the
// sources feeds every accumulator, and the elementwise work happens in registers instead of a materialised tensor.
void tryReductionFusion(RowFusionContext& ctx);

}  // namespace ThorImplementation
