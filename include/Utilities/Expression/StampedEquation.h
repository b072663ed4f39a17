// Stamped (shape- and tensor-bound) pieces of a compiled expression and the plan that runs them in order
// (reference: Utilities/Expression/StampedEquation.h:411-516 StampedEquation, :551-597 StampedReduction / StampedArgMinMax,
//  :1659-1780 StampedExecutionPlan).  A stamped object owns copies of the Tensor handles it reads and writes, so
// the storage outlives queued work; run() never allocates, compiles or re-plans.
#pragma once

#include "DeepLearning/Implementation/Tensor/Tensor.h"
#include "Utilities/Common/Stream.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "Utilities/Expression/SegmentedBroadcastKernel.h"
#include "Utilities/TensorOperations/Cub/CubReduction.h"

#include <cstdint>
#include <memory>
#include <optional>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace ThorImplementation {

// One launch of a run-time compiled elementwise / broadcast kernel, or of a row-fused kernel that also holds the
// reductions of its rows.
class StampedEquation {
   public:
    struct ScalarArgument {
        std::string name;  // runtime scalar input name
        size_t argIndex;   // position in the kernel argument list
    };

    StampedEquation(std::shared_ptr<CompiledKernel> kernel, std::vector<Tensor> inputs, std::vector<Tensor> outputs,
                    std::vector<ScalarArgument> scalars, std::vector<size_t> inputArgIndex, std::vector<size_t> outputArgIndex,
                    size_t numArgs, bool passNumel, uint64_t numel, bool numelIs64, uint32_t gridX, uint32_t threads, uint64_t flops,
                    std::string description);

    void run(Stream& stream) const { runOn(stream, {}); }
    void runOn(Stream& stream, const std::unordered_map<std::string, float>& runtime_scalars) const;

    uint32_t gpuNum() const;
    Tensor getOutputTensor() const;
    const std::vector<Tensor>& getOutputTensors() const { return outputs; }
    const std::vector<Tensor>& getInputTensors() const { return inputs; }
    const std::shared_ptr<CompiledKernel>& getCompiledKernel() const { return kernel; }
    uint64_t flopCount() const { return flops; }
    const std::string& getDescription() const { return description; }
    std::unordered_set<std::string> runtimeScalarNames() const;

    // Reduced axes become 1; the listed squeeze axes (or every singleton when squeeze_axes == {UINT64_MAX}) are removed.
    static std::vector<uint64_t> computeReductionOutputDims(const std::vector<uint64_t>& input_dims, const std::vector<uint64_t>& reduction_axes,
                                                            const std::vector<uint64_t>& squeeze_axes);

   private:
    std::shared_ptr<CompiledKernel> kernel;
    std::vector<Tensor> inputs;
    std::vector<Tensor> outputs;
    std::vector<ScalarArgument> scalars;
    std::vector<size_t> inputArgIndex, outputArgIndex;
    size_t numArgs;
    bool passNumel;
    uint64_t numel;
    bool numelIs64;
    uint32_t gridX, threads;
    uint64_t flops;
    std::string description;
};

class StampedReduction {
   public:
    explicit StampedReduction(std::shared_ptr<StampedCubReduction> stamped) : stamped(std::move(stamped)) {}
    void runOn(Stream& stream) const { stamped->runOn(stream); }
    CubReductionPath getPath() const { return stamped->getPath(); }
    Tensor getOutputTensor() const { return stamped->getOutputTensor(); }
    uint64_t flopCount() const { return stamped->getGeometry().input_elements; }
    const std::shared_ptr<StampedCubReduction>& getStamped() const { return stamped; }

   private:
    std::shared_ptr<StampedCubReduction> stamped;
};

class StampedArgMinMax {
   public:
    explicit StampedArgMinMax(std::shared_ptr<StampedCubArgReduction> stamped) : stamped(std::move(stamped)) {}
    void runOn(Stream& stream) const { stamped->runOn(stream); }
    CubReductionPath getPath() const { return stamped->getPath(); }
    Tensor getOutputTensor() const { return stamped->getIndexOutputTensor().value(); }
    uint64_t flopCount() const { return stamped->getGeometry().input_elements; }

   private:
    std::shared_ptr<StampedCubArgReduction> stamped;
};

// Several value reductions over one geometry evaluated in a single pass over their common sources, with the
// elementwise work that feeds them computed in registers (sum(x) and sum(x*x) of one tensor: one read of x), optionally
// writing same-shaped elementwise results of those sources in the same pass.
class StampedFusedReduction {
   public:
    // `segmentOffsets`: the reduction runs per segment of a ragged batch; the kernels read this offsets tensor at every run.
    StampedFusedReduction(ReductionLaunchPlan plan, std::vector<Tensor> inputs, std::vector<std::string> scalarNames, std::vector<Tensor> outputs,
                          std::vector<Tensor> elementwiseOutputs, std::optional<Tensor> workspace, uint64_t flops,
                          std::optional<Tensor> segmentOffsets = std::nullopt)
        : plan(std::move(plan)), inputs(std::move(inputs)), scalarNames(std::move(scalarNames)), outputs(std::move(outputs)),
          elementwiseOutputs(std::move(elementwiseOutputs)), workspace(std::move(workspace)), flops(flops), segmentOffsets(std::move(segmentOffsets)) {}
    void runOn(Stream& stream, const std::unordered_map<std::string, float>& runtime_scalars) const;
    const std::vector<Tensor>& getOutputTensors() const { return outputs; }
    const std::vector<std::string>& runtimeScalarNames() const { return scalarNames; }
    uint64_t flopCount() const { return flops; }
    const std::string& getDescription() const { return plan.variant; }
    const ReductionLaunchPlan& getLaunchPlan() const { return plan; }

   private:
    ReductionLaunchPlan plan;
    std::vector<Tensor> inputs;
    std::vector<std::string> scalarNames;
    std::vector<Tensor> outputs;
    std::vector<Tensor> elementwiseOutputs;  // tensors of the input's shape written by the same pass
    std::optional<Tensor> workspace;
    uint64_t flops;
    std::optional<Tensor> segmentOffsets;
};

// Per-segment reduction over a ragged batch; the offsets are read on the device each time the stage runs.
class StampedSegmentedReductionStage {
   public:
    explicit StampedSegmentedReductionStage(std::shared_ptr<StampedCubSegmentedReduction> stamped) : stamped(std::move(stamped)) {}
    void runOn(Stream& stream) const { stamped->runOn(stream); }
    Tensor getOutputTensor() const { return stamped->getOutputTensor(); }
    uint64_t flopCount() const { return stamped->getNumItems(); }
    const std::shared_ptr<StampedCubSegmentedReduction>& getStamped() const { return stamped; }

   private:
    std::shared_ptr<StampedCubSegmentedReduction> stamped;
};

// A prefix scan bound to its tensors: values along the last axis, or over the segments of an offsets tensor read at every run.
struct CubScanKernels;
class StampedScan {
   public:
    // one output: the scanned values, or (indexOutput) the UINT32 indices of an arg scan
    StampedScan(std::shared_ptr<const CubScanKernels> kernels, Tensor input, std::optional<Tensor> offsets, Tensor temp, Tensor output, bool indexOutput)
        : kernels(std::move(kernels)), input(std::move(input)), offsets(std::move(offsets)), temp(std::move(temp)) {
        (indexOutput ? indices : values) = std::move(output);
    }
    // a min / max scan that writes the running values and the indices that hold them in one pass
    StampedScan(std::shared_ptr<const CubScanKernels> kernels, Tensor input, std::optional<Tensor> offsets, Tensor temp, Tensor values, Tensor indices)
        : kernels(std::move(kernels)), input(std::move(input)), offsets(std::move(offsets)), temp(std::move(temp)), values(std::move(values)),
          indices(std::move(indices)) {}
    // the gradient of a min / max scan over rows in one launch: reads the operand and the FP32 upstream gradient, writes `routed`
    static StampedScan routing(std::shared_ptr<const CubScanKernels> kernels, Tensor input, Tensor gradient, Tensor routed) {
        StampedScan scan(std::move(kernels), std::move(input), std::nullopt, Tensor(), std::move(routed), /*indexOutput=*/false);
        scan.gradient = std::move(gradient);
        return scan;
    }
    void runOn(Stream& stream) const;
    Tensor getOutputTensor() const { return values.isInitialized() ? values : indices; }
    std::string getKernelVariant() const;

   private:
    std::shared_ptr<const CubScanKernels> kernels;
    Tensor input;
    std::optional<Tensor> offsets;
    Tensor temp, values, indices, gradient;
};

struct StampedExecutionStage {
    enum class Kind {
        FusedKernel, Reduction, ArgMinMax, FusedRowKernel, Copy, FusedReduction, SegmentedReduction, SegmentedBroadcast, ReduceMinMaxBackward, Scan,
        DependencyBarrier,  // launches nothing: a node of the dependency graph only (scheduler tests; reference StampedEquation.h:1461)
    };
    static std::string kindToString(Kind kind) {
        switch (kind) {
            case Kind::FusedKernel:
                return "FusedKernel";
            case Kind::Reduction:
                return "Reduction";
            case Kind::ArgMinMax:
                return "ArgMinMax";
            case Kind::FusedRowKernel:
                return "FusedRowKernel";
            case Kind::Copy:
                return "Copy";
            case Kind::FusedReduction:
                return "FusedReduction";
            case Kind::SegmentedReduction:
                return "SegmentedReduction";
            case Kind::SegmentedBroadcast:
                return "SegmentedBroadcast";
            case Kind::ReduceMinMaxBackward:
                return "ReduceMinMaxBackward";
            case Kind::Scan:
                return "Scan";
            case Kind::DependencyBarrier:
                return "DependencyBarrier";
        }
        return "<unknown>";
    }
    static StampedExecutionStage dependencyBarrier(uint32_t gpu_num, std::vector<uint32_t> dependency_stage_indices) {
        StampedExecutionStage stage;
        stage.kind = Kind::DependencyBarrier;
        stage.gpu_num = gpu_num;
        stage.dependency_stage_indices = std::move(dependency_stage_indices);
        return stage;
    }

    Kind kind = Kind::FusedKernel;
    std::vector<uint32_t> dependency_stage_indices;
    uint32_t gpu_num = 0;
    std::shared_ptr<StampedEquation> kernel;  // also the routing kernel of Kind::ReduceMinMaxBackward (its winners come from an ArgMinMax stage)
    std::shared_ptr<StampedReduction> reduction;
    std::shared_ptr<StampedArgMinMax> arg_minmax;
    std::shared_ptr<StampedFusedReduction> fused_reduction;
    std::shared_ptr<StampedSegmentedReductionStage> segmented_reduction;
    std::shared_ptr<StampedCubSegmentedArgReduction> segmented_arg_reduction;  // SegmentedReduction stages that find winners instead of values
    std::shared_ptr<StampedSegmentedBroadcast> segmented_broadcast;
    std::shared_ptr<StampedScan> scan;
    // Kind::Copy: a named output that is only a view of an input is copied into the caller's tensor
    Tensor copySource, copyDestination;

    uint64_t flopCount() const;
    void runOn(Stream& stream, const std::unordered_map<std::string, float>& runtime_scalars) const;
};

namespace detail {

// Where every stage of a plan runs (reference: StampedEquation.h:1637-1646, StampedEquation.cpp:3958-4047).  Lane 0 is the
// caller's stream; every other lane is a helper stream, so stages on different lanes may overlap.  A chain never leaves its
// lane: at a fork the first dependent stage continues on the producer's lane and the others open lanes of their own; a stage
// inherits the lane of a producer it continues (the caller's lane when it continues several).  A stage whose result is
// needed on another lane records a completion event; helper lanes that start from nothing wait for the caller-ready event.
struct StampedExecutionSchedule {
    std::vector<uint32_t> stage_lane_indices;
    std::vector<uint32_t> lane_gpu_nums;
    std::vector<bool> stage_has_downstream_dependency;
    std::vector<bool> stage_needs_completion_event;
    bool needs_caller_ready_event = false;
};

// Throws std::runtime_error when a stage depends on itself or on a later stage.
StampedExecutionSchedule buildStampedExecutionSchedule(const std::vector<StampedExecutionStage>& steps, uint32_t caller_gpu_num);

}  // namespace detail

class StampedExecutionPlan {
   public:
    // Builds the schedule and, when it has helper lanes, takes their streams from Expression's helper-stream pool and creates the
    // events the joins need: run() itself creates nothing.
    StampedExecutionPlan(std::vector<StampedExecutionStage> steps, std::unordered_map<std::string, Tensor> final_outputs, const Stream& stream);

    void run();
    void run(const std::unordered_map<std::string, float>& runtime_scalars);
    void runOn(Stream& run_stream) const;
    void runOn(Stream& run_stream, const std::unordered_map<std::string, float>& runtime_scalars) const;

    bool requiresRuntimeScalars() const { return !runtimeScalarNames().empty(); }
    std::unordered_set<std::string> runtimeScalarNames() const;

    uint64_t flopCount() const;
    std::vector<uint64_t> stageFlopCounts() const;
    std::vector<std::string> stageKindNames() const;
    std::vector<std::vector<uint32_t>> stageDependencyIndices() const;
    std::vector<CubReductionPath> reductionPaths() const;
    const std::vector<StampedExecutionStage>& stages() const { return steps; }
    const detail::StampedExecutionSchedule& schedule() const { return execution_schedule; }

    Tensor output(const std::string& name) const;
    Tensor output() const;
    const std::unordered_map<std::string, Tensor>& getFinalOutputs() const { return final_outputs; }

   private:
    struct LaneResources {
        std::vector<Stream> helpers;            // lanes 1 .. of the schedule
        Event caller_ready;                     // set when the schedule needs it
        std::vector<Event> stage_completion;    // one slot per stage; initialised where the schedule asks for an event
    };
    static LaneResources makeLaneResources(const detail::StampedExecutionSchedule& schedule);
    void runForked(Stream& run_stream, const detail::StampedExecutionSchedule& schedule, const LaneResources& lanes,
                   const std::unordered_map<std::string, float>& runtime_scalars) const;

    std::vector<StampedExecutionStage> steps;
    std::unordered_map<std::string, Tensor> final_outputs;
    Stream stream;
    detail::StampedExecutionSchedule execution_schedule;
    LaneResources lane_resources;
};

}  // namespace ThorImplementation
