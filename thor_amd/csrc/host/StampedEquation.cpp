#include "Utilities/Expression/StampedEquation.h"

#include "Utilities/Common/ScopedGpu.h"

#include "Utilities/Expression/Expression.h"

#include <algorithm>
#include <cstdlib>
#include <limits>
#include <stdexcept>

namespace ThorImplementation {

StampedEquation::StampedEquation(std::shared_ptr<CompiledKernel> kernel, std::vector<Tensor> inputs, std::vector<Tensor> outputs,
                                 std::vector<ScalarArgument> scalars, std::vector<size_t> inputArgIndex, std::vector<size_t> outputArgIndex,
                                 size_t numArgs, bool passNumel, uint64_t numel, bool numelIs64, uint32_t gridX, uint32_t threads,
                                 uint64_t flops, std::string description)
    : kernel(std::move(kernel)), inputs(std::move(inputs)), outputs(std::move(outputs)), scalars(std::move(scalars)),
      inputArgIndex(std::move(inputArgIndex)), outputArgIndex(std::move(outputArgIndex)), numArgs(numArgs), passNumel(passNumel),
      numel(numel), numelIs64(numelIs64), gridX(gridX), threads(threads), flops(flops), description(std::move(description)) {
    if (!this->kernel) throw std::runtime_error("StampedEquation requires a compiled kernel.");
    if (this->outputs.empty()) throw std::runtime_error("StampedEquation requires at least one output tensor.");
    for (const Tensor& t : this->inputs) {
        if (t.getPlacement().getMemDevice() != TensorPlacement::MemDevices::GPU) {
            throw std::runtime_error("Fused equation inputs must be GPU tensors.");
        }
    }
}

uint32_t StampedEquation::gpuNum() const { return outputs[0].getPlacement().getDeviceNum(); }

Tensor StampedEquation::getOutputTensor() const {
    if (outputs.size() != 1) {
        throw std::runtime_error("getOutputTensor called but there are " + std::to_string(outputs.size()) +
                                 " outputs. This function is only valid for single output equations.");
    }
    return outputs[0];
}

std::unordered_set<std::string> StampedEquation::runtimeScalarNames() const {
    std::unordered_set<std::string> names;
    for (const ScalarArgument& s : scalars) names.insert(s.name);
    return names;
}

void StampedEquation::runOn(Stream& stream, const std::unordered_map<std::string, float>& runtime_scalars) const {
    if (!stream.isInitialized() || stream.getGpuNum() != static_cast<int>(gpuNum())) {
        throw std::runtime_error("Stamped equation must run on a stream of the GPU its tensors live on.");
    }
    // argument storage: one slot per kernel argument, each holding either a pointer or a float / index value
    std::vector<const void*> pointerSlots(numArgs, nullptr);
    std::vector<float> floatSlots(numArgs, 0.0f);
    std::vector<void*> args(numArgs + (passNumel ? 1 : 0), nullptr);
    for (size_t i = 0; i < inputs.size(); ++i) {
        pointerSlots[inputArgIndex[i]] = inputs[i].getMemPtr();
        args[inputArgIndex[i]] = &pointerSlots[inputArgIndex[i]];
    }
    for (size_t i = 0; i < outputs.size(); ++i) {
        pointerSlots[outputArgIndex[i]] = outputs[i].getMemPtr();
        args[outputArgIndex[i]] = &pointerSlots[outputArgIndex[i]];
    }
    for (const ScalarArgument& s : scalars) {
        auto it = runtime_scalars.find(s.name);
        if (it == runtime_scalars.end()) throw std::runtime_error("Missing runtime scalar input: " + s.name);
        floatSlots[s.argIndex] = it->second;
        args[s.argIndex] = &floatSlots[s.argIndex];
    }
    uint32_t numel32 = static_cast<uint32_t>(numel);
    uint64_t numel64 = numel;
    if (passNumel) args[numArgs] = numelIs64 ? static_cast<void*>(&numel64) : static_cast<void*>(&numel32);
    ScopedGpu scoped(stream.getGpuNum());
    kernel->launch(gridX, 1, 1, threads, stream.getStream(), args);
}

std::vector<uint64_t> StampedEquation::computeReductionOutputDims(const std::vector<uint64_t>& input_dims,
                                                                  const std::vector<uint64_t>& reduction_axes,
                                                                  const std::vector<uint64_t>& squeeze_axes) {
    std::vector<uint64_t> out = input_dims;
    for (uint64_t axis : reduction_axes) {
        if (axis >= out.size()) throw std::runtime_error("Reduction axis out of range.");
        out[axis] = 1;
    }
    if (squeeze_axes.empty()) return out;
    std::vector<uint64_t> squeezed;
    if (squeeze_axes.size() == 1 && squeeze_axes[0] == std::numeric_limits<uint64_t>::max()) {
        for (uint64_t d : out)
            if (d != 1) squeezed.push_back(d);
    } else {
        std::vector<uint64_t> axes = squeeze_axes;
        std::sort(axes.begin(), axes.end());
        axes.erase(std::unique(axes.begin(), axes.end()), axes.end());
        for (uint64_t axis : axes) {
            if (axis >= out.size()) throw std::runtime_error("squeeze axes are invalid for the input rank.");
            if (out[axis] != 1) {
                throw std::runtime_error("Trying to squeeze axis " + std::to_string(axis) + " but it has size " + std::to_string(out[axis]) +
                                         ", can only squeeze dimensions of size 1.");
            }
        }
        for (uint64_t i = 0; i < out.size(); ++i)
            if (!std::binary_search(axes.begin(), axes.end(), i)) squeezed.push_back(out[i]);
    }
    if (squeezed.empty()) squeezed.push_back(1);
    return squeezed;
}

void StampedFusedReduction::runOn(Stream& stream, const std::unordered_map<std::string, float>& runtime_scalars) const {
    if (!stream.isInitialized() || outputs.empty() || stream.getGpuNum() != static_cast<int>(outputs[0].getPlacement().getDeviceNum())) {
        throw std::runtime_error("Stamped reduction must run on a stream of the GPU its tensors live on.");
    }
    // main kernel: sources, runtime scalars, outputs, index output (unused), partials, scale
    std::vector<const void*> sourcePointers(inputs.size());
    std::vector<float> scalarValues(scalarNames.size());
    std::vector<void*> outputPointers(outputs.size());
    void* indexOut = nullptr;
    void* partials = workspace.has_value() ? const_cast<Tensor&>(workspace.value()).getMemPtr<char>() : nullptr;
    float scale = 1.0f;
    std::vector<void*> args;
    for (size_t i = 0; i < inputs.size(); ++i) {
        sourcePointers[i] = inputs[i].getMemPtr();
        args.push_back(&sourcePointers[i]);
    }
    for (size_t i = 0; i < scalarNames.size(); ++i) {
        auto it = runtime_scalars.find(scalarNames[i]);
        if (it == runtime_scalars.end()) throw std::runtime_error("Missing runtime scalar input: " + scalarNames[i]);
        scalarValues[i] = it->second;
        args.push_back(&scalarValues[i]);
    }
    for (size_t i = 0; i < outputs.size(); ++i) {
        outputPointers[i] = const_cast<Tensor&>(outputs[i]).getMemPtr();
        args.push_back(&outputPointers[i]);
    }
    std::vector<void*> elementwisePointers(elementwiseOutputs.size());
    for (size_t i = 0; i < elementwiseOutputs.size(); ++i) {
        elementwisePointers[i] = const_cast<Tensor&>(elementwiseOutputs[i]).getMemPtr();
        args.push_back(&elementwisePointers[i]);
    }
    args.push_back(&indexOut);
    args.push_back(&partials);
    args.push_back(&scale);
    const void* offsetPointer = segmentOffsets.has_value() ? segmentOffsets->getMemPtr() : nullptr;
    if (segmentOffsets.has_value()) args.push_back(&offsetPointer);
    ScopedGpu scoped(stream.getGpuNum());
    if (plan.prepareKernel) {
        std::vector<void*> prepareArgs = {&partials, &offsetPointer};
        plan.prepareKernel->launch(plan.prepareGridX, 1, 1, plan.prepareThreads, stream.getStream(), prepareArgs);
    }
    plan.mainKernel->launch(plan.mainGridX, plan.mainGridY, 1, plan.mainThreads, stream.getStream(), args);
    if (plan.finishKernel) {
        const void* constPartials = partials;
        std::vector<void*> finishArgs = {&constPartials};
        for (size_t i = 0; i < outputs.size(); ++i) finishArgs.push_back(&outputPointers[i]);
        finishArgs.push_back(&indexOut);
        finishArgs.push_back(&scale);
        if (segmentOffsets.has_value()) finishArgs.push_back(&offsetPointer);
        plan.finishKernel->launch(plan.finishGridX, 1, 1, plan.finishThreads, stream.getStream(), finishArgs);
    }
}

uint64_t StampedExecutionStage::flopCount() const {
    switch (kind) {
        case Kind::FusedKernel:
        case Kind::FusedRowKernel:
        case Kind::ReduceMinMaxBackward:
            return kernel ? kernel->flopCount() : 0;
        case Kind::Reduction:
            return reduction ? reduction->flopCount() : 0;
        case Kind::ArgMinMax:
            return arg_minmax ? arg_minmax->flopCount() : 0;
        case Kind::Copy:
            return 0;
        case Kind::FusedReduction:
            return fused_reduction ? fused_reduction->flopCount() : 0;
        case Kind::SegmentedReduction:
            return segmented_reduction ? segmented_reduction->flopCount() : 0;
        case Kind::SegmentedBroadcast:
        case Kind::Scan:
        case Kind::DependencyBarrier:
            return 0;
    }
    return 0;
}

void StampedExecutionStage::runOn(Stream& stream, const std::unordered_map<std::string, float>& runtime_scalars) const {
    switch (kind) {
        case Kind::FusedKernel:
        case Kind::FusedRowKernel:
        case Kind::ReduceMinMaxBackward:
            if (!kernel) throw std::runtime_error("Fused execution stage is missing its stamped kernel.");
            kernel->runOn(stream, runtime_scalars);
            return;
        case Kind::Reduction:
            if (!reduction) throw std::runtime_error("Reduction execution stage is missing its stamped reduction.");
            reduction->runOn(stream);
            return;
        case Kind::ArgMinMax:
            if (!arg_minmax) throw std::runtime_error("ArgMinMax execution stage is missing its stamped reduction.");
            arg_minmax->runOn(stream);
            return;
        case Kind::Copy: {
            Tensor destination = copyDestination;
            destination.copyFromAsync(copySource, stream);
            return;
        }
        case Kind::FusedReduction:
            if (!fused_reduction) throw std::runtime_error("Fused reduction stage is missing its stamped reduction.");
            fused_reduction->runOn(stream, runtime_scalars);
            return;
        case Kind::SegmentedReduction:
            if (segmented_arg_reduction) {
                segmented_arg_reduction->runOn(stream);
                return;
            }
            if (!segmented_reduction) throw std::runtime_error("Segmented reduction stage is missing its stamped reduction.");
            segmented_reduction->runOn(stream);
            return;
        case Kind::SegmentedBroadcast:
            if (!segmented_broadcast) throw std::runtime_error("Segmented broadcast stage is missing its stamped broadcast.");
            segmented_broadcast->runOn(stream);
            return;
        case Kind::Scan:
            if (!scan) throw std::runtime_error("Scan stage is missing its stamped scan.");
            scan->runOn(stream);
            return;
        case Kind::DependencyBarrier:
            return;
    }
}

detail::StampedExecutionSchedule detail::buildStampedExecutionSchedule(const std::vector<StampedExecutionStage>& steps, uint32_t caller_gpu_num) {
    StampedExecutionSchedule schedule;
    const uint32_t count = static_cast<uint32_t>(steps.size());
    schedule.stage_lane_indices.assign(count, 0);
    schedule.stage_has_downstream_dependency.assign(count, false);
    schedule.stage_needs_completion_event.assign(count, false);
    schedule.lane_gpu_nums.push_back(caller_gpu_num);
    if (count == 0) return schedule;

    // heir[p]: the dependent stage that stays on p's lane = the first stage on p's GPU that consumes p
    constexpr uint32_t kNone = 0xffffffffu;
    std::vector<uint32_t> heir(count, kNone);
    for (uint32_t stage = 0; stage < count; ++stage) {
        for (uint32_t producer : steps[stage].dependency_stage_indices) {
            if (producer >= stage) throw std::runtime_error("StampedExecutionPlan::runOn requires dependency_stage_indices to be topologically ordered.");
            if (heir[producer] == kNone && steps[producer].gpu_num == steps[stage].gpu_num) heir[producer] = stage;
        }
    }
    bool callerLaneHasRoot = false;
    for (uint32_t stage = 0; stage < count; ++stage) {
        uint32_t lane = kNone;
        for (uint32_t producer : steps[stage].dependency_stage_indices) {
            if (heir[producer] != stage) continue;
            const uint32_t candidate = schedule.stage_lane_indices[producer];
            if (lane == kNone || candidate == 0) lane = candidate;  // heir of several producers: the caller's lane wins, else the first
            if (lane == 0) break;
        }
        if (lane == kNone && steps[stage].dependency_stage_indices.empty() && !callerLaneHasRoot && steps[stage].gpu_num == caller_gpu_num) {
            lane = 0;
            callerLaneHasRoot = true;
        }
        if (lane == kNone) {
            lane = static_cast<uint32_t>(schedule.lane_gpu_nums.size());
            schedule.lane_gpu_nums.push_back(steps[stage].gpu_num);
        }
        schedule.stage_lane_indices[stage] = lane;
    }
    for (uint32_t stage = 0; stage < count; ++stage) {
        const uint32_t lane = schedule.stage_lane_indices[stage];
        if (steps[stage].dependency_stage_indices.empty() && lane != 0) schedule.needs_caller_ready_event = true;
        for (uint32_t producer : steps[stage].dependency_stage_indices) {
            schedule.stage_has_downstream_dependency[producer] = true;
            if (schedule.stage_lane_indices[producer] != lane) schedule.stage_needs_completion_event[producer] = true;
        }
    }
    // the last stage of a helper lane that nothing consumes is joined back into the caller's stream at the end of the run
    for (uint32_t stage = 0; stage < count; ++stage) {
        if (!schedule.stage_has_downstream_dependency[stage] && schedule.stage_lane_indices[stage] != 0) schedule.stage_needs_completion_event[stage] = true;
    }
    return schedule;
}

StampedExecutionPlan::LaneResources StampedExecutionPlan::makeLaneResources(const detail::StampedExecutionSchedule& schedule) {
    LaneResources lanes;
    if (schedule.lane_gpu_nums.size() <= 1) return lanes;
    for (size_t lane = 1; lane < schedule.lane_gpu_nums.size(); ++lane) lanes.helpers.push_back(Expression::getNextHelperStream(schedule.lane_gpu_nums[lane]));
    if (schedule.needs_caller_ready_event) lanes.caller_ready = Event(static_cast<int>(schedule.lane_gpu_nums[0]));
    lanes.stage_completion.resize(schedule.stage_lane_indices.size());
    for (size_t stage = 0; stage < schedule.stage_lane_indices.size(); ++stage) {
        if (schedule.stage_needs_completion_event[stage]) {
            lanes.stage_completion[stage] = Event(static_cast<int>(schedule.lane_gpu_nums[schedule.stage_lane_indices[stage]]));
        }
    }
    return lanes;
}

StampedExecutionPlan::StampedExecutionPlan(std::vector<StampedExecutionStage> plan_steps, std::unordered_map<std::string, Tensor> outputs,
                                           const Stream& plan_stream)
    : steps(std::move(plan_steps)), final_outputs(std::move(outputs)), stream(plan_stream),
      execution_schedule(detail::buildStampedExecutionSchedule(steps, plan_stream.isInitialized() ? static_cast<uint32_t>(plan_stream.getGpuNum()) : 0u)),
      lane_resources(makeLaneResources(execution_schedule)) {}

void StampedExecutionPlan::run() { runOn(stream, {}); }
void StampedExecutionPlan::run(const std::unordered_map<std::string, float>& runtime_scalars) { runOn(stream, runtime_scalars); }
void StampedExecutionPlan::runOn(Stream& run_stream) const { runOn(run_stream, {}); }

void StampedExecutionPlan::runOn(Stream& run_stream, const std::unordered_map<std::string, float>& runtime_scalars) const {
    // Single stages and plans without a branch (every stage on the caller's lane) need no scheduler: stages are stored in
    // dependency order and stream order is the synchronisation (reference: StampedEquation.cpp:4065-4113).
    //
    // Plans with independent branches run the same way unless THOR_STAGE_OVERLAP=1 asks for the helper lanes.  Measured on
    // MI355X (one GPU, HIP events between streams): the gradient of a row maximum over 8192 x 8192 (fill | argmax -> route)
    // 91 us on one lane, 112 us forked; two large independent reductions 69 / 75 us; four small independent reduction chains
    // 17 / 67 us.  Kernels of this path fill the GPU on their own, so a second lane has nothing to overlap with, and every
    // cross-stream event costs several microseconds.
    static const bool overlapByDefault = [] {
        const char* env = std::getenv("THOR_STAGE_OVERLAP");
        return env != nullptr && std::atoi(env) != 0;
    }();
    const char* now = std::getenv("THOR_STAGE_OVERLAP");  // re-read so that a caller (or a test) can switch between runs
    const bool overlap = now != nullptr ? std::atoi(now) != 0 : overlapByDefault;
    if (execution_schedule.lane_gpu_nums.size() <= 1 || !overlap) {
        for (const StampedExecutionStage& step : steps) step.runOn(run_stream, runtime_scalars);
        return;
    }
    if (run_stream.getGpuNum() == stream.getGpuNum()) {
        runForked(run_stream, execution_schedule, lane_resources, runtime_scalars);
        return;
    }
    // a run on another GPU's stream than the plan was stamped for: its own schedule and lanes, made for this run
    const detail::StampedExecutionSchedule other = detail::buildStampedExecutionSchedule(steps, static_cast<uint32_t>(run_stream.getGpuNum()));
    const LaneResources lanes = makeLaneResources(other);
    runForked(run_stream, other, lanes, runtime_scalars);
}

// Independent branches on helper streams, joined with events (reference: StampedEquation.cpp:4115-4207).  Events are the plan's
// own, created when it was stamped; a wait captures the event's latest record at the time of the call, so the next run may
// record the same events again without waiting for this one.
void StampedExecutionPlan::runForked(Stream& run_stream, const detail::StampedExecutionSchedule& schedule, const LaneResources& lanes,
                                     const std::unordered_map<std::string, float>& runtime_scalars) const {
    auto laneStream = [&](uint32_t lane) -> const Stream& { return lane == 0 ? run_stream : lanes.helpers[lane - 1]; };
    if (schedule.needs_caller_ready_event) {
        Event ready = lanes.caller_ready;
        run_stream.putEvent(ready);
    }
    for (uint32_t index = 0; index < steps.size(); ++index) {
        const StampedExecutionStage& stage = steps[index];
        const uint32_t lane = schedule.stage_lane_indices[index];
        Stream launch = laneStream(lane);
        if (stage.dependency_stage_indices.empty() && lane != 0) launch.waitEvent(lanes.caller_ready);  // work queued on the caller's stream comes first
        for (uint32_t producer : stage.dependency_stage_indices) {
            const Stream& producerStream = laneStream(schedule.stage_lane_indices[producer]);
            if (launch == producerStream) continue;
            if (!lanes.stage_completion[producer].isInitialized()) {
                throw std::runtime_error("StampedExecutionPlan::runOn missing completion event for cross-stream dependency stage.");
            }
            launch.waitEvent(lanes.stage_completion[producer]);
        }
        stage.runOn(launch, runtime_scalars);
        if (schedule.stage_needs_completion_event[index]) {
            Event done = lanes.stage_completion[index];
            launch.putEvent(done);
        }
    }
    // helper work that nothing consumed joins the caller's stream; branches that fed a stage on it are joined already
    for (uint32_t index = 0; index < steps.size(); ++index) {
        const uint32_t lane = schedule.stage_lane_indices[index];
        if (schedule.stage_has_downstream_dependency[index] || lane == 0 || laneStream(lane) == run_stream) continue;
        run_stream.waitEvent(lanes.stage_completion[index]);
    }
}

std::unordered_set<std::string> StampedExecutionPlan::runtimeScalarNames() const {
    std::unordered_set<std::string> names;
    for (const StampedExecutionStage& step : steps) {
        if (step.kernel) {
            for (const std::string& n : step.kernel->runtimeScalarNames()) names.insert(n);
        }
        if (step.fused_reduction) {
            for (const std::string& n : step.fused_reduction->runtimeScalarNames()) names.insert(n);
        }
    }
    return names;
}

uint64_t StampedExecutionPlan::flopCount() const {
    uint64_t total = 0;
    for (const StampedExecutionStage& step : steps) {
        const uint64_t f = step.flopCount();
        if (std::numeric_limits<uint64_t>::max() - total < f) throw std::runtime_error("StampedExecutionPlan::flopCount overflow.");
        total += f;
    }
    return total;
}

std::vector<uint64_t> StampedExecutionPlan::stageFlopCounts() const {
    std::vector<uint64_t> out;
    for (const StampedExecutionStage& step : steps) out.push_back(step.flopCount());
    return out;
}

std::vector<std::string> StampedExecutionPlan::stageKindNames() const {
    std::vector<std::string> out;
    for (const StampedExecutionStage& step : steps) out.push_back(StampedExecutionStage::kindToString(step.kind));
    return out;
}

std::vector<std::vector<uint32_t>> StampedExecutionPlan::stageDependencyIndices() const {
    std::vector<std::vector<uint32_t>> out;
    for (const StampedExecutionStage& step : steps) out.push_back(step.dependency_stage_indices);
    return out;
}

std::vector<CubReductionPath> StampedExecutionPlan::reductionPaths() const {
    std::vector<CubReductionPath> out;
    for (const StampedExecutionStage& step : steps) {
        if (step.kind == StampedExecutionStage::Kind::Reduction) {
            if (!step.reduction) throw std::runtime_error("Reduction execution stage is missing its stamped reduction.");
            out.push_back(step.reduction->getPath());
        }
    }
    return out;
}

Tensor StampedExecutionPlan::output(const std::string& name) const {
    auto it = final_outputs.find(name);
    if (it == final_outputs.end()) throw std::runtime_error("No such output in stamped execution plan: " + name);
    return it->second;
}

Tensor StampedExecutionPlan::output() const {
    if (final_outputs.size() != 1) {
        throw std::runtime_error("StampedEquation.output() called to return the single output tensor, but there are " +
                                 std::to_string(final_outputs.size()) + " output tensors.");
    }
    return final_outputs.begin()->second;
}

}  // namespace ThorImplementation
