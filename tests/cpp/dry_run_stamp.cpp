// Stamps a matrix of expressions without a GPU: this program defines the device C-ABI entry points for memory, streams,
// modules and launches itself (the dynamic linker binds the library's calls to these definitions), so planning, source
// generation and the run-time compilation for gfx950 run exactly as on a GPU box while nothing is launched.  What it
// guards: every kernel variant the planner can emit for these expressions compiles.  A compiler failure inside the
// in-process compiler aborts the process, so each case prints its name first.
#include "thorhip.h"

#include "Utilities/Expression/CompiledEquation.h"
#include "Utilities/Expression/FusedEquation.h"
#include "Utilities/Expression/RaggedExpression.h"
#include "Utilities/TensorOperations/Cub/CubDevicePrimitives.h"
#include "Utilities/TensorOperations/Cub/CubReduction.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <stdexcept>
#include <string>
#include <vector>

extern "C" {
int thorhip_device_count(int* count) { return *count = 1, 0; }
int thorhip_set_device(int) { return 0; }
int thorhip_get_device(int* device) { return *device = 0, 0; }
int thorhip_device_get_info(int, thorhip_device_info* info) {
    std::memset(info, 0, sizeof *info);
    info->compute_units = 256;
    info->wavefront_size = 64;
    info->max_threads_per_block = 1024;
    std::strcpy(info->arch_name, "gfx950");
    return 0;
}
int thorhip_device_synchronize(void) { return 0; }
int thorhip_malloc(void** ptr, size_t bytes) { return posix_memalign(ptr, 256, bytes ? bytes : 256) ? -1 : 0; }
int thorhip_free(void* ptr) { return std::free(ptr), 0; }
int thorhip_host_malloc(void** ptr, size_t bytes) { return posix_memalign(ptr, 256, bytes ? bytes : 256) ? -1 : 0; }
int thorhip_host_free(void* ptr) { return std::free(ptr), 0; }
int thorhip_memcpy_async(void* dst, const void* src, size_t bytes, int, void*) { return std::memcpy(dst, src, bytes), 0; }
int thorhip_memset_async(void* dst, int value, size_t bytes, void*) { return std::memset(dst, value, bytes), 0; }
int thorhip_mem_get_info(size_t* free_bytes, size_t* total_bytes) { return *free_bytes = *total_bytes = size_t(1) << 38, 0; }
int thorhip_stream_create(void** stream) { return *stream = std::malloc(8), 0; }
int thorhip_stream_destroy(void* stream) { return std::free(stream), 0; }
int thorhip_stream_synchronize(void*) { return 0; }
int thorhip_stream_wait_event(void*, void*) { return 0; }
int thorhip_stream_enqueue_host_function(void*, thorhip_host_fn fn, void* user_data) { return fn(user_data), 0; }
int thorhip_event_create(void** event, int) { return *event = std::malloc(8), 0; }
int thorhip_event_destroy(void* event) { return std::free(event), 0; }
int thorhip_event_record(void*, void*) { return 0; }
int thorhip_event_synchronize(void*) { return 0; }
int thorhip_event_elapsed_ms(float* ms, void*, void*) { return *ms = 0.0f, 0; }
int thorhip_module_load(void** module, const void*, size_t) { return *module = std::malloc(8), 0; }
int thorhip_module_unload(void* module) { return std::free(module), 0; }
int thorhip_module_get_function(void** function, void* module, const char*) { return *function = module, 0; }
int thorhip_function_get_attributes(void*, int* vgprs, int* lds, int* threads) {
    if (vgprs) *vgprs = 0;
    if (lds) *lds = 0;
    if (threads) *threads = 1024;
    return 0;
}
int thorhip_launch(void*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, void*, void**) { return 0; }
}

using namespace ThorImplementation;

static const TensorPlacement gpuPlacement(TensorPlacement::MemDevices::GPU, 0);
static int stamped = 0;

static void stampOne(const std::string& name, const Expression& e, const std::unordered_map<std::string, Tensor>& inputs, Stream& stream,
                     const char* expectKinds = nullptr) {
    std::printf("[ RUN  ] %s\n", name.c_str());
    std::fflush(stdout);
    FusedEquation eq = FusedEquation::compile(Expression::outputs({{"y", e}}).physicalOutputs(), 0);
    std::unordered_map<std::string, Tensor> used;
    for (const std::string& input : e.getInputNames()) used.emplace(input, inputs.at(input));
    StampedExecutionPlan plan = eq.stamp(used, stream);
    std::string kinds;
    for (const std::string& k : plan.stageKindNames()) kinds += (kinds.empty() ? "" : ",") + k;
    if (expectKinds && kinds != expectKinds) {
        std::printf("  unexpected plan: %s (wanted %s)\n", kinds.c_str(), expectKinds);
        std::exit(1);
    }
    ++stamped;
}

// the gradients of `e` with respect to every tensor input, for an upstream gradient of the output's shape
static void stampBackward(const std::string& name, const Expression& e, std::unordered_map<std::string, Tensor> inputs, const Tensor& upstream, Stream& stream,
                          const char* expectKinds = nullptr) {
    std::printf("[ RUN  ] %s\n", name.c_str());
    std::fflush(stdout);
    const FusedEquation forward = FusedEquation::compile(Expression::outputs({{"y", e}}).physicalOutputs(), 0);
    const FusedEquation backward = forward.compileBackward({}, std::string("__grad_output"));
    std::unordered_map<std::string, Tensor> used{{"__grad_output", upstream}};
    for (const std::string& input : e.getInputNames()) used.emplace(input, inputs.at(input));
    StampedExecutionPlan plan = backward.stamp(used, stream);
    std::string kinds;
    for (const std::string& k : plan.stageKindNames()) kinds += (kinds.empty() ? "" : ",") + k;
    if (expectKinds && kinds != expectKinds) {
        std::printf("  unexpected plan: %s (wanted %s)\n", kinds.c_str(), expectKinds);
        std::exit(1);
    }
    ++stamped;
}

static int runAll();

int main() {
    try {
        return runAll();
    } catch (const std::exception& e) {
        std::printf("  exception: %s\n", e.what());
        return 1;
    }
}

static int runAll() {
    Stream stream(0);
    const std::vector<std::pair<const char*, DataType>> floats = {{"fp16", DataType::FP16}, {"bf16", DataType::BF16}, {"fp32", DataType::FP32},
                                                                  {"e4m3", DataType::FP8_E4M3}};
    // a unary function feeding arithmetic with another tensor, flat kernels, every float dtype (16-bit float arithmetic is
    // where conversions meet packed instructions)
    const std::vector<std::pair<const char*, std::function<Expression(const Expression&)>>> unary = {
        {"exp", [](const Expression& v) { return v.exp(); }},       {"ln", [](const Expression& v) { return v.ln(); }},
        {"sqrt", [](const Expression& v) { return v.sqrt(); }},     {"tanh", [](const Expression& v) { return v.tanh(); }},
        {"sin", [](const Expression& v) { return v.sin(); }},       {"erf", [](const Expression& v) { return v.erf(); }},
        {"lgamma", [](const Expression& v) { return v.lgamma(); }}, {"sigmoid", [](const Expression& v) { return v.sigmoid(); }},
        {"gelu", [](const Expression& v) { return v.gelu(); }},     {"softplus", [](const Expression& v) { return v.softplus(); }},
        {"normcdf", [](const Expression& v) { return v.normcdf(); }}, {"log1p", [](const Expression& v) { return v.log1p(); }},
        {"abs", [](const Expression& v) { return v.abs(); }},       {"floor", [](const Expression& v) { return v.floor(); }}};
    for (const auto& [dtypeName, dtype] : floats) {
        Tensor a(gpuPlacement, TensorDescriptor(dtype, {4096, 24})), b(gpuPlacement, TensorDescriptor(dtype, {4096, 24}));
        const std::unordered_map<std::string, Tensor> inputs{{"a", a}, {"b", b}};
        const Expression x = Expression::input("a"), y = Expression::input("b");
        for (const auto& [opName, op] : unary) {
            stampOne(std::string("flat ") + dtypeName + " a - " + opName + "(b)", x - op(y), inputs, stream, "FusedKernel");
            stampOne(std::string("flat ") + dtypeName + " " + opName + "(a) * b + a", op(x) * y + x, inputs, stream, "FusedKernel");
        }
        stampOne(std::string("rows ") + dtypeName + " softmax", x.softmax(), inputs, stream);
        stampOne(std::string("rows ") + dtypeName + " log softmax", x.logSoftmax(), inputs, stream);
        stampOne(std::string("rows ") + dtypeName + " standardise",
                 (x - x.reduce_mean({1})) / ((x - x.reduce_mean({1})) * (x - x.reduce_mean({1}))).reduce_mean({1}).sqrt(), inputs, stream);
        stampOne(std::string("columns ") + dtypeName + " sum of a * ln(b)", (x * y.abs().ln()).reduce_sum({0}), inputs, stream);
        {  // operands that are broadcast along some of the kept axes: their offsets are worked out of the output's number
            Tensor image(gpuPlacement, TensorDescriptor(dtype, {6, 10, 9, 12})), bias(gpuPlacement, TensorDescriptor(dtype, {10, 1, 1}));
            Tensor gain(gpuPlacement, TensorDescriptor(dtype, {6, 1, 1, 1}));
            const Expression v = (Expression::input("image") + Expression::input("bias")) * Expression::input("gain");
            stampOne(std::string("per-image sums ") + dtypeName + " of (x + bias[C,1,1]) * gain[N,1,1,1]", v.reduce_sum({2, 3}),
                     {{"image", image}, {"bias", bias}, {"gain", gain}}, stream, "FusedReduction");
        }
        // backward equations: gradients of fused chains, row kernels that recompute the forward value, winner routing
        Tensor rowGradient(gpuPlacement, TensorDescriptor(dtype, {4096})), fullGradient(gpuPlacement, TensorDescriptor(dtype, {4096, 24}));
        stampBackward(std::string("backward ") + dtypeName + " tanh(a) * b + exp(a)", x.tanh() * y + x.exp(), inputs, fullGradient, stream, "FusedKernel");
        stampBackward(std::string("backward ") + dtypeName + " gelu(a) / softplus(b)", x.gelu() / y.softplus(), inputs, fullGradient, stream, "FusedKernel");
        stampBackward(std::string("backward ") + dtypeName + " softmax", x.softmax(), inputs, fullGradient, stream, "FusedRowKernel");
        stampBackward(std::string("backward ") + dtypeName + " log softmax", x.logSoftmax(), inputs, fullGradient, stream, "FusedRowKernel");
        stampBackward(std::string("backward ") + dtypeName + " row norms of a * b", (x * y).reduce_norm2({1}, {1}), inputs, rowGradient, stream);
        stampBackward(std::string("backward ") + dtypeName + " row max", x.reduce_max({1}, {1}), inputs, rowGradient, stream);
        stampBackward(std::string("backward ") + dtypeName + " column min of exp", x.exp().reduce_min({0}, {}),
                      inputs, Tensor(gpuPlacement, TensorDescriptor(dtype, {1, 24})), stream);
        // scans along the last axis, forward and as the backward of a sum scan; arg scans
        if (dtype != DataType::FP8_E4M3) {
            stampOne(std::string("scan ") + dtypeName + " running max of a * b", (x * y).scan(ScanOp::Max), inputs, stream, "FusedKernel,Scan");
            stampOne(std::string("scan ") + dtypeName + " exclusive sum - argmin", x.scan(ScanOp::Sum, -1, false), inputs, stream, "Scan");
            stampOne(std::string("scan ") + dtypeName + " argmin", x.scan(ScanOp::ArgMin), inputs, stream, "Scan");
            stampBackward(std::string("backward ") + dtypeName + " sum scan", x.scan(ScanOp::Sum), inputs, fullGradient, stream, "Scan");
            // one flat scan over several chunks: the kernels whose blocks publish their totals to each other
            stampOne(std::string("scan ") + dtypeName + " flat sum over 12 chunks", x.reshape({4096 * 24}).scan(ScanOp::Sum), inputs, stream, "Scan");
            stampOne(std::string("scan ") + dtypeName + " flat exclusive argmax over 12 chunks", x.reshape({4096 * 24}).scan(ScanOp::ArgMax, -1, false), inputs,
                     stream, "Scan");
        }
        // a scalar kept in device memory next to flat operands
        {
            std::printf("[ RUN  ] tensor scalar %s\n", dtypeName);
            std::fflush(stdout);
            const FusedEquation eq = FusedEquation::compile(Expression::outputs({{"y", (x * Expression::tensorRuntimeScalar("step") + y).tanh()}}).physicalOutputs(), 0);
            Tensor buffer(gpuPlacement, TensorDescriptor(DataType::FP32, {4}));
            StampedExecutionPlan plan = eq.stamp(inputs, stream, {{"step", TensorScalarBinding{buffer, 8, DataType::FP32}}});
            if (plan.stageKindNames() != std::vector<std::string>{"FusedKernel"}) {
                std::printf("  unexpected plan\n");
                std::exit(1);
            }
            ++stamped;
        }
        // gathers along an axis, with indices the same equation computes
        stampOne(std::string("gather ") + dtypeName + " value at the row argmax", (x * y).takeAlongAxis(x.argmax({1}, {}), 1), inputs, stream);
        stampOne(std::string("gather ") + dtypeName + " column picks", x.takeAlongAxis(y.argmin({0}, {}), 0) + 1.0, inputs, stream);
        // min / max scans backward: arg scan, cleared FP32 tensor, scatter-add
        if (dtype != DataType::FP8_E4M3) {
            Tensor upstream(gpuPlacement, TensorDescriptor(dtype, {4096, 24}));
            stampBackward(std::string("backward ") + dtypeName + " running max", x.scan(ScanOp::Max) * y, inputs, upstream, stream);
            stampBackward(std::string("backward ") + dtypeName + " exclusive reverse running min", x.reverseScan(ScanOp::Min, -1, false), inputs, upstream, stream);
        }
        // rotary position embedding: vector and scalar layouts, every scaling rule, explicit positions, backward
        {
            Tensor q(gpuPlacement, TensorDescriptor(dtype, {2, 4, 48, 64})), odd(gpuPlacement, TensorDescriptor(dtype, {3, 30, 7, 5}));
            Tensor positions(gpuPlacement, TensorDescriptor(DataType::UINT32, {48})), length(gpuPlacement, TensorDescriptor(DataType::INT32, {1}));
            const std::unordered_map<std::string, Tensor> ropeInputs{{"q", q}, {"odd", odd}, {"positions", positions}, {"length", length}};
            const Expression iq = Expression::input("q"), iodd = Expression::input("odd");
            RotaryPositionEmbeddingOptions o;
            stampOne(std::string("rope ") + dtypeName + " plain", iq.rope(o) * 2.0, ropeInputs, stream, "FusedKernel");
            stampOne(std::string("rope ") + dtypeName + " between products and sums", (iq * iq + iq.tanh()).rope(o) * iq + iq * 0.5, ropeInputs, stream,
                     "FusedKernel");
            o.interleaved = true;
            o.rotary_dim = 32;
            stampOne(std::string("rope ") + dtypeName + " interleaved partial", (iq + 1.0).rope(o), ropeInputs, stream);
            o = {};
            o.sequence_axis = 3;
            o.head_dim_axis = 1;
            stampOne(std::string("rope ") + dtypeName + " head dimension before sequence", iodd.rope(o), ropeInputs, stream);
            o = {};
            o.scaling_kind = RotaryScalingKind::Linear;
            o.scaling_factor = 2.0;
            stampOne(std::string("rope ") + dtypeName + " linear with ids", iq.rotaryPositionEmbeddingWithPositionIds(Expression::input("positions"), o), ropeInputs, stream);
            o.scaling_kind = RotaryScalingKind::DynamicNTK;
            o.original_max_position_embeddings = 16;
            stampOne(std::string("rope ") + dtypeName + " dynamic ntk with length",
                     iq.rotaryPositionEmbeddingWithEffectiveSequenceLength(Expression::input("length"), o), ropeInputs, stream);
            o.scaling_kind = RotaryScalingKind::Yarn;
            o.scaling_factor = 4.0;
            stampOne(std::string("rope ") + dtypeName + " yarn", iq.rope(o), ropeInputs, stream);
            o.scaling_kind = RotaryScalingKind::Llama3;
            o.inverse = true;
            stampOne(std::string("rope ") + dtypeName + " llama3 inverse", iq.rope(o), ropeInputs, stream);
            o = {};
            o.scaling_kind = RotaryScalingKind::LongRope;
            o.rotary_dim = 8;
            o.scaling_factor = 4.0;
            o.original_max_position_embeddings = 16;
            o.long_rope_short_factors = {1.0, 1.1, 1.2, 1.3};
            o.long_rope_long_factors = {2.0, 2.2, 2.4, 2.6};
            stampOne(std::string("rope ") + dtypeName + " longrope with ids and length",
                     iq.rotaryPositionEmbeddingWithPositionIdsAndEffectiveSequenceLength(Expression::input("positions"), Expression::input("length"), o),
                     ropeInputs, stream);
            if (dtype != DataType::FP8_E4M3) {
                Tensor upstream(gpuPlacement, TensorDescriptor(dtype, {2, 4, 48, 64}));
                stampBackward(std::string("backward rope ") + dtypeName + " longrope with ids", (iq * 3.0).rotaryPositionEmbeddingWithPositionIds(Expression::input("positions"), o),
                              ropeInputs, upstream, stream);
            }
        }
        // transposed and sliced operands: LDS-tiled and broadcast-form kernels, reductions over views
        Tensor t(gpuPlacement, TensorDescriptor(dtype, {24, 4096}));
        const std::unordered_map<std::string, Tensor> withT{{"a", a}, {"b", b}, {"t", t}};
        const Expression z = Expression::input("t");
        stampOne(std::string("tiled ") + dtypeName + " exp(t^T) - a", z.transpose().exp() - x, withT, stream, "FusedKernel");
        stampOne(std::string("tiled ") + dtypeName + " (a + t^T)^T", (x + z.transpose()).transpose() * z, withT, stream);
        stampOne(std::string("view ") + dtypeName + " half columns", x.stridedView({4096, 12}, {24, 1}, 12).tanh() * y.stridedView({4096, 12}, {24, 1}, 0),
                 withT, stream, "FusedKernel");
        stampOne(std::string("view ") + dtypeName + " row sums of t^T", z.transpose().reduce_sum({1}), withT, stream);
        if (dtype != DataType::FP8_E4M3) {
            Tensor halfUpstream(gpuPlacement, TensorDescriptor(dtype, {4096, 12}));
            stampBackward(std::string("backward ") + dtypeName + " gated halves of one input", x.stridedView({4096, 12}, {24, 1}, 12).tanh() * x.stridedView({4096, 12}, {24, 1}, 0),
                          inputs, halfUpstream, stream);
        }
    }
    // ragged batches: scalar and vector values, both offset dtypes, fused and index-gather paths
    for (const auto& [dtypeName, dtype] : floats) {
        if (dtype == DataType::FP8_E4M3) continue;
        for (uint64_t elements : {uint64_t(1), uint64_t(16), uint64_t(3)}) {
            for (DataType offsetsType : {DataType::UINT32, DataType::UINT64}) {
                const std::vector<uint64_t> trailing = elements > 1 ? std::vector<uint64_t>{elements} : std::vector<uint64_t>{};
                const RaggedExpression r = RaggedExpression::input("x", RaggedTensorDescriptor(dtype, trailing, 200, 6000, offsetsType));
                std::vector<uint64_t> dims{6000};
                if (elements > 1) dims.push_back(elements);
                const std::unordered_map<std::string, Tensor> inputs{{"x.values", Tensor(gpuPlacement, TensorDescriptor(dtype, dims))},
                                                                    {"x.offsets", Tensor(gpuPlacement, TensorDescriptor(offsetsType, {201}))}};
                const std::string tag = std::string("ragged ") + dtypeName + " E=" + std::to_string(elements) + (offsetsType == DataType::UINT64 ? " u64 " : " u32 ");
                // fp32 values: maximum and sum of exponentials come out of one pass over the values
                const char* softmaxStages = dtype == DataType::FP32 ? "FusedReduction,SegmentedBroadcast,FusedKernel"
                                                                    : "SegmentedReduction,FusedReduction,SegmentedBroadcast,FusedKernel";
                stampOne(tag + "softmax", r.segment_softmax().getValues(), inputs, stream, softmaxStages);
                stampOne(tag + "log softmax", r.segment_log_softmax().getValues(), inputs, stream, softmaxStages);
                stampOne(tag + "mean", r.segment_mean(), inputs, stream, "SegmentedReduction");
                {
                    std::vector<uint64_t> perSegment{200};
                    if (elements > 1) perSegment.push_back(elements);
                    stampBackward(tag + "backward of mean", r.segment_mean(), inputs, Tensor(gpuPlacement, TensorDescriptor(dtype, perSegment)), stream);
                    stampBackward(tag + "backward of max", r.segment_max(), inputs, Tensor(gpuPlacement, TensorDescriptor(dtype, perSegment)), stream);
                    stampBackward(tag + "backward of exp(sum) spread over rows",
                                  r.getValues().exp() * Expression::segmentedBroadcast(r.segment_sum(), r.getOffsets(), 200, 6000, elements, false), inputs,
                                  Tensor(gpuPlacement, TensorDescriptor(dtype, dims)), stream);
                }
                stampOne(tag + "relu * exp", (r.relu() * r.exp()).getValues(), inputs, stream, "FusedKernel");
                if (elements == 16) {
                    stampOne(tag + "sliced gate", (r.sliceLastDimension(0, 8).exp() * r.sliceLastDimension(8, 8)).getValues(), inputs, stream, "FusedKernel");
                    stampOne(tag + "sliced sum", r.sliceLastDimension(4, 8).segment_sum(), inputs, stream);
                }
            }
        }
    }
    // The primitives next to the expressions: their kernels are generated and compiled when a plan is prepared.  Top-k with and
    // without candidates (long and short inputs, keys and pairs, 32- and 16-bit keys), rows, select-flagged, scans over the
    // segments of an offsets tensor and over rows longer than a chunk, column reductions over an inner extent no vector divides.
    auto primitive = [&](const std::string& name, const std::function<void()>& prepare) {
        std::printf("[ RUN  ] %s\n", name.c_str());
        std::fflush(stdout);
        prepare();
        ++stamped;
    };
    for (const auto& [dtypeName, dtype] : std::vector<std::pair<const char*, DataType>>{{"fp32", DataType::FP32}, {"bf16", DataType::BF16}}) {
        for (const uint64_t n : {uint64_t(5000), uint64_t(1) << 21}) {
            Tensor keys(gpuPlacement, TensorDescriptor(dtype, {n})), best(gpuPlacement, TensorDescriptor(dtype, {64}));
            Tensor values(gpuPlacement, TensorDescriptor(DataType::UINT32, {n})), bestValues(gpuPlacement, TensorDescriptor(DataType::UINT32, {64}));
            primitive(std::string("top-k keys ") + dtypeName + " of " + std::to_string(n), [&] { (void)prepareCubDeviceTopKKeys(keys, best, n, 64, CubTopKOrder::Largest); });
            primitive(std::string("top-k pairs ") + dtypeName + " of " + std::to_string(n),
                      [&] { (void)prepareCubDeviceTopKPairs(keys, best, values, bestValues, n, 64, CubTopKOrder::Smallest); });
        }
        Tensor rows(gpuPlacement, TensorDescriptor(dtype, {256, 4096})), rowBest(gpuPlacement, TensorDescriptor(dtype, {256, 64}));
        primitive(std::string("top-k of rows ") + dtypeName, [&] { (void)prepareCubDeviceSegmentedTopKKeys(rows, rowBest, 256, 4096, 64, CubTopKOrder::Largest); });
        {  // rows a wavefront cannot hold (one block per row), rows searched bit by bit (more than 64 keys wanted), with values
            Tensor longRows(gpuPlacement, TensorDescriptor(dtype, {16, 8192})), longBest(gpuPlacement, TensorDescriptor(dtype, {16, 100}));
            Tensor rowValues(gpuPlacement, TensorDescriptor(DataType::UINT32, {16, 8192})), bestRowValues(gpuPlacement, TensorDescriptor(DataType::UINT32, {16, 100}));
            primitive(std::string("top-k pairs of long rows ") + dtypeName,
                      [&] { (void)prepareCubDeviceSegmentedTopKPairs(longRows, longBest, rowValues, bestRowValues, 16, 8192, 100, CubTopKOrder::Smallest); });
            primitive(std::string("top-k pairs of rows, k = 100 ") + dtypeName,
                      [&] { (void)prepareCubDeviceSegmentedTopKPairs(longRows, longBest, rowValues, bestRowValues, 16, 4096, 100, CubTopKOrder::Largest); });
            Tensor manyKeys(gpuPlacement, TensorDescriptor(dtype, {uint64_t(1) << 24})), manyBest(gpuPlacement, TensorDescriptor(dtype, {uint64_t(1) << 16}));
            primitive(std::string("top-k keys ") + dtypeName + ", 65536 of 2^24",
                      [&] { (void)prepareCubDeviceTopKKeys(manyKeys, manyBest, uint64_t(1) << 24, uint64_t(1) << 16, CubTopKOrder::Largest); });
        }
        Tensor x(gpuPlacement, TensorDescriptor(dtype, {uint64_t(1) << 20})), y(gpuPlacement, TensorDescriptor(dtype, {uint64_t(1) << 20}));
        Tensor flags(gpuPlacement, TensorDescriptor(DataType::UINT8, {uint64_t(1) << 20})), count(gpuPlacement, TensorDescriptor(DataType::UINT32, {1}));
        primitive(std::string("select-flagged ") + dtypeName, [&] { (void)prepareCubDeviceSelectFlagged(x, flags, y, count, uint64_t(1) << 20); });
        Tensor offsets(gpuPlacement, TensorDescriptor(DataType::UINT32, {101}));
        for (uint32_t i = 0; i <= 100; ++i) static_cast<uint32_t*>(offsets.getMemPtr())[i] = i * 10000u;
        primitive(std::string("scan over offset segments ") + dtypeName,
                  [&] { (void)prepareCubDeviceSegmentedScan(x, y, offsets, 1000000, 100, CubScanOp::Max, CubScanMode::Exclusive, CubScanDirection::Reverse); });
        primitive(std::string("scan over rows longer than a chunk ") + dtypeName, [&] {
            (void)prepareCubDeviceSegmentedUniformScan(x, y, uint64_t(1) << 20, 16, uint64_t(1) << 16, CubScanOp::Sum, CubScanMode::Inclusive, CubScanDirection::Forward);
        });
        Tensor odd(gpuPlacement, TensorDescriptor(dtype, {300, 1001}));
        primitive(std::string("column sum over an inner extent of 1001 ") + dtypeName, [&] { (void)CubReduction(CubReductionOp::Sum, {0}, DataType::FP32).stamp(odd, stream); });
        primitive(std::string("column arg-max over an inner extent of 1001 ") + dtypeName, [&] { (void)CubArgReduction(CubArgReductionOp::ArgMax, {0}).stamp(odd, stream); });
    }
    // A kernel whose machine code shifts 64 bits by an amount held in a vector register numbered 8n+7 must be refused when it is
    // loaded (the device computes that shift wrong when the register is the last one a wavefront owns); the same kernel with the
    // amount one register lower must load.
    {
        const auto shifting = [](int amountRegister) {
            const std::string reg = "v" + std::to_string(amountRegister);
            return "extern \"C\" __global__ void shift_probe(unsigned long long* out) {\n    unsigned long long r;\n    const unsigned lane = threadIdx.x & 63u;\n"
                   "    asm volatile(\"v_mov_b32 " + reg + ", %1\\n s_nop 4\\n v_lshlrev_b64 %0, " + reg + ", -1\" : \"=&v\"(r) : \"v\"(lane) : \"" + reg +
                   "\");\n    out[threadIdx.x] = r;\n}\n";
        };
        std::printf("[ RUN  ] a 64-bit shift by v14 loads, by v15 is refused\n");
        (void)compileKernel(shifting(14), "shift_probe", 0, false);
        bool refused = false;
        try {
            (void)compileKernel(shifting(15), "shift_probe", 0, false);
        } catch (const std::runtime_error& e) {
            refused = std::string(e.what()).find("64-bit vector shift") != std::string::npos;
        }
        if (!refused) {
            std::printf("  a kernel with v_lshlrev_b64 by v15 was loaded\n");
            return 1;
        }
    }
    std::printf("%d expressions stamped, 0 failures\n", stamped);
    return 0;
}
