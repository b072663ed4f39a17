// Exercises the C++ API (namespace ThorImplementation) directly, the way the reference's gtest suites do
// (test/Utilities/TensorOperations/CubReductionValueOperationsTest.cpp, CubArgReductionTest.cpp,
//  CubReductionGeometryTest.cpp, test/Utilities/Expression/CommonInputFusionTest.cpp,
//  test/Utilities/TensorOperations/DataTypeConversions).  Plain asserts instead of gtest: the image has no gtest.
// Usage: test_cpp_api [host|gpu]   (host: the cases that need no GPU)
#include "DeepLearning/Implementation/Tensor/Tensor.h"
#include "Utilities/Common/Stream.h"
#include "Utilities/Expression/Expression.h"
#include "Utilities/Expression/ExpressionDTypeResolution.h"
#include "Utilities/Expression/AutoDiff.h"
#include "Utilities/Expression/FusedEquation.h"
#include "Utilities/Expression/RaggedExpression.h"
#include "Utilities/TensorOperations/Cub/CubDevicePrimitives.h"
#include "Utilities/TensorOperations/Cub/CubReduction.h"
#include "Utilities/TensorOperations/DataTypeConversions/TypeConverter.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <limits>
#include <optional>
#include <set>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

using namespace ThorImplementation;

static int failures = 0;
static int checks = 0;
#define CHECK(cond)                                                                     \
    do {                                                                                \
        ++checks;                                                                       \
        if (!(cond)) {                                                                  \
            ++failures;                                                                 \
            std::printf("  CHECK failed %s:%d: %s\n", __FILE__, __LINE__, #cond);       \
        }                                                                               \
    } while (0)
#define CHECK_NEAR(a, b, tol) CHECK(std::fabs(double(a) - double(b)) <= (tol))
template <typename E, typename F>
static bool throwsAs(F&& f) {
    try {
        f();
    } catch (const E&) {
        return true;
    } catch (...) {
        return false;
    }
    return false;
}

static const TensorPlacement cpuPlacement(TensorPlacement::MemDevices::CPU);
static const TensorPlacement gpuPlacement(TensorPlacement::MemDevices::GPU, 0);

static Tensor gpuFrom(const std::vector<float>& values, const std::vector<uint64_t>& dims, Stream& stream, DataType dtype = DataType::FP32) {
    Tensor host(cpuPlacement, TensorDescriptor(DataType::FP32, dims));
    std::memcpy(host.getMemPtr<float>(), values.data(), values.size() * sizeof(float));
    Tensor device(gpuPlacement, TensorDescriptor(dtype, dims));
    device.copyFromAsync(host, stream);  // converts when the dtypes differ
    stream.synchronize();
    return device;
}

static std::vector<float> toHostF32(const Tensor& t, Stream& stream) {
    Tensor host(cpuPlacement, TensorDescriptor(DataType::FP32, t.getDimensions()));
    host.copyFromAsync(t, stream);
    stream.synchronize();
    const float* p = host.getMemPtr<float>();
    return std::vector<float>(p, p + host.getTotalNumElements());
}

template <typename T>
static std::vector<T> toHostRaw(const Tensor& t, Stream& stream) {
    Tensor host(cpuPlacement, TensorDescriptor(t.getDataType(), t.getDimensions()));
    host.copyFromAsync(t, stream);
    stream.synchronize();
    const T* p = host.getMemPtr<T>();
    return std::vector<T>(p, p + host.getTotalNumElements());
}

// ---- host-only cases -----------------------------------------------------------------------------------------------------
static void geometryPathsAndErrors() {
    // CubReductionGeometryTest.cpp: path selection and argument validation by exception type
    CHECK(CubReduction::analyzeGeometry({8192, 8192}, std::vector<uint32_t>{0, 1}).path == CubReductionPath::DeviceTransformReduce);
    const CubReductionGeometry rows = CubReduction::analyzeGeometry({8192, 4096}, 1);
    CHECK(rows.path == CubReductionPath::ContiguousFixedSegment && rows.outer_size == 8192 && rows.reduction_size == 4096 && rows.inner_size == 1);
    const CubReductionGeometry tiled = CubReduction::analyzeGeometry({4, 5, 6}, 1);
    CHECK(tiled.path == CubReductionPath::TiledFixedSegment && tiled.outer_size == 4 && tiled.reduction_size == 5 && tiled.inner_size == 6);
    const CubReductionGeometry strided = CubReduction::analyzeGeometry({64, 256, 56, 56}, std::vector<uint32_t>{0, 2, 3});
    CHECK(strided.path == CubReductionPath::StridedFixedSegment && strided.output_elements == 256 && strided.reduction_size == 64ull * 56 * 56);
    CHECK((strided.squeezed_output_dimensions == std::vector<uint64_t>{256}));
    CHECK(throwsAs<std::invalid_argument>([] { CubReduction::analyzeGeometry({4, 5}, 2); }));
    CHECK(throwsAs<std::invalid_argument>([] { CubReduction::analyzeGeometry({4, 5}, std::vector<uint32_t>{1, 1}); }));
    CHECK(throwsAs<std::invalid_argument>([] { CubReduction::analyzeGeometry({}, 0); }));
    CHECK(CubReduction::getFp32EmptyReductionValue(CubReductionOp::Product) == 1.0f);
    CHECK(CubReduction::getFp32EmptyReductionValue(CubReductionOp::Min) == std::numeric_limits<float>::infinity());
    CHECK(CubArgReduction::getEmptyReductionIndex() == std::numeric_limits<uint64_t>::max());
    // logical (output, reduction) coordinates -> physical offsets on a [2,3,2] tensor reduced over {0,2}
    const CubReductionGeometry g = CubReduction::analyzeGeometry({2, 3, 2}, std::vector<uint32_t>{0, 2});
    CHECK(CubReduction::mapLogicalReductionIndexToPhysicalIndex(g, 1, 0) == 2);
    CHECK(CubReduction::mapLogicalReductionIndexToPhysicalIndex(g, 1, 3) == 6 + 2 + 1);
}

static void dtypeResolutionAndStageSplit() {
    // CommonInputFusionTest.cpp:281-303: a reduction boundary splits stages; dtype rules of ExpressionDTypeResolution.cpp
    Expression x = Expression::input("x"), y = Expression::input("y");
    Expression trunk = x + y;
    Outputs outs = Expression::outputs({{"trunk", trunk}, {"sum_last", trunk.reduce_sum({1}, {})}});
    PhysicalOutputs physical = outs.physicalOutputs();
    resolveOutputsDTypesInPlace(physical, {DataType::FP16, DataType::BF16});
    for (const NamedOutput& o : physical.outputs) {
        const ExprNode& node = physical.expr->nodes[o.node_idx];
        if (o.name == "trunk") CHECK(node.output_dtype == DataType::FP32);  // fp16 with bf16 promotes to fp32
        if (o.name == "sum_last") CHECK(node.output_dtype == DataType::FP32 && node.compute_dtype == DataType::FP32);
    }
    Expression s = Expression::input("d").sigmoid();
    const PhysicalExpression p = s.expression();
    CHECK(canonicalize(p) == "div(exp(neg(max(neg(input#0),scalar(0)))),add(exp(neg(abs(input#0))),scalar(1)))");
    CHECK(throwsAs<std::runtime_error>([&] {
        PhysicalOutputs bad = Expression::outputs({{"o", x + y}}).physicalOutputs();
        resolveOutputsDTypesInPlace(bad, {DataType::UINT8, DataType::FP16});
    }));
}

static void cpuTypeConverter() {
    // the reference's CPU path (TypeConverter.cpp:899-942): RNE, +-Inf on overflow, gradual underflow, fp8 satfinite
    const std::vector<float> in = {1.0f, 65504.0f, 65520.0f, 1e5f, -1e5f, 5.9604645e-8f, 2.9802322e-8f, 1e-40f, 448.0f, 1e6f};
    std::vector<uint16_t> h(in.size()), b(in.size());
    std::vector<uint8_t> e4(in.size()), e5(in.size());
    TypeConverter::cpuConvertNow(in.data(), h.data(), DataType::FP32, DataType::FP16, in.size());
    TypeConverter::cpuConvertNow(in.data(), b.data(), DataType::FP32, DataType::BF16, in.size());
    TypeConverter::cpuConvertNow(in.data(), e4.data(), DataType::FP32, DataType::FP8_E4M3, in.size());
    TypeConverter::cpuConvertNow(in.data(), e5.data(), DataType::FP32, DataType::FP8_E5M2, in.size());
    CHECK(h[0] == 0x3C00 && h[1] == 0x7BFF && h[2] == 0x7C00 && h[3] == 0x7C00 && h[4] == 0xFC00);
    CHECK(h[5] == 0x0001 && h[6] == 0x0000 && h[7] == 0x0000);  // 2^-24 is the smallest subnormal; 2^-25 ties to even (zero)
    CHECK(b[0] == 0x3F80 && b[3] == 0x47C3 && b[7] == 0x0001);  // 1e5 -> 0x47C35000 rounds to 0x47C3 ; 1e-40 is a bf16 subnormal
    CHECK(e4[8] == 0x7E && e4[9] == 0x7E);                      // 448 is the largest e4m3 value and everything above saturates to it
    CHECK(e5[9] == 0x7B);                                       // 57344 saturating
    std::vector<float> back(in.size());
    TypeConverter::cpuConvertNow(h.data(), back.data(), DataType::FP16, DataType::FP32, in.size());
    CHECK(back[0] == 1.0f && back[1] == 65504.0f && std::isinf(back[2]) && back[5] == 5.9604645e-8f);
}

// ---- GPU cases -------------------------------------------------------------------------------------------------------------
static void valueReductionsSmallExact(Stream& stream) {
    // CubReductionValueOperationsTest.cpp: small integers, exact in fp32 whatever the order
    Tensor v = gpuFrom({-2.0f, 3.0f, -4.0f}, {3}, stream);
    auto run = [&](CubReductionOp op, const Tensor& t, std::vector<uint32_t> axes, float scale = 1.0f) {
        auto stamped = CubReduction(op, axes, DataType::FP32, scale).stamp(t, stream);
        stamped->run();
        return toHostF32(stamped->getOutputTensor(), stream);
    };
    CHECK(run(CubReductionOp::Sum, v, {0})[0] == -3.0f);
    CHECK(run(CubReductionOp::Min, v, {0})[0] == -4.0f);
    CHECK(run(CubReductionOp::Max, v, {0})[0] == 3.0f);
    CHECK(run(CubReductionOp::Product, v, {0})[0] == 24.0f);
    CHECK(run(CubReductionOp::Mean, v, {0})[0] == -1.0f);
    CHECK(run(CubReductionOp::L1Norm, v, {0})[0] == 9.0f);
    CHECK_NEAR(run(CubReductionOp::L2Norm, v, {0})[0], std::sqrt(29.0), 1e-6);
    CHECK(run(CubReductionOp::Sum, v, {0}, 0.5f)[0] == -1.5f);
    Tensor m = gpuFrom({-1, 2, -3, 4, -5, 6}, {2, 3}, stream);
    CHECK((run(CubReductionOp::Sum, m, {1}) == std::vector<float>{-2, 5}));
    CHECK((run(CubReductionOp::Sum, m, {0}) == std::vector<float>{3, -3, 3}));
    CHECK((run(CubReductionOp::Max, m, {0, 1}) == std::vector<float>{6}));
    Tensor nan = gpuFrom({1.0f, std::nanf(""), 3.0f}, {3}, stream);
    CHECK(std::isnan(run(CubReductionOp::Max, nan, {0})[0]) && std::isnan(run(CubReductionOp::Min, nan, {0})[0]));
    // output dtype and satfinite for fp8 (CubReductionDTypeAndLifecycleTest.cpp:205-222)
    Tensor big = gpuFrom({400.0f, 400.0f}, {2}, stream);
    auto e4 = CubReduction(CubReductionOp::Sum, 0u, DataType::FP8_E4M3).stamp(big, stream);
    e4->run();
    CHECK(toHostF32(e4->getOutputTensor(), stream)[0] == 448.0f);
    CHECK(e4->getOutputDataType() == DataType::FP8_E4M3 && e4->getAccumulatorDataType() == DataType::FP32);
    CHECK(throwsAs<std::invalid_argument>([&] { CubReduction(CubReductionOp::Sum, 3u).stamp(m, stream); }));
}

static Tensor gpuOffsets(const std::vector<uint64_t>& values, Stream& stream, DataType dtype = DataType::UINT32) {
    Tensor host(cpuPlacement, TensorDescriptor(dtype, {values.size()}));
    for (size_t i = 0; i < values.size(); ++i) {
        if (dtype == DataType::UINT64)
            host.getMemPtr<uint64_t>()[i] = values[i];
        else
            host.getMemPtr<uint32_t>()[i] = static_cast<uint32_t>(values[i]);
    }
    Tensor device(gpuPlacement, TensorDescriptor(dtype, {values.size()}));
    device.copyFromAsync(host, stream);
    stream.synchronize();
    return device;
}

static void offsetSegmentedReductions(Stream& stream) {
    const float inf = std::numeric_limits<float>::infinity();
    // CubOffsetSegmentedReductionTest.cpp:29-45: scalar rows, an empty segment, skewed lengths
    Tensor x = gpuFrom({1, -2, 4, 5, 7, -1, 8, 99, 100}, {9}, stream);
    Tensor offsets = gpuOffsets({0, 3, 3, 5, 7}, stream);
    auto run = [&](CubReductionOp op) {
        auto stamped = CubSegmentedReduction(op, DataType::FP32).stamp(x, offsets, stream);
        CHECK(stamped->getPath() == CubReductionPath::OffsetSegmented);
        stamped->run();
        return toHostF32(stamped->getOutputTensor(), stream);
    };
    CHECK((run(CubReductionOp::Sum) == std::vector<float>{3, 0, 12, 7}));
    CHECK((run(CubReductionOp::Mean) == std::vector<float>{1, 0, 6, 3.5f}));
    CHECK((run(CubReductionOp::Min) == std::vector<float>{-2, inf, 5, -1}));
    CHECK((run(CubReductionOp::Max) == std::vector<float>{4, -inf, 7, 8}));
    // :116-157: vector values, packed indices row * D + d, NaN wins, lowest index wins ties, all-ones for empty segments
    Tensor v = gpuFrom({2, 7, 5, -1, 7, 6, -1, 4, std::nanf(""), 6, 1, 9, 5, 1, 8}, {5, 3}, stream);
    Tensor vOffsets = gpuOffsets({0, 3, 3, 5}, stream, DataType::UINT64);
    const uint64_t none = std::numeric_limits<uint64_t>::max();
    auto argMin = CubSegmentedArgReduction(CubArgReductionOp::ArgMin).stamp(v, vOffsets, stream);
    argMin->run();
    CHECK((toHostRaw<uint64_t>(argMin->getIndexOutputTensor(), stream) == std::vector<uint64_t>{3, 7, 8, none, none, none, 12, 10, 14}));
    auto argMax = CubSegmentedArgReduction(CubArgReductionOp::ArgMax, DataType::UINT32).stamp(v, vOffsets, stream);
    argMax->run();
    const uint32_t none32 = std::numeric_limits<uint32_t>::max();
    CHECK((toHostRaw<uint32_t>(argMax->getIndexOutputTensor(), stream) == std::vector<uint32_t>{0, 1, 8, none32, none32, none32, 9, 10, 11}));
    // :239-295: runtime offsets are read by the kernels, not by the stamp
    Tensor y = gpuFrom({1, 2, 3, 4, 5, 6}, {6}, stream);
    Tensor runtimeOffsets = gpuOffsets({9, 9, 9, 9}, stream);
    Tensor out(gpuPlacement, TensorDescriptor(DataType::FP32, {3}));
    CHECK(throwsAs<std::invalid_argument>([&] { CubSegmentedReduction(CubReductionOp::Mean, DataType::FP32).stamp(y, out, runtimeOffsets, stream); }));
    auto dynamic = CubSegmentedReduction(CubReductionOp::Mean, DataType::FP32).stampRuntimeOffsets(y, out, runtimeOffsets, stream);
    runtimeOffsets.copyFromAsync(gpuOffsets({0, 2, 2, 6}, stream), stream);
    dynamic->run();
    CHECK((toHostF32(out, stream) == std::vector<float>{1.5f, 0.0f, 4.5f}));
    runtimeOffsets.copyFromAsync(gpuOffsets({0, 1, 4, 6}, stream), stream);
    dynamic->run();
    CHECK((toHostF32(out, stream) == std::vector<float>{1.0f, 3.0f, 5.5f}));
    // :457-511: contract violations
    CHECK(throwsAs<std::invalid_argument>([&] { CubSegmentedReduction(CubReductionOp::Product); }));
    CHECK(throwsAs<std::invalid_argument>([&] { CubSegmentedReduction(CubReductionOp::Sum).stamp(x, gpuOffsets({1, 3, 9}, stream), stream); }));
    CHECK(throwsAs<std::invalid_argument>([&] { CubSegmentedReduction(CubReductionOp::Sum).stamp(x, gpuOffsets({0, 5, 3}, stream), stream); }));
    CHECK(throwsAs<std::invalid_argument>([&] { CubSegmentedReduction(CubReductionOp::Sum).stamp(x, gpuOffsets({0, 5, 10}, stream), stream); }));
}

static void autodiffGraphStructure() {
    // buildBackwardOutputs builds gradients as one more expression graph (AutoDiff.h:15-27, AutoDiff.cpp:2486-2581 there)
    const Expression x = Expression::input("x"), w = Expression::input("w");
    const PhysicalOutputs forward = Expression::outputs({{"y", (x * w).tanh()}}).physicalOutputs();
    const std::unordered_map<std::string, std::vector<uint64_t>> dims{{"x", {4, 3}}, {"w", {3}}};
    const PhysicalOutputs backward = buildBackwardOutputs(forward, {"x", "w"}, std::string(DEFAULT_BACKWARD_UPSTREAM_INPUT_NAME), dims);
    CHECK(backward.outputs.size() == 2 && backward.outputs[0].name == "x_grad" && backward.outputs[1].name == "w_grad");
    CHECK((backward.expr->getInputNames() == std::set<std::string>{"x", "w", "__grad_output"}));
    auto count = [&](ExprOp op) {
        int n = 0;
        for (const ExprNode& node : backward.expr->nodes) n += node.op == op;
        return n;
    };
    CHECK(count(ExprOp::TANH) == 1);        // the forward value is copied once and shared by both gradients
    CHECK(count(ExprOp::REDUCE_SUM) == 1);  // w was broadcast over rows: its gradient is summed back to [3]
    for (const ExprNode& node : backward.expr->nodes) {
        if (node.op == ExprOp::REDUCE_SUM) CHECK(node.reduction_axes == (std::vector<uint64_t>{0}) && node.squeeze_axes == (std::vector<uint64_t>{0}));
    }
    // implicit upstream: ones of the output's shape; a gradient nothing reaches is zeros of the input's shape
    const PhysicalOutputs implicit = buildBackwardOutputs(Expression::outputs({{"y", x.exp()}, }).physicalOutputs(), {"x"}, std::nullopt, dims);
    bool seeded = false;
    for (const ExprNode& node : implicit.expr->nodes) seeded = seeded || (node.op == ExprOp::FILL && node.scalar_fp == 1.0 && node.fill_dims == dims.at("x"));
    CHECK(seeded);
    CHECK(throwsAs<std::runtime_error>([&] { (void)buildBackwardOutputs(forward, {"x"}, std::string("w"), dims); }));        // collides with an input
    CHECK(throwsAs<std::runtime_error>([&] { (void)buildBackwardOutputs(forward, {"nope"}, std::nullopt, dims); }));         // unknown input
    CHECK(throwsAs<std::runtime_error>([&] { (void)buildBackwardOutputs(forward, {"x", "x"}, std::nullopt, dims); }));       // duplicate
    {
        // the shape-free forms (AutoDiff.h:15-27 there: forward_input_dims defaults to nullopt in every overload): the implicit seed
        // is the scalar 1, nothing is summed back or expanded, rules that need a shape say so
        const PhysicalOutputs shapeless = buildBackwardOutputs(forward, {"x", "w"});
        CHECK(shapeless.outputs.size() == 2 && shapeless.outputs[0].name == "x_grad" && shapeless.outputs[1].name == "w_grad");
        int sums = 0, fills = 0, ones = 0;
        for (const ExprNode& node : shapeless.expr->nodes) {
            sums += node.op == ExprOp::REDUCE_SUM;
            fills += node.op == ExprOp::FILL;
            ones += node.op == ExprOp::SCALAR_FP && node.scalar_fp == 1.0;
        }
        CHECK(sums == 0 && fills == 0 && ones >= 1);
        CHECK((shapeless.expr->getInputNames() == std::set<std::string>{"x", "w"}));
        const PhysicalOutputs named = buildBackwardOutputs(forward, {"x"}, std::unordered_map<std::string, std::string>{{"y", "__gy"}});
        CHECK((named.expr->getInputNames() == std::set<std::string>{"x", "w", "__gy"}));
        const PhysicalOutputs summed = buildBackwardOutputs(Expression::outputs({{"s", (x * x).reduce_sum({1}, {})}}).physicalOutputs(), {"x"});
        CHECK(summed.outputs.size() == 1);  // a reduction that keeps its axes broadcasts back by itself
        CHECK(throwsAs<std::runtime_error>([&] { (void)buildBackwardOutputs(Expression::outputs({{"r", x.reshape({12})}}).physicalOutputs(), {"x"}); }));
        CHECK(throwsAs<std::runtime_error>([&] { (void)buildBackwardOutputs(Expression::outputs({{"m", x.reduce_mean({1}, {})}}).physicalOutputs(), {"x"}); }));
        CHECK(throwsAs<std::runtime_error>([&] { (void)buildBackwardOutputs(Expression::outputs({{"m", x.reduce_sum({1}, {1})}}).physicalOutputs(), {"x"}); }));
        // the overloads that carry the seeds' runtime dtypes, or take the seeds from the forward graph (AutoDiff.h:29-48 there)
        const std::unordered_map<std::string, std::string> seedNames{{"y", "__gy"}};
        const PhysicalOutputs typedSeed = buildBackwardOutputs(forward, {"x"}, seedNames, std::unordered_map<std::string, DataType>{{"y", DataType::FP16}}, dims);
        bool carries = false;
        for (const ExprNode& node : typedSeed.expr->nodes) {
            carries = carries || (node.op == ExprOp::INPUT && typedSeed.expr->inputs.at(node.input_slot).name == "__gy" && node.output_dtype == DataType::FP16);
        }
        CHECK(carries);
        CHECK(throwsAs<std::runtime_error>([&] { (void)buildBackwardOutputs(forward, {"x"}, seedNames, std::unordered_map<std::string, DataType>{}, dims); }));
        const PhysicalOutputs nodeSeed =
            buildBackwardOutputs(forward, {"x"}, seedNames, std::unordered_map<std::string, uint32_t>{{"y", forward.outputs[0].node_idx}}, dims);
        CHECK((nodeSeed.expr->getInputNames() == std::set<std::string>{"x", "w"}));  // the seed is tanh(x * w) itself: no gradient input
    }
    {
        // the reference's softmax spelling (Expression.h:736-738 there takes cuDNN's enumerations): the same nodes as this build's own
        const Expression a = x.softmax(CUDNN_SOFTMAX_ACCURATE, CUDNN_SOFTMAX_MODE_CHANNEL), b = x.softmax(SoftmaxAlgorithm::Accurate, SoftmaxMode::Channel);
        CHECK(a.expression().nodes.back().softmax_algorithm == b.expression().nodes.back().softmax_algorithm);
        CHECK(a.expression().nodes.back().softmax_mode == SoftmaxMode::Channel);
        CHECK(x.softmax(CUDNN_SOFTMAX_FAST, CUDNN_SOFTMAX_MODE_INSTANCE).expression().nodes.back().softmax_mode == SoftmaxMode::Instance);
        CHECK(x.logSoftmax(CUDNN_SOFTMAX_MODE_INSTANCE).expression().nodes.back().softmax_algorithm == SoftmaxAlgorithm::Log);
        CHECK(throwsAs<std::invalid_argument>([&] { (void)x.softmax(CUDNN_SOFTMAX_LOG); }));
    }
    CHECK(throwsAs<std::runtime_error>([&] {
        (void)buildBackwardOutputs(Expression::outputs({{"y", x.floor() * w}}).physicalOutputs(), {"x"}, std::nullopt, dims);  // no rule for floor
    }));
    const PhysicalOutputs two = Expression::outputs({{"a", x + w}, {"b", x - w}}).physicalOutputs();
    CHECK(throwsAs<std::runtime_error>([&] { (void)buildBackwardOutputs(two, {"x"}, std::nullopt, dims); }));  // several outputs need a seed map
    const PhysicalOutputs partial = buildBackwardOutputs(two, {"w"}, std::unordered_map<std::string, std::string>{{"b", "__gb"}}, dims);
    CHECK((partial.expr->getInputNames() == std::set<std::string>{"__gb"}));  // d(x - w)/dw = -g, summed over rows: no forward value needed
    // take_along_axis is an index-aware binary op: the axis rides in reduction_axes, indices must be integral
    // (ExpressionConvenienceOpsTest.cpp:357-383 there)
    PhysicalOutputs take = Expression::outputs({{"y", x.takeAlongAxis(w, 1)}}).physicalOutputs();
    const ExprNode& takeNode = take.expr->nodes.at(take.outputs[0].node_idx);
    CHECK(takeNode.op == ExprOp::TAKE_ALONG_AXIS && takeNode.reduction_axes == (std::vector<uint64_t>{1}));
    CHECK(take.expr->nodes.at(takeNode.lhs).op == ExprOp::INPUT && take.expr->nodes.at(takeNode.rhs).op == ExprOp::INPUT);
    CHECK(throwsAs<std::runtime_error>([&] {
        PhysicalOutputs floatIndices = Expression::outputs({{"y", x.takeAlongAxis(w, 1)}}).physicalOutputs();
        resolveOutputsDTypesInPlace(floatIndices, {DataType::FP32, DataType::FP32});
    }));
    resolveOutputsDTypesInPlace(take, {DataType::FP16, DataType::UINT32});
    CHECK(take.expr->nodes.at(take.outputs[0].node_idx).output_dtype == DataType::FP16);
    CHECK(throwsAs<std::invalid_argument>([&] { (void)x.takeAlongAxis(w, -2); }));
    // offsets of a ragged batch are structure
    const Expression offsets = Expression::input("offsets");
    const PhysicalOutputs ragged = Expression::outputs({{"s", Expression::segmentedReduceSum(x, offsets)}}).physicalOutputs();
    CHECK(throwsAs<std::runtime_error>([&] { (void)buildBackwardOutputs(ragged, {"offsets"}, std::nullopt, {{{"x", {4, 3}}, {"offsets", {3}}}}); }));
    CHECK((normalizeBackwardWrtNames(*ragged.expr, {}) == std::vector<std::string>{"x"}));
}

static void scanExpressionStructure() {
    // Expression::scan builds a SCAN node that carries op, mode and axis (Expression.cpp:3908-3922 there); arg scans resolve to
    // UINT32, value scans keep the input dtype; segmented scans take offsets as structure
    const Expression x = Expression::input("x"), offsets = Expression::input("offsets");
    PhysicalOutputs scan = Expression::outputs({{"y", x.scan(ScanOp::Max, -1, false)}}).physicalOutputs();
    const ExprNode& node = scan.expr->nodes.at(scan.outputs[0].node_idx);
    CHECK(node.op == ExprOp::SCAN && node.scan_op == ScanOp::Max && node.scan_mode == ScanMode::Exclusive && node.scan_axis == UINT64_MAX && !node.scan_reverse);
    resolveOutputsDTypesInPlace(scan, {DataType::BF16});
    CHECK(scan.expr->nodes.at(scan.outputs[0].node_idx).output_dtype == DataType::BF16);
    PhysicalOutputs arg = Expression::outputs({{"y", x.segmentedScan(offsets, ScanOp::ArgMin, true, true)}}).physicalOutputs();
    const ExprNode& argNode = arg.expr->nodes.at(arg.outputs[0].node_idx);
    CHECK(argNode.op == ExprOp::SEGMENTED_SCAN && argNode.scan_reverse && arg.expr->nodes.at(argNode.rhs).op == ExprOp::INPUT);
    resolveOutputsDTypesInPlace(arg, {DataType::FP32, DataType::UINT64});
    CHECK(arg.expr->nodes.at(arg.outputs[0].node_idx).output_dtype == DataType::UINT32);
    CHECK(throwsAs<std::runtime_error>([&] {
        PhysicalOutputs bad = Expression::outputs({{"y", x.scan(ScanOp::Sum)}}).physicalOutputs();
        resolveOutputsDTypesInPlace(bad, {DataType::INT32});
    }));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)x.scan(ScanOp::Sum, -2); }));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)x.scanWithIndices(ScanOp::Sum); }));
    const auto [values, indices] = x.scanWithIndices(ScanOp::Min);
    CHECK(values.expression().nodes.back().scan_op == ScanOp::Min && indices.expression().nodes.back().scan_op == ScanOp::ArgMin);
    const PhysicalExpression count = (x > Expression(0.0)).prefixCount().expression();
    CHECK(count.nodes.back().op == ExprOp::SCAN && count.nodes.at(count.nodes.back().lhs).op == ExprOp::CAST);
    // the gradient of a sum scan is the scan from the other end (AutoDiff.cpp there: reverse-scan lowering)
    const PhysicalOutputs forward = Expression::outputs({{"y", x.scan(ScanOp::Sum, -1, false)}}).physicalOutputs();
    const PhysicalOutputs backward = buildBackwardOutputs(forward, {"x"}, std::string("__grad_output"), {{{"x", {3, 5}}}});
    bool reversed = false;
    for (const ExprNode& n : backward.expr->nodes) reversed = reversed || (n.op == ExprOp::SCAN && n.scan_reverse && n.scan_mode == ScanMode::Exclusive);
    CHECK(reversed);
    // min / max scans route every position's gradient to the running winner: an FP32 SCAN_MAX_BACKWARD node over the operand and
    // the FP32 gradient (AutoDiff.cpp:5743-5760 there); product scans have no rule
    const PhysicalOutputs maxBackward =
        buildBackwardOutputs(Expression::outputs({{"y", x.scan(ScanOp::Max, -1, false)}}).physicalOutputs(), {"x"}, std::nullopt, {{{"x", {3, 5}}}});
    int routed = 0;
    for (const ExprNode& n : maxBackward.expr->nodes) {
        if (n.op != ExprOp::SCAN_MAX_BACKWARD) continue;
        ++routed;
        CHECK(n.scan_mode == ScanMode::Exclusive && !n.scan_reverse && n.aux == UINT32_MAX && n.output_dtype == DataType::FP32);
        CHECK(maxBackward.expr->nodes.at(n.lhs).op == ExprOp::INPUT && maxBackward.expr->nodes.at(n.rhs).output_dtype == DataType::FP32);
    }
    CHECK(routed == 1);
    const PhysicalOutputs raggedMin = buildBackwardOutputs(Expression::outputs({{"y", x.segmentedScan(offsets, ScanOp::Min)}}).physicalOutputs(), {"x"},
                                                           std::string("__grad_output"), {{{"x", {9}}, {"offsets", {4}}}});
    bool segmentedRouting = false;
    for (const ExprNode& n : raggedMin.expr->nodes) segmentedRouting = segmentedRouting || (n.op == ExprOp::SEGMENTED_SCAN_MIN_BACKWARD && n.aux != UINT32_MAX);
    CHECK(segmentedRouting);
    CHECK(throwsAs<std::runtime_error>([&] {
        (void)buildBackwardOutputs(Expression::outputs({{"y", x.scan(ScanOp::Product)}}).physicalOutputs(), {"x"}, std::nullopt, {{{"x", {3, 5}}}});
    }));
}

static void ropeExpressionStructure() {
    // ROPE nodes carry every option; explicit positions and the effective length ride as operands that precede the rotation and
    // are cast to fp32 (Expression.cpp:4334-4507, ExpressionConvenienceOpsTest.cpp:3670-3700 there)
    RotaryPositionEmbeddingOptions options;
    options.sequence_axis = 1;
    options.head_dim_axis = 2;
    options.rotary_dim = 4;
    options.scaling_kind = RotaryScalingKind::Yarn;
    options.scaling_factor = 4.0;
    options.original_max_position_embeddings = 16;
    const Expression x = Expression::input("x");
    PhysicalOutputs outputs =
        Expression::outputs({{"y", x.rotaryPositionEmbeddingWithPositionIds(Expression::input("positions"), options)}}).physicalOutputs();
    const ExprNode& node = outputs.expr->nodes.at(outputs.outputs[0].node_idx);
    CHECK(node.op == ExprOp::ROPE && node.rhs != UINT32_MAX && node.aux == UINT32_MAX && node.rhs < outputs.outputs[0].node_idx);
    CHECK(outputs.expr->nodes.at(node.rhs).op == ExprOp::CAST && outputs.expr->nodes.at(node.rhs).output_dtype == DataType::FP32);
    CHECK(node.rope_sequence_axis == 1 && node.rope_head_dim_axis == 2 && node.rope_rotary_dim == 4 && node.rope_scaling_kind == RotaryScalingKind::Yarn);
    CHECK(std::fabs(node.rope_attention_factor - (0.1 * std::log(4.0) + 1.0)) < 1e-15);  // YaRN's own magnitude correction
    resolveOutputsDTypesInPlace(outputs, {DataType::UINT32, DataType::BF16});  // slots in order of appearance: positions come first
    CHECK(outputs.expr->nodes.at(outputs.outputs[0].node_idx).output_dtype == DataType::BF16);
    options.position_offset = 1;
    CHECK(throwsAs<std::runtime_error>([&] { (void)x.rotaryPositionEmbeddingWithPositionIds(Expression::input("positions"), options); }));
    options.position_offset = 0;
    options.rotary_dim = 3;
    CHECK(throwsAs<std::runtime_error>([&] { (void)x.rope(options); }));
    options.rotary_dim = 4;
    options.scaling_kind = RotaryScalingKind::LongRope;
    CHECK(throwsAs<std::runtime_error>([&] { (void)x.rope(options); }));  // factor lists missing
    options.long_rope_short_factors = {1.0, 1.0};
    options.long_rope_long_factors = {2.0, 2.0};
    const PhysicalExpression both =
        x.rotaryPositionEmbeddingWithPositionIdsAndEffectiveSequenceLength(Expression::input("positions"), Expression::input("lengths"), options).expression();
    CHECK(both.nodes.back().op == ExprOp::ROPE && both.nodes.back().rhs != UINT32_MAX && both.nodes.back().aux != UINT32_MAX);
    CHECK(std::fabs(both.nodes.back().rope_attention_factor - std::sqrt(1.0 + std::log(4.0) / std::log(16.0))) < 1e-15);
    // equal parameters, equal text; any parameter tells two rotations apart
    RotaryPositionEmbeddingOptions a, b;
    b.base = 500000.0;
    CHECK(canonicalize(x.rope(a).expression()) == canonicalize(x.rope(a).expression()));
    CHECK(canonicalize(x.rope(a).expression()) != canonicalize(x.rope(b).expression()));
    // the gradient is the same rotation turned the other way, positions and all (AutoDiff.cpp:4672-4693 there)
    options.inverse = false;
    const PhysicalOutputs forward = Expression::outputs({{"y", x.rotaryPositionEmbeddingWithPositionIds(Expression::input("positions"), options)}}).physicalOutputs();
    const PhysicalOutputs backward = buildBackwardOutputs(forward, {"x"}, std::string("__grad_output"), {{{"x", {2, 5, 8}}, {"positions", {5}}}});
    int turnedBack = 0;
    for (const ExprNode& n : backward.expr->nodes) turnedBack += n.op == ExprOp::ROPE && n.rope_inverse && n.rhs != UINT32_MAX && n.rope_rotary_dim == 4;
    CHECK(turnedBack == 1);
}

static void raggedExpressionStructure() {
    // RaggedExpressionTest.cpp:739-795,907-957,2037-2055 there: names, descriptors and markers, no device work
    const RaggedTensorDescriptor descriptor(DataType::FP32, {4}, 3, 9);
    CHECK(descriptor.getValuesDimensions() == (std::vector<uint64_t>{9, 4}) && descriptor.getOffsetsDescriptor().getDimensions() == (std::vector<uint64_t>{4}));
    CHECK(descriptor.getOffsetsDataType() == DataType::UINT32);
    CHECK(throwsAs<std::invalid_argument>([] { RaggedTensorDescriptor(DataType::FP32, {4}, 3, 0); }));
    CHECK(throwsAs<std::invalid_argument>([] { RowPartitionDescriptor(3, 9, DataType::INT32); }));
    CHECK(throwsAs<std::invalid_argument>([] { RowPartitionDescriptor(3, 1ull << 33, DataType::UINT32); }));

    const RaggedExpression x = RaggedExpression::input("x", descriptor);
    CHECK((x.getInputNames() == std::set<std::string>{"x.values", "x.offsets"}));
    CHECK((x.getMetadataInputNames() == std::set<std::string>{"x.offsets"}));
    CHECK((x.getDifferentiableInputNames() == std::set<std::string>{"x.values"}));
    CHECK(x.getRuntimeExtent().maxLaunchElements() == 36);
    const PhysicalExpression marked = x.mapValues([](const Expression& v) { return (v.swish() + Expression(0.25)).tanh(); }).getValues().expression();
    const ExprNode& marker = marked.nodes.at(marked.output_node);
    CHECK(marker.op == ExprOp::RAGGED_VALUEWISE_EXTENT && marker.ragged_runtime_batch_size == 3 && marker.ragged_runtime_max_active_values == 9 &&
          marker.ragged_runtime_elements_per_value == 4);
    CHECK(marked.nodes.at(marker.lhs).op == ExprOp::TANH && marked.nodes.at(marker.rhs).op == ExprOp::INPUT);

    const Expression shared = Expression::input("shared.offsets");
    const RaggedExpression a(Expression::input("a.values"), shared, descriptor), b(Expression::input("b.values"), shared, descriptor);
    const RaggedExpression sum = a + b;
    CHECK(sum.getOffsets().isSameLogicalNode(shared) && sum.getDescriptor() == descriptor);
    const RaggedExpression less = a.lessThan(b);
    CHECK(less.getValuesDataType() == DataType::BOOLEAN && less.getOffsets().isSameLogicalNode(shared));
    CHECK(a.cast(DataType::FP16).getValuesDataType() == DataType::FP16 && a.cast(DataType::FP16).getRuntimeExtent().elementsPerValue == 4);
    const RaggedExpression other(Expression::input("c.values"), Expression::input("c.offsets"), descriptor);
    CHECK(throwsAs<std::invalid_argument>([&] { (void)(a + other); }));
    const RaggedExpression wider(Expression::input("d.values"), shared, RaggedTensorDescriptor(DataType::FP32, {5}, 3, 9));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)(a + wider); }));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)a.withValues(Expression::input("e"), RaggedTensorDescriptor(DataType::FP32, {4}, 2, 9)); }));
    CHECK(throwsAs<std::runtime_error>([] { (void)RaggedExpression().getValues(); }));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)RaggedExpression::input("i", RaggedTensorDescriptor(DataType::INT32, {}, 3, 9)).segment_mean(); }));

    const PhysicalExpression reduced = x.reduce_sum().expression();
    const ExprNode& reduction = reduced.nodes.at(reduced.output_node);
    CHECK(reduction.op == ExprOp::SEGMENTED_REDUCE_SUM && reduction.ragged_runtime_elements_per_value == 4 && reduction.ragged_runtime_batch_size == 3);
    CHECK(canonicalize(reduced).find("segmented_reduce_sum:ragged=[3,9,4]") != std::string::npos);
    CHECK(throwsAs<std::invalid_argument>([&] { (void)(Expression::input("v") + 1.0).withRaggedRuntimeExtent(Expression::input("o") + 1.0, 3, 9, 4); }));

    // RaggedExpressionTest.cpp:800-871 there: trailing slices keep the partition and use storage strides; nested slices compose
    const RaggedExpression wide = RaggedExpression::input("w", RaggedTensorDescriptor(DataType::FP32, {2, 6}, 3, 9));
    const RaggedExpression inner = wide.sliceLastDimension(2, 4).sliceLastDimension(1, 2);
    CHECK((inner.getValuesDimensions() == std::vector<uint64_t>{9, 2, 2}) && inner.getRuntimeExtent().elementsPerValue == 4);
    const PhysicalExpression sliced = inner.getValues().expression();
    const ExprNode& view = sliced.nodes.at(sliced.nodes.at(sliced.output_node).lhs);
    CHECK(view.op == ExprOp::STRIDED_VIEW && (view.view_strides == std::vector<uint64_t>{12, 6, 1}) && view.view_element_offset == 3);
    CHECK(sliced.nodes.at(view.lhs).op == ExprOp::INPUT);  // one view of the original storage, not a view of a view
    const RaggedExpression outer = wide.sliceTrailingDimension(0, 1, 1);
    CHECK((outer.getValuesDimensions() == std::vector<uint64_t>{9, 1, 6}));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)wide.sliceLastDimension(4, 3); }));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)wide.sliceTrailingDimension(2, 0, 1); }));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)wide.sliceLastDimension(0, 0); }));
}

static void raggedExpressionExecution(Stream& stream) {
    // RaggedExpressionTest.cpp:1795-1824 there: empty and skewed rows
    auto runOne = [&](const Expression& e, const std::unordered_map<std::string, Tensor>& inputs, const std::optional<Tensor>& into = std::nullopt) {
        FusedEquation eq = FusedEquation::compile(Expression::outputs({{"out", e}}).physicalOutputs(), 0);
        std::unordered_map<std::string, Tensor> pre;
        if (into.has_value()) pre.emplace("out", into.value());
        StampedExecutionPlan plan = eq.stamp(inputs, stream, {}, pre);
        plan.run();
        return plan.output("out");
    };
    const float inf = std::numeric_limits<float>::infinity();
    {
        const RaggedExpression x = RaggedExpression::input("x", RaggedTensorDescriptor(DataType::FP32, {}, 4, 9));
        const std::unordered_map<std::string, Tensor> inputs{{"x.values", gpuFrom({1, -2, 4, 5, 7, -1, 8, 99, 100}, {9}, stream)},
                                                            {"x.offsets", gpuOffsets({0, 3, 3, 5, 7}, stream)}};
        CHECK((toHostF32(runOne(x.segment_sum(), inputs), stream) == std::vector<float>{3, 0, 12, 7}));
        CHECK((toHostF32(runOne(x.segment_mean(), inputs), stream) == std::vector<float>{1, 0, 6, 3.5f}));
        CHECK((toHostF32(runOne(x.segment_min(), inputs), stream) == std::vector<float>{-2, inf, 5, -1}));
        CHECK((toHostF32(runOne(x.segment_max(), inputs), stream) == std::vector<float>{4, -inf, 7, 8}));
    }
    {
        // :1983-2035 there: [6, 2, 2] values, UINT64 offsets, one empty row, one row of capacity nobody owns
        const RaggedExpression x = RaggedExpression::input("x", RaggedTensorDescriptor(DataType::FP32, {2, 2}, 3, 6, DataType::UINT64));
        const std::unordered_map<std::string, Tensor> inputs{
            {"x.values", gpuFrom({1, 2, 3, 4, 5, 6, 7, 8, -1, -2, -3, -4, 9, 10, 11, 12, 13, 14, 15, 16, 101, 102, 103, 104}, {6, 2, 2}, stream)},
            {"x.offsets", gpuOffsets({0, 2, 2, 5}, stream, DataType::UINT64)}};
        const Tensor sum = runOne(x.segment_sum(), inputs);
        CHECK((sum.getDimensions() == std::vector<uint64_t>{3, 2, 2}));
        CHECK((toHostF32(sum, stream) == std::vector<float>{6, 8, 10, 12, 0, 0, 0, 0, 21, 22, 23, 24}));
        const float small = 1.0f / (1.0f + std::exp(4.0f)), large = 1.0f - small;
        const Tensor softmax = runOne(x.segment_softmax().getValues(), inputs, gpuFrom(std::vector<float>(24, 555.0f), {6, 2, 2}, stream));
        const std::vector<float> p = toHostF32(softmax, stream);
        for (int c = 0; c < 4; ++c) {
            CHECK_NEAR(p[c], small, 3e-5);
            CHECK_NEAR(p[4 + c], large, 3e-5);
        }
        for (int i = 20; i < 24; ++i) CHECK(p[i] == 555.0f);
        const Tensor logSoftmax = runOne(x.segment_log_softmax().getValues(), inputs, gpuFrom(std::vector<float>(24, -555.0f), {6, 2, 2}, stream));
        const std::vector<float> lp = toHostF32(logSoftmax, stream);
        for (int c = 0; c < 4; ++c) {
            CHECK_NEAR(lp[c], std::log(small), 3e-5);
            CHECK_NEAR(lp[4 + c], std::log(large), 3e-5);
        }
        for (int i = 20; i < 24; ++i) CHECK(lp[i] == -555.0f);
    }
    {
        // :1826-1854 there: scalar values
        const RaggedExpression x = RaggedExpression::input("x", RaggedTensorDescriptor(DataType::FP32, {}, 3, 8));
        const std::unordered_map<std::string, Tensor> inputs{{"x.values", gpuFrom({1, 2, 0, -1, 1, 50, 60, 70}, {8}, stream)},
                                                            {"x.offsets", gpuOffsets({0, 2, 2, 5}, stream)}};
        const std::vector<float> p = toHostF32(runOne(x.softmax().getValues(), inputs, gpuFrom(std::vector<float>(8, 321.0f), {8}, stream)), stream);
        const float d0 = std::exp(1.0f) + std::exp(2.0f), d2 = std::exp(0.0f) + std::exp(-1.0f) + std::exp(1.0f);
        const std::vector<float> want{std::exp(1.0f) / d0, std::exp(2.0f) / d0, std::exp(0.0f) / d2, std::exp(-1.0f) / d2, std::exp(1.0f) / d2, 321, 321, 321};
        for (size_t i = 0; i < want.size(); ++i) CHECK_NEAR(p[i], want[i], 2e-5);
        // relu and a comparison, valuewise, over the active rows only
        const RaggedExpression y = x.relu() * x.relu();
        const std::vector<float> q = toHostF32(runOne(y.getValues(), inputs, gpuFrom(std::vector<float>(8, -7.0f), {8}, stream)), stream);
        CHECK((q == std::vector<float>{1, 4, 0, 0, 1, -7, -7, -7}));
    }
    {
        // trailing slices of [6, 4] values compose and only the active rows are computed (:1348-1404 there)
        const RaggedExpression x = RaggedExpression::input("x", RaggedTensorDescriptor(DataType::FP32, {4}, 2, 6));
        std::vector<float> host(24);
        for (size_t i = 0; i < host.size(); ++i) host[i] = static_cast<float>(i);
        const std::unordered_map<std::string, Tensor> inputs{{"x.values", gpuFrom(host, {6, 4}, stream)}, {"x.offsets", gpuOffsets({0, 1, 4}, stream)}};
        const RaggedExpression product = x.sliceLastDimension(0, 2) * x.sliceLastDimension(2, 2);
        const std::vector<float> p = toHostF32(runOne(product.getValues(), inputs, gpuFrom(std::vector<float>(12, -1.0f), {6, 2}, stream)), stream);
        CHECK((p == std::vector<float>{0 * 2, 1 * 3, 4 * 6, 5 * 7, 8 * 10, 9 * 11, 12 * 14, 13 * 15, -1, -1, -1, -1}));
        const std::vector<float> sums = toHostF32(runOne(x.sliceLastDimension(1, 2).sliceLastDimension(1, 1).segment_sum(), inputs), stream);
        CHECK((sums == std::vector<float>{2, 6 + 10 + 14}));
    }
}

static void argReductionsTiesAndNaN(Stream& stream) {
    // CubArgReductionTest.cpp: lowest index wins ties, NaN wins, index is the position inside the reduction domain
    Tensor t = gpuFrom({1, 1, 3, 1, std::nanf(""), 0, std::nanf(""), -4}, {2, 4}, stream);
    CubArgReductionOutputOptions options;
    options.produce_value = true;
    auto amin = CubArgReduction(CubArgReductionOp::ArgMin, 1u, options).stamp(t, stream);
    amin->run();
    CHECK((toHostRaw<uint32_t>(amin->getIndexOutputTensor().value(), stream) == std::vector<uint32_t>{0, 0}));
    const std::vector<float> values = toHostF32(amin->getValueOutputTensor().value(), stream);
    CHECK(values[0] == 1.0f && std::isnan(values[1]));
    Tensor u = gpuFrom({5, 5, 3, 5, -1, std::nanf(""), std::nanf(""), 8}, {2, 4}, stream);
    options.produce_value = false;
    options.index_output_dtype = DataType::UINT64;
    auto amax = CubArgReduction(CubArgReductionOp::ArgMax, 1u, options).stamp(u, stream);
    amax->run();
    CHECK((toHostRaw<uint64_t>(amax->getIndexOutputTensor().value(), stream) == std::vector<uint64_t>{0, 1}));
    CHECK(!amax->getValueOutputTensor().has_value());
}

static void expressionConfig1AndRuntimeScalars(Stream& stream) {
    const size_t n = 1000;
    std::vector<float> a(n), b(n), c(n), d(n);
    for (size_t i = 0; i < n; ++i) {
        a[i] = std::sin(0.1f * i);
        b[i] = std::cos(0.3f * i);
        c[i] = 0.001f * i - 0.5f;
        d[i] = 0.02f * i - 10.0f;
    }
    Expression ea = Expression::input("a"), eb = Expression::input("b"), ec = Expression::input("c"), ed = Expression::input("d");
    FusedEquation eq = FusedEquation::compile(((ea * eb + ec) * ed.sigmoid()).expression(), 0);
    std::unordered_map<std::string, Tensor> inputs = {{"a", gpuFrom(a, {n}, stream)}, {"b", gpuFrom(b, {n}, stream)}, {"c", gpuFrom(c, {n}, stream)},
                                                      {"d", gpuFrom(d, {n}, stream)}};
    StampedExecutionPlan plan = eq.stamp(inputs, stream);
    CHECK((plan.stageKindNames() == std::vector<std::string>{"FusedKernel"}));
    plan.run();
    const std::vector<float> got = toHostF32(plan.output(), stream);
    for (size_t i = 0; i < n; i += 37) {
        const double want = (double(a[i]) * b[i] + c[i]) / (1.0 + std::exp(-double(d[i])));
        CHECK_NEAR(got[i], want, 4e-7 * std::max(1.0, std::fabs(want)) + 2e-7);
    }
    // a scalar kept in device memory: read at every run through a TensorScalarBinding (CompiledEquation.h:15-19 there), bound as
    // the third argument of stamp like in the reference
    {
        const Expression stepped = Expression::input("x") * Expression::tensorRuntimeScalar("step") + 1.0;
        const FusedEquation eq3 = FusedEquation::compile(stepped.expression(), 0);
        Tensor xs = gpuFrom({1, 2, 3, 4}, {4}, stream), buffer = gpuFrom({123.0f, 0.25f}, {2}, stream);
        StampedExecutionPlan byOffset = eq3.stamp({{"x", xs}}, stream, {{"step", TensorScalarBinding{buffer, 4, DataType::FP32}}});
        CHECK((byOffset.stageKindNames() == std::vector<std::string>{"FusedKernel"}));
        byOffset.run();
        CHECK((toHostF32(byOffset.output(), stream) == std::vector<float>{1.25f, 1.5f, 1.75f, 2.0f}));
        buffer.copyFromAsync(gpuFrom({123.0f, -1.5f}, {2}, stream), stream);
        byOffset.run();
        CHECK((toHostF32(byOffset.output(), stream) == std::vector<float>{-0.5f, -2.0f, -3.5f, -5.0f}));
        CHECK(throwsAs<std::runtime_error>([&] { (void)eq3.stamp({{"x", xs}}, stream); }));                                                          // unbound
        CHECK(throwsAs<std::runtime_error>([&] { (void)eq3.stamp({{"x", xs}}, stream, {{"step", TensorScalarBinding{buffer, 2, DataType::FP32}}}); }));  // misaligned
        CHECK(throwsAs<std::runtime_error>([&] { (void)eq3.stamp({{"x", xs}}, stream, {{"step", TensorScalarBinding{buffer, 8, DataType::FP32}}}); }));  // past the end
        CHECK(throwsAs<std::runtime_error>([&] { (void)eq3.stamp({{"x", xs}}, stream, {{"step", TensorScalarBinding{buffer, 0, DataType::FP16}}}); }));  // dtype
    }
    // convenience run into a caller-provided tensor, with a runtime scalar
    Expression scaled = Expression::input("x") * Expression::runtimeScalar("alpha") + 1.0;
    FusedEquation eq2 = FusedEquation::compile(scaled.expression(), 0);
    Tensor x = gpuFrom({1, 2, 3, 4}, {4}, stream);
    Tensor out(gpuPlacement, TensorDescriptor(DataType::FP32, {4}));
    eq2.run({{"x", x}}, {{"alpha", 2.5f}}, out, stream);
    CHECK((toHostF32(out, stream) == std::vector<float>{3.5f, 6.0f, 8.5f, 11.0f}));
    CHECK(throwsAs<std::runtime_error>([&] { eq2.run({{"x", x}}, out, stream); }));  // missing runtime scalar
}

static void autodiffExecution(Stream& stream) {
    // d/dx, d/dw of sum(tanh(x * w)) with w broadcast over rows; then the same with an explicit upstream gradient
    const std::vector<float> xv{0.5f, -1.0f, 2.0f, 1.5f, 0.25f, -0.75f}, wv{2.0f, -0.5f, 1.0f}, gv{1.0f, 2.0f, -1.0f, 0.5f, 0.0f, 3.0f};
    const Expression x = Expression::input("x"), w = Expression::input("w");
    const FusedEquation forward = FusedEquation::compile(Expression::outputs({{"y", (x * w).tanh()}}).physicalOutputs(), 0);
    const std::unordered_map<std::string, Tensor> inputs{{"x", gpuFrom(xv, {2, 3}, stream)}, {"w", gpuFrom(wv, {3}, stream)}};
    const FusedEquation implicit = forward.compileBackward({"x", "w"});
    CHECK((implicit.getOutputNames() == std::vector<std::string>{"x_grad", "w_grad"}));
    CHECK((implicit.getOutputShapes(inputs).at("w_grad") == std::vector<uint64_t>{3}));
    StampedExecutionPlan plan = implicit.stamp(inputs, stream);
    plan.run();
    std::vector<float> gx = toHostF32(plan.output("x_grad"), stream), gw = toHostF32(plan.output("w_grad"), stream);
    for (int r = 0; r < 2; ++r) {
        for (int c = 0; c < 3; ++c) {
            const double t = std::tanh(double(xv[r * 3 + c]) * wv[c]);
            CHECK_NEAR(gx[r * 3 + c], (1 - t * t) * wv[c], 1e-6);
        }
    }
    for (int c = 0; c < 3; ++c) {
        double want = 0;
        for (int r = 0; r < 2; ++r) {
            const double t = std::tanh(double(xv[r * 3 + c]) * wv[c]);
            want += (1 - t * t) * xv[r * 3 + c];
        }
        CHECK_NEAR(gw[c], want, 1e-6);
    }
    std::unordered_map<std::string, Tensor> withUpstream = inputs;
    withUpstream.emplace("__grad_output", gpuFrom(gv, {2, 3}, stream));
    StampedExecutionPlan seeded = forward.compileBackward({"x"}, std::string(DEFAULT_BACKWARD_UPSTREAM_INPUT_NAME)).stamp(withUpstream, stream);
    seeded.run();
    gx = toHostF32(seeded.output("x_grad"), stream);
    for (int i = 0; i < 6; ++i) {
        const double t = std::tanh(double(xv[i]) * wv[i % 3]);
        CHECK_NEAR(gx[i], gv[i] * (1 - t * t) * wv[i % 3], 1e-6);
    }
    // min/max reductions hand the gradient to the first winner
    const FusedEquation rowMax = FusedEquation::compile(Expression::outputs({{"m", x.reduce_max({1}, {1})}}).physicalOutputs(), 0);
    StampedExecutionPlan routed = rowMax.compileBackward({"x"}).stamp({{"x", gpuFrom({1, 3, 3, 2, 2, 0}, {2, 3}, stream)}}, stream);
    CHECK((routed.stageKindNames() == std::vector<std::string>{"FusedKernel", "ArgMinMax", "ReduceMinMaxBackward"}));
    routed.run();
    CHECK((toHostF32(routed.output("x_grad"), stream) == std::vector<float>{0, 1, 0, 1, 0, 0}));
    CHECK(throwsAs<std::runtime_error>([&] { (void)forward.compileBackward({"x"}, std::string("w")); }));
    CHECK(throwsAs<std::runtime_error>([&] { (void)implicit.compileBackward({"x"}); }));  // no second derivative of a backward equation
}

static void ropeExecution(Stream& stream) {
    // the equivalences ExpressionConvenienceOpsTest.cpp:3503-3668 there asserts, and the closed form of the first pair
    std::vector<float> values(1 * 2 * 8 * 8);
    for (size_t i = 0; i < values.size(); ++i) values[i] = 0.25f * static_cast<float>(static_cast<int>(i % 17) - 8);
    const Tensor x = gpuFrom(values, {1, 2, 8, 8}, stream);
    auto run = [&](const Expression& e, std::unordered_map<std::string, Tensor> inputs) {
        FusedEquation eq = FusedEquation::compile(Expression::outputs({{"y", e}}).physicalOutputs(), 0);
        StampedExecutionPlan plan = eq.stamp(inputs, stream);
        plan.run();
        return toHostF32(plan.output("y"), stream);
    };
    const Expression ix = Expression::input("x");
    RotaryPositionEmbeddingOptions plainOptions;
    plainOptions.rotary_dim = 4;
    const std::vector<float> plain = run(ix.rope(plainOptions), {{"x", x}});
    // pair 0 turns by the position itself: (a, b) -> (a cos p - b sin p, a sin p + b cos p); the tail is untouched
    for (int p = 0; p < 8; ++p) {
        const float a = values[p * 8 + 0], b = values[p * 8 + 2];
        CHECK(std::fabs(plain[p * 8 + 0] - (a * std::cos((float)p) - b * std::sin((float)p))) < 1e-5f);
        CHECK(std::fabs(plain[p * 8 + 2] - (a * std::sin((float)p) + b * std::cos((float)p))) < 1e-5f);
        for (int d = 4; d < 8; ++d) CHECK(plain[p * 8 + d] == values[p * 8 + d]);
    }
    Tensor lengthHost(cpuPlacement, TensorDescriptor(DataType::UINT32, {1}));
    lengthHost.getMemPtr<uint32_t>()[0] = 3;
    Tensor length(gpuPlacement, TensorDescriptor(DataType::UINT32, {1}));
    length.copyFromAsync(lengthHost, stream);
    stream.synchronize();
    RotaryPositionEmbeddingOptions ntk = plainOptions;
    ntk.scaling_kind = RotaryScalingKind::DynamicNTK;
    ntk.scaling_factor = 2.0;
    ntk.original_max_position_embeddings = 4;
    // a short effective length leaves Dynamic NTK unscaled; the physical extent (8 > 4) does not
    CHECK(run(ix.rotaryPositionEmbeddingWithEffectiveSequenceLength(Expression::input("length"), ntk), {{"x", x}, {"length", length}}) == plain);
    CHECK(run(ix.rope(ntk), {{"x", x}}) != plain);
    RotaryPositionEmbeddingOptions longRope = plainOptions;
    longRope.scaling_kind = RotaryScalingKind::LongRope;
    longRope.original_max_position_embeddings = 4;
    longRope.long_rope_short_factors = {1.0, 1.0};
    longRope.long_rope_long_factors = {2.0, 2.0};
    // (1 / (1 * base^(2j/d)) against base^(-2j/d): the same frequency up to the rounding of the two power evaluations)
    const std::vector<float> shortLength = run(ix.rotaryPositionEmbeddingWithEffectiveSequenceLength(Expression::input("length"), longRope), {{"x", x}, {"length", length}});
    const std::vector<float> physicalLength = run(ix.rope(longRope), {{"x", x}});
    float shortGap = 0.0f, physicalGap = 0.0f;
    for (size_t i = 0; i < plain.size(); ++i) {
        shortGap = std::max(shortGap, std::fabs(shortLength[i] - plain[i]));
        physicalGap = std::max(physicalGap, std::fabs(physicalLength[i] - plain[i]));
    }
    CHECK(shortGap < 1e-5f);
    CHECK(physicalGap > 1e-2f);
    // explicit absolute positions equal the offset they spell out; turning back returns the input
    Tensor idsHost(cpuPlacement, TensorDescriptor(DataType::UINT32, {8}));
    for (uint32_t p = 0; p < 8; ++p) idsHost.getMemPtr<uint32_t>()[p] = p + 5;
    Tensor ids(gpuPlacement, TensorDescriptor(DataType::UINT32, {8}));
    ids.copyFromAsync(idsHost, stream);
    stream.synchronize();
    RotaryPositionEmbeddingOptions shifted = plainOptions;
    shifted.position_offset = 5;
    CHECK(run(ix.rotaryPositionEmbeddingWithPositionIds(Expression::input("positions"), plainOptions), {{"x", x}, {"positions", ids}}) == run(ix.rope(shifted), {{"x", x}}));
    RotaryPositionEmbeddingOptions back = shifted;
    back.inverse = true;
    const std::vector<float> round = run(ix.rope(shifted).rope(back), {{"x", x}});
    for (size_t i = 0; i < values.size(); ++i) CHECK(std::fabs(round[i] - values[i]) < 2e-6f);
}

static void devicePrefixScans(Stream& stream) {
    // cubDeviceScan / cubDeviceSegmentedUniformScan / cubDeviceSegmentedScan and arg forms: plan, temporary storage, run
    // (CubDevicePrimitivesTest.cpp there; literal vectors of test_expression_scan.py / test_expression_segmented_scan.py)
    auto upload = [&](const std::vector<uint32_t>& v, const std::vector<uint64_t>& dims) {
        Tensor host(cpuPlacement, TensorDescriptor(DataType::UINT32, dims));
        std::memcpy(host.getMemPtr<uint32_t>(), v.data(), v.size() * 4);
        Tensor device(gpuPlacement, TensorDescriptor(DataType::UINT32, dims));
        device.copyFromAsync(host, stream);
        stream.synchronize();
        return device;
    };
    const Tensor rows = upload({2, 3, 1, 4, 5, 1, 2, 3}, {2, 4});
    Tensor out(gpuPlacement, TensorDescriptor(DataType::UINT32, {2, 4}));
    auto uniform = [&](CubScanOp op, CubScanMode mode, CubScanDirection direction = CubScanDirection::Forward) {
        const CubDeviceSegmentedUniformScanPlan plan = prepareCubDeviceSegmentedUniformScan(rows, out, 8, 2, 4, op, mode, direction);
        CHECK(plan.temp_storage_bytes >= 1 && plan.num_segments == 2 && plan.segment_size == 4 && plan.dtype == DataType::UINT32);
        CHECK(cubDeviceSegmentedUniformScanTempBytes(rows, out, 8, 2, 4, op, mode, direction) == plan.temp_storage_bytes);
        const Tensor temp = allocateCubTemporaryStorage(gpuPlacement, plan.temp_storage_bytes);
        cubDeviceSegmentedUniformScan(plan, temp, rows, out, stream);
        return toHostRaw<uint32_t>(out, stream);
    };
    CHECK((uniform(CubScanOp::Sum, CubScanMode::Inclusive) == std::vector<uint32_t>{2, 5, 6, 10, 5, 6, 8, 11}));
    CHECK((uniform(CubScanOp::Sum, CubScanMode::Exclusive) == std::vector<uint32_t>{0, 2, 5, 6, 0, 5, 6, 8}));
    CHECK((uniform(CubScanOp::Min, CubScanMode::Exclusive) == std::vector<uint32_t>{0xffffffffu, 2, 2, 1, 0xffffffffu, 5, 1, 1}));
    CHECK((uniform(CubScanOp::Max, CubScanMode::Inclusive) == std::vector<uint32_t>{2, 3, 3, 4, 5, 5, 5, 5}));
    CHECK((uniform(CubScanOp::Product, CubScanMode::Inclusive) == std::vector<uint32_t>{2, 6, 6, 24, 5, 5, 10, 30}));
    CHECK((uniform(CubScanOp::Sum, CubScanMode::Inclusive, CubScanDirection::Reverse) == std::vector<uint32_t>{10, 8, 5, 4, 11, 6, 5, 3}));
    // one flat scan over the same eight elements
    const CubDeviceScanPlan flat = prepareCubDeviceScan(rows, out, 8, CubScanOp::Sum, CubScanMode::Inclusive);
    cubDeviceScan(flat, allocateCubTemporaryStorage(gpuPlacement, flat.temp_storage_bytes), rows, out, stream);
    CHECK((toHostRaw<uint32_t>(out, stream) == std::vector<uint32_t>{2, 5, 6, 10, 15, 16, 18, 21}));
    // segments of an offsets tensor, and the flattened index of the running maximum
    const Tensor values = upload({8, 6, 7, 5, 3, 2, 9}, {7}), offsets = upload({0, 2, 5, 7}, {4});
    Tensor ragged(gpuPlacement, TensorDescriptor(DataType::UINT32, {7}));
    const CubDeviceSegmentedScanPlan segmented = prepareCubDeviceSegmentedScan(values, ragged, offsets, 7, 3, CubScanOp::Max, CubScanMode::Exclusive);
    CHECK(segmented.offset_dtype == DataType::UINT32 && segmented.num_segments == 3);
    cubDeviceSegmentedScan(segmented, allocateCubTemporaryStorage(gpuPlacement, segmented.temp_storage_bytes), values, ragged, offsets, stream);
    CHECK((toHostRaw<uint32_t>(ragged, stream) == std::vector<uint32_t>{0, 8, 0, 7, 7, 0, 2}));
    const CubDeviceSegmentedArgScanPlan winners = prepareCubDeviceSegmentedArgScan(values, ragged, offsets, 7, 3, CubArgScanOp::ArgMin, CubScanMode::Inclusive);
    cubDeviceSegmentedArgScan(winners, allocateCubTemporaryStorage(gpuPlacement, winners.temp_storage_bytes), values, ragged, offsets, stream);
    CHECK((toHostRaw<uint32_t>(ragged, stream) == std::vector<uint32_t>{0, 1, 2, 3, 4, 5, 5}));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceSegmentedUniformScan(rows, out, 8, 3, 3, CubScanOp::Sum, CubScanMode::Inclusive); }));
    CHECK(throwsAs<std::invalid_argument>([&] {
        cubDeviceScan(flat, allocateCubTemporaryStorage(gpuPlacement, 1), rows, out, stream);  // flat over 8 elements needs no storage: one chunk
        const Tensor big(gpuPlacement, TensorDescriptor(DataType::UINT32, {1 << 20}));
        Tensor bigOut(gpuPlacement, TensorDescriptor(DataType::UINT32, {1 << 20}));
        const CubDeviceScanPlan carried = prepareCubDeviceScan(big, bigOut, 1 << 20, CubScanOp::Sum, CubScanMode::Inclusive);
        cubDeviceScan(carried, allocateCubTemporaryStorage(gpuPlacement, 1), big, bigOut, stream);  // too little temporary storage
    }));
    CHECK(isCubScanDTypeSupported(DataType::BF16) && !isCubScanDTypeSupported(DataType::INT32) && isCubSegmentOffsetDTypeSupported(DataType::UINT64));
    {
        // A bounded wait between blocks that gives up (forced: a bound of zero polls) works the totals it lacks out of the input:
        // the plan / run entry point hands back complete results (CubScan.cu there never returns a partial result either), and
        // the diagnostic says that waits took the way out.
        setenv("THOR_SCAN_WAIT_LIMIT", "0", 1);
        const uint64_t n = 1 << 20;
        const Tensor ones = upload(std::vector<uint32_t>(n, 1u), {n});
        Tensor counted(gpuPlacement, TensorDescriptor(DataType::UINT32, {n}));
        const CubDeviceScanPlan impatient = prepareCubDeviceScan(ones, counted, n, CubScanOp::Sum, CubScanMode::Inclusive);
        unsetenv("THOR_SCAN_WAIT_LIMIT");
        CHECK(cubScanKernelVariant(impatient.kernels).find("published_totals") != std::string::npos);
        const Tensor temp = allocateCubTemporaryStorage(gpuPlacement, impatient.temp_storage_bytes);
        cubDeviceScan(impatient, temp, ones, counted, stream);
        const std::vector<uint32_t> got = toHostRaw<uint32_t>(counted, stream);
        bool counts = got.size() == n;
        for (uint64_t i = 0; counts && i < n; ++i) counts = got[i] == i + 1;
        CHECK(counts);
        CHECK(cubScanWaitsRecovered(impatient.kernels, temp, stream) > 0);
        const CubDeviceScanPlan patient = prepareCubDeviceScan(ones, counted, n, CubScanOp::Sum, CubScanMode::Inclusive);
        cubDeviceScan(patient, temp, ones, counted, stream);
        CHECK(cubScanWaitsRecovered(patient.kernels, temp, stream) == 0);
    }
    // through the Expression: one Scan stage
    const FusedEquation running = FusedEquation::compile(Expression::outputs({{"y", Expression::input("x").scan(ScanOp::Max)}}).physicalOutputs(), 0);
    StampedExecutionPlan plan = running.stamp({{"x", rows}}, stream);
    CHECK((plan.stageKindNames() == std::vector<std::string>{"Scan"}));
    plan.run();
    CHECK((toHostRaw<uint32_t>(plan.output("y"), stream) == std::vector<uint32_t>{2, 3, 3, 4, 5, 5, 5, 5}));
}

static void deviceSelectAndTopK(Stream& stream) {
    // plan / shared temporary storage / run of select-flagged and the four top-k families, on the reference's literal vectors
    // (CubDevicePrimitivesTest.cpp:664-1030 there: TopKKeysLargestAndSmallestUseCubDeviceTopK, TopKPairsCarriesUint32IndexValues,
    // TopKCapsKToNumItems, SelectFlagged*, SegmentedTopK*, the *Rejects* cases)
    auto upload = [&](const std::vector<uint32_t>& v) {
        Tensor host(cpuPlacement, TensorDescriptor(DataType::UINT32, {v.size()}));
        std::memcpy(host.getMemPtr<uint32_t>(), v.data(), v.size() * 4);
        Tensor device(gpuPlacement, TensorDescriptor(DataType::UINT32, {v.size()}));
        device.copyFromAsync(host, stream);
        stream.synchronize();
        return device;
    };
    auto uploadBytes = [&](const std::vector<uint8_t>& v, DataType dtype) {
        Tensor host(cpuPlacement, TensorDescriptor(dtype, {v.size()}));
        std::memcpy(host.getMemPtr(), v.data(), v.size());
        Tensor device(gpuPlacement, TensorDescriptor(dtype, {v.size()}));
        device.copyFromAsync(host, stream);
        stream.synchronize();
        return device;
    };
    {
        const Tensor keys = upload({5, 3, 1, 7, 8, 2, 4, 6});
        Tensor largestOut(gpuPlacement, TensorDescriptor(DataType::UINT32, {3})), smallestOut(gpuPlacement, TensorDescriptor(DataType::UINT32, {4}));
        const CubDeviceTopKKeysPlan largest = prepareCubDeviceTopKKeys(keys, largestOut, 8, 3, CubTopKOrder::Largest);
        const CubDeviceTopKKeysPlan smallest = prepareCubDeviceTopKKeys(keys, smallestOut, 8, 4, CubTopKOrder::Smallest);
        CHECK(largest.key_dtype == DataType::UINT32 && largest.num_items == 8 && largest.k == 3 && largest.order == CubTopKOrder::Largest);
        CHECK(cubDeviceTopKKeysTempBytes(keys, largestOut, 8, 3, CubTopKOrder::Largest) == largest.temp_storage_bytes);
        const CubTemporaryStoragePlan shared = cubMaxTemporaryStoragePlan(
            {cubTemporaryStoragePlan(gpuPlacement, largest.temp_storage_bytes), cubTemporaryStoragePlan(gpuPlacement, smallest.temp_storage_bytes)});
        CHECK(shared.bytes >= largest.temp_storage_bytes && shared.bytes >= smallest.temp_storage_bytes);
        const Tensor temp = allocateCubTemporaryStorage(shared);
        cubDeviceTopKKeys(largest, temp, keys, largestOut, stream);
        cubDeviceTopKKeys(smallest, temp, keys, smallestOut, stream);
        std::vector<uint32_t> l = toHostRaw<uint32_t>(largestOut, stream), sm = toHostRaw<uint32_t>(smallestOut, stream);
        std::sort(l.begin(), l.end(), std::greater<uint32_t>());
        std::sort(sm.begin(), sm.end());
        CHECK((l == std::vector<uint32_t>{8, 7, 6}));
        CHECK((sm == std::vector<uint32_t>{1, 2, 3, 4}));
        // k beyond the input is capped; the one-call form takes the byte count
        const Tensor three = upload({5, 3, 7});
        Tensor capped(gpuPlacement, TensorDescriptor(DataType::UINT32, {3}));
        cubDeviceTopKKeys(temp, shared.bytes, three, capped, 3, 99, stream);
        std::vector<uint32_t> c = toHostRaw<uint32_t>(capped, stream);
        std::sort(c.begin(), c.end(), std::greater<uint32_t>());
        CHECK((c == std::vector<uint32_t>{7, 5, 3}));
        CHECK(throwsAs<std::invalid_argument>([&] { cubDeviceTopKKeys(temp, 1, three, capped, 3, 2, stream); }));
        CHECK(throwsAs<std::invalid_argument>([&] { cubDeviceTopKKeys(largest, allocateCubTemporaryStorage(gpuPlacement, 1), keys, largestOut, stream); }));
        Tensor fpOut(gpuPlacement, TensorDescriptor(DataType::FP32, {2})), smallOut(gpuPlacement, TensorDescriptor(DataType::UINT32, {1}));
        CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceTopKKeys(three, fpOut, 3, 2); }));
        CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceTopKKeys(three, smallOut, 3, 2); }));
        const Tensor fp8In(gpuPlacement, TensorDescriptor(DataType::FP8_E4M3, {2}));
        Tensor fp8Out(gpuPlacement, TensorDescriptor(DataType::FP8_E4M3, {1}));
        CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceTopKKeys(fp8In, fp8Out, 2, 1); }));
        CHECK(isCubTopKKeyDTypeSupported(DataType::BF16) && !isCubTopKKeyDTypeSupported(DataType::FP8_E4M3) && !isCubTopKKeyDTypeSupported(DataType::UINT64));
        CHECK(isCubTopKValueDTypeSupported(DataType::UINT32) && !isCubTopKValueDTypeSupported(DataType::FP32));
    }
    {
        const Tensor keys = gpuFrom({5.0f, -3.0f, 1.0f, 7.0f, 8.0f, 2.0f, 4.0f, 6.0f}, {8}, stream);
        const Tensor values = upload({0, 1, 2, 3, 4, 5, 6, 7});
        Tensor keysOut(gpuPlacement, TensorDescriptor(DataType::FP32, {4})), valuesOut(gpuPlacement, TensorDescriptor(DataType::UINT32, {4}));
        const CubDeviceTopKPairsPlan plan = prepareCubDeviceTopKPairs(keys, keysOut, values, valuesOut, 8, 4, CubTopKOrder::Largest);
        CHECK(plan.value_dtype == DataType::UINT32);
        cubDeviceTopKPairs(plan, allocateCubTemporaryStorage(cubTemporaryStoragePlan(gpuPlacement, plan.temp_storage_bytes)), keys, keysOut, values, valuesOut,
                           stream);
        const std::vector<float> k = toHostF32(keysOut, stream);
        const std::vector<uint32_t> v = toHostRaw<uint32_t>(valuesOut, stream);
        std::vector<std::pair<float, uint32_t>> pairs;
        for (size_t i = 0; i < k.size(); ++i) pairs.emplace_back(k[i], v[i]);
        std::sort(pairs.begin(), pairs.end(), [](const auto& a, const auto& b) { return a.first > b.first; });
        CHECK((pairs == std::vector<std::pair<float, uint32_t>>{{8.0f, 4u}, {7.0f, 3u}, {6.0f, 7u}, {5.0f, 0u}}));
        const Tensor fpValues = gpuFrom({10.0f, 20.0f, 30.0f}, {3}, stream);
        Tensor fpValuesOut(gpuPlacement, TensorDescriptor(DataType::FP32, {2}));
        const Tensor three = upload({1, 2, 3});
        Tensor twoOut(gpuPlacement, TensorDescriptor(DataType::UINT32, {2}));
        CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceTopKPairs(three, twoOut, fpValues, fpValuesOut, 3, 2); }));
    }
    {
        const Tensor input = upload({10, 20, 30, 40, 50, 60});
        const Tensor flags = uploadBytes({1, 0, 1, 0, 0, 1}, DataType::BOOLEAN);
        Tensor output(gpuPlacement, TensorDescriptor(DataType::UINT32, {6})), count(gpuPlacement, TensorDescriptor(DataType::UINT32, {1}));
        const CubDeviceSelectFlaggedPlan plan = prepareCubDeviceSelectFlagged(input, flags, output, count, 6);
        CHECK(plan.input_dtype == DataType::UINT32 && plan.flag_dtype == DataType::BOOLEAN && plan.num_items == 6);
        CHECK(cubDeviceSelectFlaggedTempBytes(input, flags, output, count, 6) == plan.temp_storage_bytes);
        const Tensor temp = allocateCubTemporaryStorage(cubTemporaryStoragePlan(gpuPlacement, plan.temp_storage_bytes));
        cubDeviceSelectFlagged(plan, temp, input, flags, output, count, stream);
        CHECK((toHostRaw<uint32_t>(count, stream) == std::vector<uint32_t>{3}));
        const std::vector<uint32_t> selected = toHostRaw<uint32_t>(output, stream);
        CHECK((std::vector<uint32_t>(selected.begin(), selected.begin() + 3) == std::vector<uint32_t>{10, 30, 60}));
        // no items: only the count is written
        Tensor dirty = upload({77});
        const Tensor byteFlags = uploadBytes({1}, DataType::UINT8);
        Tensor one(gpuPlacement, TensorDescriptor(DataType::UINT32, {1}));
        const CubDeviceSelectFlaggedPlan none = prepareCubDeviceSelectFlagged(upload({123}), byteFlags, one, dirty, 0);
        cubDeviceSelectFlagged(none, allocateCubTemporaryStorage(gpuPlacement, none.temp_storage_bytes), upload({123}), byteFlags, one, dirty, stream);
        CHECK((toHostRaw<uint32_t>(dirty, stream) == std::vector<uint32_t>{0}));
        const Tensor fpFlags(gpuPlacement, TensorDescriptor(DataType::FP32, {6}));
        Tensor fpOut(gpuPlacement, TensorDescriptor(DataType::FP32, {6})), fpCount(gpuPlacement, TensorDescriptor(DataType::FP32, {1}));
        CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceSelectFlagged(input, fpFlags, output, count, 6); }));
        CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceSelectFlagged(input, flags, fpOut, count, 6); }));
        CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceSelectFlagged(input, flags, output, fpCount, 6); }));
        CHECK(throwsAs<std::invalid_argument>([&] { cubDeviceSelectFlagged(temp, 0, input, flags, output, count, 6, stream); }));
        CHECK(isCubSelectFlagDTypeSupported(DataType::BOOLEAN) && isCubSelectFlagDTypeSupported(DataType::UINT8) && !isCubSelectFlagDTypeSupported(DataType::UINT32));
        CHECK(isCubSelectValueDTypeSupported(DataType::FP16) && !isCubSelectValueDTypeSupported(DataType::FP8_E5M2));
    }
    {
        const Tensor keys = upload({1, 5, 3, 9, 2, 10, 4, 8, 6, 7, 11, 15, 12, 14, 13});
        Tensor largestOut(gpuPlacement, TensorDescriptor(DataType::UINT32, {6})), smallestOut(gpuPlacement, TensorDescriptor(DataType::UINT32, {6}));
        const CubDeviceSegmentedTopKKeysPlan largest = prepareCubDeviceSegmentedTopKKeys(keys, largestOut, 3, 5, 2, CubTopKOrder::Largest);
        const CubDeviceSegmentedTopKKeysPlan smallest = prepareCubDeviceSegmentedTopKKeys(keys, smallestOut, 3, 5, 2, CubTopKOrder::Smallest);
        CHECK(largest.num_segments == 3 && largest.segment_size == 5 && largest.k == 2);
        const Tensor temp = allocateCubTemporaryStorage(cubMaxTemporaryStoragePlan(
            {cubTemporaryStoragePlan(gpuPlacement, largest.temp_storage_bytes), cubTemporaryStoragePlan(gpuPlacement, smallest.temp_storage_bytes)}));
        cubDeviceSegmentedTopKKeys(largest, temp, keys, largestOut, stream);
        cubDeviceSegmentedTopKKeys(smallest, temp, keys, smallestOut, stream);
        std::vector<uint32_t> l = toHostRaw<uint32_t>(largestOut, stream), sm = toHostRaw<uint32_t>(smallestOut, stream);
        for (size_t at = 0; at < 6; at += 2) {
            std::sort(l.begin() + at, l.begin() + at + 2, std::greater<uint32_t>());
            std::sort(sm.begin() + at, sm.begin() + at + 2);
        }
        CHECK((l == std::vector<uint32_t>{9, 5, 10, 8, 15, 14}));
        CHECK((sm == std::vector<uint32_t>{1, 2, 4, 6, 11, 12}));
        const Tensor floatKeys = gpuFrom({1, 5, 3, 9, 2, 10, 4, 8, 6, 7, 11, 15, 12, 14, 13}, {15}, stream);
        const Tensor values = upload({100, 101, 102, 103, 104, 200, 201, 202, 203, 204, 300, 301, 302, 303, 304});
        Tensor keysOut(gpuPlacement, TensorDescriptor(DataType::FP32, {6})), valuesOut(gpuPlacement, TensorDescriptor(DataType::UINT32, {6}));
        const CubDeviceSegmentedTopKPairsPlan pairsPlan = prepareCubDeviceSegmentedTopKPairs(floatKeys, keysOut, values, valuesOut, 3, 5, 2, CubTopKOrder::Largest);
        cubDeviceSegmentedTopKPairs(pairsPlan, temp, floatKeys, keysOut, values, valuesOut, stream);
        const std::vector<float> k = toHostF32(keysOut, stream);
        const std::vector<uint32_t> v = toHostRaw<uint32_t>(valuesOut, stream);
        std::vector<std::pair<float, uint32_t>> pairs;
        for (size_t i = 0; i < k.size(); ++i) pairs.emplace_back(k[i], v[i]);
        for (size_t at = 0; at < 6; at += 2) std::sort(pairs.begin() + at, pairs.begin() + at + 2, [](const auto& a, const auto& b) { return a.first > b.first; });
        CHECK((pairs == std::vector<std::pair<float, uint32_t>>{{9.0f, 103u}, {5.0f, 101u}, {10.0f, 200u}, {8.0f, 202u}, {15.0f, 301u}, {14.0f, 303u}}));
        CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceSegmentedTopKKeys(keys, largestOut, 3, 5, 5); }));  // k must stay below the segment
        CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceSegmentedTopKKeys(keys, largestOut, 3, 0, 1); }));
        CHECK(throwsAs<std::invalid_argument>([&] { (void)prepareCubDeviceSegmentedTopKKeys(keys, largestOut, 4, 5, 1); }));  // keys_in too small
        const CubDeviceSegmentedTopKKeysPlan nothing = prepareCubDeviceSegmentedTopKKeys(keys, largestOut, 3, 5, 0);
        cubDeviceSegmentedTopKKeys(nothing, temp, keys, largestOut, stream);  // k == 0: nothing to do, nothing thrown
    }
}

static void softmaxPlansAndRowKernel(Stream& stream) {
    const uint64_t rows = 7, cols = 130;
    std::vector<float> x(rows * cols);
    for (size_t i = 0; i < x.size(); ++i) x[i] = 3.0f * std::sin(0.37f * i);
    Tensor tx = gpuFrom(x, {rows, cols}, stream, DataType::BF16);
    const std::vector<float> xb = toHostF32(tx, stream);  // the bf16-rounded values the kernels see
    Expression ix = Expression::input("x");
    Expression e = (ix - ix.reduce_max({1})).exp();
    FusedEquation eq = FusedEquation::compile((e / e.reduce_sum({1})).expression(), 0);
    auto check = [&](const StampedExecutionPlan& plan) {
        const std::vector<float> got = toHostF32(plan.output(), stream);
        for (uint64_t r = 0; r < rows; ++r) {
            double m = -1e30, sum = 0;
            for (uint64_t c = 0; c < cols; ++c) m = std::max<double>(m, xb[r * cols + c]);
            for (uint64_t c = 0; c < cols; ++c) sum += std::exp(xb[r * cols + c] - m);
            for (uint64_t c = 0; c < cols; c += 11) CHECK_NEAR(got[r * cols + c], std::exp(xb[r * cols + c] - m) / sum, 2e-6);
        }
    };
    StampedExecutionPlan fused = eq.stamp({{"x", tx}}, stream);
    CHECK((fused.stageKindNames() == std::vector<std::string>{"FusedRowKernel"}));
    CHECK(fused.output().getDataType() == DataType::FP32);
    fused.run();
    check(fused);
    setenv("THOR_DISABLE_ROW_FUSION", "1", 1);
    StampedExecutionPlan staged = eq.stamp({{"x", tx}}, stream);
    unsetenv("THOR_DISABLE_ROW_FUSION");
    // the reference's lowering (CommonInputFusionTest.cpp:281-327)
    CHECK((staged.stageKindNames() == std::vector<std::string>{"Reduction", "FusedKernel", "Reduction", "FusedKernel"}));
    CHECK((staged.reductionPaths() == std::vector<CubReductionPath>{CubReductionPath::ContiguousFixedSegment, CubReductionPath::ContiguousFixedSegment}));
    staged.run();
    check(staged);
    // Expression::softmax(): the same function, result in the input's dtype (the reference's softmax stage keeps it)
    FusedEquation method = FusedEquation::compile(ix.softmax().expression(), 0);
    StampedExecutionPlan viaMethod = method.stamp({{"x", tx}}, stream);
    CHECK((viaMethod.stageKindNames() == std::vector<std::string>{"FusedRowKernel"}));
    CHECK(viaMethod.output().getDataType() == DataType::BF16);
    viaMethod.run();
    const std::vector<float> rounded = toHostF32(viaMethod.output(), stream), exact = toHostF32(fused.output(), stream);
    for (size_t i = 0; i < rounded.size(); i += 7) CHECK_NEAR(rounded[i], exact[i], 4e-3 * exact[i] + 1e-9);
    CHECK(throwsAs<std::invalid_argument>([&] { (void)ix.softmax(SoftmaxAlgorithm::Log); }));
}

// ---- smaller entry points of the boundary (Expression.h:664,683-684,711-714,1010 and FusedEquation.h:594-599 there) ---------------
static void boundaryShorthandsAndSubstitution() {
    Expression x = Expression::input("x");
    const PhysicalExpression inclusive = x.inclusiveScanSum().expression(), exclusive = Expression::exclusiveScanSum(x, 1).expression();
    CHECK(inclusive.nodes.back().op == ExprOp::SCAN && inclusive.nodes.back().scan_op == ScanOp::Sum && inclusive.nodes.back().scan_mode == ScanMode::Inclusive);
    CHECK(exclusive.nodes.back().op == ExprOp::SCAN && exclusive.nodes.back().scan_mode == ScanMode::Exclusive && exclusive.nodes.back().scan_axis == 1);
    CHECK(Expression::prefixCount(x, false).expression().nodes.back().op == ExprOp::SCAN);
    // substituteInput: every use of b reads exp(d) instead; b disappears from the inputs, d appears
    Expression a = Expression::input("a"), b = Expression::input("b"), c = Expression::input("c"), d = Expression::input("d");
    Expression composed = ((a * b + c) * b).substituteInput("b", d.exp());
    CHECK((composed.getInputNames() == std::set<std::string>{"a", "c", "d"}));
    Expression untouched = (a + c).substituteInput("b", d);
    CHECK((untouched.getInputNames() == std::set<std::string>{"a", "c"}));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)a.substituteInput("", d); }));
    // stridedViewBackward: validation of the reference, node carries the view and the source shape
    Expression g = Expression::input("g");
    const PhysicalExpression routed = g.stridedViewBackward({4, 6}, {2, 3}, {6, 1}, 7).expression();
    CHECK(routed.nodes.back().op == ExprOp::STRIDED_VIEW_BACKWARD && (routed.nodes.back().fill_dims == std::vector<uint64_t>{4, 6}));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)g.stridedViewBackward({}, {2, 3}, {6, 1}); }));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)g.stridedViewBackward({4, 6}, {2, 3}, {6}); }));
    CHECK(throwsAs<std::invalid_argument>([&] { (void)g.stridedViewBackward({4, 6}, {2, 3}, {1, 1}); }));  // overlapping rows
    // RoPE options that this build does not implement are refused, not ignored
    RotaryPositionEmbeddingOptions options;
    options.compute_dtype = DataType::BF16;
    CHECK(throwsAs<std::invalid_argument>([&] { (void)x.rotaryPositionEmbedding(options); }));
    options.compute_dtype = DataType::FP32;
    options.allow_in_place_materialization = true;  // a permission: accepted
    (void)x.rotaryPositionEmbedding(options);
    // conditional outputs: same branch names in the same order, at least one elif for ifElifElse (Expression.cpp:5342-5390 there)
    const Expression selector = Expression::input("selector");
    const Outputs thenOutputs = Expression::outputs({{"y", x + 10.0}}), elseOutputs = Expression::outputs({{"y", x + 40.0}});
    const Outputs chosen = Outputs::ifElse(selector > 0.0, thenOutputs, elseOutputs);
    CHECK(!chosen.isConditional() && chosen.namedOutputs().size() == 1 && chosen.namedOutputs()[0].name == "y");
    CHECK(chosen.expression()->nodes[chosen.namedOutputs()[0].node_idx].op == ExprOp::WHERE);
    CHECK(throwsAs<std::runtime_error>([&] { (void)Outputs::ifElse(selector > 0.0, thenOutputs, Expression::outputs({{"z", x}})); }));
    CHECK(throwsAs<std::runtime_error>([&] { (void)Outputs::ifElifElse(selector > 2.0, thenOutputs, {}, elseOutputs); }));
    const Outputs ladder = Outputs::ifElifElse(selector > 2.0, thenOutputs, {{selector > 1.0, Expression::outputs({{"y", x + 20.0}})}}, elseOutputs);
    CHECK(FusedEquation::compile(ladder.physicalOutputs(), 0).getOutputShapes({{"x", Tensor(cpuPlacement, TensorDescriptor(DataType::FP32, {4, 5}))},
                                                                               {"selector", Tensor(cpuPlacement, TensorDescriptor(DataType::FP32, {1}))}})
              .at("y") == std::vector<uint64_t>({4, 5}));
}

static void boundaryRequestedShapesAndSubstitutionExecution(Stream& stream) {
    const uint64_t rows = 6, cols = 50;
    std::vector<float> xs(rows * cols), ds(rows * cols);
    for (size_t i = 0; i < xs.size(); ++i) {
        xs[i] = float(int(i % 9) - 4);
        ds[i] = 0.01f * float(int(i % 7));
    }
    Tensor tx = gpuFrom(xs, {rows, cols}, stream), td = gpuFrom(ds, {rows, cols}, stream);
    Expression x = Expression::input("x");
    FusedEquation rowSum = FusedEquation::compile(x.reduce_sum({1}).expression(), 0);
    StampedExecutionPlan plain = rowSum.stamp({{"x", tx}}, stream);
    CHECK((plain.output().getDimensions() == std::vector<uint64_t>{rows, 1}));
    StampedExecutionPlan flat = rowSum.stamp({{"x", tx}}, stream, {}, {}, {{"output", {rows}}});
    CHECK((flat.output().getDimensions() == std::vector<uint64_t>{rows}));
    flat.run();
    const std::vector<float> sums = toHostF32(flat.output(), stream);
    for (uint64_t r = 0; r < rows; ++r) {
        double want = 0;
        for (uint64_t c = 0; c < cols; ++c) want += xs[r * cols + c];
        CHECK(sums[r] == float(want));
    }
    StampedExecutionPlan single = rowSum.stampSingleOutput({{"x", tx}}, stream, {}, std::nullopt, {1, rows, 1});
    CHECK((single.output().getDimensions() == std::vector<uint64_t>{1, rows, 1}));
    CHECK(throwsAs<std::runtime_error>([&] { (void)rowSum.stamp({{"x", tx}}, stream, {}, {}, {{"output", {rows + 1}}}); }));
    CHECK(throwsAs<std::runtime_error>([&] { (void)rowSum.stamp({{"x", tx}}, stream, {}, {}, {{"nonesuch", {rows}}}); }));
    Tensor own(gpuPlacement, TensorDescriptor(DataType::FP32, {rows, 1}));
    StampedExecutionPlan kept = rowSum.stamp({{"x", tx}}, stream, {}, {{"output", own}}, {{"output", {rows}}});
    CHECK((kept.output().getDimensions() == std::vector<uint64_t>{rows, 1}));  // the caller's tensor keeps its dimensions

    // substituteInput runs like the expression written out by hand
    Expression b = Expression::input("b"), d = Expression::input("d");
    FusedEquation viaSubstitution = FusedEquation::compile(((x * b + 1.0) * b).substituteInput("b", d.exp()).expression(), 0);
    FusedEquation byHand = FusedEquation::compile(((x * d.exp() + 1.0) * d.exp()).expression(), 0);
    StampedExecutionPlan p1 = viaSubstitution.stamp({{"x", tx}, {"d", td}}, stream), p2 = byHand.stamp({{"x", tx}, {"d", td}}, stream);
    p1.run();
    p2.run();
    CHECK(toHostF32(p1.output(), stream) == toHostF32(p2.output(), stream));

    // stridedViewBackward places a gradient shaped like the view into zeros shaped like the source
    std::vector<float> gs = {1, 2, 3, 4, 5, 6};
    Tensor tg = gpuFrom(gs, {2, 3}, stream);
    FusedEquation place = FusedEquation::compile(Expression::input("g").stridedViewBackward({4, 6}, {2, 3}, {6, 1}, 7).expression(), 0);
    StampedExecutionPlan placed = place.stamp({{"g", tg}}, stream);
    placed.run();
    const std::vector<float> routed = toHostF32(placed.output(), stream);
    CHECK(routed.size() == 24);
    for (size_t i = 0; i < routed.size(); ++i) {
        float want = 0;
        for (int r = 0; r < 2; ++r)
            for (int c = 0; c < 3; ++c)
                if (i == size_t(7 + 6 * r + c)) want = gs[r * 3 + c];
        CHECK(routed[i] == want);
    }
}

// ---- stage scheduling: lanes, forks and joins (test/Utilities/Expression/StampedExecutionPlanSchedulerTest.cpp:18-89 there) ----------
static StampedExecutionStage barrierStage(std::vector<uint32_t> dependencies = {}, uint32_t gpu = 0) {
    return StampedExecutionStage::dependencyBarrier(gpu, std::move(dependencies));
}

static void stagePlanScheduler() {
    typedef std::vector<uint32_t> U;
    typedef std::vector<bool> B;
    {  // a linear chain stays on the caller's lane: no events at all
        std::vector<StampedExecutionStage> stages = {barrierStage(), barrierStage({0}), barrierStage({1}), barrierStage({2})};
        const detail::StampedExecutionSchedule s = detail::buildStampedExecutionSchedule(stages, 0);
        CHECK((s.stage_lane_indices == U{0, 0, 0, 0}));
        CHECK((s.lane_gpu_nums == U{0}));
        CHECK(!s.needs_caller_ready_event);
        CHECK((s.stage_needs_completion_event == B{false, false, false, false}));
    }
    {  // a fork opens one helper lane, the join comes back to the caller's lane
        std::vector<StampedExecutionStage> stages = {barrierStage(), barrierStage({0}), barrierStage({0}), barrierStage({1, 2}), barrierStage({3})};
        const detail::StampedExecutionSchedule s = detail::buildStampedExecutionSchedule(stages, 0);
        CHECK((s.stage_lane_indices == U{0, 0, 1, 0, 0}));
        CHECK((s.lane_gpu_nums == U{0, 0}));
        CHECK(!s.needs_caller_ready_event);
        CHECK((s.stage_needs_completion_event == B{true, false, true, false, false}));
    }
    {  // two independent roots: the helper root waits for the caller-ready event, one event joins it back
        std::vector<StampedExecutionStage> stages = {barrierStage(), barrierStage(), barrierStage({0, 1}), barrierStage({2})};
        const detail::StampedExecutionSchedule s = detail::buildStampedExecutionSchedule(stages, 0);
        CHECK((s.stage_lane_indices == U{0, 1, 0, 0}));
        CHECK((s.lane_gpu_nums == U{0, 0}));
        CHECK(s.needs_caller_ready_event);
        CHECK((s.stage_needs_completion_event == B{false, true, false, false}));
    }
    {  // nested forks: only parallel branches get lanes
        std::vector<StampedExecutionStage> stages = {barrierStage(),    barrierStage({0}), barrierStage({0}),    barrierStage({1}),
                                                     barrierStage({1}), barrierStage({2}), barrierStage({3, 4}), barrierStage({5, 6})};
        const detail::StampedExecutionSchedule s = detail::buildStampedExecutionSchedule(stages, 0);
        CHECK((s.stage_lane_indices == U{0, 0, 1, 0, 2, 1, 0, 0}));
        CHECK((s.lane_gpu_nums == U{0, 0, 0}));
    }
    {  // a helper branch that nothing consumes still gets an event: the run joins it at the end
        std::vector<StampedExecutionStage> stages = {barrierStage(), barrierStage({0}), barrierStage({0})};
        const detail::StampedExecutionSchedule s = detail::buildStampedExecutionSchedule(stages, 0);
        CHECK((s.stage_lane_indices == U{0, 0, 1}));
        CHECK((s.stage_needs_completion_event == B{true, false, true}));
    }
    {  // dependencies must point backwards
        std::vector<StampedExecutionStage> stages = {barrierStage({1}), barrierStage()};
        CHECK(throwsAs<std::runtime_error>([&] { (void)detail::buildStampedExecutionSchedule(stages, 0); }));
    }
}

static void stagePlanForksAndJoins(Stream& stream) {
    // barrier-only plan, submitted many times without synchronising in between: events are reused from run to run
    {
        std::vector<StampedExecutionStage> stages = {barrierStage(), barrierStage({0}), barrierStage({0}), barrierStage({1, 2})};
        StampedExecutionPlan plan(std::move(stages), {}, stream);
        CHECK(plan.schedule().lane_gpu_nums.size() == 2);
        setenv("THOR_STAGE_OVERLAP", "1", 1);  // helper lanes are opt-in: on this hardware one lane measured faster
        for (int run = 0; run < 64; ++run) plan.run();
        unsetenv("THOR_STAGE_OVERLAP");
        stream.synchronize();
    }
    // two independent reductions of different inputs, then arithmetic on both: the branches run on two lanes and the result is the
    // staged one, run after run, with the inputs rewritten on the caller's stream between runs (the helper lane must wait for them)
    // (rows of different lengths, so that the two reductions cannot share one pass)
    const uint64_t rows = 300, cols = 1000, colsB = 500;
    std::vector<float> a(rows * cols), b(rows * colsB);
    for (size_t i = 0; i < a.size(); ++i) a[i] = float(int(i % 17) - 8);
    for (size_t i = 0; i < b.size(); ++i) b[i] = float(int(i % 13) - 6);
    Tensor ta = gpuFrom(a, {rows, cols}, stream), tb = gpuFrom(b, {rows, colsB}, stream);
    Expression ia = Expression::input("a"), ib = Expression::input("b");
    Expression combined = ia.reduce_sum({1}) * 2.0 + ib.reduce_max({1});
    FusedEquation eq = FusedEquation::compile(combined.expression(), 0);
    StampedExecutionPlan plan = eq.stamp({{"a", ta}, {"b", tb}}, stream);
    const detail::StampedExecutionSchedule& schedule = plan.schedule();
    CHECK(schedule.lane_gpu_nums.size() == 2);
    CHECK(schedule.needs_caller_ready_event);
    auto expect = [&](const std::vector<float>& av, const std::vector<float>& bv) {
        const std::vector<float> got = toHostF32(plan.output(), stream);
        for (uint64_t r = 0; r < rows; ++r) {
            double sum = 0, top = -1e30;
            for (uint64_t c = 0; c < cols; ++c) sum += av[r * cols + c];
            for (uint64_t c = 0; c < colsB; ++c) top = std::max<double>(top, bv[r * colsB + c]);
            CHECK(got[r] == float(sum * 2.0 + top));  // small integers: exact in any order
        }
    };
    setenv("THOR_STAGE_OVERLAP", "1", 1);
    plan.run();
    expect(a, b);
    Tensor hostB(cpuPlacement, TensorDescriptor(DataType::FP32, {rows, colsB}));
    for (int round = 1; round <= 3; ++round) {
        for (size_t i = 0; i < b.size(); ++i) b[i] = float(int((i + round) % 11) - 5);
        std::memcpy(hostB.getMemPtr<float>(), b.data(), b.size() * sizeof(float));
        tb.copyFromAsync(hostB, stream);  // queued on the caller's stream; the helper lane's reduction of b must see it
        plan.run();
        expect(a, b);
    }
    // the same plan on one lane (the default) gives the same values
    unsetenv("THOR_STAGE_OVERLAP");
    plan.run();
    expect(a, b);
}

static void typeConverterOnGpuAndTensorViews(Stream& stream) {
    const uint64_t n = 100003;
    std::vector<float> x(n);
    for (uint64_t i = 0; i < n; ++i) x[i] = (i % 100 == 0 ? 1e5f : 1.0f) * std::sin(0.001f * i) * (i % 100 == 1 ? 1e-40f : 1.0f);
    Tensor src = gpuFrom(x, {n}, stream);
    Tensor half(gpuPlacement, TensorDescriptor(DataType::FP16, {n}));
    TypeConverter::convertType(src.getMemPtr(), half.getMemPtr(), DataType::FP32, DataType::FP16, (long)n, stream, 0);
    const std::vector<uint16_t> got = toHostRaw<uint16_t>(half, stream);
    std::vector<uint16_t> want(n);
    TypeConverter::cpuConvertNow(x.data(), want.data(), DataType::FP32, DataType::FP16, (long)n);
    CHECK(got == want);
    // in place, widening back (walks backwards)
    Tensor wide(gpuPlacement, TensorDescriptor(DataType::FP32, {n}));
    wide.copyFromAsync(half, stream);  // device-to-device copy with conversion
    const std::vector<float> back = toHostF32(wide, stream);
    std::vector<float> wantBack(n);
    TypeConverter::cpuConvertNow(want.data(), wantBack.data(), DataType::FP16, DataType::FP32, (long)n);
    CHECK(std::memcmp(back.data(), wantBack.data(), n * 4) == 0);
    // a transposed view reduces through the strided path
    Tensor m = gpuFrom({1, 2, 3, 4, 5, 6}, {2, 3}, stream);
    Tensor view = m.aliasView({3, 2}, {1, 3});
    auto stamped = CubReduction(CubReductionOp::Sum, 1u).stamp(view, stream);
    stamped->run();
    CHECK((toHostF32(stamped->getOutputTensor(), stream) == std::vector<float>{5, 7, 9}));
    CHECK(throwsAs<std::invalid_argument>([&] { Tensor outside = m.aliasView({4, 2}, {1, 3}); }));  // would read past the allocation
}

int main(int argc, char** argv) {
    const std::string mode = argc > 1 ? argv[1] : "gpu";
    struct Case {
        const char* name;
        std::function<void()> body;
    };
    std::vector<Case> cases = {{"geometryPathsAndErrors", geometryPathsAndErrors},
                               {"dtypeResolutionAndStageSplit", dtypeResolutionAndStageSplit},
                               {"cpuTypeConverter", cpuTypeConverter},
                               {"raggedExpressionStructure", raggedExpressionStructure},
                               {"autodiffGraphStructure", autodiffGraphStructure},
                               {"scanExpressionStructure", scanExpressionStructure},
                               {"ropeExpressionStructure", ropeExpressionStructure},
                               {"stagePlanScheduler", stagePlanScheduler},
                               {"boundaryShorthandsAndSubstitution", boundaryShorthandsAndSubstitution}};
    if (mode == "gpu") {
        auto withStream = [](void (*f)(Stream&)) {
            return [f] {
                Stream stream(0);
                f(stream);
            };
        };
        cases.push_back({"valueReductionsSmallExact", withStream(valueReductionsSmallExact)});
        cases.push_back({"argReductionsTiesAndNaN", withStream(argReductionsTiesAndNaN)});
        cases.push_back({"offsetSegmentedReductions", withStream(offsetSegmentedReductions)});
        cases.push_back({"raggedExpressionExecution", withStream(raggedExpressionExecution)});
        cases.push_back({"expressionConfig1AndRuntimeScalars", withStream(expressionConfig1AndRuntimeScalars)});
        cases.push_back({"softmaxPlansAndRowKernel", withStream(softmaxPlansAndRowKernel)});
        cases.push_back({"autodiffExecution", withStream(autodiffExecution)});
        cases.push_back({"devicePrefixScans", withStream(devicePrefixScans)});
        cases.push_back({"deviceSelectAndTopK", withStream(deviceSelectAndTopK)});
        cases.push_back({"ropeExecution", withStream(ropeExecution)});
        cases.push_back({"stagePlanForksAndJoins", withStream(stagePlanForksAndJoins)});
        cases.push_back({"boundaryRequestedShapesAndSubstitutionExecution", withStream(boundaryRequestedShapesAndSubstitutionExecution)});
        cases.push_back({"typeConverterOnGpuAndTensorViews", withStream(typeConverterOnGpuAndTensorViews)});
    }
    for (const Case& c : cases) {
        const int before = failures;
        std::printf("[ RUN  ] %s\n", c.name);
        std::fflush(stdout);
        try {
            c.body();
        } catch (const std::exception& e) {
            ++failures;
            std::printf("  unexpected exception: %s\n", e.what());
        }
        std::printf("[ %s ] %s\n", failures == before ? " OK " : "FAIL", c.name);
    }
    std::printf("%d checks, %d failures\n", checks, failures);
    return failures == 0 ? 0 : 1;
}
