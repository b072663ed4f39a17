// Internal: turns a reduction geometry into a kernel shape (vector width, lanes per row, split factor, grid), generates
// the traits struct that specialises the device templates for that shape, and compiles it.
#pragma once

#include "Utilities/TensorOperations/Cub/CubReduction.h"

#include <cstdint>
#include <optional>
#include <string>
#include <vector>

namespace ThorImplementation {

struct ReductionKernelRequest {
    bool isArg = false;
    CubReductionOp valueOp = CubReductionOp::Sum;
    CubArgReductionOp argOp = CubArgReductionOp::ArgMax;
    DataType inputDType = DataType::FP32;
    DataType valueOutputDType = DataType::FP32;
    DataType indexOutputDType = DataType::UINT32;
    bool writeValue = true;
    bool writeIndex = false;
    CubReductionGeometry geometry;
    uint64_t inputAlignmentBytes = 256;  // largest power of two (capped at 256) dividing every source base address
    int deviceNum = 0;

    // ---- offset-segmented form: values [rows, trailing] reduced over row ranges given by an offsets tensor at run time ----
    // geometry.output_elements = segments * trailing, geometry.input_elements = rows * trailing; the kernels take the
    // offsets pointer as their last argument.
    bool segmented = false;
    uint64_t segments = 0, segmentedRows = 0, trailing = 1;
    bool offsetsAre64 = false;

    // ---- fused form: several value reductions over the same geometry, fed by an elementwise prologue ------------------
    // When `values` is empty the request is the plain one above: one source of inputDType, the value itself reduced.
    struct Source {
        enum class Kind : uint8_t {
            Vector,  // same layout as the reduction input: read at the element offset
            Scalar,  // one element, read at [0]
            Kept,    // one element per output (numbered row-major over the kept axes), read at [output]: a per-channel scale
        };
        DataType storage = DataType::FP32;
        Kind kind = Kind::Vector;
        // Kept sources that are broadcast along some of the kept axes as well (a [C, 1, 1] bias under [N, C, H, W] -> [N, C]): the
        // element's offset as a C expression of `slot`, the output's number; empty: the output's number itself.
        std::string keptOffset;
    };
    struct Value {
        CubReductionOp op = CubReductionOp::Sum;
        DataType outputDType = DataType::FP32;
        std::string expression;  // fp32 C expression of the value to accumulate, in terms of the prologue's names
    };
    // Two values that are the statistics of a softmax over the same elements: values[0] = their maximum, values[1] = the sum of
    // exp(element - maximum); values[0].expression is the element, one accumulator ({max, sum}) gathers both in one pass.
    bool onlineSoftmax = false;
    struct Elementwise {
        DataType outputDType = DataType::FP32;
        std::string expression;  // storage-typed C expression of the element to store, in terms of the prologue's names
    };
    std::vector<Source> sources;         // kernel arguments in0, in1, ...
    std::vector<uint32_t> scalarSlots;   // runtime scalars passed by value as float s<slot>, after the sources
    // Statements evaluated once per element before the values are accumulated.  Element k of vector source i is
    // `l.p<i>.v[k]`, scalar and kept source i is `kk.z<i>`, runtime scalars are `s.s<slot>`.
    std::string prologue;
    std::vector<Value> values;           // outputs out0, out1, ... in this order
    // Tensors of the reduction input's shape written by the same pass (arguments e0, e1, ... after the reduction outputs).
    std::vector<Elementwise> elementwise;
};

struct ReductionShape {
    enum class Kernel { All, Rows, Columns, Strided, Segments } kernel = Kernel::All;
    int vec = 1;
    int threads = 256;
    int threadsPerRow = 64;
    int unroll = 4;
    uint64_t blocks = 1;
    uint64_t split = 1;
    bool indexIs64 = false;
    uint32_t gridX = 1, gridY = 1;
    size_t workspaceBytes = 0;
    // Blocks that share an output count in on ticket words and the last one folds the partials (no finishing launch): the
    // words live in the workspace at ticketOffset and must be zero before the first run.
    bool tickets = false;
    uint64_t ticketCount = 0;
    size_t ticketOffset = 0;
    // collapsed axes of the strided kernel
    std::vector<uint64_t> keptDims, keptStrides, reducedDims, reducedStrides;
    // Columns kernel over a view: index (into keptDims) of the kept axis that is contiguous in memory, or -1 for the
    // dense [outer, R, inner] layout
    int laneAxis = -1;
    // Columns whose lanes do not lie on the output's fastest axis: a block reduces this many consecutive coordinates of that axis
    // and writes them out together through LDS (0: every lane stores its own outputs)
    int transposeRows = 0;
    // Segments kernel: rows per block, number of such chunks, smallest team of threads that shares a segment, columns per
    // block of the finishing launch
    uint64_t chunkRows = 0, chunks = 1;
    int minTeam = 1, finishLanes = 1, finishThreads = 256;
    // Segments kernel: rows dealt out to lanes (reduceSegmentsByRows) instead of segments dealt out to teams (reduceSegments)
    bool segmentsByRows = false;
    // Rows kernel: vectors at addresses that are only aligned to the element; the last reduction_size % vec elements of a row go one by one
    bool unalignedVectors = false;
    // Rows kernel over [outer, R, inner] with a small inner extent: outputs per row, their elements interleaved along the row
    int interleave = 1;
    int walkGroup = 4;  // reduceSegmentsByRows: rows of a lane's range that are walked together
    std::string describe() const;
};

uint64_t pointerAlignment(const void* p);

// Length of the runs of adjacent blocks that the row kernels give to one XCD (thor::xcdBlock in the device prelude); 1 = the
// hardware's round-robin order.  THOR_XCD_RUN overrides the kernel's preferred length (tuning switch).
int xcdRunLength(int preferred);
ReductionShape planReductionShape(const ReductionKernelRequest& request);
std::string generateReductionSource(const ReductionKernelRequest& request, const ReductionShape& shape);
ReductionLaunchPlan buildReductionKernels(const ReductionKernelRequest& request);
// The workspace a launch plan needs (nothing when it needs none), with its ticket words cleared; `stream` is synchronised.
std::optional<Tensor> allocateReductionWorkspace(const ReductionLaunchPlan& plan, const TensorPlacement& placement, const Stream& stream);

const char* deviceTypeName(DataType dtype);  // "thor::f16", "float", ...

}  // namespace ThorImplementation
