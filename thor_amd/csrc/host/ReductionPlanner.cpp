#include "ReductionPlanner.h"

#include "Utilities/Common/ScopedGpu.h"
#include "Utilities/Common/Stream.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "thorhip_numeric_embed.h"

#include <algorithm>
#include <cstdlib>
#include <sstream>
#include <stdexcept>

namespace ThorImplementation {

namespace {

constexpr uint64_t kTargetThreads = 256ull * 512ull;  // threads that keep 256 CUs busy with loads in flight
constexpr uint64_t kMaxGridY = 65535;

uint64_t pow2Ceil(uint64_t v) {
    uint64_t p = 1;
    while (p < v) p <<= 1;
    return p;
}

uint64_t ceilDiv(uint64_t a, uint64_t b) { return (a + b - 1) / b; }

// Largest power-of-two element count whose byte size is <= 16, divides every listed extent and fits the alignment.
int chooseVector(uint32_t elementBytes, uint64_t alignmentBytes, std::initializer_list<uint64_t> mustDivide) {
    int vec = static_cast<int>(16 / elementBytes);
    while (vec > 1) {
        bool ok = alignmentBytes % (static_cast<uint64_t>(vec) * elementBytes) == 0;
        for (uint64_t extent : mustDivide) ok = ok && (extent % vec == 0);
        if (ok) break;
        vec /= 2;
    }
    return vec;
}

size_t partialBytes(uint64_t slots, bool isArg, bool indexIs64) {
    size_t bytes = ((slots * 4 + 7) / 8) * 8;
    if (isArg) bytes += slots * (indexIs64 ? 8 : 4);
    return bytes;
}

// Outputs that lanes would scatter (the lane axis is not the output's fastest one) leave through an LDS transpose when the
// writes are a visible share of the traffic and one block can own whole columns: no split of R, R at most 512, at least 16
// coordinates along the output's fastest axis.  Measured on fp32 [512, 8, 16384] seen as [16384, 8, 512], sum over the middle
// axis: 84 us with scattered stores.
int transposeRowsFor(uint64_t split, uint64_t reductionSize, uint64_t fastestOutputExtent, uint64_t laneOutputStride, uint64_t rowBytes) {
    if (std::getenv("THOR_REDUCE_NO_TRANSPOSE") != nullptr) return 0;
    if (split != 1 || laneOutputStride == 1 || reductionSize > 512 || fastestOutputExtent < 16) return 0;
    if (16 * rowBytes > 65536) return 0;  // the block's results wait in LDS: 16 rows of lanes x vector + 1 accumulators
    return 16;
}

// Merges adjacent axes that address memory as one longer axis (outer stride == inner dim * inner stride) and drops
// singleton axes.  Order is preserved, so row-major positions inside the collapsed domain are unchanged.
void collapseAxes(std::vector<uint64_t>& dims, std::vector<uint64_t>& strides) {
    std::vector<uint64_t> d, s;
    for (size_t i = 0; i < dims.size(); ++i) {
        if (dims[i] == 1) continue;
        if (!d.empty() && s.back() == dims[i] * strides[i]) {
            d.back() *= dims[i];
            s.back() = strides[i];
        } else {
            d.push_back(dims[i]);
            s.push_back(strides[i]);
        }
    }
    dims = d;
    strides = s;
}

const char* valueAccumulatorType(CubReductionOp op, int& finalize);

const char* accumulatorType(const ReductionKernelRequest& r, bool indexIs64, int& finalize) {
    finalize = 0;
    if (r.isArg) {
        if (r.argOp == CubArgReductionOp::ArgMax) return indexIs64 ? "ArgAcc<true, u64>" : "ArgAcc<true, u32>";
        return indexIs64 ? "ArgAcc<false, u64>" : "ArgAcc<false, u32>";
    }
    return valueAccumulatorType(r.valueOp, finalize);
}

const char* valueAccumulatorType(CubReductionOp op, int& finalize) {
    finalize = 0;
    switch (op) {
        case CubReductionOp::Sum:
            return "ValueAcc<SumOp>";
        case CubReductionOp::Mean:
            finalize = 1;
            return "ValueAcc<SumOp>";
        case CubReductionOp::L1Norm:
            return "ValueAcc<AbsSumOp>";
        case CubReductionOp::L2Norm:
            finalize = 2;
            return "ValueAcc<SquareSumOp>";
        case CubReductionOp::Product:
            return "ValueAcc<ProductOp>";
        case CubReductionOp::Min:
            return "ValueAcc<MinOp>";
        case CubReductionOp::Max:
            return "ValueAcc<MaxOp>";
    }
    throw std::invalid_argument("Unsupported tensor reduction operation.");
}

std::string offsetFunction(const char* name, const std::vector<uint64_t>& dims, const std::vector<uint64_t>& strides) {
    std::ostringstream out;
    out << "    static __device__ __forceinline__ u64 " << name << "(u64 i) {\n        u64 offset = 0;\n";
    for (size_t a = dims.size(); a-- > 0;) {
        if (a == 0) {
            out << "        offset += i * " << strides[a] << "ull;\n";
        } else {
            out << "        offset += (i % " << dims[a] << "ull) * " << strides[a] << "ull;\n        i /= " << dims[a] << "ull;\n";
        }
    }
    out << "        return offset;\n    }\n";
    return out.str();
}

}  // namespace

int xcdRunLength(int preferred) {
    if (const char* env = std::getenv("THOR_XCD_RUN")) {
        const long v = std::atol(env);
        if (v >= 1 && v <= 1024) return static_cast<int>(v);
    }
    return preferred;
}

uint64_t pointerAlignment(const void* p) {
    const uint64_t address = reinterpret_cast<uint64_t>(p);
    uint64_t alignment = 256;
    while (alignment > 1 && address % alignment != 0) alignment /= 2;
    return alignment;
}

const char* deviceTypeName(DataType dtype) {
    switch (dtype) {
        case DataType::FP16: return "thor::f16";
        case DataType::BF16: return "thor::bf16";
        case DataType::FP8_E4M3: return "thor::e4m3";
        case DataType::FP8_E5M2: return "thor::e5m2";
        case DataType::FP32: return "float";
        case DataType::FP64: return "double";
        case DataType::INT8: return "thor::i8";
        case DataType::INT16: return "thor::i16";
        case DataType::INT32: return "thor::i32";
        case DataType::INT64: return "thor::i64";
        case DataType::UINT8: return "thor::u8";
        case DataType::UINT16: return "thor::u16";
        case DataType::UINT32: return "thor::u32";
        case DataType::UINT64: return "thor::u64";
        case DataType::BOOLEAN: return "thor::boolean";
        default: break;
    }
    throw std::invalid_argument(std::string("No device type for dtype ") + dataTypeName(dtype));
}

std::string ReductionShape::describe() const {
    std::ostringstream out;
    switch (kernel) {
        case Kernel::All:
            out << "all(blocks=" << blocks << ",unroll=" << unroll;
            break;
        case Kernel::Rows:
            out << "rows(lanes_per_row=" << threadsPerRow << ",split=" << split;
            if (unalignedVectors) out << ",unaligned_vectors";
            if (interleave > 1) out << ",outputs_per_row=" << interleave;
            break;
        case Kernel::Columns:
            out << (laneAxis < 0 ? "columns(lanes_x=" : "view_columns(lanes_x=") << threadsPerRow << ",rows_in_flight=" << unroll << ",split=" << split;
            if (unalignedVectors) out << ",unaligned_vectors";
            if (transposeRows > 0) out << ",transposed_store=" << transposeRows;
            break;
        case Kernel::Segments:
            out << "segments(" << (segmentsByRows ? "by_rows," : "by_teams,") << "lanes_x=" << threadsPerRow << ",rows_in_flight=" << unroll << ",chunk_rows=" << chunkRows;
            if (!segmentsByRows) out << ",min_team=" << minTeam;
            break;
        case Kernel::Strided:
            out << "strided(kept_rank=" << keptDims.size() << ",reduced_rank=" << reducedDims.size() << ",split=" << split;
            break;
    }
    out << ",vec=" << vec << ",threads=" << threads << ",grid=" << gridX << "x" << gridY << (tickets ? ",last_share_folds" : "") << ")";
    return out.str();
}

namespace {
ReductionShape planShapeWithoutTickets(const ReductionKernelRequest& request);
}

ReductionShape planReductionShape(const ReductionKernelRequest& request) {
    ReductionShape shape = planShapeWithoutTickets(request);
    // Finishing inside the main launch: whole-tensor reductions over several blocks, and split reductions whose shares of one
    // output group are whole blocks.  THOR_REDUCE_TICKETS=0 keeps the finishing launch (tuning switch).
    // Measured on MI355X, finishing launch against last share: per-channel sums of an NCHW tensor (strided, 256 x 16 blocks) 21.0 /
    // 21.2 us, 16 rows of 2^22 (rows, 16 x 8 blocks) 49.5 / 48.9 us: as fast with one launch fewer, so these two kinds take
    // tickets.  Whole-tensor sums (1024 arrivals on one word: 42 / 47 us) and column sums (47.5 / 53.9 us with the shares of one
    // output apart and adjacent lanes on adjacent words, 84 us before that; with 48 shares instead of 64 the two are equal) keep
    // the finishing launch unless THOR_REDUCE_TICKETS=2 forces tickets everywhere.
    const char* env = std::getenv("THOR_REDUCE_TICKETS");
    const bool wanted = env == nullptr || std::atoi(env) != 0;
    const bool forced = env != nullptr && std::atoi(env) == 2;
    uint64_t count = 0;
    switch (shape.kernel) {
        case ReductionShape::Kernel::All: count = forced && shape.blocks > 1 ? 1 : 0; break;
        case ReductionShape::Kernel::Rows: count = shape.split > 1 && shape.threadsPerRow > 64 ? request.geometry.outer_size : 0; break;
        case ReductionShape::Kernel::Columns: count = forced && shape.split > 1 ? shape.gridX : 0; break;
        case ReductionShape::Kernel::Strided: count = shape.split > 1 ? request.geometry.output_elements : 0; break;
        case ReductionShape::Kernel::Segments: break;
    }
    if (wanted && count > 0 && shape.workspaceBytes > 0) {
        shape.tickets = true;
        shape.ticketCount = count;
        shape.ticketOffset = (shape.workspaceBytes + 255) / 256 * 256;
        shape.workspaceBytes = shape.ticketOffset + count * 4;
    }
    return shape;
}

namespace {
ReductionShape planShapeWithoutTickets(const ReductionKernelRequest& request) {
    const CubReductionGeometry& g = request.geometry;
    uint32_t elementBytes = dataTypeSizeInBytes(request.inputDType);
    if (!request.values.empty()) {
        elementBytes = 1;
        for (const ReductionKernelRequest::Source& source : request.sources)
            if (source.kind == ReductionKernelRequest::Source::Kind::Vector) elementBytes = std::max(elementBytes, dataTypeSizeInBytes(source.storage));
        for (const ReductionKernelRequest::Elementwise& e : request.elementwise) elementBytes = std::max(elementBytes, dataTypeSizeInBytes(e.outputDType));
    }
    const uint64_t accumulators = request.values.empty() ? 1 : request.values.size();
    ReductionShape shape;
    shape.indexIs64 = g.input_elements >= (1ull << 31) || g.reduction_size >= (1ull << 31);
    const uint64_t accumulatorBytes = request.isArg ? (shape.indexIs64 ? 16 : 8) : 4 * accumulators;

    auto finishSplit = [&](uint64_t outputs) {
        if (shape.split > 1) shape.workspaceBytes = accumulators * partialBytes(outputs * shape.split, request.isArg, shape.indexIs64);
    };

    if (request.segmented) {
        shape.kernel = ReductionShape::Kernel::Segments;
        // candidates carry the row of the element (32 bits while rows fit: half the registers, shuffles and partial bytes); the
        // store packs row * trailing + element into the output's index type and keeps the all-ones mark of an empty segment
        shape.indexIs64 = request.segmentedRows >= 0xffffffffull;
        shape.vec = chooseVector(elementBytes, request.inputAlignmentBytes, {request.trailing});
        shape.threads = 256;
        shape.unroll = 8;
        if (const char* env = std::getenv("THOR_SEGMENT_BATCH")) {  // tuning switch: rows in flight per lane
            const long requested = std::atol(env);
            if (requested == 1 || requested == 2 || requested == 4 || requested == 8 || requested == 16) shape.unroll = static_cast<int>(requested);
        }
        const uint64_t columnsPerRow = request.trailing / shape.vec;
        shape.threadsPerRow = static_cast<int>(std::min<uint64_t>(64, pow2Ceil(columnsPerRow)));
        const uint64_t lanesX = static_cast<uint64_t>(shape.threadsPerRow);
        const uint64_t tiles = ceilDiv(columnsPerRow, lanesX);
        // A block streams a chunk of rows whatever the partition is.  Chunks are about as long as an average segment, so
        // that the teams of one block get pieces of similar length, between one pass of the block and about 128 KiB;
        // shorter while that leaves fewer than eight blocks per CU.
        const uint64_t averageRows = std::max<uint64_t>(request.segmentedRows / std::max<uint64_t>(request.segments, 1), 1);
        const uint64_t rowsPerPass = (256 / lanesX) * shape.unroll;
        const uint64_t passBytes = rowsPerPass * lanesX * shape.vec * elementBytes;
        uint64_t passesPerChunk = std::min<uint64_t>(std::max<uint64_t>(131072 / passBytes, 1), std::max<uint64_t>(pow2Ceil(averageRows / rowsPerPass + 1) / 2, 1));
        while (passesPerChunk > 1 && ceilDiv(request.segmentedRows, rowsPerPass * passesPerChunk) * tiles < 2048) passesPerChunk /= 2;
        shape.chunkRows = rowsPerPass * passesPerChunk;
        shape.chunks = std::max<uint64_t>(ceilDiv(request.segmentedRows, shape.chunkRows), 1);
        // the smallest team that shares one segment: eight rows in flight per lane should cover an average segment
        const uint64_t rowLanes = std::min<uint64_t>(std::max<uint64_t>(pow2Ceil(averageRows) / shape.unroll, 1), 8);
        // ... and a team no wider than a wavefront folds with shuffles alone (no LDS round, no barriers): log-normal segments
        // of 64 rows x 64 fp32 on average, teams of 128 -> 64 threads: sum 209 -> 193 us, arg-max 340 -> 282 us
        shape.minTeam = static_cast<int>(std::min<uint64_t>(lanesX * rowLanes, std::max<uint64_t>(lanesX, 64)));
        if (const char* env = std::getenv("THOR_SEGMENT_MIN_TEAM")) {  // tuning switch: threads of the smallest team
            const uint64_t requested = static_cast<uint64_t>(std::atol(env));
            if (requested >= lanesX && requested <= 256 && (requested & (requested - 1)) == 0) shape.minTeam = static_cast<int>(requested);
        }
        // Work dealt out by rows (every lane owns `unroll` consecutive rows and loads them before it looks at the offsets)
        // when a row lane reads whole cache lines and segments are long enough that most ranges hold one or two of them:
        // log-normal segments of 64 rows x 64 fp32 on average: see the measurements beside the kernel's bench lines.
        const bool wholeLines = lanesX * shape.vec * elementBytes >= 128;
        uint64_t vectorSources = 0;
        for (const ReductionKernelRequest::Source& source : request.sources) vectorSources += source.kind == ReductionKernelRequest::Source::Kind::Vector;
        vectorSources = std::max<uint64_t>(vectorSources, 1);
        shape.segmentsByRows = wholeLines && averageRows >= 8;
        if (const char* env = std::getenv("THOR_SEGMENT_KERNEL")) {  // tuning / test switch: "teams" or "rows"
            if (std::string(env) == "teams") shape.segmentsByRows = false;
            if (std::string(env) == "rows") shape.segmentsByRows = true;
        }
        if (shape.segmentsByRows) {
            if (std::getenv("THOR_SEGMENT_BATCH") == nullptr) shape.unroll = averageRows >= 32 ? 16 : 8;
            // at most 64 registers of rows, and 64 elements per lane in the unrolled walk (fp8 vectors of 16 x 16 rows compile for minutes)
            while (shape.unroll > 1 && (static_cast<uint64_t>(shape.unroll) * shape.vec * elementBytes * vectorSources > 256 ||
                                        static_cast<uint64_t>(shape.unroll) * shape.vec > 64))
                shape.unroll /= 2;
            // Smaller blocks when the accumulation is longer: the wavefronts of a block meet at two barriers and their walks
            // differ with the partition.  Log-normal segments of 64 rows x 64 fp32 on average, 256 / 128 / 64 threads:
            // arg-max 227 / 208 / 250 us, the pair of a one-pass softmax 290 / 265 / 255 us, sums 190 / 195 / 202 us.
            if (request.onlineSoftmax) shape.threads = 64;
            else if (request.isArg) shape.threads = 128;
            shape.threads = std::max<int>(shape.threads, static_cast<int>(lanesX));
            if (const char* env = std::getenv("THOR_SEGMENT_THREADS")) {  // tuning switch: threads per block
                const uint64_t requested = static_cast<uint64_t>(std::atol(env));
                if ((requested == 64 || requested == 128 || requested == 256) && requested >= lanesX) shape.threads = static_cast<int>(requested);
            }
            shape.chunkRows = (static_cast<uint64_t>(shape.threads) / lanesX) * static_cast<uint64_t>(shape.unroll);
            shape.chunks = std::max<uint64_t>(ceilDiv(request.segmentedRows, shape.chunkRows), 1);
            if (const char* env = std::getenv("THOR_SEGMENT_GROUP")) {  // tuning switch: rows walked together
                const long requested = std::atol(env);
                if (requested == 1 || requested == 2 || requested == 4 || requested == 8 || requested == 16) shape.walkGroup = static_cast<int>(requested);
            }
        }
        shape.finishLanes = static_cast<int>(std::min<uint64_t>(64, pow2Ceil(request.trailing)));
        // a segment of average length runs over averageRows / chunkRows chunks, folded by finishThreads / finishLanes row
        // lanes: one wavefront while that leaves each lane a handful of partials, else a block
        shape.finishThreads = (averageRows / shape.chunkRows) * shape.finishLanes > 8 * 64 ? 256 : 64;
        shape.blocks = tiles;
        shape.gridX = static_cast<uint32_t>(shape.chunks * tiles);
        shape.gridY = 1;
        if (shape.chunks > 1) {
            shape.workspaceBytes = accumulators * partialBytes(shape.chunks * 2 * request.trailing, request.isArg, shape.indexIs64) + shape.chunks * 16;
        }
        return shape;
    }

    if (g.path == CubReductionPath::DeviceTransformReduce && !g.device_transform_uses_affine_stride) {
        shape.kernel = ReductionShape::Kernel::All;
        shape.vec = chooseVector(elementBytes, request.inputAlignmentBytes, {g.input_elements});
        shape.threads = 256;
        shape.unroll = 4;
        const uint64_t vectors = g.input_elements / shape.vec;
        // four resident blocks per CU that stride over the tensor: measured 6.4 TB/s at 2^26 fp32 elements against
        // 5.9 TB/s with one chunk per block (16 384 blocks), and the finishing launch folds 1024 partials instead of 16 384
        shape.blocks = std::min<uint64_t>(std::max<uint64_t>(ceilDiv(vectors, 256ull * shape.unroll), 1), 1024);
        shape.gridX = static_cast<uint32_t>(shape.blocks);
        if (shape.blocks > 1) shape.workspaceBytes = accumulators * partialBytes(shape.blocks, request.isArg, shape.indexIs64);
        return shape;
    }

    if (g.path == CubReductionPath::ContiguousFixedSegment) {
        shape.kernel = ReductionShape::Kernel::Rows;
        shape.vec = chooseVector(elementBytes, request.inputAlignmentBytes, {g.reduction_size});
        // A row length (or a pointer) that no vector fits: the lanes still read 16-byte vectors, at addresses that are only
        // aligned to the element, and the last row_length % vec elements of a row one by one.
        const int wide = static_cast<int>(16 / elementBytes);
        if (shape.vec < wide && request.elementwise.empty() && g.reduction_size >= 4ull * wide && request.inputAlignmentBytes % elementBytes == 0) {
            shape.vec = wide;
            shape.unalignedVectors = true;
        }
        const uint64_t vectorsPerRow = std::max<uint64_t>(g.reduction_size / shape.vec, 1);
        // aim at about 8 vector loads in flight per lane
        uint64_t lanes = std::min<uint64_t>(std::max<uint64_t>(pow2Ceil(ceilDiv(vectorsPerRow, 8)), 1), 1024);
        // ... but never fewer than 8 lanes on a row that has the vectors for them: the lanes of a row read adjacent vectors, and
        // fewer than 8 of them touch part of a cache line per load (rows of 56 fp16, one lane per row: 52 us for 98 MiB; 8 lanes: 19 us)
        lanes = std::max<uint64_t>(lanes, std::min<uint64_t>(8, pow2Ceil(vectorsPerRow)));
        shape.threadsPerRow = static_cast<int>(lanes);
        shape.threads = lanes <= 64 ? 256 : static_cast<int>(lanes);
        const uint64_t totalThreads = g.outer_size * lanes;
        if (totalThreads < kTargetThreads && vectorsPerRow > lanes * 16) {
            shape.split = std::min<uint64_t>({ceilDiv(kTargetThreads, totalThreads), vectorsPerRow / (lanes * 8), kMaxGridY});
            if (shape.split < 2) shape.split = 1;
        }
        const uint64_t rowsPerBlock = lanes <= 64 ? 256 / lanes : 1;
        shape.gridX = static_cast<uint32_t>(ceilDiv(g.outer_size, rowsPerBlock));
        shape.gridY = static_cast<uint32_t>(shape.split);
        finishSplit(g.outer_size);
        return shape;
    }

    if (g.path == CubReductionPath::TiledFixedSegment) {
        // [outer, R, inner] with an inner extent of a few elements (a 16-byte vector holds a whole number of inner rows): lanes
        // across the outputs would each walk a stream of their own, 16 bytes at a time.  The rows kernel reads the
        // contiguous row of R * inner elements instead and keeps one accumulator per inner element
        // ([4096, 4096, 4] fp32 over the middle axis: 178 us with lanes across outputs).
        {
            const uint64_t innerBytes = g.inner_size * elementBytes;
            bool keptSources = false;
            for (const ReductionKernelRequest::Source& source : request.sources) keptSources = keptSources || source.kind != ReductionKernelRequest::Source::Kind::Vector;
            const int vec = static_cast<int>(16 / elementBytes);
            const uint64_t rowElements = g.reduction_size * g.inner_size;
            const bool denseOutput = g.tiled_output_inner_stride == 1 && g.tiled_output_outer_stride == g.inner_size;
            if (g.inner_size > 1 && innerBytes <= 16 && 16 % innerBytes == 0 && !keptSources && request.elementwise.empty() && denseOutput &&
                rowElements % vec == 0 && request.inputAlignmentBytes % 16 == 0 && std::getenv("THOR_REDUCE_NO_INTERLEAVE") == nullptr) {
                const uint64_t vectorsPerRow = rowElements / vec;
                uint64_t lanes = std::min<uint64_t>(std::max<uint64_t>(pow2Ceil(ceilDiv(vectorsPerRow, 8)), 1), 1024);
                lanes = std::max<uint64_t>(lanes, std::min<uint64_t>(8, pow2Ceil(vectorsPerRow)));
                if (g.outer_size * lanes >= kTargetThreads || vectorsPerRow <= lanes * 16) {  // enough rows that none has to be split
                    shape.kernel = ReductionShape::Kernel::Rows;
                    shape.vec = vec;
                    shape.interleave = static_cast<int>(g.inner_size);
                    shape.threadsPerRow = static_cast<int>(lanes);
                    shape.threads = lanes <= 64 ? 256 : static_cast<int>(lanes);
                    const uint64_t rowsPerBlock = lanes <= 64 ? 256 / lanes : 1;
                    shape.gridX = static_cast<uint32_t>(ceilDiv(g.outer_size, rowsPerBlock));
                    shape.gridY = 1;
                    return shape;
                }
            }
        }
        shape.kernel = ReductionShape::Kernel::Columns;
        shape.vec = chooseVector(elementBytes, request.inputAlignmentBytes, {g.inner_size});
        // An inner extent (or a pointer) that no vector fits: the lanes still own 16-byte vectors of outputs and read them at
        // addresses that are only aligned to the element; the last vector of the inner extent is moved back to end with it, and
        // the outputs it shares with the vector before it are stored by that one.
        const int wideColumns = static_cast<int>(16 / elementBytes);
        if (shape.vec < wideColumns && request.elementwise.empty() && g.inner_size >= 2ull * wideColumns && g.tiled_output_outer_stride != 1 &&
            request.inputAlignmentBytes % elementBytes == 0 && std::getenv("THOR_COLUMNS_NO_UNALIGNED") == nullptr) {
            shape.vec = wideColumns;
            shape.unalignedVectors = true;
        }
        const uint64_t innerColumns = ceilDiv(g.inner_size, shape.vec);
        shape.threads = 256;
        shape.unroll = 8;  // rows in flight per thread
        if (const char* env = std::getenv("THOR_COLUMNS_BATCH")) shape.unroll = std::min<long>(std::max<long>(std::atol(env), 1), 16);  // tuning switch
        const uint64_t columns = g.outer_size * innerColumns;
        // a block is up to one wavefront of columns wide; the rest of its threads are row groups folded through LDS
        shape.threadsPerRow = static_cast<int>(std::min<uint64_t>(64, pow2Ceil(columns)));
        if (g.tiled_output_outer_stride != 1 && std::getenv("THOR_COLUMNS_POW2_LANES") == nullptr) {
            // as many blocks across the columns as 64-lane blocks would take, each as wide as its share of the columns: 20
            // columns are 20 lanes and 12 row groups (not 32 lanes of which 12 idle), 77 columns two blocks of 39 (not 64 + 13)
            shape.threadsPerRow = static_cast<int>(ceilDiv(columns, ceilDiv(columns, 64)));
        }
        if (const char* env = std::getenv("THOR_COLUMNS_LANES")) {  // tuning switch: lanes across the columns of a block
            const long requested = std::atol(env);
            if ((requested == 64 || requested == 128 || requested == 256) && static_cast<uint64_t>(requested) <= pow2Ceil(columns)) shape.threadsPerRow = static_cast<int>(requested);
        }
        const uint64_t groups = 256 / shape.threadsPerRow;
        // enough threads to keep loads in flight on every CU, but at least 16 rows per thread and partials that stay small
        // next to the input (measured on 8192 x 8192 fp32: 512 Ki threads reach 5.3 TB/s, 128 Ki threads 3.8 TB/s)
        const uint64_t wantedThreads = 4 * kTargetThreads;
        if (columns * groups < wantedThreads && g.reduction_size >= groups * 32) {
            shape.split = std::min<uint64_t>({ceilDiv(wantedThreads, columns * groups), g.reduction_size / (groups * 16), kMaxGridY});
            if (shape.split < 2) shape.split = 1;
        }
        if (const char* env = std::getenv("THOR_COLUMNS_SPLIT")) {  // tuning switch
            shape.split = std::min<uint64_t>({static_cast<uint64_t>(std::max<long>(std::atol(env), 1)), std::max<uint64_t>(g.reduction_size / groups, 1), kMaxGridY});
        }
        shape.gridX = static_cast<uint32_t>(ceilDiv(columns, shape.threadsPerRow));
        shape.gridY = static_cast<uint32_t>(shape.split);
        if (g.tiled_output_outer_stride == 1) {
            // [inner, outer] output: consecutive outer coordinates are adjacent in the output
            shape.transposeRows = transposeRowsFor(shape.split, g.reduction_size, g.outer_size, g.tiled_output_inner_stride,
                                                    (static_cast<uint64_t>(shape.threadsPerRow) * shape.vec + 1) * accumulatorBytes);
            if (shape.transposeRows > 0) {
                shape.gridX = static_cast<uint32_t>(ceilDiv(innerColumns, shape.threadsPerRow) * ceilDiv(g.outer_size, shape.transposeRows));
            }
        }
        finishSplit(g.output_elements);
        return shape;
    }

    // Strided: arbitrary kept / reduced axes, including views and the affine rank-1 whole-tensor case.
    shape.kernel = ReductionShape::Kernel::Strided;
    shape.threads = 256;
    if (const char* env = std::getenv("THOR_STRIDED_THREADS")) {  // tuning switch: threads per block
        const long requested = std::atol(env);
        if (requested == 256 || requested == 512 || requested == 1024) shape.threads = static_cast<int>(requested);
    }
    for (size_t a = 0; a < g.indexing.retained_axes.size(); ++a) {
        shape.keptDims.push_back(g.indexing.retained_dimensions[a]);
        shape.keptStrides.push_back(g.indexing.input_strides[g.indexing.retained_axes[a]]);
    }
    for (size_t a = 0; a < g.indexing.reduced_axes.size(); ++a) {
        shape.reducedDims.push_back(g.indexing.reduced_dimensions[a]);
        shape.reducedStrides.push_back(g.indexing.input_strides[g.indexing.reduced_axes[a]]);
    }
    collapseAxes(shape.keptDims, shape.keptStrides);
    collapseAxes(shape.reducedDims, shape.reducedStrides);
    if (shape.keptDims.empty()) {
        shape.keptDims = {1};
        shape.keptStrides = {0};
    }
    if (shape.reducedDims.empty()) {
        shape.reducedDims = {1};
        shape.reducedStrides = {0};
    }
    // A view whose contiguous axis is a kept one (a transposed matrix reduced along its rows): lanes go across that axis,
    // every lane owns outputs, and memory is still read in contiguous runs.  Lanes across the reduction domain, below,
    // would read one element per cache line.
    int laneAxis = -1;
    bool reducedContiguous = false;
    for (size_t a = 0; a < shape.reducedDims.size(); ++a) reducedContiguous = reducedContiguous || (shape.reducedStrides[a] == 1 && shape.reducedDims[a] > 1);
    if (!reducedContiguous) {
        for (size_t a = 0; a < shape.keptDims.size(); ++a)
            if (shape.keptStrides[a] == 1 && shape.keptDims[a] >= 16) laneAxis = static_cast<int>(a);
    }
    if (laneAxis >= 0) {
        shape.kernel = ReductionShape::Kernel::Columns;
        shape.laneAxis = laneAxis;
        int vec = static_cast<int>(16 / elementBytes);
        while (vec > 1) {
            bool ok = request.inputAlignmentBytes % (static_cast<uint64_t>(vec) * elementBytes) == 0 && shape.keptDims[laneAxis] % vec == 0;
            for (size_t a = 0; a < shape.keptStrides.size(); ++a) ok = ok && (static_cast<int>(a) == laneAxis || shape.keptStrides[a] % vec == 0);
            for (uint64_t st : shape.reducedStrides) ok = ok && st % vec == 0;
            if (ok) break;
            vec /= 2;
        }
        shape.vec = vec;
        shape.unroll = 8;
        const uint64_t columns = g.output_elements / vec;
        shape.threadsPerRow = static_cast<int>(std::min<uint64_t>(64, pow2Ceil(columns)));
        const uint64_t groups = 256 / shape.threadsPerRow;
        const uint64_t wantedThreads = 4 * kTargetThreads;
        if (columns * groups < wantedThreads && g.reduction_size >= groups * 32) {
            shape.split = std::min<uint64_t>({ceilDiv(wantedThreads, columns * groups), g.reduction_size / (groups * 16), kMaxGridY});
            if (shape.split < 2) shape.split = 1;
        }
        shape.gridX = static_cast<uint32_t>(ceilDiv(columns, shape.threadsPerRow));
        shape.gridY = static_cast<uint32_t>(shape.split);
        if (static_cast<size_t>(laneAxis) + 1 != shape.keptDims.size()) {
            // the columns after the lane axis run along the last kept axis, the output's fastest one
            uint64_t laneOutputStride = 1;
            for (size_t a = static_cast<size_t>(laneAxis) + 1; a < shape.keptDims.size(); ++a) laneOutputStride *= shape.keptDims[a];
            shape.transposeRows = transposeRowsFor(shape.split, g.reduction_size, shape.keptDims.back(), laneOutputStride,
                                                    (static_cast<uint64_t>(shape.threadsPerRow) * vec + 1) * accumulatorBytes);
            if (shape.transposeRows > 0) {
                const uint64_t laneVectors = shape.keptDims[laneAxis] / vec;
                shape.gridX = static_cast<uint32_t>(ceilDiv(laneVectors, shape.threadsPerRow) * ceilDiv(columns / laneVectors, shape.transposeRows));
            }
        }
        finishSplit(g.output_elements);
        return shape;
    }
    shape.vec = 1;
    if (shape.reducedStrides.back() == 1) {
        int vec = static_cast<int>(16 / elementBytes);
        while (vec > 1) {
            bool ok = request.inputAlignmentBytes % (static_cast<uint64_t>(vec) * elementBytes) == 0 && shape.reducedDims.back() % vec == 0;
            for (size_t a = 0; a + 1 < shape.reducedStrides.size(); ++a) ok = ok && shape.reducedStrides[a] % vec == 0;
            for (uint64_t s : shape.keptStrides) ok = ok && s % vec == 0;
            if (ok) break;
            vec /= 2;
        }
        shape.vec = vec;
    }
    const uint64_t reductionVectors = g.reduction_size / shape.vec;
    const uint64_t outputs = g.output_elements;
    // About one output per compute unit or more, each over a long reduction: one 1024-thread block per output reads it whole.
    // Nothing is split, so no share waits to fold the others (per-channel sums of [64, 256, 56, 56] fp16, 98 MiB: 20.5 us as
    // 16 shares of 256 threads per channel with the last share folding, 18.1 us this way).
    // (Not with an elementwise output: twice the bytes per launch make the fold a smaller share, 38.3 against 39.5 us.)
    const bool wholeOutputs = outputs >= 192 && outputs < 2048 && reductionVectors >= 1024ull * 16 && request.elementwise.empty() && std::getenv("THOR_STRIDED_BLOCKS") == nullptr &&
                              std::getenv("THOR_STRIDED_THREADS") == nullptr;
    if (wholeOutputs) {
        shape.threads = 1024;
    } else if (outputs < 2048 && reductionVectors > 256ull * 8) {
        uint64_t wantedBlocks = 4096;
        if (const char* env = std::getenv("THOR_STRIDED_BLOCKS")) wantedBlocks = std::max<long>(std::atol(env), 1);  // tuning switch
        shape.split = std::min<uint64_t>({ceilDiv(wantedBlocks, outputs), reductionVectors / (256ull * 4), kMaxGridY});
        if (shape.split < 2) shape.split = 1;
    }
    shape.unroll = 4;
    if (const char* env = std::getenv("THOR_STRIDED_BATCH")) shape.unroll = std::min<long>(std::max<long>(std::atol(env), 1), 16);  // tuning switch
    shape.gridX = static_cast<uint32_t>(outputs);
    shape.gridY = static_cast<uint32_t>(shape.split);
    finishSplit(outputs);
    return shape;
}
}  // namespace

std::string generateReductionSource(const ReductionKernelRequest& request, const ReductionShape& shape) {
    const CubReductionGeometry& g = request.geometry;
    // the plain request is the fused form with one source and the value itself
    std::vector<ReductionKernelRequest::Source> sources = request.sources;
    std::vector<ReductionKernelRequest::Value> values = request.values;
    std::string prologue = request.prologue;
    if (values.empty()) {
        sources = {{request.inputDType, ReductionKernelRequest::Source::Kind::Vector, std::string()}};
        values = {{request.valueOp, request.valueOutputDType, "x0"}};
        prologue = "        const float x0 = toFloat(l.p0.v[k]);\n";
    } else if (request.isArg) {
        throw std::invalid_argument("Arg reductions cannot be fused with other reductions.");
    }
    const char* indexType = shape.indexIs64 ? "u64" : "u32";

    std::ostringstream s;
    s << thor_embed::kDevicePrelude << thor_embed::kReduceKernels;
    s << "namespace gen {\nusing namespace thor;\nstruct Cfg {\n";
    s << "    typedef " << indexType << " IndexT;\n";
    s << "    static constexpr int kVec = " << shape.vec << ";\n";
    s << "    static constexpr int kThreads = " << shape.threads << ";\n";
    s << "    static constexpr bool kTickets = " << (shape.tickets ? "true" : "false") << ";\n";
    s << "    static constexpr u64 kTicketOffset = " << shape.ticketOffset << "ull;\n";
    // one block per row of 8192 fp32: runs of 4 rows (128 KiB) per XCD measured +1.5 % (6.57 -> 6.67 TB/s), runs of 2 -3 %; rows
    // that share a block and whole-tensor sums gain nothing from any run length
    s << "    static constexpr int kXcdRun = " << xcdRunLength(shape.kernel == ReductionShape::Kernel::Rows && shape.threadsPerRow > 64 ? 4 : 1) << ";\n";
    s << "    static constexpr u64 kSplit = " << shape.split << "ull;\n";
    s << "    static constexpr u64 kOutputs = " << g.output_elements << "ull;\n";
    s << "    static constexpr float kDivisor = (float)" << g.reduction_size << "ull;\n";

    // what the prologue reads
    typedef ReductionKernelRequest::Source::Kind SourceKind;
    s << "    struct Sources {\n";
    for (size_t i = 0; i < sources.size(); ++i) s << "        const " << deviceTypeName(sources[i].storage) << "* in" << i << ";\n";
    for (uint32_t slot : request.scalarSlots) s << "        float s" << slot << ";\n";
    s << "    };\n    struct Loaded {\n";
    for (size_t i = 0; i < sources.size(); ++i)
        if (sources[i].kind == SourceKind::Vector) s << "        Pack<" << deviceTypeName(sources[i].storage) << ", kVec> p" << i << ";\n";
    s << "    };\n";
    s << "    static __device__ __forceinline__ void load(const Sources& s, u64 offset, Loaded& l) {\n";
    for (size_t i = 0; i < sources.size(); ++i)
        if (sources[i].kind == SourceKind::Vector)
            s << "        l.p" << i << (shape.unalignedVectors ? ".loadStreamUnaligned(s.in" : ".loadStream(s.in") << i << " + offset);\n";
    s << "        (void)s; (void)offset; (void)l;\n    }\n";
    s << "    static __device__ __forceinline__ void loadFirstOnly(const Sources& s, u64 offset, Loaded& l) {\n";  // element 0 of every vector source
    for (size_t i = 0; i < sources.size(); ++i)
        if (sources[i].kind == SourceKind::Vector) s << "        l.p" << i << ".v[0] = s.in" << i << "[offset];\n";
    s << "        (void)s; (void)offset; (void)l;\n    }\n";
    // values that depend only on the output
    s << "    struct Kept {\n";
    for (size_t i = 0; i < sources.size(); ++i)
        if (sources[i].kind != SourceKind::Vector) s << "        " << deviceTypeName(sources[i].storage) << " z" << i << ";\n";
    s << "    };\n";
    s << "    static __device__ __forceinline__ void loadKept(const Sources& s, u64 slot, Kept& kk) {\n";
    for (size_t i = 0; i < sources.size(); ++i) {
        if (sources[i].kind == SourceKind::Scalar) s << "        kk.z" << i << " = s.in" << i << "[0];\n";
        if (sources[i].kind == SourceKind::Kept) {
            s << "        kk.z" << i << " = s.in" << i << "[" << (sources[i].keptOffset.empty() ? std::string("slot") : sources[i].keptOffset) << "];\n";
        }
    }
    s << "        (void)s; (void)slot; (void)kk;\n    }\n";

    // accumulators
    std::vector<int> finalize(values.size(), 0);
    if (request.isArg) {
        int f = 0;
        s << "    typedef " << accumulatorType(request, shape.indexIs64, f) << " Acc;\n";
    } else if (request.onlineSoftmax) {
        if (values.size() != 2) throw std::invalid_argument("The one-pass softmax statistics are two values: the maximum and the sum of exponentials.");
        s << "    typedef OnlineSoftmaxAcc Acc;\n";
    } else if (values.size() == 1) {
        s << "    typedef " << valueAccumulatorType(values[0].op, finalize[0]) << " Acc;\n";
    } else {
        s << "    struct Acc {\n";
        for (size_t j = 0; j < values.size(); ++j) s << "        " << valueAccumulatorType(values[j].op, finalize[j]) << " a" << j << ";\n";
        s << "        __device__ __forceinline__ void reset() {";
        for (size_t j = 0; j < values.size(); ++j) s << " a" << j << ".reset();";
        s << " }\n        __device__ __forceinline__ void merge(const Acc& o) {";
        for (size_t j = 0; j < values.size(); ++j) s << " a" << j << ".merge(o.a" << j << ");";
        s << " }\n        __device__ __forceinline__ Acc shuffleXor(int mask) const {\n            Acc r;\n";
        for (size_t j = 0; j < values.size(); ++j) s << "            r.a" << j << " = a" << j << ".shuffleXor(mask);\n";
        s << "            return r;\n        }\n";
        // partials: one float array per member, back to back
        s << "        template <bool DEVICE_WIDE = false>\n        __device__ __forceinline__ void storePartial(void* partials, u64 slot, u64 slots) const {\n"
             "            char* base = static_cast<char*>(partials);\n            const u64 stride = ((slots * 4 + 7) / 8) * 8;\n";
        for (size_t j = 0; j < values.size(); ++j) s << "            a" << j << ".template storePartial<DEVICE_WIDE>(base + " << j << " * stride, slot, slots);\n";
        s << "        }\n        template <bool DEVICE_WIDE = false>\n        __device__ __forceinline__ void loadPartial(const void* partials, u64 slot, u64 slots) {\n"
             "            const char* base = static_cast<const char*>(partials);\n            const u64 stride = ((slots * 4 + 7) / 8) * 8;\n";
        for (size_t j = 0; j < values.size(); ++j) s << "            a" << j << ".template loadPartial<DEVICE_WIDE>(base + " << j << " * stride, slot, slots);\n";
        s << "        }\n    };\n";
    }
    s << "    static constexpr bool kOnlineSoftmax = " << (request.onlineSoftmax ? "true" : "false") << ";\n";
    s << "    static __device__ __forceinline__ float valueOne(const Loaded& l, const Sources& s, const Kept& kk, int k) {\n" << prologue;
    s << "        (void)l; (void)s; (void)kk; (void)k;\n        return " << values[0].expression << ";\n    }\n";
    s << "    static __device__ __forceinline__ void accumulateOne(Acc& acc, const Loaded& l, const Sources& s, const Kept& kk, int k, IndexT index) {\n";
    s << prologue;
    if (request.isArg || values.size() == 1 || request.onlineSoftmax) {
        s << "        acc.add(" << values[0].expression << ", index);\n";
    } else {
        for (size_t j = 0; j < values.size(); ++j) s << "        acc.a" << j << ".add(" << values[j].expression << ", index);\n";
    }
    s << "        (void)l; (void)s; (void)kk; (void)k; (void)index;\n    }\n";

    // results
    s << "    struct Outputs {\n";
    for (size_t j = 0; j < values.size(); ++j) s << "        " << deviceTypeName(values[j].outputDType) << "* out" << j << ";\n";
    for (size_t j = 0; j < request.elementwise.size(); ++j) s << "        " << deviceTypeName(request.elementwise[j].outputDType) << "* e" << j << ";\n";
    s << "        " << (request.indexOutputDType == DataType::UINT64 ? "u64" : "u32") << "* indexOut;\n    };\n";
    // same-shaped outputs written by the pass that reads the sources
    s << "    template <int KS>\n    static __device__ __forceinline__ void elementwise(const Sources& s, const Outputs& o, u64 offset, const Loaded& l, "
         "const Kept* kept) {\n";
    if (!request.elementwise.empty()) {
        for (size_t j = 0; j < request.elementwise.size(); ++j)
            s << "        Pack<" << deviceTypeName(request.elementwise[j].outputDType) << ", kVec> q" << j << ";\n";
        s << "#pragma unroll\n        for (int k = 0; k < kVec; ++k) {\n        const Kept& kk = kept[k * KS];\n" << prologue;
        for (size_t j = 0; j < request.elementwise.size(); ++j) s << "        q" << j << ".v[k] = " << request.elementwise[j].expression << ";\n";
        s << "        }\n";
        for (size_t j = 0; j < request.elementwise.size(); ++j) s << "        q" << j << ".storeStream(o.e" << j << " + offset);\n";
    }
    s << "        (void)s; (void)o; (void)offset; (void)l; (void)kept;\n    }\n";
    s << "    static __device__ __forceinline__ void store(const Acc& acc, u64 outIndex, const Outputs& o, float scale, float divisor = kDivisor) {\n";
    if (request.isArg) {
        if (request.writeValue) s << "        o.out0[outIndex] = fromFloat<" << deviceTypeName(values[0].outputDType) << ">(acc.v);\n";
        if (request.writeIndex) {
            const char* stored = request.indexOutputDType == DataType::UINT64 ? "u64" : "u32";
            if (request.segmented) {
                // the candidate holds a row; the packed position adds the trailing element this output belongs to
                s << "        o.indexOut[outIndex] = acc.i == ~(IndexT)0 ? ~(" << stored << ")0 : (" << stored << ")((u64)acc.i * " << request.trailing
                  << "ull + outIndex % " << request.trailing << "ull);\n";
            } else {
                s << "        o.indexOut[outIndex] = acc.i == ~(IndexT)0 ? ~(" << stored << ")0 : (" << stored << ")acc.i;\n";
            }
        }
        s << "        (void)scale;\n";
    } else if (request.onlineSoftmax) {
        s << "        o.out0[outIndex] = fromFloat<" << deviceTypeName(values[0].outputDType) << ">(acc.m);\n";
        s << "        o.out1[outIndex] = fromFloat<" << deviceTypeName(values[1].outputDType) << ">(acc.s);\n";
        s << "        (void)scale;\n";
    } else {
        for (size_t j = 0; j < values.size(); ++j) {
            const std::string member = values.size() == 1 ? "acc.v" : "acc.a" + std::to_string(j) + ".v";
            s << "        o.out" << j << "[outIndex] = fromFloat<" << deviceTypeName(values[j].outputDType) << ">(finalizeValue<" << finalize[j] << ">("
              << member << ", divisor, scale));\n";
        }
    }
    s << "        (void)acc; (void)outIndex; (void)o; (void)divisor;\n    }\n";

    const char* body = "";
    switch (shape.kernel) {
        case ReductionShape::Kernel::All:
            s << "    static constexpr u64 kN = " << g.input_elements << "ull;\n";
            s << "    static constexpr int kUnroll = " << shape.unroll << ";\n";
            s << "    static constexpr u64 kBlocks = " << shape.blocks << "ull;\n";
            s << "    static constexpr int kFinishThreads = 1024;\n";
            body = "thor::reduceAll<gen::Cfg>(src, out, partials, scale);";
            break;
        case ReductionShape::Kernel::Rows:
            s << "    static constexpr u64 kOuter = " << g.outer_size << "ull;\n";
            s << "    static constexpr u64 kR = " << g.reduction_size * static_cast<uint64_t>(shape.interleave) << "ull;\n";  // elements of a row
            s << "    static constexpr int kInterleave = " << shape.interleave << ";\n";
            s << "    static constexpr int kThreadsPerRow = " << shape.threadsPerRow << ";\n";
            body = "thor::reduceRows<gen::Cfg>(src, out, partials, scale);";
            break;
        case ReductionShape::Kernel::Columns:
            s << "    static constexpr u64 kR = " << g.reduction_size << "ull;\n";
            s << "    static constexpr int kBatch = " << shape.unroll << ";\n";
            s << "    static constexpr int kLanesX = " << shape.threadsPerRow << ";\n";
            if (shape.laneAxis < 0) {
                // dense [outer, R, inner]: a column begins at a multiple of the vector width, except the last one of an inner
                // extent that the width does not divide, which ends with the extent and owns only what the one before does not
                const uint64_t innerVectors = ceilDiv(g.inner_size, static_cast<uint64_t>(shape.vec));
                const uint64_t lastFirst = g.inner_size - static_cast<uint64_t>(shape.vec);
                const uint64_t shared = innerVectors * shape.vec - g.inner_size;  // leading elements of the last column that the one before owns
                s << "    static constexpr u64 kColumns = " << (g.outer_size * innerVectors) << "ull;\n";
                s << "    static __device__ __forceinline__ u64 columnFirst(u64 c) { const u64 first = (c % " << innerVectors << "ull) * " << shape.vec
                  << "ull; return first < " << lastFirst << "ull ? first : " << lastFirst << "ull; }\n";
                s << "    static __device__ __forceinline__ bool ownsElement(u64 c, int k) { return " << (shared == 0 ? "true" : "") ;
                if (shared != 0) s << "c % " << innerVectors << "ull != " << (innerVectors - 1) << "ull || k >= " << shared;
                s << "; }\n";
                s << "    static __device__ __forceinline__ u64 columnBase(u64 c) { return (c / " << innerVectors << "ull) * " << (g.reduction_size * g.inner_size)
                  << "ull + columnFirst(c); }\n";
                s << "    static __device__ __forceinline__ u64 rowOffset(u64 r) { return r * " << g.inner_size << "ull; }\n";
                s << "    static __device__ __forceinline__ u64 partialSlot(u64 c, int k) { return (c / " << innerVectors << "ull) * " << g.inner_size
                  << "ull + columnFirst(c) + k; }\n";
                s << "    static __device__ __forceinline__ u64 outputIndex(u64 c, int k) { return (c / " << innerVectors << "ull) * "
                  << g.tiled_output_outer_stride << "ull + (columnFirst(c) + k) * " << g.tiled_output_inner_stride << "ull; }\n";
            } else {
                s << "    static constexpr u64 kColumns = " << (g.output_elements / shape.vec) << "ull;\n";
                s << "    static __device__ __forceinline__ bool ownsElement(u64, int) { return true; }\n";
                // a view: columns enumerate the kept coordinates with the contiguous axis fastest (in vectors); outputs are
                // numbered row-major over the kept axes in their logical order
                const size_t lane = static_cast<size_t>(shape.laneAxis);
                std::vector<uint64_t> logicalStride(shape.keptDims.size(), 1);
                for (size_t a = shape.keptDims.size(); a-- > 1;) logicalStride[a - 1] = logicalStride[a] * shape.keptDims[a];
                const uint64_t laneVectors = shape.keptDims[lane] / shape.vec;
                std::ostringstream base, slot;
                base << "    static __device__ __forceinline__ u64 columnBase(u64 c) {\n        u64 offset = (c % " << laneVectors << "ull) * " << shape.vec
                     << "ull;\n        c /= " << laneVectors << "ull;\n";
                slot << "    static __device__ __forceinline__ u64 partialSlot(u64 c, int k) {\n        u64 index = ((c % " << laneVectors << "ull) * " << shape.vec
                     << "ull + k) * " << logicalStride[lane] << "ull;\n        c /= " << laneVectors << "ull;\n";
                for (size_t a = shape.keptDims.size(); a-- > 0;) {
                    if (a == lane) continue;
                    base << "        offset += (c % " << shape.keptDims[a] << "ull) * " << shape.keptStrides[a] << "ull;\n        c /= " << shape.keptDims[a] << "ull;\n";
                    slot << "        index += (c % " << shape.keptDims[a] << "ull) * " << logicalStride[a] << "ull;\n        c /= " << shape.keptDims[a] << "ull;\n";
                }
                base << "        return offset;\n    }\n";
                slot << "        return index;\n    }\n";
                s << base.str() << slot.str();
                s << "    static __device__ __forceinline__ u64 outputIndex(u64 c, int k) { return partialSlot(c, k); }\n";
                s << offsetFunction("rowOffset", shape.reducedDims, shape.reducedStrides);
            }
            body = "thor::reduceColumns<gen::Cfg>(src, out, partials, scale);";
            if (shape.transposeRows > 0) {
                const uint64_t laneVectors = (shape.laneAxis < 0 ? g.inner_size : shape.keptDims[static_cast<size_t>(shape.laneAxis)]) / shape.vec;
                s << "    static constexpr int kTransposeRows = " << shape.transposeRows << ";\n";
                s << "    static constexpr u64 kLaneVectors = " << laneVectors << "ull;\n";
                s << "    static constexpr u64 kQ = " << (g.output_elements / shape.vec / laneVectors) << "ull;\n";
                body = "thor::reduceColumnsTransposed<gen::Cfg>(src, out, scale);";
            }
            break;
        case ReductionShape::Kernel::Segments:
            s << "    typedef " << (request.offsetsAre64 ? "u64" : "u32") << " OffsetT;\n";
            s << "    static constexpr u64 kD = " << request.trailing << "ull;\n";
            s << "    static constexpr u64 kSegments = " << request.segments << "ull;\n";
            s << "    static constexpr u64 kColumnTiles = " << shape.blocks << "ull;\n";
            s << "    static constexpr int kBatch = " << shape.unroll << ";\n";
            s << "    static constexpr int kLanesX = " << shape.threadsPerRow << ";\n";
            s << "    static constexpr u64 kRows = " << request.segmentedRows << "ull;\n";
            s << "    static constexpr u64 kChunkRows = " << shape.chunkRows << "ull;\n";
            s << "    static constexpr u64 kChunks = " << shape.chunks << "ull;\n";
            s << "    static constexpr int kMinTeam = " << shape.minTeam << ";\n";
            s << "    static constexpr int kWalkGroup = " << shape.walkGroup << ";\n";
            s << "    static constexpr int kFinishLanes = " << shape.finishLanes << ";\n";
            s << "    static constexpr int kFinishThreads = " << shape.finishThreads << ";\n";
            body = shape.segmentsByRows ? "thor::reduceSegmentsByRows<gen::Cfg>(src, out, partials, scale, static_cast<const gen::Cfg::OffsetT*>(offsets));"
                                        : "thor::reduceSegments<gen::Cfg>(src, out, partials, scale, static_cast<const gen::Cfg::OffsetT*>(offsets));";
            break;
        case ReductionShape::Kernel::Strided: {
            std::vector<uint64_t> rd = shape.reducedDims, rs = shape.reducedStrides;
            if (shape.vec > 1) {
                rd.back() /= shape.vec;
                rs.back() = shape.vec;  // one step of the innermost axis = one vector
            }
            s << "    static constexpr u64 kReduction = " << (g.reduction_size / shape.vec) << "ull;\n";
            s << "    static constexpr int kBatch = " << shape.unroll << ";\n";
            s << offsetFunction("keptOffset", shape.keptDims, shape.keptStrides);
            s << offsetFunction("reducedOffset", rd, rs);
            body = "thor::reduceStrided<gen::Cfg>(src, out, partials, scale);";
            break;
        }
    }
    // layout of the final store made by the second stage of split kernels
    if (shape.kernel == ReductionShape::Kernel::Columns && shape.laneAxis < 0) {
        s << "    static constexpr u64 kFinishInner = " << g.inner_size << "ull;\n";
        s << "    static constexpr u64 kFinishOuterStride = " << g.tiled_output_outer_stride << "ull;\n";
        s << "    static constexpr u64 kFinishInnerStride = " << g.tiled_output_inner_stride << "ull;\n";
    } else {
        s << "    static constexpr u64 kFinishInner = 1ull;\n    static constexpr u64 kFinishOuterStride = 1ull;\n"
             "    static constexpr u64 kFinishInnerStride = 0ull;\n";
    }
    s << "};\n}  // namespace gen\n";

    // kernel signatures: sources, runtime scalars, reduction outputs, elementwise outputs, index output, partials, scale
    std::ostringstream outputParams, outputInit, finishParams, finishInit;
    for (size_t j = 0; j < values.size(); ++j) {
        outputParams << deviceTypeName(values[j].outputDType) << "* out" << j << ", ";
        outputInit << "out" << j << ", ";
    }
    finishParams << outputParams.str();
    finishInit << outputInit.str();
    for (size_t j = 0; j < request.elementwise.size(); ++j) {
        outputParams << deviceTypeName(request.elementwise[j].outputDType) << "* e" << j << ", ";
        outputInit << "e" << j << ", ";
        finishInit << "nullptr, ";
    }
    outputParams << "void* indexOut";
    finishParams << "void* indexOut";
    outputInit << "static_cast<decltype(gen::Cfg::Outputs::indexOut)>(indexOut)";
    finishInit << "static_cast<decltype(gen::Cfg::Outputs::indexOut)>(indexOut)";
    s << "extern \"C\" __global__ __launch_bounds__(" << shape.threads << ") ";
    if (const char* env = std::getenv("THOR_REDUCE_WAVES_PER_SIMD")) {  // tuning switch: register budget for N resident wavefronts per SIMD
        const long requested = std::atol(env);
        if (requested >= 1 && requested <= 8) s << "__attribute__((amdgpu_waves_per_eu(" << requested << "))) ";
    }
    s << "void thor_reduce_main(";
    for (size_t i = 0; i < sources.size(); ++i) s << "const " << deviceTypeName(sources[i].storage) << "* in" << i << ", ";
    for (uint32_t slot : request.scalarSlots) s << "float s" << slot << ", ";
    s << outputParams.str() << ", void* partials, float scale" << (request.segmented ? ", const void* offsets" : "") << ") {\n    const gen::Cfg::Sources src{";
    for (size_t i = 0; i < sources.size(); ++i) s << (i ? ", " : "") << "in" << i;
    for (uint32_t slot : request.scalarSlots) s << ", s" << slot;
    s << "};\n    const gen::Cfg::Outputs out{" << outputInit.str() << "};\n    (void)partials;\n    " << body << "\n}\n";
    const bool twoStageAll = shape.kernel == ReductionShape::Kernel::All && shape.blocks > 1;
    if (request.segmented && shape.chunks > 1) {
        s << "extern \"C\" __global__ __launch_bounds__(256) void thor_reduce_finish(const void* partials, "
          << finishParams.str() << ", float scale, const void* offsets) {\n    const gen::Cfg::Outputs out{" << finishInit.str()
          << "};\n    thor::finishSegments<gen::Cfg>(partials, out, scale, static_cast<const gen::Cfg::OffsetT*>(offsets));\n}\n";
        s << "extern \"C\" __global__ __launch_bounds__(256) void thor_reduce_prepare(void* partials, const void* offsets) {\n"
             "    thor::prepareSegments<gen::Cfg>(partials, static_cast<const gen::Cfg::OffsetT*>(offsets));\n}\n";
    } else if ((twoStageAll || shape.split > 1) && !shape.tickets) {
        s << "extern \"C\" __global__ __launch_bounds__(" << (twoStageAll ? 1024 : 256) << ") void thor_reduce_finish(const void* partials, "
          << finishParams.str() << ", float scale) {\n    const gen::Cfg::Outputs out{" << finishInit.str() << "};\n    thor::"
          << (twoStageAll ? "finishAll" : "finishPartials") << "<gen::Cfg>(partials, out, scale);\n}\n";
    }
    return s.str();
}

ReductionLaunchPlan buildReductionKernels(const ReductionKernelRequest& request) {
    const ReductionShape shape = planReductionShape(request);
    const std::string source = generateReductionSource(request, shape);
    ReductionLaunchPlan plan;
    // fp32 accumulation order is part of the result: never let the compiler fuse or reassociate across elements
    plan.mainKernel = compileKernel(source, "thor_reduce_main", request.deviceNum, /*fastContract=*/false);
    if (shape.tickets) {
        plan.ticketOffset = shape.ticketOffset;
        plan.ticketBytes = shape.ticketCount * 4;
    } else if (shape.kernel == ReductionShape::Kernel::All && shape.blocks > 1) {
        plan.finishKernel = compileKernel(source, "thor_reduce_finish", request.deviceNum, false);
        plan.finishThreads = 1024;
        plan.finishGridX = 1;
    } else if (shape.kernel == ReductionShape::Kernel::Segments) {
        if (shape.chunks > 1) {
            plan.prepareKernel = compileKernel(source, "thor_reduce_prepare", request.deviceNum, false);
            plan.prepareThreads = 256;
            plan.prepareGridX = static_cast<uint32_t>(ceilDiv(request.segments + 1, 256));
            plan.finishKernel = compileKernel(source, "thor_reduce_finish", request.deviceNum, false);
            plan.finishThreads = 256;
            plan.finishGridX = static_cast<uint32_t>(
                ceilDiv(shape.chunks * ceilDiv(request.trailing, static_cast<uint64_t>(shape.finishLanes)) * shape.finishThreads, 256));
        }
    } else if (shape.split > 1) {
        plan.finishKernel = compileKernel(source, "thor_reduce_finish", request.deviceNum, false);
        plan.finishThreads = 256;
        plan.finishGridX = static_cast<uint32_t>((request.geometry.output_elements * 64 + 255) / 256);
    }
    plan.mainGridX = shape.gridX;
    plan.mainGridY = shape.gridY;
    plan.mainThreads = static_cast<uint32_t>(shape.threads);
    plan.workspaceBytes = shape.workspaceBytes;
    plan.variant = shape.describe() + " [" + plan.mainKernel->kernelName + "]";
    return plan;
}

std::optional<Tensor> allocateReductionWorkspace(const ReductionLaunchPlan& plan, const TensorPlacement& placement, const Stream& stampStream) {
    if (plan.workspaceBytes == 0) return std::nullopt;
    Tensor workspace(placement, TensorDescriptor(DataType::UINT8, {plan.workspaceBytes}));
    if (plan.ticketBytes > 0) {
        Stream stream = stampStream;
        ScopedGpu scoped(stream.getGpuNum());
        THOR_HIP_CHECK(thorhip_memset_async(workspace.getMemPtr<char>() + plan.ticketOffset, 0, plan.ticketBytes, stream.getStream()));
        stream.synchronize();
    }
    return workspace;
}

}  // namespace ThorImplementation
