// Expression::rotaryPositionEmbedding: pairs of the head dimension turned by an angle that grows with the position
// (reference behaviour: Utilities/Expression/CudaSourceEmitter.cpp:3538-3697 angle, frequency rules and the rotation;
// Expression.cpp:4334-4426 parameters).
//
// The angle depends on the position and the pair only, so a thread owns one (position, group of pairs) item, works its sines
// and cosines out once and keeps them in registers while it walks every other coordinate of the tensor (batch, heads): the
// transcendental work is spread over that walk and the kernel stays a stream of 16-byte loads and stores.  The tensor is read
// as [O, first special axis, M, second special axis, I] whichever order the sequence and head-dimension axes come in; when the
// head dimension is the last axis a thread moves whole vectors along it, otherwise single elements.
#include "RotaryEmbedding.h"

#include "HipSourceEmitter.h"
#include "ReductionPlanner.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "thorhip_numeric_embed.h"

#include <algorithm>
#include <cstdlib>
#include <sstream>
#include <stdexcept>

namespace ThorImplementation {

namespace {

std::string floatArray(const std::vector<double>& values) {
    std::string s = "{";
    for (size_t i = 0; i < values.size(); ++i) s += (i ? ", " : "") + floatLiteral(values[i]);
    return s + "}";
}

// Statements that leave the frequency of pair `j` (a float expression) in `freq`; every rule in fp32, operation by operation as
// the reference emits it.
std::string frequencyStatements(const ExprNode& n, uint64_t rotary, const std::string& j, const std::string& ind) {
    std::ostringstream s;
    const std::string rot = "(float)" + std::to_string(rotary) + "ull";
    const std::string base = floatLiteral(n.rope_base), factor = floatLiteral(n.rope_scaling_factor);
    const std::string originalMax = floatLiteral(static_cast<double>(n.rope_original_max_position_embeddings));
    switch (n.rope_scaling_kind) {
        case RotaryScalingKind::DynamicNTK:
            s << ind << "float base = " << base << ";\n";
            s << ind << "if (seqLen > " << originalMax << " && " << rotary << "ull > 2ull) {\n";
            s << ind << "    const float ratio = (" << factor << " * seqLen / " << originalMax << ") - (" << factor << " - 1.0f);\n";
            s << ind << "    base = base * powf(ratio, " << rot << " / (float)" << (rotary - 2) << "ull);\n";
            s << ind << "}\n";
            s << ind << "freq = powf(base, -2.0f * " << j << " / " << rot << ");\n";
            break;
        case RotaryScalingKind::Yarn:
            s << ind << "const float posFreq = powf(" << base << ", 2.0f * " << j << " / " << rot << ");\n";
            s << ind << "const float extrapolated = 1.0f / posFreq;\n";
            s << ind << "const float interpolated = 1.0f / (" << factor << " * posFreq);\n";
            s << ind << "const float logBase = logf(" << base << ");\n";
            s << ind << "float low = (" << rot << " * logf(" << originalMax << " / (" << floatLiteral(n.rope_yarn_beta_fast)
              << " * 6.2831853071795864769f))) / (2.0f * logBase);\n";
            s << ind << "float high = (" << rot << " * logf(" << originalMax << " / (" << floatLiteral(n.rope_yarn_beta_slow)
              << " * 6.2831853071795864769f))) / (2.0f * logBase);\n";
            s << ind << "low = fmaxf(floorf(low), 0.0f);\n";
            s << ind << "high = fminf(ceilf(high), (float)" << (rotary - 1) << "ull);\n";
            s << ind << "if (low == high) high += 0.001f;\n";
            s << ind << "const float ramp = fminf(fmaxf((" << j << " - low) / (high - low), 0.0f), 1.0f);\n";
            s << ind << "freq = interpolated * ramp + extrapolated * (1.0f - ramp);\n";
            break;
        case RotaryScalingKind::LongRope:
            s << ind << "const float stretch = seqLen > " << originalMax << " ? thor_rope_long_factors[pair] : thor_rope_short_factors[pair];\n";
            s << ind << "freq = 1.0f / (stretch * powf(" << base << ", 2.0f * " << j << " / " << rot << "));\n";
            break;
        case RotaryScalingKind::Llama3: {
            const std::string lowFactor = floatLiteral(n.rope_llama3_low_freq_factor), highFactor = floatLiteral(n.rope_llama3_high_freq_factor);
            s << ind << "const float plain = powf(" << base << ", -2.0f * " << j << " / " << rot << ");\n";
            s << ind << "const float wavelength = 6.2831853071795864769f / plain;\n";
            s << ind << "const float lowWavelength = " << originalMax << " / " << lowFactor << ";\n";
            s << ind << "const float highWavelength = " << originalMax << " / " << highFactor << ";\n";
            s << ind << "if (wavelength > lowWavelength) {\n";
            s << ind << "    freq = plain / " << factor << ";\n";
            s << ind << "} else if (wavelength < highWavelength) {\n";
            s << ind << "    freq = plain;\n";
            s << ind << "} else {\n";
            s << ind << "    const float smooth = (" << originalMax << " / wavelength - " << lowFactor << ") / (" << highFactor << " - " << lowFactor << ");\n";
            s << ind << "    freq = (1.0f - smooth) * (plain / " << factor << ") + smooth * plain;\n";
            s << ind << "}\n";
            break;
        }
        case RotaryScalingKind::None:
        case RotaryScalingKind::Linear:
            s << ind << "freq = powf(" << base << ", -2.0f * " << j << " / " << rot << ");\n";
            break;
    }
    return s.str();
}

}  // namespace

std::shared_ptr<StampedEquation> stampRotaryEmbedding(const Tensor& values, const std::optional<Tensor>& positionIds,
                                                      const std::optional<Tensor>& effectiveLength, const Tensor& output, const ExprNode& n,
                                                      int deviceNum) {
    return stampRotaryEmbedding(values, positionIds, effectiveLength, output, n, deviceNum, RopeFusion{});
}

std::shared_ptr<StampedEquation> stampRotaryEmbedding(const Tensor& values, const std::optional<Tensor>& positionIds,
                                                      const std::optional<Tensor>& effectiveLength, const Tensor& output, const ExprNode& n,
                                                      int deviceNum, const RopeFusion& fusion) {
    if (!values.isInitialized() || !output.isInitialized()) throw std::runtime_error("RoPE requires initialized tensors.");
    const std::vector<uint64_t>& dims = values.getDimensions();
    const uint32_t seqAxis = n.rope_sequence_axis, dimAxis = n.rope_head_dim_axis;
    if (seqAxis >= dims.size() || dimAxis >= dims.size() || seqAxis == dimAxis) {
        throw std::runtime_error("RoPE sequence and head-dimension axes must be distinct axes of the input.");
    }
    if (output.getDimensions() != dims) throw std::runtime_error("RoPE output must have the shape of its input.");
    for (uint64_t d : dims)
        if (d == 0) throw std::runtime_error("RoPE does not support zero-sized dimensions.");
    if (!values.isDenseContiguous() || !output.isDenseContiguous()) throw std::runtime_error("RoPE requires dense tensors.");
    const uint64_t seq = dims[seqAxis], headDim = dims[dimAxis];
    const uint64_t rotary = n.rope_rotary_dim == 0 ? headDim : n.rope_rotary_dim;
    if (rotary == 0 || rotary > headDim || (rotary & 1ull) != 0) throw std::runtime_error("RoPE rotary_dim must be even and no larger than the head dimension.");
    const uint64_t half = rotary / 2;
    if (n.rope_base <= 0.0 || n.rope_scaling_factor <= 0.0) throw std::runtime_error("Invalid RoPE base/scaling factor during code generation.");
    if (n.rope_scaling_kind == RotaryScalingKind::LongRope &&
        (n.rope_long_rope_short_factors.size() != half || n.rope_long_rope_long_factors.size() != half)) {
        throw std::runtime_error("LongRoPE code generation requires short/long factor lists of length rotary_dim / 2.");
    }
    if (positionIds.has_value()) {
        if (!positionIds->isInitialized() || !positionIds->isDenseContiguous() || positionIds->getTotalNumElements() != seq) {
            throw std::runtime_error("RoPE position ids must hold one position per element of the sequence axis.");
        }
    }
    if (effectiveLength.has_value()) {
        if (!effectiveLength->isInitialized() || effectiveLength->getTotalNumElements() != 1) {
            throw std::runtime_error("RoPE effective sequence length must be a single element.");
        }
    }

    // [O, first, M, second, I] around the two special axes
    const uint32_t firstAxis = std::min(seqAxis, dimAxis), secondAxis = std::max(seqAxis, dimAxis);
    uint64_t outerCount = 1, middleCount = 1, innerCount = 1;
    for (size_t d = 0; d < dims.size(); ++d) {
        if (d < firstAxis) outerCount *= dims[d];
        if (d > firstAxis && d < secondAxis) middleCount *= dims[d];
        if (d > secondAxis) innerCount *= dims[d];
    }
    auto strideOf = [&](uint32_t axis) {
        uint64_t s = 1;
        for (size_t d = axis + 1; d < dims.size(); ++d) s *= dims[d];
        return s;
    };
    const uint64_t seqStride = strideOf(seqAxis), dimStride = strideOf(dimAxis);
    const uint64_t middleStride = dims[secondAxis] * innerCount, outerStride = dims[firstAxis] * middleCount * middleStride;
    const uint64_t walk = outerCount * middleCount * innerCount;  // coordinates a thread visits with one set of angles
    const uint64_t total = walk * seq * headDim;

    // every tensor the kernel streams: the operand (or what the prologue computes it from), what the epilogue reads, the output
    std::vector<Tensor> streamed;
    if (fusion.prologue.has_value()) {
        streamed = fusion.prologue->tensors;
    } else {
        streamed.push_back(values);
    }
    if (fusion.epilogue.has_value()) streamed.insert(streamed.end(), fusion.epilogue->tensors.begin(), fusion.epilogue->tensors.end());
    streamed.push_back(output);
    uint32_t widest = 1;
    for (const Tensor& t : streamed) {
        if (!t.isInitialized() || !t.isDenseContiguous() || t.getDimensions() != dims) throw std::runtime_error("RoPE streams dense tensors of the rotated shape.");
        widest = std::max<uint32_t>(widest, dataTypeSizeInBytes(t.getDataType()));
    }
    const uint64_t tail = headDim - rotary;
    int vec = dimStride == 1 ? static_cast<int>(16 / widest) : 1;
    auto fits = [&](int v) {
        if (v == 1) return true;
        if (tail % v != 0) return false;
        if (n.rope_interleaved ? rotary % v != 0 : half % v != 0) return false;
        for (const Tensor& t : streamed)
            if (pointerAlignment(t.getMemPtr()) % (static_cast<uint64_t>(v) * dataTypeSizeInBytes(t.getDataType())) != 0) return false;
        return true;
    };
    while (!fits(vec)) vec /= 2;
    const bool pairsInsideVector = n.rope_interleaved && vec > 1;
    const uint64_t pairSlots = n.rope_interleaved ? (vec > 1 ? rotary / vec : half) : half / vec;
    const int pairsPerThread = n.rope_interleaved ? (vec > 1 ? vec / 2 : 1) : vec;
    const uint64_t slots = pairSlots + tail / vec;
    // Half-rotated layout whose halves are not whole 64-byte sectors (head dimensions of 80 or 96 halves, 80 floats): a lane
    // that reads both vectors of its pairs touches every sector of the row in each of its two loads and uses part of it.  Two
    // adjacent lanes then share the pairs: each reads, turns and writes one of the two vectors and gets the other operand from
    // its neighbour, so one load of the wavefront covers the rows whole ([8, 32, 4096, 80] bf16: 137 us the other way).
    uint32_t narrowest = 8;
    for (const Tensor& t : streamed) narrowest = std::min<uint32_t>(narrowest, dataTypeSizeInBytes(t.getDataType()));
    const bool pairedLanes = !n.rope_interleaved && vec > 1 && (half * narrowest) % 64 != 0 && std::getenv("THOR_ROPE_NO_PAIRED_LANES") == nullptr;
    const uint64_t walkSlots = pairedLanes ? (2 * pairSlots + tail / vec + 1) / 2 * 2 : slots;  // an even count keeps the two lanes of a pair adjacent
    const uint64_t items = seq * walkSlots;
    const uint32_t threads = 256;
    const uint64_t blocksPerChunk = (items + threads - 1) / threads;
    // Many blocks, each thread walking at least two coordinates with its angles (measured on [8, 32, 4096, 128] bf16: 88 us
    // with walks of 2 in 16384 blocks, 97 us with walks of 8, 136 us with walks of 1, where the sines are not shared at all).
    uint64_t wantedBlocks = 32768;
    if (const char* text = std::getenv("THOR_ROPE_BLOCKS")) {
        const long long asked = std::atoll(text);
        if (asked >= 1 && asked <= (1 << 24)) wantedBlocks = static_cast<uint64_t>(asked);
    }
    uint64_t chunks = std::min<uint64_t>(std::max<uint64_t>(1, walk / 2), std::max<uint64_t>(1, (wantedBlocks + blocksPerChunk - 1) / blocksPerChunk));
    const uint64_t walkPerChunk = (walk + chunks - 1) / chunks;
    chunks = (walk + walkPerChunk - 1) / walkPerChunk;
    // Heads between the sequence axis and a last-axis head dimension ([.., S, heads.., D]): everything at one position is one
    // contiguous run, so a block takes a few consecutive positions, leaves their sines and cosines in LDS (one per thread) and
    // streams the run, every head reading the same table.
    const bool tileLayout = middleCount > 1 && innerCount == 1 && dimStride == 1 && seqAxis < dimAxis && std::getenv("THOR_ROPE_NO_TILES") == nullptr;
    uint64_t tilePositions = std::max<uint64_t>(1, threads / half);
    while (tilePositions * middleCount * walkSlots < 2 * threads && tilePositions * 2 * half <= 4096) tilePositions *= 2;
    tilePositions = std::min(tilePositions, seq);
    const uint64_t tiles = (seq + tilePositions - 1) / tilePositions;
    const bool tileFits = tilePositions * middleCount * walkSlots < (1ull << 31);  // the tiled kernel counts a block's items in 32 bits
    const bool tiled = tileLayout && tileFits;
    const uint64_t blocks = tiled ? outerCount * tiles : blocksPerChunk * chunks;
    if (blocks > 0x7fffffffull) throw std::runtime_error("RoPE: the tensor is too large for one launch.");

    const std::string inType = deviceTypeName(values.getDataType()), outType = deviceTypeName(output.getDataType());
    const bool needsLength = n.rope_scaling_kind == RotaryScalingKind::DynamicNTK || n.rope_scaling_kind == RotaryScalingKind::LongRope;
    // a block shares the table of frequencies when that saves work: more than one thread of the block per pair
    const bool sharedFrequencies = half <= 8192 && items >= 2 * half;
    const bool hasPrologue = fusion.prologue.has_value(), hasEpilogue = fusion.epilogue.has_value();

    // ---- the three things a site (one vector of elements at one offset) does, with or without fused elementwise work ----
    auto replaceAll = [](std::string text, const std::string& what, const std::string& with) {
        for (size_t at = text.find(what); at != std::string::npos; at = text.find(what, at + with.size())) text.replace(at, what.size(), with);
        return text;
    };
    auto indented = [](const std::string& statements, const std::string& ind) {
        std::string out;
        size_t at = 0;
        while (at < statements.size()) {
            const size_t eol = statements.find('\n', at);
            const std::string line = statements.substr(at, eol == std::string::npos ? std::string::npos : eol - at);
            const size_t firstText = line.find_first_not_of(' ');
            if (firstText != std::string::npos) out += ind + line.substr(firstText) + "\n";
            if (eol == std::string::npos) break;
            at = eol + 1;
        }
        return out;
    };
    const char* contractOn = "#pragma clang fp contract(fast)\n";
    // loads of one site: the operand's sources and what the epilogue reads, all at `offset`
    auto loadSite = [&](const std::string& ind, const std::string& site, const std::string& offset) {
        std::string out;
        if (hasPrologue) {
            for (size_t i = 0; i < fusion.prologue->tensors.size(); ++i) {
                const std::string name = site + "_" + std::to_string(i);
                out += ind + "thor::Pack<" + deviceTypeName(fusion.prologue->tensors[i].getDataType()) + ", V> " + name + ";\n";
                out += ind + name + ".loadStream(p" + std::to_string(i) + " + " + offset + ");\n";
            }
        } else {
            out += ind + "thor::Pack<" + inType + ", V> " + site + ";\n" + ind + site + ".loadStream(x + " + offset + ");\n";
        }
        if (hasEpilogue) {
            for (size_t i = 0; i < fusion.epilogue->tensors.size(); ++i) {
                const std::string name = site + "_e" + std::to_string(i);
                out += ind + "thor::Pack<" + deviceTypeName(fusion.epilogue->tensors[i].getDataType()) + ", V> " + name + ";\n";
                out += ind + name + ".loadStream(e" + std::to_string(i) + " + " + offset + ");\n";
            }
        }
        return out;
    };
    // `float var` = element k of the site as the rotation reads it
    auto operandOf = [&](const std::string& ind, const std::string& var, const std::string& site, const std::string& k) {
        if (!hasPrologue) return ind + "const float " + var + " = thor::toFloat(" + site + ".v[" + k + "]);\n";
        std::string text = fusion.prologue->statements;
        for (size_t i = 0; i < fusion.prologue->tensors.size(); ++i) {
            text = replaceAll(text, "@P" + std::to_string(i) + "@", site + "_" + std::to_string(i) + ".v[" + k + "]");
        }
        std::string out = ind + "float " + var + ";\n" + ind + "{\n";
        if (fusion.prologue->contract) out += contractOn;
        out += indented(text, ind + "    ");
        out += ind + "    " + var + " = " + fusion.prologue->value + ";\n" + ind + "}\n";
        return out;
    };
    // element k of the output site from the rotated (or, beyond the rotary part, untouched) fp32 value
    auto resultTo = [&](const std::string& ind, const std::string& outSite, const std::string& site, const std::string& k, const std::string& rotated) {
        if (!hasEpilogue) return ind + outSite + ".v[" + k + "] = thor::fromFloat<" + outType + ">(" + rotated + ");\n";
        std::string text = fusion.epilogue->statements;
        for (size_t i = 0; i < fusion.epilogue->tensors.size(); ++i) {
            text = replaceAll(text, "@E" + std::to_string(i) + "@", site + "_e" + std::to_string(i) + ".v[" + k + "]");
        }
        std::string out = ind + "{\n";
        out += ind + "    const float turned = " + rotated + ";\n";
        out += ind + "    const " + std::string(valueCType(fusion.rotatedDType)) + " rotatedValue = " + castValueExpr("turned", DataType::FP32, fusion.rotatedDType) +
               ";\n";
        out += ind + "    {\n";
        if (fusion.epilogue->contract) out += contractOn;
        out += indented(replaceAll(text, "@R@", "rotatedValue"), ind + "        ");
        out += ind + "        " + outSite + ".v[" + k + "] = " + fusion.epilogue->value + ";\n";
        out += ind + "    }\n" + ind + "}\n";
        return out;
    };
    // a vector of the part of the head dimension that is not rotated: through the same elementwise work, unturned
    auto copySite = [&](const std::string& ind, const std::string& offset) {
        std::string out = loadSite(ind, "p", offset);
        out += ind + "thor::Pack<" + outType + ", V> q;\n";
        out += "#pragma unroll\n" + ind + "for (int k = 0; k < V; ++k) {\n";
        out += operandOf(ind + "    ", "a", "p", "k");
        out += resultTo(ind + "    ", "q", "p", "k", "a");
        out += ind + "}\n" + ind + "q.storeStream(out + " + offset + ");\n";
        return out;
    };
    // pairs that lie inside one vector (interleaved layout)
    auto turnInsideVector = [&](const std::string& ind, const std::string& offset) {
        std::string out = loadSite(ind, "p", offset);
        out += ind + "thor::Pack<" + outType + ", V> q;\n";
        out += "#pragma unroll\n" + ind + "for (int k = 0; k < P; ++k) {\n";
        out += operandOf(ind + "    ", "a", "p", "2 * k");
        out += operandOf(ind + "    ", "b", "p", "2 * k + 1");
        out += resultTo(ind + "    ", "q", "p", "2 * k", "a * cs[k] - b * sn[k]");
        out += resultTo(ind + "    ", "q", "p", "2 * k + 1", "a * sn[k] + b * cs[k]");
        out += ind + "}\n" + ind + "q.storeStream(out + " + offset + ");\n";
        return out;
    };
    // the two elements of a pair in two vectors `apart` coordinates from each other
    auto turnAcrossVectors = [&](const std::string& ind, const std::string& offsetA, const std::string& offsetB) {
        std::string out = loadSite(ind, "pa", offsetA) + loadSite(ind, "pb", offsetB);
        out += ind + "thor::Pack<" + outType + ", V> qa, qb;\n";
        out += "#pragma unroll\n" + ind + "for (int k = 0; k < V; ++k) {\n";
        out += operandOf(ind + "    ", "a", "pa", "k");
        out += operandOf(ind + "    ", "b", "pb", "k");
        out += resultTo(ind + "    ", "qa", "pa", "k", "a * cs[k] - b * sn[k]");
        out += resultTo(ind + "    ", "qb", "pb", "k", "a * sn[k] + b * cs[k]");
        out += ind + "}\n" + ind + "qa.storeStream(out + " + offsetA + ");\n" + ind + "qb.storeStream(out + " + offsetB + ");\n";
        return out;
    };

    std::ostringstream s;
    s << thor_embed::kDevicePrelude;
    if (n.rope_scaling_kind == RotaryScalingKind::LongRope) {
        s << "__device__ const float thor_rope_short_factors[" << half << "] = " << floatArray(n.rope_long_rope_short_factors) << ";\n";
        s << "__device__ const float thor_rope_long_factors[" << half << "] = " << floatArray(n.rope_long_rope_long_factors) << ";\n";
    }
    s << "extern \"C\" __global__ __launch_bounds__(256) void thor_rope(";
    if (hasPrologue) {
        for (size_t i = 0; i < fusion.prologue->tensors.size(); ++i) {
            s << (i ? ", " : "") << "const " << deviceTypeName(fusion.prologue->tensors[i].getDataType()) << "* __restrict__ p" << i;
        }
    } else {
        s << "const " << inType << "* __restrict__ x";
    }
    if (positionIds.has_value()) s << ", const " << deviceTypeName(positionIds->getDataType()) << "* __restrict__ ids";
    if (effectiveLength.has_value()) s << ", const " << deviceTypeName(effectiveLength->getDataType()) << "* __restrict__ length";
    if (hasEpilogue) {
        for (size_t i = 0; i < fusion.epilogue->tensors.size(); ++i) {
            s << ", const " << deviceTypeName(fusion.epilogue->tensors[i].getDataType()) << "* __restrict__ e" << i;
        }
    }
    for (uint32_t slot : fusion.scalarSlots) s << ", float s" << slot;
    s << ", " << outType << "* __restrict__ out) {\n";
    s << "    constexpr int V = " << vec << ", P = " << pairsPerThread << ";\n";
    if (needsLength) {
        const std::string extent = effectiveLength.has_value() ? std::string("thor::toFloat(length[0])") : floatLiteral(static_cast<double>(seq));
        s << "    const float seqLen = fmaxf(" << extent << " + " << floatLiteral(static_cast<double>(std::max<int64_t>(0, n.rope_position_offset)))
          << ", 1.0f);\n";
    }
    const std::string attention = floatLiteral(n.rope_attention_factor);
    // the two elements of a pair lie `apart` coordinates from each other along the head dimension
    const uint64_t apart = n.rope_interleaved ? 1 : half;
    if (tiled) {
        const uint64_t table = tilePositions * half;
        s << "    __shared__ float sines[" << table << "], cosines[" << table << "];\n";
        s << "    const thor::u64 outer = blockIdx.x / " << tiles << "u, firstPosition = (thor::u64)(blockIdx.x % " << tiles << "u) * " << tilePositions << "ull;\n";
        s << "    for (thor::u32 t = threadIdx.x; t < " << table << "u; t += " << threads << "u) {\n";
        s << "        const thor::u32 pair = t % " << half << "u;\n";
        s << "        const thor::u64 position = firstPosition + t / " << half << "u;\n";
        s << "        float sn = 0.0f, cs = 0.0f;\n";
        s << "        if (position < " << seq << "ull) {\n";
        if (positionIds.has_value()) {
            s << "            float angleBase = thor::toFloat(ids[position]);\n";
        } else {
            s << "            float angleBase = thor::toFloat(position) + " << floatLiteral(static_cast<double>(n.rope_position_offset)) << ";\n";
        }
        if (n.rope_scaling_kind == RotaryScalingKind::Linear) s << "            angleBase = angleBase / " << floatLiteral(n.rope_scaling_factor) << ";\n";
        s << "            float freq = 0.0f;\n";
        s << "            {\n" << frequencyStatements(n, rotary, "thor::toFloat(pair)", "                ") << "            }\n";
        s << "            const float theta = angleBase * freq;\n";
        s << "            sincosf(theta, &sn, &cs);\n";  // one argument reduction for both (a third fewer instructions than sinf + cosf)
        if (n.rope_attention_factor != 1.0) s << "            sn *= " << attention << ";\n            cs *= " << attention << ";\n";
        if (n.rope_inverse) s << "            sn = -sn;\n";
        s << "        }\n        sines[t] = sn;\n        cosines[t] = cs;\n    }\n";
        s << "    __syncthreads();\n";
        s << "    const thor::u64 base = outer * " << outerStride << "ull + firstPosition * " << seqStride << "ull;\n";
        s << "    const thor::u64 left = " << seq << "ull - firstPosition;\n";
        const uint64_t tileTurningSlots = pairedLanes ? 2 * pairSlots : pairSlots;
        s << "    const thor::u32 liveItems = (thor::u32)(left < " << tilePositions << "ull ? left : " << tilePositions << "ull) * " << middleCount * walkSlots << "u;\n";
        s << "    for (thor::u32 item = threadIdx.x; item < liveItems; item += " << threads << "u) {\n";
        s << "        const thor::u32 row = item / " << walkSlots << "u, slot = item % " << walkSlots << "u;\n";
        s << "        const thor::u64 rowBase = base + (thor::u64)row * " << headDim << "ull;\n";
        if (tail != 0 || walkSlots != tileTurningSlots) {
            s << "        if (slot >= " << tileTurningSlots << "u) {\n";
            if (walkSlots != tileTurningSlots + tail / vec) s << "            if (slot >= " << tileTurningSlots + tail / vec << "u) continue;  // the slot that makes the count even\n";
            s << "            const thor::u64 e = rowBase + " << rotary << "ull + (slot - " << tileTurningSlots << "u) * V;\n";
            s << copySite("            ", "e");
            s << "            continue;\n        }\n";
        }
        if (pairedLanes) {
            s << "        const thor::u32 firstPair = (slot / 2u) * P;\n        const bool second = (slot & 1u) != 0;\n";
        } else {
            s << "        const thor::u32 firstPair = slot * P;\n";
        }
        s << "        const float* sn = sines + (row / " << middleCount << "u) * " << half << "u + firstPair;\n";
        s << "        const float* cs = cosines + (row / " << middleCount << "u) * " << half << "u + firstPair;\n";
        if (pairedLanes) {
            s << "        const thor::u64 e = rowBase + firstPair + (second ? " << apart << "u : 0u);\n";
            s << loadSite("        ", "p", "e");
            s << "        thor::Pack<" << outType << ", V> q;\n";
            s << "#pragma unroll\n        for (int k = 0; k < V; ++k) {\n";
            s << operandOf("            ", "a", "p", "k");
            s << "            const float b = __shfl_xor(a, 1);\n";
            s << resultTo("            ", "q", "p", "k", "a * cs[k] + b * (second ? sn[k] : -sn[k])");
            s << "        }\n        q.storeStream(out + e);\n";
        } else if (pairsInsideVector) {
            s << "        const thor::u64 e = rowBase + firstPair * 2;\n";
            s << turnInsideVector("        ", "e");
        } else {
            s << "        const thor::u64 ea = rowBase + " << (n.rope_interleaved ? "firstPair * 2" : "firstPair") << ", eb = ea + " << apart << "ull;\n";
            s << turnAcrossVectors("        ", "ea", "eb");
        }
        s << "    }\n}\n";
    } else {
    if (sharedFrequencies) {
        // one frequency per pair, worked out once per block
        s << "    __shared__ float frequencies[" << half << "];\n";
        s << "    for (thor::u32 pair = threadIdx.x; pair < " << half << "u; pair += " << threads << "u) {\n";
        s << "        float freq = 0.0f;\n";
        s << "        {\n" << frequencyStatements(n, rotary, "thor::toFloat(pair)", "            ") << "        }\n";
        s << "        frequencies[pair] = freq;\n    }\n";
        s << "    __syncthreads();\n";
    }
    s << "    const thor::u64 chunk = blockIdx.x / " << blocksPerChunk << "u;\n";
    s << "    const thor::u64 item = (thor::u64)(blockIdx.x % " << blocksPerChunk << "u) * " << threads << " + threadIdx.x;\n";
    s << "    if (item >= " << items << "ull) return;\n";
    s << "    const thor::u64 position = item / " << walkSlots << "ull, slot = item % " << walkSlots << "ull;\n";
    s << "    const thor::u64 walkFirst = chunk * " << walkPerChunk << "ull;\n";
    s << "    const thor::u64 walkLast = walkFirst + " << walkPerChunk << "ull < " << walk << "ull ? walkFirst + " << walkPerChunk << "ull : " << walk << "ull;\n";
    // address of (walk coordinate w, this position, head-dimension coordinate d)
    s << "    auto at = [&](thor::u64 w, thor::u64 d) {\n";
    s << "        const thor::u64 i = w % " << innerCount << "ull, m = (w / " << innerCount << "ull) % " << middleCount << "ull, o = w / " << innerCount * middleCount
      << "ull;\n";
    s << "        return o * " << outerStride << "ull + m * " << middleStride << "ull + i + position * " << seqStride << "ull + d * " << dimStride << "ull;\n";
    s << "    };\n";
    const uint64_t turningSlots = pairedLanes ? 2 * pairSlots : pairSlots;
    if (tail != 0 || walkSlots != turningSlots) {
        s << "    if (slot >= " << turningSlots << "ull) {\n";
        if (walkSlots != turningSlots + tail / vec) s << "        if (slot >= " << turningSlots + tail / vec << "ull) return;  // the slot that makes the count even\n";
        s << "        // beyond the rotary part: a copy\n";
        s << "        const thor::u64 d = " << rotary << "ull + (slot - " << turningSlots << "ull) * V;\n";
        s << "        for (thor::u64 w = walkFirst; w < walkLast; ++w) {\n";
        s << "            const thor::u64 e = at(w, d);\n";
        s << copySite("            ", "e");
        s << "        }\n        return;\n    }\n";
    }
    if (pairedLanes) {
        s << "    const thor::u64 firstPair = (slot / 2) * P;\n    const bool second = (slot & 1ull) != 0;\n";
    } else {
        s << "    const thor::u64 firstPair = slot * P;\n";
    }
    if (positionIds.has_value()) {
        s << "    float angleBase = thor::toFloat(ids[position]);\n";
    } else {
        s << "    float angleBase = thor::toFloat(position) + " << floatLiteral(static_cast<double>(n.rope_position_offset)) << ";\n";
    }
    if (n.rope_scaling_kind == RotaryScalingKind::Linear) s << "    angleBase = angleBase / " << floatLiteral(n.rope_scaling_factor) << ";\n";
    s << "    float sn[P], cs[P];\n";
    s << "#pragma unroll\n    for (int k = 0; k < P; ++k) {\n";
    s << "        const thor::u64 pair = firstPair + k;\n";
    if (sharedFrequencies) {
        s << "        const float freq = frequencies[pair];\n";
    } else {
        s << "        float freq = 0.0f;\n";
        s << "        {\n" << frequencyStatements(n, rotary, "thor::toFloat(pair)", "            ") << "        }\n";
    }
    s << "        const float theta = angleBase * freq;\n";
    s << "        sincosf(theta, &sn[k], &cs[k]);\n";
    if (n.rope_attention_factor != 1.0) {
        s << "        sn[k] *= " << floatLiteral(n.rope_attention_factor) << ";\n        cs[k] *= " << floatLiteral(n.rope_attention_factor) << ";\n";
    }
    if (n.rope_inverse) s << "        sn[k] = -sn[k];\n";
    s << "    }\n";
    if (pairedLanes) {
        // own * cos + other * (+-sin): the first lane of a pair holds a (a cos - b sin), the second b (b cos + a sin)
        s << "    float turn[P];\n#pragma unroll\n    for (int k = 0; k < P; ++k) turn[k] = second ? sn[k] : -sn[k];\n";
    }
    s << "#pragma unroll 1\n";
    s << "    for (thor::u64 w = walkFirst; w < walkLast; ++w) {\n";
    if (pairedLanes) {
        s << "        const thor::u64 e = at(w, firstPair + (second ? " << apart << "ull : 0ull));\n";
        s << loadSite("        ", "p", "e");
        s << "        thor::Pack<" << outType << ", V> q;\n";
        s << "#pragma unroll\n        for (int k = 0; k < V; ++k) {\n";
        s << operandOf("            ", "a", "p", "k");
        s << "            const float b = __shfl_xor(a, 1);\n";
        s << resultTo("            ", "q", "p", "k", "a * cs[k] + b * turn[k]");
        s << "        }\n        q.storeStream(out + e);\n";
    } else if (pairsInsideVector) {
        s << "        const thor::u64 e = at(w, firstPair * 2);\n";
        s << turnInsideVector("        ", "e");
    } else {
        const std::string firstCoordinate = n.rope_interleaved ? "firstPair * 2" : "firstPair";
        s << "        const thor::u64 ea = at(w, " << firstCoordinate << "), eb = at(w, " << firstCoordinate << " + " << apart << "ull);\n";
        s << turnAcrossVectors("        ", "ea", "eb");
    }
    s << "    }\n}\n";
    }

    const std::shared_ptr<CompiledKernel> kernel = compileKernel(s.str(), "thor_rope", deviceNum, /*fastContract=*/false);
    std::ostringstream description;
    description << "rope(seq=" << seq << ",head_dim=" << headDim << ",rotary=" << rotary << (n.rope_interleaved ? ",interleaved" : "")
                << (n.rope_inverse ? ",inverse" : "");
    if (tiled) {
        description << ",tile=" << tilePositions << "x" << middleCount << (pairedLanes ? ",paired_lanes" : "");
    } else {
        description << ",walk=" << walk << "/" << chunks << (pairedLanes ? ",paired_lanes" : "");
    }
    description << ",vec=" << vec << ",grid=" << blocks << ") [" << kernel->kernelName << "]";
    std::vector<Tensor> inputs;
    if (hasPrologue) {
        inputs = fusion.prologue->tensors;
    } else {
        inputs.push_back(values);
    }
    if (positionIds.has_value()) inputs.push_back(*positionIds);
    if (effectiveLength.has_value()) inputs.push_back(*effectiveLength);
    if (hasEpilogue) inputs.insert(inputs.end(), fusion.epilogue->tensors.begin(), fusion.epilogue->tensors.end());
    std::vector<size_t> inputArgs;
    for (size_t i = 0; i < inputs.size(); ++i) inputArgs.push_back(i);
    std::vector<StampedEquation::ScalarArgument> scalarArgs;
    size_t next = inputs.size();
    for (const std::string& name : fusion.scalarNames) scalarArgs.push_back({name, next++});
    std::string text = description.str();
    if (hasPrologue || hasEpilogue) {
        text = std::string("fused ") + (hasPrologue ? "prologue+" : "") + text.substr(0, text.find(" [")) + (hasEpilogue ? "+epilogue" : "") + text.substr(text.find(" ["));
    }
    return std::make_shared<StampedEquation>(kernel, inputs, std::vector<Tensor>{output}, scalarArgs, inputArgs, std::vector<size_t>{next}, next + 1,
                                             /*passNumel=*/false, total, total > UINT32_MAX, static_cast<uint32_t>(blocks), threads,
                                             /*flops=*/fusion.extraFlopsPerElement * total, text);
}

}  // namespace ThorImplementation
