// Reduction kernels for gfx950, instantiated by generated code through a `Cfg` traits struct (appended after the device
// prelude at run-time compilation).  They replace cub::DeviceReduce / DeviceSegmentedReduce and the reference's tiled
// kernels (Utilities/TensorOperations/Cub/CubReductionOperation.cuh:2482-3054, CubArgReductionOperation.cuh:1054-1186).
//
// Cfg provides
//   In, Out                       storage types of the input and of the value output
//   Acc                           ValueAcc<Op> or ArgAcc<IS_MAX, IndexT>
//   IndexT                        u32 or u64: type of element offsets and of arg indices inside the kernel
//   OutIndex                      u32 or u64: storage type of the arg index output
//   kIsArg, kWriteValue, kWriteIndex
//   kFinalize, kDivisor           0 none / 1 divide by kDivisor / 2 square root
//   kVec                          elements per vector load (all shapes and base addresses are multiples of it)
//   kThreads                      threads per block
// plus the geometry constants each kernel names below.  Shapes are compile-time constants: trip counts are known, loops
// unroll, and every divide is a divide by a constant.
#pragma once

namespace thor {

template <typename Cfg>
__device__ __forceinline__ void loadAsFloat(const typename Cfg::In* p, float (&x)[Cfg::kVec]) {
    Pack<typename Cfg::In, Cfg::kVec> pack;
    pack.loadStream(p);
#pragma unroll
    for (int k = 0; k < Cfg::kVec; ++k) x[k] = toFloat(pack.v[k]);
}

template <typename Cfg>
__device__ __forceinline__ void storeResult(const typename Cfg::Acc& acc, u64 outIndex, void* valueOut, void* indexOut, float scale) {
    if constexpr (Cfg::kIsArg) {
        if (Cfg::kWriteValue) static_cast<typename Cfg::Out*>(valueOut)[outIndex] = fromFloat<typename Cfg::Out>(acc.v);
        if (Cfg::kWriteIndex) static_cast<typename Cfg::OutIndex*>(indexOut)[outIndex] = (typename Cfg::OutIndex)acc.i;
    } else {
        static_cast<typename Cfg::Out*>(valueOut)[outIndex] =
            fromFloat<typename Cfg::Out>(finalizeValue<Cfg::kFinalize>(acc.v, Cfg::kDivisor, scale));
    }
}

// Partials live in a float array followed (arg reductions only) by an IndexT array of the same length.
template <typename Cfg>
__device__ __forceinline__ void storePartial(const typename Cfg::Acc& acc, void* partials, u64 slot, u64 slots) {
    static_cast<float*>(partials)[slot] = acc.v;
    if constexpr (Cfg::kIsArg) {
        typename Cfg::IndexT* ip = reinterpret_cast<typename Cfg::IndexT*>(static_cast<char*>(partials) + ((slots * 4 + 7) / 8) * 8);
        ip[slot] = acc.i;
    }
}
template <typename Cfg>
__device__ __forceinline__ typename Cfg::Acc loadPartial(const void* partials, u64 slot, u64 slots) {
    typename Cfg::Acc acc;
    acc.v = static_cast<const float*>(partials)[slot];
    if constexpr (Cfg::kIsArg) {
        const typename Cfg::IndexT* ip =
            reinterpret_cast<const typename Cfg::IndexT*>(static_cast<const char*>(partials) + ((slots * 4 + 7) / 8) * 8);
        acc.i = ip[slot];
    }
    return acc;
}

// ---- whole tensor -> one value ------------------------------------------------------------------------------------------
// Cfg: kN (elements), kUnroll (vectors in flight per thread), kBlocks (grid size).
// Each block folds a block-strided set of chunks into one partial; finishAll (a second, single-block launch) folds the
// partials.  A single-launch variant in which the last block to finish (atomic ticket after a device-scope fence) does
// the final fold was measured at 1.98 ms for 2^26 fp32 elements on MI355X against 0.04 ms for the streaming part alone:
// a device-scope release per block has to write back a non-coherent per-XCD L2, and 16 384 tickets serialise on one
// address.  Two launches cost a few microseconds.
template <typename Cfg>
__device__ __forceinline__ void reduceAll(const typename Cfg::In* in, void* valueOut, void* indexOut, void* partials, float scale) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    constexpr IndexT kVectors = (IndexT)(Cfg::kN / Cfg::kVec);
    constexpr IndexT kChunk = (IndexT)Cfg::kThreads * Cfg::kUnroll;
    __shared__ Acc scratch[Cfg::kThreads / kWave];
    Acc acc;
    acc.reset();
    for (IndexT base = (IndexT)blockIdx.x * kChunk; base < kVectors; base += (IndexT)Cfg::kBlocks * kChunk) {
        float x[Cfg::kUnroll][Cfg::kVec];
        bool live[Cfg::kUnroll];
#pragma unroll
        for (int u = 0; u < Cfg::kUnroll; ++u) {
            const IndexT v = base + (IndexT)u * Cfg::kThreads + threadIdx.x;
            live[u] = v < kVectors;
            if (live[u]) loadAsFloat<Cfg>(in + v * Cfg::kVec, x[u]);
        }
#pragma unroll
        for (int u = 0; u < Cfg::kUnroll; ++u) {
            if (live[u]) {
                const IndexT v = base + (IndexT)u * Cfg::kThreads + threadIdx.x;
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) acc.add(x[u][k], v * Cfg::kVec + k);
            }
        }
    }
    blockReduce<Cfg::kThreads, false>(acc, scratch);
    if (threadIdx.x == 0) {
        if (Cfg::kBlocks == 1) {
            storeResult<Cfg>(acc, 0, valueOut, indexOut, scale);
        } else {
            storePartial<Cfg>(acc, partials, blockIdx.x, Cfg::kBlocks);
        }
    }
}

// One block of kFinishThreads threads folds the kBlocks partials of reduceAll.
template <typename Cfg>
__device__ __forceinline__ void finishAll(const void* partials, void* valueOut, void* indexOut, float scale) {
    typedef typename Cfg::Acc Acc;
    __shared__ Acc scratch[Cfg::kFinishThreads / kWave];
    Acc total;
    total.reset();
    for (u32 b = threadIdx.x; b < (u32)Cfg::kBlocks; b += Cfg::kFinishThreads) total.merge(loadPartial<Cfg>(partials, b, Cfg::kBlocks));
    blockReduce<Cfg::kFinishThreads, false>(total, scratch);
    if (threadIdx.x == 0) storeResult<Cfg>(total, 0, valueOut, indexOut, scale);
}

// ---- contiguous rows: [kOuter, kR] -> [kOuter] ----------------------------------------------------------------------------
// Cfg: kOuter, kR, kThreadsPerRow (power of two; <= 64: kThreads / kThreadsPerRow rows per block, else one row per block
// and kThreads == kThreadsPerRow), kSplit (row segments; 1 = whole row).  With kSplit > 1 the block at (x = row,
// y = segment) writes a partial and finishPartials folds them.
template <typename Cfg>
__device__ __forceinline__ void reduceRows(const typename Cfg::In* in, void* valueOut, void* indexOut, void* partials, float scale) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    constexpr int TPR = Cfg::kThreadsPerRow;
    constexpr bool kSubWave = TPR <= kWave;
    constexpr int kRowsPerBlock = kSubWave ? Cfg::kThreads / TPR : 1;
    constexpr u64 kVectorsPerRow = Cfg::kR / Cfg::kVec;
    constexpr u64 kVectorsPerSegment = (kVectorsPerRow + Cfg::kSplit - 1) / Cfg::kSplit;
    constexpr u64 kIters = (kVectorsPerSegment + TPR - 1) / TPR;

    u64 row;
    int lane;
    if (kSubWave) {
        row = (u64)blockIdx.x * kRowsPerBlock + threadIdx.x / TPR;
        lane = threadIdx.x % TPR;
    } else {
        row = blockIdx.x;
        lane = threadIdx.x;
    }
    const u64 segment = Cfg::kSplit > 1 ? blockIdx.y : 0;
    const u64 vBegin = segment * kVectorsPerSegment;
    const u64 vEnd = (vBegin + kVectorsPerSegment < kVectorsPerRow) ? vBegin + kVectorsPerSegment : kVectorsPerRow;
    const bool rowLive = row < Cfg::kOuter;
    const typename Cfg::In* rowPtr = in + (rowLive ? row : 0) * Cfg::kR;

    Acc acc;
    acc.reset();
    constexpr int kBatch = kIters >= 8 ? 8 : (int)(kIters > 0 ? kIters : 1);
    for (u64 it = 0; it < kIters; it += kBatch) {
        float x[kBatch][Cfg::kVec];
        bool live[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const u64 v = vBegin + (it + u) * TPR + lane;
            live[u] = rowLive && v < vEnd;
            if (live[u]) loadAsFloat<Cfg>(rowPtr + v * Cfg::kVec, x[u]);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (live[u]) {
                const u64 v = vBegin + (it + u) * TPR + lane;
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) acc.add(x[u][k], (IndexT)(v * Cfg::kVec + k));
            }
        }
    }
    if (kSubWave) {
        groupReduce<TPR>(acc);
    } else {
        __shared__ Acc scratch[Cfg::kThreads / kWave];
        blockReduce<Cfg::kThreads, false>(acc, scratch);
    }
    if (lane == 0 && rowLive) {
        if (Cfg::kSplit > 1) {
            storePartial<Cfg>(acc, partials, row * Cfg::kSplit + segment, Cfg::kOuter * Cfg::kSplit);
        } else {
            storeResult<Cfg>(acc, row, valueOut, indexOut, scale);
        }
    }
}

// ---- middle axis: [kOuter, kR, kInner] -> [kOuter, kInner] ------------------------------------------------------------------
// One thread owns kVec adjacent inner positions and walks its share of the kR rows; adjacent threads read adjacent
// memory.  Cfg: kOuter, kR, kInner, kSplit (shares of kR, grid y), kOutOuterStride / kOutInnerStride (output layout).
template <typename Cfg>
__device__ __forceinline__ void reduceColumns(const typename Cfg::In* in, void* valueOut, void* indexOut, void* partials, float scale) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    constexpr u64 kInnerVectors = Cfg::kInner / Cfg::kVec;
    constexpr u64 kColumns = Cfg::kOuter * kInnerVectors;
    constexpr u64 kRowsPerShare = (Cfg::kR + Cfg::kSplit - 1) / Cfg::kSplit;
    const u64 column = (u64)blockIdx.x * Cfg::kThreads + threadIdx.x;
    if (column >= kColumns) return;
    const u64 outer = column / kInnerVectors, iv = column % kInnerVectors;
    const u64 share = Cfg::kSplit > 1 ? blockIdx.y : 0;
    const u64 rBegin = share * kRowsPerShare;
    const u64 rEnd = (rBegin + kRowsPerShare < Cfg::kR) ? rBegin + kRowsPerShare : Cfg::kR;
    const typename Cfg::In* base = in + outer * Cfg::kR * Cfg::kInner + iv * Cfg::kVec;

    Acc acc[Cfg::kVec];
#pragma unroll
    for (int k = 0; k < Cfg::kVec; ++k) acc[k].reset();
    constexpr int kBatch = 4;
    for (u64 r = rBegin; r < rEnd; r += kBatch) {
        float x[kBatch][Cfg::kVec];
#pragma unroll
        for (int u = 0; u < kBatch; ++u)
            if (r + u < rEnd) loadAsFloat<Cfg>(base + (r + u) * Cfg::kInner, x[u]);
#pragma unroll
        for (int u = 0; u < kBatch; ++u)
            if (r + u < rEnd) {
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) acc[k].add(x[u][k], (IndexT)(r + u));
            }
    }
#pragma unroll
    for (int k = 0; k < Cfg::kVec; ++k) {
        const u64 inner = iv * Cfg::kVec + k;
        if (Cfg::kSplit > 1) {
            const u64 logical = outer * Cfg::kInner + inner;
            storePartial<Cfg>(acc[k], partials, logical * Cfg::kSplit + share, Cfg::kOuter * Cfg::kInner * Cfg::kSplit);
        } else {
            storeResult<Cfg>(acc[k], outer * Cfg::kOutOuterStride + inner * Cfg::kOutInnerStride, valueOut, indexOut, scale);
        }
    }
}

// ---- arbitrary kept / reduced axes, dense or strided -------------------------------------------------------------------------
// Cfg: keptOffset(output) and reducedOffset(r) -- generated straight-line address arithmetic over the collapsed kept /
// reduced axes (the innermost reduced axis is counted in vectors of kVec when it is contiguous) -- kOutputs, kReduction
// (vector count of the reduction domain), kSplit (shares of the reduction domain, grid y; outputs on grid x).
template <typename Cfg>
__device__ __forceinline__ void reduceStrided(const typename Cfg::In* in, void* valueOut, void* indexOut, void* partials, float scale) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    constexpr u64 kPerShare = (Cfg::kReduction + Cfg::kSplit - 1) / Cfg::kSplit;
    const u64 output = blockIdx.x;
    const u64 share = blockIdx.y;
    const u64 rBegin = share * kPerShare;
    const u64 rEnd = (rBegin + kPerShare < Cfg::kReduction) ? rBegin + kPerShare : Cfg::kReduction;
    const typename Cfg::In* base = in + Cfg::keptOffset(output);
    __shared__ Acc scratch[Cfg::kThreads / kWave];

    Acc acc;
    acc.reset();
    constexpr int kBatch = 4;
    for (u64 r0 = rBegin + threadIdx.x; r0 < rEnd; r0 += (u64)Cfg::kThreads * kBatch) {
        float x[kBatch][Cfg::kVec];
        bool live[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const u64 r = r0 + (u64)u * Cfg::kThreads;
            live[u] = r < rEnd;
            if (live[u]) loadAsFloat<Cfg>(base + Cfg::reducedOffset(r), x[u]);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (live[u]) {
                const u64 r = r0 + (u64)u * Cfg::kThreads;
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) acc.add(x[u][k], (IndexT)(r * Cfg::kVec + k));
            }
        }
    }
    blockReduce<Cfg::kThreads, false>(acc, scratch);
    if (threadIdx.x == 0) {
        if (Cfg::kSplit > 1) {
            storePartial<Cfg>(acc, partials, output * Cfg::kSplit + share, Cfg::kOutputs * Cfg::kSplit);
        } else {
            storeResult<Cfg>(acc, output, valueOut, indexOut, scale);
        }
    }
}

// ---- second stage of the split kernels: [kOutputs, kSplit] partials -> [kOutputs] -------------------------------------------
// One wavefront per output.  Cfg: kOutputs, kSplit, kFinishOuterStride/kFinishInnerStride/kFinishInner (output layout:
// logical index o = outer * kFinishInner + inner is stored at outer * kFinishOuterStride + inner * kFinishInnerStride).
template <typename Cfg>
__device__ __forceinline__ void finishPartials(const void* partials, void* valueOut, void* indexOut, float scale) {
    typedef typename Cfg::Acc Acc;
    const u64 output = ((u64)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    const int lane = threadIdx.x % kWave;
    const bool live = output < Cfg::kOutputs;
    Acc acc;
    acc.reset();
    if (live) {
        for (u64 s = lane; s < Cfg::kSplit; s += kWave) acc.merge(loadPartial<Cfg>(partials, output * Cfg::kSplit + s, Cfg::kOutputs * Cfg::kSplit));
    }
    groupReduce<kWave>(acc);
    if (live && lane == 0) {
        const u64 outer = output / Cfg::kFinishInner, inner = output % Cfg::kFinishInner;
        storeResult<Cfg>(acc, outer * Cfg::kFinishOuterStride + inner * Cfg::kFinishInnerStride, valueOut, indexOut, scale);
    }
}

}  // namespace thor
