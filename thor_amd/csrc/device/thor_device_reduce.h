// Reduction kernels for gfx950, instantiated by generated code through a `Cfg` traits struct (appended after the device
// prelude at run-time compilation).  They replace cub::DeviceReduce / DeviceSegmentedReduce and the reference's tiled
// kernels (Utilities/TensorOperations/Cub/CubReductionOperation.cuh:2482-3054, CubArgReductionOperation.cuh:1054-1186).
//
// One kernel may reduce several values at once from several tensors of the same layout: the generated Cfg describes
// what is read at an element offset, how the loaded words turn into the values that are accumulated (an elementwise
// prologue evaluated in registers), and where the results go.  Cfg provides
//   Sources                       the tensors (and by-value scalars) the prologue reads
//   Loaded                        the words loaded for one vector position: Cfg::load(sources, elementOffset, loaded)
//   Acc                           ValueAcc<Op>, ArgAcc<IS_MAX, IndexT> or a generated struct of several ValueAcc members with
//                                 the same protocol (reset, merge, shuffleXor, storePartial, loadPartial, partialBytes)
//   Kept, loadKept(sources, outputSlot, kept)       values that depend only on the output (per-channel scale, scalars)
//   accumulateOne(acc, loaded, sources, kept, k, index)   evaluates element k of a loaded vector and adds it under `index`
//   elementwise<KS>(sources, outputs, offset, loaded, kept)   optional same-shaped outputs computed from the loaded vector
//                                 and stored at the same offset (element k uses kept[k * KS])
//   Outputs, store(acc, outIndex, outputs, scale)   finalises (mean divide, L2 square root), scales, converts, stores
//   IndexT                        u32 or u64: type of element offsets and of arg indices inside the kernel
//   kVec                          elements per vector load (all shapes and base addresses are multiples of it)
//   kThreads                      threads per block
// plus the geometry constants each kernel names below.  Shapes are compile-time constants: trip counts are known, loops
// unroll, and every divide is a divide by a constant.
#pragma once

namespace thor {

// ---- whole tensor -> one value ------------------------------------------------------------------------------------------
// Cfg: kN (elements), kUnroll (vectors in flight per thread), kBlocks (grid size).
// Each block folds a block-strided set of chunks into one partial; finishAll (a second, single-block launch) folds the
// partials.  A single-launch variant in which the last block to finish (atomic ticket after a device-scope fence) does
// the final fold was measured at 1.98 ms for 2^26 fp32 elements on MI355X against 0.04 ms for the streaming part alone:
// a device-scope release per block has to write back a non-coherent per-XCD L2, and 16 384 tickets serialise on one
// address.  Two launches cost a few microseconds.
template <typename Cfg>
__device__ __forceinline__ void reduceAll(const typename Cfg::Sources& src, const typename Cfg::Outputs& out, void* partials, float scale) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    constexpr IndexT kVectors = (IndexT)(Cfg::kN / Cfg::kVec);
    constexpr IndexT kChunk = (IndexT)Cfg::kThreads * Cfg::kUnroll;
    __shared__ Acc scratch[Cfg::kThreads / kWave];
    Acc acc;
    acc.reset();
    typename Cfg::Kept kept;
    Cfg::loadKept(src, 0, kept);
    for (IndexT base = (IndexT)blockIdx.x * kChunk; base < kVectors; base += (IndexT)Cfg::kBlocks * kChunk) {
        typename Cfg::Loaded x[Cfg::kUnroll];
        bool live[Cfg::kUnroll];
#pragma unroll
        for (int u = 0; u < Cfg::kUnroll; ++u) {
            const IndexT v = base + (IndexT)u * Cfg::kThreads + threadIdx.x;
            live[u] = v < kVectors;
            if (live[u]) Cfg::load(src, (u64)v * Cfg::kVec, x[u]);
        }
#pragma unroll
        for (int u = 0; u < Cfg::kUnroll; ++u) {
            if (live[u]) {
                const IndexT v = base + (IndexT)u * Cfg::kThreads + threadIdx.x;
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) Cfg::accumulateOne(acc, x[u], src, kept, k, (IndexT)(v * Cfg::kVec + k));
                Cfg::template elementwise<0>(src, out, (u64)v * Cfg::kVec, x[u], &kept);
            }
        }
    }
    blockReduce<Cfg::kThreads, false>(acc, scratch);
    if (threadIdx.x == 0) {
        if (Cfg::kBlocks == 1) {
            Cfg::store(acc, 0, out, scale);
        } else {
            acc.storePartial(partials, blockIdx.x, Cfg::kBlocks);
        }
    }
}

// One block of kFinishThreads threads folds the kBlocks partials of reduceAll.
template <typename Cfg>
__device__ __forceinline__ void finishAll(const void* partials, const typename Cfg::Outputs& out, float scale) {
    typedef typename Cfg::Acc Acc;
    __shared__ Acc scratch[Cfg::kFinishThreads / kWave];
    Acc total;
    total.reset();
    for (u32 b = threadIdx.x; b < (u32)Cfg::kBlocks; b += Cfg::kFinishThreads) {
        Acc part;
        part.loadPartial(partials, b, Cfg::kBlocks);
        total.merge(part);
    }
    blockReduce<Cfg::kFinishThreads, false>(total, scratch);
    if (threadIdx.x == 0) Cfg::store(total, 0, out, scale);
}

// ---- contiguous rows: [kOuter, kR] -> [kOuter] ----------------------------------------------------------------------------
// Cfg: kOuter, kR, kThreadsPerRow (power of two; <= 64: kThreads / kThreadsPerRow rows per block, else one row per block
// and kThreads == kThreadsPerRow), kSplit (row segments; 1 = whole row).  With kSplit > 1 the block at (x = row,
// y = segment) writes a partial and finishPartials folds them.
template <typename Cfg>
__device__ __forceinline__ void reduceRows(const typename Cfg::Sources& src, const typename Cfg::Outputs& out, void* partials, float scale) {
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
    const u64 rowBase = (rowLive ? row : 0) * Cfg::kR;

    Acc acc;
    acc.reset();
    typename Cfg::Kept kept;
    Cfg::loadKept(src, rowLive ? row : 0, kept);
    constexpr int kBatch = kIters >= 8 ? 8 : (int)(kIters > 0 ? kIters : 1);
    for (u64 it = 0; it < kIters; it += kBatch) {
        typename Cfg::Loaded x[kBatch];
        bool live[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const u64 v = vBegin + (it + u) * TPR + lane;
            live[u] = rowLive && v < vEnd;
            if (live[u]) Cfg::load(src, rowBase + v * Cfg::kVec, x[u]);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (live[u]) {
                const u64 v = vBegin + (it + u) * TPR + lane;
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) Cfg::accumulateOne(acc, x[u], src, kept, k, (IndexT)(v * Cfg::kVec + k));
                Cfg::template elementwise<0>(src, out, rowBase + v * Cfg::kVec, x[u], &kept);
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
            acc.storePartial(partials, row * Cfg::kSplit + segment, Cfg::kOuter * Cfg::kSplit);
        } else {
            Cfg::store(acc, row, out, scale);
        }
    }
}

// ---- lanes across outputs: [kOuter, kR, kInner] -> [kOuter, kInner], and views whose kept axis is the contiguous one --------
// A column is kVec outputs that are adjacent in memory; adjacent lanes own adjacent columns, so a wavefront reads up to
// 1 KiB of contiguous memory per step of the reduction.  A block is kLanesX columns wide and kThreads / kLanesX row
// groups deep: row group g of share s walks reduction positions rBegin + g, rBegin + g + groups, ...; the groups are
// then folded through LDS, so the depth adds parallelism without adding partials.
// Cfg: kColumns, kR (reduction positions), kLanesX (power of two <= 64), kBatch (positions in flight per thread), kSplit
// (shares of kR, grid y), and the generated address functions columnBase(column), rowOffset(r), outputIndex(column, k)
// (where element k of the column is stored) and partialSlot(column, k) (its row-major output number).
template <typename Cfg>
__device__ __forceinline__ void reduceColumns(const typename Cfg::Sources& src, const typename Cfg::Outputs& out, void* partials, float scale) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    constexpr u64 kRowsPerShare = (Cfg::kR + Cfg::kSplit - 1) / Cfg::kSplit;
    constexpr int kGroups = Cfg::kThreads / Cfg::kLanesX;
    constexpr int kBatch = Cfg::kBatch;
    const int lx = threadIdx.x % Cfg::kLanesX, group = threadIdx.x / Cfg::kLanesX;
    const u64 column = (u64)blockIdx.x * Cfg::kLanesX + lx;
    const bool columnLive = column < Cfg::kColumns;
    const u64 safeColumn = columnLive ? column : 0;
    const u64 share = Cfg::kSplit > 1 ? blockIdx.y : 0;
    const u64 rBegin = share * kRowsPerShare;
    const u64 rEnd = (rBegin + kRowsPerShare < Cfg::kR) ? rBegin + kRowsPerShare : Cfg::kR;
    const u64 base = Cfg::columnBase(safeColumn);

    Acc acc[Cfg::kVec];
    typename Cfg::Kept kept[Cfg::kVec];
#pragma unroll
    for (int k = 0; k < Cfg::kVec; ++k) {
        acc[k].reset();
        Cfg::loadKept(src, Cfg::partialSlot(safeColumn, k), kept[k]);
    }
    for (u64 r0 = rBegin + group; r0 < rEnd; r0 += (u64)kGroups * kBatch) {
        typename Cfg::Loaded x[kBatch];
        bool live[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const u64 r = r0 + (u64)u * kGroups;
            live[u] = columnLive && r < rEnd;
            if (live[u]) Cfg::load(src, base + Cfg::rowOffset(r), x[u]);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (live[u]) {
                const u64 r = r0 + (u64)u * kGroups;
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) Cfg::accumulateOne(acc[k], x[u], src, kept[k], k, (IndexT)r);
                Cfg::template elementwise<1>(src, out, base + Cfg::rowOffset(r), x[u], kept);
            }
        }
    }
    if (kGroups > 1) {
        // fold the row groups: group g > 0 parks its accumulators, group 0 merges them in group order
        __shared__ Acc parked[(kGroups > 1 ? kGroups - 1 : 1) * Cfg::kLanesX * Cfg::kVec];
        if (group > 0) {
#pragma unroll
            for (int k = 0; k < Cfg::kVec; ++k) parked[((group - 1) * Cfg::kLanesX + lx) * Cfg::kVec + k] = acc[k];
        }
        __syncthreads();
        if (group == 0) {
            for (int g = 1; g < kGroups; ++g) {
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) acc[k].merge(parked[((g - 1) * Cfg::kLanesX + lx) * Cfg::kVec + k]);
            }
        }
    }
    if (group != 0 || !columnLive) return;
#pragma unroll
    for (int k = 0; k < Cfg::kVec; ++k) {
        if (Cfg::kSplit > 1) {
            acc[k].storePartial(partials, Cfg::partialSlot(column, k) * Cfg::kSplit + share, Cfg::kOutputs * Cfg::kSplit);
        } else {
            Cfg::store(acc[k], Cfg::outputIndex(column, k), out, scale);
        }
    }
}

// ---- arbitrary kept / reduced axes, dense or strided -------------------------------------------------------------------------
// Cfg: keptOffset(output) and reducedOffset(r) -- generated straight-line address arithmetic over the collapsed kept /
// reduced axes (the innermost reduced axis is counted in vectors of kVec when it is contiguous) -- kOutputs, kReduction
// (vector count of the reduction domain), kSplit (shares of the reduction domain, grid y; outputs on grid x).
template <typename Cfg>
__device__ __forceinline__ void reduceStrided(const typename Cfg::Sources& src, const typename Cfg::Outputs& out, void* partials, float scale) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    constexpr u64 kPerShare = (Cfg::kReduction + Cfg::kSplit - 1) / Cfg::kSplit;
    const u64 output = blockIdx.x;
    const u64 share = blockIdx.y;
    const u64 rBegin = share * kPerShare;
    const u64 rEnd = (rBegin + kPerShare < Cfg::kReduction) ? rBegin + kPerShare : Cfg::kReduction;
    const u64 base = Cfg::keptOffset(output);
    __shared__ Acc scratch[Cfg::kThreads / kWave];

    Acc acc;
    acc.reset();
    typename Cfg::Kept kept;
    Cfg::loadKept(src, output, kept);
    constexpr int kBatch = 4;
    for (u64 r0 = rBegin + threadIdx.x; r0 < rEnd; r0 += (u64)Cfg::kThreads * kBatch) {
        typename Cfg::Loaded x[kBatch];
        bool live[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const u64 r = r0 + (u64)u * Cfg::kThreads;
            live[u] = r < rEnd;
            if (live[u]) Cfg::load(src, base + Cfg::reducedOffset(r), x[u]);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (live[u]) {
                const u64 r = r0 + (u64)u * Cfg::kThreads;
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) Cfg::accumulateOne(acc, x[u], src, kept, k, (IndexT)(r * Cfg::kVec + k));
                Cfg::template elementwise<0>(src, out, base + Cfg::reducedOffset(r), x[u], &kept);
            }
        }
    }
    blockReduce<Cfg::kThreads, false>(acc, scratch);
    if (threadIdx.x == 0) {
        if (Cfg::kSplit > 1) {
            acc.storePartial(partials, output * Cfg::kSplit + share, Cfg::kOutputs * Cfg::kSplit);
        } else {
            Cfg::store(acc, output, out, scale);
        }
    }
}

// ---- second stage of the split kernels: [kOutputs, kSplit] partials -> [kOutputs] -------------------------------------------
// One wavefront per output.  Cfg: kOutputs, kSplit, kFinishOuterStride/kFinishInnerStride/kFinishInner (output layout:
// logical index o = outer * kFinishInner + inner is stored at outer * kFinishOuterStride + inner * kFinishInnerStride).
template <typename Cfg>
__device__ __forceinline__ void finishPartials(const void* partials, const typename Cfg::Outputs& out, float scale) {
    typedef typename Cfg::Acc Acc;
    const u64 output = ((u64)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    const int lane = threadIdx.x % kWave;
    const bool live = output < Cfg::kOutputs;
    Acc acc;
    acc.reset();
    if (live) {
        for (u64 s = lane; s < Cfg::kSplit; s += kWave) {
            Acc part;
            part.loadPartial(partials, output * Cfg::kSplit + s, Cfg::kOutputs * Cfg::kSplit);
            acc.merge(part);
        }
    }
    groupReduce<kWave>(acc);
    if (live && lane == 0) {
        const u64 outer = output / Cfg::kFinishInner, inner = output % Cfg::kFinishInner;
        Cfg::store(acc, outer * Cfg::kFinishOuterStride + inner * Cfg::kFinishInnerStride, out, scale);
    }
}

}  // namespace thor
