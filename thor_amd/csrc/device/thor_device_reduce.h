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

// ---- finishing inside the launch that made the partials ---------------------------------------------------------------------
// With Cfg::kTickets the blocks that share an output count themselves in on a ticket word (one u32 per output group, in
// the workspace at byte Cfg::kTicketOffset, zero between launches) after their partials are out; the block that counts in
// last folds the partials and stores the result, so no second launch is needed.  Partials are device-wide words
// (storeDeviceWide / loadDeviceWide: they pass the per-XCD L2), so a thread that stored one only waits for its stores
// to be acknowledged (partialsWritten) before the block's barrier; thread 0 then takes the ticket with a device-scope
// atomic, and the last block reads the partials without any cache maintenance.  (A release / acquire fence pair does
// the same by writing back and invalidating the whole L2 of the XCD: measured 180 us instead of 20 us for the 4096
// blocks of a per-channel sum.)  The fold walks the partials in their fixed order, never in arrival order, so results
// are reproducible bit for bit; the folding block resets the ticket, which nobody else touches any more in this launch,
// so a stamped plan can run again without a clear.
template <typename Cfg>
__device__ __forceinline__ bool lastToArrive(void* partials, u64 ticket, u32 arrivals) {
    __shared__ u32 last;
    __syncthreads();
    if (threadIdx.x == 0) {
        u32* word = reinterpret_cast<u32*>(static_cast<char*>(partials) + Cfg::kTicketOffset) + ticket;
        const u32 before = __hip_atomic_fetch_add(word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last = before + 1u == arrivals ? 1u : 0u;
        if (last) storeDeviceWide(word, 0u);
    }
    __syncthreads();
    return last != 0u;
}

// The fold of one output's kSplit partials by one wavefront, in share order; lane 0 stores.  `lane` in [0, 64).
template <typename Cfg>
__device__ __forceinline__ void foldShares(const void* partials, u64 output, const typename Cfg::Outputs& out, float scale, int lane) {
    typedef typename Cfg::Acc Acc;
    Acc acc;
    acc.reset();
    for (u64 s = lane; s < Cfg::kSplit; s += kWave) {
        Acc part;
        part.template loadPartial<Cfg::kTickets>(partials, output * Cfg::kSplit + s, Cfg::kOutputs * Cfg::kSplit);
        acc.merge(part);
    }
    groupReduce<kWave>(acc);
    if (lane == 0) {
        const u64 outer = output / Cfg::kFinishInner, inner = output % Cfg::kFinishInner;
        Cfg::store(acc, outer * Cfg::kFinishOuterStride + inner * Cfg::kFinishInnerStride, out, scale);
    }
}

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
    const u32 block = xcdBlock<Cfg::kXcdRun>(blockIdx.x, gridDim.x);
    for (IndexT base = (IndexT)block * kChunk; base < kVectors; base += (IndexT)Cfg::kBlocks * kChunk) {
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
            acc.template storePartial<Cfg::kTickets>(partials, block, Cfg::kBlocks);
            if (Cfg::kTickets) partialsWritten();
        }
    }
    if (Cfg::kTickets && Cfg::kBlocks > 1) {
        if (!lastToArrive<Cfg>(partials, 0, (u32)Cfg::kBlocks)) return;
        __shared__ Acc finishScratch[Cfg::kThreads / kWave];
        Acc total;
        total.reset();
        for (u32 b = threadIdx.x; b < (u32)Cfg::kBlocks; b += Cfg::kThreads) {
            Acc part;
            part.template loadPartial<true>(partials, b, Cfg::kBlocks);
            total.merge(part);
        }
        blockReduce<Cfg::kThreads, false>(total, finishScratch);
        if (threadIdx.x == 0) Cfg::store(total, 0, out, scale);
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
    const u32 block = xcdBlock<Cfg::kXcdRun>(blockIdx.x, gridDim.x);
    if (kSubWave) {
        row = (u64)block * kRowsPerBlock + threadIdx.x / TPR;
        lane = threadIdx.x % TPR;
    } else {
        row = block;
        lane = threadIdx.x;
    }
    const u64 segment = Cfg::kSplit > 1 ? blockIdx.y : 0;
    const u64 vBegin = segment * kVectorsPerSegment;
    const u64 vEnd = (vBegin + kVectorsPerSegment < kVectorsPerRow) ? vBegin + kVectorsPerSegment : kVectorsPerRow;
    const bool rowLive = row < Cfg::kOuter;
    const u64 rowBase = (rowLive ? row : 0) * Cfg::kR;

    // kInterleave > 1: the row holds kInterleave outputs element by element ([outer, R, inner] with an inner extent that
    // divides the vector): element e of the row belongs to output e % kInterleave and to reduction position e / kInterleave
    constexpr int J = Cfg::kInterleave;
    static_assert(Cfg::kVec % J == 0 && (J == 1 || Cfg::kSplit == 1), "interleaved outputs: whole groups per vector, rows not split");
    Acc acc[J];
#pragma unroll
    for (int j = 0; j < J; ++j) acc[j].reset();
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
                for (int k = 0; k < Cfg::kVec; ++k) Cfg::accumulateOne(acc[k % J], x[u], src, kept, k, (IndexT)((v * Cfg::kVec + k) / J));
                Cfg::template elementwise<0>(src, out, rowBase + v * Cfg::kVec, x[u], &kept);
            }
        }
    }
    if constexpr (Cfg::kR % Cfg::kVec != 0) {
        // a row length no vector divides (the vectors above were read at unaligned addresses): the rest of the row, one
        // element per lane, by the block that holds the row's last segment
        constexpr u64 kTail = Cfg::kR % Cfg::kVec;
        if (rowLive && segment == (u64)Cfg::kSplit - 1) {
            for (u64 t = (u64)lane; t < kTail; t += TPR) {
                typename Cfg::Loaded x;
                Cfg::loadFirstOnly(src, rowBase + kVectorsPerRow * Cfg::kVec + t, x);
                Cfg::accumulateOne(acc[0], x, src, kept, 0, (IndexT)(kVectorsPerRow * Cfg::kVec + t));
            }
        }
    }
    if (kSubWave) {
#pragma unroll
        for (int j = 0; j < J; ++j) groupReduce<TPR>(acc[j]);
    } else {
        __shared__ Acc scratch[J][Cfg::kThreads / kWave];
#pragma unroll
        for (int j = 0; j < J; ++j) blockReduce<Cfg::kThreads, false>(acc[j], scratch[j]);
    }
    if (lane == 0 && rowLive) {
        if (Cfg::kSplit > 1) {
            acc[0].template storePartial<Cfg::kTickets>(partials, row * Cfg::kSplit + segment, Cfg::kOuter * Cfg::kSplit);
            if (Cfg::kTickets) partialsWritten();
        } else {
#pragma unroll
            for (int j = 0; j < J; ++j) Cfg::store(acc[j], row * J + j, out, scale);
        }
    }
    if (Cfg::kTickets && Cfg::kSplit > 1 && !kSubWave && rowLive) {  // one row per block: the row's last share folds
        if (lastToArrive<Cfg>(partials, row, (u32)Cfg::kSplit) && threadIdx.x < kWave) foldShares<Cfg>(partials, row, out, scale, threadIdx.x);
    }
}

// ---- lanes across outputs: [kOuter, kR, kInner] -> [kOuter, kInner], and views whose kept axis is the contiguous one --------
// A column is kVec outputs that are adjacent in memory; adjacent lanes own adjacent columns, so a wavefront reads up to
// 1 KiB of contiguous memory per step of the reduction.  A block is kLanesX columns wide and kThreads / kLanesX row
// groups deep: row group g of share s walks reduction positions rBegin + g, rBegin + g + groups, ...; the groups are
// then folded through LDS, so the depth adds parallelism without adding partials.
// Cfg: kColumns, kR (reduction positions), kLanesX (<= 64, any width; a power of two for the transposed form), kBatch (positions in flight per thread), kSplit
// (shares of kR, grid y), and the generated address functions columnBase(column), rowOffset(r), outputIndex(column, k)
// (where element k of the column is stored), partialSlot(column, k) (its row-major output number) and ownsElement(column, k)
// (false for the outputs that the last column of an inner extent shares with the one before it, when the vector width does
// not divide the extent: that column is moved back to end with the extent).
template <typename Cfg>
__device__ __forceinline__ void reduceColumns(const typename Cfg::Sources& src, const typename Cfg::Outputs& out, void* partials, float scale) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    constexpr u64 kRowsPerShare = (Cfg::kR + Cfg::kSplit - 1) / Cfg::kSplit;
    constexpr int kGroups = Cfg::kThreads / Cfg::kLanesX;
    constexpr int kBatch = Cfg::kBatch;
    const int lx = threadIdx.x % Cfg::kLanesX, group = threadIdx.x / Cfg::kLanesX;
    const u64 column = (u64)blockIdx.x * Cfg::kLanesX + lx;
    // a width that does not divide the block leaves its last threads without a row group
    const bool columnLive = column < Cfg::kColumns && group < kGroups;
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
        if (group > 0 && group < kGroups) {
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
    if (group == 0 && columnLive) {
#pragma unroll
        for (int k = 0; k < Cfg::kVec; ++k) {
            if (!Cfg::ownsElement(column, k)) continue;  // an output that the column before this one holds as well
            if (Cfg::kSplit > 1) {
                // for a finishing launch the shares of one output lie together; when the last share folds, the outputs of one
                // share do: adjacent lanes then write, and later read, adjacent words
                const u64 slot = Cfg::kTickets ? share * Cfg::kOutputs + Cfg::partialSlot(column, k) : Cfg::partialSlot(column, k) * Cfg::kSplit + share;
                acc[k].template storePartial<Cfg::kTickets>(partials, slot, Cfg::kOutputs * Cfg::kSplit);
            } else {
                Cfg::store(acc[k], Cfg::outputIndex(column, k), out, scale);
            }
        }
        if (Cfg::kTickets && Cfg::kSplit > 1) partialsWritten();
    }
    if (Cfg::kTickets && Cfg::kSplit > 1) {
        // the last share of this block's columns folds them: a thread per output, the shares in their order
        if (!lastToArrive<Cfg>(partials, blockIdx.x, (u32)Cfg::kSplit)) return;
        for (int o = threadIdx.x; o < Cfg::kLanesX * Cfg::kVec; o += Cfg::kThreads) {
            const u64 c = (u64)blockIdx.x * Cfg::kLanesX + o / Cfg::kVec;
            if (c >= Cfg::kColumns || !Cfg::ownsElement(c, o % Cfg::kVec)) continue;
            const u64 output = Cfg::partialSlot(c, o % Cfg::kVec);
            Acc total;
            total.reset();
            // the loads of eight shares are issued together, then merged in share order (all 64 in flight cost the main loop its
            // registers: 60.6 us against 53.9 us for 8192 x 8192 fp32 over axis 0)
            constexpr int kInFlight = Cfg::kSplit < 8 ? (int)Cfg::kSplit : 8;
            for (u64 s0 = 0; s0 < Cfg::kSplit; s0 += kInFlight) {
                Acc part[kInFlight];
#pragma unroll
                for (int j = 0; j < kInFlight; ++j) {
                    part[j].reset();
                    if (s0 + j < Cfg::kSplit) part[j].template loadPartial<true>(partials, (s0 + j) * Cfg::kOutputs + output, Cfg::kOutputs * Cfg::kSplit);
                }
#pragma unroll
                for (int j = 0; j < kInFlight; ++j) total.merge(part[j]);
            }
            const u64 outer = output / Cfg::kFinishInner, inner = output % Cfg::kFinishInner;
            Cfg::store(total, outer * Cfg::kFinishOuterStride + inner * Cfg::kFinishInnerStride, out, scale);
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
    constexpr int kBatch = Cfg::kBatch;
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
            acc.template storePartial<Cfg::kTickets>(partials, output * Cfg::kSplit + share, Cfg::kOutputs * Cfg::kSplit);
            if (Cfg::kTickets) partialsWritten();
        } else {
            Cfg::store(acc, output, out, scale);
        }
    }
    if (Cfg::kTickets && Cfg::kSplit > 1) {
        if (lastToArrive<Cfg>(partials, output, (u32)Cfg::kSplit) && threadIdx.x < kWave) foldShares<Cfg>(partials, output, out, scale, threadIdx.x);
    }
}

// reduceColumns for outputs whose fastest axis is not the one the lanes lie on (a transposed matrix reduced along its rows,
// the [inner, outer] outputs of the reference's tiled kernels: Utilities/TensorOperations/Cub/CubReductionOperation.cuh:
// 2165-2534 there): lanes along the input's contiguous kept axis would scatter single elements over the output.  Here a
// block owns kLanesX * kVec lane positions times kTransposeRows consecutive values of the next kept coordinate q (the
// output's fastest axis); every row group reduces whole columns of its own q values (nothing is folded between threads),
// the results meet in LDS and leave along q: the writes of a block are runs of kTransposeRows adjacent elements.
// Cfg additionally: kTransposeRows, kLaneVectors (vectors along the lane axis), kQ (= kColumns / kLaneVectors); column
// c = q * kLaneVectors + vector.  Only without a split of R.
template <typename Cfg>
__device__ __forceinline__ void reduceColumnsTransposed(const typename Cfg::Sources& src, const typename Cfg::Outputs& out, float scale) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    constexpr int kGroups = Cfg::kThreads / Cfg::kLanesX;
    constexpr int kBatch = Cfg::kBatch;
    constexpr int kRows = Cfg::kTransposeRows, kWidth = Cfg::kLanesX * Cfg::kVec;
    constexpr u64 kTilesPerRow = (Cfg::kLaneVectors + Cfg::kLanesX - 1) / Cfg::kLanesX;
    __shared__ Acc tile[kRows][kWidth + 1];
    const int lx = threadIdx.x % Cfg::kLanesX, group = threadIdx.x / Cfg::kLanesX;
    const u64 firstVector = (blockIdx.x % kTilesPerRow) * Cfg::kLanesX, firstQ = (blockIdx.x / kTilesPerRow) * kRows;
    const bool vectorLive = firstVector + lx < Cfg::kLaneVectors;
    for (int j = group; j < kRows; j += kGroups) {
        const u64 q = firstQ + j;
        if (!vectorLive || q >= Cfg::kQ) continue;
        const u64 column = q * Cfg::kLaneVectors + firstVector + lx;
        const u64 base = Cfg::columnBase(column);
        Acc acc[Cfg::kVec];
        typename Cfg::Kept kept[Cfg::kVec];
#pragma unroll
        for (int k = 0; k < Cfg::kVec; ++k) {
            acc[k].reset();
            Cfg::loadKept(src, Cfg::partialSlot(column, k), kept[k]);
        }
        for (u64 r0 = 0; r0 < Cfg::kR; r0 += kBatch) {
            typename Cfg::Loaded x[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u)
                if (r0 + u < Cfg::kR) Cfg::load(src, base + Cfg::rowOffset(r0 + u), x[u]);
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                if (r0 + u < Cfg::kR) {
#pragma unroll
                    for (int k = 0; k < Cfg::kVec; ++k) Cfg::accumulateOne(acc[k], x[u], src, kept[k], k, (IndexT)(r0 + u));
                    Cfg::template elementwise<1>(src, out, base + Cfg::rowOffset(r0 + u), x[u], kept);
                }
            }
        }
#pragma unroll
        for (int k = 0; k < Cfg::kVec; ++k) tile[j][lx * Cfg::kVec + k] = acc[k];
    }
    __syncthreads();
    for (int slot = threadIdx.x; slot < kRows * kWidth; slot += Cfg::kThreads) {
        const int j = slot % kRows, i = slot / kRows;
        const u64 q = firstQ + j, vector = firstVector + i / Cfg::kVec;
        if (q < Cfg::kQ && vector < Cfg::kLaneVectors) Cfg::store(tile[j][i], Cfg::outputIndex(q * Cfg::kLaneVectors + vector, i % Cfg::kVec), out, scale);
    }
}

// ---- offset-segmented rows: values [N, D] and offsets [B + 1] -> [B, D] ---------------------------------------------------------
// Segment b is the row range [offsets[b], offsets[b + 1]); the offsets are read when the kernels run, so a stamped
// reduction follows whatever partition is in the tensor at that moment (replaces cub::DeviceSegmentedReduce and the
// reference's vector-valued segmented kernels, Utilities/TensorOperations/Cub/CubReductionOffsetSegmented.cu).
//
// Work is split by rows, not by segments, so the load of a block does not depend on the partition.  Three launches:
//   prepareSegments  writes, for every chunk of kChunkRows rows, the first segment that touches it
//   reduceSegments   block (chunk, column tile) hands the pieces [segment ∩ chunk] to teams of threads; the team size is
//                    picked per chunk from the number of pieces: the whole block inside a long segment, teams of
//                    kMinTeam lanes when the chunk holds many short segments.  A piece that is a whole segment is
//                    finalised and stored at once; a piece of a segment that began in an earlier chunk goes to the
//                    chunk's `head` partial, a piece of a segment that continues into the next chunk to its `tail` partial
//   finishSegments   folds tail[c] with head[c + 1 .. c1] for every segment that spans chunks
// Offsets are clamped to the row count, so an invalid partition gives meaningless results but never reads outside the
// values tensor.  An element's index (arg reductions) is its packed position row * kD + d; the candidates carry the row alone
// (every thread, team and partial belongs to one trailing element d, so rows order like positions) and Cfg::store packs it.
// Empty segments keep the accumulator's identity (sum 0, min +inf, max -inf, index all-ones) and a mean over zero rows is 0.
// Workspace: accumulators [kChunks][2][kD]; u64 tails[kChunks] (the segment whose tail the chunk holds, or all-ones);
// u64 firstSegment[kChunks].
// Cfg: kD, kRows, kSegments, kColumnTiles, kLanesX, kBatch, kChunkRows, kChunks, kMinTeam, kFinishLanes, kFinishThreads,
// OffsetT (u32 or u64).
template <typename Cfg>
__device__ __forceinline__ u64 segmentOffset(const typename Cfg::OffsetT* offsets, u64 s) {
    const u64 o = (u64)offsets[s];
    return o < Cfg::kRows ? o : Cfg::kRows;
}

template <typename Cfg>
struct SegmentWorkspace {
    static constexpr u64 kPartialSlots = Cfg::kChunks * 2 * Cfg::kD;
    __device__ __forceinline__ static u64* tails(void* workspace) {
        return reinterpret_cast<u64*>(static_cast<char*>(workspace) + Cfg::Acc::partialBytes(kPartialSlots));
    }
    __device__ __forceinline__ static u64* firstSegment(void* workspace) { return tails(workspace) + Cfg::kChunks; }
};

__device__ __forceinline__ u64 shuffleFrom(u64 v, int sourceLane) {
    const u32 lo = __shfl((u32)(v & 0xffffffffu), sourceLane, kWave);
    const u32 hi = __shfl((u32)(v >> 32), sourceLane, kWave);
    return ((u64)hi << 32) | lo;
}

// firstSegment[c] = the first segment that touches chunk c: the first one that ends after the chunk's first row or begins
// at or after it (an empty segment belongs to the chunk its position lies in); bit 63 is set when that segment began
// before the chunk.  One thread per segment (and one for "no segment") writes the entries of the chunks it is first in:
// with reach(s) = the last row position that still belongs to s (last - 1, or first for an empty segment), those are
// the chunks whose first row lies in (reach(s - 1), reach(s)].  Most threads own no chunk; a long range is written by
// the whole wavefront.  Launched with 256 threads per block over kSegments + 1 threads.
template <typename Cfg>
__device__ __forceinline__ void prepareSegments(void* workspace, const typename Cfg::OffsetT* offsets) {
    constexpr u64 kStraddles = (u64)1 << 63;
    u64* table = SegmentWorkspace<Cfg>::firstSegment(workspace);
    const u64 s = (u64)blockIdx.x * blockDim.x + threadIdx.x;
    const int lane = threadIdx.x % kWave;
    u64 chunkLo = 0, count = 0, first = 0;
    if (s <= Cfg::kSegments) {
        u64 afterPrevious = 0;  // reach(s - 1) + 1
        if (s > 0) {
            const u64 f = segmentOffset<Cfg>(offsets, s - 1), l = segmentOffset<Cfg>(offsets, s);
            afterPrevious = l > f ? l : f + 1;
        }
        u64 chunkEnd = Cfg::kChunks;  // the thread after the last segment takes every chunk that is left
        if (s < Cfg::kSegments) {
            first = segmentOffset<Cfg>(offsets, s);
            const u64 last = segmentOffset<Cfg>(offsets, s + 1);
            const u64 reach = last > first ? last - 1 : first;
            chunkEnd = reach / Cfg::kChunkRows + 1;
            if (chunkEnd > Cfg::kChunks) chunkEnd = Cfg::kChunks;
        } else {
            first = Cfg::kRows;
        }
        chunkLo = (afterPrevious + Cfg::kChunkRows - 1) / Cfg::kChunkRows;
        count = chunkEnd > chunkLo ? chunkEnd - chunkLo : 0;
    }
    if (count <= 4) {
        for (u64 i = 0; i < count; ++i) table[chunkLo + i] = s | (first < (chunkLo + i) * Cfg::kChunkRows ? kStraddles : 0);
    }
    u64 longRanges = __builtin_amdgcn_ballot_w64(count > 4);
    while (longRanges) {
        const int owner = __builtin_ctzll(longRanges);
        longRanges &= longRanges - 1;
        const u64 lo = shuffleFrom(chunkLo, owner), n = shuffleFrom(count, owner), value = shuffleFrom(s, owner), begin = shuffleFrom(first, owner);
        for (u64 i = lane; i < n; i += kWave) table[lo + i] = value | (begin < (lo + i) * Cfg::kChunkRows ? kStraddles : 0);
    }
}

constexpr __device__ int floorLog2(int x) { return x <= 1 ? 0 : 1 + floorLog2(x / 2); }

// Folds the threads of a team of 2^teamBits consecutive threads that share a column (thread-in-team modulo LANES_X):
// shuffles inside a wavefront, then LDS between the wavefronts of a team.  The result is valid in the team's first
// LANES_X threads.  teamBits must be the same for the whole block; `parked` holds THREADS / 64 * LANES_X * VEC accumulators.
template <int THREADS, int LANES_X, int VEC, typename Acc>
__device__ __forceinline__ void teamReduce(Acc (&acc)[VEC], int teamBits, Acc* parked) {
    const int inWave = teamBits < 6 ? (1 << teamBits) : kWave;
    for (int mask = inWave / 2; mask >= LANES_X; mask >>= 1) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[k].merge(acc[k].shuffleXor(mask));
    }
    if (THREADS > kWave && teamBits > 6) {
        const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
        const int wavesPerTeam = 1 << (teamBits - 6);
        const int waveInTeam = wave & (wavesPerTeam - 1);
        if (waveInTeam != 0 && lane < LANES_X) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) parked[(wave * LANES_X + lane) * VEC + k] = acc[k];
        }
        __syncthreads();
        if (waveInTeam == 0 && lane < LANES_X) {
            for (int w = 1; w < wavesPerTeam; ++w) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) acc[k].merge(parked[((wave + w) * LANES_X + lane) * VEC + k]);
            }
        }
        __syncthreads();
    }
}

template <typename Cfg>
__device__ __forceinline__ void reduceSegments(const typename Cfg::Sources& src, const typename Cfg::Outputs& out, void* workspace, float scale,
                                               const typename Cfg::OffsetT* offsets) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    typedef SegmentWorkspace<Cfg> Workspace;
    constexpr u64 kColumnsPerRow = Cfg::kD / Cfg::kVec;
    constexpr int kBatch = Cfg::kBatch;
    constexpr int kThreadBits = floorLog2(Cfg::kThreads);
    constexpr int kMaxTeamBits = kThreadBits - floorLog2(Cfg::kMinTeam);
    __shared__ Acc parked[Cfg::kThreads / kWave * Cfg::kLanesX * Cfg::kVec];

    const u64 chunk = blockIdx.x / Cfg::kColumnTiles, tile = blockIdx.x % Cfg::kColumnTiles;
    const u64 cBegin = chunk * Cfg::kChunkRows;
    const u64 cEnd = cBegin + Cfg::kChunkRows < Cfg::kRows ? cBegin + Cfg::kChunkRows : Cfg::kRows;
    // segments [sLo, sEnd) touch the chunk: from the prepared first one up to the first one that begins at or after the
    // chunk's end, which is the next chunk's first one unless that one began before the boundary; the last chunk also
    // takes the empty segments at the very end
    u64 sLo = 0, sEnd = Cfg::kSegments;
    if (Cfg::kChunks > 1) {
        constexpr u64 kStraddles = (u64)1 << 63;
        sLo = Workspace::firstSegment(workspace)[chunk] & ~kStraddles;
        if (sLo > Cfg::kSegments) sLo = Cfg::kSegments;
        if (chunk + 1 < Cfg::kChunks) {
            const u64 entry = Workspace::firstSegment(workspace)[chunk + 1];
            sEnd = (entry & ~kStraddles) + (entry >> 63);
            if (sEnd > Cfg::kSegments) sEnd = Cfg::kSegments;
        }
    }
    const u64 pieces = sEnd > sLo ? sEnd - sLo : 0;

    // one team per piece: as many teams as pieces (a power of two), teams never smaller than kMinTeam threads
    int teamCountBits = 0;
    while (teamCountBits < kMaxTeamBits && (u64)(1u << teamCountBits) < pieces) ++teamCountBits;
    const int teamBits = kThreadBits - teamCountBits;
    const u64 team = threadIdx.x >> teamBits;
    const int inTeam = threadIdx.x & ((1 << teamBits) - 1);
    const int lx = inTeam % Cfg::kLanesX;
    const u64 rowLane = inTeam / Cfg::kLanesX, rowLanes = (u64)(1 << teamBits) / Cfg::kLanesX;
    const u64 column = tile * Cfg::kLanesX + lx;
    const bool columnLive = column < kColumnsPerRow;
    const u64 columnOffset = (columnLive ? column : 0) * Cfg::kVec;  // dead lanes read column 0 and store nothing
    const u64 teams = (u64)(1u << teamCountBits);
    const u64 passes = shiftRightBelow32(pieces + teams - 1, (u32)teamCountBits);

    for (u64 pass = 0; pass < passes; ++pass) {
        const u64 segment = sLo + pass * teams + team;
        const bool pieceLive = segment < sEnd;
        u64 first = 0, last = 0;
        if (pieceLive) {
            first = segmentOffset<Cfg>(offsets, segment);
            last = segmentOffset<Cfg>(offsets, segment + 1);
            if (last < first) last = first;
        }
        const u64 pBegin = first > cBegin ? first : cBegin;
        const u64 pEnd = last < cEnd ? last : cEnd;

        Acc acc[Cfg::kVec];
        typename Cfg::Kept kept[Cfg::kVec];  // per-output operands: one element per (segment, trailing element)
#pragma unroll
        for (int k = 0; k < Cfg::kVec; ++k) {
            Cfg::loadKept(src, (pieceLive ? segment : 0) * Cfg::kD + columnOffset + k, kept[k]);
            acc[k].reset();
        }
        for (u64 r0 = pBegin + rowLane; r0 < pEnd; r0 += rowLanes * kBatch) {
            typename Cfg::Loaded x[kBatch];
            if (r0 + (u64)(kBatch - 1) * rowLanes < pEnd) {
#pragma unroll
                for (int u = 0; u < kBatch; ++u) Cfg::load(src, (r0 + (u64)u * rowLanes) * Cfg::kD + columnOffset, x[u]);
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const IndexT row = (IndexT)(r0 + (u64)u * rowLanes);
#pragma unroll
                    for (int k = 0; k < Cfg::kVec; ++k) Cfg::accumulateOne(acc[k], x[u], src, kept[k], k, row);
                }
            } else {
                bool live[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const u64 r = r0 + (u64)u * rowLanes;
                    live[u] = r < pEnd;
                    if (live[u]) Cfg::load(src, r * Cfg::kD + columnOffset, x[u]);
                }
                // (selects over re-read rows instead of these branches measured 15-25 % slower for sums of short segments)
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    if (live[u]) {
                        const IndexT row = (IndexT)(r0 + (u64)u * rowLanes);
#pragma unroll
                        for (int k = 0; k < Cfg::kVec; ++k) Cfg::accumulateOne(acc[k], x[u], src, kept[k], k, row);
                    }
                }
            }
        }
        teamReduce<Cfg::kThreads, Cfg::kLanesX, Cfg::kVec>(acc, teamBits, parked);
        if (pieceLive && rowLane == 0 && columnLive) {
#pragma unroll
            for (int k = 0; k < Cfg::kVec; ++k) {
                const u64 d = column * Cfg::kVec + k;
                if (first < cBegin) {
                    acc[k].storePartial(workspace, (chunk * 2 + 0) * Cfg::kD + d, Workspace::kPartialSlots);
                } else if (last > cEnd) {
                    acc[k].storePartial(workspace, (chunk * 2 + 1) * Cfg::kD + d, Workspace::kPartialSlots);
                } else {
                    Cfg::store(acc[k], segment * Cfg::kD + d, out, scale, toFloat((u64)(last - first)));
                }
            }
        }
    }
    if (Cfg::kChunks > 1 && tile == 0 && threadIdx.x == 0) {
        u64 tailSegment = ~(u64)0;
        if (pieces > 0) {
            const u64 first = segmentOffset<Cfg>(offsets, sEnd - 1), last = segmentOffset<Cfg>(offsets, sEnd);
            if (first >= cBegin && first < cEnd && last > cEnd) tailSegment = sEnd - 1;
        }
        Workspace::tails(workspace)[chunk] = tailSegment;
    }
}

// The same chunks, partials and finishing launch with the work dealt out by rows instead of by segments: thread
// (row lane, column) owns kBatch consecutive rows of the chunk and issues all of their loads before it knows where the
// segments lie, so the data in flight depends on neither the partition nor the offsets' latency, and every thread does the same
// amount of work whatever the lengths are.  The chunk's offsets are staged in LDS meanwhile.  A thread then walks its
// rows run by run (a run = the rows of one segment inside the thread's range):
//   * a segment that begins and ends inside the range is finalised and stored by the thread itself;
//   * the first run, when its segment began before the range, is parked as the thread's `head`; the last run, when its
//     segment goes on after the range, as its `tail` (a range in the middle of a long segment has only a tail);
//   * one row of threads then goes over the row lanes in order, folding tails into heads: segments that end here are stored
//     (or go to the chunk's head partial when they began in an earlier chunk), what is left is the chunk's tail partial.
// Empty segments are stored (identity) by the thread that owns the row before their position; those at position 0 by the
// first thread of the first chunk.  Rows outside every segment are skipped.  Meant for segments of kBatch rows or more on
// average: the rows are walked kWalkGroup at a time, and a group is walked once per segment that touches it.  (Resident
// blocks that stride over the chunks measured slower than one block per chunk: a block's loads, walk and fold do not overlap.)
// Cfg as for reduceSegments; kChunkRows == kThreads / kLanesX * kBatch.
template <typename Cfg>
__device__ __forceinline__ void reduceSegmentsByRows(const typename Cfg::Sources& src, const typename Cfg::Outputs& out, void* workspace, float scale,
                                                     const typename Cfg::OffsetT* offsets) {
    typedef typename Cfg::IndexT IndexT;
    typedef typename Cfg::Acc Acc;
    typedef SegmentWorkspace<Cfg> Workspace;
    constexpr u64 kColumnsPerRow = Cfg::kD / Cfg::kVec;
    constexpr int kBatch = Cfg::kBatch;
    constexpr int kGroup = kBatch < Cfg::kWalkGroup ? kBatch : Cfg::kWalkGroup;  // rows walked together: a run costs a pass over the groups it touches
    constexpr int kRowLanes = Cfg::kThreads / Cfg::kLanesX;
    constexpr int kWindow = Cfg::kThreads;  // offsets staged per chunk: kWindow + 1
    constexpr u64 kNone = ~(u64)0;
    static_assert(Cfg::kChunkRows == (u64)kRowLanes * kBatch, "a chunk is one range of rows per row lane");
    __shared__ u64 bounds[kWindow + 1];
    __shared__ Acc heads[kRowLanes * Cfg::kLanesX * Cfg::kVec];
    __shared__ Acc tails[kRowLanes * Cfg::kLanesX * Cfg::kVec];
    __shared__ u64 headSegment[kRowLanes];
    __shared__ u64 tailSegment[kRowLanes];

    const int lx = threadIdx.x % Cfg::kLanesX;
    const int rowLane = threadIdx.x / Cfg::kLanesX;
    const int slot = (rowLane * Cfg::kLanesX + lx) * Cfg::kVec;

    {
        const u64 chunk = blockIdx.x / Cfg::kColumnTiles, tile = blockIdx.x % Cfg::kColumnTiles;
        const u64 cBegin = chunk * Cfg::kChunkRows;
        const u64 cEnd = cBegin + Cfg::kChunkRows < Cfg::kRows ? cBegin + Cfg::kChunkRows : Cfg::kRows;
        const u64 column = tile * Cfg::kLanesX + lx;
        const bool columnLive = column < kColumnsPerRow;
        const u64 columnOffset = (columnLive ? column : 0) * Cfg::kVec;  // dead lanes read column 0 and store nothing
        const u64 rowBegin = cBegin + (u64)rowLane * kBatch;
        const u64 rowEnd = rowBegin + kBatch < cEnd ? rowBegin + kBatch : cEnd;
        const int liveRows = rowEnd > rowBegin ? (int)(rowEnd - rowBegin) : 0;

        // every load of the thread, before anything that depends on the offsets
        typename Cfg::Loaded x[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            if (u < liveRows) Cfg::load(src, (rowBegin + (u64)u) * Cfg::kD + columnOffset, x[u]);
        }

        u64 sLo = 0, sEnd = Cfg::kSegments;
        if (Cfg::kChunks > 1) {
            constexpr u64 kStraddles = (u64)1 << 63;
            sLo = Workspace::firstSegment(workspace)[chunk] & ~kStraddles;
            if (sLo > Cfg::kSegments) sLo = Cfg::kSegments;
            if (chunk + 1 < Cfg::kChunks) {
                const u64 entry = Workspace::firstSegment(workspace)[chunk + 1];
                sEnd = (entry & ~kStraddles) + (entry >> 63);
                if (sEnd > Cfg::kSegments) sEnd = Cfg::kSegments;
            }
        }
        for (int i = threadIdx.x; i <= kWindow; i += Cfg::kThreads) {
            const u64 at = sLo + (u64)i;
            bounds[i] = segmentOffset<Cfg>(offsets, at < Cfg::kSegments ? at : Cfg::kSegments);
        }
        __syncthreads();
        auto bound = [&](u64 at) -> u64 {  // offsets[at], clamped; at <= kSegments
            return at - sLo <= (u64)kWindow ? bounds[at - sLo] : segmentOffset<Cfg>(offsets, at);
        };

        // the first segment that ends after the range's first row (kSegments when none does)
        u64 s = sLo;
        {
            u64 hi = sEnd;
            while (s < hi) {
                const u64 mid = (s + hi) / 2;
                if (bound(mid + 1) > rowBegin) hi = mid; else s = mid + 1;
            }
        }
        auto storeEmpty = [&](u64 segment) {
            if (!columnLive) return;
#pragma unroll
            for (int k = 0; k < Cfg::kVec; ++k) {
                Acc identity;
                identity.reset();
                Cfg::store(identity, segment * Cfg::kD + column * Cfg::kVec + k, out, scale, 0.0f);
            }
        };
        if (liveRows > 0 && rowBegin == 0) {
            for (u64 e = 0; e < s; ++e) storeEmpty(e);  // empty segments at position 0 have no row before them
        }

        u64 myHead = kNone, myTail = kNone;
        if (liveRows > 0) {
            Acc acc[Cfg::kVec];
            typename Cfg::Kept kept[Cfg::kVec];
            u64 first = 0, last = 0;  // rows of segment s
            auto enter = [&]() {
                first = bound(s);
                last = bound(s + 1);
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) {
                    Cfg::loadKept(src, s * Cfg::kD + columnOffset + k, kept[k]);
                    acc[k].reset();
                }
            };
            if (s < Cfg::kSegments) enter();
#pragma unroll
            for (int g = 0; g < kBatch; g += kGroup) {
                if (g < liveRows) {
                    const u64 groupEnd = rowBegin + g + kGroup < rowEnd ? rowBegin + g + kGroup : rowEnd;
                    while (s < Cfg::kSegments && first < groupEnd) {
                        const int lo = first > rowBegin ? (int)(first - rowBegin) : 0;
                        const int hi = last < groupEnd ? (last > rowBegin ? (int)(last - rowBegin) : 0) : (int)(groupEnd - rowBegin);
                        if constexpr (Cfg::kOnlineSoftmax) {
                            // the rows of the run at once: their maximum first, then independent exponentials (rows outside
                            // the run count as -inf and add nothing), one merge into the running pair
                            float v[kGroup][Cfg::kVec];
#pragma unroll
                            for (int u = g; u < g + kGroup; ++u) {
                                const bool inRun = u >= lo && u < hi;
#pragma unroll
                                for (int k = 0; k < Cfg::kVec; ++k) v[u - g][k] = inRun ? Cfg::valueOne(x[u], src, kept[k], k) : -__builtin_inff();
                            }
#pragma unroll
                            for (int k = 0; k < Cfg::kVec; ++k) {
                                float values[kGroup];
#pragma unroll
                                for (int u = 0; u < kGroup; ++u) values[u] = v[u][k];
                                acc[k].template addMany<kGroup>(values);
                            }
                        } else {
#pragma unroll
                            for (int u = g; u < g + kGroup; ++u) {
                                if (u >= lo && u < hi) {
                                    const IndexT row = (IndexT)(rowBegin + (u64)u);
#pragma unroll
                                    for (int k = 0; k < Cfg::kVec; ++k) Cfg::accumulateOne(acc[k], x[u], src, kept[k], k, row);
                                }
                            }
                        }
                        if (last > groupEnd) break;  // goes on after these rows
                        if (first < rowBegin) {      // began before the range and ends in it
                            myHead = s;
#pragma unroll
                            for (int k = 0; k < Cfg::kVec; ++k) heads[slot + k] = acc[k];
                        } else if (columnLive) {
#pragma unroll
                            for (int k = 0; k < Cfg::kVec; ++k)
                                Cfg::store(acc[k], s * Cfg::kD + column * Cfg::kVec + k, out, scale, toFloat((u64)(last > first ? last - first : 0)));
                        }
                        ++s;
                        if (s < Cfg::kSegments) enter();
                    }
                }
            }
            if (s < Cfg::kSegments && first < rowEnd && last > rowEnd) {
                myTail = s;  // goes on after the range
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k) tails[slot + k] = acc[k];
            } else {
                // nothing goes on past the range: the empty segments at the position after its last row belong to this thread
                while (s < Cfg::kSegments && bound(s) == rowEnd && bound(s + 1) == rowEnd) {
                    storeEmpty(s);
                    ++s;
                }
            }
        }
        if (lx == 0) {
            headSegment[rowLane] = myHead;
            tailSegment[rowLane] = myTail;
        }
        __syncthreads();

        // one row of threads folds the parked runs in row order
        if (rowLane == 0) {
            Acc running[Cfg::kVec];
            u64 runningSegment = kNone;
#pragma unroll
            for (int k = 0; k < Cfg::kVec; ++k) running[k].reset();
            for (int j = 0; j < kRowLanes; ++j) {
                const int parked = (j * Cfg::kLanesX + lx) * Cfg::kVec;
                const u64 ended = headSegment[j];
                if (ended != kNone) {
                    const u64 first = bound(ended), last = bound(ended + 1);
#pragma unroll
                    for (int k = 0; k < Cfg::kVec; ++k) {
                        Acc total = heads[parked + k];
                        if (runningSegment == ended) {
                            total = running[k];
                            total.merge(heads[parked + k]);
                        }
                        if (columnLive) {
                            const u64 d = column * Cfg::kVec + k;
                            if (first < cBegin) {
                                total.storePartial(workspace, (chunk * 2 + 0) * Cfg::kD + d, Workspace::kPartialSlots);
                            } else {
                                Cfg::store(total, ended * Cfg::kD + d, out, scale, toFloat((u64)(last > first ? last - first : 0)));
                            }
                        }
                        running[k].reset();
                    }
                    runningSegment = kNone;
                }
                const u64 open = tailSegment[j];
                if (open != kNone) {
#pragma unroll
                    for (int k = 0; k < Cfg::kVec; ++k) {
                        if (runningSegment == open) {
                            running[k].merge(tails[parked + k]);
                        } else {
                            running[k] = tails[parked + k];
                        }
                    }
                    runningSegment = open;
                }
            }
            bool holdsTail = false;
            if (runningSegment != kNone) {
                holdsTail = bound(runningSegment) >= cBegin;
                if (columnLive) {
#pragma unroll
                    for (int k = 0; k < Cfg::kVec; ++k)
                        running[k].storePartial(workspace, (chunk * 2 + (holdsTail ? 1 : 0)) * Cfg::kD + column * Cfg::kVec + k, Workspace::kPartialSlots);
                }
            }
            if (Cfg::kChunks > 1 && tile == 0 && lx == 0) Workspace::tails(workspace)[chunk] = holdsTail ? runningSegment : kNone;
        }
    }
}

// Last launch: block (c, column tile) finishes the segment whose tail chunk c holds, if any: tail[c] and the heads of the
// chunks the segment runs on into, spread over the block's kFinishThreads / kFinishLanes row lanes.  The mean's divisor is
// the row count the offsets hold now.  kFinishLanes = columns (single trailing elements) per block, a power of two <= 64.
template <typename Cfg>
__device__ __forceinline__ void finishSegments(const void* workspace, const typename Cfg::Outputs& out, float scale, const typename Cfg::OffsetT* offsets) {
    typedef typename Cfg::Acc Acc;
    typedef SegmentWorkspace<Cfg> Workspace;
    constexpr int kThreads = Cfg::kFinishThreads;  // threads that finish one segment: 64, or the whole block of 256
    constexpr u64 kTiles = (Cfg::kD + Cfg::kFinishLanes - 1) / Cfg::kFinishLanes;
    __shared__ Acc parked[kThreads / kWave * Cfg::kFinishLanes];
    const u64 job = ((u64)blockIdx.x * blockDim.x + threadIdx.x) / kThreads;
    const u64 chunk = job / kTiles, tile = job % kTiles;
    if (chunk >= Cfg::kChunks) return;  // (groups of kThreads leave together: barriers are only used when that is the block)
    const u64 segment = Workspace::tails(const_cast<void*>(workspace))[chunk];
    if (segment >= Cfg::kSegments) return;  // no segment continues past this chunk
    const u64 first = segmentOffset<Cfg>(offsets, segment), last = segmentOffset<Cfg>(offsets, segment + 1);
    if (last <= first) return;
    u64 lastChunk = (last - 1) / Cfg::kChunkRows;
    if (lastChunk >= Cfg::kChunks) lastChunk = Cfg::kChunks - 1;
    const int lx = threadIdx.x % Cfg::kFinishLanes;
    const u64 rowLane = (threadIdx.x % kThreads) / Cfg::kFinishLanes, rowLanes = kThreads / Cfg::kFinishLanes;
    const u64 d = tile * Cfg::kFinishLanes + lx;
    const bool columnLive = d < Cfg::kD;
    Acc acc[1];
    acc[0].reset();
    if (columnLive) {
        if (rowLane == 0) acc[0].loadPartial(workspace, (chunk * 2 + 1) * Cfg::kD + d, Workspace::kPartialSlots);
#pragma unroll 4
        for (u64 c = chunk + 1 + rowLane; c <= lastChunk; c += rowLanes) {
            Acc part;
            part.loadPartial(workspace, (c * 2 + 0) * Cfg::kD + d, Workspace::kPartialSlots);
            acc[0].merge(part);
        }
    }
    teamReduce<kThreads, Cfg::kFinishLanes, 1>(acc, floorLog2(kThreads), parked);
    if (rowLane == 0 && columnLive) Cfg::store(acc[0], segment * Cfg::kD + d, out, scale, toFloat((u64)(last - first)));
}

// ---- segmented broadcast: per-segment values [B, E] -> rows [N, E] ---------------------------------------------------------------
// out[r, :] = values[b, :] for every row r of segment b = [offsets[b], offsets[b + 1]), optionally divided by the
// segment's length in fp32 and rounded once to the storage type (reference: Utilities/Expression/SegmentedBroadcastKernel.cu:82-104,
// one block per segment).  Rows that belong to no segment are left untouched.  Here the *output* is split into chunks of
// rows, so the stores stream at the same rate whatever the partition is: a block searches the offsets once for the
// first segment that reaches into its chunk, stages a window of kWindow + 1 offsets in LDS, and every thread finds the
// segment of the vector it writes with a binary search in that window (further windows follow while segments are
// shorter than kChunkRows / kWindow on average).
// First s in [0, n] for which pred(s) holds, for a predicate that is false up to some point and true from there on
// (pred(n) is taken as true).  A wavefront with all 64 lanes active runs the search: each round probes 64 evenly spaced
// candidates, so the depth is log64(n) dependent loads instead of log2(n).
template <typename Pred>
__device__ __forceinline__ u64 waveLowerBound(u64 n, Pred pred) {
    const u64 lane = threadIdx.x % kWave;
    u64 lo = 0, hi = n;
    while (hi > lo) {
        const u64 step = (hi - lo + kWave - 1) / kWave;
        const u64 probe = lo + lane * step;
        const bool holds = probe < hi ? pred(probe) : true;
        const u64 mask = __builtin_amdgcn_ballot_w64(holds);
        const u64 firstTrue = mask ? (u64)__builtin_ctzll(mask) : (u64)kWave;
        if (firstTrue == 0) return lo;
        const u64 newLo = lo + (firstTrue - 1) * step + 1;
        const u64 newHi = lo + firstTrue * step;
        lo = newLo;
        hi = newHi < hi ? newHi : hi;
    }
    return lo;
}

// Cfg: T (storage type), OffsetT, kE (elements per value), kRows, kSegments, kChunkRows, kVec (elements per store; kChunkRows * kE
// is a multiple of it), kThreads, kWindow (a power of two), kNormalize, kViaHalf (round through fp16 first: e5m2), kIds (write
// the segment's number instead of a value: the row -> segment index that fused kernels gather per-segment values through).
template <typename Cfg>
__device__ __forceinline__ typename Cfg::T broadcastValue(typename Cfg::T value, u64 length) {
    if constexpr (!Cfg::kNormalize) {
        return value;
    } else {
        float x = toFloat(value) / toFloat(length);
        if (Cfg::kViaHalf) x = roundF16(x);
        return fromFloat<typename Cfg::T>(x);
    }
}

template <typename Cfg>
__device__ __forceinline__ void broadcastSegments(const typename Cfg::T* values, const typename Cfg::OffsetT* offsets, typename Cfg::T* out) {
    typedef typename Cfg::T T;
    constexpr int kWindow = Cfg::kWindow;
    constexpr u64 kE = Cfg::kE;
    constexpr int kVec = Cfg::kVec;
    constexpr bool kRowVectors = kE % kVec == 0;  // a vector never crosses a row
    __shared__ u64 bounds[kWindow + 1];
    const u64 cBegin = (u64)blockIdx.x * Cfg::kChunkRows;
    const u64 cEnd = cBegin + Cfg::kChunkRows < Cfg::kRows ? cBegin + Cfg::kChunkRows : Cfg::kRows;
    u64 window = waveLowerBound(Cfg::kSegments, [&](u64 s) { return segmentOffset<Cfg>(offsets, s + 1) > cBegin; });
    while (window < Cfg::kSegments) {
        for (int i = threadIdx.x; i <= kWindow; i += Cfg::kThreads) {
            const u64 s = window + i;
            bounds[i] = segmentOffset<Cfg>(offsets, s < Cfg::kSegments ? s : Cfg::kSegments);
        }
        __syncthreads();
        const u64 rLo = bounds[0] > cBegin ? bounds[0] : cBegin;
        const u64 rHi = bounds[kWindow] < cEnd ? bounds[kWindow] : cEnd;
        if (rLo < rHi) {
            const u64 vLo = rLo * kE / kVec, vHi = (rHi * kE + kVec - 1) / kVec;
            u64 vFirst = vLo + threadIdx.x;
            if constexpr (kRowVectors && !Cfg::kIds) {
                // four vectors of a thread at a time: their searches interleave and their four loads of per-segment values
                // are in flight together (one vector per round leaves the chain search -> load -> store to wait alone:
                // 1 GiB written in 223 us; four: see the bench line)
                constexpr int kRound = 4;
                for (; vFirst + (u64)(kRound - 1) * Cfg::kThreads < vHi; vFirst += (u64)kRound * Cfg::kThreads) {
                    int j[kRound];
                    u64 component[kRound];
                    bool live[kRound];
#pragma unroll
                    for (int u = 0; u < kRound; ++u) {
                        const u64 e0 = (vFirst + (u64)u * Cfg::kThreads) * kVec;
                        const u64 row = e0 / kE;
                        component[u] = e0 % kE;
                        live[u] = row >= rLo && row < rHi;
                        const u64 searched = row > rLo ? row : rLo;
                        j[u] = 0;
#pragma unroll
                        for (int step = kWindow / 2; step >= 1; step /= 2) {
                            if (bounds[j[u] + step] <= searched) j[u] += step;
                        }
                    }
                    Pack<T, kVec> x[kRound];
#pragma unroll
                    for (int u = 0; u < kRound; ++u)
                        if (live[u]) x[u].load(values + (window + j[u]) * kE + component[u]);
#pragma unroll
                    for (int u = 0; u < kRound; ++u) {
                        if (live[u]) {
                            const u64 length = bounds[j[u] + 1] - bounds[j[u]];
#pragma unroll
                            for (int k = 0; k < kVec; ++k) x[u].v[k] = broadcastValue<Cfg>(x[u].v[k], length);
                            x[u].storeStream(out + (vFirst + (u64)u * Cfg::kThreads) * kVec);
                        }
                    }
                }
            }
            for (u64 v = vFirst; v < vHi; v += Cfg::kThreads) {
                const u64 e0 = v * kVec;
                u64 row = e0 / kE;
                u64 component = e0 % kE;
                const u64 searched = row > rLo ? row : rLo;
                int j = 0;  // bounds[j] <= searched < bounds[j + step] holds throughout
#pragma unroll
                for (int step = kWindow / 2; step >= 1; step /= 2) {
                    if (bounds[j + step] <= searched) j += step;
                }
                if (kRowVectors && !Cfg::kIds) {
                    if (row >= rLo && row < rHi) {
                        const u64 length = bounds[j + 1] - bounds[j];
                        Pack<T, kVec> x;
                        x.load(values + (window + j) * kE + component);
#pragma unroll
                        for (int k = 0; k < kVec; ++k) x.v[k] = broadcastValue<Cfg>(x.v[k], length);
                        x.storeStream(out + e0);
                    }
                } else {
                    Pack<T, kVec> x;
                    bool live[kVec];
                    bool all = true;
#pragma unroll
                    for (int k = 0; k < kVec; ++k) {
                        live[k] = row >= rLo && row < rHi;
                        all = all && live[k];
                        if (live[k]) {
                            while (bounds[j + 1] <= row) ++j;
                            if constexpr (Cfg::kIds) {
                                x.v[k] = (T)(window + j);
                            } else {
                                x.v[k] = broadcastValue<Cfg>(values[(window + j) * kE + component], bounds[j + 1] - bounds[j]);
                            }
                        }
                        if (++component == kE) {
                            component = 0;
                            ++row;
                        }
                    }
                    if (all) {
                        x.storeStream(out + e0);
                    } else {
#pragma unroll
                        for (int k = 0; k < kVec; ++k)
                            if (live[k]) out[e0 + k] = x.v[k];
                    }
                }
            }
        }
        const bool finished = bounds[kWindow] >= cEnd;
        __syncthreads();
        if (finished) break;
        window += kWindow;
    }
}

// ---- second stage of the split kernels: [kOutputs, kSplit] partials -> [kOutputs] -------------------------------------------
// One wavefront per output.  Cfg: kOutputs, kSplit, kFinishOuterStride/kFinishInnerStride/kFinishInner (output layout:
// logical index o = outer * kFinishInner + inner is stored at outer * kFinishOuterStride + inner * kFinishInnerStride).
template <typename Cfg>
__device__ __forceinline__ void finishPartials(const void* partials, const typename Cfg::Outputs& out, float scale) {
    const u64 output = ((u64)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
    if (output < Cfg::kOutputs) foldShares<Cfg>(partials, output, out, scale, threadIdx.x % kWave);
}

}  // namespace thor
