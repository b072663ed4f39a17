// Prefix scans (sum / product / min / max and arg-min / arg-max) over one logical sequence that segment heads cut into
// independent scans: rows of equal length, the segments of a row partition, or nothing (one flat scan).  Instantiated by
// run-time generated traits structs (placed after thor_device_prelude.h).
//
// A block owns a chunk of consecutive logical positions and keeps it in registers: lane-interleaved 16-byte vectors, so
// loads and stores coalesce.  Order inside the chunk is (vector round, thread, element).  Each thread scans its vectors
// serially, the per-vector totals are scanned across the wavefront with shuffles, the wavefront totals across the block
// through a few words of LDS, and the prefix is folded back into the elements: one read and one write per element.  The
// state that flows is {value, index of the value (arg scans), "a head lies in the summarised range"}; combining an earlier
// state with a later one keeps the later one alone when it holds a head.
//
// Chunks that start inside a segment need the state of what precedes them.  When segments are rows that chunks hold whole,
// there is nothing to carry.  Otherwise (Cfg::kLookback) a block takes its chunk by ticket, publishes the chunk's total as
// soon as it has it, and folds the totals of what precedes it from a fixed tree of base 64: the totals of the earlier chunks
// of its group of 64, of the earlier groups of its super-group of 64 groups, and of the earlier super-groups (the last chunk
// of a group publishes the group's total, the last of a super-group that one's).  A block only ever waits for chunks with
// smaller tickets, which are running or done, and the shape of the fold does not depend on who arrived when: results are
// the same from run to run.  Waits are bounded (kWaitLimit polls).  A block whose wait gives up finishes its chunk with what it
// has, then - its registers free again - works the totals it lacks out of the input, in the order their owners would have, and
// does its chunk once more: the result is the same bits whether or not a wait gave up.  Every element is read once and written once.  Beyond 64^3 chunks three launches, none of which
// waits on another block, do the same: the kernel without stores writes each chunk's total, one block turns the totals into
// carries, the full kernel applies them.
//
// A reverse scan walks the same code over mirrored positions (logical p = total - 1 - physical q).
//
// Cfg: T (storage), Acc (u32 for UINT32, float otherwise), kUnsigned, kOp (0 sum, 1 min, 2 max, 3 product), kArg, kInclusive, kReverse,
// kTotal, kRow (row length; 0 = heads come from a bitmap), kThreads, kVec, kItems, kChunkElems (positions per block, a
// multiple of kVec, at most kThreads * kVec * kItems), kChunks, kCarry, kLookback (with kCarry: what precedes a chunk comes
// from the published totals, not from a carries array; kWaitLimit polls bound every wait), kClearWords, kWriteValue, kWriteIndex.
#pragma once

namespace thor {

constexpr u32 kNoIndex = 0xffffffffu;

template <typename Cfg>
struct ScanState {
    typename Cfg::Acc v;
    u32 i;
    u32 head;
};

template <typename Cfg>
__device__ __forceinline__ typename Cfg::Acc scanIdentity() {
    typedef typename Cfg::Acc Acc;
    if (Cfg::kOp == 0) return (Acc)0;
    if (Cfg::kOp == 3) return (Acc)1;
    if (Cfg::kUnsigned) return Cfg::kOp == 1 ? (Acc)0xffffffffu : (Acc)0;  // largest / smallest value
    return Cfg::kOp == 1 ? (Acc)__builtin_inff() : (Acc)(-__builtin_inff());
}

template <typename Cfg>
__device__ __forceinline__ ScanState<Cfg> scanEmpty() {
    ScanState<Cfg> s;
    s.v = scanIdentity<Cfg>();
    s.i = kNoIndex;
    s.head = 0;
    return s;
}

// `a` summarises positions before those of `b`.  Min / max keep the earlier value unless the later one is strictly better
// (so equal values keep the first index); an empty earlier state loses against any element.
template <typename Cfg>
__device__ __forceinline__ void scanOp(typename Cfg::Acc av, u32 ai, typename Cfg::Acc bv, u32 bi, typename Cfg::Acc& rv, u32& ri) {
    if (Cfg::kOp == 0) {
        rv = av + bv;
        ri = kNoIndex;
    } else if (Cfg::kOp == 3) {
        rv = av * bv;
        ri = kNoIndex;
    } else {
        // an index also says "holds an element": the first element of a scan is taken as it is, whatever its value (a NaN
        // that comes first stays, one that comes later never wins: no comparison with it holds)
        const bool takeLater = ((Cfg::kOp == 1 ? (bv < av) : (av < bv)) | (ai == kNoIndex)) & (bi != kNoIndex);
        rv = takeLater ? bv : av;
        ri = takeLater ? bi : ai;
    }
}

template <typename Cfg>
__device__ __forceinline__ ScanState<Cfg> scanCombine(const ScanState<Cfg>& a, const ScanState<Cfg>& b) {
    ScanState<Cfg> r;
    scanOp<Cfg>(a.v, a.i, b.v, b.i, r.v, r.i);
    r.v = b.head ? b.v : r.v;
    r.i = b.head ? b.i : r.i;
    r.head = a.head | b.head;
    return r;
}

template <typename Cfg>
__device__ __forceinline__ ScanState<Cfg> scanShuffleUp(const ScanState<Cfg>& s, int delta) {
    ScanState<Cfg> r;
    r.v = __shfl_up(s.v, delta, kWave);
    r.i = (Cfg::kOp == 1 || Cfg::kOp == 2) ? __shfl_up(s.i, delta, kWave) : kNoIndex;
    r.head = __shfl_up(s.head, delta, kWave);
    return r;
}

// Lane-to-lane moves of the data-parallel primitive kind: the value of the lane `shift` places earlier inside a row of 16
// lanes (CTRL 0x110 + shift), lane 15 of the previous row (0x142, rows 1 and 3) or lane 31 (0x143, rows 2 and 3).  Lanes
// with no source, and rows outside ROW_MASK, receive `empty`.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ u32 scanMoveBits(u32 empty, u32 x) {
    return (u32)__builtin_amdgcn_update_dpp((int)empty, (int)x, CTRL, ROW_MASK, 0xf, false);
}
template <typename Cfg, bool WITH_HEAD, int CTRL, int ROW_MASK>
__device__ __forceinline__ ScanState<Cfg> scanStep(const ScanState<Cfg>& s) {
    typedef typename Cfg::Acc Acc;
    ScanState<Cfg> earlier;
    earlier.v = __builtin_bit_cast(Acc, scanMoveBits<CTRL, ROW_MASK>(__builtin_bit_cast(u32, scanIdentity<Cfg>()), __builtin_bit_cast(u32, s.v)));
    earlier.i = (Cfg::kOp == 1 || Cfg::kOp == 2) ? scanMoveBits<CTRL, ROW_MASK>(kNoIndex, s.i) : kNoIndex;
    earlier.head = WITH_HEAD ? scanMoveBits<CTRL, ROW_MASK>(0u, s.head) : 0u;
    return scanCombine<Cfg>(earlier, s);  // an empty earlier state leaves s as it is
}

// Inclusive scan of one state per lane across the wavefront: four steps inside rows of 16 lanes, then the total of row 0
// into row 1 and of row 2 into row 3, then the total of the lower half into the upper half.  WITH_HEAD = false: no state
// holds a segment head except possibly lane 0's (which nothing is combined into), so the head words stay where they are.
template <typename Cfg, bool WITH_HEAD = true>
__device__ __forceinline__ ScanState<Cfg> scanWave(ScanState<Cfg> s) {
    s = scanStep<Cfg, WITH_HEAD, 0x111, 0xf>(s);
    s = scanStep<Cfg, WITH_HEAD, 0x112, 0xf>(s);
    s = scanStep<Cfg, WITH_HEAD, 0x114, 0xf>(s);
    s = scanStep<Cfg, WITH_HEAD, 0x118, 0xf>(s);
    s = scanStep<Cfg, WITH_HEAD, 0x142, 0xa>(s);
    s = scanStep<Cfg, WITH_HEAD, 0x143, 0xc>(s);
    return s;
}

__device__ __forceinline__ float scanLoad(float x) { return x; }
__device__ __forceinline__ float scanLoad(f16 x) { return toFloat(x); }
__device__ __forceinline__ float scanLoad(bf16 x) { return toFloat(x); }
__device__ __forceinline__ u32 scanLoad(u32 x) { return x; }
template <typename T>
__device__ __forceinline__ T scanStore(float x) {
    return fromFloat<T>(x);
}
template <typename T>
__device__ __forceinline__ T scanStore(u32 x) {
    return (T)x;
}

// chunk states in memory: kChunks values, then kChunks indices, then kChunks head words
template <typename Cfg>
__device__ __forceinline__ ScanState<Cfg> scanLoadState(const void* buffer, u64 slot) {
    ScanState<Cfg> s;
    const u32* words = static_cast<const u32*>(buffer);
    s.v = __builtin_bit_cast(typename Cfg::Acc, words[slot]);
    s.i = words[Cfg::kChunks + slot];
    s.head = words[2 * Cfg::kChunks + slot];
    return s;
}
template <typename Cfg>
__device__ __forceinline__ void scanStoreState(void* buffer, u64 slot, const ScanState<Cfg>& s) {
    u32* words = static_cast<u32*>(buffer);
    words[slot] = __builtin_bit_cast(u32, s.v);
    words[Cfg::kChunks + slot] = s.i;
    words[2 * Cfg::kChunks + slot] = s.head;
}

// the traits of the sum over runs that routes a min / max scan's gradient (only what the combining code looks at)
struct ScanRunSum {
    typedef float T;
    typedef float Acc;
    static constexpr bool kUnsigned = false;
    static constexpr int kOp = 0;
};

// bit k set: logical position p + k starts a segment (p is a multiple of kVec)
template <typename Cfg>
__device__ __forceinline__ u32 scanHeadBits(const u32* heads, u64 p) {
    constexpr int V = Cfg::kVec;
    if (Cfg::kRow == 0) return (heads[p / 32] >> (p % 32)) & ((1u << V) - 1u);
    if (Cfg::kRow % V == 0) return p % Cfg::kRow == 0 ? 1u : 0u;
    u32 bits = 0;
#pragma unroll
    for (int k = 0; k < V; ++k) bits |= ((p + k) % Cfg::kRow == 0 ? 1u : 0u) << k;
    return bits;
}

// ---- published totals (Cfg::kLookback) ----------------------------------------------------------------------------------------
// The block of memory a scan with published totals works in: 32 control words of 8 bytes (word 0: the ticket counter, word 1:
// the number of waits that gave up and worked their totals out again), then one entry of two 8-byte words per chunk, per group and per super-group.  A word
// holds 32 bits of state above a tag (bit 0: written, bit 1: a head lies in the summarised range); the first word carries
// the value, the second (min / max only) the index.  Every word is written once per run, whole, after the block was
// cleared, so a reader that sees the tag sees the state: no fences.
constexpr u32 kScanControlWords = 32;

template <typename Cfg>
__device__ __forceinline__ void scanPublish(u64* entries, u64 entry, const ScanState<Cfg>& s) {
    const u64 tag = 1u | (s.head ? 2u : 0u);
    __hip_atomic_store(entries + 2 * entry, ((u64)__builtin_bit_cast(u32, s.v) << 32) | tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (Cfg::kOp == 1 || Cfg::kOp == 2) {
        __hip_atomic_store(entries + 2 * entry + 1, ((u64)s.i << 32) | tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// One look at entries [first, first + count), count <= 64, by a whole wavefront: lane l reads entry first + l.
struct ScanGlimpse {
    u64 w0, w1;
};
template <typename Cfg>
__device__ __forceinline__ ScanGlimpse scanGlimpse(u64* entries, u64 first, u32 count) {
    const u32 lane = threadIdx.x % kWave;
    ScanGlimpse g = {0, 0};
    if (lane < count) {
        u64* slot = entries + 2 * (first + lane);
        g.w0 = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (Cfg::kOp == 1 || Cfg::kOp == 2) g.w1 = __hip_atomic_load(slot + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return g;
}

// ---- totals worked out again from the input (the way out of a wait that gave up) -----------------------------------------------
// Every published total is a function of the input alone, folded in a fixed order.  A block whose wait for an entry gave up
// therefore computes that entry itself, with the operations and the order of the block that owes it, so the scan's result does
// not depend on whether the wait succeeded (same bits, float sums included).  Slow (one wavefront walks whole chunks) and, while
// blocks take chunks by ticket, never needed: it is what makes a bounded wait safe to give up.  The code runs between the two
// passes a block then makes over its chunk, when none of the chunk is held in registers.
template <typename Cfg>
struct ScanSource {
    const typename Cfg::T* in;
    const u32* heads;
};

template <typename Cfg>
__device__ __forceinline__ ScanState<Cfg> scanLastLane(const ScanState<Cfg>& s) {
    ScanState<Cfg> all;
    all.v = __shfl(s.v, kWave - 1, kWave);
    all.i = (Cfg::kOp == 1 || Cfg::kOp == 2) ? __shfl(s.i, kWave - 1, kWave) : kNoIndex;
    all.head = __shfl(s.head, kWave - 1, kWave);
    return all;
}

// the total of chunk `chunk` as its block computes it (scanChunkCore: vectors serially, lanes, then the wavefronts' totals),
// by one whole wavefront that plays the block's wavefronts in turn; every lane returns it
template <typename Cfg>
__device__ __noinline__ ScanState<Cfg> scanChunkTotalAgain(ScanSource<Cfg> src, u64 chunk) {
    typedef typename Cfg::T T;
    typedef ScanState<Cfg> S;
    constexpr int V = Cfg::kVec, ITEMS = Cfg::kItems, THREADS = Cfg::kThreads, WAVES = THREADS / kWave;
    constexpr bool kPlain = Cfg::kRow != 0 && (Cfg::kRow % ((u64)THREADS * V) == 0 || Cfg::kRow == Cfg::kTotal);
    const int lane = threadIdx.x % kWave;
    const u64 chunkBase = chunk * Cfg::kChunkElems;
    S mine = scanEmpty<Cfg>();
#pragma unroll 1
    for (int slot = 0; slot < ITEMS * WAVES; ++slot) {
        const int it = slot / WAVES, wave = slot % WAVES;
        const u64 local = ((u64)it * THREADS + (u64)wave * kWave + lane) * V;
        const u64 p = chunkBase + local;
        const bool live = local < Cfg::kChunkElems && p < Cfg::kTotal;
        const u64 physical = Cfg::kReverse ? Cfg::kTotal - (live ? p : 0) - V : (live ? p : 0);
        Pack<T, V> x;
        u32 headBits = 0;
        if (live) {
            x.load(src.in + physical);
            headBits = scanHeadBits<Cfg>(src.heads, p);
        }
        S run = scanEmpty<Cfg>();
#pragma unroll
        for (int k = 0; k < V; ++k) {
            S e;
            e.v = live ? scanLoad(x.v[Cfg::kReverse ? V - 1 - k : k]) : scanIdentity<Cfg>();
            e.i = live ? (u32)(physical + (Cfg::kReverse ? V - 1 - k : k)) : kNoIndex;
            e.head = (headBits >> k) & 1u;
            run = scanCombine<Cfg>(run, e);
        }
        S inclusive;
        if (kPlain) {
            const u32 roundHead = (chunkBase + (u64)it * THREADS * V) % Cfg::kRow == 0 ? 1u : 0u;
            inclusive = scanWave<Cfg, false>(run);
            inclusive.head = wave == 0 ? roundHead : 0u;
        } else {
            inclusive = scanWave<Cfg, true>(run);
        }
        const S total = scanLastLane<Cfg>(inclusive);
        if (lane == slot) mine = total;
    }
    return scanLastLane<Cfg>(scanWave<Cfg>(mine));
}

// LEVEL 0: the total of chunk `entry`; 1: of group `entry` (64 chunks); 2: of super-group `entry` (64 groups) - each folded
// like scanLookBack folds what it publishes: the first 63 parts across a wavefront, then the last part
template <typename Cfg, int LEVEL>
__device__ __forceinline__ ScanState<Cfg> scanTotalAgain(ScanSource<Cfg> src, u64 entry) {
    typedef ScanState<Cfg> S;
    if constexpr (LEVEL == 0) {
        return scanChunkTotalAgain<Cfg>(src, entry);
    } else {
        const u32 lane = threadIdx.x % kWave;
        S mine = scanEmpty<Cfg>();
#pragma unroll 1
        for (u32 part = 0; part < 63; ++part) {
            const S t = scanTotalAgain<Cfg, LEVEL - 1>(src, entry * 64 + part);
            if (lane == part) mine = t;
        }
        const S before = scanLastLane<Cfg>(scanWave<Cfg>(mine));
        return scanCombine<Cfg>(before, scanTotalAgain<Cfg, LEVEL - 1>(src, entry * 64 + 63));
    }
}

// The combination, in order, of entries [first, first + count), count <= 64, of level LEVEL: called by one whole wavefront,
// lane l waits for entry first + l (`seen`: an earlier look at the same entries, or zeros); every lane returns the result.
// RECOVER false: polls until every entry is there; after kWaitLimit polls the wait gives up: `gaveUp` is set (in every lane) and
// the result means nothing.  RECOVER true: one look, and the entries that are not there are computed from the input.
template <typename Cfg, int LEVEL, bool RECOVER>
__device__ __forceinline__ ScanState<Cfg> scanAwait(u64* entries, u64 first, u32 count, u64* control, ScanGlimpse seen, ScanSource<Cfg> src,
                                                    bool& gaveUp) {
    typedef ScanState<Cfg> S;
    constexpr bool kIndexed = Cfg::kOp == 1 || Cfg::kOp == 2;
    const u32 lane = threadIdx.x % kWave;
    const bool mine = lane < count;
    if constexpr (RECOVER) {
        seen = scanGlimpse<Cfg>(entries, first, count);
        const bool ready = !mine || ((seen.w0 & 1u) != 0 && (!kIndexed || (seen.w1 & 1u) != 0));
        u64 missing = __ballot(!ready);
        while (missing) {
            const u32 l = (u32)__builtin_ctzll(missing);
            missing &= missing - 1;
            const S again = scanTotalAgain<Cfg, LEVEL>(src, first + l);
            if (lane == l) {
                const u64 tag = 1u | (again.head ? 2u : 0u);
                seen.w0 = ((u64)__builtin_bit_cast(u32, again.v) << 32) | tag;
                seen.w1 = ((u64)again.i << 32) | tag;
            }
        }
    } else {
        for (u32 polls = 0;; ++polls) {
            const bool ready = !mine || ((seen.w0 & 1u) != 0 && (!kIndexed || (seen.w1 & 1u) != 0));
            if (__ballot(!ready) == 0) break;
            if (polls >= Cfg::kWaitLimit) {  // polls before a wait gives up: seconds' worth, never reached while earlier tickets run
                if (lane == 0) atomicAdd(reinterpret_cast<u32*>(control + 1), 1u);
                gaveUp = true;
                return scanEmpty<Cfg>();
            }
            if (polls) __builtin_amdgcn_s_sleep(1);
            if (!ready) seen = scanGlimpse<Cfg>(entries, first, count);
        }
    }
    S s = scanEmpty<Cfg>();
    if (mine) {
        s.v = __builtin_bit_cast(typename Cfg::Acc, (u32)(seen.w0 >> 32));
        s.i = kIndexed ? (u32)(seen.w1 >> 32) : kNoIndex;
        s.head = (u32)(seen.w0 >> 1) & 1u;
    }
    return scanLastLane<Cfg>(scanWave<Cfg>(s));
}

// Where chunk `chunk` sits in the tree of totals, and the arrays of the tree inside the block of memory.
template <typename Cfg>
struct ScanPlace {
    u64 *control, *chunkTotals, *groupTotals, *superTotals;
    u64 group, super;
    u32 inGroup, inSuper;
    __device__ __forceinline__ ScanPlace(void* block, u64 chunk) {
        constexpr u64 kGroups = (Cfg::kChunks + 63) / 64;
        control = static_cast<u64*>(block);
        chunkTotals = control + kScanControlWords;
        groupTotals = chunkTotals + 2 * Cfg::kChunks;
        superTotals = groupTotals + 2 * kGroups;
        inGroup = (u32)(chunk % 64);
        group = chunk / 64;
        inSuper = (u32)(group % 64);
        super = group / 64;
    }
};

// The totals of earlier groups and super-groups are old news by the time a chunk starts: a first look at them, taken before
// the chunk's own data is loaded, is usually all it takes.
template <typename Cfg>
struct ScanEarlyLook {
    ScanGlimpse groups, supers;
};
template <typename Cfg>
__device__ __forceinline__ ScanEarlyLook<Cfg> scanLookEarly(void* block, u64 chunk) {
    const ScanPlace<Cfg> at(block, chunk);
    ScanEarlyLook<Cfg> early;
    early.groups = scanGlimpse<Cfg>(at.groupTotals, at.group - at.inSuper, at.inSuper);
    early.supers = scanGlimpse<Cfg>(at.superTotals, 0, (u32)at.super);
    return early;
}

// What precedes chunk `chunk`, given its own total (the same in every lane of the calling wavefront); publishes the totals
// this chunk owes to later ones.  RECOVER false: the first call; when a wait gives up `gaveUp` is set, the totals not yet
// published stay owed and the result means nothing.  RECOVER true: the call that follows such a first one: nothing is waited
// for, what is missing is computed from the input, what is still owed is published.
template <typename Cfg, bool RECOVER>
__device__ __forceinline__ ScanState<Cfg> scanLookBack(void* block, u64 chunk, const ScanState<Cfg>& total, const ScanEarlyLook<Cfg>& early,
                                                       ScanSource<Cfg> src, bool& gaveUp) {
    typedef ScanState<Cfg> S;
    const ScanPlace<Cfg> at(block, chunk);
    const u32 lane = threadIdx.x % kWave;
    const bool closesGroup = at.inGroup == 63, closesSuper = closesGroup && at.inSuper == 63;
    // the closing chunk's own total has no reader; a second call finds the chunk's total published by the first
    if (!RECOVER && lane == 0 && !closesGroup) scanPublish<Cfg>(at.chunkTotals, chunk, total);
    S chunksBefore = scanEmpty<Cfg>(), groupsBefore = scanEmpty<Cfg>(), supersBefore = scanEmpty<Cfg>();
    const ScanGlimpse nothing = {0, 0};
    if (at.inGroup > 0) chunksBefore = scanAwait<Cfg, 0, RECOVER>(at.chunkTotals, chunk - at.inGroup, at.inGroup, at.control, nothing, src, gaveUp);
    if (gaveUp) return chunksBefore;
    const S groupTotal = scanCombine<Cfg>(chunksBefore, total);
    // (publishing an entry twice writes the same words twice: a first call may have come this far before a later wait gave up)
    if (closesGroup && lane == 0) scanPublish<Cfg>(at.groupTotals, at.group, groupTotal);
    // a head in what was folded so far cuts off everything earlier: no need to wait for it
    if (at.inSuper > 0 && (!chunksBefore.head || closesSuper)) {
        groupsBefore = scanAwait<Cfg, 1, RECOVER>(at.groupTotals, at.group - at.inSuper, at.inSuper, at.control, early.groups, src, gaveUp);
        if (gaveUp) return groupsBefore;
    }
    if (closesSuper && lane == 0) scanPublish<Cfg>(at.superTotals, at.super, scanCombine<Cfg>(groupsBefore, groupTotal));
    const S lower = scanCombine<Cfg>(groupsBefore, chunksBefore);
    if (at.super > 0 && !lower.head) supersBefore = scanAwait<Cfg, 2, RECOVER>(at.superTotals, 0, (u32)at.super, at.control, early.supers, src, gaveUp);
    return scanCombine<Cfg>(supersBefore, lower);
}

// AGGREGATE_ONLY: write the chunk's total to `aggregates` and nothing else.  Otherwise: take the chunk's carry from
// `carries` (when Cfg::kCarry) and write the scanned values and / or indices.
//
// ROUTE (the gradient of a min / max scan; chunks hold whole rows, nothing is carried): the winners stay in registers.  Position
// p's gradient belongs to the element that won p's prefix, and the positions one element wins are consecutive: they begin at
// the element itself (after it, for an exclusive scan) and end before the next element that beats it.  So a second scan over
// the same chunk sums `gradient` over those runs, the last position of each run puts the run's sum where the winner lies in a
// zeroed copy of the chunk in LDS, and the copy is written out with full vectors: every element of `routed` is written once.
//
// SECOND (published totals only): the pass that follows a first pass one of whose waits gave up.  The chunk is `again[0]`, its
// total `again[1..3]` (LDS of the block, written by the first pass); what precedes the chunk is taken from the totals that are
// there and, for the rest, worked out of the input before the chunk is loaded; nothing is waited for.
template <typename Cfg>
__device__ __forceinline__ void scanChunkSecondPass(const typename Cfg::T* in, const u32* heads, const void* carries, typename Cfg::T* outValue,
                                                 u32* outIndex, u32* again);

template <typename Cfg, bool AGGREGATE_ONLY, bool ROUTE, bool SECOND = false>
__device__ __forceinline__ void scanChunkCore(const typename Cfg::T* in, const u32* heads, const void* carries, void* aggregates,
                                              typename Cfg::T* outValue, u32* outIndex, const float* gradient, float* routed, u32* again = nullptr) {
    typedef typename Cfg::T T;
    typedef typename Cfg::Acc Acc;
    typedef ScanState<Cfg> S;
    constexpr int V = Cfg::kVec, ITEMS = Cfg::kItems, THREADS = Cfg::kThreads, WAVES = THREADS / kWave;
    static_assert(ITEMS * WAVES <= kWave, "the wavefront totals of a chunk are scanned by one wavefront");
    // rows that start only where a round of the block starts (or one flat scan): heads need not travel between lanes
    constexpr bool kPlain = Cfg::kRow != 0 && (Cfg::kRow % ((u64)THREADS * V) == 0 || Cfg::kRow == Cfg::kTotal);
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    constexpr bool kLook = Cfg::kLookback && Cfg::kCarry && !AGGREGATE_ONLY && !ROUTE;
    u64 chunk = blockIdx.x;
    // first pass: [0] the chunk, [1..3] its total, [4] a wait gave up; second pass: [1..3] become what precedes the chunk
    __shared__ u32 recovery[kLook && !SECOND ? 5 : 1];
    if constexpr (kLook && !SECOND) {
        // chunks in the order blocks start: whoever a block waits for has started before it
        if (threadIdx.x == 0) {
            recovery[0] = atomicAdd(static_cast<u32*>(const_cast<void*>(carries)), 1u);
            recovery[4] = 0;
        }
        __syncthreads();
        chunk = recovery[0];
    }
    if constexpr (SECOND) chunk = again[0];
    const u64 chunkBase = chunk * Cfg::kChunkElems;

    __shared__ u32 totalValue[ITEMS * WAVES], totalIndex[ITEMS * WAVES], totalHead[ITEMS * WAVES];

    Acc pre[ITEMS][V];
    u32 preIndex[ITEMS][V];
    u32 sealed[ITEMS];
    bool live[ITEMS];
    u64 physical[ITEMS];  // first element of the vector in memory
    S laneExclusive[ITEMS];
    __shared__ float routeTile[ROUTE ? ITEMS * THREADS * V : 1];  // indexed by the position inside the chunk
    Pack<float, V> upstream[ROUTE ? ITEMS : 1];
    u32 rowHeads[ROUTE ? ITEMS : 1];
    u32 winners[ROUTE ? ITEMS : 1][V];  // in scan order
    ScanEarlyLook<Cfg> early = {};
    if constexpr (kLook && !SECOND) {
        if (wave == 0) early = scanLookEarly<Cfg>(const_cast<void*>(carries), chunk);
    }
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const u64 local = ((u64)it * THREADS + threadIdx.x) * V;
        const u64 p = chunkBase + local;
        live[it] = local < Cfg::kChunkElems && p < Cfg::kTotal;
        physical[it] = Cfg::kReverse ? Cfg::kTotal - (live[it] ? p : 0) - V : (live[it] ? p : 0);
        Pack<T, V> x;
        u32 headBits = 0;
        if (live[it]) {
            x.loadStream(in + physical[it]);
            headBits = scanHeadBits<Cfg>(heads, p);
        }
        if constexpr (ROUTE) {
            if (live[it]) upstream[it].loadStream(gradient + physical[it]);
            rowHeads[it] = headBits;
#pragma unroll
            for (int k = 0; k < V; ++k) routeTile[local + k] = 0.0f;
        }
        S run = scanEmpty<Cfg>();
        sealed[it] = 0;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            S e;
            e.v = live[it] ? scanLoad(x.v[Cfg::kReverse ? V - 1 - k : k]) : scanIdentity<Cfg>();
            e.i = live[it] ? (u32)(physical[it] + (Cfg::kReverse ? V - 1 - k : k)) : kNoIndex;
            e.head = (headBits >> k) & 1u;
            if (!Cfg::kInclusive) {
                pre[it][k] = e.head ? scanIdentity<Cfg>() : run.v;
                preIndex[it][k] = e.head ? kNoIndex : run.i;
                sealed[it] |= (run.head | e.head) << k;
            }
            run = scanCombine<Cfg>(run, e);
            if (Cfg::kInclusive) {
                pre[it][k] = run.v;
                preIndex[it][k] = run.i;
                sealed[it] |= run.head << k;
            }
        }
        S inclusive;
        if (kPlain) {
            // only the first lane of the block can hold a head in this round, and nothing is combined into it
            const u32 roundHead = (chunkBase + (u64)it * THREADS * V) % Cfg::kRow == 0 ? 1u : 0u;
            inclusive = scanWave<Cfg, false>(run);
            inclusive.head = wave == 0 ? roundHead : 0u;
        } else {
            inclusive = scanWave<Cfg, true>(run);
        }
        laneExclusive[it] = scanShuffleUp<Cfg>(inclusive, 1);
        if (lane == 0) laneExclusive[it] = scanEmpty<Cfg>();
        if (lane == kWave - 1) {
            totalValue[it * WAVES + wave] = __builtin_bit_cast(u32, inclusive.v);
            totalIndex[it * WAVES + wave] = inclusive.i;
            totalHead[it * WAVES + wave] = inclusive.head;
        }
    }
    __syncthreads();
    if (wave == 0) {
        S mine = scanEmpty<Cfg>();
        if (lane < ITEMS * WAVES) {
            mine.v = __builtin_bit_cast(Acc, totalValue[lane]);
            mine.i = totalIndex[lane];
            mine.head = totalHead[lane];
        }
        const S inclusive = scanWave<Cfg>(mine);
        if (AGGREGATE_ONLY) {
            if (lane == kWave - 1) scanStoreState<Cfg>(aggregates, chunk, inclusive);
        } else {
            S before = scanShuffleUp<Cfg>(inclusive, 1);
            if (lane == 0) before = scanEmpty<Cfg>();
            if constexpr (kLook && !SECOND) {
                const S total = scanLastLane<Cfg>(inclusive);
                const ScanSource<Cfg> src = {in, heads};
                bool gaveUp = false;
                // a wait that gave up leaves this pass with a result that means nothing: a second pass follows
                before = scanCombine<Cfg>(scanLookBack<Cfg, false>(const_cast<void*>(carries), chunk, total, early, src, gaveUp), before);
                if (gaveUp && lane == 0) {
                    recovery[1] = __builtin_bit_cast(u32, total.v);
                    recovery[2] = total.i;
                    recovery[3] = total.head;
                    recovery[4] = 1;
                }
            } else if constexpr (SECOND) {
                S preceding;
                preceding.v = __builtin_bit_cast(Acc, again[1]);
                preceding.i = again[2];
                preceding.head = again[3];
                before = scanCombine<Cfg>(preceding, before);
            } else if (Cfg::kCarry) {
                before = scanCombine<Cfg>(scanLoadState<Cfg>(carries, chunk), before);
            }
            if (lane < ITEMS * WAVES) {
                totalValue[lane] = __builtin_bit_cast(u32, before.v);
                totalIndex[lane] = before.i;
                totalHead[lane] = before.head;
            }
        }
    }
    if (AGGREGATE_ONLY) return;
    __syncthreads();
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        if (!live[it]) continue;
        S base;
        base.v = __builtin_bit_cast(Acc, totalValue[it * WAVES + wave]);
        base.i = totalIndex[it * WAVES + wave];
        base.head = totalHead[it * WAVES + wave];
        base = scanCombine<Cfg>(base, laneExclusive[it]);
        Pack<T, V> values;
        Pack<u32, V> indices;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            Acc v;
            u32 i;
            scanOp<Cfg>(base.v, base.i, pre[it][k], preIndex[it][k], v, i);
            const bool own = (sealed[it] >> k) & 1u;
            v = own ? pre[it][k] : v;
            i = own ? preIndex[it][k] : i;
            values.v[Cfg::kReverse ? V - 1 - k : k] = scanStore<T>(v);
            indices.v[Cfg::kReverse ? V - 1 - k : k] = i;
            if constexpr (ROUTE) winners[it][k] = i;
        }
        if constexpr (!ROUTE) {
            if (Cfg::kWriteValue) values.storeStream(outValue + physical[it]);
            if (Cfg::kWriteIndex) indices.storeStream(outIndex + physical[it]);
        }
    }
    if constexpr (kLook && !SECOND) {
        // the flag was written before the barrier above: every thread of the block reads the same value.  Nothing of the first
        // pass is needed any more, so the call costs the ordinary pass no registers.
        if (recovery[4] != 0) scanChunkSecondPass<Cfg>(in, heads, carries, outValue, outIndex, recovery);
    }
    if constexpr (ROUTE) {
        typedef ScanRunSum R;
        typedef ScanState<R> RS;
        // a run begins where a position is won by itself (inclusive) or by the position just before it (exclusive), and at
        // every row head; positions outside the chunk's data count as heads so that the last run ends before them
        float sums[ITEMS][V];
        u32 runHeads[ITEMS], runSealed[ITEMS];
        RS runExclusive[ITEMS];
        __syncthreads();  // the totals of the first scan have been read
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) {
            RS run = scanEmpty<R>();
            runHeads[it] = 0;
            runSealed[it] = 0;
#pragma unroll
            for (int k = 0; k < V; ++k) {
                const u32 own = (u32)(physical[it] + (Cfg::kReverse ? V - 1 - k : k));
                const u32 opener = Cfg::kInclusive ? own : (Cfg::kReverse ? own + 1u : own - 1u);
                RS e;
                e.v = live[it] ? upstream[it].v[Cfg::kReverse ? V - 1 - k : k] : 0.0f;
                e.i = kNoIndex;
                e.head = !live[it] || winners[it][k] == opener || winners[it][k] == kNoIndex || ((rowHeads[it] >> k) & 1u) ? 1u : 0u;
                runHeads[it] |= e.head << k;
                run = scanCombine<R>(run, e);
                sums[it][k] = run.v;
                runSealed[it] |= run.head << k;
            }
            const RS inclusive = scanWave<R, true>(run);
            runExclusive[it] = scanShuffleUp<R>(inclusive, 1);
            if (lane == 0) runExclusive[it] = scanEmpty<R>();
            if (lane == kWave - 1) {
                totalValue[it * WAVES + wave] = __builtin_bit_cast(u32, inclusive.v);
                totalHead[it * WAVES + wave] = inclusive.head;
            }
            if (lane == 0) totalIndex[it * WAVES + wave] = runHeads[it] & 1u;  // does this wavefront's round begin with a head
        }
        __syncthreads();
        u32 nextWaveBegins[ITEMS];  // the head bit of the position after this wavefront's round
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) nextWaveBegins[it] = it * WAVES + wave + 1 < ITEMS * WAVES ? totalIndex[it * WAVES + wave + 1] : 1u;
        __syncthreads();
        if (wave == 0) {
            RS mine = scanEmpty<R>();
            if (lane < ITEMS * WAVES) {
                mine.v = __builtin_bit_cast(float, totalValue[lane]);
                mine.head = totalHead[lane];
            }
            const RS inclusive = scanWave<R>(mine);
            RS before = scanShuffleUp<R>(inclusive, 1);
            if (lane == 0) before = scanEmpty<R>();
            if (lane < ITEMS * WAVES) {
                totalValue[lane] = __builtin_bit_cast(u32, before.v);
                totalHead[lane] = before.head;
            }
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) {
            RS base;
            base.v = __builtin_bit_cast(float, totalValue[it * WAVES + wave]);
            base.i = kNoIndex;
            base.head = totalHead[it * WAVES + wave];
            base = scanCombine<R>(base, runExclusive[it]);
            // the head bit of the position after this vector: the next lane's first, or the next wavefront's
            u32 following = __shfl_down(runHeads[it] & 1u, 1, kWave);
            if (lane == kWave - 1) following = nextWaveBegins[it];
            if (!live[it]) continue;
            const u32 ends = (runHeads[it] >> 1) | (following << (V - 1));  // bit k: position k closes its run
#pragma unroll
            for (int k = 0; k < V; ++k) {
                const float sum = ((runSealed[it] >> k) & 1u) ? sums[it][k] : base.v + sums[it][k];
                const u32 winner = winners[it][k];
                if (((ends >> k) & 1u) && winner != kNoIndex) {
                    const u64 position = Cfg::kReverse ? Cfg::kTotal - 1 - winner : (u64)winner;
                    routeTile[position - chunkBase] = sum;
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) {
            if (!live[it]) continue;
            const u64 local = ((u64)it * THREADS + threadIdx.x) * V;
            Pack<float, V> out;
#pragma unroll
            for (int k = 0; k < V; ++k) out.v[Cfg::kReverse ? V - 1 - k : k] = routeTile[local + k];
            out.storeStream(routed + physical[it]);
        }
    }
}

// again[1..3]: the total of chunk again[0] -> what precedes that chunk (called by the block's first wavefront)
template <typename Cfg>
__device__ __forceinline__ void scanPrecedingAgain(const typename Cfg::T* in, const u32* heads, const void* carries, u32* again) {
    typedef ScanState<Cfg> S;
    S total;
    total.v = __builtin_bit_cast(typename Cfg::Acc, again[1]);
    total.i = again[2];
    total.head = again[3];
    const ScanSource<Cfg> src = {in, heads};
    const ScanEarlyLook<Cfg> unused = {};
    bool never = false;
    const S preceding = scanLookBack<Cfg, true>(const_cast<void*>(carries), again[0], total, unused, src, never);
    if (threadIdx.x % kWave == 0) {
        again[1] = __builtin_bit_cast(u32, preceding.v);
        again[2] = preceding.i;
        again[3] = preceding.head;
    }
}

template <typename Cfg>
__device__ __forceinline__ void scanChunkSecondPass(const typename Cfg::T* in, const u32* heads, const void* carries, typename Cfg::T* outValue,
                                                 u32* outIndex, u32* again) {
    if (threadIdx.x < kWave) scanPrecedingAgain<Cfg>(in, heads, carries, again);
    scanChunkCore<Cfg, false, false, true>(in, heads, carries, nullptr, outValue, outIndex, nullptr, nullptr, again);
}

template <typename Cfg, bool AGGREGATE_ONLY>
__device__ __forceinline__ void scanChunk(const typename Cfg::T* in, const u32* heads, const void* carries, void* aggregates,
                                          typename Cfg::T* outValue, u32* outIndex) {
    scanChunkCore<Cfg, AGGREGATE_ONLY, false>(in, heads, carries, aggregates, outValue, outIndex, nullptr, nullptr);
}
template <typename Cfg>
__device__ __forceinline__ void scanRoute(const typename Cfg::T* in, const float* gradient, float* routed) {
    scanChunkCore<Cfg, false, true>(in, nullptr, nullptr, nullptr, nullptr, nullptr, gradient, routed);
}

// One block: the totals of kChunks chunks -> the state that precedes each chunk.  A thread owns a run of consecutive chunks.
template <typename Cfg>
__device__ __forceinline__ void scanCarries(const void* aggregates, void* carries) {
    typedef ScanState<Cfg> S;
    constexpr int THREADS = 1024, WAVES = THREADS / kWave;
    constexpr u64 PER = (Cfg::kChunks + THREADS - 1) / THREADS;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const u64 first = (u64)threadIdx.x * PER;
    __shared__ u32 totalValue[WAVES], totalIndex[WAVES], totalHead[WAVES];
    // a thread's totals are loaded at once (independent loads), then folded from registers
    constexpr bool kHeld = PER <= 32;
    S held[kHeld ? PER : 1];
    if (kHeld) {
#pragma unroll
        for (u64 j = 0; j < PER; ++j) held[j] = first + j < Cfg::kChunks ? scanLoadState<Cfg>(aggregates, first + j) : scanEmpty<Cfg>();
    }
    S run = scanEmpty<Cfg>();
    if (kHeld) {
#pragma unroll
        for (u64 j = 0; j < PER; ++j) run = scanCombine<Cfg>(run, held[j]);
    } else {
        for (u64 c = first; c < first + PER && c < Cfg::kChunks; ++c) run = scanCombine<Cfg>(run, scanLoadState<Cfg>(aggregates, c));
    }
    const S inclusive = scanWave<Cfg>(run);
    S before = scanShuffleUp<Cfg>(inclusive, 1);
    if (lane == 0) before = scanEmpty<Cfg>();
    if (lane == kWave - 1) {
        totalValue[wave] = __builtin_bit_cast(u32, inclusive.v);
        totalIndex[wave] = inclusive.i;
        totalHead[wave] = inclusive.head;
    }
    __syncthreads();
    S earlierWaves = scanEmpty<Cfg>();
    for (int w = 0; w < wave; ++w) {
        S t;
        t.v = __builtin_bit_cast(typename Cfg::Acc, totalValue[w]);
        t.i = totalIndex[w];
        t.head = totalHead[w];
        earlierWaves = scanCombine<Cfg>(earlierWaves, t);
    }
    run = scanCombine<Cfg>(earlierWaves, before);
    if (kHeld) {
#pragma unroll
        for (u64 j = 0; j < PER; ++j) {
            if (first + j < Cfg::kChunks) scanStoreState<Cfg>(carries, first + j, run);
            run = scanCombine<Cfg>(run, held[j]);
        }
    } else {
        for (u64 c = first; c < first + PER && c < Cfg::kChunks; ++c) {
            scanStoreState<Cfg>(carries, c, run);
            run = scanCombine<Cfg>(run, scanLoadState<Cfg>(aggregates, c));
        }
    }
}

// Segment heads of a row partition as one bit per logical position.  scanClear zeroes the bitmap, and the block of the
// published totals behind it, first: Cfg::kClearWords words from the start of the temporary storage.
// Cfg: OffsetT, kSegments, kTotal, kReverse.
template <typename Cfg>
__device__ __forceinline__ void scanClear(u32* words) {
    const u64 word = (u64)blockIdx.x * blockDim.x + threadIdx.x;
    if (word < Cfg::kClearWords) words[word] = 0;
}
template <typename Cfg>
__device__ __forceinline__ void scanMarkHeads(const typename Cfg::OffsetT* offsets, u32* heads) {
    const u64 s = (u64)blockIdx.x * blockDim.x + threadIdx.x;
    if (s > Cfg::kSegments) return;
    u64 begin = (u64)offsets[s];
    begin = begin < Cfg::kTotal ? begin : Cfg::kTotal;
    if (s == Cfg::kSegments) {
        // rows past the partition form a segment of their own, so nothing of theirs flows into a real one
        if (!Cfg::kReverse && begin < Cfg::kTotal) atomicOr(&heads[begin / 32], 1u << (begin % 32));
        return;
    }
    u64 end = (u64)offsets[s + 1];
    end = end < Cfg::kTotal ? end : Cfg::kTotal;
    if (end <= begin) return;
    const u64 position = Cfg::kReverse ? Cfg::kTotal - end : begin;
    atomicOr(&heads[position / 32], 1u << (position % 32));
}

}  // namespace thor
