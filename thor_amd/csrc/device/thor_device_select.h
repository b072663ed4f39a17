// Stream compaction (select-flagged) and top-k selection, device-wide and over rows of one length.  Instantiated by run-time
// generated traits structs (placed after thor_device_prelude.h).  Replaces cub::DeviceSelect::Flagged and cub::DeviceTopK /
// the batched fixed-size top-k the reference calls (Utilities/TensorOperations/Cub/CubSelect.cu:26-50, CubTopK.cu:27-330).
//
// Select-flagged keeps the input's order.  A block owns a chunk of consecutive positions: one launch counts the raised flags
// of every chunk, one block turns the counts into output offsets (and writes the total), and the last launch reads the flags
// and the elements with lane-interleaved vector loads, ranks the flagged ones in position order, gathers them in LDS and
// writes the chunk's run of the output with adjacent lanes on adjacent elements.  No block waits for another one.
//
// Top-k is a radix selection on an order-preserving unsigned image of the key (sign handling for floats and signed integers;
// for "smallest" the image is complemented, so the code always looks for the largest images).  From the most significant
// digit down (11, 11 and 10 bits of a 32-bit key; 8-bit digits of narrower ones): a histogram of the digit over the keys
// that still match the digits fixed so far, then the bucket that holds the k-th largest image is fixed (by the block of the
// counting pass that finishes last).  After the last digit the image T of the k-th key and the number of keys equal to T
// that belong to the answer are known; one more pass writes every key above T and that many keys equal to T.  Long inputs
// are read once: see "candidates" below.  The answer is
// the k best keys (with their values, for pairs) in no particular order, like the reference's (its library calls ask for
// unsorted, not run-to-run deterministic output); which of several equal keys at the threshold are taken is not fixed either.
// Rows (fixed-size segments of at most 8192 keys) run the same selection inside one block, keys in registers, histogram in LDS.
#pragma once

namespace thor {

// Exclusive prefix sum of one word per thread over a block; `total` receives the block's sum in every thread.  `lds` holds
// THREADS / 64 words and may be reused after the call.
template <int THREADS>
__device__ __forceinline__ u32 blockExclusiveSum(u32 x, u32* lds, u32& total) {
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    u32 inclusive = x;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const u32 y = __shfl_up(inclusive, d, kWave);
        if (lane >= d) inclusive += y;
    }
    if (lane == kWave - 1) lds[wave] = inclusive;
    __syncthreads();
    u32 before = 0, sum = 0;
#pragma unroll
    for (int w = 0; w < THREADS / kWave; ++w) {
        const u32 t = lds[w];
        before += w < wave ? t : 0u;
        sum += t;
    }
    total = sum;
    __syncthreads();
    return before + inclusive - x;
}

// How many of the lanes below this one are set in `votes` (the result of a ballot).
__device__ __forceinline__ u32 votesBelow(u64 votes) {
    return __builtin_amdgcn_mbcnt_hi((u32)(votes >> 32), __builtin_amdgcn_mbcnt_lo((u32)votes, 0u));
}

// ---- select-flagged ----------------------------------------------------------------------------------------------------------
// Cfg: Word (u8 / u16 / u32: elements are copied as raw words), kTotal, kThreads (256), kVec (4 when the tensors are aligned to
// four elements, else 1), kRounds (4), kChunks.  A block owns kThreads * kVec * kRounds consecutive positions, read in rounds of
// lane-interleaved vectors: vector v = round * kThreads + thread holds positions [v * kVec, v * kVec + kVec) of the chunk.
template <typename Cfg>
struct SelectChunk {
    static constexpr u64 kElems = (u64)Cfg::kThreads * Cfg::kVec * Cfg::kRounds;
};

// bit k set: the flag of position `first + k` is raised (k < kVec; positions at or past kTotal count as not raised)
template <typename Cfg>
__device__ __forceinline__ u32 selectFlagBits(const u8* flags, u64 first) {
    u32 bits = 0;
    if (Cfg::kVec == 4 && first + 4 <= Cfg::kTotal) {
        const u32 w = *reinterpret_cast<const u32*>(flags + first);
        // the top bit of every byte that is not zero
        const u32 raised = (((w & 0x7f7f7f7fu) + 0x7f7f7f7fu) | w) & 0x80808080u;
        bits = ((raised >> 7) & 1u) | ((raised >> 14) & 2u) | ((raised >> 21) & 4u) | ((raised >> 28) & 8u);
    } else {
#pragma unroll
        for (int k = 0; k < Cfg::kVec; ++k)
            if (first + k < Cfg::kTotal) bits |= (flags[first + k] != 0 ? 1u : 0u) << k;
    }
    return bits;
}

// The raised flags of every chunk.  A wavefront counts one chunk (the count does not care in which order the scattering pass
// will read the chunk): sixteen flag bytes per lane and load, all loads of the chunk in flight, no LDS and no barrier.  Launched
// with kChunks / (kThreads / 64) blocks, rounded up.
template <typename Cfg>
__device__ __forceinline__ void selectCount(const u8* flags, u32* counts) {
    constexpr u64 kElems = SelectChunk<Cfg>::kElems;
    const int lane = threadIdx.x % kWave;
    const u64 chunk = (u64)blockIdx.x * (Cfg::kThreads / kWave) + threadIdx.x / kWave;
    if (chunk >= Cfg::kChunks) return;
    const u64 chunkBase = chunk * kElems;
    u32 mine = 0;
    if (Cfg::kVec == 4 && kElems % (kWave * 16) == 0 && chunkBase + kElems <= Cfg::kTotal) {
        constexpr int kLoads = (int)(kElems / (kWave * 16));
        Pack<u32, 4> words[kLoads];
#pragma unroll
        for (int j = 0; j < kLoads; ++j) words[j].loadStream(reinterpret_cast<const u32*>(flags + chunkBase) + ((u64)j * kWave + lane) * 4);
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const u32 w = words[j].v[k];
                mine += (u32)__builtin_popcount((((w & 0x7f7f7f7fu) + 0x7f7f7f7fu) | w) & 0x80808080u);  // bytes that are not zero
            }
        }
    } else {
        for (u64 first = chunkBase + (u64)lane * Cfg::kVec; first < chunkBase + kElems && first < Cfg::kTotal; first += (u64)kWave * Cfg::kVec) {
            mine += (u32)__builtin_popcount(selectFlagBits<Cfg>(flags, first));
        }
    }
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) mine += __shfl_xor(mine, d, kWave);
    if (lane == 0) counts[chunk] = mine;
}

// One block of 1024 threads: counts[kChunks] -> bases[kChunks] (exclusive), the grand total -> *numSelected.  A thread owns a
// run of consecutive chunks, so one block-wide scan serves any number of them.
template <typename Cfg>
__device__ __forceinline__ void selectOffsets(const u32* counts, u32* bases, u32* numSelected) {
    __shared__ u32 lds[1024 / kWave];
    constexpr u64 kPer = (Cfg::kChunks + 1023) / 1024;
    constexpr bool kHeld = kPer <= 64;  // a thread's counts are loaded at once (independent loads) and kept
    const u64 first = (u64)threadIdx.x * kPer;
    u32 held[kHeld ? kPer : 1];
    u32 mine = 0;
    if (kHeld) {
#pragma unroll
        for (u64 j = 0; j < kPer; ++j) held[j] = first + j < Cfg::kChunks ? counts[first + j] : 0u;
#pragma unroll
        for (u64 j = 0; j < kPer; ++j) mine += held[j];
    } else {
        for (u64 c = first; c < first + kPer && c < Cfg::kChunks; ++c) mine += counts[c];
    }
    u32 total;
    u32 running = blockExclusiveSum<1024>(mine, lds, total);
    if (kHeld) {
#pragma unroll
        for (u64 j = 0; j < kPer; ++j) {
            if (first + j < Cfg::kChunks) bases[first + j] = running;
            running += held[j];
        }
    } else {
        for (u64 c = first; c < first + kPer && c < Cfg::kChunks; ++c) {
            bases[c] = running;
            running += counts[c];
        }
    }
    if (threadIdx.x == 0) *numSelected = total;
}

// The flagged elements of the chunk are ranked in position order, gathered in LDS and written out as one contiguous run.
template <typename Cfg>
__device__ __forceinline__ void selectScatter(const typename Cfg::Word* in, const u8* flags, const u32* bases, typename Cfg::Word* out) {
    typedef typename Cfg::Word Word;
    static_assert(Cfg::kRounds == 4, "the ranks of four rounds travel in the four 16-bit fields of one 64-bit sum");
    __shared__ u32 lds[2 * (Cfg::kThreads / kWave)];
    __shared__ Word kept[SelectChunk<Cfg>::kElems];
    const u64 chunkBase = (u64)blockIdx.x * SelectChunk<Cfg>::kElems;
    u32 bits[Cfg::kRounds];
    Pack<Word, Cfg::kVec> values[Cfg::kRounds];
    u64 packed = 0;  // field r: flagged elements this thread holds in round r
#pragma unroll
    for (int round = 0; round < Cfg::kRounds; ++round) {
        const u64 first = chunkBase + ((u64)round * Cfg::kThreads + threadIdx.x) * Cfg::kVec;
        bits[round] = 0;
        if (first < Cfg::kTotal) {
            bits[round] = selectFlagBits<Cfg>(flags, first);
            if (first + Cfg::kVec <= Cfg::kTotal) {
                values[round].loadStream(in + first);
            } else {
#pragma unroll
                for (int k = 0; k < Cfg::kVec; ++k)
                    if (first + k < Cfg::kTotal) values[round].v[k] = in[first + k];
            }
        }
        packed |= (u64)__builtin_popcount(bits[round]) << (16 * round);
    }
    // exclusive sums over the threads of every field at once (a field stays below 2^16: at most kThreads * kVec per round)
    u32 totalLo, totalHi;
    const u32 beforeLo = blockExclusiveSum<Cfg::kThreads>((u32)packed, lds, totalLo);
    const u32 beforeHi = blockExclusiveSum<Cfg::kThreads>((u32)(packed >> 32), lds + Cfg::kThreads / kWave, totalHi);
    const u32 roundTotal[4] = {totalLo & 0xffffu, totalLo >> 16, totalHi & 0xffffu, totalHi >> 16};
    const u32 before[4] = {beforeLo & 0xffffu, beforeLo >> 16, beforeHi & 0xffffu, beforeHi >> 16};
    u32 roundBase = 0;
#pragma unroll
    for (int round = 0; round < Cfg::kRounds; ++round) {
        u32 at = roundBase + before[round];
#pragma unroll
        for (int k = 0; k < Cfg::kVec; ++k)
            if (bits[round] & (1u << k)) kept[at++] = values[round].v[k];
        roundBase += roundTotal[round];
    }
    __syncthreads();
    Word* run = out + bases[blockIdx.x];
    for (u32 i = threadIdx.x; i < roundBase; i += Cfg::kThreads) run[i] = kept[i];
}

// ---- key images ----------------------------------------------------------------------------------------------------------------
// Cfg::kKind: 0 unsigned integer, 1 signed integer, 2 float (sign and magnitude).  Cfg::kBits: 8, 16 or 32.  The image orders like
// the key; for kLargest == false it is complemented.  Floats order by their bits: -0 below +0, NaNs beyond the infinities.
template <typename Cfg>
__device__ __forceinline__ u32 topkImage(typename Cfg::Raw raw) {
    constexpr u32 kMask = Cfg::kBits == 32 ? 0xffffffffu : ((1u << Cfg::kBits) - 1u);
    constexpr u32 kSign = 1u << (Cfg::kBits - 1);
    u32 u = (u32)raw & kMask;
    if (Cfg::kKind == 1) u ^= kSign;
    if (Cfg::kKind == 2) u = (u & kSign) ? (~u & kMask) : (u | kSign);
    return Cfg::kLargest ? u : (~u & kMask);
}

// The key whose image is `image` (topkImage is a bijection of the key's bits).
template <typename Cfg>
__device__ __forceinline__ typename Cfg::Raw topkKeyOfImage(u32 image) {
    constexpr u32 kMask = Cfg::kBits == 32 ? 0xffffffffu : ((1u << Cfg::kBits) - 1u);
    constexpr u32 kSign = 1u << (Cfg::kBits - 1);
    u32 u = Cfg::kLargest ? image : (~image & kMask);
    if (Cfg::kKind == 1) u ^= kSign;
    if (Cfg::kKind == 2) u = (u & kSign) ? (u & ~kSign) : (~u & kMask);
    return (typename Cfg::Raw)u;
}

// Digits are taken from the most significant end: 11, 11 and 10 bits of a 32-bit image, 8 and 8 of a 16-bit one, 8 of an 8-bit one.
constexpr int kTopkMaxBins = 2048;
constexpr int kTopkBinsPerThread = kTopkMaxBins / 256;

// The bucket of a histogram of `numBins` bins (a power of two, at most 2048) that holds the `wanted`-th largest digit (1-based,
// wanted <= the histogram's total, which `totalOut` receives: the result means nothing otherwise), found by the 256 threads of a block: thread t looks at the 8 bins of descending ranks
// [8 t, 8 t + 8).  Returns the bucket in every thread; `above` receives the number of entries in larger buckets.  `lds`: 6 words.
template <typename Bins>
__device__ __forceinline__ u32 topkPickBucket(const Bins& bins, u32 numBins, u32 wanted, u32* lds, u32& above, u32* totalOut = nullptr) {
    u32 counts[kTopkBinsPerThread];
    u32 mine = 0;
#pragma unroll
    for (int i = 0; i < kTopkBinsPerThread; ++i) {
        const u32 rank = threadIdx.x * kTopkBinsPerThread + i;
        counts[i] = rank < numBins ? bins(numBins - 1u - rank) : 0u;
        mine += counts[i];
    }
    u32 total;
    u32 before = blockExclusiveSum<256>(mine, lds, total);  // entries in the bins of the threads before this one: all larger
    if (totalOut) *totalOut = total;
    if (before < wanted && wanted <= before + mine) {
#pragma unroll
        for (int i = 0; i < kTopkBinsPerThread; ++i) {
            if (before < wanted && wanted <= before + counts[i]) {
                lds[4] = numBins - 1u - (threadIdx.x * kTopkBinsPerThread + i);
                lds[5] = before;
            }
            before += counts[i];
        }
    }
    __syncthreads();
    const u32 bucket = lds[4];
    above = lds[5];
    __syncthreads();
    return bucket;
}

// ---- device-wide top-k -----------------------------------------------------------------------------------------------------------
// Cfg: Raw (u8 / u16 / u32 word of the key), kKind, kBits, kLargest, kTotal, kK (already capped at kTotal, > 0), kPairs, kVec (keys
// per vector load: 16 bytes' worth when the key tensor is aligned and kTotal divides, else 1), kItems (vectors per thread of the
// gathering pass).  Temporary storage: 2048 histogram words, then the sixteen state words below (then the candidates, see there).
struct TopkState {
    u32 prefix;     // the digits fixed so far, in place
    u32 remaining;  // the rank (1-based) of the wanted key among the keys that match the prefix
    u32 taken;      // output slots handed out to keys above the threshold
    u32 ties;       // keys equal to the threshold seen so far by the gathering pass
    u32 arrived;    // blocks of the running launch that have finished their part (zero between launches)
    // candidates (below)
    u32 reserved[2];
    u32 overflow;    // a region of the candidate list was too short for this input: the third launch walks the whole input
    u32 floorTies;   // keys equal to F whose positions were asked to be noted
    u32 ambiguous;   // entries asked for in the second list
    u32 unused[6];
};
constexpr int kTopkStateWords = 16;

template <typename Cfg>
__device__ __forceinline__ void topkInit(u32* temp) {
    for (int b = threadIdx.x; b < kTopkMaxBins; b += 256) temp[b] = 0;
    if (threadIdx.x < kTopkStateWords) temp[kTopkMaxBins + threadIdx.x] = 0;
    __syncthreads();
    if (threadIdx.x == 0) reinterpret_cast<TopkState*>(temp + kTopkMaxBins)->remaining = (u32)Cfg::kK;
}

// One block of 256 threads: fixes the digit at `shift` and clears the histogram for the next pass.  The histogram words were
// added to by blocks all over the device: they are read at device scope.
template <typename Cfg>
__device__ __forceinline__ void topkPick(u32* temp, u32 shift, u32 bits) {
    __shared__ u32 lds[8];
    TopkState* state = reinterpret_cast<TopkState*>(temp + kTopkMaxBins);
    const u32 wanted = state->remaining, prefix = state->prefix;
    u32 above;
    const u32 bucket = topkPickBucket([&](u32 b) { return loadDeviceWide(&temp[b]); }, 1u << bits, wanted, lds, above);
    for (int b = threadIdx.x; b < kTopkMaxBins; b += 256) temp[b] = 0;
    if (threadIdx.x == 0) {
        state->prefix = prefix | (bucket << shift);
        state->remaining = wanted - above;
    }
}

// The end of a counting pass, called by every block (256 threads) once it has added its histogram to the shared one: the
// block waits until those additions are acknowledged and counts itself in; the block that counts in last fixes the digit,
// so the pass needs no launch of its own for that.
template <typename Cfg>
__device__ __forceinline__ void topkPickWhenLast(u32* temp, u32 shift, u32 bits) {
    __shared__ u32 last;
    partialsWritten();
    __syncthreads();
    TopkState* state = reinterpret_cast<TopkState*>(temp + kTopkMaxBins);
    if (threadIdx.x == 0) {
        const u32 before = __hip_atomic_fetch_add(&state->arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last = before + 1u == gridDim.x ? 1u : 0u;
        if (last) storeDeviceWide(&state->arrived, 0u);
    }
    __syncthreads();
    if (last) topkPick<Cfg>(temp, shift, bits);
}

// Histogram of the `bits`-wide digit at `shift` over the keys whose higher digits equal the prefix.  Blocks stride over the keys
// in vectors, four vectors of a thread in flight.
template <typename Cfg>
__device__ __forceinline__ void topkHistogram(const typename Cfg::Raw* keys, u32* temp, u32 shift, u32 bits) {
    typedef typename Cfg::Raw Raw;
    constexpr int V = Cfg::kVec, kUnroll = 4;
    __shared__ u32 bins[kTopkMaxBins];
    const u32 numBins = 1u << bits;
    for (u32 b = threadIdx.x; b < numBins; b += 256) bins[b] = 0;
    __syncthreads();
    const u32 prefix = reinterpret_cast<const TopkState*>(temp + kTopkMaxBins)->prefix;
    const u32 fixedBits = shift + bits >= 32 ? 0u : (0xffffffffu << (shift + bits));
    const u32 digitMask = numBins - 1u;
    constexpr u64 kVectors = Cfg::kTotal / V;  // kTotal is a multiple of V
    const u64 stride = (u64)gridDim.x * 256;
    for (u64 v0 = (u64)blockIdx.x * 256 + threadIdx.x; v0 < kVectors; v0 += stride * kUnroll) {
        Pack<Raw, V> x[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
            if (v0 + u * stride < kVectors) x[u].loadStream(keys + (v0 + u * stride) * V);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (v0 + u * stride < kVectors) {
#pragma unroll
                for (int k = 0; k < V; ++k) {
                    const u32 image = topkImage<Cfg>(x[u].v[k]);
                    if ((image & fixedBits) == (prefix & fixedBits)) atomicAdd(&bins[(image >> shift) & digitMask], 1u);
                }
            }
        }
    }
    __syncthreads();
    for (u32 b = threadIdx.x; b < numBins; b += 256) {
        const u32 mine = bins[b];
        if (mine != 0) atomicAdd(&temp[b], mine);
    }
    topkPickWhenLast<Cfg>(temp, shift, bits);
}

// Writes the keys above the threshold image (kK - remaining of them) and `remaining` of the keys equal to it.  Every
// wavefront counts its qualifying keys with votes, the block adds the counts up and asks once for that many output slots
// (requests for slots from all over the grid meet at one address, and the memory system serves those one after the other:
// one request per wavefront vote cost 0.7 ms at k = 65 536); a block without qualifying keys, the usual case when k is
// small next to the input, leaves after the count.
template <typename Cfg>
__device__ __forceinline__ void topkGather(const typename Cfg::Raw* keys, const u32* values, u32* temp, typename Cfg::Raw* outKeys, u32* outValues) {
    typedef typename Cfg::Raw Raw;
    constexpr int V = Cfg::kVec, kWaves = Cfg::kThreads / kWave;
    __shared__ u32 waveAbove[kWaves], waveTies[kWaves], bases[2];
    TopkState* state = reinterpret_cast<TopkState*>(temp + kTopkMaxBins);
    const u32 threshold = state->prefix, wantedTies = state->remaining, firstTieSlot = (u32)Cfg::kK - wantedTies;
    constexpr u64 kVectors = Cfg::kTotal / V;
    constexpr u64 kChunkVectors = (u64)Cfg::kThreads * Cfg::kItems;
    constexpr u64 kChunks = (kVectors + kChunkVectors - 1) / kChunkVectors;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    for (u64 chunk = blockIdx.x; chunk < kChunks; chunk += gridDim.x) {
        if (chunk != blockIdx.x) __syncthreads();  // the previous chunk's counts and bases have been read
        const u64 blockFirst = chunk * kChunkVectors;
        Pack<Raw, V> x[Cfg::kItems];
#pragma unroll
        for (int it = 0; it < Cfg::kItems; ++it) {
            const u64 v = blockFirst + (u64)it * Cfg::kThreads + threadIdx.x;
            if (v < kVectors) x[it].loadStream(keys + v * V);
        }
        u32 above = 0, ties = 0;  // of this wavefront
#pragma unroll
        for (int it = 0; it < Cfg::kItems; ++it) {
            const bool live = blockFirst + (u64)it * Cfg::kThreads + threadIdx.x < kVectors;
#pragma unroll
            for (int k = 0; k < V; ++k) {
                const u32 image = live ? topkImage<Cfg>(x[it].v[k]) : 0u;
                above += (u32)__builtin_popcountll(__builtin_amdgcn_ballot_w64(live && image > threshold));
                ties += (u32)__builtin_popcountll(__builtin_amdgcn_ballot_w64(live && image == threshold));
            }
        }
        if (lane == 0) {
            waveAbove[wave] = above;
            waveTies[wave] = ties;
        }
        __syncthreads();
        u32 aboveAt = 0, tieAt = 0, blockAbove = 0, blockTies = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            aboveAt += w < wave ? waveAbove[w] : 0u;
            tieAt += w < wave ? waveTies[w] : 0u;
            blockAbove += waveAbove[w];
            blockTies += waveTies[w];
        }
        if (blockAbove + blockTies == 0) continue;
        if (threadIdx.x == 0) {
            bases[0] = blockAbove ? atomicAdd(&state->taken, blockAbove) : 0u;
            bases[1] = blockTies ? atomicAdd(&state->ties, blockTies) : 0u;
        }
        __syncthreads();
        aboveAt += bases[0];
        tieAt += bases[1];
        if (above + ties == 0) continue;  // nothing in this wavefront
#pragma unroll
        for (int it = 0; it < Cfg::kItems; ++it) {
            const u64 v = blockFirst + (u64)it * Cfg::kThreads + threadIdx.x;
            const bool live = v < kVectors;
#pragma unroll
            for (int k = 0; k < V; ++k) {
                const u32 image = live ? topkImage<Cfg>(x[it].v[k]) : 0u;
                const bool isAbove = live && image > threshold, isTie = live && image == threshold;
                const u64 aboveVotes = __builtin_amdgcn_ballot_w64(isAbove), tieVotes = __builtin_amdgcn_ballot_w64(isTie);
                u32 slot = 0xffffffffu;
                if (isAbove) slot = aboveAt + votesBelow(aboveVotes);
                if (isTie) {
                    const u32 rank = tieAt + votesBelow(tieVotes);
                    if (rank < wantedTies) slot = firstTieSlot + rank;
                }
                aboveAt += (u32)__builtin_popcountll(aboveVotes);
                tieAt += (u32)__builtin_popcountll(tieVotes);
                if (slot != 0xffffffffu) {
                    outKeys[slot] = x[it].v[k];
                    if (Cfg::kPairs) outValues[slot] = values[v * V + k];
                }
            }
        }
    }
}

// ---- candidates ------------------------------------------------------------------------------------------------------------------
// Long inputs are read in full once, in three launches:
//   1. the floor (topkFloor): wavefronts read a sample of the input (runs of 256 vectors spread evenly), every lane keeps the
//      largest images of eight groups of its vectors, and each wavefront finds, by a bit search over votes, a value that at least
//      kFloorRank of those maxima reach.  The smallest of the wavefronts' values is the floor F: wavefronts * kFloorRank >= kK
//      sampled keys lie at or above it, so the kK-th largest key of the input does too, whatever the sample missed.  Block 0
//      also clears the shared histogram and the state words (no launch of its own for that).
//   2. the pass over the input (topkCollect): keys above F, the candidates, go into the candidate list (image and position;
//      every wavefront owns a region of kRegion entries and counts what it wrote), and their distance from F is counted in a
//      histogram whose buckets grow with the distance (below), so one histogram resolves keys just above F and keys far
//      above it alike.  Keys equal to F are not listed: they can be any part of the input (many equal keys); the positions
//      of the first kK of them are noted (pairs).
//   3. the output (topkFinish): every block picks the bucket that holds the kK-th largest key out of the histogram, or finds
//      that fewer than kK keys lie above F: then the answer is all candidates plus keys equal to F.  Blocks walk the list;
//      candidates in buckets above the picked one are written out, those in
//      the picked bucket go to a second, short list; the block that finishes last selects from that list (digits of the
//      distance inside the bucket, histogram in LDS) and writes the rest of the output, or the keys equal to F.
// A region that would overflow (the sample was not representative: inputs that repeat with the sample's period) raises
// `overflow`: the histogram still counted every candidate, and the third launch walks the whole input instead of the list.
// A picked bucket that holds more than kAmbiguous keys which are not all equal (clustered keys around the threshold that the
// sample did not see) makes the last block of the third launch walk the list (the input) by itself: slow, and correct.
// Cfg additionally: kCompact, kFloorBlocks (blocks of 256 threads of the first launch), kFloorItems (vectors per lane there),
// kFloorRank, kSampleRunStride (vectors from one run of the sample to the next), kRegion, kRegions (wavefronts of the second
// launch), kAmbiguous (entries of the second list).
// Temporary storage after the state: kFloorBlocks * 4 floors, kK positions of keys equal to F, the second list (images,
// positions), kRegions counts, the candidate list (kRegions * kRegion images, as many positions for pairs).
template <typename Cfg>
struct TopkCandidates {
    static constexpr u32 kFloors = Cfg::kFloorBlocks * 4;
    __device__ __forceinline__ static u32* floors(u32* temp) { return temp + kTopkMaxBins + kTopkStateWords; }
    __device__ __forceinline__ static u32* tiePositions(u32* temp) { return floors(temp) + kFloors; }
    __device__ __forceinline__ static u32* ambiguousImages(u32* temp) { return tiePositions(temp) + (u32)Cfg::kK; }
    __device__ __forceinline__ static u32* ambiguousPositions(u32* temp) { return ambiguousImages(temp) + Cfg::kAmbiguous; }
    __device__ __forceinline__ static u32* counts(u32* temp) { return ambiguousPositions(temp) + Cfg::kAmbiguous; }
    __device__ __forceinline__ static u32* images(u32* temp) { return counts(temp) + Cfg::kRegions; }
    __device__ __forceinline__ static u32* positions(u32* temp) { return images(temp) + (u64)Cfg::kRegions * Cfg::kRegion; }
};

// The bucket of a distance d >= 0 (image - F - 1), B = Cfg::kBucketBits (3 .. 6): d itself below 2^B, else the position q of
// d's leading bit and the B bits after it: ((q - B + 1) << B) | those bits, at most (33 - B) * 2^B - 1 < 2048.  Buckets order
// like distances.  More bits: fewer keys share the bucket of the kK-th largest; fewer bits: fewer histogram words that every
// block of the second launch adds to at its end.
template <typename Cfg>
__device__ __forceinline__ u32 topkDistanceBucket(u32 d) {
    constexpr u32 B = Cfg::kBucketBits;
    if (d < (1u << B)) return d;
    const u32 q = 31u - (u32)__builtin_clz(d);
    return ((q - B + 1u) << B) | ((d >> (q - B)) & ((1u << B) - 1u));
}
// The distances of a bucket: [first, first + 2^bits).
template <typename Cfg>
__device__ __forceinline__ void topkBucketRange(u32 bucket, u32& first, u32& bits) {
    constexpr u32 B = Cfg::kBucketBits;
    if (bucket < (1u << B)) {
        first = bucket;
        bits = 0;
        return;
    }
    const u32 q = (bucket >> B) + B - 1u;
    bits = q - B;
    first = ((1u << B) | (bucket & ((1u << B) - 1u))) << bits;
}

// First launch: kFloorBlocks blocks of 256 threads.  A lane reads kFloorItems vectors (a multiple of kTopkFloorGroups) and keeps
// kTopkFloorGroups maxima.
constexpr int kTopkFloorGroups = 8;
template <typename Cfg>
__device__ __forceinline__ void topkFloor(const typename Cfg::Raw* keys, u32* temp) {
    typedef typename Cfg::Raw Raw;
    constexpr int V = Cfg::kVec, I = Cfg::kFloorItems;
    if (blockIdx.x == 0) topkInit<Cfg>(temp);  // nothing else touches the histogram or the state during this launch
    if (Cfg::kFloorRank == 0) {  // no sample: every key lies at or above zero
        if (threadIdx.x % kWave == 0) TopkCandidates<Cfg>::floors(temp)[blockIdx.x * 4 + threadIdx.x / kWave] = 0;
        return;
    }
    Pack<Raw, V> x[I];
#pragma unroll
    for (int it = 0; it < I; ++it) {
        // run `run` of the sample lies somewhere in the run-th stretch of kSampleRunStride vectors: evenly spaced runs would
        // show a sample of few distinct keys when the input repeats itself with a period that the spacing divides
        const u64 run = (u64)it * Cfg::kFloorBlocks + blockIdx.x;
        const u64 shift = (u64)(((u32)run * 2654435761u) >> 8) % (Cfg::kSampleRunStride - 255);
        x[it].load(keys + (run * Cfg::kSampleRunStride + shift + threadIdx.x) * V);
    }
    constexpr int G = kTopkFloorGroups;  // maxima per lane: of the vectors it, it + G, ...
    u32 largest[G];
    u32 all = 0;
#pragma unroll
    for (int g = 0; g < G; ++g) largest[g] = 0;
#pragma unroll
    for (int it = 0; it < I; ++it) {
#pragma unroll
        for (int k = 0; k < V; ++k) {
            const u32 image = topkImage<Cfg>(x[it].v[k]);
            largest[it % G] = image > largest[it % G] ? image : largest[it % G];
        }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) all = largest[g] > all ? largest[g] : all;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const u32 other = (u32)__shfl_xor((int)all, d, kWave);
        all = other > all ? other : all;
    }
    // The largest value, with the bits below the 20 under the wavefront's leading bit left zero, that kFloorRank of the
    // wavefront's 64 * G maxima reach (zero is reached by all of them).
    u32 value = 0;
    if (all != 0) {
        const int top = 31 - __builtin_clz(all);
        const int low = top > 19 ? top - 19 : 0;
        for (int bit = top; bit >= low; --bit) {
            const u32 trial = value | (1u << bit);
            u32 reached = 0;
#pragma unroll
            for (int g = 0; g < G; ++g) reached += (u32)__builtin_popcountll(__builtin_amdgcn_ballot_w64(largest[g] >= trial));
            if (reached >= Cfg::kFloorRank) value = trial;
        }
    }
    if (threadIdx.x % kWave == 0) TopkCandidates<Cfg>::floors(temp)[blockIdx.x * 4 + threadIdx.x / kWave] = value;
}

// The smallest of the first launch's values, in every thread of a block of 256.  `lds`: 4 words.
template <typename Cfg>
__device__ __forceinline__ u32 topkFloorOfAll(const u32* temp, u32* lds) {
    const u32* floors = TopkCandidates<Cfg>::floors(const_cast<u32*>(temp));
    u32 smallest = 0xffffffffu;
    for (u32 i = threadIdx.x; i < TopkCandidates<Cfg>::kFloors; i += 256) {
        const u32 f = floors[i];
        smallest = f < smallest ? f : smallest;
    }
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const u32 other = (u32)__shfl_xor((int)smallest, d, kWave);
        smallest = other < smallest ? other : smallest;
    }
    if (threadIdx.x % kWave == 0) lds[threadIdx.x / kWave] = smallest;
    __syncthreads();
    u32 result = lds[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) result = lds[w] < result ? lds[w] : result;
    __syncthreads();
    return result;
}

// Second launch: kRegions / 4 blocks of 256 threads stride over the input in vectors, the next turn's vectors on their way
// while this turn's are looked at.  Every wavefront owns a region of the list and counts what it wrote: no wavefront asks
// another for room, and no block waits for anything at its end (the bucket is picked by the third launch).  A wavefront
// gathers its candidates in LDS and copies them to its region when kTopkStage have come together, as a rule once, at the
// end: a store in the loop would make the wait for the next turn's vectors a wait for that store as well (the compiler
// cannot count the memory operations in flight across the branches around the stores, and waits for all of them).
constexpr u32 kTopkStage = 512;
template <typename Cfg>
__device__ __forceinline__ void topkCollect(const typename Cfg::Raw* keys, u32* temp) {
    typedef typename Cfg::Raw Raw;
    constexpr int V = Cfg::kVec, kUnroll = Cfg::kCompactUnroll;
    __shared__ u32 bins[kTopkMaxBins];
    __shared__ u32 lds[8];
    __shared__ u32 stageImages[256 / kWave][kTopkStage];
    __shared__ u32 stagePositions[Cfg::kPairs ? 256 / kWave : 1][Cfg::kPairs ? kTopkStage : 1];
    constexpr u64 kVectors = Cfg::kTotal / V;
    const u64 stride = (u64)gridDim.x * 256;
    u64 v0 = (u64)blockIdx.x * 256 + threadIdx.x;
    Pack<Raw, V> x[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
        if (v0 + u * stride < kVectors) x[u].loadStream(keys + (v0 + u * stride) * V);
    for (u32 b = threadIdx.x; b < kTopkMaxBins; b += 256) bins[b] = 0;
    TopkState* state = reinterpret_cast<TopkState*>(temp + kTopkMaxBins);
    const u32 floorImage = topkFloorOfAll<Cfg>(temp, lds);  // (its barriers also order the cleared bins)
    const int lane = threadIdx.x % kWave;
    const u32 region = blockIdx.x * (256 / kWave) + threadIdx.x / kWave;
    u32* regionImages = TopkCandidates<Cfg>::images(temp) + (u64)region * Cfg::kRegion;
    u32* regionPositions = TopkCandidates<Cfg>::positions(temp) + (u64)region * Cfg::kRegion;
    u32* tiePositions = TopkCandidates<Cfg>::tiePositions(temp);
    const int wave = threadIdx.x / kWave;
    u32 cursor = 0;          // candidates of this wavefront so far: the same in every lane
    u32 copied = 0;          // of them, in the region already (the rest is in LDS)
    bool tiesNoted = false;  // kK keys equal to F have been noted (by anyone): no more requests
    auto copyStage = [&]() {  // (the wavefront's LDS writes and reads are in program order)
        for (u32 i = lane; i < cursor - copied; i += kWave) {
            if (copied + i < Cfg::kRegion) {
                regionImages[copied + i] = stageImages[wave][i];
                if (Cfg::kPairs) regionPositions[copied + i] = stagePositions[Cfg::kPairs ? wave : 0][Cfg::kPairs ? i : 0];
            }
        }
        copied = cursor;
    };
    while ((v0 - lane) < kVectors) {  // (every lane of a wavefront makes the same number of turns)
        const u64 next = v0 + stride * kUnroll;
        Pack<Raw, V> y[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
            if (next + u * stride < kVectors) y[u].loadStream(keys + (next + u * stride) * V);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const bool live = v0 + u * stride < kVectors;
            u32 image[V];
            u32 mask = 0;  // bit k: key k of the vector is a candidate
            bool tie = false;
#pragma unroll
            for (int k = 0; k < V; ++k) {
                image[k] = live ? topkImage<Cfg>(x[u].v[k]) : 0u;
                mask |= (live && image[k] > floorImage ? 1u : 0u) << k;
                tie |= Cfg::kPairs && live && image[k] == floorImage;
            }
            if (__builtin_amdgcn_ballot_w64(mask != 0 || (tie && !tiesNoted)) == 0) continue;  // the usual case when k is small next to the input
            // The lanes' candidate counts (0 .. V) turn into places in the region through votes on the counts' bits.
            const u32 mine = (u32)__builtin_popcount(mask);
            u32 before = 0, all = 0;
#pragma unroll
            for (int b = 0; (1 << b) <= V; ++b) {
                const u64 votes = __builtin_amdgcn_ballot_w64(((mine >> b) & 1u) != 0);
                before += votesBelow(votes) << b;
                all += (u32)__builtin_popcountll(votes) << b;
            }
            if (cursor - copied + all > kTopkStage) copyStage();
            u32 slot = cursor - copied + before;
            cursor += all;
            while (mask != 0) {  // (as many turns as the lane with most candidates has: one, as a rule)
                const int k = __builtin_ctz(mask);
                mask &= mask - 1u;
                u32 chosen = image[0];
#pragma unroll
                for (int j = 1; j < V; ++j) chosen = k == j ? image[j] : chosen;
                stageImages[wave][slot] = chosen;
                if (Cfg::kPairs) stagePositions[Cfg::kPairs ? wave : 0][Cfg::kPairs ? slot : 0] = (u32)((v0 + u * stride) * V + k);
                atomicAdd(&bins[topkDistanceBucket<Cfg>(chosen - floorImage - 1u)], 1u);
                ++slot;
            }
            if (Cfg::kPairs && !tiesNoted) {
#pragma unroll
                for (int k = 0; k < V; ++k) {
                    const bool tieHere = live && image[k] == floorImage;
                    const u64 tieVotes = __builtin_amdgcn_ballot_w64(tieHere);
                    if (tieVotes != 0 && !tiesNoted) {
                        const int first = __builtin_ctzll(tieVotes);
                        u32 noted = 0;
                        if (lane == first) noted = atomicAdd(&state->floorTies, (u32)__builtin_popcountll(tieVotes));
                        noted = (u32)__shfl((int)noted, first, kWave);
                        if (tieHere) {
                            const u32 rank = noted + votesBelow(tieVotes);
                            if (rank < (u32)Cfg::kK) tiePositions[rank] = (u32)((v0 + u * stride) * V + k);
                        }
                        tiesNoted = noted >= (u32)Cfg::kK;
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) x[u] = y[u];
        v0 = next;
    }
    copyStage();
    if (lane == 0) {
        TopkCandidates<Cfg>::counts(temp)[region] = cursor < Cfg::kRegion ? cursor : Cfg::kRegion;
        if (cursor > Cfg::kRegion) atomicOr(&state->overflow, 1u);
    }
    __syncthreads();
    for (u32 b = threadIdx.x; b < (33u - Cfg::kBucketBits) << Cfg::kBucketBits; b += 256) {
        const u32 mine = bins[b];
        if (mine != 0) atomicAdd(&temp[b], mine);
    }
}

// A walk over the candidates: `visit(image, position)` sees every key above F of the wavefront's share once and in the same
// order for every run; `position()` is the key's place in the input.  Wavefront `first` of `step`: regions first,
// first + step, ..., the counts of kTopkRegionBatch regions loaded together, then up to kWalkPerLane * 64 entries of each at a
// time, so a region costs no round trip of its own.  issue() asks for the first regions' counts, settle() (any time later)
// takes them; the first entries of the first regions stay in registers from one run to the next.  When a region overflowed,
// the whole input is walked instead (the same share of it for every run).
constexpr int kTopkRegionBatch = 4;
template <typename Cfg>
struct TopkWalk {
    static constexpr int kPerLane = Cfg::kRegion < Cfg::kWalkPerLane * kWave ? (int)((Cfg::kRegion + kWave - 1) / kWave) : Cfg::kWalkPerLane;
    const typename Cfg::Raw* keys;
    u32* temp;
    u32 first, step, floorImage;
    u32 overflow;
    u32 firstCounts[kTopkRegionBatch];
    u32 firstWords[kTopkRegionBatch][kPerLane];
    bool haveWords;

    __device__ __forceinline__ void loadCounts(u32 r0, u32 (&count)[kTopkRegionBatch]) const {
        const u32* counts = TopkCandidates<Cfg>::counts(temp);
#pragma unroll
        for (int j = 0; j < kTopkRegionBatch; ++j) {
            const u32 r = r0 + j * step;
            count[j] = counts[r < Cfg::kRegions ? r : Cfg::kRegions - 1];
        }
    }
    __device__ __forceinline__ void issue(const typename Cfg::Raw* keys_, u32* temp_, u32 first_, u32 step_) {
        keys = keys_;
        temp = temp_;
        first = first_;
        step = step_;
        haveWords = false;
        overflow = reinterpret_cast<const TopkState*>(temp + kTopkMaxBins)->overflow;
        loadCounts(first, firstCounts);
    }
    __device__ __forceinline__ void settle(u32 floorImage_) {
        floorImage = floorImage_;
#pragma unroll
        for (int j = 0; j < kTopkRegionBatch; ++j) {
            firstCounts[j] = first + j * step < Cfg::kRegions ? (u32)__builtin_amdgcn_readfirstlane((int)firstCounts[j]) : 0u;
        }
    }
    template <typename Visit>
    __device__ __forceinline__ void run(const Visit& visit) {
        const u32 lane = threadIdx.x % kWave;
        if (overflow != 0) {
            for (u64 i = (u64)first * kWave + lane; i < Cfg::kTotal; i += (u64)step * kWave) {
                const u32 image = topkImage<Cfg>(keys[i]);
                if (image > floorImage) visit(image, [&]() { return (u32)i; });
            }
            return;
        }
        const u32* images = TopkCandidates<Cfg>::images(temp);
        const u32* positions = TopkCandidates<Cfg>::positions(temp);
        for (u32 r0 = first; r0 < Cfg::kRegions; r0 += step * kTopkRegionBatch) {
            u32 count[kTopkRegionBatch];
            u32 most = 0;
            if (r0 == first) {
#pragma unroll
                for (int j = 0; j < kTopkRegionBatch; ++j) count[j] = firstCounts[j];
            } else {
                loadCounts(r0, count);
#pragma unroll
                for (int j = 0; j < kTopkRegionBatch; ++j) count[j] = r0 + j * step < Cfg::kRegions ? (u32)__builtin_amdgcn_readfirstlane((int)count[j]) : 0u;
            }
#pragma unroll
            for (int j = 0; j < kTopkRegionBatch; ++j) most = count[j] > most ? count[j] : most;
            for (u32 at = 0; at < most; at += kPerLane * kWave) {
                const bool kept = r0 == first && at == 0;  // these entries stay in registers for the next run
                u32 word[kTopkRegionBatch][kPerLane];
                if (!(kept && haveWords)) {
#pragma unroll
                    for (int j = 0; j < kTopkRegionBatch; ++j) {
#pragma unroll
                        for (int e = 0; e < kPerLane; ++e) {
                            const u32 i = at + e * kWave + lane;
                            word[j][e] = i < count[j] ? images[(u64)(r0 + j * step) * Cfg::kRegion + i] : 0u;
                        }
                    }
                }
                if (kept) {
#pragma unroll
                    for (int j = 0; j < kTopkRegionBatch; ++j) {
#pragma unroll
                        for (int e = 0; e < kPerLane; ++e) {
                            if (haveWords) word[j][e] = firstWords[j][e];
                            else firstWords[j][e] = word[j][e];
                        }
                    }
                    haveWords = true;
                }
#pragma unroll
                for (int j = 0; j < kTopkRegionBatch; ++j) {
#pragma unroll
                    for (int e = 0; e < kPerLane; ++e) {
                        const u32 i = at + e * kWave + lane;
                        if (i < count[j]) visit(word[j][e], [&]() { return positions[(u64)(r0 + j * step) * Cfg::kRegion + i]; });
                    }
                }
            }
        }
    }
};

// Third launch: kFinishBlocks blocks of 256 threads.  Every block finds F and picks the bucket out of the second launch's
// histogram by itself.  Every thread counts the candidates of its share above the picked bucket and those in it, a block scan
// turns the counts into ranks inside the block, one thread asks for the block's output slots and its room in the second
// list (requests from all over the grid meet at one address each, and the memory system serves those one after the other:
// about 10 ns a request), and a second walk over the same candidates puts them into LDS in rank order, from where the block
// writes them out (a store between the walk's loads would make every later load wait for it).
constexpr int kTopkAmbiguousPerThread = 8;  // a second list of up to 256 * this entries stays in the last block's registers
constexpr u32 kTopkStageOut = 1792, kTopkStageAmbiguous = 256;  // entries of a block that go through LDS (the rest: stored from the walk)
template <typename Cfg>
__device__ __forceinline__ void topkFinish(const typename Cfg::Raw* keys, const u32* values, u32* temp, typename Cfg::Raw* outKeys, u32* outValues) {
    typedef typename Cfg::Raw Raw;
    __shared__ u32 stage[Cfg::kPairs ? 2 : 1][kTopkMaxBins];  // [0]: images (later the digit histogram), [1]: positions
    __shared__ u32 lds[8];
    __shared__ u32 bases[2];
    __shared__ u32 last;
    static_assert(kTopkStageOut + kTopkStageAmbiguous == kTopkMaxBins, "the stage is the histogram's memory");
    u32* bins = stage[0];
    TopkState* state = reinterpret_cast<TopkState*>(temp + kTopkMaxBins);
    const u32 firstWave = blockIdx.x * (256 / kWave) + threadIdx.x / kWave, waveStep = gridDim.x * (256 / kWave);
    TopkWalk<Cfg> share;  // this wavefront's share of the candidates
    share.issue(keys, temp, firstWave, waveStep);
    const u32 floorImage = topkFloorOfAll<Cfg>(temp, lds);
    u32 aboveBucket, listed;
    const u32 picked = topkPickBucket([&](u32 b) { return temp[b]; }, kTopkMaxBins, (u32)Cfg::kK, lds, aboveBucket, &listed);
    // fewer than kK keys above F: every candidate belongs to the answer (bucket -1), and `wanted` keys equal to F
    const int bucket = listed >= (u32)Cfg::kK ? (int)picked : -1;
    const u32 wanted = listed >= (u32)Cfg::kK ? (u32)Cfg::kK - aboveBucket : (u32)Cfg::kK - listed;
    u32* ambiguousImages = TopkCandidates<Cfg>::ambiguousImages(temp);
    u32* ambiguousPositions = TopkCandidates<Cfg>::ambiguousPositions(temp);
    share.settle(floorImage);
    {
        u32 out = 0, ambiguous = 0;
        share.run([&](u32 image, auto) {
            const int mine = (int)topkDistanceBucket<Cfg>(image - floorImage - 1u);
            out += mine > bucket;
            ambiguous += mine == bucket;
        });
        u32 blockOut, blockAmbiguous;
        u32 outAt = blockExclusiveSum<256>(out, lds, blockOut);                    // ranks inside the block
        u32 ambiguousAt = blockExclusiveSum<256>(ambiguous, lds, blockAmbiguous);
        if (blockOut + blockAmbiguous != 0) {  // (the same in every thread)
            if (threadIdx.x == 0) {
                bases[0] = blockOut ? atomicAdd(&state->taken, blockOut) : 0u;
                bases[1] = blockAmbiguous ? atomicAdd(&state->ambiguous, blockAmbiguous) : 0u;
            }
            __syncthreads();
            const u32 outBase = bases[0], ambiguousBase = bases[1];
            if (out + ambiguous != 0) {
                share.run([&](u32 image, auto position) {
                    const int mine = (int)topkDistanceBucket<Cfg>(image - floorImage - 1u);
                    if (mine > bucket) {
                        const u32 rank = outAt++;
                        if (rank < kTopkStageOut) {
                            stage[0][rank] = image;
                            if (Cfg::kPairs) stage[Cfg::kPairs ? 1 : 0][rank] = position();
                        } else if (outBase + rank < (u32)Cfg::kK) {
                            outKeys[outBase + rank] = topkKeyOfImage<Cfg>(image);
                            if (Cfg::kPairs) outValues[outBase + rank] = values[position()];
                        }
                    } else if (mine == bucket) {
                        const u32 rank = ambiguousAt++;
                        if (rank < kTopkStageAmbiguous) {
                            stage[0][kTopkStageOut + rank] = image;
                            if (Cfg::kPairs) stage[Cfg::kPairs ? 1 : 0][kTopkStageOut + rank] = position();
                        } else if (ambiguousBase + rank < Cfg::kAmbiguous) {
                            storeDeviceWide(&ambiguousImages[ambiguousBase + rank], image);  // read by the last block of this launch
                            if (Cfg::kPairs) storeDeviceWide(&ambiguousPositions[ambiguousBase + rank], position());
                        }
                    }
                });
            }
            __syncthreads();
            const u32 stagedOut = blockOut < kTopkStageOut ? blockOut : kTopkStageOut;
            for (u32 i = threadIdx.x; i < stagedOut; i += 256) {
                if (outBase + i < (u32)Cfg::kK) {  // (always, when the histogram and the list agree)
                    outKeys[outBase + i] = topkKeyOfImage<Cfg>(stage[0][i]);
                    if (Cfg::kPairs) outValues[outBase + i] = values[stage[Cfg::kPairs ? 1 : 0][i]];
                }
            }
            const u32 stagedAmbiguous = blockAmbiguous < kTopkStageAmbiguous ? blockAmbiguous : kTopkStageAmbiguous;
            for (u32 i = threadIdx.x; i < stagedAmbiguous; i += 256) {
                if (ambiguousBase + i < Cfg::kAmbiguous) {
                    storeDeviceWide(&ambiguousImages[ambiguousBase + i], stage[0][kTopkStageOut + i]);
                    if (Cfg::kPairs) storeDeviceWide(&ambiguousPositions[ambiguousBase + i], stage[Cfg::kPairs ? 1 : 0][kTopkStageOut + i]);
                }
            }
        }
    }
    partialsWritten();
    __syncthreads();
    if (threadIdx.x == 0) {
        const u32 before = __hip_atomic_fetch_add(&state->arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last = before + 1u == gridDim.x ? 1u : 0u;
        if (last) storeDeviceWide(&state->arrived, 0u);
    }
    __syncthreads();
    if (!last) return;
    if (bucket < 0) {
        // the rest of the answer are keys equal to F, from the positions noted by the second launch
        const u32* tiePositions = TopkCandidates<Cfg>::tiePositions(temp);
        for (u32 j = threadIdx.x; j < wanted; j += 256) {
            outKeys[listed + j] = topkKeyOfImage<Cfg>(floorImage);
            if (Cfg::kPairs) {
                const u32 position = tiePositions[j];
                outValues[listed + j] = values[position < Cfg::kTotal ? position : 0];
            }
        }
        return;
    }
    // The picked bucket holds `held` keys and `wanted` of them belong to the answer: the largest ones, into the output's last
    // `wanted` slots.  The keys are in the second list, which the block holds in registers when it is short (thread t: entries
    // t, t + 256, ...), or, when that list was too short, found by walking the candidates again for every step.
    const u32 held = loadDeviceWide(&state->ambiguous);
    const bool listedAll = held <= Cfg::kAmbiguous;
    u32 firstDistance, bits;
    topkBucketRange<Cfg>((u32)bucket, firstDistance, bits);
    const u32 firstImage = floorImage + 1u + firstDistance;  // images of the bucket: firstImage + [0, 2^bits)
    constexpr int E = kTopkAmbiguousPerThread;
    u32 offsets[E], places[E];
    const bool inRegisters = listedAll && held <= 256u * E;
    if (inRegisters) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
            offsets[e] = 0;
            places[e] = 0;
            const u32 i = (u32)e * 256 + threadIdx.x;
            if (i < held) {
                offsets[e] = loadDeviceWide(&ambiguousImages[i]) - firstImage;
                if (Cfg::kPairs) places[e] = loadDeviceWide(&ambiguousPositions[i]);
            }
        }
    }
    TopkWalk<Cfg> all;  // every candidate, for this block alone
    if (!listedAll) {
        all.issue(keys, temp, threadIdx.x / kWave, 256 / kWave);
        all.settle(floorImage);
    }
    auto walk = [&](const auto& visit) {  // visit(offset inside the bucket, position): the same order for every call
        if (inRegisters) {
#pragma unroll
            for (int e = 0; e < E; ++e) {
                if ((u32)e * 256 + threadIdx.x < held) visit(offsets[e], [&]() { return places[e]; });
            }
        } else if (listedAll) {
            for (u32 i = threadIdx.x; i < held; i += 256) {
                visit(loadDeviceWide(&ambiguousImages[i]) - firstImage, [&]() { return Cfg::kPairs ? loadDeviceWide(&ambiguousPositions[i]) : 0u; });
            }
        } else {
            all.run([&](u32 image, auto position) {
                if ((int)topkDistanceBucket<Cfg>(image - floorImage - 1u) == bucket) visit(image - firstImage, position);
            });
        }
    };
    // digits of the offset, from the top: 11 bits at a time
    u32 prefix = 0, remaining = wanted;
    for (int shift = (int)bits; shift > 0;) {
        const u32 digitBits = shift >= 11 ? 11u : (u32)shift;
        shift -= (int)digitBits;
        const u32 fixedBits = shift + digitBits >= 32 ? 0u : (0xffffffffu << (shift + digitBits));
        __syncthreads();
        for (u32 b = threadIdx.x; b < (1u << digitBits); b += 256) bins[b] = 0;
        __syncthreads();
        walk([&](u32 offset, auto) {
            if ((offset & fixedBits) == (prefix & fixedBits)) atomicAdd(&bins[(offset >> shift) & ((1u << digitBits) - 1u)], 1u);
        });
        __syncthreads();
        u32 above;
        const u32 digit = topkPickBucket([&](u32 b) { return bins[b]; }, 1u << digitBits, remaining, lds, above);
        prefix |= digit << shift;
        remaining -= above;
    }
    // `prefix` is the offset of the kK-th largest key; `remaining` keys equal to it belong to the answer
    u32 above = 0, ties = 0;
    walk([&](u32 offset, auto) {
        above += offset > prefix;
        ties += offset == prefix;
    });
    u32 total;
    u32 aboveAt = blockExclusiveSum<256>(above, lds, total) + ((u32)Cfg::kK - wanted);
    u32 tieAt = blockExclusiveSum<256>(ties, lds, total);
    auto slotOf = [&](u32 offset) {
        u32 slot = 0xffffffffu;
        if (offset > prefix) slot = aboveAt++;
        if (offset == prefix) {
            const u32 rank = tieAt++;
            if (rank < remaining) slot = (u32)Cfg::kK - remaining + rank;
        }
        return slot;
    };
    if (inRegisters) {  // the values of all entries are asked for before the first one is stored
        u32 slots[E], taken[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            slots[e] = (u32)e * 256 + threadIdx.x < held ? slotOf(offsets[e]) : 0xffffffffu;
            taken[e] = 0;
            if (Cfg::kPairs && slots[e] < (u32)Cfg::kK) taken[e] = values[places[e]];
        }
#pragma unroll
        for (int e = 0; e < E; ++e) {
            if (slots[e] < (u32)Cfg::kK) {
                outKeys[slots[e]] = topkKeyOfImage<Cfg>(firstImage + offsets[e]);
                if (Cfg::kPairs) outValues[slots[e]] = taken[e];
            }
        }
        return;
    }
    walk([&](u32 offset, auto position) {
        const u32 slot = slotOf(offset);
        if (slot < (u32)Cfg::kK) {
            outKeys[slot] = topkKeyOfImage<Cfg>(firstImage + offset);
            if (Cfg::kPairs) outValues[slot] = values[position()];
        }
    });
}

// ---- top-k of every row: one block per row ------------------------------------------------------------------------------------------
// Cfg additionally: kSegment (row length, <= kThreads * kItems), kK < kSegment; kItems counts single keys here.  Output row r
// holds kK keys at outKeys + r * kK.
template <typename Cfg>
__device__ __forceinline__ void topkRows(const typename Cfg::Raw* keys, const u32* values, typename Cfg::Raw* outKeys, u32* outValues) {
    __shared__ u32 bins[kTopkMaxBins];
    __shared__ u32 lds[8];
    __shared__ u32 counters[2];
    const u64 rowBase = (u64)blockIdx.x * Cfg::kSegment;
    u32 image[Cfg::kItems];
#pragma unroll
    for (int k = 0; k < Cfg::kItems; ++k) {
        const u32 p = (u32)k * Cfg::kThreads + threadIdx.x;
        image[k] = p < Cfg::kSegment ? topkImage<Cfg>(keys[rowBase + p]) : 0u;
    }
    u32 prefix = 0, remaining = (u32)Cfg::kK;
    int high = Cfg::kBits;  // digits below `high` are still open
    while (high > 0) {
        const int bits = Cfg::kBits == 32 ? (high > 10 ? 11 : 10) : 8;
        const int shift = high - bits;
        const u32 numBins = 1u << bits;
        for (u32 b = threadIdx.x; b < numBins; b += Cfg::kThreads) bins[b] = 0;
        __syncthreads();
        const u32 fixedBits = high >= 32 ? 0u : (0xffffffffu << high);
#pragma unroll
        for (int k = 0; k < Cfg::kItems; ++k) {
            const u32 p = (u32)k * Cfg::kThreads + threadIdx.x;
            if (p < Cfg::kSegment && (image[k] & fixedBits) == (prefix & fixedBits)) atomicAdd(&bins[(image[k] >> shift) & (numBins - 1u)], 1u);
        }
        __syncthreads();
        u32 above;
        const u32 bucket = topkPickBucket([&](u32 b) { return bins[b]; }, numBins, remaining, lds, above);
        prefix |= bucket << shift;
        remaining -= above;
        high = shift;
    }
    if (threadIdx.x < 2) counters[threadIdx.x] = 0;
    __syncthreads();
    const u32 firstTieSlot = (u32)Cfg::kK - remaining;
    typename Cfg::Raw* rowKeys = outKeys + (u64)blockIdx.x * Cfg::kK;
    u32* rowValues = Cfg::kPairs ? outValues + (u64)blockIdx.x * Cfg::kK : nullptr;
#pragma unroll
    for (int k = 0; k < Cfg::kItems; ++k) {
        const u32 p = (u32)k * Cfg::kThreads + threadIdx.x;
        if (p >= Cfg::kSegment) continue;
        u32 slot = 0xffffffffu;
        if (image[k] > prefix) {
            slot = atomicAdd(&counters[0], 1u);
        } else if (image[k] == prefix) {
            const u32 rank = atomicAdd(&counters[1], 1u);
            if (rank < remaining) slot = firstTieSlot + rank;
        }
        if (slot != 0xffffffffu) {
            rowKeys[slot] = keys[rowBase + p];
            if (Cfg::kPairs) rowValues[slot] = values[rowBase + p];
        }
    }
}

// ---- top-k of every row: one wavefront per row ---------------------------------------------------------------------------------------
// Rows of at most 64 * kVec * kItems keys (kVec = 16 bytes' worth of keys, at most 64 keys per lane; the kernel above takes
// longer rows).  A wavefront keeps its row in registers as images - lane l holds vector (it * 64 + l) of the row for every
// it < kItems, read with 16-byte loads at whatever alignment the row has; 16-bit keys stay two to a register - and finds the
// image of the kK-th largest key bit by bit: the largest T with count(image >= T) >= kK.  Nothing is shared between
// wavefronts, so the kernel has no barrier; a block of kThreads / 64 wavefronts takes that many consecutive rows.  The
// kernel is bound by instruction issue (a row of 4096 16-bit keys is 8 KiB: at the memory's rate a wavefront may spend about
// a dozen instructions per key), so the work per key is what is designed:
//   * Direct form: every lane counts its own keys against T (a compare and an add-with-carry per key and bit), the counts
//     meet in a wavefront sum: kBits steps over all kVec * kItems keys of a lane.
//   * Few keys wanted (kK <= 64, rows of at least two vectors per lane): every lane takes the maxima of the first and of the
//     second half of its keys, and the kK-th largest of those 128 maxima is a floor: kK different keys, at least, lie at or
//     above it.  For keys in random order that leaves about 1.4 kK candidates (for kK = 64 of 4096), which every lane pushes
//     on a small stack of its own in LDS (entry e of lane l at word e * 64 + l: no two lanes share a bank); the bit-by-bit
//     search and the output then run over the stacks alone.  A row that overflows a stack (many equal keys at the top, a
//     lane that holds most of the large keys) takes the direct form.
// Cfg additionally: kRows.  Positions inside a row: p = (it * 64 + lane) * kVec + e.
constexpr int kTopkRowStack = 8;  // candidates per lane
template <int N>
struct TopkSlots {
    static constexpr int value = N;
};

template <typename Cfg>
__device__ __forceinline__ u32 topkWaveSum(u32 x) {
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) x += __shfl_xor(x, d, kWave);
    return x;
}

typedef unsigned short topk_u16x2 __attribute__((ext_vector_type(2)));
typedef short topk_i16x2 __attribute__((ext_vector_type(2)));

// The images of the two 16-bit keys of one word, in place (see topkImage).
template <typename Cfg>
__device__ __forceinline__ u32 topkImagePair(u32 w) {
    if (Cfg::kKind == 1) w ^= 0x80008000u;
    if (Cfg::kKind == 2) {
        const topk_i16x2 negative = __builtin_bit_cast(topk_i16x2, w) >> (short)15;  // all ones in the halves whose sign is set
        w ^= __builtin_bit_cast(u32, negative) | 0x80008000u;
    }
    return Cfg::kLargest ? w : ~w;
}
__device__ __forceinline__ u32 topkMaxPair(u32 a, u32 b) {
    return __builtin_bit_cast(u32, __builtin_elementwise_max(__builtin_bit_cast(topk_u16x2, a), __builtin_bit_cast(topk_u16x2, b)));
}

// Output of one row from `SLOTS` keys per lane: image(j) counts only where live(j), position(j) is the key's place in the row.
// prefix: the image of the kK-th largest key; `remaining`: how many keys equal to it belong to the answer.
template <typename Cfg, int SLOTS, typename Image, typename Position, typename Live>
__device__ __forceinline__ void topkRowEmit(const Image& image, const Position& position, const Live& live, u32 prefix, u32 remaining,
                                            const u32* rowValuesIn, typename Cfg::Raw* rowKeys, u32* rowValues) {
    const int lane = threadIdx.x % kWave;
    const u32 firstTieSlot = (u32)Cfg::kK - remaining;
    u32 aboveAt = 0, tieAt = 0;
#pragma unroll
    for (int j = 0; j < SLOTS; ++j) {
        const bool isAbove = live(j) && image(j) > prefix, isTie = live(j) && image(j) == prefix;
        const u64 aboveVotes = __builtin_amdgcn_ballot_w64(isAbove), tieVotes = __builtin_amdgcn_ballot_w64(isTie);
        if ((aboveVotes | tieVotes) == 0) continue;
        u32 slot = 0xffffffffu;
        if (isAbove) slot = aboveAt + votesBelow(aboveVotes);
        if (isTie) {
            const u32 rank = tieAt + votesBelow(tieVotes);
            if (rank < remaining) slot = firstTieSlot + rank;
        }
        aboveAt += (u32)__builtin_popcountll(aboveVotes);
        tieAt += (u32)__builtin_popcountll(tieVotes);
        if (slot != 0xffffffffu) {
            rowKeys[slot] = topkKeyOfImage<Cfg>(image(j));  // the key's bits, from its image: no second read of the row
            if (Cfg::kPairs) rowValues[slot] = rowValuesIn[position(j)];
        }
    }
}

template <typename Cfg>
__device__ __forceinline__ void topkRowsWave(const typename Cfg::Raw* keys, const u32* values, typename Cfg::Raw* outKeys, u32* outValues) {
    typedef typename Cfg::Raw Raw;
    constexpr int V = Cfg::kVec, ITEMS = Cfg::kItems, R = V * ITEMS, kWaves = Cfg::kThreads / kWave;
    constexpr int P = Cfg::kBits == 16 ? 2 : 1;  // images per register
    constexpr int W = R / P;
    constexpr int E = kTopkRowStack;
    constexpr bool kFullRows = Cfg::kSegment == (u32)(kWave * R);  // no slot lies past the row
    // the floor wants two groups of whole vectors in every lane, all of the first group inside the row, and at most one wanted
    // key for every two groups
    constexpr bool kFloor = Cfg::kK <= (u64)kWave && ITEMS % 2 == 0 && Cfg::kSegment >= (u32)(kWave * R / 2) && R > 2 * E;
    constexpr bool kWideEntries = Cfg::kBits == 32;  // an entry of a stack is (image << 16 | slot), or two words for 32-bit images
    constexpr int kRows = 2 * E;  // a stack's height in LDS: E entries are the rule, up to twice as many take the wider search below
    __shared__ u32 stackEntries[kFloor ? kWaves * (kRows + 1) * kWave : 1];
    __shared__ u32 stackImages[kFloor && kWideEntries ? kWaves * (kRows + 1) * kWave : 1];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const u64 row = (u64)blockIdx.x * kWaves + wave;
    if (row >= Cfg::kRows) return;  // the whole wavefront leaves; nothing in this kernel waits for it
    const Raw* rowIn = keys + row * Cfg::kSegment;
    const u32* rowValuesIn = Cfg::kPairs ? values + row * Cfg::kSegment : nullptr;
    Raw* rowKeys = outKeys + row * Cfg::kK;
    u32* rowValues = Cfg::kPairs ? outValues + row * Cfg::kK : nullptr;

    const auto position = [&](int j) { return (u32)((j / V) * kWave + lane) * V + (u32)(j % V); };
    const auto live = [&](int j) { return kFullRows || position(j) < Cfg::kSegment; };
    u32 words[W];  // a test image is never 0: slots past the row hold 0 and count for nothing
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const u32 first = (u32)(it * kWave + lane) * V;
        Pack<Raw, V> x;
        const bool whole = kFullRows || first + V <= Cfg::kSegment;
        if (whole) {
            x.loadStreamUnaligned(rowIn + first);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) x.v[e] = first + e < Cfg::kSegment ? rowIn[first + e] : (Raw)0;
        }
        if constexpr (P == 2) {
#pragma unroll
            for (int e = 0; e < V; e += 2) {
                const u32 pair = (u32)x.v[e] | ((u32)x.v[e + 1] << 16);
                u32 images = topkImagePair<Cfg>(pair);
                if (!whole) images = (live(it * V + e) ? images & 0xffffu : 0u) | (live(it * V + e + 1) ? images & 0xffff0000u : 0u);
                words[(it * V + e) / 2] = images;
            }
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) words[it * V + e] = live(it * V + e) ? topkImage<Cfg>(x.v[e]) : 0u;
        }
    }
    const auto image = [&](int j) { return P == 2 ? (j % 2 ? words[j / 2] >> 16 : words[j / 2] & 0xffffu) : words[j]; };

    if constexpr (kFloor) {
        // the maxima of the two halves of the lane's keys
        u32 group[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            u32 best = words[t * (W / 2)];
#pragma unroll
            for (int w = 1; w < W / 2; ++w) {
                const u32 other = words[t * (W / 2) + w];
                best = P == 2 ? topkMaxPair(best, other) : (other > best ? other : best);
            }
            if (P == 2) best = (best >> 16) > (best & 0xffffu) ? best >> 16 : best & 0xffffu;
            group[t] = best;
        }
        // the kK-th largest of the 128 maxima (0 when fewer than kK groups hold a key: then every key is a candidate)
        u32 floorImage = 0;
#pragma unroll 1
        for (int bit = Cfg::kBits - 1; bit >= 0; --bit) {
            const u32 test = floorImage | (1u << bit);
            const u32 count = (u32)__builtin_popcountll(__builtin_amdgcn_ballot_w64(group[0] >= test)) +
                              (u32)__builtin_popcountll(__builtin_amdgcn_ballot_w64(group[1] >= test));
            if (count >= (u32)Cfg::kK) floorImage = test;
        }
        // every lane pushes its candidates on its own stack; pushes beyond the stack's height land in one more, unused, row
        u32* entries = stackEntries + wave * (kRows + 1) * kWave + lane;
        u32* wideImages = stackImages + (kWideEntries ? wave * (kRows + 1) * kWave + lane : 0);
        u32 height = 0;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            if (live(j) && image(j) >= floorImage) {
                const u32 at = (height < (u32)kRows ? height : (u32)kRows) * kWave;
                entries[at] = kWideEntries ? (u32)j : (image(j) << 16) | (u32)j;
                if (kWideEntries) wideImages[at] = image(j);
                ++height;
            }
        }
        // The search over the stacks, S entries of every lane in registers.  Almost every row fits E; a row in which some lane
        // holds more (2 in 1 000 rows of 4 096 normal keys, k = 64) would otherwise take the search over all registers below,
        // several times the time of a row that fits, and a few such rows near the end of the grid lengthen the whole launch.
        const auto overStacks = [&](auto slots) {
            constexpr int S = decltype(slots)::value;
            u32 cImage[S], cSlot[S];
#pragma unroll
            for (int e = 0; e < S; ++e) {
                const u32 entry = (u32)e < height ? entries[e * kWave] : 0u;
                cImage[e] = kWideEntries ? ((u32)e < height ? wideImages[e * kWave] : 0u) : entry >> 16;
                cSlot[e] = entry & 0xffffu;
            }
            // the wanted image lies between the floor and the row's largest image: the bits those two share are its own
            u32 largest = group[0] > group[1] ? group[0] : group[1];
#pragma unroll
            for (int d = kWave / 2; d > 0; d >>= 1) {
                const u32 other = __shfl_xor(largest, d, kWave);
                largest = other > largest ? other : largest;
            }
            const int open = 32 - __builtin_clz((floorImage ^ largest) | 1u);  // bits below this one may differ
            u32 prefix = open >= 32 ? 0u : (floorImage >> open) << open;
#pragma unroll 1
            for (int bit = open - 1; bit >= 0; --bit) {
                const u32 test = prefix | (1u << bit);
                u32 count = 0;
#pragma unroll
                for (int e = 0; e < S; ++e) count += (u32)__builtin_popcountll(__builtin_amdgcn_ballot_w64(cImage[e] >= test));
                if (count >= (u32)Cfg::kK) prefix = test;
            }
            const auto cLive = [&](int e) { return (u32)e < height; };
            u32 above = 0;
#pragma unroll
            for (int e = 0; e < S; ++e) above += (u32)__builtin_popcountll(__builtin_amdgcn_ballot_w64(cLive(e) && cImage[e] > prefix));
            topkRowEmit<Cfg, S>([&](int e) { return cImage[e]; },
                                [&](int e) { return ((cSlot[e] / (u32)V) * kWave + (u32)lane) * (u32)V + cSlot[e] % (u32)V; }, cLive, prefix,
                                (u32)Cfg::kK - above, rowValuesIn, rowKeys, rowValues);
        };
        if (__builtin_amdgcn_ballot_w64(height > (u32)E) == 0) {
            overStacks(TopkSlots<E>());
            return;
        }
        if (__builtin_amdgcn_ballot_w64(height > (u32)kRows) == 0) {
            overStacks(TopkSlots<kRows>());
            return;
        }
    }

    u32 prefix = 0;
#pragma unroll 1
    for (int bit = Cfg::kBits - 1; bit >= 0; --bit) {
        const u32 test = prefix | (1u << bit);
        u32 mine = 0;
#pragma unroll
        for (int j = 0; j < R; ++j) mine += image(j) >= test ? 1u : 0u;
        if (topkWaveSum<Cfg>(mine) >= (u32)Cfg::kK) prefix = test;
    }
    u32 mineAbove = 0;
#pragma unroll
    for (int j = 0; j < R; ++j) mineAbove += live(j) && image(j) > prefix ? 1u : 0u;
    const u32 above = topkWaveSum<Cfg>(mineAbove);
    topkRowEmit<Cfg, R>(image, position, live, prefix, (u32)Cfg::kK - above, rowValuesIn, rowKeys, rowValues);
}

}  // namespace thor
