// Stream compaction (select-flagged) and top-k selection, device-wide and over rows of one length.  Instantiated by run-time
// generated traits structs (placed after thor_device_prelude.h).  Replaces cub::DeviceSelect::Flagged and cub::DeviceTopK /
// the batched fixed-size top-k the reference calls (Utilities/TensorOperations/Cub/CubSelect.cu:26-50, CubTopK.cu:27-330).
//
// Select-flagged keeps the input's order.  A block owns a chunk of consecutive positions, 16 per thread: one launch counts the
// raised flags of every chunk, one block turns the counts into output offsets (and writes the total), and the last launch
// reads the flags again, ranks them inside the block with wavefront shuffles and copies the flagged elements to their places.
// No block waits for another one.
//
// Top-k is a radix selection on an order-preserving unsigned image of the key (sign handling for floats and signed integers;
// for "smallest" the image is complemented, so the code always looks for the largest images).  From the most significant
// 8-bit digit down: a histogram of the digit over the keys that still match the digits fixed so far, then the bucket that
// holds the k-th largest image is fixed.  After the last digit the image T of the k-th key and the number of keys equal to T
// that belong to the answer are known; one more pass writes every key above T and that many keys equal to T.  The answer is
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

// ---- select-flagged ----------------------------------------------------------------------------------------------------------
// Cfg: Word (u8 / u16 / u32: elements are copied as raw words), kTotal, kThreads (256), kItems (16), kChunks.
template <typename Cfg>
__device__ __forceinline__ u32 selectFlagBits(const u8* flags, u64 first) {
    // bit k set: the flag of position first + k is raised
    u32 bits = 0;
    if (first + Cfg::kItems <= Cfg::kTotal) {
#pragma unroll
        for (int k = 0; k < Cfg::kItems; ++k) bits |= (flags[first + k] != 0 ? 1u : 0u) << k;
    } else {
        for (int k = 0; k < Cfg::kItems; ++k)
            if (first + k < Cfg::kTotal) bits |= (flags[first + k] != 0 ? 1u : 0u) << k;
    }
    return bits;
}

template <typename Cfg>
__device__ __forceinline__ void selectCount(const u8* flags, u32* counts) {
    __shared__ u32 lds[Cfg::kThreads / kWave];
    const u64 first = ((u64)blockIdx.x * Cfg::kThreads + threadIdx.x) * Cfg::kItems;
    const u32 mine = first < Cfg::kTotal ? (u32)__builtin_popcount(selectFlagBits<Cfg>(flags, first)) : 0u;
    u32 total;
    (void)blockExclusiveSum<Cfg::kThreads>(mine, lds, total);
    if (threadIdx.x == 0) counts[blockIdx.x] = total;
}

// One block of 1024 threads: counts[kChunks] -> bases[kChunks] (exclusive), the grand total -> *numSelected.
template <typename Cfg>
__device__ __forceinline__ void selectOffsets(const u32* counts, u32* bases, u32* numSelected) {
    __shared__ u32 lds[1024 / kWave];
    u32 carry = 0;
    for (u64 c0 = 0; c0 < Cfg::kChunks; c0 += 1024) {
        const u64 c = c0 + threadIdx.x;
        const u32 mine = c < Cfg::kChunks ? counts[c] : 0u;
        u32 total;
        const u32 before = blockExclusiveSum<1024>(mine, lds, total);
        if (c < Cfg::kChunks) bases[c] = carry + before;
        carry += total;
    }
    if (threadIdx.x == 0) *numSelected = carry;
}

template <typename Cfg>
__device__ __forceinline__ void selectScatter(const typename Cfg::Word* in, const u8* flags, const u32* bases, typename Cfg::Word* out) {
    __shared__ u32 lds[Cfg::kThreads / kWave];
    const u64 first = ((u64)blockIdx.x * Cfg::kThreads + threadIdx.x) * Cfg::kItems;
    const u32 bits = first < Cfg::kTotal ? selectFlagBits<Cfg>(flags, first) : 0u;
    u32 total;
    u32 at = bases[blockIdx.x] + blockExclusiveSum<Cfg::kThreads>((u32)__builtin_popcount(bits), lds, total);
#pragma unroll
    for (int k = 0; k < Cfg::kItems; ++k) {
        if (bits & (1u << k)) out[at++] = in[first + k];
    }
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

// The bucket of a 256-bin histogram that holds the `wanted`-th largest digit (1-based, wanted <= the histogram's total), found
// by the 256 threads of a block: thread t looks at bin 255 - t.  Returns the bucket in every thread; `above` receives the
// number of entries in larger buckets.  `lds`: 4 + 2 words.
__device__ __forceinline__ u32 topkPickBucket(u32 binCount, u32 wanted, u32* lds, u32& above) {
    u32 total;
    const u32 before = blockExclusiveSum<256>(binCount, lds, total);  // entries in larger bins
    if (before < wanted && wanted <= before + binCount) {
        lds[4] = 255u - threadIdx.x;
        lds[5] = before;
    }
    __syncthreads();
    const u32 bucket = lds[4];
    above = lds[5];
    __syncthreads();
    return bucket;
}

// ---- device-wide top-k -----------------------------------------------------------------------------------------------------------
// Cfg: Raw (u8 / u16 / u32 word of the key), kKind, kBits, kLargest, kTotal, kK (already capped at kTotal, > 0), kPairs, kItems
// (keys per thread of the gathering pass).  Temporary storage: 256 histogram words, then the state words below.
struct TopkState {
    u32 prefix;     // the digits fixed so far, in place
    u32 remaining;  // the rank (1-based) of the wanted key among the keys that match the prefix
    u32 taken;      // output slots handed out to keys above the threshold
    u32 ties;       // keys equal to the threshold seen so far by the gathering pass
};

template <typename Cfg>
__device__ __forceinline__ void topkInit(u32* temp) {
    temp[threadIdx.x] = 0;
    if (threadIdx.x == 0) {
        TopkState* state = reinterpret_cast<TopkState*>(temp + 256);
        state->prefix = 0;
        state->remaining = (u32)Cfg::kK;
        state->taken = 0;
        state->ties = 0;
    }
}

// Histogram of the digit at `shift` over the keys whose higher digits equal the prefix.  Blocks stride over the keys.
template <typename Cfg>
__device__ __forceinline__ void topkHistogram(const typename Cfg::Raw* keys, u32* temp, u32 shift) {
    __shared__ u32 bins[256];
    bins[threadIdx.x] = 0;
    __syncthreads();
    const u32 prefix = reinterpret_cast<const TopkState*>(temp + 256)->prefix;
    const u32 fixedBits = shift + 8 >= 32 ? 0u : (0xffffffffu << (shift + 8));
    for (u64 i = (u64)blockIdx.x * 256 + threadIdx.x; i < Cfg::kTotal; i += (u64)gridDim.x * 256) {
        const u32 image = topkImage<Cfg>(keys[i]);
        if ((image & fixedBits) == (prefix & fixedBits)) atomicAdd(&bins[(image >> shift) & 255u], 1u);
    }
    __syncthreads();
    const u32 mine = bins[threadIdx.x];
    if (mine != 0) atomicAdd(&temp[threadIdx.x], mine);
}

// One block of 256 threads: fixes the digit at `shift` and clears the histogram for the next pass.
template <typename Cfg>
__device__ __forceinline__ void topkPick(u32* temp, u32 shift) {
    __shared__ u32 lds[8];
    TopkState* state = reinterpret_cast<TopkState*>(temp + 256);
    const u32 wanted = state->remaining, prefix = state->prefix;
    u32 above;
    const u32 bucket = topkPickBucket(temp[255 - threadIdx.x], wanted, lds, above);
    temp[threadIdx.x] = 0;
    if (threadIdx.x == 0) {
        state->prefix = prefix | (bucket << shift);
        state->remaining = wanted - above;
    }
}

// Writes the keys above the threshold image (kK - remaining of them) and `remaining` of the keys equal to it.
template <typename Cfg>
__device__ __forceinline__ void topkGather(const typename Cfg::Raw* keys, const u32* values, u32* temp, typename Cfg::Raw* outKeys, u32* outValues) {
    __shared__ u32 lds[Cfg::kThreads / kWave];
    __shared__ u32 bases[2];
    TopkState* state = reinterpret_cast<TopkState*>(temp + 256);
    const u32 threshold = state->prefix, wantedTies = state->remaining, firstTieSlot = (u32)Cfg::kK - wantedTies;
    const u64 first = ((u64)blockIdx.x * Cfg::kThreads + threadIdx.x) * Cfg::kItems;
    u32 aboveBits = 0, tieBits = 0;
    for (int k = 0; k < Cfg::kItems; ++k) {
        if (first + k < Cfg::kTotal) {
            const u32 image = topkImage<Cfg>(keys[first + k]);
            aboveBits |= (image > threshold ? 1u : 0u) << k;
            tieBits |= (image == threshold ? 1u : 0u) << k;
        }
    }
    u32 blockAbove, blockTies;
    u32 aboveAt = blockExclusiveSum<Cfg::kThreads>((u32)__builtin_popcount(aboveBits), lds, blockAbove);
    u32 tieAt = blockExclusiveSum<Cfg::kThreads>((u32)__builtin_popcount(tieBits), lds, blockTies);
    if (threadIdx.x == 0) {
        bases[0] = blockAbove ? atomicAdd(&state->taken, blockAbove) : 0u;
        bases[1] = blockTies ? atomicAdd(&state->ties, blockTies) : 0u;
    }
    __syncthreads();
    aboveAt += bases[0];
    tieAt += bases[1];
    for (int k = 0; k < Cfg::kItems; ++k) {
        u32 slot = 0xffffffffu;
        if (aboveBits & (1u << k)) slot = aboveAt++;
        if (tieBits & (1u << k)) {
            if (tieAt < wantedTies) slot = firstTieSlot + tieAt;
            ++tieAt;
        }
        if (slot != 0xffffffffu) {
            outKeys[slot] = keys[first + k];
            if (Cfg::kPairs) outValues[slot] = values[first + k];
        }
    }
}

// ---- top-k of every row: one block per row ------------------------------------------------------------------------------------------
// Cfg additionally: kSegment (row length, <= kThreads * kItems), kK < kSegment.  Output row r holds kK keys at outKeys + r * kK.
template <typename Cfg>
__device__ __forceinline__ void topkRows(const typename Cfg::Raw* keys, const u32* values, typename Cfg::Raw* outKeys, u32* outValues) {
    __shared__ u32 bins[256];
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
    for (int shift = Cfg::kBits - 8; shift >= 0; shift -= 8) {
        bins[threadIdx.x] = 0;
        __syncthreads();
        const u32 fixedBits = shift + 8 >= 32 ? 0u : (0xffffffffu << (shift + 8));
#pragma unroll
        for (int k = 0; k < Cfg::kItems; ++k) {
            const u32 p = (u32)k * Cfg::kThreads + threadIdx.x;
            if (p < Cfg::kSegment && (image[k] & fixedBits) == (prefix & fixedBits)) atomicAdd(&bins[(image[k] >> shift) & 255u], 1u);
        }
        __syncthreads();
        u32 above;
        const u32 bucket = topkPickBucket(bins[255 - threadIdx.x], remaining, lds, above);
        prefix |= bucket << shift;
        remaining -= above;
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

}  // namespace thor
