// Stable least-significant-digit radix sort of (key, primitive index) pairs for 16-, 32- and 64-bit keys: 8 bits per pass,
// 9 bits for the 64-bit tile|depth keys (their 44 or 45 significant bits then take five passes instead of six).  Replaces cub::DeviceRadixSort::SortPairs(begin_bit = 0, end_bit)
// at R/src/hybrid_blend/inference.cu:145-153 (64-bit tile|depth keys:
// R/src/alpha_blend_global_ordering/inference.cu:117-124).
//
// One pass = three launches and no inter-block waiting:
//   digit_histogram : per-block digit counts, stored digit-major   hist[digit][block]
//   digit_row_scan  : one block per digit: exclusive scan along its row, row total
//   digit_scatter   : re-reads the block's items, ranks them stably with wave64 ballots, scatters
// Item order inside a block is (wave, round, lane); every rank below is computed in that order,
// which is what keeps equal keys in their input order.
#include "common.h"

namespace htgs {

constexpr int kSortItems = 16;                              // rounds per wave
// digit width per key type; kRadix digits, the first kRadix threads of a block own one digit each
template <typename KeyT> struct SortDigit { static constexpr int bits = sizeof(KeyT) == 8 ? 9 : 8; };
constexpr int kMaxRadix = 512;
constexpr int kScanThreads = 1024;
// Items per block = threads x 16 = 8192.  Longer blocks give longer runs per digit, i.e. fuller cache lines in the
// scatter; two blocks fit a CU's LDS for every key width (8-byte keys share one array between keys and values).
template <typename KeyT> struct SortShape { static constexpr int threads = 512; };
constexpr int kSortTileMin = 256 * kSortItems;              // sizes the histogram scratch (half a block: room to spare)

template <typename KeyT>
__device__ __forceinline__ uint32_t digit_of(KeyT k, int shift, uint32_t mask) { return (uint32_t)(k >> shift) & mask; }

// Workgroups go round the eight XCDs of the device in launch order, and each XCD has an L2 of its own.  Blocks that are
// neighbours in the input write neighbouring runs of every digit, a run being shorter than a cache line or two; handing
// every XCD a contiguous eighth of the input lets those partial lines meet in one L2 before they are written back.
constexpr uint32_t kXcds = 8;
__device__ __forceinline__ uint32_t xcd_contiguous_block(uint32_t launched, uint32_t n_blocks)
{
    const uint32_t per_xcd = (n_blocks + kXcds - 1) / kXcds;
    return (launched % kXcds) * per_xcd + launched / kXcds;           // >= n_blocks: nothing to do
}
inline uint32_t xcd_padded_grid(uint32_t n_blocks) { return (n_blocks + kXcds - 1) / kXcds * kXcds; }

template <typename KeyT, int THREADS = SortShape<KeyT>::threads, int BITS = SortDigit<KeyT>::bits>
__global__ void __launch_bounds__(THREADS) digit_histogram_kernel(const KeyT *__restrict__ keys, uint32_t *__restrict__ hist,
                                                                uint64_t n, uint32_t n_blocks, int shift, uint32_t mask)
{
    constexpr int kSortThreads = THREADS, kSortTile = kSortThreads * kSortItems, kRadix = 1 << BITS;
    static_assert(kRadix <= kSortThreads, "one thread per digit");
    __shared__ uint32_t counts[kRadix];
    const uint32_t block = xcd_contiguous_block(blockIdx.x, n_blocks);
    if (block >= n_blocks) return;
    if (threadIdx.x < kRadix) counts[threadIdx.x] = 0;
    __syncthreads();
    // the order of the keys does not matter here, so every thread reads 16-byte words: kPer keys at a time
    const uint64_t base = (uint64_t)block * kSortTile;
    constexpr int kPer = 16 / sizeof(KeyT);
    if (base + kSortTile <= n) {
        const uint4 *words = reinterpret_cast<const uint4 *>(keys + base);      // kSortTile keys are a multiple of 16 bytes
#pragma unroll
        for (int r = 0; r < kSortItems / kPer; ++r) {
            const uint4 word = words[r * kSortThreads + threadIdx.x];
            KeyT k[kPer];
            __builtin_memcpy(k, &word, 16);
#pragma unroll
            for (int j = 0; j < kPer; ++j) atomicAdd(&counts[digit_of(k[j], shift, mask)], 1u);
        }
    } else {
#pragma unroll
        for (int r = 0; r < kSortItems; ++r) {
            const uint64_t i = base + (uint64_t)r * kSortThreads + threadIdx.x;
            if (i < n) atomicAdd(&counts[digit_of(keys[i], shift, mask)], 1u);
        }
    }
    __syncthreads();
    if (threadIdx.x < kRadix) hist[(size_t)threadIdx.x * n_blocks + block] = counts[threadIdx.x];
}

// block d scans row d of hist in place (exclusive) and writes the row total to totals[d]
__global__ void __launch_bounds__(kScanThreads) digit_row_scan_kernel(uint32_t *__restrict__ hist, uint32_t *__restrict__ totals, uint32_t n_blocks)
{
    constexpr int kSortThreads = kScanThreads, kSortWaves = kScanThreads / kWave;
    __shared__ uint32_t wave_sums[kSortWaves];
    uint32_t *row = hist + (size_t)blockIdx.x * n_blocks;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    uint32_t carry = 0;
    for (uint32_t start = 0; start < n_blocks; start += kSortThreads) {
        const uint32_t i = start + threadIdx.x;
        const uint32_t v = i < n_blocks ? row[i] : 0u;
        uint32_t inc = v;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            const uint32_t t = __shfl_up(inc, d, kWave);
            if (lane >= d) inc += t;
        }
        if (lane == kWave - 1) wave_sums[wave] = inc;
        __syncthreads();
        uint32_t before = 0, all = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            const uint32_t s = wave_sums[w];
            if (w < wave) before += s;
            all += s;
        }
        __syncthreads();
        if (i < n_blocks) row[i] = carry + before + inc - v;
        carry += all;
    }
    if (threadIdx.x == 0) totals[blockIdx.x] = carry;
}

// RECTANGLES (a sort of one pass over the Gaussians, whose values are their indices in the order of the input): the
// Gaussians' tile rectangles, four 16-bit bounds each, travel with the pairs -- read in the order of the input, which is
// theirs, written in sorted order, with the number of tiles each covers beside them (none for the key `culled`, whose
// rectangle was never written).
template <typename KeyT, int THREADS = SortShape<KeyT>::threads, int BITS = SortDigit<KeyT>::bits, bool RECTANGLES = false>
__global__ void __launch_bounds__(THREADS) digit_scatter_kernel(
    const KeyT *__restrict__ keys_in, const uint32_t *__restrict__ vals_in, KeyT *__restrict__ keys_out, uint32_t *__restrict__ vals_out,
    const uint32_t *__restrict__ hist, const uint32_t *__restrict__ totals, uint64_t n, uint32_t n_blocks, int shift, uint32_t mask,
    bool last_pass = false, const uint2 *__restrict__ rectangles_in = nullptr, uint2 *__restrict__ rectangles_out = nullptr,
    uint32_t *__restrict__ counts_out = nullptr, uint32_t culled = 0)
{
    constexpr int kSortThreads = THREADS, kSortWaves = kSortThreads / kWave, kSortTile = kSortThreads * kSortItems;
    constexpr int kBits = BITS, kRadix = 1 << kBits, kDigitWaves = kRadix / kWave;
    // (16-bit counters: a block holds 8192 items; with 512 digits and 8-byte keys two blocks still fit a CU's LDS)
    __shared__ uint16_t counts[kSortWaves][kRadix];    // per wave: running digit count, later the wave's base inside the block
    __shared__ uint32_t digit_start[kRadix];           // first slot of each digit in the block-local order
    __shared__ uint32_t global_base[kRadix];           // where the block's run of each digit starts in the output
    __shared__ uint32_t wave_sums[kDigitWaves], wave_sums_g[kDigitWaves];
    // The block's items grouped by digit (stable).  8-byte keys: the values follow the keys through the same memory, in a
    // second round, which halves the block's LDS and allows 8192-item blocks here as well (sort of 9 M pairs 0.61 -> 0.47 ms); for the
    // short keys the second round costs more than the third resident block gains (0.24 -> 0.29 ms), so keys and values
    // have their own arrays there.
    constexpr bool kTwoRounds = sizeof(KeyT) == 8;
    __shared__ __attribute__((aligned(16))) unsigned char local_raw[kSortTile * (kTwoRounds ? sizeof(KeyT) : sizeof(KeyT) + 4)];
    KeyT *local_keys = reinterpret_cast<KeyT *>(local_raw);
    uint32_t *local_vals = reinterpret_cast<uint32_t *>(local_raw + (kTwoRounds ? 0 : kSortTile * sizeof(KeyT)));
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const uint32_t block = xcd_contiguous_block(blockIdx.x, n_blocks);
    if (block >= n_blocks) return;
    for (int c = threadIdx.x; c < kSortWaves * kRadix / 2; c += kSortThreads) reinterpret_cast<uint32_t *>(&counts[0][0])[c] = 0;
    __syncthreads();

    const uint64_t block_base = (uint64_t)block * kSortTile;
    const uint64_t wave_base = block_base + (uint64_t)wave * (kWave * kSortItems);
    KeyT key[kSortItems];
    uint32_t val[kSortItems];
    uint32_t rank[kSortItems];
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const uint64_t i = wave_base + (uint64_t)r * kWave + lane;
        const bool valid = i < n;
        // (the last reads of these buffers before they are written again: streaming, nothing to keep in the caches)
        key[r] = valid ? __builtin_nontemporal_load(keys_in + i) : (KeyT)0;
        val[r] = valid ? __builtin_nontemporal_load(vals_in + i) : 0u;
        const uint32_t d = digit_of(key[r], shift, mask);
        // lanes of this wave holding the same digit: per digit bit, keep the lanes whose bit equals this lane's.
        // (bit as 0 / ~0 by a signed bit-field extract; keep = peers & ~(vote ^ bit) is one three-input operation per half)
        const uint64_t present = __ballot(valid);
        uint32_t peers_lo = (uint32_t)present, peers_hi = (uint32_t)(present >> 32);
#pragma unroll
        for (int b = 0; b < kBits; ++b) {
            const uint32_t bit = (uint32_t)__builtin_amdgcn_sbfe((int)d, b, 1);
            const uint64_t vote = __ballot(bit != 0u);
            peers_lo &= ~((uint32_t)vote ^ bit);
            peers_hi &= ~((uint32_t)(vote >> 32) ^ bit);
        }
        const uint32_t below = __builtin_amdgcn_mbcnt_hi(peers_hi, __builtin_amdgcn_mbcnt_lo(peers_lo, 0u));
        uint32_t seen = 0;
        if (valid) {
            seen = counts[wave][d];
            if (below == 0) counts[wave][d] = (uint16_t)(seen + (uint32_t)(__builtin_popcount(peers_lo) + __builtin_popcount(peers_hi)));
        }
        rank[r] = seen + below;
    }
    __syncthreads();

    // thread d of the first four waves owns digit d: block-local start of the digit, base of each wave inside it,
    // global start of the run
    {
        const bool owner = threadIdx.x < kRadix;
        const uint32_t d = threadIdx.x & (kRadix - 1);
        uint32_t block_count = 0;
        if (owner) {
#pragma unroll
            for (int w = 0; w < kSortWaves; ++w) block_count += counts[w][d];
        }
        // exclusive scans over the 256 digits: of this block's counts (local order) and of the global totals
        uint32_t inc_local = block_count, inc_global = owner ? totals[d] : 0u;
        const uint32_t total = inc_global;
#pragma unroll
        for (int s = 1; s < kWave; s <<= 1) {
            const uint32_t tl = __shfl_up(inc_local, s, kWave), tg = __shfl_up(inc_global, s, kWave);
            if (lane >= s) { inc_local += tl; inc_global += tg; }
        }
        if (owner && lane == kWave - 1) { wave_sums[wave] = inc_local; wave_sums_g[wave] = inc_global; }
        __syncthreads();
        if (owner) {
            uint32_t before_l = 0, before_g = 0;
#pragma unroll
            for (int w = 0; w < kDigitWaves; ++w)
                if (w < wave) { before_l += wave_sums[w]; before_g += wave_sums_g[w]; }
            const uint32_t start = before_l + inc_local - block_count;
            digit_start[d] = start;
            global_base[d] = before_g + inc_global - total + hist[(size_t)d * n_blocks + block];
            uint32_t run = start;
#pragma unroll
            for (int w = 0; w < kSortWaves; ++w) {
                const uint32_t c = counts[w][d];
                counts[w][d] = (uint16_t)run;
                run += c;
            }
        }
    }
    __syncthreads();

    // group the block's items by digit in LDS (stable), ...
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const uint64_t i = wave_base + (uint64_t)r * kWave + lane;
        rank[r] += counts[wave][digit_of(key[r], shift, mask)];          // now the item's slot in the block-local order
        if (i < n) {
            local_keys[rank[r]] = key[r];
            if (!kTwoRounds) local_vals[rank[r]] = val[r];
        }
    }
    __syncthreads();
    // ... then stream them out: neighbouring threads write neighbouring addresses inside each digit's run
    const uint32_t n_local = n - block_base < (uint64_t)kSortTile ? (uint32_t)(n - block_base) : (uint32_t)kSortTile;
    uint32_t digits[kSortItems / 2];           // two rounds: the digits, two to a register, for the values' turn
#pragma unroll
    for (int r = 0; r < kSortItems / 2; ++r) digits[r] = 0u;
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const uint32_t i = (uint32_t)r * kSortThreads + threadIdx.x;
        if (i < n_local) {
            const KeyT k = local_keys[i];
            const uint32_t d = digit_of(k, shift, mask);
            const uint32_t pos = global_base[d] + (i - digit_start[d]);
            keys_out[pos] = k;
            if (kTwoRounds || RECTANGLES) digits[r / 2] |= d << (16 * (r % 2));
            if (!kTwoRounds) {
                // (the sorted values are read once more, by the walk of their tile's list: streaming stores leave the
                // caches to the records that the tiles share)
                if (last_pass) __builtin_nontemporal_store(local_vals[i], vals_out + pos);
                else vals_out[pos] = local_vals[i];
            }
        }
    }
    if constexpr (RECTANGLES) {
        static_assert(!kTwoRounds && sizeof(KeyT) == 4, "the rectangles take the room of the keys and the values");
        uint2 *local_rectangles = reinterpret_cast<uint2 *>(local_raw);
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kSortItems; ++r) {
            const uint64_t i = wave_base + (uint64_t)r * kWave + lane;
            if (i < n) local_rectangles[rank[r]] = key[r] == (KeyT)culled ? make_uint2(0u, 0u) : rectangles_in[i];
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kSortItems; ++r) {
            const uint32_t i = (uint32_t)r * kSortThreads + threadIdx.x;
            if (i < n_local) {
                const uint32_t d = digits[r / 2] >> (16 * (r % 2)) & 0xffffu;
                const uint32_t pos = global_base[d] + (i - digit_start[d]);
                const uint2 b = local_rectangles[i];                 // x0 | x1 << 16, y0 | y1 << 16
                rectangles_out[pos] = b;
                counts_out[pos] = ((b.x >> 16) - (b.x & 0xffffu)) * ((b.y >> 16) - (b.y & 0xffffu));
            }
        }
    }
    if (kTwoRounds) {
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kSortItems; ++r) {
            const uint64_t i = wave_base + (uint64_t)r * kWave + lane;
            if (i < n) local_vals[rank[r]] = val[r];
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kSortItems; ++r) {
            const uint32_t i = (uint32_t)r * kSortThreads + threadIdx.x;
            if (i < n_local) {
                const uint32_t d = digits[r / 2] >> (16 * (r % 2)) & 0xffffu;
                uint32_t *out = vals_out + (global_base[d] + (i - digit_start[d]));
                if (last_pass) __builtin_nontemporal_store(local_vals[i], out);
                else *out = local_vals[i];
            }
        }
    }
}

// streaming_result: the sorted values leave the last pass as streaming stores (the instance lists, which the blend reads once)
template <typename KeyT, int THREADS = SortShape<KeyT>::threads, int BITS = SortDigit<KeyT>::bits>
static int sort_pairs(hipStream_t s, void *const keys[2], uint32_t *const vals[2], uint32_t *sort_tmp, uint64_t n, int end_bit, int *selector,
                      bool streaming_result = false)
{
    constexpr int kSortThreads = THREADS, kSortTile = kSortThreads * kSortItems;
    const uint32_t n_blocks = (uint32_t)((n + kSortTile - 1) / kSortTile);
    constexpr int kBits = BITS, kRadix = 1 << kBits;
    uint32_t *hist = sort_tmp;
    uint32_t *totals = sort_tmp + (size_t)kRadix * n_blocks;
    int cur = 0;
    // the passes share the key's bits evenly (14 bits: 7 + 7 rather than 8 + 6): fewer digits per pass are longer runs
    // per digit in every block's output
    const int passes = (end_bit + kBits - 1) / kBits, step = passes > 0 ? (end_bit + passes - 1) / passes : kBits;
    for (int shift = 0; shift < end_bit; shift += step) {
        const int bits = end_bit - shift < step ? end_bit - shift : step;
        const uint32_t mask = (1u << bits) - 1u;
        const KeyT *kin = (const KeyT *)keys[cur];
        KeyT *kout = (KeyT *)keys[cur ^ 1];
        hipLaunchKernelGGL((digit_histogram_kernel<KeyT, THREADS, BITS>), dim3(xcd_padded_grid(n_blocks)), dim3(kSortThreads), 0, s, kin, hist, n, n_blocks, shift, mask);
        hipLaunchKernelGGL(digit_row_scan_kernel, dim3(kRadix), dim3(kScanThreads), 0, s, hist, totals, n_blocks);
        hipLaunchKernelGGL((digit_scatter_kernel<KeyT, THREADS, BITS>), dim3(xcd_padded_grid(n_blocks)), dim3(kSortThreads), 0, s, kin, vals[cur], kout, vals[cur ^ 1],
                           hist, totals, n, n_blocks, shift, mask, streaming_result && shift + step >= end_bit);
        cur ^= 1;
    }
    *selector = cur;
    return check_launch("sort");
}

int sort_u32_pairs_with_rectangles(void *stream, uint32_t *const keys[2], uint32_t *const vals[2], uint32_t *sort_tmp, uint64_t n, int bits,
                                   const uint16_t *rectangles_in, uint16_t *rectangles_out, uint32_t *counts_out, uint32_t culled)
{
    if (n == 0) return HTGS_OK;
    if (bits < 1 || bits > 8) return fail(HTGS_ERR_ARGUMENT, "sort: one pass takes at most eight bits");
    // (blocks of 4096 items, the smallest the kernels take: a few million pairs are three rounds of such blocks)
    constexpr int kThreads = kSortTileMin / kSortItems, kBits = 8, kRadix = 1 << kBits, kTile = kThreads * kSortItems;
    hipStream_t s = (hipStream_t)stream;
    const uint32_t n_blocks = (uint32_t)((n + kTile - 1) / kTile);
    uint32_t *hist = sort_tmp, *totals = sort_tmp + (size_t)kRadix * n_blocks;
    const uint32_t mask = (1u << bits) - 1u;
    hipLaunchKernelGGL((digit_histogram_kernel<uint32_t, kThreads, kBits>), dim3(xcd_padded_grid(n_blocks)), dim3(kThreads), 0, s, keys[0], hist, n, n_blocks, 0, mask);
    hipLaunchKernelGGL(digit_row_scan_kernel, dim3(kRadix), dim3(kScanThreads), 0, s, hist, totals, n_blocks);
    hipLaunchKernelGGL((digit_scatter_kernel<uint32_t, kThreads, kBits, true>), dim3(xcd_padded_grid(n_blocks)), dim3(kThreads), 0, s, keys[0], vals[0], keys[1],
                       vals[1], hist, totals, n, n_blocks, 0, mask, false, reinterpret_cast<const uint2 *>(rectangles_in),
                       reinterpret_cast<uint2 *>(rectangles_out), counts_out, culled);
    return check_launch("sort");
}

int sort_u32_pairs(void *stream, uint32_t *const keys[2], uint32_t *const vals[2], uint32_t *sort_tmp, uint64_t n, int end_bit, int digit_bits,
                   int *selector)
{
    *selector = 0;
    if (n == 0) return HTGS_OK;
    void *const k[2] = { keys[0], keys[1] };
    // a few million pairs: with 8-bit digits blocks of 4096 items, the smallest the kernels take, so that every compute
    // unit has several; 9-bit digits need a thread per digit (8192 items)
    if (digit_bits == 9) return sort_pairs<uint32_t, 512, 9>((hipStream_t)stream, k, vals, sort_tmp, n, end_bit, selector);
    return sort_pairs<uint32_t, kSortTileMin / kSortItems, 8>((hipStream_t)stream, k, vals, sort_tmp, n, end_bit, selector);
}

}  // namespace htgs

using namespace htgs;

extern "C" size_t htgs_sort_tmp_words(uint64_t n_instances)
{
    const uint64_t n_blocks = (n_instances + kSortTileMin - 1) / kSortTileMin;
    // (256 digits x blocks of half the real size = 512 digits x real blocks: either digit width fits)
    return (size_t)(256 * (n_blocks > 0 ? n_blocks : 1) + 2 * kMaxRadix);
}

extern "C" int htgs_sort_instances(const htgs_frame *f, int *selector)
{
    if (!f || !selector) return fail(HTGS_ERR_ARGUMENT, "htgs_sort_instances: null argument");
    if (f->mode < 0 || f->mode > 3) return fail(HTGS_ERR_MODE, "unsupported rasterizer mode");
    *selector = 0;
    if (f->n_instances == 0) return HTGS_OK;
    if (f->n_instances > 0xfffffffeull) return fail(HTGS_ERR_ARGUMENT, "htgs_sort_instances: more than 2^32-2 instances");
    if (!f->keys[0] || !f->keys[1] || !f->vals[0] || !f->vals[1] || !f->sort_tmp)
        return fail(HTGS_ERR_ARGUMENT, "htgs_sort_instances: null pointer");
    if (((uintptr_t)f->keys[0] | (uintptr_t)f->keys[1]) & 15) return fail(HTGS_ERR_ARGUMENT, "htgs_sort_instances: keys must be 16-byte aligned");
    const int end_bit = htgs_frame_end_bit(f);
    hipStream_t s = (hipStream_t)f->stream;
    switch (htgs_frame_key_bytes(f)) {
        case 8: return sort_pairs<uint64_t>(s, f->keys, f->vals, f->sort_tmp, f->n_instances, end_bit, selector, true);
        case 4: return sort_pairs<uint32_t>(s, f->keys, f->vals, f->sort_tmp, f->n_instances, end_bit, selector, true);
        default: return sort_pairs<uint16_t>(s, f->keys, f->vals, f->sort_tmp, f->n_instances, end_bit, selector, true);
    }
}
