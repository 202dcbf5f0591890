// The walks of the three modes with 8x8 tiles (HYBRID_BLEND, ALPHA_BLEND_FIRST_K, OIT_BLEND), the inference kernels with one
// wave per tile and the kernels for tiles with very long lists.  The latter are shared by the inference and the training
// forward pass: what is done with a pixel's finished core, tail or sums is a function object of the launch (Finish), and
// the size of a record of `prim` a template parameter (REC4, in 16-byte words).
// Restates blend_cu of R/include/hybrid_blend/kernels/inference.cuh:78-216,
// R/include/alpha_blend_first_k/kernels/inference.cuh:78-206 and R/include/oit_blend/kernels/inference.cuh:78-177.
#pragma once

#include "blend_common.h"

namespace htgs {

__device__ __forceinline__ void store_pixel(float *__restrict__ image, float *__restrict__ depths, uint32_t w, uint32_t h,
                                            uint32_t x, uint32_t y, bool chw, float r, float g, float b, float depth)
{
    const size_t pix = (size_t)w * y + x, np = (size_t)w * h;
    r = saturate(r); g = saturate(g); b = saturate(b);
    if (chw) { image[pix] = r; image[np + pix] = g; image[2 * np + pix] = b; }
    else { image[3 * pix] = r; image[3 * pix + 1] = g; image[3 * pix + 2] = b; }
    if (depths) depths[pix] = depth;
}

// ---------------------------------------------------------------------------------------------
// HYBRID_BLEND: K nearest fragments with alpha >= 1/20 are alpha-blended in depth order, everything
// else is merged order-independently into one tail fragment behind them.
// ---------------------------------------------------------------------------------------------
// The tail of a pixel: colour sums (every fragment's alpha * colour; the final core's share is taken out when the pixel
// is composited), alpha sum, depth sum and transmittance of what is not in the core.
struct HybridTail {
    float T, c0, c1, c2, alpha, depth;
};
__device__ __forceinline__ void hybrid_tail_init(HybridTail &t) { t.T = 1.0f; t.c0 = t.c1 = t.c2 = t.alpha = t.depth = 0.0f; }
// what joins the tail: a fragment itself, the entry it pushed out of the core, or an empty slot (alpha 0)
template <bool FAST>
__device__ __forceinline__ void hybrid_tail_add(HybridTail &t, float depth, float alpha)
{
    t.alpha += alpha;
    if (!FAST) t.depth = __builtin_fmaf(depth, alpha, t.depth);      // (not used for the median depth)
    t.T *= 1.0f - alpha;
}
template <int K>
__device__ __forceinline__ void hybrid_core_init(float (&cd)[K], float (&ca)[K], float (&ci)[K])
{
#pragma unroll
    for (int i = 0; i < K; ++i) {
        cd[i] = __FLT_MAX__; ca[i] = 0.0f; ci[i] = 0.0f;
        asm volatile("" : "+v"(cd[i]), "+v"(ca[i]), "+v"(ci[i]));      // one register per slot, never a 16-wide tuple
    }
}

// The walk over instances [first, last) of a tile's list (whole batches of 64 from `first` on) by one wave: lanes =
// pixels, by quadrants.  A core slot holds depth, alpha and the Gaussian's index (an exchange moves three registers); the
// colours are fetched once, when the sorted core is blended.  Every fragment's alpha * colour goes into the tail sums
// when it is evaluated, and the share of the fragments that end up in the core is taken out again at the end, so an
// entry pushed out of the core needs no colour: its alpha and depth, which the tail also needs, are in the slot.
// SOLO: the wave is the whole workgroup (its barriers are the workgroup's).
// TIES (the walks of blend_hybrid_long_kernel): `tie` receives the least depth at which an entry was pushed out of the core
// that is exactly as deep as the entry that is now last.  (A candidate as deep as the last slot of a share's own core
// needs no note: at least K fragments of the share are not farther and came earlier, so it is in nobody's final core.)
// PIXELS: only the pixels of the lanes in pixel_lanes are wanted; instances that do not reach one of them are left out
// (the other lanes' cores and tails come out incomplete).
template <int K, bool FAST, bool SOLO, bool TIES = false, bool PIXELS = false, int REC4 = HTGS_PRIM_FLOATS / 4>
__device__ __forceinline__ void hybrid_walk(TileStageQ &st, QuadrantLists &ql, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
                                            uint32_t first, uint32_t last, uint32_t lane, const PixelTerms &pt, float cx, float cy, float (&cd)[K],
                                            float (&ca)[K], float (&ci)[K], HybridTail &tail, float *tie = nullptr, uint64_t pixel_lanes = 0)
{
    constexpr int MODE = HTGS_MODE_HYBRID_BLEND;
    constexpr int N = kStageSlots;
    tile_list_walk<MODE, true, PIXELS ? kCullPixels : kCullAlpha, SOLO, REC4, FAST>(st, ql, prim, inst, first, last, lane, cx, cy, [&](uint32_t addr) {
        // cut-off and alpha threshold are tested together: the lanes of a quadrant that its instance does not
        // reach run along to the second test (one exec level less for the scalar unit to manage; the staging
        // cull leaves hardly a turn in which no lane passes, so there is nothing to skip)
        TileFrag f;
        bool fragment;
        if constexpr (FAST) fragment = tile_frag_fast<MODE, N>(addr, pt, f);
        else {
            const bool in_reach = tile_frag_cutoff<N>(addr, pt, f);
            f.den_rcp = frag_rcp<FAST>(f.den);
            fragment = tile_frag_alpha<MODE, FAST>(stage_opacity<N>(addr), f) && in_reach;
        }
        const float4 col = stage_row<N, 5>(addr);
        if (!fragment) return;
        float depth = tile_frag_depth<N>(addr, pt, f);
        float p3 = f.alpha;
        tail.c0 = __builtin_fmaf(p3, col.x, tail.c0);
        tail.c1 = __builtin_fmaf(p3, col.y, tail.c1);
        tail.c2 = __builtin_fmaf(p3, col.z, tail.c2);
        if (depth < cd[K - 1] && f.alpha >= kMinAlphaCore) {
            float pi = col.w;
            if constexpr (FAST && !TIES) core_quick_walk<K>(depth, p3, pi, cd, ca, ci);
            else core_exchange_walk<K>(depth, p3, pi, cd, ca, ci);
            if (TIES && p3 > 0.0f && depth == cd[K - 1]) *tie = depth < *tie ? depth : *tie;
        }
        hybrid_tail_add<FAST>(tail, depth, p3);
    }, pixel_lanes);
}

// ---------------------------------------------------------------------------------------------
// HYBRID_BLEND's core as sorted 64-bit keys (the kernel with one wave per tile, inference).  A slot is one register pair:
// the high word holds the depth, the low word alpha as a fraction of 19 to 23 bits (rounded: an absolute error of 2^-20 at
// most, 2^-24 in the tiles with short lists; KeyFormat) above the instance's place in the tile's list (at most 13 bits: the
// lists this kernel walks are no longer than the threshold beyond which a tile goes to the other kernel, at most
// kPackedListMost).  Floats of one sign order like their bit patterns
// and so do the doubles made of (depth, low word): one step of the insertion is slot' = min(carried, slot), carried' =
// max(carried, slot), two instructions without exec masks or moves (a third of the exchange of three registers), and what
// is pushed out carries the alpha that the tail needs.  The Gaussian's index, which only the final core needs, is looked
// up from the place in the list when the pixel is composited.  Which of two fragments of equal depth comes first is
// decided by the low word here, not by the reference's insertion: the image-only fast path leaves it at that; with exact
// arithmetic the walk notes where it can matter (hybrid_key_walk) and such pixels are walked again.
// ---------------------------------------------------------------------------------------------
typedef double CoreKey;
constexpr uint32_t kPackedListMost = 8192;
// How a tile's keys divide the low word (the same for every pixel of the tile: scalar registers).  The place takes the bits
// that the length of the tile's list asks for, nine at least, and alpha the other 19 to 23: a fraction of 23 bits is within
// 2^-24 of the float, so in the tiles with up to 512 instances a key holds its alpha almost as the float does.
struct KeyFormat {
    uint32_t shift, place_mask;     // bits of the place; 2^shift - 1
    float one, one_rcp;             // 2^(32 - shift) - 1, the fraction that stands for alpha = 1, and its reciprocal
};
__device__ __forceinline__ KeyFormat key_format(uint32_t list_length)      // 1 .. kPackedListMost
{
    KeyFormat f;
    f.shift = 32u - (uint32_t)__builtin_clz((list_length - 1u) | 0x1ffu);
    f.place_mask = (1u << f.shift) - 1u;
    f.one = (float)((1u << (32u - f.shift)) - 1u);
    f.one_rcp = 1.0f / f.one;
    return f;
}
__device__ __forceinline__ float key_depth(CoreKey k) { return bits_to_float((uint32_t)__double2hiint(k)); }
__device__ __forceinline__ uint32_t key_low(CoreKey k) { return (uint32_t)__double2loint(k); }
__device__ __forceinline__ CoreKey make_key(float depth, uint32_t low) { return __hiloint2double((int)float_to_bits(depth), (int)low); }
__device__ __forceinline__ uint32_t key_pack(float alpha, uint32_t place, const KeyFormat &f)      // alpha in [0, 1]
{
    return (uint32_t)__builtin_fmaf(alpha, f.one, 0.5f) << f.shift | place;
}
__device__ __forceinline__ float key_alpha(uint32_t low, const KeyFormat &f) { return (float)(low >> f.shift) * f.one_rcp; }
__device__ __forceinline__ void key_step(CoreKey &carried, CoreKey &slot)
{
    CoreKey out;
    asm("v_max_f64 %0, %2, %1\n\tv_min_f64 %1, %2, %1" : "=&v"(out), "+v"(slot) : "v"(carried));
    carried = out;
}
template <int K>
__device__ __forceinline__ void core_key_walk(CoreKey &carried, CoreKey (&core)[K])
{
#pragma unroll
    for (int g0 = 0; g0 < K; g0 += kInsertGroup) {
        const int g1 = g0 + kInsertGroup < K ? g0 + kInsertGroup : K;
        if (K > kInsertGroup && !__any(key_depth(carried) < key_depth(core[g1 - 1]))) continue;
#pragma unroll
        for (int i = g0; i < g1; ++i) key_step(carried, core[i]);
    }
}
// FAST or not is the arithmetic of a fragment alone.  Without FAST, `tie` receives the least depth at which the keys may not
// have kept what the reference's insertion keeps: an entry left the core that is exactly as deep as the entry that is now
// last (which of the two stays is the insertion's choice; it matters if the finished core still reaches that deep.  Two
// such entries that both stay are seen in the finished core, key_core_tied).
template <int K, bool FAST, bool SOLO, int REC4 = HTGS_PRIM_FLOATS / 4, bool AHEAD = false>
__device__ __forceinline__ void hybrid_key_walk(TileStageQ &st, QuadrantLists &ql, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
                                                uint32_t first, uint32_t last, uint32_t lane, const PixelTerms &pt, float cx, float cy,
                                                CoreKey (&core)[K], HybridTail &tail, float &tie, const KeyFormat &fmt)
{
    constexpr int MODE = HTGS_MODE_HYBRID_BLEND;
    constexpr int N = kStageSlots;
    tile_list_walk<MODE, true, kCullAlpha, SOLO, REC4, FAST, true, AHEAD>(st, ql, prim, inst, first, last, lane, cx, cy, [&](uint32_t addr) {
        TileFrag f;
        bool fragment;
        if constexpr (FAST) fragment = tile_frag_fast<MODE, N>(addr, pt, f);
        else {
            const bool in_reach = tile_frag_cutoff<N>(addr, pt, f);
            f.den_rcp = frag_rcp<FAST>(f.den);
            fragment = tile_frag_alpha<MODE, FAST>(stage_opacity<N>(addr), f) && in_reach;
        }
        const float4 col = stage_row<N, 5>(addr);
        if (!fragment) return;
        float depth = tile_frag_depth<N>(addr, pt, f);
        float p3 = f.alpha;
        if (depth < key_depth(core[K - 1]) && f.alpha >= kMinAlphaCore) {
            // (a fragment that enters the core has the alpha that its key holds from here on: what the colour sums
            // receive now is what is taken out of them again for the entries of the finished core)
            // (the fast path's alpha is opacity * 2^t with the opacity held to 1 and t <= 0 up to the rounding of the staged
            // quadratic: held to 1 here, the fraction has no room for more; the exact path's is held to 1 when it is evaluated)
            if constexpr (FAST) p3 = p3 < 1.0f ? p3 : 1.0f;
            const uint32_t low = key_pack(p3, float_to_bits(col.w) - first, fmt);
            p3 = key_alpha(low, fmt);
            tail.c0 = __builtin_fmaf(p3, col.x, tail.c0);
            tail.c1 = __builtin_fmaf(p3, col.y, tail.c1);
            tail.c2 = __builtin_fmaf(p3, col.z, tail.c2);
            CoreKey carried = make_key(depth, low);
            core_key_walk<K>(carried, core);
            depth = key_depth(carried);
            p3 = key_alpha(key_low(carried), fmt);
            if constexpr (!FAST) tie = p3 > 0.0f && depth == key_depth(core[K - 1]) && depth < tie ? depth : tie;
        } else {
            tail.c0 = __builtin_fmaf(p3, col.x, tail.c0);
            tail.c1 = __builtin_fmaf(p3, col.y, tail.c1);
            tail.c2 = __builtin_fmaf(p3, col.z, tail.c2);
        }
        hybrid_tail_add<FAST>(tail, depth, p3);
    });
}
// two entries of the finished core are exactly as deep as each other (their order is the reference's insertion's to choose)
template <int K>
__device__ __forceinline__ bool key_core_tied(const CoreKey (&core)[K], const KeyFormat &fmt)
{
    bool tied = false;
#pragma unroll
    for (int i = 0; i + 1 < K; ++i) tied = tied || (key_low(core[i + 1]) >> fmt.shift != 0u && __double2hiint(core[i]) == __double2hiint(core[i + 1]));
    return tied;
}
// the finished keys as the three arrays the composite takes
template <int K>
__device__ __forceinline__ void key_core_unpack(const CoreKey (&core)[K], const uint32_t *__restrict__ inst, uint32_t first, uint32_t last, float (&cd)[K],
                                                float (&ca)[K], float (&ci)[K], const KeyFormat &fmt)
{
#pragma unroll
    for (int i = 0; i < K; ++i) {
        const uint32_t low = key_low(core[i]), place = low & fmt.place_mask;
        cd[i] = key_depth(core[i]);
        ca[i] = key_alpha(low, fmt);
        ci[i] = ca[i] > 0.0f && first + place < last ? bits_to_float(inst[first + place]) : 0.0f;
    }
}

// core + tail -> pixel (R/include/hybrid_blend/kernels/inference.cuh:172-213)
template <int K, int REC4 = HTGS_PRIM_FLOATS / 4>
__device__ __forceinline__ void hybrid_composite(const float4 *__restrict__ prim, float (&cd)[K], float (&ca)[K], float (&ci)[K], HybridTail &tail,
                                                 float *__restrict__ image, float *__restrict__ depths, uint32_t width, uint32_t height,
                                                 uint32_t x, uint32_t y, int chw, int median)
{
    constexpr int MODE = HTGS_MODE_HYBRID_BLEND;
    float tail0 = tail.c0, tail1 = tail.c1, tail2 = tail.c2;
    const float tail3 = tail.alpha, depth_tail = tail.depth, T_tail = tail.T;
    float r = 0.0f, g = 0.0f, b = 0.0f, depth_pixel = 0.0f, T_core = 1.0f;
    float4 cc[K];
#pragma unroll
    for (int i = 0; i < K; ++i)
        cc[i] = ca[i] > 0.0f ? prim[(size_t)float_to_bits(ci[i]) * REC4 + 4] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
    for (int i = 0; i < K; ++i) {                      // the core's share of the colour sums
        tail0 = __builtin_fmaf(-ca[i], cc[i].x, tail0);
        tail1 = __builtin_fmaf(-ca[i], cc[i].y, tail1);
        tail2 = __builtin_fmaf(-ca[i], cc[i].z, tail2);
    }
    tail0 = clamp_pos(tail0); tail1 = clamp_pos(tail1); tail2 = clamp_pos(tail2);   // colours are >= 0, so is the exact difference
#pragma unroll
    for (int i = 0; i < K; ++i) {
        if (T_core >= kTransmittanceThreshold) {
            const float w = T_core * ca[i];
            r = __builtin_fmaf(w, cc[i].x, r);
            g = __builtin_fmaf(w, cc[i].y, g);
            b = __builtin_fmaf(w, cc[i].z, b);
            if (median) depth_pixel = (T_core > 0.5f && cd[i] < __FLT_MAX__) ? cd[i] : depth_pixel;
            else depth_pixel = __builtin_fmaf(w, cd[i], depth_pixel);
            T_core *= 1.0f - ca[i];
        }
    }
    float total_alpha = 0.0f;
    if (!median) total_alpha = 1.0f - T_core;
    if (T_core >= kTransmittanceThreshold && tail3 >= ModeCfg<MODE>::min_alpha) {
        const float weight_tail = T_core * (1.0f - T_tail);
        const float wn = weight_tail * (1.0f / tail3);
        r = __builtin_fmaf(wn, tail0, r);
        g = __builtin_fmaf(wn, tail1, g);
        b = __builtin_fmaf(wn, tail2, b);
        if (!median) { depth_pixel = __builtin_fmaf(wn, depth_tail, depth_pixel); total_alpha += weight_tail; }
    }
    if (!median) depth_pixel = total_alpha > 0.0f ? depth_pixel / total_alpha : 0.0f;
    store_pixel(image, depths, width, height, x, y, chw, r, g, b, depth_pixel);
}

// what the inference kernels do with a pixel's finished core and tail: composite and store
struct HybridImage {
    float *image, *depths;
    uint32_t width, height;
    int chw, median;
    template <int K>
    __device__ __forceinline__ void operator()(const float4 *__restrict__ prim, uint32_t, const TilePixel &px, float (&cd)[K], float (&ca)[K], float (&ci)[K],
                                               HybridTail &tail) const
    {
        hybrid_composite<K>(prim, cd, ca, ci, tail, image, depths, width, height, px.x, px.y, chw, median);
    }
};

// One tile by one wave with the core as keys; finish(prim, tile, px, cd, ca, ci, tail) is called once per pixel inside the
// image.  Without FAST, the pixels at which fragments of exactly equal depth met where they decide the core (a pixel or
// two in a tile in a hundred) are walked again afterwards, over the instances that reach one of them, with the
// reference's insertion.
template <int K, bool FAST, int REC4, typename Finish>
__device__ __forceinline__ void hybrid_tile_by_keys(TileStageQ &st, QuadrantLists &ql, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
                                                    uint32_t tile, uint32_t first, uint32_t last, uint32_t lane, const TilePixel &px, uint32_t grid_w,
                                                    uint32_t width, uint32_t height, const Finish &finish)
{
    HybridTail tail;
    hybrid_tail_init(tail);
    float cd[K], ca[K], ci[K];                 // ci: the index's bit pattern
    CoreKey core[K];
#pragma unroll
    for (int i = 0; i < K; ++i) {
        core[i] = make_key(__FLT_MAX__, 0u);
        asm volatile("" : "+v"(core[i]));      // one register pair per slot, never a wide tuple
    }
    float tie = __FLT_MAX__;
    const KeyFormat fmt = key_format(last > first ? last - first : 1u);
    hybrid_key_walk<K, FAST, true, REC4, true>(st, ql, inst, prim, first, last, lane, px.pt, px.cx, px.cy, core, tail, tie, fmt);
    if constexpr (FAST) {
        if (!px.inside) return;
        key_core_unpack<K>(core, inst, first, last, cd, ca, ci, fmt);
        finish(prim, tile, px, cd, ca, ci, tail);
    } else {
        const bool again = px.inside && ((tie < __FLT_MAX__ && tie <= key_depth(core[K - 1])) || key_core_tied<K>(core, fmt));
        const uint64_t again_lanes = __ballot(again);
        key_core_unpack<K>(core, inst, first, last, cd, ca, ci, fmt);
        if (px.inside && !again) finish(prim, tile, px, cd, ca, ci, tail);
        if (again_lanes == 0) return;
        // (the lane and its pixel are worked out afresh, so that nothing the first walk keeps in registers has to
        // live through the pixels' finish for the sake of this rare second walk)
        uint32_t lane_again = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
        asm volatile("" : "+v"(lane_again));
        const TilePixel px_again = quadrant_tile_pixel(tile, grid_w, lane_again, width, height);
        hybrid_tail_init(tail);
        hybrid_core_init<K>(cd, ca, ci);
        hybrid_walk<K, false, true, false, true, REC4>(st, ql, inst, prim, first, last, lane_again, px_again.pt, px_again.cx, px_again.cy, cd, ca, ci, tail, nullptr,
                                                       again_lanes);
        if ((again_lanes >> lane_again & 1ull) != 0) finish(prim, tile, px_again, cd, ca, ci, tail);
    }
}

// ---------------------------------------------------------------------------------------------
// Tiles with very long lists (HYBRID_BLEND, ALPHA_BLEND_FIRST_K and OIT_BLEND, which walk all of a list): the kernel
// with one wave per tile puts a tile whose list is longer than long_threshold on a list instead of walking it, if the
// caller provided that list, and a second launch of workgroups of kLongWaves waves takes those: one wave walks one tile at some
// 200 ns per instance once it has a SIMD to itself, so a single list of 300 000 instances would otherwise hold the
// launch for 70 ms.
// long_tiles[0] = entries on the list, [1..3] = work counters, [4] = workgroups done, [5] = unused -- all zeroed with the
// ranges and again by the last workgroup of the second launch; [6], [7] = tiles with pixels settled by a second look / walked again in one piece (upper half: of these, after a second look that ran out of
// room) since the ranges were made (for the tests); then 2 n_tiles words for the entries (tile | part << 20 |
// (parts - 1) << 25: a tile is on the list once per part, and the parts beyond the first of all tiles together are held
// to n_tiles, so the list cannot overflow) and n_tiles words that count a tile's finished parts.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kLongHeader = 8, kLongRounds = 3, kLongParts = 32;
constexpr int kLongWaves = 16;
// waves of a workgroup of the K-buffer kernels: sixteen share a compute unit's registers at 128 a lane, which a K-buffer of
// 32 slots (96 registers) leaves too few of; eight have 256
template <int K> constexpr int long_waves() { return K > 16 ? 8 : kLongWaves; }
constexpr uint32_t kLongListDefault = 8192;
// What a workgroup leaves of its part of a list, in 64-lane rows: HYBRID's core, tail and the depth of a tie.
template <int K> constexpr uint32_t long_part_words() { return (3u * K + 7u) * 64u; }
// The parts a list of this length is walked in by separate workgroups (1: by one).  A part is at least four times the
// threshold long, long enough that what the parts leave behind (part_words each) fits into the list's own stretch of
// the spare value buffer, and at least as long as the frame's average list (part_floor = instances / tiles, rounded
// up): the parts beyond the first of all tiles together then cannot exceed the number of tiles, which is what the list
// of entries has room for, and how a list is split is a function of its length and of the frame alone -- no budget
// shared between workgroups, nothing that depends on the order in which they run.
__device__ __forceinline__ uint32_t long_parts(uint32_t length, uint32_t long_threshold, uint32_t part_words, uint32_t part_floor)
{
    uint32_t least = 4u * long_threshold > part_words ? 4u * long_threshold : part_words;
    least = least > part_floor ? least : part_floor;
    const uint32_t parts = length / least;
    return parts < 1u ? 1u : parts > kLongParts ? kLongParts : parts;
}
// (one lane of the tile's wave) enters the tile; part_floor = 0: in one part
__device__ __forceinline__ void long_tile_enter(uint32_t *__restrict__ long_tiles, uint32_t tile, uint32_t n_tiles, uint32_t length,
                                                uint32_t long_threshold, uint32_t part_words, uint32_t part_floor)
{
    const uint32_t parts = part_floor != 0u ? long_parts(length, long_threshold, part_words, part_floor) : 1u;
    if (parts > 1u) long_tiles[kLongHeader + 2u * n_tiles + tile] = 0u;
    const uint32_t at = kLongHeader + atomicAdd(long_tiles, parts);
    for (uint32_t part = 0; part < parts; ++part) long_tiles[at + part] = tile | part << 20 | (parts - 1u) << 25;
}
// An entry of the list: part `part` of `parts` of the tile's list [tile_first, tile_last) is [first, last), whole batches of 64.
struct LongEntry {
    uint32_t tile, part, parts, tile_first, tile_last, first, last;
};
// The workgroups take the entries off the list one by one, the longest first: the list is gone through kLongRounds times
// (a counter per round, `round` starts at 0), and a round takes the entries of its length class only -- more than 16, more
// than 4 and up to 4 times the threshold.  The lists differ in length by orders of magnitude, and the launch ends when the
// workgroup with the longest one does.  Called by all threads of the workgroup (barriers inside); false: the list is
// through.  The last workgroup to find that clears the list's header, so that the list is empty again for the next blend of
// this frame (htgs_blend called again without htgs_extract_ranges).
__device__ __forceinline__ bool long_tile_take(const uint32_t *long_tiles, const uint32_t *__restrict__ ranges, uint32_t long_threshold,
                                               uint32_t &round, uint32_t *s_next, LongEntry &e)
{
    const uint32_t n_long = long_tiles[0];
    for (;;) {
        __syncthreads();
        if (threadIdx.x == 0) *s_next = atomicAdd(const_cast<uint32_t *>(long_tiles) + 1 + round, 1u);
        __syncthreads();
        const uint32_t j = (uint32_t)__builtin_amdgcn_readfirstlane((int)*s_next);     // (the same in every lane: what follows stays in scalar registers)
        if (j >= n_long) {
            if (++round < kLongRounds) continue;
            if (threadIdx.x == 0) {
                uint32_t *header = const_cast<uint32_t *>(long_tiles);
                __threadfence();
                if (atomicAdd(header + 4, 1u) == gridDim.x - 1) {
#pragma unroll
                    for (uint32_t k = 0; k < 6; ++k) header[k] = 0u;
                }
            }
            return false;
        }
        const uint32_t entry = long_tiles[kLongHeader + j];
        e.tile = entry & 0xfffffu; e.part = entry >> 20 & 31u; e.parts = (entry >> 25) + 1u;
        e.tile_first = ranges[2 * e.tile]; e.tile_last = ranges[2 * e.tile + 1];
        const uint32_t tile_batches = (e.tile_last - e.tile_first + 63u) / 64u;
        e.first = e.tile_first + 64u * (uint32_t)((uint64_t)tile_batches * e.part / e.parts);
        e.last = e.tile_first + 64u * (uint32_t)((uint64_t)tile_batches * (e.part + 1u) / e.parts);
        e.last = e.last < e.tile_last ? e.last : e.tile_last;
        const uint32_t length = e.last - e.first;
        const uint32_t length_class = length > 16u * long_threshold ? 0u : length > 4u * long_threshold ? 1u : 2u;
        if (length_class == round) return true;
    }
}
// share of wave `wave` of [first, last): whole batches of 64
__device__ __forceinline__ void long_wave_share(uint32_t first, uint32_t last, uint32_t wave, uint32_t &share_first, uint32_t &share_last,
                                                uint32_t waves = kLongWaves)
{
    const uint32_t n_batches = (last - first + 63u) / 64u;
    share_first = first + 64u * (uint32_t)((uint64_t)n_batches * wave / waves);
    share_last = first + 64u * (uint32_t)((uint64_t)n_batches * (wave + 1) / waves);
    share_last = share_last < last ? share_last : last;
}
// One of several parts is done and the first wave has written what it left (and called __threadfence()): whether the
// other parts are there already, so that this workgroup ends the tile.  Called by all threads; the first wave calls
// __threadfence() again before it reads the other parts.
__device__ __forceinline__ bool long_part_done(const uint32_t *long_tiles, uint32_t n_tiles, const LongEntry &e, uint32_t *s_whole)
{
    if (threadIdx.x == 0) *s_whole = atomicAdd(const_cast<uint32_t *>(long_tiles) + kLongHeader + 2u * n_tiles + e.tile, 1u) == e.parts - 1u;
    __syncthreads();
    return *s_whole != 0;
}

// One wave per tile; the tiles with very long lists are left to blend_hybrid_long_kernel.
// KEYS (with long_tiles and a threshold of no more than kPackedListMost): the core as sorted 64-bit keys, hybrid_tile_by_keys.
// (K = 32: two registers a slot leave room for four waves per SIMD instead of three -- cfg2 442 -> 488 FPS)
template <int K, bool FAST, bool KEYS = false>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(K <= 16 ? 5 : KEYS ? 4 : 3))) blend_hybrid_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
    float *__restrict__ image, float *__restrict__ depths, uint32_t width, uint32_t height, uint32_t grid_w, int chw, int median,
    uint32_t *__restrict__ long_tiles, uint32_t long_threshold, uint32_t part_floor, const uint32_t *__restrict__ tile_order)
{
    __shared__ TileStageQ st;
    __shared__ QuadrantLists ql;
    const uint32_t tile = block_tile(tile_order);
    const uint32_t lane = threadIdx.x;
    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    if (long_tiles != nullptr && last - first > long_threshold) {
        if (lane == 0) long_tile_enter(long_tiles, tile, gridDim.x, last - first, long_threshold, long_part_words<K>(), part_floor);
        return;
    }
    const TilePixel px = quadrant_tile_pixel(tile, grid_w, lane, width, height);
    if constexpr (KEYS) {
        hybrid_tile_by_keys<K, FAST, HTGS_PRIM_FLOATS / 4>(st, ql, inst, prim, tile, first, last, lane, px, grid_w, width, height,
                                                           HybridImage{ image, depths, width, height, chw, median });
    } else {
        HybridTail tail;
        hybrid_tail_init(tail);
        float cd[K], ca[K], ci[K];                 // ci: the index's bit pattern
        hybrid_core_init<K>(cd, ca, ci);
        hybrid_walk<K, FAST, true>(st, ql, inst, prim, first, last, lane, px.pt, px.cx, px.cy, cd, ca, ci, tail);
        if (!px.inside) return;
        hybrid_composite<K>(prim, cd, ca, ci, tail, image, depths, width, height, px.x, px.y, chw, median);
    }
}

__device__ __forceinline__ float wave_total(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ float wave_product(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v *= __shfl_xor(v, o);
    return v;
}
constexpr int kAgainPixels = 2;       // pixels a pass of pixels_again takes at once
constexpr int kAgainMost = 8;         // pixels of a tile beyond which they are walked again in one piece instead

// The second look at the pixels of pixel_lanes, whose cores the merge could not settle: lanes = instances.  Every wave
// goes through its share [first, last) of the tile's list once per kAgainPixels pixels and evaluates each instance at these
// pixels with the walk's own arithmetic.  A fragment that cannot be in the pixel's final core -- farther than the merged
// core's last entry (last_depth[pixel]: which depths the K nearest have is certain, which fragments of equal depth they
// are is not), or too faint for the core -- joins the pixel's tail in sums[][j] (this wave's sums and product, to be combined
// over the waves; the colour sums take every fragment); the others, the few that decide the core, are put down in list
// order at `out` as (pixel, depth, alpha, index) for the walk's insertion to be replayed on them alone.  Returns their
// number, or ~0u when `room` entries were not enough.  pass_done(pixels) is called, by the whole workgroup, after each pass.
// ALPHA_BLEND_FIRST_K has no tail: its fragments that are not farther than the core's last entry are put down, no sums.
template <int MODE, bool FAST, int REC4, typename PassDone>
__device__ __forceinline__ uint32_t pixels_again(TileStage<64> &st, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, uint32_t first,
                                                        uint32_t last, uint32_t lane, float cx, float cy, uint64_t pixel_lanes,
                                                        const float *last_depth, float (*sums)[6], uint32_t *__restrict__ out, uint32_t room,
                                                        PassDone pass_done)
{
    constexpr bool kTail = MODE == HTGS_MODE_HYBRID_BLEND;
    uint32_t n_out = 0;
    bool fits = true;
    for (uint64_t todo = pixel_lanes; todo != 0;) {
        uint32_t pixel[kAgainPixels];
        PixelTerms pt[kAgainPixels];
        float farthest[kAgainPixels];
        HybridTail acc[kAgainPixels];
#pragma unroll
        for (int j = 0; j < kAgainPixels; ++j) {
            pixel[j] = todo != 0 ? (uint32_t)__builtin_ctzll(todo) : 64u;
            todo &= todo - 1;                                       // (0 stays 0)
            uint32_t local_x, local_y;
            quadrant_pixel(pixel[j] & 63u, local_x, local_y);
            pt[j] = pixel_terms(local_x, local_y, 8);
            farthest[j] = last_depth[pixel[j] & 63u];
            hybrid_tail_init(acc[j]);
        }
        for (uint32_t base = first; base < last; base += 64) {
            wave_lds_sync();
            tile_stage_load<MODE, 64, true, kCullNone, true, REC4>(st, prim, inst, base + lane, last, lane, cx, cy);
            wave_lds_sync();
            const bool loaded = base + lane < last;
            const uint32_t addr = stage_address(st) + 16u * lane;
#pragma unroll
            for (int j = 0; j < kAgainPixels; ++j) {
                if (pixel[j] >= 64u) continue;                      // (wave-uniform)
                TileFrag f;
                const bool in_reach = tile_frag_cutoff<64>(addr, pt[j], f);
                f.den_rcp = frag_rcp<FAST>(f.den);
                const float4 col = stage_row<64, 5>(addr);
                const bool fragment = tile_frag_alpha<MODE, FAST>(stage_opacity<64>(addr), f) && in_reach && loaded;
                const float depth = tile_frag_depth<64>(addr, pt[j], f);
                bool decides = false;
                if (fragment) {
                    if (kTail) {
                        acc[j].c0 = __builtin_fmaf(f.alpha, col.x, acc[j].c0);
                        acc[j].c1 = __builtin_fmaf(f.alpha, col.y, acc[j].c1);
                        acc[j].c2 = __builtin_fmaf(f.alpha, col.z, acc[j].c2);
                    }
                    decides = depth <= farthest[j] && (!kTail || f.alpha >= kMinAlphaCore);
                    if (kTail && !decides) hybrid_tail_add<false>(acc[j], depth, f.alpha);
                }
                const uint64_t deciding = __ballot(decides);
                if (deciding != 0) {
                    const uint32_t at = n_out + (uint32_t)__popcll(deciding & ((1ull << lane) - 1ull));
                    n_out += (uint32_t)__popcll(deciding);
                    fits = fits && n_out <= room;
                    if (decides && fits) {
                        out[4 * at] = pixel[j]; out[4 * at + 1] = float_to_bits(depth); out[4 * at + 2] = float_to_bits(f.alpha);
                        out[4 * at + 3] = float_to_bits(col.w);
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; kTail && j < kAgainPixels; ++j) {
            const float T = wave_product(acc[j].T), c0 = wave_total(acc[j].c0), c1 = wave_total(acc[j].c1), c2 = wave_total(acc[j].c2),
                        alpha = wave_total(acc[j].alpha), depth = wave_total(acc[j].depth);
            if (lane == 0) { sums[j][0] = T; sums[j][1] = c0; sums[j][2] = c1; sums[j][3] = c2; sums[j][4] = alpha; sums[j][5] = depth; }
        }
        pass_done(pixel);
    }
    return fits ? n_out : ~0u;
}

// A core, a tail and a tie depth (3K + 7 rows of 64 lanes at from[]) join the running ones: they cover the stretch of the
// list that follows.
template <int K, bool FAST>
__device__ __forceinline__ void hybrid_merge(const float *from, uint32_t lane, float (&cd)[K], float (&ca)[K], float (&ci)[K], HybridTail &tail,
                                             float &tie)
{
    constexpr bool kTies = !FAST;
    from += lane;
#pragma unroll
    for (int i = 0; i < K; ++i) {
        float depth = from[(3 * i) * 64], alpha = from[(3 * i + 1) * 64], index = from[(3 * i + 2) * 64];
        if (alpha > 0.0f) {                    // a filled slot
            if (kTies && depth == cd[K - 1]) tie = depth < tie ? depth : tie;
            if (depth < cd[K - 1]) {
                core_exchange_walk<K>(depth, alpha, index, cd, ca, ci);
                if (kTies && alpha > 0.0f && depth == cd[K - 1]) tie = depth < tie ? depth : tie;
            }
            hybrid_tail_add<FAST>(tail, depth, alpha);
        }
    }
    tail.T *= from[(3 * K) * 64];
    tail.c0 += from[(3 * K + 1) * 64]; tail.c1 += from[(3 * K + 2) * 64]; tail.c2 += from[(3 * K + 3) * 64];
    tail.alpha += from[(3 * K + 4) * 64]; tail.depth += from[(3 * K + 5) * 64];
    const float other = from[(3 * K + 6) * 64];
    tie = other < tie ? other : tie;
}
// The long tiles: a workgroup of kLongWaves waves takes a tile, every wave walks a contiguous share of the list (whole
// batches of 64) into a core and a tail of its own, and the shares are then merged into the first wave's, in list
// order, through LDS: the entries of the incoming core enter the running core like fragments (what does not stay in
// the core, of either, joins the tail), the tails add up.  The pixel gets the K nearest fragments of the whole list and
// everything else in its tail, as in a single walk; what differs from the single walk is the order in which the tail's
// sums are added (rounding) and which of two stored fragments of exactly equal depth is kept when a nearer one arrives.
// finish(prim, tile, px, cd, ca, ci, tail) is called by the lanes of the first wave whose pixels lie inside the image, once
// per pixel, with the pixel's finished core and tail.
template <int K, bool FAST, int REC4, typename Finish>
__global__ void __launch_bounds__(64 * long_waves<K>()) blend_hybrid_long_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, const uint32_t *long_tiles,
    uint32_t width, uint32_t height, uint32_t grid_w, uint32_t *__restrict__ shortlist, uint32_t long_threshold, const Finish finish)
{
    constexpr int kWaves = long_waves<K>();
    __shared__ TileStageQ st[kWaves];
    __shared__ QuadrantLists ql[kWaves];
    __shared__ float s_merge[3 * K + 7][64];          // one wave's core, tail and least depth of a tie, lane-minor
    __shared__ uint32_t s_next;
    __shared__ uint32_t s_redo[2];                    // the pixels (lanes) to walk again
    __shared__ uint32_t s_short[kWaves];          // how many instances of each share reach one of them
    __shared__ uint32_t s_whole;                      // this workgroup finished the last part of its tile
    __shared__ float s_last_depth[64];                // depth of the merged core's last entry
    __shared__ float s_sums[kWaves][kAgainPixels][6], s_tails[64][6];   // tails of the pixels looked at again: per wave, whole
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
    if (long_tiles[0] == 0) return;                   // (the ordinary frame)
    const uint32_t n_tiles = grid_w * ((height + 7u) / 8u);
    uint32_t round = 0;
    LongEntry entry;
    while (long_tile_take(long_tiles, ranges, long_threshold, round, &s_next, entry)) {
        // (the same in every lane; said so, they live in scalar registers through the walks that follow)
        const auto uniform = [](uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
        const uint32_t tile = uniform(entry.tile), part = uniform(entry.part), parts = uniform(entry.parts), tile_first = uniform(entry.tile_first),
                       tile_last = uniform(entry.tile_last);
        uint32_t first = uniform(entry.first), last = uniform(entry.last);
        const TilePixel px = quadrant_tile_pixel(tile, grid_w, lane, width, height);
        uint32_t n_batches = (last - first + 63u) / 64u;
        uint32_t seg_first, seg_last;
        long_wave_share(first, last, wave, seg_first, seg_last, kWaves);
        constexpr bool kTies = !FAST;
        HybridTail tail;
        hybrid_tail_init(tail);
        float cd[K], ca[K], ci[K];
        hybrid_core_init<K>(cd, ca, ci);
        float tie = __FLT_MAX__;                        // least depth at which two fragments of equal depth met at the end of a core
        hybrid_walk<K, FAST, false, kTies, false, REC4>(st[wave], ql[wave], inst, prim, seg_first, seg_last, lane, px.pt, px.cx, px.cy, cd, ca, ci, tail, &tie);
        for (uint32_t s = 1; s < (uint32_t)kWaves; ++s) {
            __syncthreads();                               // the buffer is free
            if (wave == s) {
#pragma unroll
                for (int i = 0; i < K; ++i) { s_merge[3 * i][lane] = cd[i]; s_merge[3 * i + 1][lane] = ca[i]; s_merge[3 * i + 2][lane] = ci[i]; }
                s_merge[3 * K][lane] = tail.T; s_merge[3 * K + 1][lane] = tail.c0; s_merge[3 * K + 2][lane] = tail.c1;
                s_merge[3 * K + 3][lane] = tail.c2; s_merge[3 * K + 4][lane] = tail.alpha; s_merge[3 * K + 5][lane] = tail.depth;
                s_merge[3 * K + 6][lane] = tie;
            }
            __syncthreads();
            if (wave == 0) hybrid_merge<K, FAST>(&s_merge[0][0], lane, cd, ca, ci, tail, tie);
        }
        if (parts > 1u) {
            // One of several parts: what it came to goes to the tile's stretch of the spare value buffer (which is as long as the
            // list and unused until pixels are walked again), and the workgroup that finds the other parts there already
            // merges them all, in list order, and goes on with the whole tile.
            float *const left = reinterpret_cast<float *>(shortlist + tile_first);
            if (wave == 0) {
                float *mine = left + (size_t)part * long_part_words<K>() + lane;
#pragma unroll
                for (int i = 0; i < K; ++i) { mine[(3 * i) * 64] = cd[i]; mine[(3 * i + 1) * 64] = ca[i]; mine[(3 * i + 2) * 64] = ci[i]; }
                mine[(3 * K) * 64] = tail.T; mine[(3 * K + 1) * 64] = tail.c0; mine[(3 * K + 2) * 64] = tail.c1;
                mine[(3 * K + 3) * 64] = tail.c2; mine[(3 * K + 4) * 64] = tail.alpha; mine[(3 * K + 5) * 64] = tail.depth;
                mine[(3 * K + 6) * 64] = tie;
                __threadfence();
            }
            if (!long_part_done(long_tiles, n_tiles, entry, &s_whole)) continue;
            if (wave == 0) {
                __threadfence();
                hybrid_tail_init(tail);
                hybrid_core_init<K>(cd, ca, ci);
                tie = __FLT_MAX__;
                for (uint32_t other = 0; other < parts; ++other)
                    hybrid_merge<K, FAST>(left + (size_t)other * long_part_words<K>(), lane, cd, ca, ci, tail, tie);
            }
            first = tile_first; last = tile_last; n_batches = (last - first + 63u) / 64u;
            long_wave_share(first, last, wave, seg_first, seg_last, kWaves);
            __syncthreads();                               // (the parts are read before the shortlist overwrites them)
        }
        if (kTies) {
            // Equal depths matter where they can change the final core: a tie no deeper than its last entry (both
            // fragments of a deeper tie end in the tail either way), or two equal depths next to each other in it.
            // There the merged walk and the single walk can keep different fragments, or keep them in another order: the
            // reference's insertion lets a displaced entry hop over a stored one of exactly equal depth.  Such pixels (a
            // handful per frame of very long lists) are walked again in one piece by the first wave, over the instances
            // that reach one of them; every wave picks those out of its share first (into the tile's own stretch of the
            // shortlist, in list order), since the walk of one wave alone is bound by the latency of staging.
            bool redo = false;
            if (wave == 0) {
                redo = tie <= cd[K - 1];
#pragma unroll
                for (int i = 0; i + 1 < K; ++i) redo = redo || (ca[i + 1] > 0.0f && cd[i] == cd[i + 1]);
                const uint64_t lanes = __ballot(redo);
                if (lane == 0) { s_redo[0] = (uint32_t)lanes; s_redo[1] = (uint32_t)(lanes >> 32); }
            }
            __syncthreads();
            const uint64_t redo_lanes = (uint64_t)s_redo[0] | (uint64_t)s_redo[1] << 32;
            if (redo_lanes != 0) {
                bool others_done = false;                       // the pixels that need no second look are composited
                if (shortlist != nullptr && __popcll(redo_lanes) <= kAgainMost) {
                    // All waves look at these pixels again, lanes = instances (pixels_again), into the tile's stretch of
                    // the shortlist, four words per fragment that decides a core: a wave has a quarter as many entries as
                    // its share has instances, which is ample unless depths coincide by the hundred -- then, and when the
                    // pixels are many (a pass over the list serves kAgainPixels of them), the other way below is taken.
                    others_done = true;
                    if (wave == 0) {
                        s_last_depth[lane] = cd[K - 1];
                        if (px.inside && !redo) finish(prim, tile, px, cd, ca, ci, tail);
                    }
                    __syncthreads();
                    const uint32_t listed = pixels_again<HTGS_MODE_HYBRID_BLEND, false, REC4>(
                        reinterpret_cast<TileStage<64> &>(st[wave]), inst, prim, seg_first, seg_last, lane, px.cx, px.cy, redo_lanes, s_last_depth, s_sums[wave], shortlist + seg_first,
                        (seg_last - seg_first) / 4u, [&](const uint32_t (&pixel)[kAgainPixels]) {
                            __syncthreads();
                            if (wave == 0 && lane < (uint32_t)kAgainPixels) {      // the waves' sums of a pixel, in list order
                                uint32_t mine = pixel[0];
#pragma unroll
                                for (int j = 1; j < kAgainPixels; ++j) mine = lane == (uint32_t)j ? pixel[j] : mine;
                                if (mine < 64u) {
                                    float T = 1.0f, sum[5] = { 0.0f, 0.0f, 0.0f, 0.0f, 0.0f };
                                    for (int w = 0; w < kWaves; ++w) {
                                        T *= s_sums[w][lane][0];
#pragma unroll
                                        for (int k = 0; k < 5; ++k) sum[k] += s_sums[w][lane][1 + k];
                                    }
                                    s_tails[mine][0] = T;
#pragma unroll
                                    for (int k = 0; k < 5; ++k) s_tails[mine][1 + k] = sum[k];
                                }
                            }
                            __syncthreads();
                        });
                    if (lane == 0) s_short[wave] = listed;
                    __syncthreads();
                    bool settled = true;
                    for (int w = 0; w < kWaves; ++w) settled = settled && s_short[w] != ~0u;
                    __syncthreads();                            // (s_short is written again below)
                    if (settled) {
                        if (wave == 0) {
                            // The walk's insertion, on the fragments that decide the cores alone, in list order; every pixel's lane
                            // takes its own.
                            hybrid_core_init<K>(cd, ca, ci);
                            tail.T = s_tails[lane][0]; tail.c0 = s_tails[lane][1]; tail.c1 = s_tails[lane][2]; tail.c2 = s_tails[lane][3];
                            tail.alpha = s_tails[lane][4]; tail.depth = s_tails[lane][5];
                            for (uint32_t w = 0; w < (uint32_t)kWaves; ++w) {
                                const uint32_t *entry = shortlist + first + 64u * (uint32_t)((uint64_t)n_batches * w / kWaves);
                                for (uint32_t left = s_short[w]; left != 0; --left, entry += 4) {
                                    float depth = bits_to_float(entry[1]), alpha = bits_to_float(entry[2]), index = bits_to_float(entry[3]);
                                    if (lane == entry[0]) {
                                        if (depth < cd[K - 1]) core_exchange_walk<K>(depth, alpha, index, cd, ca, ci);
                                        hybrid_tail_add<false>(tail, depth, alpha);
                                    }
                                }
                            }
                            if (px.inside && redo) finish(prim, tile, px, cd, ca, ci, tail);
                        }
                        if (threadIdx.x == 0) atomicAdd(const_cast<uint32_t *>(long_tiles) + 6, 1u);
                        continue;
                    }
                }
                if (threadIdx.x == 0) atomicAdd(const_cast<uint32_t *>(long_tiles) + 7, others_done ? 0x10001u : 1u);
                if (shortlist != nullptr) {
                    uint32_t kept = 0;
                    for (uint32_t base = seg_first; base < seg_last; base += 64) {
                        const uint32_t fetch = base + lane;
                        const bool reaches = tile_stage_load<HTGS_MODE_HYBRID_BLEND, 64, true, kCullPixels, true, REC4>(reinterpret_cast<TileStage<64> &>(st[wave]), prim, inst, fetch, seg_last, lane,
                                                                                                               px.cx, px.cy, redo_lanes) != 0;
                        const uint64_t keep = __ballot(reaches);
                        if (reaches) shortlist[seg_first + kept + (uint32_t)__popcll(keep & ((1ull << lane) - 1ull))] = inst[fetch];
                        kept += (uint32_t)__popcll(keep);
                    }
                    if (lane == 0) s_short[wave] = kept;
                    __syncthreads();
                }
                if (wave == 0) {
                    if (!others_done && px.inside && !redo)
                        finish(prim, tile, px, cd, ca, ci, tail);
                    hybrid_tail_init(tail);
                    hybrid_core_init<K>(cd, ca, ci);
                    if (shortlist != nullptr) {
                        for (uint32_t s = 0; s < (uint32_t)kWaves; ++s) {
                            const uint32_t from = first + 64u * (uint32_t)((uint64_t)n_batches * s / kWaves);
                            hybrid_walk<K, FAST, false, false, true, REC4>(st[0], ql[0], shortlist, prim, from, from + s_short[s], lane, px.pt, px.cx, px.cy, cd, ca, ci,
                                                                     tail, nullptr, redo_lanes);
                        }
                    } else {
                        hybrid_walk<K, FAST, false, false, true, REC4>(st[0], ql[0], inst, prim, first, last, lane, px.pt, px.cx, px.cy, cd, ca, ci, tail, nullptr, redo_lanes);
                    }
                    if (px.inside && redo) finish(prim, tile, px, cd, ca, ci, tail);
                }
                continue;
            }
        }
        if (wave == 0 && px.inside) finish(prim, tile, px, cd, ca, ci, tail);
    }
}

// ---------------------------------------------------------------------------------------------
// ALPHA_BLEND_FIRST_K: the K nearest fragments with alpha >= 1/20, alpha-blended; no tail.
// ---------------------------------------------------------------------------------------------
template <int K>
__device__ __forceinline__ void first_k_core_init(float (&cd)[K], float (&ca)[K], uint32_t (&ci)[K])
{
#pragma unroll
    for (int i = 0; i < K; ++i) {
        ca[i] = 0.0f; cd[i] = __FLT_MAX__; ci[i] = 0xffffffffu;
        asm volatile("" : "+v"(cd[i]), "+v"(ca[i]), "+v"(ci[i]));      // one register per slot
    }
}
// The walk over instances [first, last) of a tile's list by one wave (SOLO: the wave is the whole workgroup).  TIES (the
// walks of blend_first_k_long_kernel): `tie` receives the least depth at which an entry was pushed out of the core that is
// exactly as deep as the entry that is now last.
// PIXELS: only the pixels of the lanes in pixel_lanes are wanted; instances that do not reach one of them are left out.
template <int K, bool FAST, bool SOLO, bool TIES = false, int REC4 = HTGS_PRIM_FLOATS / 4, bool PIXELS = false>
__device__ __forceinline__ void first_k_walk(TileStageQ &st, QuadrantLists &ql, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
                                             uint32_t first, uint32_t last, uint32_t lane, const PixelTerms &pt, float cx, float cy, float (&cd)[K],
                                             float (&ca)[K], uint32_t (&ci)[K], float *tie = nullptr, uint64_t pixel_lanes = 0)
{
    constexpr int MODE = HTGS_MODE_ALPHA_BLEND_FIRST_K;
    constexpr int N = kStageSlots;
    tile_list_walk<MODE, true, PIXELS ? kCullPixels : kCullAlpha, SOLO, REC4>(st, ql, prim, inst, first, last, lane, cx, cy, [&](uint32_t addr) {
        TileFrag f;
        const bool in_reach = tile_frag_cutoff<N>(addr, pt, f);
        f.den_rcp = frag_rcp<FAST>(f.den);
        float depth = tile_frag_depth<N>(addr, pt, f);
        if (!(in_reach && depth < cd[K - 1])) return;          // depth test before the exponential (:151)
        if (!tile_frag_alpha<MODE, FAST>(stage_opacity<N>(addr), f)) return;
        float alpha = f.alpha;
        uint32_t idx = stage_index<N>(addr);
        core_exchange_walk<K>(depth, alpha, idx, cd, ca, ci);
        if (TIES && alpha > 0.0f && depth == cd[K - 1]) *tie = depth < *tie ? depth : *tie;
    }, pixel_lanes);
}
// The same walk with the core as sorted 64-bit keys (above HYBRID_BLEND's: depth | alpha as a fraction | place in the list),
// exact arithmetic; `tie` as in hybrid_key_walk.
template <int K, bool SOLO, int REC4 = HTGS_PRIM_FLOATS / 4>
__device__ __forceinline__ void first_k_key_walk(TileStageQ &st, QuadrantLists &ql, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
                                                 uint32_t first, uint32_t last, uint32_t lane, const PixelTerms &pt, float cx, float cy,
                                                 CoreKey (&core)[K], float &tie, const KeyFormat &fmt)
{
    constexpr int MODE = HTGS_MODE_ALPHA_BLEND_FIRST_K;
    constexpr int N = kStageSlots;
    tile_list_walk<MODE, true, kCullAlpha, SOLO, REC4, false, true, true>(st, ql, prim, inst, first, last, lane, cx, cy, [&](uint32_t addr) {
        TileFrag f;
        const bool in_reach = tile_frag_cutoff<N>(addr, pt, f);
        f.den_rcp = frag_rcp<false>(f.den);
        float depth = tile_frag_depth<N>(addr, pt, f);
        if (!(in_reach && depth < key_depth(core[K - 1]))) return;          // depth test before the exponential (:151)
        if (!tile_frag_alpha<MODE, false>(stage_opacity<N>(addr), f)) return;
        CoreKey carried = make_key(depth, key_pack(f.alpha, stage_index<N>(addr) - first, fmt));      // (the slot's last word is the place in the list)
        core_key_walk<K>(carried, core);
        depth = key_depth(carried);
        tie = key_low(carried) >> fmt.shift != 0u && depth == key_depth(core[K - 1]) && depth < tie ? depth : tie;
    });
}
// the finished keys as the three arrays the composite takes (an empty slot has the index 0xffffffff)
template <int K>
__device__ __forceinline__ void first_k_core_unpack(const CoreKey (&core)[K], const uint32_t *__restrict__ inst, uint32_t first, uint32_t last, float (&cd)[K],
                                                    float (&ca)[K], uint32_t (&ci)[K], const KeyFormat &fmt)
{
#pragma unroll
    for (int i = 0; i < K; ++i) {
        const uint32_t low = key_low(core[i]), place = low & fmt.place_mask;
        cd[i] = key_depth(core[i]);
        ca[i] = key_alpha(low, fmt);
        ci[i] = low >> fmt.shift != 0u && first + place < last ? inst[first + place] : 0xffffffffu;
    }
}
template <int K, int REC4 = HTGS_PRIM_FLOATS / 4>
__device__ __forceinline__ void first_k_composite(const float4 *__restrict__ prim, const float (&cd)[K], const float (&ca)[K], const uint32_t (&ci)[K],
                                                  float *__restrict__ image, float *__restrict__ depths, uint32_t width, uint32_t height, uint32_t x,
                                                  uint32_t y, int chw, int median)
{
    float r = 0.0f, g = 0.0f, b = 0.0f, depth_pixel = 0.0f, T = 1.0f;
    bool open = true;
#pragma unroll
    for (int i = 0; i < K; ++i) {
        open = open && T >= kTransmittanceThreshold && ci[i] != 0xffffffffu;
        if (open) {
            const float wgt = T * ca[i];
            const float4 col = prim[(size_t)ci[i] * REC4 + 4];
            r = __builtin_fmaf(wgt, col.x, r);
            g = __builtin_fmaf(wgt, col.y, g);
            b = __builtin_fmaf(wgt, col.z, b);
            if (median) depth_pixel = T > 0.5f ? cd[i] : depth_pixel;
            else depth_pixel = __builtin_fmaf(wgt, cd[i], depth_pixel);
            T *= 1.0f - ca[i];
        }
    }
    if (!median) depth_pixel = T < 1.0f ? depth_pixel / (1.0f - T) : 0.0f;
    store_pixel(image, depths, width, height, x, y, chw, r, g, b, depth_pixel);
}
struct FirstKImage {
    float *image, *depths;
    uint32_t width, height;
    int chw, median;
    template <int K>
    __device__ __forceinline__ void operator()(const float4 *__restrict__ prim, uint32_t, const TilePixel &px, const float (&cd)[K], const float (&ca)[K],
                                               const uint32_t (&ci)[K]) const
    {
        first_k_composite<K>(prim, cd, ca, ci, image, depths, width, height, px.x, px.y, chw, median);
    }
};
// what a workgroup leaves of its part of a list: the core and the depth of a tie
template <int K> constexpr uint32_t first_k_part_words() { return (3u * K + 1u) * 64u; }
// KEYS (exact arithmetic, with long_tiles and a threshold of no more than kPackedListMost): the core as sorted 64-bit keys;
// the pixels at which fragments of exactly equal depth met where they decide the core are walked again afterwards, over the
// instances that reach one of them, with the reference's insertion (as in hybrid_tile_by_keys).
template <int K, bool FAST, bool KEYS = false>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(K <= 16 ? 5 : 2))) blend_first_k_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
    float *__restrict__ image, float *__restrict__ depths, uint32_t width, uint32_t height, uint32_t grid_w, int chw, int median,
    uint32_t *__restrict__ long_tiles, uint32_t long_threshold, uint32_t part_floor, const uint32_t *__restrict__ tile_order)
{
    static_assert(!(KEYS && FAST), "the keys of this mode are for the exact path");
    __shared__ TileStageQ st;
    __shared__ QuadrantLists ql;
    const uint32_t tile = block_tile(tile_order);
    const uint32_t lane = threadIdx.x;
    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    if (long_tiles != nullptr && last - first > long_threshold) {
        if (lane == 0) long_tile_enter(long_tiles, tile, gridDim.x, last - first, long_threshold, first_k_part_words<K>(), part_floor);
        return;
    }
    const TilePixel px = quadrant_tile_pixel(tile, grid_w, lane, width, height);
    float ca[K], cd[K];
    uint32_t ci[K];
    if constexpr (KEYS) {
        CoreKey core[K];
#pragma unroll
        for (int i = 0; i < K; ++i) {
            core[i] = make_key(__FLT_MAX__, 0u);
            asm volatile("" : "+v"(core[i]));      // one register pair per slot, never a wide tuple
        }
        float tie = __FLT_MAX__;
        const KeyFormat fmt = key_format(last > first ? last - first : 1u);
        first_k_key_walk<K, true>(st, ql, inst, prim, first, last, lane, px.pt, px.cx, px.cy, core, tie, fmt);
        const bool again = px.inside && ((tie < __FLT_MAX__ && tie <= key_depth(core[K - 1])) || key_core_tied<K>(core, fmt));
        const uint64_t again_lanes = __ballot(again);
        first_k_core_unpack<K>(core, inst, first, last, cd, ca, ci, fmt);
        if (px.inside && !again) first_k_composite<K>(prim, cd, ca, ci, image, depths, width, height, px.x, px.y, chw, median);
        if (again_lanes == 0) return;
        // (the lane and its pixel are worked out afresh: nothing of the first walk has to live through the composite for this)
        uint32_t lane_again = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
        asm volatile("" : "+v"(lane_again));
        const TilePixel px_again = quadrant_tile_pixel(tile, grid_w, lane_again, width, height);
        first_k_core_init<K>(cd, ca, ci);
        first_k_walk<K, false, true, false, HTGS_PRIM_FLOATS / 4, true>(st, ql, inst, prim, first, last, lane_again, px_again.pt, px_again.cx, px_again.cy, cd, ca, ci,
                                                                         nullptr, again_lanes);
        if ((again_lanes >> lane_again & 1ull) != 0)
            first_k_composite<K>(prim, cd, ca, ci, image, depths, width, height, px_again.x, px_again.y, chw, median);
    } else {
        first_k_core_init<K>(cd, ca, ci);
        first_k_walk<K, FAST, true>(st, ql, inst, prim, first, last, lane, px.pt, px.cx, px.cy, cd, ca, ci);
        if (!px.inside) return;
        first_k_composite<K>(prim, cd, ca, ci, image, depths, width, height, px.x, px.y, chw, median);
    }
}

// A core and a tie depth (3K + 1 rows of 64 lanes at from[]) join the running ones: they cover the stretch of the list
// that follows.
template <int K, bool FAST>
__device__ __forceinline__ void first_k_merge(const float *from, uint32_t lane, float (&cd)[K], float (&ca)[K], uint32_t (&ci)[K], float &tie)
{
    constexpr bool kTies = true;
    from += lane;
#pragma unroll
    for (int i = 0; i < K; ++i) {
        float depth = from[(3 * i) * 64], alpha = from[(3 * i + 1) * 64];
        uint32_t index = float_to_bits(from[(3 * i + 2) * 64]);
        if (alpha > 0.0f) {                    // a filled slot
            if (kTies && depth == cd[K - 1]) tie = depth < tie ? depth : tie;
            if (depth < cd[K - 1]) {
                core_exchange_walk<K>(depth, alpha, index, cd, ca, ci);
                if (kTies && alpha > 0.0f && depth == cd[K - 1]) tie = depth < tie ? depth : tie;
            }
        }
    }
    const float other = from[(3 * K) * 64];
    tie = other < tie ? other : tie;
}
template <int K>
__device__ __forceinline__ void first_k_put(float *to, uint32_t lane, const float (&cd)[K], const float (&ca)[K], const uint32_t (&ci)[K], float tie)
{
    to += lane;
#pragma unroll
    for (int i = 0; i < K; ++i) { to[(3 * i) * 64] = cd[i]; to[(3 * i + 1) * 64] = ca[i]; to[(3 * i + 2) * 64] = bits_to_float(ci[i]); }
    to[(3 * K) * 64] = tie;
}

// The tiles with very long lists, as in blend_hybrid_long_kernel: every wave of the workgroup walks a share of the list
// into a core of its own, the cores are merged in list order (and so are those of the parts of a list that several
// workgroups walked, through the tile's stretch of the spare value buffer `spare`), and the pixels at which fragments of
// exactly equal depth met where they can change the final core get a second look (pixels_again) with the insertion
// replayed on the fragments that are not farther than the merged core's last entry -- or, when they are many or the room
// for those fragments does not do, the first wave walks the whole list again for them.
// finish(prim, tile, px, cd, ca, ci): as for blend_hybrid_long_kernel, with the pixel's finished core.
template <int K, bool FAST, int REC4, typename Finish>
__global__ void __launch_bounds__(64 * long_waves<K>()) blend_first_k_long_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, const uint32_t *long_tiles,
    uint32_t width, uint32_t height, uint32_t grid_w, uint32_t *__restrict__ spare, uint32_t long_threshold, const Finish finish)
{
    constexpr int kWaves = long_waves<K>();
    __shared__ TileStageQ st[kWaves];
    __shared__ QuadrantLists ql[kWaves];
    __shared__ float s_merge[3 * K + 1][64];
    __shared__ uint32_t s_next, s_whole, s_redo[2], s_listed[kWaves];
    __shared__ float s_last_depth[64];
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
    if (long_tiles[0] == 0) return;                   // (the ordinary frame)
    const uint32_t n_tiles = grid_w * ((height + 7u) / 8u);
    constexpr bool kTies = true;                      // (the fast variant too: a tie decides which fragment a pixel shows)
    uint32_t round = 0;
    LongEntry entry;
    while (long_tile_take(long_tiles, ranges, long_threshold, round, &s_next, entry)) {
        // (the same in every lane; said so, they live in scalar registers through the walks that follow)
        const auto uniform = [](uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
        const LongEntry e = { uniform(entry.tile), uniform(entry.part), uniform(entry.parts), uniform(entry.tile_first), uniform(entry.tile_last),
                              uniform(entry.first), uniform(entry.last) };
        const TilePixel px = quadrant_tile_pixel(e.tile, grid_w, lane, width, height);
        uint32_t share_first, share_last;
        long_wave_share(e.first, e.last, wave, share_first, share_last, kWaves);
        float ca[K], cd[K];
        uint32_t ci[K];
        first_k_core_init<K>(cd, ca, ci);
        float tie = __FLT_MAX__;
        first_k_walk<K, FAST, false, kTies, REC4>(st[wave], ql[wave], inst, prim, share_first, share_last, lane, px.pt, px.cx, px.cy, cd, ca, ci, &tie);
        for (uint32_t s = 1; s < (uint32_t)kWaves; ++s) {
            __syncthreads();                               // the buffer is free
            if (wave == s) first_k_put<K>(&s_merge[0][0], lane, cd, ca, ci, tie);
            __syncthreads();
            if (wave == 0) first_k_merge<K, FAST>(&s_merge[0][0], lane, cd, ca, ci, tie);
        }
        if (e.parts > 1u) {
            float *const left = reinterpret_cast<float *>(spare + e.tile_first);
            if (wave == 0) {
                first_k_put<K>(left + (size_t)e.part * first_k_part_words<K>(), lane, cd, ca, ci, tie);
                __threadfence();
            }
            if (!long_part_done(long_tiles, n_tiles, e, &s_whole)) continue;
            if (wave == 0) {
                __threadfence();
                first_k_core_init<K>(cd, ca, ci);
                tie = __FLT_MAX__;
                for (uint32_t other = 0; other < e.parts; ++other)
                    first_k_merge<K, FAST>(left + (size_t)other * first_k_part_words<K>(), lane, cd, ca, ci, tie);
            }
            long_wave_share(e.tile_first, e.tile_last, wave, share_first, share_last, kWaves);
            __syncthreads();                               // (the parts are read before the second look overwrites them)
        }
        if (kTies) {
            bool redo = false;
            if (wave == 0) {
                redo = tie <= cd[K - 1];
#pragma unroll
                for (int i = 0; i + 1 < K; ++i) redo = redo || (ca[i + 1] > 0.0f && cd[i] == cd[i + 1]);
                const uint64_t lanes = __ballot(redo);
                if (lane == 0) { s_redo[0] = (uint32_t)lanes; s_redo[1] = (uint32_t)(lanes >> 32); }
                s_last_depth[lane] = cd[K - 1];
                if (lanes != 0 && px.inside && !redo) finish(prim, e.tile, px, cd, ca, ci);
            }
            __syncthreads();
            const uint64_t redo_lanes = (uint64_t)s_redo[0] | (uint64_t)s_redo[1] << 32;
            if (redo_lanes != 0) {
                bool settled = false, looked = false;
                if (spare != nullptr && __popcll(redo_lanes) <= kAgainMost) {
                    looked = true;
                    const uint32_t listed = pixels_again<HTGS_MODE_ALPHA_BLEND_FIRST_K, FAST, REC4>(
                        reinterpret_cast<TileStage<64> &>(st[wave]), inst, prim, share_first, share_last, lane, px.cx, px.cy, redo_lanes, s_last_depth, nullptr, spare + share_first,
                        (share_last - share_first) / 4u, [](const uint32_t (&)[kAgainPixels]) {});
                    if (lane == 0) s_listed[wave] = listed;
                    __syncthreads();
                    settled = true;
                    for (int w = 0; w < kWaves; ++w) settled = settled && s_listed[w] != ~0u;
                }
                if (threadIdx.x == 0) atomicAdd(const_cast<uint32_t *>(long_tiles) + (settled ? 6 : 7), settled || !looked ? 1u : 0x10001u);
                if (wave == 0) {
                    first_k_core_init<K>(cd, ca, ci);
                    if (settled) {
                        for (uint32_t w = 0; w < (uint32_t)kWaves; ++w) {
                            uint32_t from, to;
                            long_wave_share(e.tile_first, e.tile_last, w, from, to, kWaves);
                            const uint32_t *candidate = spare + from;
                            for (uint32_t todo = s_listed[w]; todo != 0; --todo, candidate += 4) {
                                float depth = bits_to_float(candidate[1]), alpha = bits_to_float(candidate[2]);
                                uint32_t index = candidate[3];
                                if (lane == candidate[0] && depth < cd[K - 1]) core_exchange_walk<K>(depth, alpha, index, cd, ca, ci);
                            }
                        }
                    } else {
                        first_k_walk<K, FAST, false, false, REC4>(st[0], ql[0], inst, prim, e.tile_first, e.tile_last, lane, px.pt, px.cx, px.cy, cd, ca, ci);
                    }
                    if (px.inside && redo) finish(prim, e.tile, px, cd, ca, ci);
                }
                continue;
            }
        }
        if (wave == 0 && px.inside) finish(prim, e.tile, px, cd, ca, ci);
    }
}

// ---------------------------------------------------------------------------------------------
// OIT_BLEND: weighted-sum order-independent transparency over all fragments.
// ---------------------------------------------------------------------------------------------
// what a pixel has summed up: alpha * (colour, depth), alpha, and the transmittance
struct OitSums {
    float a0, a1, a2, a3, alpha, T;
};
// The walk over instances [first, last) of a tile's list by one wave (SOLO: the wave is the whole workgroup).
// DEPTH: the depth sum is wanted (the training pass has no use for it)
template <bool FAST, bool SOLO, int REC4 = HTGS_PRIM_FLOATS / 4, bool DEPTH = !FAST>
__device__ __forceinline__ void oit_walk(TileStageQ &st, QuadrantLists &ql, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, uint32_t first,
                                         uint32_t last, uint32_t lane, const PixelTerms &pt, float cx, float cy, OitSums &sum)
{
    constexpr int MODE = HTGS_MODE_OIT_BLEND;
    constexpr int N = kStageSlots;
    tile_list_walk<MODE, DEPTH, kCullAlpha, SOLO, REC4, FAST>(st, ql, prim, inst, first, last, lane, cx, cy, [&](uint32_t addr) {
        TileFrag f;
        bool fragment;
        if constexpr (FAST) fragment = tile_frag_fast<MODE, N>(addr, pt, f);
        else {
            const bool in_reach = tile_frag_cutoff<N>(addr, pt, f);
            f.den_rcp = frag_rcp<FAST>(f.den);
            fragment = tile_frag_alpha<MODE, FAST>(stage_opacity<N>(addr), f) && in_reach;
        }
        const float4 col = stage_row<N, 5>(addr);
        if (!fragment) return;
        const float depth = DEPTH ? tile_frag_depth<N>(addr, pt, f) : 0.0f;
        sum.a0 = __builtin_fmaf(f.alpha, col.x, sum.a0);
        sum.a1 = __builtin_fmaf(f.alpha, col.y, sum.a1);
        sum.a2 = __builtin_fmaf(f.alpha, col.z, sum.a2);
        if (DEPTH) sum.a3 = __builtin_fmaf(f.alpha, depth, sum.a3);
        sum.alpha += f.alpha;
        sum.T *= 1.0f - f.alpha;
    });
}
__device__ __forceinline__ void oit_composite(const OitSums &sum, float *__restrict__ image, float *__restrict__ depths, uint32_t width, uint32_t height,
                                              uint32_t x, uint32_t y, int chw)
{
    float r = 0.0f, g = 0.0f, b = 0.0f, d = 0.0f;
    if (sum.alpha >= ModeCfg<HTGS_MODE_OIT_BLEND>::min_alpha) {
        const float alpha = 1.0f - sum.T;
        const float s = alpha * (1.0f / sum.alpha);
        r = s * sum.a0; g = s * sum.a1; b = s * sum.a2;
        d = (s * sum.a3) / alpha;
    }
    store_pixel(image, depths, width, height, x, y, chw, r, g, b, d);
}
struct OitImage {
    float *image, *depths;
    uint32_t width, height;
    int chw;
    __device__ __forceinline__ void operator()(uint32_t, const TilePixel &px, const OitSums &sum) const
    {
        oit_composite(sum, image, depths, width, height, px.x, px.y, chw);
    }
};
constexpr uint32_t kOitPartWords = 6u * 64u;
template <bool FAST>
__global__ void __launch_bounds__(64) blend_oit_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
    float *__restrict__ image, float *__restrict__ depths, uint32_t width, uint32_t height, uint32_t grid_w, int chw,
    uint32_t *__restrict__ long_tiles, uint32_t long_threshold, uint32_t part_floor, const uint32_t *__restrict__ tile_order)
{
    __shared__ TileStageQ st;
    __shared__ QuadrantLists ql;
    const uint32_t tile = block_tile(tile_order);
    const uint32_t lane = threadIdx.x;
    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    if (long_tiles != nullptr && last - first > long_threshold) {
        if (lane == 0) long_tile_enter(long_tiles, tile, gridDim.x, last - first, long_threshold, kOitPartWords, part_floor);
        return;
    }
    const TilePixel px = quadrant_tile_pixel(tile, grid_w, lane, width, height);
    OitSums sum = { 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 1.0f };
    oit_walk<FAST, true>(st, ql, inst, prim, first, last, lane, px.pt, px.cx, px.cy, sum);
    if (!px.inside) return;
    oit_composite(sum, image, depths, width, height, px.x, px.y, chw);
}

// The tiles with very long lists: every wave of the workgroup walks a share of the list, the sums add up in the order of
// the shares (the transmittances multiply), and so do those of the parts of a list that several workgroups walked
// (`left`: the spare value buffer, where the parts of a tile leave their sums in the tile's own stretch).  The pixel's
// result is that of the single walk up to the order of its sums.
// finish(tile, px, sum): as for blend_hybrid_long_kernel, with the pixel's finished sums.
template <bool FAST, int REC4, typename Finish, bool DEPTH = !FAST>
__global__ void __launch_bounds__(64 * kLongWaves) blend_oit_long_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, const uint32_t *long_tiles,
    uint32_t width, uint32_t height, uint32_t grid_w, uint32_t *__restrict__ left, uint32_t long_threshold, const Finish finish)
{
    __shared__ TileStageQ st[kLongWaves];
    __shared__ QuadrantLists ql[kLongWaves];
    __shared__ float s_sums[kLongWaves][6][64];
    __shared__ uint32_t s_next, s_whole;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
    if (long_tiles[0] == 0) return;                   // (the ordinary frame)
    const uint32_t n_tiles = grid_w * ((height + 7u) / 8u);
    uint32_t round = 0;
    LongEntry entry;
    while (long_tile_take(long_tiles, ranges, long_threshold, round, &s_next, entry)) {
        const TilePixel px = quadrant_tile_pixel(entry.tile, grid_w, lane, width, height);
        uint32_t share_first, share_last;
        long_wave_share(entry.first, entry.last, wave, share_first, share_last);
        OitSums sum = { 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 1.0f };
        oit_walk<FAST, false, REC4, DEPTH>(st[wave], ql[wave], inst, prim, share_first, share_last, lane, px.pt, px.cx, px.cy, sum);
        s_sums[wave][0][lane] = sum.a0; s_sums[wave][1][lane] = sum.a1; s_sums[wave][2][lane] = sum.a2; s_sums[wave][3][lane] = sum.a3;
        s_sums[wave][4][lane] = sum.alpha; s_sums[wave][5][lane] = sum.T;
        __syncthreads();
        if (wave == 0) {
            for (int w = 1; w < kLongWaves; ++w) {
                sum.a0 += s_sums[w][0][lane]; sum.a1 += s_sums[w][1][lane]; sum.a2 += s_sums[w][2][lane]; sum.a3 += s_sums[w][3][lane];
                sum.alpha += s_sums[w][4][lane]; sum.T *= s_sums[w][5][lane];
            }
        }
        if (entry.parts > 1u) {
            float *const parts = reinterpret_cast<float *>(left + entry.tile_first);
            if (wave == 0) {
                float *mine = parts + (size_t)entry.part * kOitPartWords + lane;
                mine[0] = sum.a0; mine[64] = sum.a1; mine[128] = sum.a2; mine[192] = sum.a3; mine[256] = sum.alpha; mine[320] = sum.T;
                __threadfence();
            }
            if (!long_part_done(long_tiles, n_tiles, entry, &s_whole)) continue;
            if (wave == 0) {
                __threadfence();
                sum = { 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 1.0f };
                for (uint32_t part = 0; part < entry.parts; ++part) {
                    const float *its = parts + (size_t)part * kOitPartWords + lane;
                    sum.a0 += its[0]; sum.a1 += its[64]; sum.a2 += its[128]; sum.a3 += its[192]; sum.alpha += its[256]; sum.T *= its[320];
                }
            }
        }
        if (wave == 0 && px.inside) finish(entry.tile, px, sum);
    }
}

}  // namespace htgs
