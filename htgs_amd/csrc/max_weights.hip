// Per-Gaussian maximum blending weight of a view (used by the reference's importance-based pruning).
// Restates update_max_weights_cu of R/include/hybrid_blend/kernels/update_max_weights.cuh:59-212,
// R/include/alpha_blend_first_k/kernels/update_max_weights.cuh:59-161,
// R/include/alpha_blend_global_ordering/kernels/update_max_weights.cuh:59-131 and
// R/include/oit_blend/kernels/update_max_weights.cuh:58-165.  The maximum is taken on the bit patterns of the
// (non-negative) weights with integer atomicMax, which makes the result independent of the order of arrival.
#include "blend_long.h"

namespace htgs {

__device__ __forceinline__ void raise_max(uint32_t *__restrict__ max_weights, uint32_t g, float w)
{
    if (g == 0xffffffffu) return;
    const uint32_t bits = float_to_bits(w);
    if (max_weights[g] < bits) atomicMax(max_weights + g, bits);
}

// HYBRID_BLEND (TAIL = true, CORE = true), ALPHA_BLEND_FIRST_K (CORE only), OIT_BLEND (TAIL only, K unused)
template <int K, int MODE>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(K <= 16 ? 5 : 2))) max_weights_tile_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
    uint32_t *__restrict__ max_weights, uint32_t width, uint32_t height, uint32_t grid_w, float weight_threshold, const uint32_t *__restrict__ tile_order,
    uint32_t *__restrict__ long_tiles, uint32_t long_threshold, uint32_t part_floor)
{
    constexpr bool kCore = MODE != HTGS_MODE_OIT_BLEND;
    constexpr bool kTail = MODE != HTGS_MODE_ALPHA_BLEND_FIRST_K;
    constexpr int KS = kCore ? K : 1;
    __shared__ TileStageQ st;
    __shared__ QuadrantLists ql;
    const uint32_t tile = block_tile(tile_order);
    const uint32_t lane = threadIdx.x;
    {
        // a tile with a very long list is left to the kernels that share a list between waves and workgroups
        const uint32_t length = ranges[2 * tile + 1] - ranges[2 * tile];
        if (long_tiles != nullptr && length > long_threshold) {
            constexpr uint32_t part_words = MODE == HTGS_MODE_HYBRID_BLEND ? long_part_words<KS>() : MODE == HTGS_MODE_OIT_BLEND ? kOitPartWords : first_k_part_words<KS>();
            if (lane == 0) long_tile_enter(long_tiles, tile, gridDim.x, length, long_threshold, part_words, part_floor);
            return;
        }
    }
    const TilePixel px = quadrant_tile_pixel(tile, grid_w, lane, width, height);
    const bool inside = px.inside;
    const PixelTerms pt = px.pt;
    const float cx = px.cx, cy = px.cy;

    float alpha_sum = 0.0f, T_tail = 1.0f;
    float ca[KS], cd[KS];
    uint32_t ci[KS];
#pragma unroll
    for (int i = 0; i < KS; ++i) {
        ca[i] = 0.0f; cd[i] = __FLT_MAX__; ci[i] = 0xffffffffu;
        asm volatile("" : "+v"(cd[i]), "+v"(ca[i]), "+v"(ci[i]));      // one register per slot
    }

    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    tile_list_walk<MODE, kCore, kCullAlpha, true>(st, ql, prim, inst, first, last, lane, cx, cy, [&](uint32_t addr) {
        TileFrag f;
        bool in_reach = tile_frag_cutoff<kStageSlots>(addr, pt, f);
        f.den_rcp = rcp_exact(f.den);
        float depth = 0.0f;
        if (MODE == HTGS_MODE_ALPHA_BLEND_FIRST_K) {
            depth = tile_frag_depth<kStageSlots>(addr, pt, f);
            in_reach = in_reach && depth < cd[KS - 1];
        }
        if (!(tile_frag_alpha<MODE>(stage_opacity<kStageSlots>(addr), f) && in_reach)) return;
        float alpha = f.alpha;
        if (MODE == HTGS_MODE_HYBRID_BLEND) depth = tile_frag_depth<kStageSlots>(addr, pt, f);
        if (kCore && (MODE == HTGS_MODE_ALPHA_BLEND_FIRST_K || (depth < cd[KS - 1] && alpha >= kMinAlphaCore))) {
            uint32_t idx = stage_index<kStageSlots>(addr);
            core_exchange_walk<KS>(depth, alpha, idx, cd, ca, ci);
        }
        if (kTail) { alpha_sum += alpha; T_tail *= 1.0f - alpha; }
    });
    float T_core = 1.0f;
    if (kCore && inside) {
#pragma unroll
        for (int i = 0; i < KS; ++i) {
            const float w = T_core * ca[i];
            T_core *= 1.0f - ca[i];
            if (T_core < kTransmittanceThreshold) T_core = 0.0f;
            if (!(w < weight_threshold)) raise_max(max_weights, ci[i], w);
        }
    }
    if (!kTail) return;
    float tail_weight = 0.0f;
    if (inside && alpha_sum >= weight_threshold) tail_weight = (T_core * (1.0f - T_tail)) * (1.0f / alpha_sum);
    const bool active = inside && tail_weight >= weight_threshold;
    if (!__any(active)) return;
    // second walk over the tile's list: alpha * tail weight for every fragment that passes the cut-off (no alpha
    // threshold here, R/include/hybrid_blend/kernels/update_max_weights.cuh:197-204)
    tile_list_walk<MODE, false, kCullCutoff, true>(st, ql, prim, inst, first, last, lane, cx, cy, [&](uint32_t addr) {
        TileFrag f;
        if (!active || !tile_frag_cutoff<kStageSlots>(addr, pt, f)) return;
        const float G = d_exp2((f.num * ModeCfg<MODE>::exp2_scale) * rcp_exact(f.den));
        const float a = stage_opacity<kStageSlots>(addr) * G;
        const float w = (a < kMaxFragmentAlpha ? a : kMaxFragmentAlpha) * tail_weight;
        if (!(w < weight_threshold)) raise_max(max_weights, stage_index<kStageSlots>(addr), w);
    });
}

__global__ void __launch_bounds__(256) max_weights_global_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
    uint32_t *__restrict__ max_weights, uint32_t width, uint32_t height, uint32_t grid_w, float weight_threshold, const uint32_t *__restrict__ tile_order)
{
    constexpr int MODE = HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING;
    __shared__ TileStage<256> st;
    __shared__ uint16_t s_reach[256];                  // per staged slot: the quadrants of the tile it can reach
    const uint32_t tile = block_tile(tile_order);
    const uint32_t t = threadIdx.x, wave = t >> 6, lane = t & 63;
    const uint32_t x0 = (tile % grid_w) * 16, y0 = (tile / grid_w) * 16;
    uint32_t local_x, local_y;
    subtile_pixel(t, local_x, local_y);                // a wave = an 8x8 sub-tile, walked by quadrants
    const uint32_t x = x0 + local_x, y = y0 + local_y;
    const bool inside = x < width && y < height;
    const PixelTerms pt = pixel_terms(local_x, local_y, 16);
    const float cx = tile_centre(x0, 16), cy = tile_centre(y0, 16);
    float T = 1.0f;
    bool done = !inside;
    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    for (uint32_t base = first; base < last; base += 256) {
        if (__syncthreads_count(done) == 256) break;
        s_reach[t] = (uint16_t)tile_stage_load<MODE, 256, false, kCullAlpha, true>(st, prim, inst, base + t, last, t, cx, cy);
        __syncthreads();
        const uint32_t stage_base = __builtin_amdgcn_readfirstlane(stage_address(st));
        subtile_walk(s_reach, stage_base, last - base < 256u ? last - base : 256u, wave, lane,
                     [&]() { return __ballot(!done) == 0; },
                     [&](uint32_t addr) {
            TileFrag f;
            if (done || !tile_frag_cutoff<256>(addr, pt, f)) return;
            f.den_rcp = rcp_exact(f.den);
            if (!tile_frag_alpha<MODE>(stage_opacity<256>(addr), f)) return;
            const float w = T * f.alpha;
            T *= 1.0f - f.alpha;
            if (T < kTransmittanceThreshold) done = true;
            if (!(w < weight_threshold)) raise_max(max_weights, stage_index<256>(addr), w);
        });
    }
}

// What the pass does with a pixel's finished core and tail when the tile's list was walked by the kernels for very long
// lists: the weights of the core's entries, and the weight of a tail fragment per unit of alpha into tail_weights[64 tile +
// lane] (0: no tail fragment of this pixel can reach the threshold) for the second walk (max_weights_tail_long_kernel).
struct MaxWeightsHybrid {
    uint32_t *max_weights;
    float *tail_weights;
    float weight_threshold;
    template <int K>
    __device__ __forceinline__ void operator()(const float4 *__restrict__, uint32_t tile, const TilePixel &, float (&)[K], float (&ca)[K], float (&ci)[K],
                                               HybridTail &tail) const
    {
        float T_core = 1.0f;
#pragma unroll
        for (int i = 0; i < K; ++i) {
            const float w = T_core * ca[i];
            T_core *= 1.0f - ca[i];
            if (T_core < kTransmittanceThreshold) T_core = 0.0f;
            if (ca[i] > 0.0f && !(w < weight_threshold)) raise_max(max_weights, float_to_bits(ci[i]), w);
        }
        float tail_weight = 0.0f;
        if (tail.alpha >= weight_threshold) tail_weight = (T_core * (1.0f - tail.T)) * (1.0f / tail.alpha);
        tail_weights[64u * (size_t)tile + (threadIdx.x & 63u)] = tail_weight >= weight_threshold ? tail_weight : 0.0f;
    }
};
struct MaxWeightsFirstK {
    uint32_t *max_weights;
    float weight_threshold;
    template <int K>
    __device__ __forceinline__ void operator()(const float4 *__restrict__, uint32_t, const TilePixel &, const float (&)[K], const float (&ca)[K],
                                               const uint32_t (&ci)[K]) const
    {
        float T_core = 1.0f;
#pragma unroll
        for (int i = 0; i < K; ++i) {
            const float w = T_core * ca[i];
            T_core *= 1.0f - ca[i];
            if (T_core < kTransmittanceThreshold) T_core = 0.0f;
            if (!(w < weight_threshold)) raise_max(max_weights, ci[i], w);
        }
    }
};
struct MaxWeightsOit {
    float *tail_weights;
    float weight_threshold;
    __device__ __forceinline__ void operator()(uint32_t tile, const TilePixel &, const OitSums &sum) const
    {
        float tail_weight = 0.0f;
        if (sum.alpha >= weight_threshold) tail_weight = (1.0f * (1.0f - sum.T)) * (1.0f / sum.alpha);
        tail_weights[64u * (size_t)tile + (threadIdx.x & 63u)] = tail_weight >= weight_threshold ? tail_weight : 0.0f;
    }
};

// After the kernels for very long lists have left the tail weights of such tiles: the tiles are entered on the list again,
// in parts, for the second walk.
__global__ void __launch_bounds__(256) max_weights_tail_enter_kernel(const uint32_t *__restrict__ ranges, uint32_t *__restrict__ long_tiles, uint32_t n_tiles,
                                                                    uint32_t long_threshold, uint32_t part_floor)
{
    const uint32_t tile = blockIdx.x * 256 + threadIdx.x;
    if (tile >= n_tiles) return;
    const uint32_t length = ranges[2 * tile + 1] - ranges[2 * tile];
    if (length > long_threshold) long_tile_enter(long_tiles, tile, n_tiles, length, long_threshold / 4u, 0u, part_floor);   // (parts of one threshold's length)
}
// The second walk (alpha * tail weight for every fragment that passes the cut-off) over the parts of the very long lists:
// a workgroup of four waves per part, every wave a share of it; the maximum is order independent, nothing to merge.
constexpr int kTailWaves = 4;
template <int MODE>
__global__ void __launch_bounds__(64 * kTailWaves) max_weights_tail_long_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, const uint32_t *long_tiles,
    uint32_t *__restrict__ max_weights, const float *__restrict__ tail_weights, uint32_t width, uint32_t height, uint32_t grid_w, float weight_threshold,
    uint32_t long_threshold)
{
    __shared__ TileStageQ st[kTailWaves];
    __shared__ QuadrantLists ql[kTailWaves];
    __shared__ uint32_t s_next;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
    if (long_tiles[0] == 0) return;                   // (the ordinary frame)
    uint32_t round = 0;
    LongEntry e;
    while (long_tile_take(long_tiles, ranges, long_threshold, round, &s_next, e)) {
        const TilePixel px = quadrant_tile_pixel(e.tile, grid_w, lane, width, height);
        const PixelTerms pt = px.pt;
        const float tail_weight = px.inside ? tail_weights[64u * (size_t)e.tile + lane] : 0.0f;
        const bool active = tail_weight > 0.0f;
        if (__syncthreads_or(active) == 0) continue;
        uint32_t share_first, share_last;
        long_wave_share(e.first, e.last, wave, share_first, share_last, kTailWaves);
        tile_list_walk<MODE, false, kCullCutoff, false>(st[wave], ql[wave], prim, inst, share_first, share_last, lane, px.cx, px.cy, [&](uint32_t addr) {
            TileFrag f;
            if (!active || !tile_frag_cutoff<kStageSlots>(addr, pt, f)) return;
            const float G = d_exp2((f.num * ModeCfg<MODE>::exp2_scale) * rcp_exact(f.den));
            const float a = stage_opacity<kStageSlots>(addr) * G;
            const float w = (a < kMaxFragmentAlpha ? a : kMaxFragmentAlpha) * tail_weight;
            if (!(w < weight_threshold)) raise_max(max_weights, stage_index<kStageSlots>(addr), w);
        });
    }
}

// the least length of a part of a long list; 0: lists are not split (there is no spare value buffer for what the parts leave behind)
static uint32_t part_floor_of(const htgs_frame *f, int sel, uint32_t n_tiles, bool needs_spare)
{
    if (needs_spare && f->vals[sel ^ 1] == nullptr) return 0u;
    const uint64_t floor = (f->n_instances + n_tiles - 1) / n_tiles;
    return floor < 1u ? 1u : (uint32_t)floor;
}
// the tiles with very long lists are taken by the kernels that share a list only when the caller provided the list for such
// tiles and, in the modes with a tail, the per-pixel scratch for the tail weights between the two walks
template <int MODE>
static bool shares_long_lists(const htgs_frame *f) { return f->long_tiles != nullptr && (MODE == HTGS_MODE_ALPHA_BLEND_FIRST_K || f->pixel_scratch != nullptr); }

template <int K, int MODE>
static void launch_tile(const htgs_frame *f, int sel, uint32_t *max_weights, float thr, uint32_t grid_w, uint32_t n_tiles)
{
    hipStream_t s = (hipStream_t)f->stream;
    const uint32_t threshold = f->long_list_threshold > 0 ? (uint32_t)f->long_list_threshold : kLongListDefault;
    const bool shared = shares_long_lists<MODE>(f);
    const uint32_t w = (uint32_t)f->width, h = (uint32_t)f->height;
    hipLaunchKernelGGL((max_weights_tile_kernel<K, MODE>), dim3(n_tiles), dim3(64), 0, s, f->ranges, f->vals[sel], (const float4 *)f->prim, max_weights, w, h, grid_w,
                       thr, f->tile_order, shared ? f->long_tiles : nullptr, threshold, part_floor_of(f, sel, n_tiles, true));
    if (!shared) return;
    constexpr int REC4 = HTGS_PRIM_FLOATS / 4;
    if constexpr (MODE == HTGS_MODE_HYBRID_BLEND)
        hipLaunchKernelGGL((blend_hybrid_long_kernel<K, false, REC4, MaxWeightsHybrid>), dim3(256 * kLongWaves / long_waves<K>()), dim3(64 * long_waves<K>()), 0, s,
                           f->ranges, f->vals[sel], (const float4 *)f->prim, f->long_tiles, w, h, grid_w, f->vals[sel ^ 1], threshold,
                           MaxWeightsHybrid{ max_weights, f->pixel_scratch, thr });
    else if constexpr (MODE == HTGS_MODE_ALPHA_BLEND_FIRST_K)
        hipLaunchKernelGGL((blend_first_k_long_kernel<K, false, REC4, MaxWeightsFirstK>), dim3(256 * kLongWaves / long_waves<K>()), dim3(64 * long_waves<K>()), 0, s,
                           f->ranges, f->vals[sel], (const float4 *)f->prim, f->long_tiles, w, h, grid_w, f->vals[sel ^ 1], threshold, MaxWeightsFirstK{ max_weights, thr });
    else
        hipLaunchKernelGGL((blend_oit_long_kernel<false, REC4, MaxWeightsOit, false>), dim3(256), dim3(64 * kLongWaves), 0, s, f->ranges, f->vals[sel],
                           (const float4 *)f->prim, f->long_tiles, w, h, grid_w, f->vals[sel ^ 1], threshold, MaxWeightsOit{ f->pixel_scratch, thr });
    if constexpr (MODE != HTGS_MODE_ALPHA_BLEND_FIRST_K) {
        hipLaunchKernelGGL(max_weights_tail_enter_kernel, dim3((n_tiles + 255) / 256), dim3(256), 0, s, f->ranges, f->long_tiles, n_tiles, threshold,
                           part_floor_of(f, sel, n_tiles, false));
        hipLaunchKernelGGL(max_weights_tail_long_kernel<MODE>, dim3(1024), dim3(64 * kTailWaves), 0, s, f->ranges, f->vals[sel], (const float4 *)f->prim, f->long_tiles,
                           max_weights, f->pixel_scratch, w, h, grid_w, thr, threshold);
    }
}

template <int MODE>
static void dispatch_tile(const htgs_frame *f, int sel, uint32_t *mw, float thr, uint32_t grid_w, uint32_t n_tiles)
{
    switch (htgs_effective_k(f->K)) {
        case 32: launch_tile<32, MODE>(f, sel, mw, thr, grid_w, n_tiles); break;
        case 16: launch_tile<16, MODE>(f, sel, mw, thr, grid_w, n_tiles); break;
        case 8: launch_tile<8, MODE>(f, sel, mw, thr, grid_w, n_tiles); break;
        case 4: launch_tile<4, MODE>(f, sel, mw, thr, grid_w, n_tiles); break;
        case 2: launch_tile<2, MODE>(f, sel, mw, thr, grid_w, n_tiles); break;
        default: launch_tile<1, MODE>(f, sel, mw, thr, grid_w, n_tiles); break;
    }
}

}  // namespace htgs

using namespace htgs;

extern "C" int htgs_max_weights_front(const htgs_frame *f)
{
    if (!f) return fail(HTGS_ERR_ARGUMENT, "htgs_max_weights_front: null frame");
    htgs_frame t = *f;
    t.scale_modifier = 1.0f;      // update_max_weights.cuh:46: the scale modifier is not applied
    t.sh_0 = nullptr;             // no colours
    t.sh_rest = nullptr;
    t.active_sh_bases = 1;
    t.total_sh_bases = 0;
    t.clamp_info = nullptr;
    int rc = htgs_preprocess(&t);
    if (rc != HTGS_OK) return rc;
    return htgs_scan_offsets(&t);
}

extern "C" int htgs_max_weights_blend(const htgs_frame *f, int selector, float *max_weights, float weight_threshold)
{
    if (!f) return fail(HTGS_ERR_ARGUMENT, "htgs_max_weights_blend: null frame");
    if (f->mode < 0 || f->mode > 3) return fail(HTGS_ERR_MODE, "unsupported rasterizer mode");
    if (selector < 0 || selector > 1 || f->width <= 0 || f->height <= 0) return fail(HTGS_ERR_ARGUMENT, "htgs_max_weights_blend: bad argument");
    if (frame_prim_floats(f) != HTGS_PRIM_FLOATS) return fail(HTGS_ERR_ARGUMENT, "htgs_max_weights_blend: reads records of HTGS_PRIM_FLOATS floats (prim_floats)");
    if (f->n_instances == 0 || f->n_primitives == 0) return HTGS_OK;
    if (!f->ranges || !f->vals[selector] || !f->prim || !max_weights) return fail(HTGS_ERR_ARGUMENT, "htgs_max_weights_blend: null pointer");
    const int tile = tile_size(f->mode);
    const uint32_t grid_w = div_up(f->width, tile), grid_h = div_up(f->height, tile);
    const uint32_t n_tiles = grid_w * grid_h;
    uint32_t *mw = reinterpret_cast<uint32_t *>(max_weights);
    switch (f->mode) {
        case HTGS_MODE_HYBRID_BLEND: dispatch_tile<HTGS_MODE_HYBRID_BLEND>(f, selector, mw, weight_threshold, grid_w, n_tiles); break;
        case HTGS_MODE_ALPHA_BLEND_FIRST_K: dispatch_tile<HTGS_MODE_ALPHA_BLEND_FIRST_K>(f, selector, mw, weight_threshold, grid_w, n_tiles); break;
        case HTGS_MODE_OIT_BLEND: launch_tile<1, HTGS_MODE_OIT_BLEND>(f, selector, mw, weight_threshold, grid_w, n_tiles); break;
        default:
            hipLaunchKernelGGL(max_weights_global_kernel, dim3(n_tiles), dim3(256), 0, (hipStream_t)f->stream, f->ranges, f->vals[selector],
                               (const float4 *)f->prim, mw, (uint32_t)f->width, (uint32_t)f->height, grid_w, weight_threshold, f->tile_order);
            break;
    }
    return check_launch("max_weights");
}

extern "C" int htgs_max_weights_back(const htgs_frame *f, float *max_weights, float weight_threshold)
{
    int selector = 0;
    int rc = htgs_create_instances(f);
    if (rc != HTGS_OK) return rc;
    rc = htgs_sort_instances(f, &selector);
    if (rc != HTGS_OK) return rc;
    rc = htgs_extract_ranges(f, selector);
    if (rc != HTGS_OK) return rc;
    return htgs_max_weights_blend(f, selector, max_weights, weight_threshold);
}
