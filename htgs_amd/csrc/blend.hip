// Per-tile blend kernels of the four modes (inference: image + depth).
// Restates blend_cu of R/include/hybrid_blend/kernels/inference.cuh:78-216,
// R/include/alpha_blend_first_k/kernels/inference.cuh:78-206,
// R/include/alpha_blend_global_ordering/kernels/inference.cuh:78-176 and
// R/include/oit_blend/kernels/inference.cuh:78-177.
//
// An 8x8 tile is exactly one wave64: one workgroup = one wave, Gaussian records are staged 64 at a
// time in LDS (every lane then reads the same address, a broadcast), the K-buffer lives in VGPRs.
// The 16x16 tiles of the global-ordering mode use four waves and a workgroup barrier.
// Every kernel has a second instantiation, FAST, for the image-only path of the reference's fast_inference
// kernels (R/include/<mode>/kernels/fast_inference.cuh): hardware reciprocal and 2^x, no depth.
#include "blend_common.h"

#include "blend_long.h"

namespace htgs {

// ---------------------------------------------------------------------------------------------
// ALPHA_BLEND_GLOBAL_ORDERING: instances arrive sorted by (tile, depth of the Gaussian centre);
// classic front-to-back blending, a pixel stops at T < 1e-4, the workgroup stops when all have.
// ---------------------------------------------------------------------------------------------
// A wave holds one 8x8 sub-tile of the 16x16 tile, laid out for the quadrant walk; the 256 threads stage 256 instances
// per batch, each with one bit per 4x4 quadrant of the tile it can reach, and every wave then walks the hits of its own
// four quadrants, 64 staged slots at a time.
template <bool FAST>
__global__ void __launch_bounds__(256) blend_global_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
    float *__restrict__ image, float *__restrict__ depths, uint32_t width, uint32_t height, uint32_t grid_w, int chw, int median, const uint32_t *__restrict__ tile_order)
{
    constexpr int MODE = HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING;
    __shared__ TileStage<256> st;
    __shared__ uint16_t s_reach[256];                  // per staged slot: the quadrants of the tile it can reach
    const uint32_t tile = block_tile(tile_order);
    const uint32_t t = threadIdx.x, wave = t >> 6, lane = t & 63;
    const uint32_t x0 = (tile % grid_w) * 16, y0 = (tile / grid_w) * 16;
    uint32_t local_x, local_y;
    subtile_pixel(t, local_x, local_y);
    const uint32_t x = x0 + local_x, y = y0 + local_y;
    const bool inside = x < width && y < height;
    const PixelTerms pt = pixel_terms(local_x, local_y, 16);
    const float cx = tile_centre(x0, 16), cy = tile_centre(y0, 16);
    float r = 0.0f, g = 0.0f, b = 0.0f, depth_pixel = 0.0f, T = 1.0f;
    bool done = !inside;

    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    for (uint32_t base = first; base < last; base += 256) {
        if (__syncthreads_count(done) == 256) break;
        s_reach[t] = (uint16_t)tile_stage_load<MODE, 256, false, kCullAlpha, true>(st, prim, inst, base + t, last, t, cx, cy);
        __syncthreads();
        const uint32_t stage_base = __builtin_amdgcn_readfirstlane(stage_address(st));
        subtile_walk(s_reach, stage_base, last - base < 256u ? last - base : 256u, wave, lane,
                     [&]() { return __ballot(!done) == 0; },       // every pixel of the sub-tile is opaque
                     [&](uint32_t addr) {
            TileFrag f;
            if (done || !tile_frag_cutoff<256>(addr, pt, f)) return;
            f.den_rcp = frag_rcp<FAST>(f.den);
            const float4 q4 = stage_row<256, 4>(addr);
            if (!tile_frag_alpha<MODE, FAST>(q4.w, f)) return;
            const float4 col = stage_row<256, 5>(addr);
            const float wgt = T * f.alpha;
            r = __builtin_fmaf(wgt, col.x, r);
            g = __builtin_fmaf(wgt, col.y, g);
            b = __builtin_fmaf(wgt, col.z, b);
            const float depth = q4.z;
            if (median) depth_pixel = T > 0.5f ? depth : depth_pixel;
            else depth_pixel = __builtin_fmaf(wgt, depth, depth_pixel);
            T *= 1.0f - f.alpha;
            if (T < kTransmittanceThreshold) done = true;
        });
    }
    if (!inside) return;
    if (!median) depth_pixel = T < 1.0f ? depth_pixel / (1.0f - T) : 0.0f;
    store_pixel(image, depths, width, height, x, y, chw, r, g, b, depth_pixel);
}

// Self-check of the staging cull (tile_stage_load with CULL, per quadrant): every instance of every 8x8 tile is evaluated
// at all 64 pixels with the blend kernels' own cut-off and alpha tests and the outcome is compared, quadrant by quadrant,
// with the verdict of the lane that staged it.  counts: instances looked at, instances that reach no pixel of the tile,
// instances left out of all four quadrants, (instance, quadrant) pairs left out although a pixel there is reached.
template <int MODE>
__global__ void __launch_bounds__(64) check_tile_cull_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, uint32_t grid_w,
    unsigned long long *__restrict__ counts)
{
    __shared__ TileStage<64> st;
    const uint32_t tile = blockIdx.x, lane = threadIdx.x;
    const TilePixel px = quadrant_tile_pixel(tile, grid_w, lane, 0xffffffffu, 0xffffffffu);
    const PixelTerms pt = px.pt;
    const float cx = px.cx, cy = px.cy;
    unsigned long long seen = 0, empty = 0, missed = 0, wrong = 0;
    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    for (uint32_t base = first; base < last; base += 64) {
        __syncthreads();
        QuadrantHits hits = quadrant_ballot(tile_stage_load<MODE, 64, false, kCullAlpha, true>(st, prim, inst, base + lane, last, lane, cx, cy));
        __syncthreads();
        const int nb = last - base < 64u ? (int)(last - base) : 64;
        uint32_t addr = stage_address(st);
        for (int j = 0; j < nb; ++j, stage_advance(addr)) {
            TileFrag f;
            bool pass = tile_frag_cutoff<64>(addr, pt, f);
            if (pass) {
                f.den_rcp = rcp_exact(f.den);
                pass = tile_frag_alpha<MODE>(stage_opacity<64>(addr), f);
            }
            const uint64_t reached = __ballot(pass);
            bool kept = false;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const bool keep = (hits.h[q] >> j) & 1;
                kept = kept || keep;
                wrong += !keep && ((reached >> (16 * q)) & 0xffffu) != 0;
            }
            ++seen; empty += reached == 0; missed += !kept;
        }
    }
    if (lane == 0 && seen) {
        atomicAdd(counts, seen); atomicAdd(counts + 1, empty); atomicAdd(counts + 2, missed);
        if (wrong) atomicAdd(counts + 3, wrong);
    }
}

// The same for the 16x16 tiles of ALPHA_BLEND_GLOBAL_ORDERING (sixteen quadrants per tile): every thread evaluates its
// pixel for every staged instance, the waves note which quadrants are reached, and one thread per instance compares.
__global__ void __launch_bounds__(256) check_tile_cull_16_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, uint32_t grid_w,
    unsigned long long *__restrict__ counts)
{
    constexpr int MODE = HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING;
    __shared__ TileStage<256> st;
    __shared__ uint32_t s_reach[256], s_reached[256];
    const uint32_t tile = blockIdx.x, t = threadIdx.x, wave = t >> 6, lane = t & 63;
    const uint32_t x0 = (tile % grid_w) * 16, y0 = (tile / grid_w) * 16;
    uint32_t local_x, local_y;
    subtile_pixel(t, local_x, local_y);
    const PixelTerms pt = pixel_terms(local_x, local_y, 16);
    const float cx = tile_centre(x0, 16), cy = tile_centre(y0, 16);
    unsigned long long seen = 0, empty = 0, missed = 0, wrong = 0;
    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    for (uint32_t base = first; base < last; base += 256) {
        __syncthreads();
        s_reach[t] = tile_stage_load<MODE, 256, false, kCullAlpha, true>(st, prim, inst, base + t, last, t, cx, cy);
        s_reached[t] = 0u;
        __syncthreads();
        const int nb = last - base < 256u ? (int)(last - base) : 256;
        uint32_t addr = stage_address(st);
        for (int j = 0; j < nb; ++j, stage_advance(addr)) {
            TileFrag f;
            bool pass = tile_frag_cutoff<256>(addr, pt, f);
            if (pass) {
                f.den_rcp = rcp_exact(f.den);
                pass = tile_frag_alpha<MODE>(stage_opacity<256>(addr), f);
            }
            const uint64_t reached = __ballot(pass);
            uint32_t bits = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q) bits |= (((reached >> (16 * q)) & 0xffffu) != 0 ? 1u : 0u) << (4 * wave + q);
            if (lane == 0 && bits) atomicOr(&s_reached[j], bits);
        }
        __syncthreads();
        if (t < (uint32_t)nb) {
            const uint32_t kept = s_reach[t], reached = s_reached[t];
            ++seen; empty += reached == 0; missed += kept == 0; wrong += (unsigned)__builtin_popcount(reached & ~kept);
        }
    }
    if (seen) {
        atomicAdd(counts, seen); atomicAdd(counts + 1, empty); atomicAdd(counts + 2, missed);
        if (wrong) atomicAdd(counts + 3, wrong);
    }
}

// the least length of a part of a long list (0: lists are not split, there is no spare value buffer to leave the parts' results in)
static uint32_t long_part_floor(const htgs_frame *f, int selector, uint32_t n_tiles)
{
    if (f->vals[selector ^ 1] == nullptr) return 0u;
    const uint64_t floor = (f->n_instances + n_tiles - 1) / n_tiles;
    return floor < 1u ? 1u : (uint32_t)floor;
}

template <int K, bool FAST>
static void launch_hybrid(const htgs_frame *f, int selector, uint32_t grid_w, uint32_t n_tiles)
{
    const uint32_t threshold = f->long_list_threshold > 0 ? (uint32_t)f->long_list_threshold : kLongListDefault;
    // (the fast path packs a core entry's place in its list into 13 bits where no list of the launch can be longer)
    if (f->long_tiles != nullptr && threshold <= kPackedListMost)
        hipLaunchKernelGGL((blend_hybrid_kernel<K, FAST, true>), dim3(n_tiles), dim3(64), 0, (hipStream_t)f->stream, f->ranges, f->vals[selector],
                           (const float4 *)f->prim, f->image, FAST ? nullptr : f->depth, (uint32_t)f->width, (uint32_t)f->height, grid_w, f->to_chw,
                           f->use_median_depth, f->long_tiles, threshold, long_part_floor(f, selector, n_tiles), f->tile_order);
    else
        hipLaunchKernelGGL((blend_hybrid_kernel<K, FAST>), dim3(n_tiles), dim3(64), 0, (hipStream_t)f->stream, f->ranges, f->vals[selector],
                           (const float4 *)f->prim, f->image, FAST ? nullptr : f->depth, (uint32_t)f->width, (uint32_t)f->height, grid_w, f->to_chw,
                           f->use_median_depth, f->long_tiles, threshold, long_part_floor(f, selector, n_tiles), f->tile_order);
    if (f->long_tiles)      // (one workgroup per compute unit; they find an empty list on ordinary frames)
        hipLaunchKernelGGL((blend_hybrid_long_kernel<K, FAST, HTGS_PRIM_FLOATS / 4, HybridImage>), dim3(256 * kLongWaves / long_waves<K>()), dim3(64 * long_waves<K>()), 0,
                           (hipStream_t)f->stream, f->ranges, f->vals[selector], (const float4 *)f->prim, f->long_tiles, (uint32_t)f->width, (uint32_t)f->height, grid_w,
                           f->vals[selector ^ 1], threshold,
                           HybridImage{ f->image, FAST ? nullptr : f->depth, (uint32_t)f->width, (uint32_t)f->height, f->to_chw, f->use_median_depth });
}
template <int K, bool FAST>
static void launch_first_k(const htgs_frame *f, int selector, uint32_t grid_w, uint32_t n_tiles)
{
    const uint32_t threshold = f->long_list_threshold > 0 ? (uint32_t)f->long_list_threshold : kLongListDefault;
    if (!FAST && f->long_tiles != nullptr && threshold <= kPackedListMost)
        hipLaunchKernelGGL((blend_first_k_kernel<K, false, true>), dim3(n_tiles), dim3(64), 0, (hipStream_t)f->stream, f->ranges, f->vals[selector],
                           (const float4 *)f->prim, f->image, f->depth, (uint32_t)f->width, (uint32_t)f->height, grid_w, f->to_chw,
                           f->use_median_depth, f->long_tiles, threshold, long_part_floor(f, selector, n_tiles), f->tile_order);
    else
        hipLaunchKernelGGL((blend_first_k_kernel<K, FAST>), dim3(n_tiles), dim3(64), 0, (hipStream_t)f->stream, f->ranges, f->vals[selector],
                           (const float4 *)f->prim, f->image, FAST ? nullptr : f->depth, (uint32_t)f->width, (uint32_t)f->height, grid_w, f->to_chw,
                           f->use_median_depth, f->long_tiles, threshold, long_part_floor(f, selector, n_tiles), f->tile_order);
    if (f->long_tiles)
        hipLaunchKernelGGL((blend_first_k_long_kernel<K, FAST, HTGS_PRIM_FLOATS / 4, FirstKImage>), dim3(256 * kLongWaves / long_waves<K>()), dim3(64 * long_waves<K>()), 0,
                           (hipStream_t)f->stream, f->ranges, f->vals[selector], (const float4 *)f->prim, f->long_tiles, (uint32_t)f->width, (uint32_t)f->height, grid_w,
                           f->vals[selector ^ 1], threshold,
                           FirstKImage{ f->image, FAST ? nullptr : f->depth, (uint32_t)f->width, (uint32_t)f->height, f->to_chw, f->use_median_depth });
}

template <bool FAST>
static void launch_blend(const htgs_frame *f, int selector, uint32_t grid_w, uint32_t n_tiles)
{
    const int K = htgs_effective_k(f->K);
    hipStream_t s = (hipStream_t)f->stream;
    float *depth = FAST ? nullptr : f->depth;
    switch (f->mode) {
        case HTGS_MODE_HYBRID_BLEND:
            switch (K) {
                case 32: launch_hybrid<32, FAST>(f, selector, grid_w, n_tiles); break;
                case 16: launch_hybrid<16, FAST>(f, selector, grid_w, n_tiles); break;
                case 8: launch_hybrid<8, FAST>(f, selector, grid_w, n_tiles); break;
                case 4: launch_hybrid<4, FAST>(f, selector, grid_w, n_tiles); break;
                case 2: launch_hybrid<2, FAST>(f, selector, grid_w, n_tiles); break;
                default: launch_hybrid<1, FAST>(f, selector, grid_w, n_tiles); break;
            }
            break;
        case HTGS_MODE_ALPHA_BLEND_FIRST_K:
            switch (K) {
                case 32: launch_first_k<32, FAST>(f, selector, grid_w, n_tiles); break;
                case 16: launch_first_k<16, FAST>(f, selector, grid_w, n_tiles); break;
                case 8: launch_first_k<8, FAST>(f, selector, grid_w, n_tiles); break;
                case 4: launch_first_k<4, FAST>(f, selector, grid_w, n_tiles); break;
                case 2: launch_first_k<2, FAST>(f, selector, grid_w, n_tiles); break;
                default: launch_first_k<1, FAST>(f, selector, grid_w, n_tiles); break;
            }
            break;
        case HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING:
            hipLaunchKernelGGL(blend_global_kernel<FAST>, dim3(n_tiles), dim3(256), 0, s, f->ranges, f->vals[selector], (const float4 *)f->prim,
                               f->image, depth, (uint32_t)f->width, (uint32_t)f->height, grid_w, f->to_chw, f->use_median_depth, f->tile_order);
            break;
        default:
        {
            const uint32_t threshold = f->long_list_threshold > 0 ? (uint32_t)f->long_list_threshold : kLongListDefault;
            hipLaunchKernelGGL(blend_oit_kernel<FAST>, dim3(n_tiles), dim3(64), 0, s, f->ranges, f->vals[selector], (const float4 *)f->prim,
                               f->image, depth, (uint32_t)f->width, (uint32_t)f->height, grid_w, f->to_chw, f->long_tiles, threshold,
                               long_part_floor(f, selector, n_tiles), f->tile_order);
            if (f->long_tiles)
                hipLaunchKernelGGL((blend_oit_long_kernel<FAST, HTGS_PRIM_FLOATS / 4, OitImage>), dim3(256), dim3(64 * kLongWaves), 0, s, f->ranges, f->vals[selector],
                                   (const float4 *)f->prim, f->long_tiles, (uint32_t)f->width, (uint32_t)f->height, grid_w, f->vals[selector ^ 1], threshold,
                                   OitImage{ f->image, depth, (uint32_t)f->width, (uint32_t)f->height, f->to_chw });
            break;
        }
    }
}

}  // namespace htgs

using namespace htgs;

extern "C" int htgs_effective_k(int K)
{
    return K >= 32 ? 32 : K >= 16 ? 16 : K >= 8 ? 8 : K >= 4 ? 4 : K >= 2 ? 2 : 1;
}

extern "C" int htgs_blend(const htgs_frame *f, int selector)
{
    if (!f) return fail(HTGS_ERR_ARGUMENT, "htgs_blend: null frame");
    if (f->mode < 0 || f->mode > 3) return fail(HTGS_ERR_MODE, "unsupported rasterizer mode");
    if (selector < 0 || selector > 1 || f->width <= 0 || f->height <= 0) return fail(HTGS_ERR_ARGUMENT, "htgs_blend: bad argument");
    if (frame_prim_floats(f) != HTGS_PRIM_FLOATS) return fail(HTGS_ERR_ARGUMENT, "htgs_blend: the inference kernels read records of HTGS_PRIM_FLOATS floats (prim_floats)");
    if (!f->ranges || !f->image || (!f->depth && !f->fast_math) || (f->n_instances > 0 && (!f->vals[selector] || !f->prim)))
        return fail(HTGS_ERR_ARGUMENT, "htgs_blend: null pointer");
    const int tile = tile_size(f->mode);
    const uint32_t grid_w = div_up(f->width, tile), grid_h = div_up(f->height, tile);
    const uint32_t n_tiles = grid_w * grid_h;
    // (an entry of the list of long tiles holds the tile in 20 bits; htgs_scan_offsets refuses larger grids as well)
    if ((uint64_t)grid_w * grid_h > (1ull << 20)) return fail(HTGS_ERR_ARGUMENT, "htgs_blend: more than 2^20 tiles");
    if (f->fast_math) launch_blend<true>(f, selector, grid_w, n_tiles);
    else launch_blend<false>(f, selector, grid_w, n_tiles);
    return check_launch("blend");
}

extern "C" int htgs_check_tile_cull(const htgs_frame *f, int selector, unsigned long long *counts)
{
    if (!f || !counts) return fail(HTGS_ERR_ARGUMENT, "htgs_check_tile_cull: null pointer");
    if (f->mode < 0 || f->mode > 3) return fail(HTGS_ERR_MODE, "unsupported rasterizer mode");
    if (selector < 0 || selector > 1 || f->width <= 0 || f->height <= 0) return fail(HTGS_ERR_ARGUMENT, "htgs_check_tile_cull: bad argument");
    if (!f->ranges || (f->n_instances > 0 && (!f->vals[selector] || !f->prim))) return fail(HTGS_ERR_ARGUMENT, "htgs_check_tile_cull: null pointer");
    if (frame_prim_floats(f) != HTGS_PRIM_FLOATS) return fail(HTGS_ERR_ARGUMENT, "htgs_check_tile_cull: reads records of HTGS_PRIM_FLOATS floats (prim_floats)");
    const int tile = tile_size(f->mode);
    const uint32_t grid_w = div_up(f->width, tile), n_tiles = grid_w * div_up(f->height, tile);
    hipStream_t s = (hipStream_t)f->stream;
    const float4 *prim = (const float4 *)f->prim;
    if (f->mode == HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING)
        hipLaunchKernelGGL(check_tile_cull_16_kernel, dim3(n_tiles), dim3(256), 0, s, f->ranges, f->vals[selector], prim, grid_w, counts);
    else if (f->mode == HTGS_MODE_ALPHA_BLEND_FIRST_K)
        hipLaunchKernelGGL(check_tile_cull_kernel<HTGS_MODE_ALPHA_BLEND_FIRST_K>, dim3(n_tiles), dim3(64), 0, s, f->ranges, f->vals[selector], prim, grid_w, counts);
    else if (f->mode == HTGS_MODE_OIT_BLEND)
        hipLaunchKernelGGL(check_tile_cull_kernel<HTGS_MODE_OIT_BLEND>, dim3(n_tiles), dim3(64), 0, s, f->ranges, f->vals[selector], prim, grid_w, counts);
    else
        hipLaunchKernelGGL(check_tile_cull_kernel<HTGS_MODE_HYBRID_BLEND>, dim3(n_tiles), dim3(64), 0, s, f->ranges, f->vals[selector], prim, grid_w, counts);
    return check_launch("check_tile_cull");
}
