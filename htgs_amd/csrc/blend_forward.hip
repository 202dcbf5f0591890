// Training forward blend of the four modes: unclamped [3,H,W] image plus the per-pixel records that the
// backward pass needs.  Restates blend_cu of R/include/hybrid_blend/kernels/forward.cuh:78-235,
// R/include/alpha_blend_first_k/kernels/forward.cuh:78-215,
// R/include/alpha_blend_global_ordering/kernels/forward.cuh:78-156 and
// R/include/oit_blend/kernels/forward.cuh:76-165.
//
// Records are pixel-minor ([slot][pixel]) so that a wave writes 64 consecutive words.  Where the reference
// leaves a record unwritten (tail with an alpha sum below 1/255, skipped core slots) zeros are stored, so that
// backward never reads indeterminate memory.
#include "blend_common.h"

namespace htgs {

__device__ __forceinline__ float one_minus_alpha_rcp(float one_minus_alpha)
{
    return 1.0f / (one_minus_alpha > kOneMinusAlphaEps ? one_minus_alpha : kOneMinusAlphaEps);
}

template <int K>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(K <= 16 ? 5 : 3))) blend_hybrid_forward_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
    float *__restrict__ image, uint32_t *__restrict__ core_idx, float4 *__restrict__ core_info, float *__restrict__ tail_info,
    uint32_t width, uint32_t height, uint32_t grid_w, const uint32_t *__restrict__ tile_order)
{
    constexpr int MODE = HTGS_MODE_HYBRID_BLEND;
    __shared__ TileStageQ st;
    __shared__ QuadrantLists ql;
    const uint32_t tile = block_tile(tile_order);
    const uint32_t lane = threadIdx.x;
    const TilePixel px = quadrant_tile_pixel(tile, grid_w, lane, width, height);
    const uint32_t x = px.x, y = px.y;
    const bool inside = px.inside;
    const PixelTerms pt = px.pt;
    const float cx = px.cx, cy = px.cy;

    float T_tail = 1.0f, tail0 = 0.0f, tail1 = 0.0f, tail2 = 0.0f, tail3 = 0.0f;
    // slots hold depth, alpha and index; colours are fetched at the end and the core's share of the colour sums is
    // taken out there (see blend_hybrid_kernel)
    float c3[K], cd[K];
    uint32_t ci[K];
#pragma unroll
    for (int i = 0; i < K; ++i) {
        c3[i] = 0.0f; cd[i] = __FLT_MAX__; ci[i] = 0xffffffffu;
        asm volatile("" : "+v"(cd[i]), "+v"(c3[i]), "+v"(ci[i]));      // one register per slot
    }

    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    tile_list_walk<MODE, true, kCullAlpha, true, HTGS_PRIM_FLOATS_TRAIN / 4>(st, ql, prim, inst, first, last, lane, cx, cy, [&](uint32_t addr) {
        TileFrag f;
        const bool in_reach = tile_frag_cutoff<kStageSlots>(addr, pt, f);
        f.den_rcp = rcp_exact(f.den);
        const float4 col = stage_row<kStageSlots, 5>(addr);
        if (!(tile_frag_alpha<MODE>(stage_opacity<kStageSlots>(addr), f) && in_reach)) return;
        float depth = tile_frag_depth<kStageSlots>(addr, pt, f);
        float p3 = f.alpha;
        tail0 = __builtin_fmaf(p3, col.x, tail0);
        tail1 = __builtin_fmaf(p3, col.y, tail1);
        tail2 = __builtin_fmaf(p3, col.z, tail2);
        if (depth < cd[K - 1] && f.alpha >= kMinAlphaCore) {
            uint32_t idx = stage_index<kStageSlots>(addr);
            core_exchange_walk<K>(depth, p3, idx, cd, c3, ci);
        }
        tail3 += p3;
        T_tail *= 1.0f - p3;
    });
    if (!inside) return;

    const size_t pix = (size_t)width * y + x, np = (size_t)width * height;
    const size_t rp = record_pixel(tile, x, y), rnp = record_plane();
    float c0[K], c1[K], c2[K];
#pragma unroll
    for (int i = 0; i < K; ++i) {
        float4 c = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (c3[i] > 0.0f) c = prim[(size_t)ci[i] * (HTGS_PRIM_FLOATS_TRAIN / 4) + 4];
        c0[i] = c.x; c1[i] = c.y; c2[i] = c.z;
    }
#pragma unroll
    for (int i = 0; i < K; ++i) {
        tail0 = __builtin_fmaf(-c3[i], c0[i], tail0);
        tail1 = __builtin_fmaf(-c3[i], c1[i], tail1);
        tail2 = __builtin_fmaf(-c3[i], c2[i], tail2);
    }
    tail0 = clamp_pos(tail0); tail1 = clamp_pos(tail1); tail2 = clamp_pos(tail2);   // colours are >= 0, so is the exact difference
    float r = 0.0f, g = 0.0f, b = 0.0f, T_core = 1.0f;
#pragma unroll
    for (int i = 0; i < K; ++i) {
        if (T_core >= kTransmittanceThreshold) {
            const float bw = T_core * c3[i];
            r = __builtin_fmaf(bw, c0[i], r);
            g = __builtin_fmaf(bw, c1[i], g);
            b = __builtin_fmaf(bw, c2[i], b);
            T_core *= 1.0f - c3[i];
            if (T_core < kTransmittanceThreshold) T_core = 0.0f;
        }
    }
    float w0 = 0.0f, w1 = 0.0f, w2 = 0.0f;
    float t0 = 0.0f, t1 = 0.0f, t2 = 0.0f, t3 = 0.0f, t4 = 0.0f, t5 = 0.0f;
    if (tail3 >= ModeCfg<MODE>::min_alpha) {
        const float asr = 1.0f / tail3;
        const float s = (T_core * (1.0f - T_tail)) * asr;
        w0 = s * tail0; w1 = s * tail1; w2 = s * tail2;
        t0 = tail0; t1 = tail1; t2 = tail2; t3 = asr; t4 = T_tail; t5 = T_core;
    }
    tail_info[rp] = t0; tail_info[rnp + rp] = t1; tail_info[2 * rnp + rp] = t2;
    tail_info[3 * rnp + rp] = t3; tail_info[4 * rnp + rp] = t4; tail_info[5 * rnp + rp] = t5;

    float n0 = 0.0f, n1 = 0.0f, n2 = 0.0f;
    T_core = 1.0f;
#pragma unroll
    for (int i = 0; i < K; ++i) {
        const bool skip = ci[i] == 0xffffffffu || T_core < kTransmittanceThreshold;
        core_idx[(size_t)i * rnp + rp] = skip ? 0xffffffffu : ci[i];
        float4 info = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (!skip) {
            const float bw = T_core * c3[i];
            n0 = __builtin_fmaf(bw, c0[i], n0);
            n1 = __builtin_fmaf(bw, c1[i], n1);
            n2 = __builtin_fmaf(bw, c2[i], n2);
            const float oma = 1.0f - c3[i];
            const float omar = one_minus_alpha_rcp(oma);
            info.x = __builtin_fmaf(c0[i], T_core, -(((r - n0) + w0) * omar));
            info.y = __builtin_fmaf(c1[i], T_core, -(((g - n1) + w1) * omar));
            info.z = __builtin_fmaf(c2[i], T_core, -(((b - n2) + w2) * omar));
            info.w = bw;
            T_core *= oma;
        }
        core_info[(size_t)i * rnp + rp] = info;
    }
    image[pix] = r + w0; image[np + pix] = g + w1; image[2 * np + pix] = b + w2;
}

template <int K>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(K <= 16 ? 5 : 2))) blend_first_k_forward_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
    float *__restrict__ image, uint32_t *__restrict__ core_idx, float4 *__restrict__ core_info,
    uint32_t width, uint32_t height, uint32_t grid_w, const uint32_t *__restrict__ tile_order)
{
    constexpr int MODE = HTGS_MODE_ALPHA_BLEND_FIRST_K;
    __shared__ TileStageQ st;
    __shared__ QuadrantLists ql;
    const uint32_t tile = block_tile(tile_order);
    const uint32_t lane = threadIdx.x;
    const TilePixel px = quadrant_tile_pixel(tile, grid_w, lane, width, height);
    const uint32_t x = px.x, y = px.y;
    const bool inside = px.inside;
    const PixelTerms pt = px.pt;
    const float cx = px.cx, cy = px.cy;

    float ca[K], cd[K];
    uint32_t ci[K];
#pragma unroll
    for (int i = 0; i < K; ++i) {
        ca[i] = 0.0f; cd[i] = __FLT_MAX__; ci[i] = 0xffffffffu;
        asm volatile("" : "+v"(cd[i]), "+v"(ca[i]), "+v"(ci[i]));      // one register per slot
    }

    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    tile_list_walk<MODE, true, kCullAlpha, true, HTGS_PRIM_FLOATS_TRAIN / 4>(st, ql, prim, inst, first, last, lane, cx, cy, [&](uint32_t addr) {
        TileFrag f;
        const bool in_reach = tile_frag_cutoff<kStageSlots>(addr, pt, f);
        f.den_rcp = rcp_exact(f.den);
        float depth = tile_frag_depth<kStageSlots>(addr, pt, f);
        if (!(in_reach && depth < cd[K - 1])) return;
        if (!tile_frag_alpha<MODE>(stage_opacity<kStageSlots>(addr), f)) return;
        float alpha = f.alpha;
        uint32_t idx = stage_index<kStageSlots>(addr);
        core_exchange_walk<K>(depth, alpha, idx, cd, ca, ci);
    });
    if (!inside) return;

    const size_t pix = (size_t)width * y + x, np = (size_t)width * height;
    const size_t rp = record_pixel(tile, x, y), rnp = record_plane();
    float r = 0.0f, g = 0.0f, b = 0.0f, T = 1.0f;
    float k0[K], k1[K], k2[K];
    bool open = true;
#pragma unroll
    for (int i = 0; i < K; ++i) {
        open = open && T >= kTransmittanceThreshold && ci[i] != 0xffffffffu;
        k0[i] = k1[i] = k2[i] = 0.0f;
        if (open) {
            const float bw = T * ca[i];
            const float4 col = prim[(size_t)ci[i] * (HTGS_PRIM_FLOATS_TRAIN / 4) + 4];
            k0[i] = col.x; k1[i] = col.y; k2[i] = col.z;
            r = __builtin_fmaf(bw, col.x, r);
            g = __builtin_fmaf(bw, col.y, g);
            b = __builtin_fmaf(bw, col.z, b);
            T *= 1.0f - ca[i];
        }
    }
    float n0 = 0.0f, n1 = 0.0f, n2 = 0.0f;
    T = 1.0f;
#pragma unroll
    for (int i = 0; i < K; ++i) {
        const bool skip = ci[i] == 0xffffffffu || T < kTransmittanceThreshold;
        core_idx[(size_t)i * rnp + rp] = skip ? 0xffffffffu : ci[i];
        float4 info = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (!skip) {
            const float bw = T * ca[i];
            n0 = __builtin_fmaf(bw, k0[i], n0);
            n1 = __builtin_fmaf(bw, k1[i], n1);
            n2 = __builtin_fmaf(bw, k2[i], n2);
            const float oma = 1.0f - ca[i];
            const float omar = one_minus_alpha_rcp(oma);
            info.x = __builtin_fmaf(k0[i], T, -((r - n0) * omar));
            info.y = __builtin_fmaf(k1[i], T, -((g - n1) * omar));
            info.z = __builtin_fmaf(k2[i], T, -((b - n2) * omar));
            info.w = bw;
            T *= oma;
        }
        core_info[(size_t)i * rnp + rp] = info;
    }
    image[pix] = r; image[np + pix] = g; image[2 * np + pix] = b;
}

__global__ void __launch_bounds__(64) blend_oit_forward_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
    float *__restrict__ image, float *__restrict__ tail_info, uint32_t width, uint32_t height, uint32_t grid_w, const uint32_t *__restrict__ tile_order)
{
    constexpr int MODE = HTGS_MODE_OIT_BLEND;
    __shared__ TileStageQ st;
    __shared__ QuadrantLists ql;
    const uint32_t tile = block_tile(tile_order);
    const uint32_t lane = threadIdx.x;
    const TilePixel px = quadrant_tile_pixel(tile, grid_w, lane, width, height);
    const uint32_t x = px.x, y = px.y;
    const bool inside = px.inside;
    const PixelTerms pt = px.pt;
    const float cx = px.cx, cy = px.cy;
    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, alpha_sum = 0.0f, T = 1.0f;

    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    tile_list_walk<MODE, false, kCullAlpha, true, HTGS_PRIM_FLOATS_TRAIN / 4>(st, ql, prim, inst, first, last, lane, cx, cy, [&](uint32_t addr) {
        TileFrag f;
        const bool in_reach = tile_frag_cutoff<kStageSlots>(addr, pt, f);
        f.den_rcp = rcp_exact(f.den);
        const float4 col = stage_row<kStageSlots, 5>(addr);
        if (!(tile_frag_alpha<MODE>(stage_opacity<kStageSlots>(addr), f) && in_reach)) return;
        a0 = __builtin_fmaf(f.alpha, col.x, a0);
        a1 = __builtin_fmaf(f.alpha, col.y, a1);
        a2 = __builtin_fmaf(f.alpha, col.z, a2);
        alpha_sum += f.alpha;
        T *= 1.0f - f.alpha;
    });
    if (!inside) return;
    const size_t pix = (size_t)width * y + x, np = (size_t)width * height;
    const size_t rp = record_pixel(tile, x, y), rnp = record_plane();
    float r = 0.0f, g = 0.0f, b = 0.0f, t0 = 0.0f, t1 = 0.0f, t2 = 0.0f, t3 = 0.0f, t4 = 0.0f, t5 = 0.0f;
    if (alpha_sum >= ModeCfg<MODE>::min_alpha) {
        const float asr = 1.0f / alpha_sum;
        const float s = (1.0f - T) * asr;
        r = s * a0; g = s * a1; b = s * a2;
        t0 = a0; t1 = a1; t2 = a2; t3 = asr; t4 = T; t5 = 1.0f;   // row 5 plays the hybrid mode's T_core
    }
    tail_info[rp] = t0; tail_info[rnp + rp] = t1; tail_info[2 * rnp + rp] = t2;
    tail_info[3 * rnp + rp] = t3; tail_info[4 * rnp + rp] = t4; tail_info[5 * rnp + rp] = t5;
    image[pix] = r; image[np + pix] = g; image[2 * np + pix] = b;
}

__global__ void __launch_bounds__(256) blend_global_forward_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim,
    float *__restrict__ image, uint32_t width, uint32_t height, uint32_t grid_w, const uint32_t *__restrict__ tile_order)
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
    float r = 0.0f, g = 0.0f, b = 0.0f, T = 1.0f;
    bool done = !inside;

    const uint32_t first = ranges[2 * tile], last = ranges[2 * tile + 1];
    for (uint32_t base = first; base < last; base += 256) {
        if (__syncthreads_count(done) == 256) break;
        s_reach[t] = (uint16_t)tile_stage_load<MODE, 256, false, kCullAlpha, true, HTGS_PRIM_FLOATS_TRAIN / 4>(st, prim, inst, base + t, last, t, cx, cy);
        __syncthreads();
        const uint32_t stage_base = __builtin_amdgcn_readfirstlane(stage_address(st));
        subtile_walk(s_reach, stage_base, last - base < 256u ? last - base : 256u, wave, lane,
                     [&]() { return __ballot(!done) == 0; },
                     [&](uint32_t addr) {
            TileFrag f;
            if (done || !tile_frag_cutoff<256>(addr, pt, f)) return;
            f.den_rcp = rcp_exact(f.den);
            const float4 col = stage_row<256, 5>(addr);
            if (!tile_frag_alpha<MODE>(stage_opacity<256>(addr), f)) return;
            const float bw = T * f.alpha;
            r = __builtin_fmaf(bw, col.x, r);
            g = __builtin_fmaf(bw, col.y, g);
            b = __builtin_fmaf(bw, col.z, b);
            T *= 1.0f - f.alpha;
            if (T < kTransmittanceThreshold) done = true;
        });
    }
    if (!inside) return;
    const size_t pix = (size_t)width * y + x, np = (size_t)width * height;
    image[pix] = r; image[np + pix] = g; image[2 * np + pix] = b;
}

template <int K>
static void launch_hybrid_forward(const htgs_frame *f, int sel, uint32_t grid_w, uint32_t n_tiles)
{
    hipLaunchKernelGGL((blend_hybrid_forward_kernel<K>), dim3(n_tiles), dim3(64), 0, (hipStream_t)f->stream, f->ranges, f->vals[sel],
                       (const float4 *)f->prim, f->image, f->core_idx, (float4 *)f->core_info, f->tail_info,
                       (uint32_t)f->width, (uint32_t)f->height, grid_w, f->tile_order);
}
template <int K>
static void launch_first_k_forward(const htgs_frame *f, int sel, uint32_t grid_w, uint32_t n_tiles)
{
    hipLaunchKernelGGL((blend_first_k_forward_kernel<K>), dim3(n_tiles), dim3(64), 0, (hipStream_t)f->stream, f->ranges, f->vals[sel],
                       (const float4 *)f->prim, f->image, f->core_idx, (float4 *)f->core_info,
                       (uint32_t)f->width, (uint32_t)f->height, grid_w, f->tile_order);
}

}  // namespace htgs

using namespace htgs;

extern "C" int htgs_blend_forward(const htgs_frame *f, int selector)
{
    if (!f) return fail(HTGS_ERR_ARGUMENT, "htgs_blend_forward: null frame");
    if (f->mode < 0 || f->mode > 3) return fail(HTGS_ERR_MODE, "unsupported rasterizer mode");
    if (selector < 0 || selector > 1 || f->width <= 0 || f->height <= 0) return fail(HTGS_ERR_ARGUMENT, "htgs_blend_forward: bad argument");
    if (frame_depth_ordered(f)) return fail(HTGS_ERR_ARGUMENT, "htgs_blend_forward: depth_order is for the inference entry points");
    if (f->prim_floats != HTGS_PRIM_FLOATS_TRAIN) return fail(HTGS_ERR_ARGUMENT, "htgs_blend_forward: the training kernels read records of HTGS_PRIM_FLOATS_TRAIN floats (prim_floats)");
    const bool needs_core = f->mode == HTGS_MODE_HYBRID_BLEND || f->mode == HTGS_MODE_ALPHA_BLEND_FIRST_K;
    const bool needs_tail = f->mode == HTGS_MODE_HYBRID_BLEND || f->mode == HTGS_MODE_OIT_BLEND;
    if (!f->ranges || !f->image || (f->n_instances > 0 && (!f->vals[selector] || !f->prim)) ||
        (needs_core && (!f->core_idx || !f->core_info)) || (needs_tail && !f->tail_info))
        return fail(HTGS_ERR_ARGUMENT, "htgs_blend_forward: null pointer");
    const int tile = tile_size(f->mode);
    const uint32_t grid_w = div_up(f->width, tile), grid_h = div_up(f->height, tile);
    const uint32_t n_tiles = grid_w * grid_h;
    hipStream_t s = (hipStream_t)f->stream;
    const int K = htgs_effective_k(f->K);
    switch (f->mode) {
        case HTGS_MODE_HYBRID_BLEND:
            switch (K) {
                case 32: launch_hybrid_forward<32>(f, selector, grid_w, n_tiles); break;
                case 16: launch_hybrid_forward<16>(f, selector, grid_w, n_tiles); break;
                case 8: launch_hybrid_forward<8>(f, selector, grid_w, n_tiles); break;
                case 4: launch_hybrid_forward<4>(f, selector, grid_w, n_tiles); break;
                case 2: launch_hybrid_forward<2>(f, selector, grid_w, n_tiles); break;
                default: launch_hybrid_forward<1>(f, selector, grid_w, n_tiles); break;
            }
            break;
        case HTGS_MODE_ALPHA_BLEND_FIRST_K:
            switch (K) {
                case 32: launch_first_k_forward<32>(f, selector, grid_w, n_tiles); break;
                case 16: launch_first_k_forward<16>(f, selector, grid_w, n_tiles); break;
                case 8: launch_first_k_forward<8>(f, selector, grid_w, n_tiles); break;
                case 4: launch_first_k_forward<4>(f, selector, grid_w, n_tiles); break;
                case 2: launch_first_k_forward<2>(f, selector, grid_w, n_tiles); break;
                default: launch_first_k_forward<1>(f, selector, grid_w, n_tiles); break;
            }
            break;
        case HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING:
            hipLaunchKernelGGL(blend_global_forward_kernel, dim3(n_tiles), dim3(256), 0, s, f->ranges, f->vals[selector],
                               (const float4 *)f->prim, f->image, (uint32_t)f->width, (uint32_t)f->height, grid_w, f->tile_order);
            break;
        default:
            hipLaunchKernelGGL(blend_oit_forward_kernel, dim3(n_tiles), dim3(64), 0, s, f->ranges, f->vals[selector],
                               (const float4 *)f->prim, f->image, f->tail_info, (uint32_t)f->width, (uint32_t)f->height, grid_w, f->tile_order);
            break;
    }
    return check_launch("blend_forward");
}
