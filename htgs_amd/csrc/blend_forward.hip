// Training forward blend of the four modes: unclamped [3,H,W] image plus the per-pixel records that the
// backward pass needs.  Restates blend_cu of R/include/hybrid_blend/kernels/forward.cuh:78-235,
// R/include/alpha_blend_first_k/kernels/forward.cuh:78-215,
// R/include/alpha_blend_global_ordering/kernels/forward.cuh:78-156 and
// R/include/oit_blend/kernels/forward.cuh:76-165.
//
// Records are pixel-minor ([slot][pixel]) so that a wave writes 64 consecutive words.  Where the reference
// leaves a record unwritten (tail with an alpha sum below 1/255, skipped core slots) zeros are stored, so that
// backward never reads indeterminate memory.
#include "blend_long.h"

namespace htgs {

__device__ __forceinline__ float one_minus_alpha_rcp(float one_minus_alpha)
{
    return 1.0f / (one_minus_alpha > kOneMinusAlphaEps ? one_minus_alpha : kOneMinusAlphaEps);
}

// What the training pass does with a pixel's finished core and tail (HYBRID_BLEND): the unclamped colour and the records
// of R/include/hybrid_blend/kernels/forward.cuh:170-233.  Called once per pixel inside the image, by the kernel with one wave
// per tile and by the one for tiles with very long lists.  records: entries per record plane (64 per tile of the frame).
struct HybridRecords {
    float *image;
    uint32_t *core_idx;
    float4 *core_info;
    float *tail_info;
    uint32_t width, height;
    size_t records;
    template <int K>
    __device__ __forceinline__ void operator()(const float4 *__restrict__ prim, uint32_t tile, const TilePixel &px, float (&cd)[K], float (&c3)[K], float (&ci)[K],
                                               HybridTail &tail) const
    {
        constexpr int MODE = HTGS_MODE_HYBRID_BLEND;
        const uint32_t x = px.x, y = px.y;
        float tail0 = tail.c0, tail1 = tail.c1, tail2 = tail.c2;
        const float tail3 = tail.alpha, T_tail = tail.T;
        const size_t pix = (size_t)width * y + x, np = (size_t)width * height;
        const size_t rp = record_pixel(tile, x, y), rnp = records;
        float c0[K], c1[K], c2[K];
#pragma unroll
        for (int i = 0; i < K; ++i) {
            float4 c = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (c3[i] > 0.0f) c = prim[(size_t)float_to_bits(ci[i]) * (HTGS_PRIM_FLOATS_TRAIN / 4) + 4];
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
            const bool skip = !(c3[i] > 0.0f) || T_core < kTransmittanceThreshold;      // an empty slot has alpha 0
            __builtin_nontemporal_store(skip ? 0xffffffffu : float_to_bits(ci[i]), core_idx + ((size_t)i * rnp + rp));
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
            // (0.7 GB of records per frame at 1080p, read back once by the backward pass: streaming stores)
            typedef float streamed_float4 __attribute__((ext_vector_type(4)));
            streamed_float4 packed; packed.x = info.x; packed.y = info.y; packed.z = info.z; packed.w = info.w;
            __builtin_nontemporal_store(packed, reinterpret_cast<streamed_float4 *>(core_info + ((size_t)i * rnp + rp)));
        }
        image[pix] = r + w0; image[np + pix] = g + w1; image[2 * np + pix] = b + w2;
    }
};

// One wave per tile: the walk of the inference kernel (slots hold depth, alpha and index; colours are fetched at the end and
// the core's share of the colour sums is taken out there), exact arithmetic, 128-byte records.  A tile whose list is
// longer than long_threshold is left to blend_hybrid_long_kernel if the caller provided the list for such tiles.
template <int K>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(K <= 16 ? 5 : 3))) blend_hybrid_forward_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, uint32_t width, uint32_t height, uint32_t grid_w,
    uint32_t *__restrict__ long_tiles, uint32_t long_threshold, uint32_t part_floor, const uint32_t *__restrict__ tile_order, const HybridRecords finish)
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
    HybridTail tail;
    hybrid_tail_init(tail);
    float cd[K], ca[K], ci[K];                 // ci: the index's bit pattern
    hybrid_core_init<K>(cd, ca, ci);
    hybrid_walk<K, false, true, false, false, HTGS_PRIM_FLOATS_TRAIN / 4>(st, ql, inst, prim, first, last, lane, px.pt, px.cx, px.cy, cd, ca, ci, tail);
    if (!px.inside) return;
    finish(prim, tile, px, cd, ca, ci, tail);
}

// ALPHA_BLEND_FIRST_K: R/include/alpha_blend_first_k/kernels/forward.cuh:160-213
struct FirstKRecords {
    float *image;
    uint32_t *core_idx;
    float4 *core_info;
    uint32_t width, height;
    size_t records;
    template <int K>
    __device__ __forceinline__ void operator()(const float4 *__restrict__ prim, uint32_t tile, const TilePixel &px, const float (&cd)[K], const float (&ca)[K],
                                               const uint32_t (&ci)[K]) const
    {
        const uint32_t x = px.x, y = px.y;
        const size_t pix = (size_t)width * y + x, np = (size_t)width * height;
        const size_t rp = record_pixel(tile, x, y), rnp = records;
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
            __builtin_nontemporal_store(skip ? 0xffffffffu : ci[i], core_idx + ((size_t)i * rnp + rp));     // (streaming, as in HybridRecords)
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
            typedef float streamed_float4 __attribute__((ext_vector_type(4)));
            streamed_float4 packed; packed.x = info.x; packed.y = info.y; packed.z = info.z; packed.w = info.w;
            __builtin_nontemporal_store(packed, reinterpret_cast<streamed_float4 *>(core_info + ((size_t)i * rnp + rp)));
        }
        image[pix] = r; image[np + pix] = g; image[2 * np + pix] = b;
    }
};

template <int K>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(K <= 16 ? 5 : 2))) blend_first_k_forward_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, uint32_t width, uint32_t height, uint32_t grid_w,
    uint32_t *__restrict__ long_tiles, uint32_t long_threshold, uint32_t part_floor, const uint32_t *__restrict__ tile_order, const FirstKRecords finish)
{
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
    first_k_core_init<K>(cd, ca, ci);
    first_k_walk<K, false, true, false, HTGS_PRIM_FLOATS_TRAIN / 4>(st, ql, inst, prim, first, last, lane, px.pt, px.cx, px.cy, cd, ca, ci);
    if (!px.inside) return;
    finish(prim, tile, px, cd, ca, ci);
}

// OIT_BLEND: R/include/oit_blend/kernels/forward.cuh:140-163
struct OitRecords {
    float *image, *tail_info;
    uint32_t width, height;
    size_t records;
    __device__ __forceinline__ void operator()(uint32_t tile, const TilePixel &px, const OitSums &sum) const
    {
        constexpr int MODE = HTGS_MODE_OIT_BLEND;
        const uint32_t x = px.x, y = px.y;
        const size_t pix = (size_t)width * y + x, np = (size_t)width * height;
        const size_t rp = record_pixel(tile, x, y), rnp = records;
        float r = 0.0f, g = 0.0f, b = 0.0f, t0 = 0.0f, t1 = 0.0f, t2 = 0.0f, t3 = 0.0f, t4 = 0.0f, t5 = 0.0f;
        if (sum.alpha >= ModeCfg<MODE>::min_alpha) {
            const float asr = 1.0f / sum.alpha;
            const float s = (1.0f - sum.T) * asr;
            r = s * sum.a0; g = s * sum.a1; b = s * sum.a2;
            t0 = sum.a0; t1 = sum.a1; t2 = sum.a2; t3 = asr; t4 = sum.T; t5 = 1.0f;   // row 5 plays the hybrid mode's T_core
        }
        tail_info[rp] = t0; tail_info[rnp + rp] = t1; tail_info[2 * rnp + rp] = t2;
        tail_info[3 * rnp + rp] = t3; tail_info[4 * rnp + rp] = t4; tail_info[5 * rnp + rp] = t5;
        image[pix] = r; image[np + pix] = g; image[2 * np + pix] = b;
    }
};

__global__ void __launch_bounds__(64) blend_oit_forward_kernel(
    const uint32_t *__restrict__ ranges, const uint32_t *__restrict__ inst, const float4 *__restrict__ prim, uint32_t width, uint32_t height, uint32_t grid_w,
    uint32_t *__restrict__ long_tiles, uint32_t long_threshold, uint32_t part_floor, const uint32_t *__restrict__ tile_order, const OitRecords finish)
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
    oit_walk<false, true, HTGS_PRIM_FLOATS_TRAIN / 4, false>(st, ql, inst, prim, first, last, lane, px.pt, px.cx, px.cy, sum);
    if (!px.inside) return;
    finish(tile, px, sum);
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

// the least length of a part of a long list (0: lists are not split, there is no spare value buffer to leave the parts' results in)
static uint32_t forward_part_floor(const htgs_frame *f, int sel, uint32_t n_tiles)
{
    if (f->vals[sel ^ 1] == nullptr) return 0u;
    const uint64_t floor = (f->n_instances + n_tiles - 1) / n_tiles;
    return floor < 1u ? 1u : (uint32_t)floor;
}
static uint32_t forward_threshold(const htgs_frame *f) { return f->long_list_threshold > 0 ? (uint32_t)f->long_list_threshold : kLongListDefault; }

template <int K>
static void launch_hybrid_forward(const htgs_frame *f, int sel, uint32_t grid_w, uint32_t n_tiles)
{
    constexpr int REC4 = HTGS_PRIM_FLOATS_TRAIN / 4;
    const HybridRecords finish = { f->image, f->core_idx, (float4 *)f->core_info, f->tail_info, (uint32_t)f->width, (uint32_t)f->height, (size_t)n_tiles * 64u };
    hipLaunchKernelGGL((blend_hybrid_forward_kernel<K>), dim3(n_tiles), dim3(64), 0, (hipStream_t)f->stream, f->ranges, f->vals[sel], (const float4 *)f->prim,
                       (uint32_t)f->width, (uint32_t)f->height, grid_w, f->long_tiles, forward_threshold(f), forward_part_floor(f, sel, n_tiles), f->tile_order, finish);
    if (f->long_tiles)
        hipLaunchKernelGGL((blend_hybrid_long_kernel<K, false, REC4, HybridRecords>), dim3(256 * kLongWaves / long_waves<K>()), dim3(64 * long_waves<K>()), 0,
                           (hipStream_t)f->stream, f->ranges, f->vals[sel], (const float4 *)f->prim, f->long_tiles, (uint32_t)f->width, (uint32_t)f->height, grid_w,
                           f->vals[sel ^ 1], forward_threshold(f), finish);
}
template <int K>
static void launch_first_k_forward(const htgs_frame *f, int sel, uint32_t grid_w, uint32_t n_tiles)
{
    constexpr int REC4 = HTGS_PRIM_FLOATS_TRAIN / 4;
    const FirstKRecords finish = { f->image, f->core_idx, (float4 *)f->core_info, (uint32_t)f->width, (uint32_t)f->height, (size_t)n_tiles * 64u };
    hipLaunchKernelGGL((blend_first_k_forward_kernel<K>), dim3(n_tiles), dim3(64), 0, (hipStream_t)f->stream, f->ranges, f->vals[sel], (const float4 *)f->prim,
                       (uint32_t)f->width, (uint32_t)f->height, grid_w, f->long_tiles, forward_threshold(f), forward_part_floor(f, sel, n_tiles), f->tile_order, finish);
    if (f->long_tiles)
        hipLaunchKernelGGL((blend_first_k_long_kernel<K, false, REC4, FirstKRecords>), dim3(256 * kLongWaves / long_waves<K>()), dim3(64 * long_waves<K>()), 0,
                           (hipStream_t)f->stream, f->ranges, f->vals[sel], (const float4 *)f->prim, f->long_tiles, (uint32_t)f->width, (uint32_t)f->height, grid_w,
                           f->vals[sel ^ 1], forward_threshold(f), finish);
}
static void launch_oit_forward(const htgs_frame *f, int sel, uint32_t grid_w, uint32_t n_tiles)
{
    constexpr int REC4 = HTGS_PRIM_FLOATS_TRAIN / 4;
    const OitRecords finish = { f->image, f->tail_info, (uint32_t)f->width, (uint32_t)f->height, (size_t)n_tiles * 64u };
    hipLaunchKernelGGL(blend_oit_forward_kernel, dim3(n_tiles), dim3(64), 0, (hipStream_t)f->stream, f->ranges, f->vals[sel], (const float4 *)f->prim,
                       (uint32_t)f->width, (uint32_t)f->height, grid_w, f->long_tiles, forward_threshold(f), forward_part_floor(f, sel, n_tiles), f->tile_order, finish);
    if (f->long_tiles)
        hipLaunchKernelGGL((blend_oit_long_kernel<false, REC4, OitRecords, false>), dim3(256), dim3(64 * kLongWaves), 0, (hipStream_t)f->stream, f->ranges, f->vals[sel],
                           (const float4 *)f->prim, f->long_tiles, (uint32_t)f->width, (uint32_t)f->height, grid_w, f->vals[sel ^ 1], forward_threshold(f), finish);
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
            launch_oit_forward(f, selector, grid_w, n_tiles);
            break;
    }
    return check_launch("blend_forward");
}
