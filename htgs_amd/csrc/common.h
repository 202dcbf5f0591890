// Shared host/device declarations of the gfx950 rasterizer.
//
// Rounding convention.  The whole library is compiled with -ffp-contract=off, so a fused
// multiply-add exists exactly where __builtin_fmaf is written.  The per-Gaussian stage uses none
// (operand order of the reference source, R/include/kernel_utils.cuh).  The per-pixel stage evaluates
// the reference's ray / Gaussian expressions in the tile-relative form (TileFrag, blend_common.h), in which |m|^2, |d|^2 and
// MT3.(d x m) are quadratics of the pixel offset from the tile centre.  log and 2^x are the
// polynomial routines below, sqrt and division are correctly rounded
// (-fhip-fp32-correctly-rounded-divide-sqrt; rcp_exact is the same quotient, cheaper).  The CPU
// checker used by the test-suite follows the same convention, which is what makes tile counts, sort
// order and every per-fragment accept/reject decision reproducible bit for bit.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/htgs_amd.h"

namespace htgs {

constexpr int kWave = 64;

// R/include/<mode>/config.h
constexpr float kTransmittanceThreshold = 1e-4f;
constexpr float kMaxFragmentAlpha = 1.0f;
constexpr float kOneMinusAlphaEps = 1e-8f;
constexpr float kMinAlphaCore = 1.0f / 20.0f;

template <int MODE> struct ModeCfg {
    static constexpr int tile = MODE == HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING ? 16 : 8;
    static constexpr float min_alpha_rcp = MODE == HTGS_MODE_ALPHA_BLEND_FIRST_K ? 20.0f : 255.0f;
    static constexpr float min_alpha = 1.0f / min_alpha_rcp;
    static constexpr float cutoff_sq = MODE == HTGS_MODE_ALPHA_BLEND_FIRST_K ? 5.99146454711f : 11.0825270903f;
    // tile-relative form: |m|^2 is staged divided by the cut-off (2 ln 20 resp. 2 ln 255), so the cut-off test is
    // num > den and exp(-rho^2 / 2) = 2^(-log2(20 or 255) num / den)
    static constexpr float cutoff_rcp = 1.0f / cutoff_sq;
    static constexpr float exp2_scale = MODE == HTGS_MODE_ALPHA_BLEND_FIRST_K ? -4.32192809488736235f : -7.99435343685885794f;
};

inline int tile_size(int mode) { return mode == HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING ? 16 : 8; }
inline int div_up(int a, int b) { return (a + b - 1) / b; }
// floats per record of f->prim; -1 for a value that no entry point takes
inline int frame_prim_floats(const htgs_frame *f)
{
    return f->prim_floats == 0 || f->prim_floats == HTGS_PRIM_FLOATS ? HTGS_PRIM_FLOATS : f->prim_floats == HTGS_PRIM_FLOATS_TRAIN ? HTGS_PRIM_FLOATS_TRAIN : -1;
}

// The Gaussians are sorted by depth before the instances are made (htgs_frame.depth_order): ALPHA_BLEND_GLOBAL_ORDERING,
// whose lists must be in depth order, and the image-only fast path of the two modes with a sorted core, whose lists may
// be in any order and whose insertions become rare when the fragments arrive roughly front to back (coarse keys, one pass)
inline bool frame_coarse_depth_ordered(const htgs_frame *f)
{
    return f->depth_order != nullptr && f->fast_math && (f->mode == HTGS_MODE_HYBRID_BLEND || f->mode == HTGS_MODE_ALPHA_BLEND_FIRST_K);
}
inline bool frame_depth_ordered(const htgs_frame *f)
{
    return (f->mode == HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING && f->depth_order != nullptr) || frame_coarse_depth_ordered(f);
}
// the parts of depth_order, n4 = N rounded up to a multiple of four words each: depth keys and Gaussian indices (two
// buffers each for the sort, which leaves its result in the first ones after four passes; htgs_preprocess writes the
// pairs), the counts and the tile rectangles in depth order, scratch of the sort
struct DepthOrder {
    uint32_t *keys[2], *vals[2], *counts;
    uint16_t *bounds;
    uint32_t *sort_tmp;
};
inline DepthOrder depth_order_parts(const htgs_frame *f)
{
    const size_t n4 = ((size_t)(f->n_primitives > 0 ? f->n_primitives : 0) + 3) & ~(size_t)3;
    DepthOrder d;
    d.keys[0] = f->depth_order; d.keys[1] = f->depth_order + n4;
    d.vals[0] = f->depth_order + 2 * n4; d.vals[1] = f->depth_order + 3 * n4;
    d.counts = f->depth_order + 4 * n4; d.bounds = reinterpret_cast<uint16_t *>(f->depth_order + 5 * n4); d.sort_tmp = f->depth_order + 7 * n4;
    return d;
}
// The keys that sort the Gaussians by depth: the bit pattern of the centre's camera-space depth (for positive depths the
// patterns order like the depths; these are the low 32 bits of the reference's tile | depth keys) less that of the near
// plane, which no Gaussian that is not culled lies in front of, `culled` for a culled Gaussian (behind all others).  With
// the far plane as the upper bound the keys of the usual cameras have 27 bits: three passes of 9-bit digits.
// Coarse keys (frame_coarse_depth_ordered): the same keys shifted down until eight bits are left, one pass.
struct DepthKeys {
    uint32_t base, culled;
    int end_bit, digit_bits, passes, shift;
};
constexpr int kCoarseDepthBits = 8;
inline DepthKeys depth_key_range(const htgs_frame *f)
{
    DepthKeys k = { 0u, 0xffffffffu, 32, 8, 4, 0 };
    const float near_plane = f->near_plane, far_plane = f->far_plane;
    if (near_plane > 0.0f && far_plane >= near_plane && far_plane < __builtin_huge_valf()) {
        uint32_t lo, hi;
        __builtin_memcpy(&lo, &near_plane, 4);
        __builtin_memcpy(&hi, &far_plane, 4);
        k.base = lo;
        k.culled = hi - lo + 1u;
        k.end_bit = 1;
        while (k.end_bit < 32 && (k.culled >> k.end_bit) != 0u) ++k.end_bit;
        const int passes8 = (k.end_bit + 7) / 8, passes9 = (k.end_bit + 8) / 9;
        k.digit_bits = passes9 < passes8 ? 9 : 8;
        k.passes = passes9 < passes8 ? passes9 : passes8;
    }
    if (frame_coarse_depth_ordered(f)) {
        // (culled, the largest key, must fit the bits that are left)
        while (k.end_bit - k.shift > kCoarseDepthBits || ((k.culled - 1u) >> k.shift) + 1u >= (1u << kCoarseDepthBits)) ++k.shift;
        k.culled = ((k.culled - 1u) >> k.shift) + 1u;
        k.end_bit = kCoarseDepthBits; k.digit_bits = kCoarseDepthBits; k.passes = 1;
    }
    return k;
}
// stable sort of n (32-bit key, value) pairs by the low end_bit key bits, digit_bits (8 or 9) a pass (radix_sort.hip);
// the result is in keys / vals[*selector]
int sort_u32_pairs(void *stream, uint32_t *const keys[2], uint32_t *const vals[2], uint32_t *sort_tmp, uint64_t n, int end_bit, int digit_bits,
                   int *selector);
// the same in one pass over keys of at most eight bits whose values are 0 .. n - 1 in this order, from keys / vals[0] to
// keys / vals[1]; the tile rectangles (four 16-bit bounds per value) are written in sorted order as well, with the number
// of tiles each covers (0 for the key `culled`)
int sort_u32_pairs_with_rectangles(void *stream, uint32_t *const keys[2], uint32_t *const vals[2], uint32_t *sort_tmp, uint64_t n, int bits,
                                   const uint16_t *rectangles_in, uint16_t *rectangles_out, uint32_t *counts_out, uint32_t culled);

// host side error reporting (api.hip)
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t float_to_bits(float f) { return __float_as_uint(f); }

// ln x: x = m 2^e, m in [sqrt(1/2), sqrt(2)), s = (m-1)/(m+1), ln m = 2 s (1 + s^2/3 + ... + s^10/11)
__device__ __forceinline__ float d_logf(float x)
{
    if (x != x || x < 0.0f) return __builtin_nanf("");
    if (x == 0.0f) return -__builtin_huge_valf();
    if (x == __builtin_huge_valf()) return x;
    int e = 0;
    if (x < 1.17549435e-38f) { x = x * 8388608.0f; e = -23; }
    uint32_t ix = float_to_bits(x);
    e += (int)(ix >> 23) - 127;
    ix = (ix & 0x007fffffu) | 0x3f800000u;
    float m = bits_to_float(ix);
    if (m > 1.41421356237f) { m = m * 0.5f; e += 1; }
    const float s = (m - 1.0f) / (m + 1.0f);
    const float z = s * s;
    float p = 0.0909090909f;
    p = p * z + 0.1111111111f;
    p = p * z + 0.1428571429f;
    p = p * z + 0.2f;
    p = p * z + 0.3333333333f;
    p = p * z;
    const float lnm = 2.0f * (s + s * p);
    const float fe = (float)e;
    return fe * 0.693359375f + (lnm + fe * -2.12194440e-4f);
}

// 2^t for t in [-126, 1): n = rint(t), r = t - n, degree-5 polynomial of 2^r on [-1/2, 1/2] (relative error 2.7e-7).
// rint is taken by adding and subtracting 1.5 * 2^23 (exact for |t| < 2^22, ties to even like rint), which also leaves
// n in the low bits of the sum for the exponent: two full-rate additions instead of v_rndne_f32 and v_cvt_i32_f32.
__device__ __forceinline__ float d_exp2(float t)
{
    const float shifted = t + 12582912.0f;
    const float n = shifted - 12582912.0f;
    const float r = t - n;
    float p = 1.3381302124e-3f;
    p = __builtin_fmaf(p, r, 9.6663683653e-3f);
    p = __builtin_fmaf(p, r, 5.5503811687e-2f);
    p = __builtin_fmaf(p, r, 2.4022349715e-1f);
    p = __builtin_fmaf(p, r, 6.9314718246e-1f);
    p = __builtin_fmaf(p, r, 1.0f);
    return bits_to_float(float_to_bits(p) + (float_to_bits(shifted) << 23));
}

// 1 / x.  v_rcp_f32 followed by one fused Newton step is the correctly rounded quotient for every x with
// 2^-120 <= x < 2^121 on gfx950 (htgs_check_reciprocal compares all of them with the division); a wave in
// which any active lane is outside that range takes the division.
__device__ __forceinline__ bool rcp_in_range(float x) { return float_to_bits(x) - 0x03800000u < 0x78800000u; }
__device__ __forceinline__ float rcp_refined(float x)
{
    const float x0 = __builtin_amdgcn_rcpf(x);
    const float e = __builtin_fmaf(-x, x0, 1.0f);
    return __builtin_fmaf(x0, e, x0);
}
__device__ __forceinline__ float rcp_exact(float x)
{
    // (the short form first and unconditionally, the division over it where a lane needs it: one branch around a side
    // block instead of two ways that meet again)
    float r = rcp_refined(x);
    if (__builtin_expect(__any(!rcp_in_range(x)), 0)) r = 1.0f / x;
    return r;
}

__device__ __forceinline__ float clamp_pos(float v) { return v > 0.0f ? v : 0.0f; }
__device__ __forceinline__ float saturate(float v) { return v > 0.0f ? (v < 1.0f ? v : 1.0f) : 0.0f; }

}  // namespace htgs
