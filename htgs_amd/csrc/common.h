// Shared host/device declarations of the gfx950 rasterizer.
//
// Rounding convention.  The whole library is compiled with -ffp-contract=off, so a fused
// multiply-add exists exactly where __builtin_fmaf is written.  The per-Gaussian stage uses none
// (operand order of the reference source, R/include/kernel_utils.cuh).  The per-pixel stage has two
// forms of the reference's ray / Gaussian evaluation: the plane form (frag_cutoff / frag_depth /
// frag_alpha), kept by the backward pass because it needs the intermediates, and the tile-relative
// form (TileFrag, blend_common.h) used by every forward-direction kernel, in which |m|^2, |d|^2 and
// MT3.(d x m) are quadratics of the pixel offset from the tile centre.  log, exp and 2^x are the
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

// e^x for x in [-87, 0]: n = rint(x log2 e), r = x - n ln 2, 1 + r + r^2 P(r), scaled through the exponent
__device__ __forceinline__ float d_expf(float x)
{
    const float t = x * 1.44269504088896341f;
    const float n = __builtin_rintf(t);
    float r = __builtin_fmaf(n, -0.693359375f, x);
    r = __builtin_fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    const float r2 = r * r;
    const float y = __builtin_fmaf(p, r2, r) + 1.0f;
    const int ni = (int)n;
    return bits_to_float((uint32_t)((int)float_to_bits(y) + ni * 8388608));
}

// 2^t for t in [-126, 1): n = rint(t), r = t - n, degree-5 polynomial of 2^r on [-1/2, 1/2] (relative error 2.7e-7)
__device__ __forceinline__ float d_exp2(float t)
{
    const float n = __builtin_rintf(t);
    const float r = t - n;
    float p = 1.3381302124e-3f;
    p = __builtin_fmaf(p, r, 9.6663683653e-3f);
    p = __builtin_fmaf(p, r, 5.5503811687e-2f);
    p = __builtin_fmaf(p, r, 2.4022349715e-1f);
    p = __builtin_fmaf(p, r, 6.9314718246e-1f);
    p = __builtin_fmaf(p, r, 1.0f);
    const int ni = (int)n;
    return bits_to_float((uint32_t)((int)float_to_bits(p) + ni * 8388608));
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
    if (__builtin_expect(__any(!rcp_in_range(x)), 0)) return 1.0f / x;
    return rcp_refined(x);
}

__device__ __forceinline__ float clamp_pos(float v) { return v > 0.0f ? v : 0.0f; }
__device__ __forceinline__ float saturate(float v) { return v > 0.0f ? (v < 1.0f ? v : 1.0f) : 0.0f; }

struct Frag {
    float G, alpha, depth;
    float num, den, den_rcp;
    float px[4], py[4], m[3], d[3];
};

// Ray / Gaussian evaluation of every blend kernel (R/include/hybrid_blend/kernels/inference.cuh:137-155):
// planes through the pixel in the Gaussian's local frame, distance of their intersection line from the
// origin, Gaussian weight at the point of maximum contribution.  The camera-space depth of that point is
// computed separately (frag_depth) because the modes need it at different places.
template <int MODE>
__device__ __forceinline__ bool frag_cutoff(const float4 &V1, const float4 &V2, const float4 &V4,
                                            float fx, float fy, Frag &o)
{
    o.px[0] = __builtin_fmaf(-V4.x, fx, V1.x); o.px[1] = __builtin_fmaf(-V4.y, fx, V1.y);
    o.px[2] = __builtin_fmaf(-V4.z, fx, V1.z); o.px[3] = __builtin_fmaf(-V4.w, fx, V1.w);
    o.py[0] = __builtin_fmaf(-V4.x, fy, V2.x); o.py[1] = __builtin_fmaf(-V4.y, fy, V2.y);
    o.py[2] = __builtin_fmaf(-V4.z, fy, V2.z); o.py[3] = __builtin_fmaf(-V4.w, fy, V2.w);
    const float *px = o.px, *py = o.py;
    o.m[0] = __builtin_fmaf(px[3], py[0], -(px[0] * py[3]));
    o.m[1] = __builtin_fmaf(px[3], py[1], -(px[1] * py[3]));
    o.m[2] = __builtin_fmaf(px[3], py[2], -(px[2] * py[3]));
    o.d[0] = __builtin_fmaf(px[1], py[2], -(px[2] * py[1]));
    o.d[1] = __builtin_fmaf(px[2], py[0], -(px[0] * py[2]));
    o.d[2] = __builtin_fmaf(px[0], py[1], -(px[1] * py[0]));
    o.num = __builtin_fmaf(o.m[2], o.m[2], __builtin_fmaf(o.m[1], o.m[1], o.m[0] * o.m[0]));
    o.den = __builtin_fmaf(o.d[2], o.d[2], __builtin_fmaf(o.d[1], o.d[1], o.d[0] * o.d[0]));
    return !(o.num > ModeCfg<MODE>::cutoff_sq * o.den);
}

__device__ __forceinline__ float frag_depth(const float4 &MT3, const Frag &o)
{
    const float *m = o.m, *d = o.d;
    const float e0 = __builtin_fmaf(d[1], m[2], -(d[2] * m[1])) * o.den_rcp;
    const float e1 = __builtin_fmaf(d[2], m[0], -(d[0] * m[2])) * o.den_rcp;
    const float e2 = __builtin_fmaf(d[0], m[1], -(d[1] * m[0])) * o.den_rcp;
    return __builtin_fmaf(MT3.z, e2, __builtin_fmaf(MT3.y, e1, MT3.x * e0)) + MT3.w;
}

// alpha of the fragment; false if below the mode's threshold.  Needs o.den_rcp.
template <int MODE>
__device__ __forceinline__ bool frag_alpha(float opacity, Frag &o)
{
    o.G = d_expf((-0.5f * o.num) * o.den_rcp);
    const float a = opacity * o.G;
    o.alpha = a < kMaxFragmentAlpha ? a : kMaxFragmentAlpha;
    return !(o.alpha < ModeCfg<MODE>::min_alpha);
}

}  // namespace htgs
