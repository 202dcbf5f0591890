// Pieces shared by the inference, training-forward, max-weight and backward blend kernels.
#pragma once

#include "common.h"

namespace htgs {

// ---------------------------------------------------------------------------------------------
// tile-relative form.  With px = px0 - dx VPMT4, py = py0 - dy VPMT4, where px0 / py0 are
// the reference's planes (R/include/hybrid_blend/kernels/inference.cuh:137-141) through the tile centre and
// (dx, dy) is the pixel's offset from it,
//     d = cross(px.n, py.n)     = A  + dy B  + dx C
//     m = px.w py.n - px.n py.w = Am + dy Bm + dx Cm            (the dx dy terms cancel)
// so |m|^2, |d|^2 and MT3.n . cross(d, m) are quadratics in (dx, dy).  The lane that stages an instance
// computes the 18 coefficients once; every pixel then needs 5 fused multiply-adds per quadratic.
// LDS layout per instance, coefficient order (1, dx, dy, dx^2, dx dy, dy^2):
//     q[0] = n0 nx ny nxx   q[1] = nxy nyy d0 dx   q[2] = dy dxx dxy dyy      (n = |m|^2 / cut-off)
//     q[3] = z0 zx zy zxx   q[4] = zxy zyy MT3.w opacity   q[5] = r g b (primitive index bits)
// ---------------------------------------------------------------------------------------------
template <int N>
struct TileStage {
    float4 q[6][N];
};

__device__ __forceinline__ void cross3(const float *a, const float *b, float *o)
{
    o[0] = __builtin_fmaf(a[1], b[2], -(a[2] * b[1]));
    o[1] = __builtin_fmaf(a[2], b[0], -(a[0] * b[2]));
    o[2] = __builtin_fmaf(a[0], b[1], -(a[1] * b[0]));
}
__device__ __forceinline__ float dotf(const float *a, const float *b)
{
    return __builtin_fmaf(a[2], b[2], __builtin_fmaf(a[1], b[1], a[0] * b[0]));
}

// the six vectors of the tile-relative form and what they are built from
struct TileGeometry {
    float a[3], aw, b[3], bw, v[3], vw;        // px0 = (a, aw), py0 = (b, bw), VPMT4 = (v, vw)
    float A[3], B[3], C[3], Am[3], Bm[3], Cm[3];
};
__device__ __forceinline__ void tile_geometry(const float4 &r1, const float4 &r2, const float4 &r4, float cx, float cy, TileGeometry &g)
{
    const float V1[4] = { r1.x, r1.y, r1.z, r1.w }, V2[4] = { r2.x, r2.y, r2.z, r2.w }, V4[4] = { r4.x, r4.y, r4.z, r4.w };
    float px0[4], py0[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        px0[k] = __builtin_fmaf(-V4[k], cx, V1[k]);
        py0[k] = __builtin_fmaf(-V4[k], cy, V2[k]);
    }
#pragma unroll
    for (int k = 0; k < 3; ++k) { g.a[k] = px0[k]; g.b[k] = py0[k]; g.v[k] = V4[k]; }
    g.aw = px0[3]; g.bw = py0[3]; g.vw = V4[3];
    cross3(px0, py0, g.A);
    cross3(V4, px0, g.B);
    cross3(py0, V4, g.C);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        g.Am[k] = __builtin_fmaf(px0[3], py0[k], -(px0[k] * py0[3]));
        g.Bm[k] = __builtin_fmaf(px0[k], V4[3], -(px0[3] * V4[k]));
        g.Cm[k] = __builtin_fmaf(V4[k], py0[3], -(V4[3] * py0[k]));
    }
}
// coefficients (1, dx, dy, dx^2, dx dy, dy^2) of |m|^2 / cut-off and of |d|^2
template <int MODE>
__device__ __forceinline__ void tile_quadratics(const TileGeometry &g, float (&n)[6], float (&d)[6])
{
    constexpr float kc = ModeCfg<MODE>::cutoff_rcp;
    n[0] = dotf(g.Am, g.Am) * kc; n[1] = (2.0f * dotf(g.Am, g.Cm)) * kc; n[2] = (2.0f * dotf(g.Am, g.Bm)) * kc;
    n[3] = dotf(g.Cm, g.Cm) * kc; n[4] = (2.0f * dotf(g.Bm, g.Cm)) * kc; n[5] = dotf(g.Bm, g.Bm) * kc;
    d[0] = dotf(g.A, g.A); d[1] = 2.0f * dotf(g.A, g.C); d[2] = 2.0f * dotf(g.A, g.B);
    d[3] = dotf(g.C, g.C); d[4] = 2.0f * dotf(g.B, g.C); d[5] = dotf(g.B, g.B);
}

// True when no pixel of the tile can pass both the cut-off and the alpha test of an instance, given the
// coefficients of |m|^2 / cut-off (n) and |d|^2 (d) and the opacity.  The cut-off is 2 ln(1 / min_alpha) in every
// mode, so opacity * exp(-rho^2 / 2) >= min_alpha is n / d <= 1 + log2(opacity) / log2(1 / min_alpha) =: r, and both
// tests together are  Q = n - min(r, 1) d <= 0.  Q is a quadratic of the pixel offset; per pixel row its least value
// over the row's pixels is at the pixel next to the vertex (or at a row end), so one evaluation per row gives the
// least Q over the tile.  The margin (1e-5 of the sum of the magnitudes of all terms, with r raised by 1e-5) is an
// order of magnitude above the rounding of the per-pixel evaluation, of 2^x and of this routine; non-finite
// coefficients never report a miss.
template <int MODE>
__device__ __forceinline__ bool tile_misses(const float (&n)[6], const float (&d)[6], float opacity)
{
    constexpr int rows = ModeCfg<MODE>::tile;
    constexpr float h = 0.5f * (float)(rows - 1);
    float r = __builtin_fmaf(__builtin_amdgcn_logf(opacity), -1.0f / ModeCfg<MODE>::exp2_scale, 1.0f);
    r = r < 1.0f ? r : 1.0f;                       // (also a NaN opacity: the cut-off alone decides)
    r = r > -1.0f ? r : -1.0f;
    r += 1e-5f;
    float q[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) q[i] = __builtin_fmaf(-r, d[i], n[i]);
    const float s0 = __builtin_fabsf(n[0]) + __builtin_fabsf(d[0]);
    const float s1 = (__builtin_fabsf(n[1]) + __builtin_fabsf(d[1])) + (__builtin_fabsf(n[2]) + __builtin_fabsf(d[2]));
    const float s2 = ((__builtin_fabsf(n[3]) + __builtin_fabsf(d[3])) + (__builtin_fabsf(n[4]) + __builtin_fabsf(d[4]))) +
                     (__builtin_fabsf(n[5]) + __builtin_fabsf(d[5]));
    const float margin = 1e-5f * __builtin_fmaf(h * h, s2, __builtin_fmaf(h, s1, s0));
    const bool convex = q[3] > 0.0f;
    const float to_vertex = -0.5f * __builtin_amdgcn_rcpf(q[3]);
    float least = __FLT_MAX__;
#pragma nounroll
    for (int row = 0; row < rows; ++row) {           // (kept a loop: unrolled, the rows crowd the callers' K-buffers out of registers)
        const float y = (float)row - h;
        const float b = __builtin_fmaf(q[4], y, q[1]);
        const float c = __builtin_fmaf(y, __builtin_fmaf(q[5], y, q[2]), q[0]);
        float xv = __builtin_rintf(__builtin_fmaf(b, to_vertex, 0.5f)) - 0.5f;
        xv = __builtin_fminf(__builtin_fmaxf(xv, -h), h);
        least = __builtin_fminf(least, __builtin_fmaf(xv, __builtin_fmaf(q[3], xv, b), c));
    }
    return convex && least > margin;                 // (a quadratic that is not convex along the rows is never left out)
}

// The same bound per 4x4 quadrant of the 8x8 tile: bit q = 2 (row >= 4) + (column >= 4) of the result is clear when no
// pixel of that quadrant can pass.  Per pixel row the least value of Q over a quadrant's four pixels is at the one
// nearest to the vertex, so two evaluations per row serve the row's two quadrants.
template <int MODE>
__device__ __forceinline__ uint32_t tile_quadrant_hits(const float (&n)[6], const float (&d)[6], float opacity)
{
    static_assert(ModeCfg<MODE>::tile == 8, "8x8 tiles");
    constexpr float h = 3.5f;
    float r = __builtin_fmaf(__builtin_amdgcn_logf(opacity), -1.0f / ModeCfg<MODE>::exp2_scale, 1.0f);
    r = r < 1.0f ? r : 1.0f;
    r = r > -1.0f ? r : -1.0f;
    r += 1e-5f;
    float q[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) q[i] = __builtin_fmaf(-r, d[i], n[i]);
    const float s0 = __builtin_fabsf(n[0]) + __builtin_fabsf(d[0]);
    const float s1 = (__builtin_fabsf(n[1]) + __builtin_fabsf(d[1])) + (__builtin_fabsf(n[2]) + __builtin_fabsf(d[2]));
    const float s2 = ((__builtin_fabsf(n[3]) + __builtin_fabsf(d[3])) + (__builtin_fabsf(n[4]) + __builtin_fabsf(d[4]))) +
                     (__builtin_fabsf(n[5]) + __builtin_fabsf(d[5]));
    const float margin = 1e-5f * __builtin_fmaf(h * h, s2, __builtin_fmaf(h, s1, s0));
    if (!(q[3] > 0.0f)) return 0xfu;                 // (not convex along the rows, or not a number: kept everywhere)
    const float to_vertex = -0.5f * __builtin_amdgcn_rcpf(q[3]);
    uint32_t bits = 0;
#pragma nounroll
    for (int half = 0; half < 2; ++half) {
        float least_l = __FLT_MAX__, least_r = __FLT_MAX__;
#pragma nounroll
        for (int row = 0; row < 4; ++row) {
            const float y = (float)(4 * half + row) - h;
            const float b = __builtin_fmaf(q[4], y, q[1]);
            const float c = __builtin_fmaf(y, __builtin_fmaf(q[5], y, q[2]), q[0]);
            const float xv = __builtin_rintf(__builtin_fmaf(b, to_vertex, 0.5f)) - 0.5f;
            const float xl = __builtin_fminf(__builtin_fmaxf(xv, -h), -0.5f), xr = __builtin_fminf(__builtin_fmaxf(xv, 0.5f), h);
            least_l = __builtin_fminf(least_l, __builtin_fmaf(xl, __builtin_fmaf(q[3], xl, b), c));
            least_r = __builtin_fminf(least_r, __builtin_fmaf(xr, __builtin_fmaf(q[3], xr, b), c));
        }
        bits |= (least_l > margin ? 0u : 1u << (2 * half)) | (least_r > margin ? 0u : 2u << (2 * half));
    }
    return bits;
}

// The 16x16 tile of ALPHA_BLEND_GLOBAL_ORDERING: sixteen 4x4 quadrants, four per 8x8 sub-tile.  Bit 4 s + q of the result
// stands for quadrant q (numbered as above) of sub-tile s = 2 (row >= 8) + (column >= 8).  Four evaluations per pixel
// row serve the row's four quadrants.
template <int MODE>
__device__ __forceinline__ uint32_t tile_quadrant_hits16(const float (&n)[6], const float (&d)[6], float opacity)
{
    static_assert(ModeCfg<MODE>::tile == 16, "16x16 tiles");
    constexpr float h = 7.5f;
    float r = __builtin_fmaf(__builtin_amdgcn_logf(opacity), -1.0f / ModeCfg<MODE>::exp2_scale, 1.0f);
    r = r < 1.0f ? r : 1.0f;
    r = r > -1.0f ? r : -1.0f;
    r += 1e-5f;
    float q[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) q[i] = __builtin_fmaf(-r, d[i], n[i]);
    const float s0 = __builtin_fabsf(n[0]) + __builtin_fabsf(d[0]);
    const float s1 = (__builtin_fabsf(n[1]) + __builtin_fabsf(d[1])) + (__builtin_fabsf(n[2]) + __builtin_fabsf(d[2]));
    const float s2 = ((__builtin_fabsf(n[3]) + __builtin_fabsf(d[3])) + (__builtin_fabsf(n[4]) + __builtin_fabsf(d[4]))) +
                     (__builtin_fabsf(n[5]) + __builtin_fabsf(d[5]));
    const float margin = 1e-5f * __builtin_fmaf(h * h, s2, __builtin_fmaf(h, s1, s0));
    if (!(q[3] > 0.0f)) return 0xffffu;              // (not convex along the rows, or not a number: kept everywhere)
    const float to_vertex = -0.5f * __builtin_amdgcn_rcpf(q[3]);
    uint32_t bits = 0;
#pragma nounroll
    for (int band = 0; band < 4; ++band) {           // four pixel rows: one row of quadrants
        float least[4] = { __FLT_MAX__, __FLT_MAX__, __FLT_MAX__, __FLT_MAX__ };
#pragma nounroll
        for (int row = 0; row < 4; ++row) {
            const float y = (float)(4 * band + row) - h;
            const float b = __builtin_fmaf(q[4], y, q[1]);
            const float c = __builtin_fmaf(y, __builtin_fmaf(q[5], y, q[2]), q[0]);
            const float xv = __builtin_rintf(__builtin_fmaf(b, to_vertex, 0.5f)) - 0.5f;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float lo = (float)(4 * k) - h;
                const float xc = __builtin_fminf(__builtin_fmaxf(xv, lo), lo + 3.0f);
                least[k] = __builtin_fminf(least[k], __builtin_fmaf(xc, __builtin_fmaf(q[3], xc, b), c));
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (!(least[k] > margin)) bits |= 1u << (4 * (2 * (band >> 1) + (k >> 1)) + 2 * (band & 1) + (k & 1));
    }
    return bits;
}

// Stages instance `fetch` of the sorted list in slot `slot` (the same arithmetic as tile_geometry / tile_quadratics,
// written out so that every row is stored as soon as it is complete: the kernels that call this hold a K-buffer in
// registers).  Returns whether the slot holds an instance that can reach a pixel of the tile: always true for a
// loaded slot unless CULL asks for tile_misses -- for walks that apply the cut-off and the alpha threshold
// (kCullAlpha), or the cut-off alone (kCullCutoff: the test with opacity 1).  What that leaves out contributes to
// no pixel, so a walk over the hits alone gives the results of the full walk bit for bit.
// the pixel's offset from the tile centre (exact)
struct PixelTerms {
    float X, Y;
};
__device__ __forceinline__ PixelTerms pixel_terms(uint32_t local_x, uint32_t local_y, int tile)
{
    PixelTerms p;
    p.X = (float)local_x - 0.5f * (float)(tile - 1);
    p.Y = (float)local_y - 0.5f * (float)(tile - 1);
    return p;
}
__device__ __forceinline__ float tile_centre(uint32_t first_pixel, int tile) { return (float)first_pixel + 0.5f * (float)(tile - 1); }

__device__ __forceinline__ float quad_eval(float c0, float cx, float cy, float cxx, float cxy, float cyy, const PixelTerms &p)
{
    const float tx = __builtin_fmaf(cxy, p.Y, __builtin_fmaf(cxx, p.X, cx));
    const float ty = __builtin_fmaf(cyy, p.Y, cy);
    return __builtin_fmaf(p.Y, ty, __builtin_fmaf(p.X, tx, c0));
}

// lane -> pixel of the quadrant walk (below): lanes 16 q .. 16 q + 15 hold the 4x4 pixels of quadrant q
__device__ __forceinline__ void quadrant_pixel(uint32_t lane, uint32_t &local_x, uint32_t &local_y)
{
    local_x = ((lane >> 4) & 1) * 4 + (lane & 3);
    local_y = (lane >> 5) * 4 + ((lane >> 2) & 3);
}

// the same for the banked layout (quadrant q = lanes 4 q .. 4 q + 3 of every row of sixteen lanes; the row is the pixel row)
__device__ __forceinline__ void banked_quadrant_pixel(uint32_t lane, uint32_t &local_x, uint32_t &local_y)
{
    const uint32_t q = (lane >> 2) & 3u;
    local_x = (q & 1u) * 4u + (lane & 3u);
    local_y = (q >> 1) * 4u + (lane >> 4);
}

// kCullPixels: a slot counts for a quadrant when the instance passes the cut-off -- with the walk's own arithmetic -- at
// one of the pixels named by pixel_lanes (a wave-uniform mask over the lanes of the quadrant walk) that lie in it.
enum { kCullNone = 0, kCullAlpha = 1, kCullCutoff = 2, kCullPixels = 3 };

// With QUADRANTS the result has one bit per 4x4 quadrant of the tile (tile_quadrant_hits) instead of one for the tile.
// REC4: 16-byte words per record of prim (five; eight in training frames).
// UNIT: the opacity is staged held to at most 1 (the image-only fast path, whose fragments then need no clamp of their own).
// POS: the last word of the slot holds the instance's place in the list (fetch) instead of the Gaussian's index.
// GIVEN: the caller has read inst[fetch] already (`given`).
template <int MODE, int N, bool DEPTH, int CULL = kCullNone, bool QUADRANTS = false, int REC4 = HTGS_PRIM_FLOATS / 4, bool UNIT = false, bool POS = false,
          bool GIVEN = false>
__device__ __forceinline__ uint32_t tile_stage_load(TileStage<N> &st, const float4 *__restrict__ prim, const uint32_t *__restrict__ inst,
                                                    uint32_t fetch, uint32_t last, int slot, float cx, float cy, uint64_t pixel_lanes = 0, uint32_t given = 0);

// (PixelTerms is complete by the time the template is instantiated)
template <int MODE, int N, bool DEPTH, int CULL, bool QUADRANTS, int REC4, bool UNIT, bool POS, bool GIVEN>
__device__ __forceinline__ uint32_t tile_stage_load(TileStage<N> &st, const float4 *__restrict__ prim, const uint32_t *__restrict__ inst,
                                                    uint32_t fetch, uint32_t last, int slot, float cx, float cy, uint64_t pixel_lanes, uint32_t given)
{
    if (fetch >= last) return 0;
    const uint32_t g = GIVEN ? given : inst[fetch];
    const float4 *rec = prim + (size_t)g * REC4;
    // (with CULL the record's colour row is fetched when it is needed, behind a compiler fence: it comes from a cache
    // line the other rows have just brought in, and four registers less at the peak keep the callers' K-buffers out
    // of scratch memory inside the batch loop)
    const float4 r1 = rec[0], r2 = rec[1], r4 = rec[2], r3 = rec[3];
    float4 col;
    if (CULL == kCullNone) col = rec[4];
    const float V1[4] = { r1.x, r1.y, r1.z, r1.w }, V2[4] = { r2.x, r2.y, r2.z, r2.w }, V4[4] = { r4.x, r4.y, r4.z, r4.w };
    float px0[4], py0[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        px0[k] = __builtin_fmaf(-V4[k], cx, V1[k]);
        py0[k] = __builtin_fmaf(-V4[k], cy, V2[k]);
    }
    float A[3], B[3], C[3], Am[3], Bm[3], Cm[3];
    cross3(px0, py0, A);
    cross3(V4, px0, B);
    cross3(py0, V4, C);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        Am[k] = __builtin_fmaf(px0[3], py0[k], -(px0[k] * py0[3]));
        Bm[k] = __builtin_fmaf(px0[k], V4[3], -(px0[3] * V4[k]));
        Cm[k] = __builtin_fmaf(V4[k], py0[3], -(V4[3] * py0[k]));
    }
    float zxy = 0.0f, zyy = 0.0f;
    if (DEPTH) {
        const float MT3[3] = { r3.x, r3.y, r3.z };
        float PA[3], PB[3], PC[3];
        cross3(MT3, A, PA);
        cross3(MT3, B, PB);
        cross3(MT3, C, PC);
        st.q[3][slot] = make_float4(dotf(PA, Am), dotf(PA, Cm) + dotf(PC, Am), dotf(PA, Bm) + dotf(PB, Am), dotf(PC, Cm));
        zxy = dotf(PB, Cm) + dotf(PC, Bm);
        zyy = dotf(PB, Bm);
    }
    constexpr float kc = ModeCfg<MODE>::cutoff_rcp;
    const float n[6] = { dotf(Am, Am) * kc, (2.0f * dotf(Am, Cm)) * kc, (2.0f * dotf(Am, Bm)) * kc,
                         dotf(Cm, Cm) * kc, (2.0f * dotf(Bm, Cm)) * kc, dotf(Bm, Bm) * kc };
    const float d[6] = { dotf(A, A), 2.0f * dotf(A, C), 2.0f * dotf(A, B), dotf(C, C), 2.0f * dotf(B, C), dotf(B, B) };
    st.q[0][slot] = make_float4(n[0], n[1], n[2], n[3]);
    st.q[1][slot] = make_float4(n[4], n[5], d[0], d[1]);
    st.q[2][slot] = make_float4(d[2], d[3], d[4], d[5]);
    if (CULL != kCullNone) {
        asm volatile("" ::: "memory");
        col = rec[4];
    }
    if (UNIT) col.w = col.w < 1.0f ? col.w : 1.0f;
    st.q[4][slot] = make_float4(zxy, zyy, r3.w, col.w);
    st.q[5][slot] = make_float4(col.x, col.y, col.z, bits_to_float(POS ? fetch : g));
    if constexpr (CULL == kCullNone) return QUADRANTS ? 0xfu : 1u;
    else if constexpr (CULL == kCullPixels) {
        static_assert(QUADRANTS, "per quadrant");
        uint32_t bits = 0;
        for (uint64_t m = pixel_lanes; m != 0; m &= m - 1) {      // (wave-uniform)
            const uint32_t p = (uint32_t)__builtin_ctzll(m);
            uint32_t local_x, local_y;
            quadrant_pixel(p, local_x, local_y);
            const PixelTerms pt = pixel_terms(local_x, local_y, 8);
            const float num = quad_eval(n[0], n[1], n[2], n[3], n[4], n[5], pt), den = quad_eval(d[0], d[1], d[2], d[3], d[4], d[5], pt);
            if (!(num > den)) bits |= 1u << (p >> 4);
        }
        return bits;
    }
    else if constexpr (QUADRANTS && ModeCfg<MODE>::tile == 16) return tile_quadrant_hits16<MODE>(n, d, CULL == kCullCutoff ? 1.0f : col.w);
    else if constexpr (QUADRANTS) return tile_quadrant_hits<MODE>(n, d, CULL == kCullCutoff ? 1.0f : col.w);
    else return (uint32_t)!tile_misses<MODE>(n, d, CULL == kCullCutoff ? 1.0f : col.w);
}

struct TileFrag {
    float num, den, den_rcp, alpha;
};

// The per-pixel loops address the staged instance through one VGPR that holds the LDS byte address of q[0][j] and
// is advanced by an opaque add (the compiler would otherwise rebuild the address from the scalar loop counter
// before every read).
struct __attribute__((aligned(16))) Float4Pod { float x, y, z, w; };
typedef __attribute__((address_space(3))) const Float4Pod lds_float4;
typedef __attribute__((address_space(3))) const float lds_float;
template <int N>
__device__ __forceinline__ uint32_t stage_address(const TileStage<N> &st) { return (uint32_t)(uintptr_t)(lds_float4 *)&st.q[0][0]; }
__device__ __forceinline__ void stage_advance(uint32_t &addr) { asm volatile("v_add_u32 %0, 16, %0" : "+v"(addr)); }
// Quadrant walk.  Lanes 16 q .. 16 q + 15 hold the 4x4 pixels of quadrant q of the tile and walk the hits of that
// quadrant, in list order, in lock step with the other three quadrants: a turn of the loop serves up to four instances,
// one per quadrant, and a batch takes as many turns as its busiest quadrant has hits (an instance reaches 1.9 of the four
// quadrants on average, so this is well under the number of instances that reach the tile).  Every pixel still sees its
// fragments in list order.  The four hit masks are wave-uniform (scalar registers).
constexpr uint32_t kNoHit = 0xfffffff0u;           // 16 * s_ff1(0): the address a quadrant without a hit left gets
struct QuadrantHits {
    uint64_t h[4];
};
__device__ __forceinline__ QuadrantHits quadrant_ballot(uint32_t bits)
{
    QuadrantHits w;
#pragma unroll
    for (int q = 0; q < 4; ++q) w.h[q] = __ballot((bits >> q) & 1);
    return w;
}
__device__ __forceinline__ bool quadrant_pending(const QuadrantHits &w) { return (w.h[0] | w.h[1] | w.h[2] | w.h[3]) != 0; }
// LDS address, relative to the stage, of the q[0] entry of the lane's quadrant's next hit, or kNoHit.  Per quadrant two
// scalar instructions: s_ff1 gives the slot (-1 for an empty mask, which the shift turns into kNoHit) and s_bitset0
// clears that bit (bit 63 of an empty mask).  A quadrant is one row of sixteen lanes to the data-parallel primitives, so
// its lanes take the slot by a move with that row's mask: no exec writes, and the scalar unit, which the four SIMDs of a
// compute unit share, is left to the loop's branches.
// BANKED: a quadrant is not a row of sixteen lanes but lanes 4 q .. 4 q + 3 of each of the four rows (bank q of the
// data-parallel primitives), which is the layout in which sums over a quadrant's lanes fold across the rows.
template <bool BANKED = false>
__device__ __forceinline__ uint32_t quadrant_next_hit(QuadrantHits &w)
{
    uint32_t a0, a1, a2, a3, addr, t;
    // (two statements: one with scalar results only, which the compiler then knows to be wave-uniform)
    asm volatile("s_ff1_i32_b64 %[a0], %[h0]\n\ts_ff1_i32_b64 %[a1], %[h1]\n\ts_ff1_i32_b64 %[a2], %[h2]\n\ts_ff1_i32_b64 %[a3], %[h3]\n\t"
                 "s_bitset0_b64 %[h0], %[a0]\n\ts_bitset0_b64 %[h1], %[a1]\n\ts_bitset0_b64 %[h2], %[a2]\n\ts_bitset0_b64 %[h3], %[a3]"
                 : [a0] "=&s"(a0), [a1] "=&s"(a1), [a2] "=&s"(a2), [a3] "=&s"(a3),
                   [h0] "+s"(w.h[0]), [h1] "+s"(w.h[1]), [h2] "+s"(w.h[2]), [h3] "+s"(w.h[3]));
    if constexpr (BANKED)
        asm volatile("v_mov_b32 %[addr], %[a0]\n\t"
                     "v_mov_b32 %[t], %[a1]\n\t"
                     "s_nop 1\n\t"
                     "v_mov_b32_dpp %[addr], %[t] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x2\n\t"
                     "v_mov_b32 %[t], %[a2]\n\t"
                     "s_nop 1\n\t"
                     "v_mov_b32_dpp %[addr], %[t] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x4\n\t"
                     "v_mov_b32 %[t], %[a3]\n\t"
                     "s_nop 1\n\t"
                     "v_mov_b32_dpp %[addr], %[t] quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x8\n\t"
                     "v_lshlrev_b32 %[addr], 4, %[addr]"
                     : [addr] "=&v"(addr), [t] "=&v"(t)
                     : [a0] "s"(a0), [a1] "s"(a1), [a2] "s"(a2), [a3] "s"(a3));
    else
        asm volatile("v_mov_b32 %[addr], %[a0]\n\t"
                     "v_mov_b32 %[t], %[a1]\n\t"
                     "s_nop 1\n\t"
                     "v_mov_b32_dpp %[addr], %[t] quad_perm:[0,1,2,3] row_mask:0x2 bank_mask:0xf\n\t"
                     "v_mov_b32 %[t], %[a2]\n\t"
                     "s_nop 1\n\t"
                     "v_mov_b32_dpp %[addr], %[t] quad_perm:[0,1,2,3] row_mask:0x4 bank_mask:0xf\n\t"
                     "v_mov_b32 %[t], %[a3]\n\t"
                     "s_nop 1\n\t"
                     "v_mov_b32_dpp %[addr], %[t] quad_perm:[0,1,2,3] row_mask:0x8 bank_mask:0xf\n\t"
                     "v_lshlrev_b32 %[addr], 4, %[addr]"
                     : [addr] "=&v"(addr), [t] "=&v"(t)
                     : [a0] "s"(a0), [a1] "s"(a1), [a2] "s"(a2), [a3] "s"(a3));
    return addr;
}
// orders one wave's LDS writes before its later LDS reads (the LDS serves a wave's instructions in order; this only keeps
// the compiler from moving them)
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
// The walk itself: turn(addr) is called, with the lanes of the quadrants that still have a hit, once per loop turn.
template <bool BANKED = false, typename Turn>
__device__ __forceinline__ void quadrant_walk(QuadrantHits &hits, uint32_t stage_base, Turn &&turn)
{
    // (the exit is taken from the scalar masks, not from the lanes' addresses: an exit test that the optimizer can fold
    // into the per-lane test below makes the loop, and the masks it carries, divergent in the compiler's eyes)
    while (quadrant_pending(hits)) {
        const uint32_t addr = quadrant_next_hit<BANKED>(hits);
        if (addr != kNoHit) turn(addr + stage_base);
    }
}
// Quadrant lists: the same walk with the scalar bit scans taken out of the loop.  After a batch is staged, the slots that
// reach quadrant q are written, in list order, to a short list in LDS (their LDS addresses), padded up to the length of
// the longest of the four lists with the address of a slot that no fragment passes (entry 0 of every row of a stage with
// kStageSlots entries per row: a cut-off quadratic above its |d|^2, opacity 0).  A turn of the loop is then one LDS read
// per lane -- entry `turn` of its quadrant's list -- instead of eight scalar and nine vector instructions that pick the
// next set bit of four masks and hand it to the quadrant's lanes, and a quadrant that has run out of hits evaluates the
// dummy slot, which fails the walk's own test, instead of being masked off: one exec level less.
constexpr int kStageSlots = 65;
typedef TileStage<kStageSlots> TileStageQ;
struct QuadrantLists {
    uint32_t a[4][64];
    uint32_t beyond;            // (the walk reads one entry ahead)
};
typedef __attribute__((address_space(3))) const uint32_t lds_u32;
// (one lane) the slot that fails every test: |m|^2 / cut-off = 1 everywhere, |d|^2 = 1/2, opacity 0
__device__ __forceinline__ void stage_dummy_init(TileStageQ &st, uint32_t lane)
{
    if (lane == 0) {
        st.q[0][0] = make_float4(1.0f, 0.0f, 0.0f, 0.0f);
        st.q[1][0] = make_float4(0.0f, 0.0f, 0.5f, 0.0f);
        st.q[2][0] = st.q[3][0] = st.q[4][0] = st.q[5][0] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
}
// LDS address of the q[0] entry of staged slot `slot` (0 .. 63)
__device__ __forceinline__ uint32_t stage_slot_address(const TileStageQ &st, uint32_t slot) { return stage_address(st) + 16u * (slot + 1u); }
// Called by the wave after tile_stage_load (bits: the lane's slot's quadrant bits): writes the four lists and returns the
// number of turns, the length of the longest (wave-uniform).  Every lane writes one entry per list: a slot that reaches
// the quadrant its address at the number of such slots before it, the others the dummy address behind all of them.
__device__ __forceinline__ uint32_t quadrant_lists_build(QuadrantLists &ql, uint32_t bits, uint32_t lane, const TileStageQ &st)
{
    const uint32_t dummy = stage_address(st), mine = stage_slot_address(st, lane);
    uint32_t most = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const bool hit = (bits >> q) & 1u;
        const uint64_t h = __ballot(hit);
        const uint32_t count = (uint32_t)__popcll(h);
        const uint32_t below = __builtin_amdgcn_mbcnt_hi((uint32_t)(h >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)h, 0u));
        ql.a[q][hit ? below : count + (lane - below)] = hit ? mine : dummy;
        most = most > count ? most : count;
    }
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)most);
}
// turn(addr) is called n_turns times, by all lanes: addr = the LDS address of the q[0] entry of the slot the lane's quadrant
// (lanes 16 q .. 16 q + 15) evaluates in this turn.
template <typename Turn>
__device__ __forceinline__ void quadrant_list_walk(const QuadrantLists &ql, uint32_t n_turns, uint32_t lane, Turn &&turn)
{
    // (the entry of the next turn is read while this turn's slot is evaluated: one LDS round trip per turn, not two)
    uint32_t p = (uint32_t)(uintptr_t)(lds_u32 *)&ql.a[lane >> 4][0];
    uint32_t addr = *(lds_u32 *)(uintptr_t)p;
    // (two turns per round of the loop, the entry that was read ahead changing registers, so that no turn moves it)
    uint32_t t = 0;
    for (; t + 1 < n_turns; t += 2) {
        asm volatile("v_add_u32 %0, 4, %0" : "+v"(p));
        const uint32_t next = *(lds_u32 *)(uintptr_t)p;
        turn(addr);
        asm volatile("v_add_u32 %0, 4, %0" : "+v"(p));
        addr = *(lds_u32 *)(uintptr_t)p;
        turn(next);
    }
    if (t < n_turns) turn(addr);
}
// The walk over instances [first, last) of a tile's list (whole batches of 64 from `first` on) by one wave, lanes =
// pixels by quadrants: every batch is staged (tile_stage_load with the CULL asked for), its quadrant lists are built and
// turn(addr) is called for every turn.  SOLO: the wave is the whole workgroup (its barriers are the workgroup's).
// AHEAD: a lane reads the list entry of the next batch before it walks this one (one register more through the walk; the
// entry is then there when the batch is staged, and the records' fetch does not wait for it).
template <int MODE, bool DEPTH, int CULL, bool SOLO, int REC4 = HTGS_PRIM_FLOATS / 4, bool UNIT = false, bool POS = false, bool AHEAD = false, typename Turn>
__device__ __forceinline__ void tile_list_walk(TileStageQ &st, QuadrantLists &ql, const float4 *__restrict__ prim, const uint32_t *__restrict__ inst,
                                               uint32_t first, uint32_t last, uint32_t lane, float cx, float cy, Turn &&turn, uint64_t pixel_lanes = 0)
{
    stage_dummy_init(st, lane);
    uint32_t listed = 0;
    if (AHEAD) listed = first + lane < last ? inst[first + lane] : 0u;
    for (uint32_t base = first; base < last; base += 64) {
        if (SOLO) __syncthreads(); else wave_lds_sync();
        const uint32_t bits = tile_stage_load<MODE, kStageSlots, DEPTH, CULL, true, REC4, UNIT, POS, AHEAD>(st, prim, inst, base + lane, last, lane + 1, cx, cy, pixel_lanes,
                                                                                                           listed);
        if (AHEAD) listed = base + 64u + lane < last ? inst[base + 64u + lane] : 0u;
        const uint32_t n_turns = quadrant_lists_build(ql, bits, lane, st);
        if (SOLO) __syncthreads(); else wave_lds_sync();
        // lanes outside the image run along (their results are never stored): the loop stays wave-uniform
        quadrant_list_walk(ql, n_turns, lane, turn);
    }
}
// The per-pixel records of the training pass are kept tile by tile: the 64 pixels of an 8x8 tile, row-major, are
// contiguous, so a tile's workgroup writes and reads whole lines whatever order the tiles are taken in.  A record plane
// has 64 entries per tile of the launch (gridDim.x tiles, the pixels beyond the image included).
__device__ __forceinline__ size_t record_pixel(uint32_t tile, uint32_t x, uint32_t y) { return (size_t)tile * 64u + (y & 7u) * 8u + (x & 7u); }
__device__ __forceinline__ size_t record_plane() { return (size_t)gridDim.x * 64u; }
// the tile a workgroup takes: the launch's blocks go through htgs_frame.tile_order (longest lists first) if there is one
__device__ __forceinline__ uint32_t block_tile(const uint32_t *__restrict__ tile_order) { return tile_order ? tile_order[blockIdx.x] : blockIdx.x; }
// pixel of a lane in an 8x8 tile that is walked by quadrants
struct TilePixel {
    uint32_t x, y;
    bool inside;
    PixelTerms pt;
    float cx, cy;
};
template <int N, int ROW>
__device__ __forceinline__ float4 stage_row(uint32_t addr)
{
    lds_float4 *p = (lds_float4 *)(uintptr_t)(addr + ROW * N * 16);
    return make_float4(p->x, p->y, p->z, p->w);
}
template <int N>
__device__ __forceinline__ float stage_opacity(uint32_t addr) { return *(lds_float *)(uintptr_t)(addr + 4 * N * 16 + 12); }
template <int N>
__device__ __forceinline__ uint32_t stage_index(uint32_t addr) { return float_to_bits(*(lds_float *)(uintptr_t)(addr + 5 * N * 16 + 12)); }

// |m|^2 <= cutoff |d|^2 ?  (inference.cuh:147)
template <int N>
__device__ __forceinline__ bool tile_frag_cutoff(uint32_t addr, const PixelTerms &p, TileFrag &o)
{
    const float4 q0 = stage_row<N, 0>(addr), q1 = stage_row<N, 1>(addr), q2 = stage_row<N, 2>(addr);
    o.num = quad_eval(q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, p);
    o.den = quad_eval(q1.z, q1.w, q2.x, q2.y, q2.z, q2.w, p);
    return !(o.num > o.den);
}

// camera-space depth of the point of maximum contribution (inference.cuh:151-152); needs o.den_rcp
template <int N>
__device__ __forceinline__ float tile_frag_depth(uint32_t addr, const PixelTerms &p, const TileFrag &o)
{
    const float4 q3 = stage_row<N, 3>(addr), q4 = stage_row<N, 4>(addr);
    return __builtin_fmaf(quad_eval(q3.x, q3.y, q3.z, q3.w, q4.x, q4.y, p), o.den_rcp, q4.z);
}

// The image-only fast path (FAST) takes the hardware's reciprocal and 2^x (v_rcp_f32, v_exp_f32: one ulp, a quarter of
// the instruction slots); every other kernel uses the exactly reproducible routines.
template <bool FAST>
__device__ __forceinline__ float frag_rcp(float x) { return FAST ? __builtin_amdgcn_rcpf(x) : rcp_exact(x); }

// alpha of the fragment, false below the mode's threshold; needs o.den_rcp
template <int MODE, bool FAST = false>
__device__ __forceinline__ bool tile_frag_alpha(float opacity, TileFrag &o)
{
    const float t = (o.num * ModeCfg<MODE>::exp2_scale) * o.den_rcp;
    const float G = FAST ? __builtin_amdgcn_exp2f(t) : d_exp2(t);
    const float a = opacity * G;
    o.alpha = a < kMaxFragmentAlpha ? a : kMaxFragmentAlpha;
    return !(o.alpha < ModeCfg<MODE>::min_alpha);
}

// The image-only fast path's fragment: with the opacity staged at no more than 1 (UNIT) alpha = opacity * G needs no clamp, and a
// fragment beyond the cut-off has G below the alpha threshold (the cut-off is where G equals it), so the alpha test alone
// decides; a vanishing or non-finite |d|^2 gives alpha 0 or NaN, which fails it.  Needs o.num, o.den.
template <int MODE, int N>
__device__ __forceinline__ bool tile_frag_fast(uint32_t addr, const PixelTerms &p, TileFrag &o)
{
    tile_frag_cutoff<N>(addr, p, o);
    o.den_rcp = __builtin_amdgcn_rcpf(o.den);
    o.alpha = stage_opacity<N>(addr) * __builtin_amdgcn_exp2f((o.num * ModeCfg<MODE>::exp2_scale) * o.den_rcp);
    return o.alpha >= ModeCfg<MODE>::min_alpha;
}

// Sorted insertion into a K-slot buffer (depth, alpha, index per slot) walks the slots front to back carrying the
// displaced entry (the reference's exchange walk); the slots are taken four at a time and the whole wave skips a group
// that no active lane can change (the carried depth is not below the group's last slot).  One slot: v_cmpx narrows
// exec to the lanes whose carried depth is below the slot's, three moves through a scratch register exchange each
// of the three registers (a wave64 v_mov_b32 holds the vector ALU for two cycles, v_swap_b32 for eight,
// v_cndmask_b32 for four), and exec is restored.  On return (depth, alpha, index) is what the walk pushed out.
constexpr int kInsertGroup = 4;
template <typename IndexT>
__device__ __forceinline__ void exchange_step(float &D, float &A, IndexT &I, float &d, float &a, IndexT &x, uint64_t all)
{
    static_assert(sizeof(IndexT) == 4, "one register");
    float t;
    asm volatile("v_cmpx_lt_f32 vcc, %[D], %[d]\n\t"
                 "v_mov_b32 %[t], %[d]\n\tv_mov_b32 %[d], %[D]\n\tv_mov_b32 %[D], %[t]\n\t"
                 "v_mov_b32 %[t], %[a]\n\tv_mov_b32 %[a], %[A]\n\tv_mov_b32 %[A], %[t]\n\t"
                 "v_mov_b32 %[t], %[x]\n\tv_mov_b32 %[x], %[I]\n\tv_mov_b32 %[I], %[t]\n\t"
                 "s_mov_b64 exec, %[all]"
                 : [D] "+v"(D), [A] "+v"(A), [I] "+v"(I), [d] "+v"(d), [a] "+v"(a), [x] "+v"(x), [t] "=&v"(t)
                 : [all] "s"(all)
                 : "vcc");
}
// four slots in one statement: exec is saved once and restored after every slot
#define HTGS_EXCHANGE_SLOT(n)                                                                                            \
    "v_cmpx_lt_f32 vcc, %[d], %[D" #n "]\n\t"                                                                           \
    "v_mov_b32 %[t], %[D" #n "]\n\tv_mov_b32 %[D" #n "], %[d]\n\tv_mov_b32 %[d], %[t]\n\t"                              \
    "v_mov_b32 %[t], %[A" #n "]\n\tv_mov_b32 %[A" #n "], %[a]\n\tv_mov_b32 %[a], %[t]\n\t"                              \
    "v_mov_b32 %[t], %[I" #n "]\n\tv_mov_b32 %[I" #n "], %[x]\n\tv_mov_b32 %[x], %[t]\n\t"                              \
    "s_mov_b64 exec, %[all]\n\t"
template <typename IndexT>
__device__ __forceinline__ void exchange_step4(float &d, float &a, IndexT &x, float &D0, float &A0, IndexT &I0, float &D1, float &A1, IndexT &I1,
                                               float &D2, float &A2, IndexT &I2, float &D3, float &A3, IndexT &I3)
{
    static_assert(sizeof(IndexT) == 4, "one register");
    float t;
    uint64_t all;
    asm volatile("s_mov_b64 %[all], exec\n\t" HTGS_EXCHANGE_SLOT(0) HTGS_EXCHANGE_SLOT(1) HTGS_EXCHANGE_SLOT(2) HTGS_EXCHANGE_SLOT(3)
                 : [d] "+v"(d), [a] "+v"(a), [x] "+v"(x), [D0] "+v"(D0), [A0] "+v"(A0), [I0] "+v"(I0), [D1] "+v"(D1), [A1] "+v"(A1), [I1] "+v"(I1),
                   [D2] "+v"(D2), [A2] "+v"(A2), [I2] "+v"(I2), [D3] "+v"(D3), [A3] "+v"(A3), [I3] "+v"(I3), [t] "=&v"(t), [all] "=&s"(all)
                 :
                 : "vcc");
}
#undef HTGS_EXCHANGE_SLOT
template <int K, typename IndexT>
__device__ __forceinline__ void core_exchange_walk(float &depth, float &alpha, IndexT &index, float (&cd)[K], float (&ca)[K], IndexT (&ci)[K])
{
    const uint64_t all = __ballot(true);               // the lanes that called
#pragma unroll
    for (int g0 = 0; g0 < K; g0 += kInsertGroup) {
        if (K > kInsertGroup && !__any(depth < cd[g0 + kInsertGroup - 1 < K ? g0 + kInsertGroup - 1 : K - 1])) continue;
        if constexpr (K % kInsertGroup == 0 && kInsertGroup == 4) {
            exchange_step4(depth, alpha, index, cd[g0], ca[g0], ci[g0], cd[g0 + 1], ca[g0 + 1], ci[g0 + 1], cd[g0 + 2], ca[g0 + 2], ci[g0 + 2],
                           cd[g0 + 3], ca[g0 + 3], ci[g0 + 3]);
        } else {
#pragma unroll
            for (int i = g0; i < g0 + kInsertGroup && i < K; ++i) exchange_step(depth, alpha, index, cd[i], ca[i], ci[i], all);
        }
    }
}

// The image-only fast path inserts by shifting instead: the entry that moves down the core alternates between two register
// triples, so that a slot costs two moves per register (slot -> the other triple, this triple -> slot) instead of an
// exchange through a scratch register.  Both triples start out as the fragment; a lane joins at the first slot that is
// not nearer than its fragment and from there on moves every slot down by one (<=: once it has joined, the entry it carries
// is the previous slot's, which is never deeper than the next slot's).  This is the stable insertion, not the reference's
// exchange walk: where two stored fragments have exactly the same depth the two differ in which of them ends up in front,
// which the fast path does not promise to reproduce.  On return (depth, alpha, index) is what was pushed out.
#define HTGS_QUICK_SLOT(n, R, W)                                                                                         \
    "v_cmpx_le_f32 vcc, %[d" #R "], %[D" #n "]\n\t"                                                                     \
    "v_mov_b32 %[d" #W "], %[D" #n "]\n\tv_mov_b32 %[D" #n "], %[d" #R "]\n\t"                                         \
    "v_mov_b32 %[a" #W "], %[A" #n "]\n\tv_mov_b32 %[A" #n "], %[a" #R "]\n\t"                                         \
    "v_mov_b32 %[x" #W "], %[I" #n "]\n\tv_mov_b32 %[I" #n "], %[x" #R "]\n\t"                                         \
    "s_mov_b64 exec, %[all]\n\t"
template <typename IndexT>
__device__ __forceinline__ void quick_step4(float &d0, float &a0, IndexT &x0, float &d1, float &a1, IndexT &x1, float &D0, float &A0, IndexT &I0,
                                            float &D1, float &A1, IndexT &I1, float &D2, float &A2, IndexT &I2, float &D3, float &A3, IndexT &I3)
{
    static_assert(sizeof(IndexT) == 4, "one register");
    uint64_t all;
    asm volatile("s_mov_b64 %[all], exec\n\t" HTGS_QUICK_SLOT(0, 0, 1) HTGS_QUICK_SLOT(1, 1, 0) HTGS_QUICK_SLOT(2, 0, 1) HTGS_QUICK_SLOT(3, 1, 0)
                 : [d0] "+v"(d0), [a0] "+v"(a0), [x0] "+v"(x0), [d1] "+v"(d1), [a1] "+v"(a1), [x1] "+v"(x1), [D0] "+v"(D0), [A0] "+v"(A0),
                   [I0] "+v"(I0), [D1] "+v"(D1), [A1] "+v"(A1), [I1] "+v"(I1), [D2] "+v"(D2), [A2] "+v"(A2), [I2] "+v"(I2), [D3] "+v"(D3),
                   [A3] "+v"(A3), [I3] "+v"(I3), [all] "=&s"(all)
                 :
                 : "vcc");
}
#undef HTGS_QUICK_SLOT
template <int K, typename IndexT>
__device__ __forceinline__ void core_quick_walk(float &depth, float &alpha, IndexT &index, float (&cd)[K], float (&ca)[K], IndexT (&ci)[K])
{
    if constexpr (K % 4 != 0) core_exchange_walk<K>(depth, alpha, index, cd, ca, ci);
    else {
        float d1 = depth, a1 = alpha;
        IndexT x1 = index;
#pragma unroll
        for (int g0 = 0; g0 < K; g0 += 4) {
            // (a group that no lane's entry is nearer than the end of: nothing moves there; a group is an even number of
            // slots, so the entry is back in the first triple at every group's start)
            if (K > 4 && !__any(depth < cd[g0 + 3])) continue;
            quick_step4(depth, alpha, index, d1, a1, x1, cd[g0], ca[g0], ci[g0], cd[g0 + 1], ca[g0 + 1], ci[g0 + 1], cd[g0 + 2], ca[g0 + 2], ci[g0 + 2],
                        cd[g0 + 3], ca[g0 + 3], ci[g0 + 3]);
        }
    }
}

__device__ __forceinline__ TilePixel quadrant_tile_pixel(uint32_t tile, uint32_t grid_w, uint32_t lane, uint32_t width, uint32_t height)
{
    TilePixel p;
    const uint32_t x0 = (tile % grid_w) * 8, y0 = (tile / grid_w) * 8;
    uint32_t local_x, local_y;
    quadrant_pixel(lane, local_x, local_y);
    p.x = x0 + local_x;
    p.y = y0 + local_y;
    p.inside = p.x < width && p.y < height;
    p.pt = pixel_terms(local_x, local_y, 8);
    // (the same in every lane: held in scalar registers, two vector registers less in kernels that count them)
    p.cx = bits_to_float((uint32_t)__builtin_amdgcn_readfirstlane((int)float_to_bits(tile_centre(x0, 8))));
    p.cy = bits_to_float((uint32_t)__builtin_amdgcn_readfirstlane((int)float_to_bits(tile_centre(y0, 8))));
    return p;
}

// The 16x16 tile of ALPHA_BLEND_GLOBAL_ORDERING: 256 threads, wave w holds the 8x8 sub-tile 2 (row >= 8) + (column >= 8)
// = w, laid out for the quadrant walk.
__device__ __forceinline__ void subtile_pixel(uint32_t thread, uint32_t &local_x, uint32_t &local_y)
{
    quadrant_pixel(thread & 63u, local_x, local_y);
    local_x += 8u * ((thread >> 6) & 1u);
    local_y += 8u * (thread >> 7);
}
// One batch of 256 staged instances (reach[slot]: the sixteen quadrant bits tile_stage_load returned for it): the wave
// walks the hits of its own four quadrants, 64 slots at a time, and stops early once all_done() says so (wave-uniform).
template <typename Done, typename Turn>
__device__ __forceinline__ void subtile_walk(const uint16_t *reach, uint32_t stage_base, uint32_t n_staged, uint32_t wave, uint32_t lane,
                                             Done &&all_done, Turn &&turn)
{
    for (uint32_t part = 0; part < 4 && 64u * part < n_staged; ++part) {
        if (all_done()) break;
        QuadrantHits hits = quadrant_ballot(((uint32_t)reach[64u * part + lane] >> (4u * wave)) & 0xfu);
        quadrant_walk(hits, stage_base + 64u * 16u * part, turn);
    }
}

}  // namespace htgs
