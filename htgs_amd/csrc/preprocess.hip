// Per-Gaussian stage: cull, exact perspective-correct screen bounds, VPMT rows, MT3, SH colour.
// Restates preprocess_cu of the four modes (R/include/hybrid_blend/kernels/inference.cuh:10-76 and siblings,
// forward.cuh:10-76 for the clamp flags) on top of transform_and_cull / convert_sh_to_rgb
// (R/include/kernel_utils.cuh:63-188).  No fused operations in this file: operand order of the reference.
#include "common.h"

namespace htgs {

struct Camera {
    float M3[4];
    float VPM[16];
    float cam[3];
};

__device__ __forceinline__ float dot3(const float *a, float bx, float by, float bz)
{
    return a[0] * bx + a[1] * by + a[2] * bz;
}
__device__ __forceinline__ float dot4(float ax, float ay, float az, float aw, float bx, float by, float bz, float bw)
{
    return ax * bx + ay * by + az * bz + aw * bw;
}

// min(grid, (uint)max(0, float2int_rd/ru(v))), kernel_utils.cuh:128-133; NaN -> 0, saturating.
__device__ __forceinline__ uint32_t tile_floor(float v, uint32_t grid)
{
    const float r = __builtin_floorf(v);
    if (!(r > 0.0f)) return 0u;
    if (r >= (float)grid) return grid;
    return (uint32_t)r;
}
__device__ __forceinline__ uint32_t tile_ceil(float v, uint32_t grid)
{
    const float r = __builtin_ceilf(v);
    if (!(r > 0.0f)) return 0u;
    if (r >= (float)grid) return grid;
    return (uint32_t)r;
}

struct Row { float x, y, z, w; };

__device__ __forceinline__ Row vpmt_row(const float *row, const float *u, const float *v, const float *w, const float *p)
{
    Row r;
    r.x = dot3(row, u[0], u[1], u[2]);
    r.y = dot3(row, v[0], v[1], v[2]);
    r.z = dot3(row, w[0], w[1], w[2]);
    r.w = dot3(row, p[0], p[1], p[2]) + row[3];
    return r;
}

__device__ __forceinline__ void axis_extent(const float f[4], const Row &Vi, const Row &V4, float &center, float &extent)
{
    center = dot4(f[0], f[1], f[2], f[3], Vi.x * V4.x, Vi.y * V4.y, Vi.z * V4.z, Vi.w * V4.w);
    const float q = dot4(f[0], f[1], f[2], f[3], Vi.x * Vi.x, Vi.y * Vi.y, Vi.z * Vi.z, Vi.w * Vi.w);
    extent = __builtin_sqrtf(clamp_pos(center * center - q));
}

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3))) preprocess_kernel(
    const float *__restrict__ positions, const float *__restrict__ scales, const float *__restrict__ rotations,
    const float *__restrict__ opacities, const float *__restrict__ sh_0, const float *__restrict__ sh_rest,
    const float *__restrict__ M, const float *__restrict__ VPM_in, const float *__restrict__ cam_position,
    uint32_t *__restrict__ n_touched, uint16_t *__restrict__ bounds, float *__restrict__ prim,
    uint8_t *__restrict__ clamp_info,
    int n, uint32_t grid_w, uint32_t grid_h, float tile, float min_alpha_rcp,
    int active_sh, int total_sh, float near_plane, float far_plane, float scale_modifier, int rec4,
    uint32_t *__restrict__ depth_keys, uint32_t *__restrict__ depth_vals, uint32_t depth_base, uint32_t depth_culled, int depth_shift)
{
    // One LDS buffer, used twice: first the block's slice of sh_rest (contiguous in memory, loaded with coalesced
    // 16-byte reads and then read back per Gaussian at a stride of 3 * total_sh words), then the block's records
    // (rec4 words of 16 bytes each: five, or eight in training frames, of which the last three are zeros here),
    // written back as one contiguous run of 16-byte stores.
    extern __shared__ float4 lds4[];
    float *lds = reinterpret_cast<float *>(lds4);
    __shared__ uint8_t s_visible[256];
    const int first = blockIdx.x * 256;
    const int i = first + threadIdx.x;
    const bool in_range = i < n;

    // camera: uniform addresses, the compiler turns these into scalar loads
    float M3[4], VPM[16], cam[3];
#pragma unroll
    for (int k = 0; k < 4; ++k) M3[k] = M[8 + k];
#pragma unroll
    for (int k = 0; k < 16; ++k) VPM[k] = VPM_in[k];
#pragma unroll
    for (int k = 0; k < 3; ++k) cam[k] = cam_position[k];

    // The block's slice of sh_rest is three quarters of everything this kernel reads.  Its loads are issued first,
    // into registers, so that they are in flight while the bounds are computed; they reach LDS further down.
    constexpr int kShRegs = 16;                                    // 16-byte words per thread: 256 x 3 x 21 / 4 / 256
    const int per = 3 * total_sh;                                  // words per Gaussian
    const int n_block = n - first < 256 ? n - first : 256;
    const size_t base_word = (size_t)first * per;                 // multiple of 256 words: 16-byte aligned
    const int words = active_sh > 1 ? n_block * per : 0;
    const float4 *src4 = reinterpret_cast<const float4 *>(sh_rest + base_word);
    float sh_regs[kShRegs][4];
#pragma unroll
    for (int k = 0; k < kShRegs; ++k) {
        const int q = k * 256 + threadIdx.x;
        float4 t = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (q < words / 4) {
            // (read once per frame and 576 MB on a scene of 3 M Gaussians: marked as streaming, so that it does not push the
            // records and lists the later stages come back to out of the last-level cache)
            typedef float streamed_float4 __attribute__((ext_vector_type(4)));
            const streamed_float4 v = __builtin_nontemporal_load(reinterpret_cast<const streamed_float4 *>(src4 + q));
            t = make_float4(v.x, v.y, v.z, v.w);
        }
        sh_regs[k][0] = t.x; sh_regs[k][1] = t.y; sh_regs[k][2] = t.z; sh_regs[k][3] = t.w;
    }

    uint32_t touched = 0;
    const size_t ic = in_range ? (size_t)i : 0;
    const float p[3] = { positions[3 * ic], positions[3 * ic + 1], positions[3 * ic + 2] };
    const float opacity = opacities[ic];
    const float z = dot3(M3, p[0], p[1], p[2]) + M3[3];                                   // kernel_utils.cuh:89
    bool visible = in_range && !(z < near_plane || z > far_plane);                        // :90
    float u[3], v[3], w[3];
    Row V1, V2, V4;
    uint32_t b0 = 0, b1 = 0, b2 = 0, b3 = 0;
    if (visible) {
        const float sx = scales[3 * (size_t)i], sy = scales[3 * (size_t)i + 1], sz = scales[3 * (size_t)i + 2];
        const float4 q = *reinterpret_cast<const float4 *>(rotations + 4 * (size_t)i);
        const float r = q.x, x = q.y, y = q.z, zq = q.w;                                   // :33
        const float xx = x * x, yy = y * y, zz = zq * zq;
        const float xy = x * y, xz = x * zq, yz = y * zq;
        const float rx = r * x, ry = r * y, rz = r * zq;
        const float R11 = 1.0f - 2.0f * (yy + zz), R12 = 2.0f * (xy - rz), R13 = 2.0f * (xz + ry);
        const float R21 = 2.0f * (xy + rz), R22 = 1.0f - 2.0f * (xx + zz), R23 = 2.0f * (yz - rx);
        const float R31 = 2.0f * (xz - ry), R32 = 2.0f * (yz + rx), R33 = 1.0f - 2.0f * (xx + yy);
        u[0] = (R11 * sx) * scale_modifier; u[1] = (R21 * sx) * scale_modifier; u[2] = (R31 * sx) * scale_modifier;  // :98
        v[0] = (R12 * sy) * scale_modifier; v[1] = (R22 * sy) * scale_modifier; v[2] = (R32 * sy) * scale_modifier;  // :99
        w[0] = (R13 * sz) * scale_modifier; w[1] = (R23 * sz) * scale_modifier; w[2] = (R33 * sz) * scale_modifier;  // :100
        V4 = vpmt_row(VPM + 12, u, v, w, p);                                               // :102
        const float rho = 2.0f * d_logf(opacity * min_alpha_rcp);                          // :104
        const float s = dot4(rho, rho, rho, -1.0f, V4.x * V4.x, V4.y * V4.y, V4.z * V4.z, V4.w * V4.w);  // :106
        visible = !(s == 0.0f);                                                            // :107
        if (visible) {
            const float rs = 1.0f / s;
            const float f[4] = { rs * rho, rs * rho, rs * rho, rs * -1.0f };               // :108
            const Row V3 = vpmt_row(VPM + 8, u, v, w, p);                                  // :111
            float cz, ez;
            axis_extent(f, V3, V4, cz, ez);                                                // :112-113
            visible = !(cz - ez < -1.0f || cz + ez > 1.0f);                                // :114-116
            if (visible) {
                V1 = vpmt_row(VPM + 0, u, v, w, p);                                        // :119
                V2 = vpmt_row(VPM + 4, u, v, w, p);                                        // :123
                float cx, ex, cy, ey;
                axis_extent(f, V1, V4, cx, ex);                                            // :120-121
                axis_extent(f, V2, V4, cy, ey);                                            // :124-125
                b0 = tile_floor(((cx - ex) + 0.5f) / tile, grid_w);                        // :129
                b1 = tile_ceil(((cx + ex) + 0.5f) / tile, grid_w);                         // :130
                b2 = tile_floor(((cy - ey) + 0.5f) / tile, grid_h);                        // :131
                b3 = tile_ceil(((cy + ey) + 0.5f) / tile, grid_h);                         // :132
                touched = (b1 - b0) * (b3 - b2);                                           // :136
                visible = touched != 0;
            }
        }
    }
    if (in_range) n_touched[i] = touched;
    // htgs_frame.depth_order: the pairs that sort the Gaussians by depth (depth_key_range() in common.h)
    if (depth_keys != nullptr && in_range) {
        // (a depth that is not a number passes the cull above, as in the reference, where its bit pattern sorts behind every
        // valid depth; here its key is held below `culled`, so it is neither dropped nor sorted by bits that the sort ignores)
        const uint32_t key = (float_to_bits(z) - depth_base) >> depth_shift;
        depth_keys[i] = touched != 0 ? (key < depth_culled - 1u ? key : depth_culled - 1u) : depth_culled;
        depth_vals[i] = (uint32_t)i;
    }
    s_visible[threadIdx.x] = visible;
    if (visible)
        *reinterpret_cast<ushort4 *>(bounds + 4 * (size_t)i) = make_ushort4((uint16_t)b0, (uint16_t)b1, (uint16_t)b2, (uint16_t)b3);

    // stage the block's SH coefficients
#pragma unroll
    for (int k = 0; k < kShRegs; ++k) {
        const int q = k * 256 + threadIdx.x;
        if (q < words / 4) lds4[q] = make_float4(sh_regs[k][0], sh_regs[k][1], sh_regs[k][2], sh_regs[k][3]);
    }
    for (int q = (words & ~3) + threadIdx.x; q < words; q += 256) lds[q] = sh_rest[base_word + q];
    __syncthreads();

    // view-dependent colour, kernel_utils.cuh:152-187
    float res[3] = { 0.0f, 0.0f, 0.0f };
    if (visible && sh_0) {                                         // no colour without coefficients (max-weights pass)
#pragma unroll
    for (int k = 0; k < 3; ++k) res[k] = 0.5f + 0.28209479177387814f * sh_0[3 * (size_t)i + k];
    if (active_sh > 1) {
        const float *c = lds + per * threadIdx.x;
        const float dx = p[0] - cam[0], dy = p[1] - cam[1], dz = p[2] - cam[2];
        const float inv = 1.0f / __builtin_sqrtf(dx * dx + dy * dy + dz * dz);
        const float x = dx * inv, y = dy * inv, zd = dz * inv;
        const float a0 = -0.48860251190291987f * y, a1 = 0.48860251190291987f * zd, a2 = -0.48860251190291987f * x;
#pragma unroll
        for (int k = 0; k < 3; ++k) res[k] = res[k] + a0 * c[0 + k] + a1 * c[3 + k] + a2 * c[6 + k];
        if (active_sh > 4) {
            const float xx = x * x, yy = y * y, zz = zd * zd;
            const float xy = x * y, xz = x * zd, yz = y * zd;
            const float a3 = 1.0925484305920792f * xy;
            const float a4 = -1.0925484305920792f * yz;
            const float a5 = 0.94617469575755997f * zz - 0.31539156525251999f;
            const float a6 = -1.0925484305920792f * xz;
            const float a7 = 0.54627421529603959f * xx - 0.54627421529603959f * yy;
#pragma unroll
            for (int k = 0; k < 3; ++k)
                res[k] = res[k] + a3 * c[9 + k] + a4 * c[12 + k] + a5 * c[15 + k] + a6 * c[18 + k] + a7 * c[21 + k];
            if (active_sh > 9) {
                const float a8 = 0.59004358992664352f * y * (-3.0f * xx + yy);
                const float a9 = 2.8906114426405538f * xy * zd;
                const float a10 = 0.45704579946446572f * y * (1.0f - 5.0f * zz);
                const float a11 = 0.3731763325901154f * zd * (5.0f * zz - 3.0f);
                const float a12 = 0.45704579946446572f * x * (1.0f - 5.0f * zz);
                const float a13 = 1.4453057213202769f * zd * (xx - yy);
                const float a14 = 0.59004358992664352f * x * (-xx + 3.0f * yy);
#pragma unroll
                for (int k = 0; k < 3; ++k)
                    res[k] = res[k] + a8 * c[24 + k] + a9 * c[27 + k] + a10 * c[30 + k] + a11 * c[33 + k]
                                    + a12 * c[36 + k] + a13 * c[39 + k] + a14 * c[42 + k];
            }
        }
    }
    if (clamp_info) {
        clamp_info[i] = res[0] < 0.0f;
        clamp_info[(size_t)n + i] = res[1] < 0.0f;
        clamp_info[2 * (size_t)n + i] = res[2] < 0.0f;
    }
    }
    __syncthreads();                                               // everyone is done reading the coefficients

    if (visible) {
        float4 *rec = lds4 + rec4 * threadIdx.x;
        rec[0] = make_float4(V1.x, V1.y, V1.z, V1.w);
        rec[1] = make_float4(V2.x, V2.y, V2.z, V2.w);
        rec[2] = make_float4(V4.x, V4.y, V4.z, V4.w);
        rec[3] = make_float4(dot3(M3, u[0], u[1], u[2]), dot3(M3, v[0], v[1], v[2]), dot3(M3, w[0], w[1], w[2]), z);
        rec[4] = make_float4(clamp_pos(res[0]), clamp_pos(res[1]), clamp_pos(res[2]), opacity);
        for (int k = HTGS_PRIM_FLOATS / 4; k < rec4; ++k) rec[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);   // (whole lines go out)
    }
    __syncthreads();
    float4 *dst4 = reinterpret_cast<float4 *>(prim) + (size_t)rec4 * first;
    if (rec4 == HTGS_PRIM_FLOATS / 4) {
        typedef float streamed_float4 __attribute__((ext_vector_type(4)));
        for (int q = threadIdx.x; q < n_block * (HTGS_PRIM_FLOATS / 4); q += 256)
            if (s_visible[q / (HTGS_PRIM_FLOATS / 4)]) {
                const float4 v = lds4[q];
                streamed_float4 w; w.x = v.x; w.y = v.y; w.z = v.z; w.w = v.w;
                __builtin_nontemporal_store(w, reinterpret_cast<streamed_float4 *>(dst4 + q));
            }
    } else {
        for (int q = threadIdx.x; q < n_block * (HTGS_PRIM_FLOATS_TRAIN / 4); q += 256)
            if (s_visible[q / (HTGS_PRIM_FLOATS_TRAIN / 4)]) dst4[q] = lds4[q];
    }
}

}  // namespace htgs

extern "C" int htgs_preprocess(const htgs_frame *f)
{
    using namespace htgs;
    if (!f) return fail(HTGS_ERR_ARGUMENT, "htgs_preprocess: null frame");
    if (f->mode < 0 || f->mode > 3) return fail(HTGS_ERR_MODE, "unsupported rasterizer mode");
    if (f->n_primitives < 0 || f->width <= 0 || f->height <= 0 || f->total_sh_bases < 0)
        return fail(HTGS_ERR_ARGUMENT, "htgs_preprocess: bad sizes");
    if (f->n_primitives == 0) return HTGS_OK;
    if (!f->positions || !f->scales || !f->rotations || !f->opacities || !f->M || !f->VPM ||
        !f->cam_position || !f->n_touched || !f->bounds || !f->prim)
        return fail(HTGS_ERR_ARGUMENT, "htgs_preprocess: null pointer");
    // the SH bands read from sh_rest must exist: 3, 8 and 15 coefficients for degrees 1, 2, 3
    const int need = f->active_sh_bases > 9 ? 15 : f->active_sh_bases > 4 ? 8 : f->active_sh_bases > 1 ? 3 : 0;
    if (need > f->total_sh_bases || (need > 0 && !f->sh_rest))
        return fail(HTGS_ERR_ARGUMENT, "htgs_preprocess: active_sh_bases needs more coefficients than sh_rest holds");
    const int tile = tile_size(f->mode);
    const uint32_t grid_w = div_up(f->width, tile), grid_h = div_up(f->height, tile);
    if (grid_w > 65535u || grid_h > 65535u) return fail(HTGS_ERR_ARGUMENT, "htgs_preprocess: image too large for 16-bit tile bounds");
    const float min_alpha_rcp = f->mode == HTGS_MODE_ALPHA_BLEND_FIRST_K ? 20.0f : 255.0f;
    // dynamic LDS: the larger of the block's SH coefficients (256 x 3 x total_sh words) and its records (256 x 80 or 128 bytes)
    const size_t sh_bytes = f->active_sh_bases > 1 ? (size_t)256 * 3 * f->total_sh_bases * sizeof(float) : 0;
    const int prim_floats = frame_prim_floats(f);
    if (prim_floats < 0) return fail(HTGS_ERR_ARGUMENT, "htgs_preprocess: prim_floats must be 0, %d or %d", HTGS_PRIM_FLOATS, HTGS_PRIM_FLOATS_TRAIN);
    const size_t lds_bytes = sh_bytes > 256 * prim_floats * sizeof(float) ? sh_bytes : 256 * prim_floats * sizeof(float);
    if (lds_bytes > 64 * 1024) return fail(HTGS_ERR_ARGUMENT, "htgs_preprocess: sh_rest has more than 21 coefficients per Gaussian");
    const bool ordered = frame_depth_ordered(f);
    if (ordered && ((uintptr_t)f->depth_order & 15)) return fail(HTGS_ERR_ARGUMENT, "htgs_preprocess: depth_order must be 16-byte aligned");
    const DepthOrder order = depth_order_parts(f);
    const DepthKeys order_keys = depth_key_range(f);
    hipLaunchKernelGGL(preprocess_kernel, dim3(div_up(f->n_primitives, 256)), dim3(256), lds_bytes, (hipStream_t)f->stream,
                       f->positions, f->scales, f->rotations, f->opacities, f->sh_0, f->sh_rest, f->M, f->VPM, f->cam_position,
                       f->n_touched, f->bounds, f->prim, f->clamp_info, f->n_primitives, grid_w, grid_h, (float)tile,
                       min_alpha_rcp, f->active_sh_bases, f->total_sh_bases, f->near_plane, f->far_plane, f->scale_modifier, prim_floats / 4,
                       ordered ? order.keys[0] : nullptr, ordered ? order.vals[0] : nullptr, order_keys.base, order_keys.culled, order_keys.shift);
    return check_launch("preprocess");
}
