// C ABI glue: error reporting, size helpers and the two-call frame driver.
// The launch order restates <mode>::inference (R/src/hybrid_blend/inference.cu:57-183 and its
// siblings); the reference's single blocking read of the instance count (:118-119) is the seam
// between htgs_render_front and htgs_render_back.
#include "common.h"
#include <cstdarg>
#include <cstdio>

namespace htgs {

static thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what)
{
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HTGS_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
    return HTGS_OK;
}

// extract_end_bit, R/include/rasterization_utils.h:3-13: bit width of n
static int bit_width(uint32_t n)
{
    int b = 0;
    while (n) { ++b; n >>= 1; }
    return b;
}

// every positive float whose exponent field is in [7, 247]: refined reciprocal against the division
__global__ void __launch_bounds__(256) check_reciprocal_kernel(unsigned long long *__restrict__ counts)
{
    const uint32_t tid = blockIdx.x * 256 + threadIdx.x, stride = gridDim.x * 256;
    unsigned long long tested = 0, wrong = 0;
    for (uint64_t u = tid; u < 0x80000000ull; u += stride) {
        const float x = bits_to_float((uint32_t)u);
        if (!rcp_in_range(x)) continue;
        ++tested;
        if (float_to_bits(rcp_refined(x)) != float_to_bits(1.0f / x)) ++wrong;
    }
    atomicAdd(counts, tested);
    if (wrong) atomicAdd(counts + 1, wrong);
}

}  // namespace htgs

using namespace htgs;

extern "C" int htgs_check_reciprocal(unsigned long long *counts, void *stream)
{
    if (!counts) return fail(HTGS_ERR_ARGUMENT, "htgs_check_reciprocal: null pointer");
    hipLaunchKernelGGL(check_reciprocal_kernel, dim3(4096), dim3(256), 0, (hipStream_t)stream, counts);
    return check_launch("check_reciprocal");
}

extern "C" const char *htgs_last_error(void) { return g_error; }

extern "C" int htgs_tile_size(int mode) { return tile_size(mode); }

extern "C" int htgs_end_bit(int mode, int width, int height)
{
    const int tile = tile_size(mode);
    const uint32_t n_tiles = (uint32_t)div_up(width, tile) * (uint32_t)div_up(height, tile);
    const int bits = bit_width(n_tiles - 1);
    return mode == HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING ? bits + 32 : bits;
}

extern "C" int htgs_key_bytes(int mode, int width, int height)
{
    if (mode == HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING) return 8;
    return htgs_end_bit(mode, width, height) <= 16 ? 2 : 4;
}

extern "C" int htgs_frame_end_bit(const htgs_frame *f)
{
    if (!f) return 0;
    return htgs_end_bit(f->mode, f->width, f->height) - (frame_depth_ordered(f) && f->mode == HTGS_MODE_ALPHA_BLEND_GLOBAL_ORDERING ? 32 : 0);
}

extern "C" int htgs_frame_key_bytes(const htgs_frame *f)
{
    if (!f) return 0;
    if (frame_depth_ordered(f)) return htgs_frame_end_bit(f) <= 16 ? 2 : 4;
    return htgs_key_bytes(f->mode, f->width, f->height);
}

extern "C" int htgs_frame_sort_passes(const htgs_frame *f)
{
    if (!f) return 0;
    const int bits = htgs_frame_key_bytes(f) == 8 ? 9 : 8;
    return (htgs_frame_end_bit(f) + bits - 1) / bits;
}

extern "C" int htgs_sort_passes(int mode, int width, int height)
{
    // 8 bits per pass, 9 for the 8-byte tile|depth keys (radix_sort.hip)
    const int bits = htgs_key_bytes(mode, width, height) == 8 ? 9 : 8;
    return (htgs_end_bit(mode, width, height) + bits - 1) / bits;
}

extern "C" int htgs_render_front(const htgs_frame *f)
{
    int rc = htgs_preprocess(f);
    if (rc != HTGS_OK) return rc;
    return htgs_scan_offsets(f);
}

extern "C" int htgs_render_back(const htgs_frame *f)
{
    int selector = 0;
    int rc = htgs_create_instances(f);
    if (rc != HTGS_OK) return rc;
    rc = htgs_sort_instances(f, &selector);
    if (rc != HTGS_OK) return rc;
    rc = htgs_extract_ranges(f, selector);
    if (rc != HTGS_OK) return rc;
    return htgs_blend(f, selector);
}

extern "C" int htgs_forward_front(const htgs_frame *f)
{
    if (!f) return fail(HTGS_ERR_ARGUMENT, "htgs_forward_front: null frame");
    if (!f->clamp_info && f->n_primitives > 0) return fail(HTGS_ERR_ARGUMENT, "htgs_forward_front: clamp_info is required for training");
    // (the per-Gaussian backward finds a Gaussian's gradient rows through offsets[] in index order)
    if (frame_depth_ordered(f)) return fail(HTGS_ERR_ARGUMENT, "htgs_forward_front: depth_order is for the inference entry points");
    htgs_frame t = *f;
    t.scale_modifier = 1.0f;   // the training preprocess has no scale modifier (R/include/hybrid_blend/kernels/forward.cuh:10-76)
    int rc = htgs_preprocess(&t);
    if (rc != HTGS_OK) return rc;
    return htgs_scan_offsets(&t);
}

extern "C" int htgs_forward_back(const htgs_frame *f, int *selector)
{
    if (!f || !selector) return fail(HTGS_ERR_ARGUMENT, "htgs_forward_back: null argument");
    if (frame_depth_ordered(f)) return fail(HTGS_ERR_ARGUMENT, "htgs_forward_back: depth_order is for the inference entry points");
    int rc = htgs_create_instances(f);
    if (rc != HTGS_OK) return rc;
    rc = htgs_sort_instances(f, selector);
    if (rc != HTGS_OK) return rc;
    rc = htgs_extract_ranges(f, *selector);
    if (rc != HTGS_OK) return rc;
    return htgs_blend_forward(f, *selector);
}
