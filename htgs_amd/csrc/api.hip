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

__global__ void __launch_bounds__(256) copy_bytes_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i];
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

// Issue cost of single vector instructions: every kernel below runs 64 copies of one instruction per loop turn over
// eight registers (the copies of one register depend on each other, the eight registers do not).
#define HTGS_R8(op) op(0) op(1) op(2) op(3) op(4) op(5) op(6) op(7)
#define HTGS_R64(op) HTGS_R8(op) HTGS_R8(op) HTGS_R8(op) HTGS_R8(op) HTGS_R8(op) HTGS_R8(op) HTGS_R8(op) HTGS_R8(op)
#define HTGS_ISSUE_KERNEL(name, op)                                                                                              \
    __global__ void __launch_bounds__(256) name(float *__restrict__ out, int turns)                                              \
    {                                                                                                                            \
        float a0 = threadIdx.x * 1e-3f, a1 = a0 + 1.0f, a2 = a0 + 2.0f, a3 = a0 + 3.0f, a4 = a0 + 4.0f, a5 = a0 + 5.0f,            \
              a6 = a0 + 6.0f, a7 = a0 + 7.0f;                                                                                    \
        const float m = 1.0001f, c = 0.5f;                                                                                       \
        for (int i = 0; i < turns; ++i)                                                                                          \
            asm volatile("s_mov_b64 s[40:41], 0x5555\n" HTGS_R64(op)                                                             \
                         : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7)                       \
                         : "v"(m), "v"(c)                                                                                        \
                         : "vcc", "s40", "s41");                                                                                 \
        out[blockIdx.x * 256 + threadIdx.x] = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7;                                             \
    }
#define HTGS_OP_FMA(i) "v_fma_f32 %" #i ", %" #i ", %8, %9\n"
#define HTGS_OP_ADD(i) "v_add_f32 %" #i ", %" #i ", %9\n"
#define HTGS_OP_MUL(i) "v_mul_f32 %" #i ", %" #i ", %8\n"
#define HTGS_OP_MOV(i) "v_mov_b32 %" #i ", %9\n"
#define HTGS_OP_ADDU(i) "v_add_u32 %" #i ", %" #i ", %9\n"
#define HTGS_OP_MIN(i) "v_min_f32 %" #i ", %" #i ", %9\n"
#define HTGS_OP_CMP(i) "v_cmp_lt_f32 vcc, %" #i ", %9\n"
#define HTGS_OP_CND(i) "v_cndmask_b32_e64 %" #i ", %" #i ", %9, s[40:41]\n"
#define HTGS_OP_RND(i) "v_rndne_f32 %" #i ", %" #i "\n"
#define HTGS_OP_CVT(i) "v_cvt_i32_f32 %" #i ", %" #i "\n"
#define HTGS_OP_LSHLADD(i) "v_lshl_add_u32 %" #i ", %" #i ", 3, %9\n"
#define HTGS_OP_RCP(i) "v_rcp_f32 %" #i ", %" #i "\n"
#define HTGS_OP_EXP(i) "v_exp_f32 %" #i ", %" #i "\n"
#define HTGS_OP_SWAP(i) "v_swap_b32 %" #i ", %9\n"
HTGS_ISSUE_KERNEL(issue_fma_kernel, HTGS_OP_FMA)
HTGS_ISSUE_KERNEL(issue_add_kernel, HTGS_OP_ADD)
HTGS_ISSUE_KERNEL(issue_mul_kernel, HTGS_OP_MUL)
HTGS_ISSUE_KERNEL(issue_mov_kernel, HTGS_OP_MOV)
HTGS_ISSUE_KERNEL(issue_addu_kernel, HTGS_OP_ADDU)
HTGS_ISSUE_KERNEL(issue_min_kernel, HTGS_OP_MIN)
HTGS_ISSUE_KERNEL(issue_cmp_kernel, HTGS_OP_CMP)
HTGS_ISSUE_KERNEL(issue_cnd_kernel, HTGS_OP_CND)
HTGS_ISSUE_KERNEL(issue_rnd_kernel, HTGS_OP_RND)
HTGS_ISSUE_KERNEL(issue_cvt_kernel, HTGS_OP_CVT)
HTGS_ISSUE_KERNEL(issue_lshladd_kernel, HTGS_OP_LSHLADD)
HTGS_ISSUE_KERNEL(issue_rcp_kernel, HTGS_OP_RCP)
HTGS_ISSUE_KERNEL(issue_exp_kernel, HTGS_OP_EXP)
// (v_swap_b32 writes both operands: the second one is a ninth register of its own)
__global__ void __launch_bounds__(256) issue_swap_kernel(float *__restrict__ out, int turns)
{
    float a0 = threadIdx.x * 1e-3f, a1 = a0 + 1.0f, a2 = a0 + 2.0f, a3 = a0 + 3.0f, a4 = a0 + 4.0f, a5 = a0 + 5.0f, a6 = a0 + 6.0f,
          a7 = a0 + 7.0f, c = 0.5f;
    for (int i = 0; i < turns; ++i)
        asm volatile(HTGS_R64(HTGS_OP_SWAP) : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7), "+v"(c) : "v"(c));
    out[blockIdx.x * 256 + threadIdx.x] = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7 + c;
}
struct IssueCase { const char *name; void (*kernel)(float *, int); };
static const IssueCase kIssueCases[] = {
    { "v_fma_f32", issue_fma_kernel }, { "v_add_f32", issue_add_kernel }, { "v_mul_f32", issue_mul_kernel }, { "v_mov_b32", issue_mov_kernel },
    { "v_add_u32", issue_addu_kernel }, { "v_min_f32", issue_min_kernel }, { "v_cmp_lt_f32", issue_cmp_kernel },
    { "v_cndmask_b32", issue_cnd_kernel }, { "v_rndne_f32", issue_rnd_kernel }, { "v_cvt_i32_f32", issue_cvt_kernel },
    { "v_lshl_add_u32", issue_lshladd_kernel }, { "v_rcp_f32", issue_rcp_kernel }, { "v_exp_f32", issue_exp_kernel }, { "v_swap_b32", issue_swap_kernel },
};
constexpr int kIssueCaseCount = (int)(sizeof(kIssueCases) / sizeof(kIssueCases[0]));

}  // namespace htgs

using namespace htgs;

extern "C" const char *htgs_issue_cost_name(int instruction)
{
    return instruction >= 0 && instruction < kIssueCaseCount ? kIssueCases[instruction].name : nullptr;
}

extern "C" int htgs_issue_cost_launch(int instruction, float *out, int n_blocks, int turns, void *stream)
{
    if (instruction < 0 || instruction >= kIssueCaseCount || !out || n_blocks <= 0 || turns <= 0)
        return fail(HTGS_ERR_ARGUMENT, "htgs_issue_cost_launch: bad argument");
    hipLaunchKernelGGL(kIssueCases[instruction].kernel, dim3((unsigned)n_blocks), dim3(256), 0, (hipStream_t)stream, out, turns);
    return check_launch("issue_cost");
}

extern "C" int htgs_check_reciprocal(unsigned long long *counts, void *stream)
{
    if (!counts) return fail(HTGS_ERR_ARGUMENT, "htgs_check_reciprocal: null pointer");
    hipLaunchKernelGGL(check_reciprocal_kernel, dim3(4096), dim3(256), 0, (hipStream_t)stream, counts);
    return check_launch("check_reciprocal");
}

extern "C" int htgs_copy_bytes(void *dst, const void *src, size_t n_bytes, void *stream)
{
    if (!dst || !src || (n_bytes & 15)) return fail(HTGS_ERR_ARGUMENT, "htgs_copy_bytes: null pointer or size not a multiple of 16");
    const size_t n = n_bytes / 16;
    if (n == 0) return HTGS_OK;
    if ((n + 255) / 256 > 0x7fffffffull) return fail(HTGS_ERR_ARGUMENT, "htgs_copy_bytes: too large");
    hipLaunchKernelGGL(copy_bytes_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint4 *)src, (uint4 *)dst, n);
    return check_launch("copy_bytes");
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
    htgs_frame t = *f;
    t.scale_modifier = 1.0f;   // the training preprocess has no scale modifier (R/include/hybrid_blend/kernels/forward.cuh:10-76)
    int rc = htgs_preprocess(&t);
    if (rc != HTGS_OK) return rc;
    return htgs_scan_offsets(&t);
}

extern "C" int htgs_forward_back(const htgs_frame *f, int *selector)
{
    if (!f || !selector) return fail(HTGS_ERR_ARGUMENT, "htgs_forward_back: null argument");
    int rc = htgs_create_instances(f);
    if (rc != HTGS_OK) return rc;
    rc = htgs_sort_instances(f, selector);
    if (rc != HTGS_OK) return rc;
    rc = htgs_extract_ranges(f, *selector);
    if (rc != HTGS_OK) return rc;
    return htgs_blend_forward(f, *selector);
}
