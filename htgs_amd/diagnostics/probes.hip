// Measurement probes, kept out of the rasterizer library: a plain device-to-device copy that calibrates the HBM
// traffic counters, and micro-kernels that measure how long one wave64 vector instruction holds a SIMD.  Built into
// libhtgs_probes.so (declarations: include/htgs_probes.h); only the benchmark loads it.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/htgs_probes.h"

namespace {

__global__ void __launch_bounds__(256) copy_bytes_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

// Issue cost of single vector instructions: every kernel below runs 64 copies of one instruction per loop turn over
// eight registers (the copies of one register depend on each other, the eight registers do not).
#define PROBE_R8(op) op(0) op(1) op(2) op(3) op(4) op(5) op(6) op(7)
#define PROBE_R64(op) PROBE_R8(op) PROBE_R8(op) PROBE_R8(op) PROBE_R8(op) PROBE_R8(op) PROBE_R8(op) PROBE_R8(op) PROBE_R8(op)
#define PROBE_ISSUE_KERNEL(name, op)                                                                                              \
    __global__ void __launch_bounds__(256) name(float *__restrict__ out, int turns)                                              \
    {                                                                                                                            \
        float a0 = threadIdx.x * 1e-3f, a1 = a0 + 1.0f, a2 = a0 + 2.0f, a3 = a0 + 3.0f, a4 = a0 + 4.0f, a5 = a0 + 5.0f,            \
              a6 = a0 + 6.0f, a7 = a0 + 7.0f;                                                                                    \
        const float m = 1.0001f, c = 0.5f;                                                                                       \
        for (int i = 0; i < turns; ++i)                                                                                          \
            asm volatile("s_mov_b64 s[40:41], 0x5555\n" PROBE_R64(op)                                                             \
                         : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7)                       \
                         : "v"(m), "v"(c)                                                                                        \
                         : "vcc", "s40", "s41");                                                                                 \
        out[blockIdx.x * 256 + threadIdx.x] = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7;                                             \
    }
#define PROBE_OP_FMA(i) "v_fma_f32 %" #i ", %" #i ", %8, %9\n"
#define PROBE_OP_ADD(i) "v_add_f32 %" #i ", %" #i ", %9\n"
#define PROBE_OP_MUL(i) "v_mul_f32 %" #i ", %" #i ", %8\n"
#define PROBE_OP_MOV(i) "v_mov_b32 %" #i ", %9\n"
#define PROBE_OP_ADDU(i) "v_add_u32 %" #i ", %" #i ", %9\n"
#define PROBE_OP_MIN(i) "v_min_f32 %" #i ", %" #i ", %9\n"
#define PROBE_OP_CMP(i) "v_cmp_lt_f32 vcc, %" #i ", %9\n"
#define PROBE_OP_CND(i) "v_cndmask_b32_e64 %" #i ", %" #i ", %9, s[40:41]\n"
#define PROBE_OP_RND(i) "v_rndne_f32 %" #i ", %" #i "\n"
#define PROBE_OP_CVT(i) "v_cvt_i32_f32 %" #i ", %" #i "\n"
#define PROBE_OP_LSHLADD(i) "v_lshl_add_u32 %" #i ", %" #i ", 3, %9\n"
#define PROBE_OP_RCP(i) "v_rcp_f32 %" #i ", %" #i "\n"
#define PROBE_OP_EXP(i) "v_exp_f32 %" #i ", %" #i "\n"
#define PROBE_OP_SWAP(i) "v_swap_b32 %" #i ", %9\n"
PROBE_ISSUE_KERNEL(issue_fma_kernel, PROBE_OP_FMA)
PROBE_ISSUE_KERNEL(issue_add_kernel, PROBE_OP_ADD)
PROBE_ISSUE_KERNEL(issue_mul_kernel, PROBE_OP_MUL)
PROBE_ISSUE_KERNEL(issue_mov_kernel, PROBE_OP_MOV)
PROBE_ISSUE_KERNEL(issue_addu_kernel, PROBE_OP_ADDU)
PROBE_ISSUE_KERNEL(issue_min_kernel, PROBE_OP_MIN)
PROBE_ISSUE_KERNEL(issue_cmp_kernel, PROBE_OP_CMP)
PROBE_ISSUE_KERNEL(issue_cnd_kernel, PROBE_OP_CND)
PROBE_ISSUE_KERNEL(issue_rnd_kernel, PROBE_OP_RND)
PROBE_ISSUE_KERNEL(issue_cvt_kernel, PROBE_OP_CVT)
PROBE_ISSUE_KERNEL(issue_lshladd_kernel, PROBE_OP_LSHLADD)
PROBE_ISSUE_KERNEL(issue_rcp_kernel, PROBE_OP_RCP)
PROBE_ISSUE_KERNEL(issue_exp_kernel, PROBE_OP_EXP)
// the same instruction with part of the wave switched off: does a wave64 instruction with an empty half (or with one
// row of sixteen lanes active) hold the SIMD for less time?
#define PROBE_MASKED_KERNEL(name, op, mask)                                                                                       \
    __global__ void __launch_bounds__(256) name(float *__restrict__ out, int turns)                                              \
    {                                                                                                                            \
        float a0 = threadIdx.x * 1e-3f, a1 = a0 + 1.0f, a2 = a0 + 2.0f, a3 = a0 + 3.0f, a4 = a0 + 4.0f, a5 = a0 + 5.0f,            \
              a6 = a0 + 6.0f, a7 = a0 + 7.0f;                                                                                    \
        const float m = 1.0001f, c = 0.5f;                                                                                       \
        for (int i = 0; i < turns; ++i)                                                                                          \
            asm volatile("s_mov_b64 s[40:41], exec\ns_mov_b64 exec, " mask "\n" PROBE_R64(op) "s_mov_b64 exec, s[40:41]\n"        \
                         : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7)                       \
                         : "v"(m), "v"(c)                                                                                        \
                         : "vcc", "s40", "s41");                                                                                 \
        out[blockIdx.x * 256 + threadIdx.x] = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7;                                             \
    }
PROBE_MASKED_KERNEL(issue_mov_half_kernel, PROBE_OP_MOV, "0xffffffff")
PROBE_MASKED_KERNEL(issue_mov_row_kernel, PROBE_OP_MOV, "0xffff")
PROBE_MASKED_KERNEL(issue_fma_half_kernel, PROBE_OP_FMA, "0xffffffff")
PROBE_MASKED_KERNEL(issue_cmp_half_kernel, PROBE_OP_CMP, "0xffffffff")
// (v_swap_b32 writes both operands: the second one is a ninth register of its own)
__global__ void __launch_bounds__(256) issue_swap_kernel(float *__restrict__ out, int turns)
{
    float a0 = threadIdx.x * 1e-3f, a1 = a0 + 1.0f, a2 = a0 + 2.0f, a3 = a0 + 3.0f, a4 = a0 + 4.0f, a5 = a0 + 5.0f, a6 = a0 + 6.0f,
          a7 = a0 + 7.0f, c = 0.5f;
    for (int i = 0; i < turns; ++i)
        asm volatile(PROBE_R64(PROBE_OP_SWAP) : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7), "+v"(c) : "v"(c));
    out[blockIdx.x * 256 + threadIdx.x] = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7 + c;
}
struct IssueCase { const char *name; void (*kernel)(float *, int); };
static const IssueCase kIssueCases[] = {
    { "v_fma_f32", issue_fma_kernel }, { "v_add_f32", issue_add_kernel }, { "v_mul_f32", issue_mul_kernel }, { "v_mov_b32", issue_mov_kernel },
    { "v_add_u32", issue_addu_kernel }, { "v_min_f32", issue_min_kernel }, { "v_cmp_lt_f32", issue_cmp_kernel },
    { "v_cndmask_b32", issue_cnd_kernel }, { "v_rndne_f32", issue_rnd_kernel }, { "v_cvt_i32_f32", issue_cvt_kernel },
    { "v_lshl_add_u32", issue_lshladd_kernel }, { "v_rcp_f32", issue_rcp_kernel }, { "v_exp_f32", issue_exp_kernel }, { "v_swap_b32", issue_swap_kernel },
    { "v_mov_b32, lanes 0-31 only", issue_mov_half_kernel }, { "v_mov_b32, lanes 0-15 only", issue_mov_row_kernel },
    { "v_fma_f32, lanes 0-31 only", issue_fma_half_kernel }, { "v_cmp_lt_f32, lanes 0-31 only", issue_cmp_half_kernel },
};
constexpr int kIssueCaseCount = (int)(sizeof(kIssueCases) / sizeof(kIssueCases[0]));


int launch_status()
{
    return hipGetLastError() == hipSuccess ? 0 : 3;
}

}  // namespace

extern "C" const char *htgs_probe_issue_cost_name(int instruction)
{
    return instruction >= 0 && instruction < kIssueCaseCount ? kIssueCases[instruction].name : nullptr;
}

extern "C" int htgs_probe_issue_cost_launch(int instruction, float *out, int n_blocks, int turns, void *stream)
{
    if (instruction < 0 || instruction >= kIssueCaseCount || !out || n_blocks <= 0 || turns <= 0)
        return 2;
    hipLaunchKernelGGL(kIssueCases[instruction].kernel, dim3((unsigned)n_blocks), dim3(256), 0, (hipStream_t)stream, out, turns);
    return launch_status();
}

extern "C" int htgs_probe_copy_bytes(void *dst, const void *src, size_t n_bytes, void *stream)
{
    if (!dst || !src || (n_bytes & 15)) return 2;
    const size_t n = n_bytes / 16;
    if (n == 0) return 0;
    if ((n + 255) / 256 > 0x7fffffffull) return 2;
    hipLaunchKernelGGL(copy_bytes_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint4 *)src, (uint4 *)dst, n);
    return launch_status();
}

