// Pieces shared by the inference, training-forward and backward blend kernels.
#pragma once

#include "common.h"

namespace htgs {

template <int N>
struct Stage {
    float4 v1[N], v2[N], v4[N], mt3[N], col[N];
};

// Stages one Gaussian record per lane.
template <int N>
__device__ __forceinline__ void stage_load(Stage<N> &st, const float4 *__restrict__ prim, const uint32_t *__restrict__ inst,
                                           uint32_t fetch, uint32_t last, int slot, uint32_t *idx_out)
{
    if (fetch < last) {
        const uint32_t g = inst[fetch];
        const float4 *rec = prim + (size_t)g * (HTGS_PRIM_FLOATS / 4);
        st.v1[slot] = rec[0];
        st.v2[slot] = rec[1];
        st.v4[slot] = rec[2];
        st.mt3[slot] = rec[3];
        st.col[slot] = rec[4];
        if (idx_out) idx_out[slot] = g;
    }
}

// exchange two VGPRs in the active lanes (one instruction instead of a select pair)
__device__ __forceinline__ void vswap(float &a, float &b) { asm volatile("v_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }
__device__ __forceinline__ void vswap(uint32_t &a, uint32_t &b) { asm volatile("v_swap_b32 %0, %1" : "+v"(a), "+v"(b)); }

}  // namespace htgs
