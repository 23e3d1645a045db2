// Small helpers shared by the vector-ALU register-tile kernels.
#pragma once

#include <hip/hip_runtime.h>

namespace simnets {

// Pointers in the constant address space: loads through them whose address is the same in every
// lane become scalar loads (s_load_dword*) and the values live in SGPRs.
#define SIMNETS_CONST_AS __attribute__((address_space(4)))

// Copies a wave-uniform value from its SGPR into a VGPR.  VALU instructions that read an SGPR
// operand issue at half the rate of all-VGPR ones on this chip (measured: 37 vs 64 T lane-ops/s), so
// a uniform operand that is used many times is moved once and then used from the VGPR.  The asm
// keeps the compiler from folding the SGPR back into the arithmetic.
__device__ __forceinline__ float to_vgpr(float uniform)
{
    float v;
    asm("v_mov_b32 %0, %1" : "=v"(v) : "s"(uniform));
    return v;
}

template <int N>
__device__ __forceinline__ void load_uniform(float (&dst)[N], const float SIMNETS_CONST_AS *src)
{
#pragma unroll
    for (int i = 0; i < N; ++i)
        dst[i] = src[i];
}

}  // namespace simnets
