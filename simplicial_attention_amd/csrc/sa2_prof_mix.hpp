// Profiling build only (libsa2_prof.so): what this chip sustains on a given instruction mix.
//
// A loop of independent v_mfma_f32_32x32x16_bf16 (two waves per SIMD, operands in registers) with, per MFMA, NV
// plain VALU instructions, NE exponentials and NL LDS fragment reads of 1 KiB per wave.  The rate depends on the
// operands' values: with random bf16 operands the chip lowers its clock to stay inside its power limit, with zeros
// or constants it holds the nominal clock.  The attention kernels' fractions of the nominal MFMA peak are to be read
// beside these figures: their instruction mixes (five to seven VALU instructions, one exponential every second MFMA
// and one and a half to two LDS fragment reads per MFMA) bound them much as they bound this loop.
#pragma once

#include "sa2_common.hpp"

namespace sa2 {

template <int NV, int NE, int NL>
__global__ __launch_bounds__(512) void prof_mix_kernel(const char *src, float *out, int iters, unsigned long long *clocks) {
    __shared__ __attribute__((aligned(16))) char lds[64 * 1024];
    const int tid = threadIdx.x, lane = tid & 63;
    for (int x = tid; x < 4096; x += 512) reinterpret_cast<u32x4 *>(lds)[x] = ld_global16(src + x * 16);   // src holds 64 KiB
    __syncthreads();
    u32x4 a[4], b[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        a[k] = ld_global16(src + (k * 64 + lane) * 16);
        b[k] = ld_global16(src + 8192 + (k * 64 + lane) * 16);
    }
    f32x16 acc[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) acc[k] = zero16();
    float v[8];
#pragma unroll
    for (int x = 0; x < 8; ++x) v[x] = bf16_lo(a[x & 3][x >> 2]) * 0.001f;
    u32x4 fr = {0u, 0u, 0u, 0u};
    const char *lp = lds + lane * 16;
    const unsigned long long c0 = clock64(), w0 = wall_clock64();
    for (int u = 0; u < iters; ++u) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                acc[k] = mfma32(a[(k + r) & 3], b[k], acc[k]);
#pragma unroll
                for (int x = 0; x < NV; ++x) v[x & 7] = v[x & 7] * 1.0001f + v[(x + 3) & 7];
#pragma unroll
                for (int x = 0; x < NE; ++x) v[x & 7] = fast_exp2(v[x & 7]) * 0.5f;
#pragma unroll
                for (int x = 0; x < NL; ++x) {
                    const u32x4 t = ld_lds16(lp + ((4 * r + k + x) & 15) * 1024);
                    fr[0] ^= t[0];
                    fr[1] ^= t[1];
                    fr[2] ^= t[2];
                    fr[3] ^= t[3];
                }
                __builtin_amdgcn_sched_barrier(0);
            }
    }
    const unsigned long long c1 = clock64(), w1 = wall_clock64();
    if (blockIdx.x == 0 && tid == 0) {
        clocks[0] = c1 - c0;       // shader clock
        clocks[1] = w1 - w0;       // constant 100 MHz clock
    }
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[k][r];
#pragma unroll
    for (int x = 0; x < 8; ++x) s += v[x];
    s += as_f32(fr[0] ^ fr[1] ^ fr[2] ^ fr[3]);
    out[blockIdx.x * 512 + tid] = s;
}

}  // namespace sa2
