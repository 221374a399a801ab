// Backward kernels of sliding-window 2-simplicial attention for gfx950.
//
// The reference computes the backward with two_simplicial_attn_bwd_kv1_kernel and two
// passes of two_simplicial_attn_bwd_kv2q_kernel
// (simplicial_attention/triton_two_simplicial_attention.py:298-503, 515-712) plus fp32
// atomics for a dQ that is later overwritten.  Here the backward is atomic-free:
//   delta_kernel      delta_i = sum_d o_i do_i                      (:230-286 there; this file)
//   bwd_q_kernel      owns query rows i    -> dQ, partial dK2/dV2   (sa2_bwd_q.hpp)
//   dk2_dv2_combine   sums the partial rows -> dK2, dV2             (sa2_bwd_q.hpp)
//   bwd_kv8_kernel    owns rows j of K1/V1 -> dK1, dV1              (sa2_bwd_kv8.hpp)
// With dlt = i - k, A = q_i * k2_{i-dlt} and B = do_i * v2_{i-dlt} (VALU, bf16):
//   S = A K1^T, dP = B V1^T, P = exp(scale*S - lse_i), dS = P (dP - delta_i)
//   G = dS K1 :  dq_i  += scale k2_{i-dlt} G_i     dk2_{i-dlt} += scale q_i G_i
//   T = P  V1 :  dv2_{i-dlt} += do_i T_i
//   dV1 += P^T B,  dK1 += scale dS^T A
#pragma once

#include "sa2_common.hpp"
#include "sa2_lds.hpp"

namespace sa2 {

// ------------------------------------------------------------------------------------
// delta[b,h,i] = sum_d (out + out_residual) * dout
// ------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void delta_kernel(KParams p) {
    constexpr int LP = D / 8;  // lanes per row, 16 bytes each
    const int64_t rows = (int64_t)p.B * p.H * p.N;
    const int64_t row = (int64_t)blockIdx.x * (256 / LP) + threadIdx.x / LP;
    const int piece = threadIdx.x % LP;
    float s = 0.f;
    const bool ok = row < rows;
    if (ok) {
        const int i = (int)(row % p.N);
        const int h = (int)((row / p.N) % p.H);
        const int b = (int)(row / ((int64_t)p.N * p.H));
        u32x4 o = ld_global16(p.o.ptr + b * p.o.sb + (int64_t)i * p.o.sn + h * p.o.sh + piece * 16);
        u32x4 g = ld_global16(p.dout.ptr + b * p.dout.sb + (int64_t)i * p.dout.sn + h * p.dout.sh + piece * 16);
#pragma unroll
        for (int w = 0; w < 4; ++w) s += bf16_lo(o[w]) * bf16_lo(g[w]) + bf16_hi(o[w]) * bf16_hi(g[w]);
        if (p.o_lo.ptr) {
            u32x4 r = ld_global16(p.o_lo.ptr + b * p.o_lo.sb + (int64_t)i * p.o_lo.sn + h * p.o_lo.sh + piece * 16);
#pragma unroll
            for (int w = 0; w < 4; ++w) s += bf16_lo(r[w]) * bf16_lo(g[w]) + bf16_hi(r[w]) * bf16_hi(g[w]);
        }
    }
#pragma unroll
    for (int off = LP / 2; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    if (ok && piece == 0) p.delta[row] = s;
}

}  // namespace sa2
