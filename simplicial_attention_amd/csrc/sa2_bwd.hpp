// Backward kernels of sliding-window 2-simplicial attention for gfx950.
//
// The reference computes the backward with two_simplicial_attn_bwd_kv1_kernel and two
// passes of two_simplicial_attn_bwd_kv2q_kernel
// (simplicial_attention/triton_two_simplicial_attention.py:298-503, 515-712) plus fp32
// atomics for a dQ that is later overwritten.  Here the backward is atomic-free:
//   delta_kernel      delta_i = sum_d o_i do_i                      (:230-286 there)
//   bwd_qk2_kernel    owns query rows i    -> dQ, partial dK2/dV2   (sa2_bwd_qk2.hpp)
//   dk2_dv2_combine   sums the partial rows -> dK2, dV2
//   bwd_dkv1_kernel   owns rows j of K1/V1 -> dK1, dV1
// With dlt = i - k, A = q_i * k2_{i-dlt} and B = do_i * v2_{i-dlt} (VALU, bf16):
//   S = A K1^T, dP = B V1^T, P = exp(scale*S - lse_i), dS = P (dP - delta_i)
//   G = dS K1 :  dq_i  += scale k2_{i-dlt} G_i     dk2_{i-dlt} += scale q_i G_i
//   T = P  V1 :  dv2_{i-dlt} += do_i T_i
//   dV1 += P^T B,  dK1 += scale dS^T A
#pragma once

#include "sa2_common.hpp"

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

// small GEMM helpers ---------------------------------------------------------------------

// acc(32x32, rows = staged rows, column = lane column) = sum_kk lds_rows[kk] * regfrag[kk]
template <int KS>
__device__ __forceinline__ f32x16 gemm_rows(const char *lds_row_base, const u32x4 (&frag)[KS]) {
    f32x16 s = zero16();
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) s = mfma32(ld_lds16(lds_row_base + 32 * kk), frag[kk], s);
    return s;
}

// acc[dt](rows = d, column = lane column) += transposed-chunk rows * packed C-layout fragment
template <int DT>
__device__ __forceinline__ void gemm_trans(f32x16 (&acc)[DT], const char *tbase, int pitch, const u32x4 (&pb)[2]) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const char *b = tbase + 32 * dt * pitch;
        acc[dt] = mfma32(ld_lds16(b), pb[0], acc[dt]);
        acc[dt] = mfma32(ld_lds16(b + 32), pb[1], acc[dt]);
    }
}

// ------------------------------------------------------------------------------------
// dK1/dV1: workgroup = 128 rows j of one (batch, kv head); lane column = j, K1/V1
// fragments stay in registers as B operands.  For every (32-row query tile, offset dlt)
// the workgroup builds A = q*k2 and B = do*v2 once in LDS, row-major (operands of S
// and dP) and transposed (operands of dV1^T += B^T P and dK1^T += A^T dS).
// ------------------------------------------------------------------------------------
template <int D>
struct Dkv1Buf {
    static constexpr int PK = row_pitch(D);
    static constexpr int PT = (32 + 8) * 2;
    static constexpr int AS = 0;
    static constexpr int BS = AS + 32 * PK;
    static constexpr int AT = BS + 32 * PK;
    static constexpr int BT = AT + D * PT;
    static constexpr int LSE = BT + D * PT;
    static constexpr int DEL = LSE + 32 * 4;
    static constexpr int BYTES = DEL + 32 * 4;
};

template <int D>
__global__ __launch_bounds__(256, 2) void bwd_dkv1_kernel(KParams p) {
    constexpr int KS = D / 16, DT = D / 32;
    using L = Dkv1Buf<D>;
    __shared__ __attribute__((aligned(16))) char lds[2 * L::BYTES];

    const int N = p.N;
    const int ntile = (N + 127) / 128;
    const int item = xcd_contiguous(blockIdx.x, gridDim.x);
    const int tile = item % ntile;
    const int bh = item / ntile;
    const int hk = bh % p.HK, b = bh / p.HK;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int c = lane & 31, hf = lane >> 5;
    const int j0 = tile * 128;
    const int jw = j0 + 32 * wave;
    const int j = jw + c;
    const bool j_ok = j < N;
    const int jc = j_ok ? j : N - 1;

    const char *k1row = p.k1.ptr + b * p.k1.sb + (int64_t)jc * p.k1.sn + hk * p.k1.sh;
    const char *v1row = p.v1.ptr + b * p.v1.sb + (int64_t)jc * p.v1.sn + hk * p.v1.sh;
    const char *k2g = p.k2.ptr + b * p.k2.sb + hk * p.k2.sh;
    const char *v2g = p.v2.ptr + b * p.v2.sb + hk * p.v2.sh;

    u32x4 k1f[KS], v1f[KS];
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
        k1f[kk] = ld_global16(k1row + (16 * kk + 8 * hf) * 2);
        v1f[kk] = ld_global16(v1row + (16 * kk + 8 * hf) * 2);
    }
    f32x16 dk1[DT], dv1[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        dk1[dt] = zero16();
        dv1[dt] = zero16();
    }

    const int it_begin = j0 / 32;
    const int last_i = (j0 + 127 + p.w1 - 1 < N - 1) ? j0 + 127 + p.w1 - 1 : N - 1;
    const int it_end = last_i / 32;
    const bool wave_active = jw < N;
    const int wit_lo = jw / 32;
    const int wit_hi = ((jw + 31 + p.w1 - 1 < N - 1) ? jw + 31 + p.w1 - 1 : N - 1) / 32;
    const float c2 = p.scale_log2e;
    const int vrow = dmap_row(c);
    constexpr int PPR = D / 8;

    int step = 0;
    for (int g = 0; g < p.G; ++g) {
        const int h = hk * p.G + g;
        const char *qg = p.q.ptr + b * p.q.sb + h * p.q.sh;
        const char *dog = p.dout.ptr + b * p.dout.sb + h * p.dout.sh;
        const float *lseg = p.lse + ((int64_t)b * p.H + h) * N;
        const float *delg = p.delta + ((int64_t)b * p.H + h) * N;

        for (int it = it_begin; it <= it_end; ++it) {
            const int dmax = (p.w2 - 1 < 32 * it + 31) ? p.w2 - 1 : 32 * it + 31;
            for (int dlt = 0; dlt <= dmax; ++dlt, ++step) {
                char *buf = lds + (step & 1) * L::BYTES;
                // ---- build A, B (row-major and transposed), lse, delta for this step
#pragma unroll
                for (int rep = 0; rep < 32 * PPR / 256; ++rep) {
                    const int idx = rep * 256 + tid;
                    const int il = idx / PPR, piece = idx % PPR;
                    const int i = 32 * it + il;
                    const int kr = i - dlt;
                    const bool valid = i < N && kr >= 0;
                    u32x4 a = {0u, 0u, 0u, 0u}, bb = {0u, 0u, 0u, 0u};
                    if (valid) {
                        a = mul_bf16x8(ld_global16(qg + (int64_t)i * p.q.sn + piece * 16),
                                       ld_global16(k2g + (int64_t)kr * p.k2.sn + piece * 16));
                        bb = mul_bf16x8(ld_global16(dog + (int64_t)i * p.dout.sn + piece * 16),
                                        ld_global16(v2g + (int64_t)kr * p.v2.sn + piece * 16));
                    }
                    *reinterpret_cast<u32x4 *>(buf + L::AS + il * L::PK + piece * 16) = a;
                    *reinterpret_cast<u32x4 *>(buf + L::BS + il * L::PK + piece * 16) = bb;
                    const int pos = kslot_pos(il);
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const int d = 8 * piece + 2 * w;
                        *reinterpret_cast<uint16_t *>(buf + L::AT + d * L::PT + pos * 2) = (uint16_t)(a[w] & 0xffffu);
                        *reinterpret_cast<uint16_t *>(buf + L::AT + (d + 1) * L::PT + pos * 2) = (uint16_t)(a[w] >> 16);
                        *reinterpret_cast<uint16_t *>(buf + L::BT + d * L::PT + pos * 2) = (uint16_t)(bb[w] & 0xffffu);
                        *reinterpret_cast<uint16_t *>(buf + L::BT + (d + 1) * L::PT + pos * 2) = (uint16_t)(bb[w] >> 16);
                    }
                }
                if (tid < 32) {
                    const int i = 32 * it + tid;
                    const bool valid = i < N && i - dlt >= 0;
                    reinterpret_cast<float *>(buf + L::LSE)[tid] = valid ? lseg[i] * kLog2e : INFINITY;
                    reinterpret_cast<float *>(buf + L::DEL)[tid] = valid ? delg[i] : 0.f;
                }
                __syncthreads();
                if (!wave_active || it < wit_lo || it > wit_hi) continue;

                // ---- S[i,j], dP[i,j]: rows = query rows of the tile, column = j
                const int roff = c * L::PK + 8 * hf * 2;
                f32x16 S = gemm_rows<KS>(buf + L::AS + roff, k1f);
                f32x16 dP = gemm_rows<KS>(buf + L::BS + roff, v1f);
                const bool full = (jw + 31 <= 32 * it) && (jw + p.w1 > 32 * it + 31);
                if (!full) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        int i = 32 * it + 8 * (r >> 2) + 4 * hf + (r & 3);
                        bool ok = (j <= i) && (j + p.w1 > i);
                        S[r] = ok ? S[r] : -INFINITY;
                    }
                }
                u32x4 pb[2], dsb[2];
#pragma unroll
                for (int a4 = 0; a4 < 4; ++a4) {
                    const float4 l4 = *reinterpret_cast<const float4 *>(buf + L::LSE + (8 * a4 + 4 * hf) * 4);
                    const float4 d4 = *reinterpret_cast<const float4 *>(buf + L::DEL + (8 * a4 + 4 * hf) * 4);
                    const int r = 4 * a4;
                    float p0 = fast_exp2(S[r] * c2 - l4.x);
                    float p1 = fast_exp2(S[r + 1] * c2 - l4.y);
                    float p2 = fast_exp2(S[r + 2] * c2 - l4.z);
                    float p3 = fast_exp2(S[r + 3] * c2 - l4.w);
                    pb[a4 >> 1][2 * (a4 & 1)] = pack_bf16(p0, p1);
                    pb[a4 >> 1][2 * (a4 & 1) + 1] = pack_bf16(p2, p3);
                    dsb[a4 >> 1][2 * (a4 & 1)] = pack_bf16(p0 * (dP[r] - d4.x), p1 * (dP[r + 1] - d4.y));
                    dsb[a4 >> 1][2 * (a4 & 1) + 1] = pack_bf16(p2 * (dP[r + 2] - d4.z), p3 * (dP[r + 3] - d4.w));
                }
                const int toff = vrow * L::PT + 8 * hf * 2;
                gemm_trans<DT>(dv1, buf + L::BT + toff, L::PT, pb);
                gemm_trans<DT>(dk1, buf + L::AT + toff, L::PT, dsb);
            }
        }
    }

    if (!j_ok) return;
    store_row<DT>(p.dk1.ptr + b * p.dk1.sb + (int64_t)j * p.dk1.sn + hk * p.dk1.sh + 16 * hf * 2, dk1, p.scale);
    store_row<DT>(p.dv1.ptr + b * p.dv1.sb + (int64_t)j * p.dv1.sn + hk * p.dv1.sh + 16 * hf * 2, dv1, 1.f);
}

}  // namespace sa2
