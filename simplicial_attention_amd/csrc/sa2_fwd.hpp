// Forward kernel of sliding-window 2-simplicial attention for gfx950.
//
// Replaces two_simplicial_attn_fwd_kernel of the reference
// (simplicial_attention/triton_two_simplicial_attention.py:58-228) with a different
// decomposition.  The second key set is addressed by its offset dlt = i - k in
// [0, w2): for a fixed offset every query row meets exactly one k2/v2 row, so
//     A[i,:]  = q_i * k2_{i-dlt}                  (VALU, rounded to bf16)
//     S^T     = K1 A^T                            (MFMA, j x i, banded in j)
//     P^T     = exp2(S^T * scale*log2e - m_i)     (online softmax over (j, dlt))
//     T^T    += V1^T P^T                          (MFMA, d x i)
//     O_i    += v2_{i-dlt} * T_i                  (VALU, once per offset and K1/V1 chunk)
// Computing the transposed logits puts one query row in one lane column, so the
// softmax row reductions are in-lane plus one cross-half exchange, and the
// accumulator layout of P^T is directly the B operand of the second GEMM.
//
// Work split: one workgroup = 128 query rows of one (batch, head); wave w owns rows
// [32w, 32w+32).  K1 rows and a transposed copy of V1 rows are staged in LDS in
// chunks of 128 rows that all four waves share; each wave visits only the 32-row
// tiles its own band (i-w1, i] touches and masks only the two boundary tiles.
#pragma once

#include "sa2_common.hpp"

namespace sa2 {

template <int D>
struct FwdCfg {
    static constexpr int KS = D / 16;          // k-steps of the logit GEMM
    static constexpr int DT = D / 32;          // 32-wide d tiles of the value GEMM
    static constexpr int CT = kChunkTiles;     // 32-row tiles per staged chunk (= waves)
    static constexpr int PK = row_pitch(D);    // LDS pitch of a K1 row, bytes
    static constexpr int PV = kChunkPitchT;    // LDS pitch of a V1^T row, bytes
    static constexpr int K1_BYTES = kChunkRows * PK;
    static constexpr int V1T_BYTES = D * PV;
};

template <int D>
__global__ __launch_bounds__(256, 2) void fwd_kernel(KParams p) {
    using C = FwdCfg<D>;
    __shared__ __attribute__((aligned(16))) char k1s[C::K1_BYTES];
    __shared__ __attribute__((aligned(16))) char v1t[C::V1T_BYTES];

    const int N = p.N;
    const int ntile = (N + 127) / 128;
    const int item = xcd_contiguous(blockIdx.x, gridDim.x);
    const int tile = ntile - 1 - item % ntile;   // longest windows first
    const int bh = item / ntile;
    const int h = bh % p.H, b = bh / p.H;
    const int hk = h / p.G;

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = lane & 31, hf = lane >> 5;
    const int i0 = tile * 128;
    const int iw = i0 + 32 * wave;
    const int i = iw + c;
    const bool row_ok = i < N;
    const int ic = row_ok ? i : N - 1;

    const char *qrow = p.q.ptr + b * p.q.sb + (int64_t)ic * p.q.sn + h * p.q.sh;
    const char *k1g = p.k1.ptr + b * p.k1.sb + hk * p.k1.sh;
    const char *v1g = p.v1.ptr + b * p.v1.sb + hk * p.v1.sh;
    const char *k2g = p.k2.ptr + b * p.k2.sb + hk * p.k2.sh;
    const char *v2g = p.v2.ptr + b * p.v2.sb + hk * p.v2.sh;

    u32x4 qf[C::KS];
#pragma unroll
    for (int kk = 0; kk < C::KS; ++kk) qf[kk] = ld_global16(qrow + (16 * kk + 8 * hf) * 2);

    f32x16 acc[C::DT], T[C::DT];
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt) acc[dt] = zero16();
    float m = -INFINITY, l = 0.f, acc_scale = 1.f;

    const bool wave_active = iw < N;
    const int wt_hi = iw / 32;                                   // diagonal tile of this wave
    const int wt_lo = (iw - p.w1 + 1 > 0 ? iw - p.w1 + 1 : 0) / 32;
    const int t_begin = (i0 - p.w1 + 1 > 0 ? i0 - p.w1 + 1 : 0) / 32;
    const int t_end = ((i0 + 127 < N - 1) ? i0 + 127 : N - 1) / 32;
    const int dmax = (p.w2 - 1 < iw + 31) ? p.w2 - 1 : iw + 31;
    const float c2 = p.scale_log2e;
    const int vrow = dmap_row(c);

    for (int ct0 = t_begin; ct0 <= t_end; ct0 += C::CT) {
        __syncthreads();
        stage_rows<D>(k1s, k1g, p.k1.sn, ct0 * 32, N);
        stage_rows_transposed<D>(v1t, v1g, p.v1.sn, ct0 * 32, N);
        __syncthreads();
        const int tl = ct0 > wt_lo ? ct0 : wt_lo;
        const int th = (ct0 + C::CT - 1 < wt_hi) ? ct0 + C::CT - 1 : wt_hi;
        if (!wave_active || tl > th) continue;

        for (int dlt = 0; dlt <= dmax; ++dlt) {
            const int kr = i - dlt;
            const bool col_ok = row_ok && kr >= 0;
            const bool any_bad = wave_any(!col_ok);
            const int krc = kr < 0 ? 0 : (kr > N - 1 ? N - 1 : kr);
            const char *k2row = k2g + (int64_t)krc * p.k2.sn;
            u32x4 A[C::KS];
#pragma unroll
            for (int kk = 0; kk < C::KS; ++kk) A[kk] = mul_bf16x8(qf[kk], ld_global16(k2row + (16 * kk + 8 * hf) * 2));
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt) T[dt] = zero16();

            for (int t = tl; t <= th; ++t) {
                const int lt = t - ct0;
                f32x16 S = zero16();
                const char *kbase = k1s + (32 * lt + c) * C::PK + 8 * hf * 2;
#pragma unroll
                for (int kk = 0; kk < C::KS; ++kk) S = mfma32(ld_lds16(kbase + 32 * kk), A[kk], S);

                const bool full = !any_bad && (t < wt_hi) && (32 * t + p.w1 > iw + 31);
                if (!full) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        int j = 32 * t + 8 * (r >> 2) + 4 * hf + (r & 3);
                        bool ok = col_ok && (j <= i) && (j + p.w1 > i);
                        S[r] = ok ? S[r] : -INFINITY;
                    }
                }
                float tmax = S[0];
#pragma unroll
                for (int r = 1; r < 16; ++r) tmax = fmaxf(tmax, S[r]);
                tmax *= c2;
                tmax = fmaxf(tmax, other_half(tmax));
                const float m_new = fmaxf(m, tmax);
                if (wave_any(m_new > m)) {
                    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                    const float alpha = fast_exp2(m - m_use);
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                        for (int r = 0; r < 16; ++r) T[dt][r] *= alpha;
                    l *= alpha;
                    acc_scale *= alpha;
                    m = m_new;
                }
                const float m_use = (m == -INFINITY) ? 0.f : m;
                u32x4 pb[2];
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    float p0 = fast_exp2(S[r] * c2 - m_use);
                    float p1 = fast_exp2(S[r + 1] * c2 - m_use);
                    l += p0 + p1;
                    pb[r >> 3][(r & 7) >> 1] = pack_bf16(p0, p1);
                }
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt) {
                    const char *vbase = v1t + (32 * dt + vrow) * C::PV + (32 * lt + 8 * hf) * 2;
                    T[dt] = mfma32(ld_lds16(vbase), pb[0], T[dt]);
                    T[dt] = mfma32(ld_lds16(vbase + 32), pb[1], T[dt]);
                }
            }

            // O_i += v2_{i-dlt} * T_i ; lane holds d = 32*dt + 16*hf + r
            const char *v2row = v2g + (int64_t)krc * p.v2.sn + 16 * hf * 2;
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt) {
                u32x4 va = ld_global16(v2row + dt * 64);
                u32x4 vb = ld_global16(v2row + dt * 64 + 16);
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    acc[dt][2 * w] = acc[dt][2 * w] * acc_scale + bf16_lo(va[w]) * T[dt][2 * w];
                    acc[dt][2 * w + 1] = acc[dt][2 * w + 1] * acc_scale + bf16_hi(va[w]) * T[dt][2 * w + 1];
                    acc[dt][8 + 2 * w] = acc[dt][8 + 2 * w] * acc_scale + bf16_lo(vb[w]) * T[dt][8 + 2 * w];
                    acc[dt][8 + 2 * w + 1] = acc[dt][8 + 2 * w + 1] * acc_scale + bf16_hi(vb[w]) * T[dt][8 + 2 * w + 1];
                }
            }
            acc_scale = 1.f;
        }
    }

    if (!row_ok) return;
    const float l_tot = l + other_half(l);
    const float inv = 1.f / l_tot;
    char *orow = p.o.ptr + b * p.o.sb + (int64_t)i * p.o.sn + h * p.o.sh + 16 * hf * 2;
    char *rrow = p.o_lo.ptr ? p.o_lo.ptr + b * p.o_lo.sb + (int64_t)i * p.o_lo.sn + h * p.o_lo.sh + 16 * hf * 2 : nullptr;
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt) {
        u32x4 oa, ob, ra, rb;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float x0 = acc[dt][2 * w] * inv, x1 = acc[dt][2 * w + 1] * inv;
            const float y0 = acc[dt][8 + 2 * w] * inv, y1 = acc[dt][8 + 2 * w + 1] * inv;
            oa[w] = pack_bf16(x0, x1);
            ob[w] = pack_bf16(y0, y1);
            ra[w] = pack_bf16(x0 - bf16_lo(oa[w]), x1 - bf16_hi(oa[w]));
            rb[w] = pack_bf16(y0 - bf16_lo(ob[w]), y1 - bf16_hi(ob[w]));
        }
        st_global16(orow + dt * 64, oa);
        st_global16(orow + dt * 64 + 16, ob);
        if (rrow) {
            st_global16(rrow + dt * 64, ra);
            st_global16(rrow + dt * 64 + 16, rb);
        }
    }
    if (hf == 0) p.lse[((int64_t)b * p.H + h) * N + i] = (m + __builtin_amdgcn_logf(l_tot)) * kLn2;
}

}  // namespace sa2
