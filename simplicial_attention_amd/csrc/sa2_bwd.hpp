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

// ------------------------------------------------------------------------------------
// dK1/dV1: workgroup = 128 rows j of one (batch, kv head); wave w owns rows
// [32w, 32w+32), lane column = j, and keeps its K1/V1 fragments in registers as B
// operands.  The workgroup walks "steps" = (query head of the group, 32-row query
// tile, offset dlt).  For every step the 256 threads build A = q*k2 and B = do*v2
// (32 x D each) once, row-major in LDS; the row-major fragments feed S and dP, and
// ds_read_b64_tr_b16 reads of the same tiles feed dV1^T += B^T P and dK1^T += A^T dS.
// Tiles are double buffered: the products of step s+1 are written while step s
// computes, their global loads are issued one step earlier still.
// ------------------------------------------------------------------------------------
template <int D>
struct Dkv1Cfg {
    static constexpr int TILE = 32 * tile_pitch<D>();
    static constexpr int AS = 0;                 // A tile
    static constexpr int BS = TILE;              // B tile
    static constexpr int LSE = 2 * TILE;         // 32 floats: lse * log2e (+inf for dead rows)
    static constexpr int DEL = LSE + 32 * 4;     // 32 floats: delta
    static constexpr int BYTES = DEL + 32 * 4;
    static constexpr int LPT = 32 * D / 8 / 256; // 16-byte pieces per thread and tensor
};

template <int D>
__global__ __launch_bounds__(256, 1) void bwd_dkv1_kernel(KParams p) {
    constexpr int KS = D / 16, DT = D / 32, PPR = D / 8, PITCH = tile_pitch<D>();
    using L = Dkv1Cfg<D>;
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
        pin_acc(dk1[dt]);
        pin_acc(dv1[dt]);
    }

    const int it_begin = j0 / 32;
    const int last_i = (j0 + 127 + p.w1 - 1 < N - 1) ? j0 + 127 + p.w1 - 1 : N - 1;
    const int it_end = last_i / 32;
    const bool wave_active = jw < N;
    const int wit_lo = jw / 32;
    const int wit_hi = ((jw + 31 + p.w1 - 1 < N - 1) ? jw + 31 + p.w1 - 1 : N - 1) / 32;
    const float c2 = p.scale_log2e;
    const int r_lane = c * PITCH + 16 * hf;
    const int t_lane = tr_lane_off<D>(lane);

    // ---- step iterator (g, it, dlt) for the loads, which run two steps ahead
    struct Step {
        int g, it, dlt;
    };
    auto dmax_of = [&](int it) { return (p.w2 - 1 < 32 * it + 31) ? p.w2 - 1 : 32 * it + 31; };
    auto next_step = [&](Step &s) {
        if (++s.dlt > dmax_of(s.it)) {
            s.dlt = 0;
            if (++s.it > it_end) {
                s.it = it_begin;
                ++s.g;
            }
        }
    };
    int nsteps = 0;
    for (int it = it_begin; it <= it_end; ++it) nsteps += dmax_of(it) + 1;
    nsteps *= p.G;

    // ---- operand staging: each thread owns LPT 16-byte pieces of the A and of the B tile
    u32x4 lq[L::LPT], lk[L::LPT], lo[L::LPT], lv[L::LPT];
    float l_lse = 0.f, l_del = 0.f;
    int st_off[L::LPT];
#pragma unroll
    for (int x = 0; x < L::LPT; ++x) st_off[x] = ((x * 256 + tid) / PPR) * PITCH + ((x * 256 + tid) % PPR) * 16;
    auto issue_loads = [&](const Step &s) {
        const int h = hk * p.G + s.g;
        const char *qg = p.q.ptr + b * p.q.sb + h * p.q.sh;
        const char *dog = p.dout.ptr + b * p.dout.sb + h * p.dout.sh;
#pragma unroll
        for (int x = 0; x < L::LPT; ++x) {
            const int pc = x * 256 + tid;
            int i = 32 * s.it + pc / PPR;
            int kr = i - s.dlt;
            i = i < N ? i : N - 1;
            kr = kr < 0 ? 0 : (kr < N ? kr : N - 1);
            const int col = (pc % PPR) * 16;
            lq[x] = ld_global16(qg + (int64_t)i * p.q.sn + col);
            lk[x] = ld_global16(k2g + (int64_t)kr * p.k2.sn + col);
            lo[x] = ld_global16(dog + (int64_t)i * p.dout.sn + col);
            lv[x] = ld_global16(v2g + (int64_t)kr * p.v2.sn + col);
        }
        if (tid < 32) {
            const int i = 32 * s.it + tid;
            const bool valid = i < N && i - s.dlt >= 0;
            const int icl = i < N ? i : N - 1;
            l_lse = valid ? p.lse[((int64_t)b * p.H + h) * N + icl] * kLog2e : INFINITY;
            l_del = valid ? p.delta[((int64_t)b * p.H + h) * N + icl] : 0.f;
        }
    };
    auto write_stage = [&](int buf) {
        char *stage = lds + buf * L::BYTES;
#pragma unroll
        for (int x = 0; x < L::LPT; ++x) {
            *reinterpret_cast<u32x4 *>(stage + L::AS + st_off[x]) = mul_bf16x8(lq[x], lk[x]);
            *reinterpret_cast<u32x4 *>(stage + L::BS + st_off[x]) = mul_bf16x8(lo[x], lv[x]);
        }
        if (tid < 32) {
            reinterpret_cast<float *>(stage + L::LSE)[tid] = l_lse;
            reinterpret_cast<float *>(stage + L::DEL)[tid] = l_del;
        }
    };

    Step ld = {0, it_begin, 0};   // next step to load
    Step cur = {0, it_begin, 0};  // step being computed
    issue_loads(ld);
    next_step(ld);
    write_stage(0);
    if (nsteps > 1) {
        issue_loads(ld);
        next_step(ld);
    }

    for (int s = 0; s < nsteps; ++s) {
        __syncthreads();
        if (s + 1 < nsteps) write_stage((s + 1) & 1);
        if (s + 2 < nsteps) {
            issue_loads(ld);
            next_step(ld);
        }
        const char *buf = lds + (s & 1) * L::BYTES;
        const int it = cur.it;
        next_step(cur);
        if (!wave_active || it < wit_lo || it > wit_hi) continue;

        // ---- S[i,j], dP[i,j]: rows = query rows of the tile, column = j
        f32x16 X = zero16(), dP = zero16();
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            X = mfma32(ld_lds16(buf + L::AS + r_lane + 32 * kk), k1f[kk], X);
            dP = mfma32(ld_lds16(buf + L::BS + r_lane + 32 * kk), v1f[kk], dP);
        }
        float dls[16];
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            const float4 l4 = *reinterpret_cast<const float4 *>(buf + L::LSE + (8 * a4 + 4 * hf) * 4);
            const float4 d4 = *reinterpret_cast<const float4 *>(buf + L::DEL + (8 * a4 + 4 * hf) * 4);
            X[4 * a4] = X[4 * a4] * c2 - l4.x;
            X[4 * a4 + 1] = X[4 * a4 + 1] * c2 - l4.y;
            X[4 * a4 + 2] = X[4 * a4 + 2] * c2 - l4.z;
            X[4 * a4 + 3] = X[4 * a4 + 3] * c2 - l4.w;
            dls[4 * a4] = d4.x;
            dls[4 * a4 + 1] = d4.y;
            dls[4 * a4 + 2] = d4.z;
            dls[4 * a4 + 3] = d4.w;
        }
        const bool full = (jw + 31 <= 32 * it) && (jw + p.w1 > 32 * it + 31);
        if (!full) {
            const int base = 32 * it + 4 * hf - j;   // i - j for register 0
#pragma unroll
            for (int rr = 0; rr < 16; ++rr) {
                const bool ok = (unsigned)(base + 8 * (rr >> 2) + (rr & 3)) < (unsigned)p.w1;
                X[rr] = ok ? X[rr] : -INFINITY;
            }
        }
        u32x4 pb[2], dsb[2];
#pragma unroll
        for (int rr = 0; rr < 16; rr += 2) {
            float p0 = fast_exp2(X[rr]);
            float p1 = fast_exp2(X[rr + 1]);
            pb[rr >> 3][(rr & 7) >> 1] = pack_bf16(p0, p1);
            dsb[rr >> 3][(rr & 7) >> 1] = pack_bf16(p0 * (dP[rr] - dls[rr]), p1 * (dP[rr + 1] - dls[rr + 1]));
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int k2s = 0; k2s < 2; ++k2s) {
                u32x2 blo = lds_read_tr<D>(buf + L::BS + t_lane, 16 * k2s, 32 * dt);
                u32x2 bhi = lds_read_tr<D>(buf + L::BS + t_lane, 16 * k2s + 8, 32 * dt);
                u32x2 alo = lds_read_tr<D>(buf + L::AS + t_lane, 16 * k2s, 32 * dt);
                u32x2 ahi = lds_read_tr<D>(buf + L::AS + t_lane, 16 * k2s + 8, 32 * dt);
                u32x4 bfr = {blo[0], blo[1], bhi[0], bhi[1]};
                u32x4 afr = {alo[0], alo[1], ahi[0], ahi[1]};
                dv1[dt] = mfma32(bfr, pb[k2s], dv1[dt]);
                dk1[dt] = mfma32(afr, dsb[k2s], dk1[dt]);
            }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            pin_acc(dk1[dt]);
            pin_acc(dv1[dt]);
        }
    }

    if (!j_ok) return;
    store_row<DT>(p.dk1.ptr + b * p.dk1.sb + (int64_t)j * p.dk1.sn + hk * p.dk1.sh + 16 * hf * 2, dk1, p.scale);
    store_row<DT>(p.dv1.ptr + b * p.dv1.sb + (int64_t)j * p.dv1.sn + hk * p.dv1.sh + 16 * hf * 2, dv1, 1.f);
}

}  // namespace sa2
