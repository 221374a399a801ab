// Backward kernels for dQ/dK2 and for dV2, eight-wave variant (two waves per SIMD).
//
// Same shape as the eight-wave forward: one workgroup owns 32 query rows i of one
// (batch, head), in round r wave w handles the offset dlt = i - k = 8r + w, and all
// waves walk the same K1/V1 tiles through a double-buffered LDS ring.  A fused kernel
// (S, dP, T and G accumulators together) needs more than 256 registers per wave, which
// forces one wave per SIMD, and one wave cannot overlap its own MFMA and VALU work.  So
// the work is split into two passes that each fit two waves per SIMD:
//
//   pass DQ (DQ = true), with A = q_i * k2_{i-dlt}, B = do_i * v2_{i-dlt}:
//       S^T = K1 A^T,  dP^T = V1 B^T,  dS = P (dP - delta_i),  G^T += K1^T dS^T
//       dq_i += k2_{i-dlt} * G_i,   dk2_{i-dlt} += q_i * G_i
//   pass DV (DQ = false):
//       S^T = K1 A^T,  T^T += V1^T P^T,   dv2_{i-dlt} += do_i * T_i
//
// with P = exp2(S scale log2e - lse_i).  Both recompute S (5 contractions instead of 4).
// Sums over offsets go to fp32 LDS rows shared by the workgroup; a round's additions run
// in eight barrier-separated phases in which wave w owns the d-slice (w + phase) mod 8,
// so no two waves touch one element at a time and the order is fixed (bitwise
// reproducible, no atomics).  dk2/dv2 rows k in [i0-31, i0+31] go to the fp32 workspace
// that dk2_dv2_combine_kernel reduces (same layout as the fused kernel, 63 rows per tile).
// Offsets up to 32 only (the staged rows and the scatter rows are sized for a halo of 31).
#pragma once

#include <type_traits>

#include "sa2_common.hpp"
#include "sa2_lds.hpp"

namespace sa2 {

template <int D, bool DQ>
struct Q8Cfg {
    static constexpr int KS = D / 16;
    static constexpr int DT = D / 32;
    static constexpr int CT = DQ ? 1 : 2;             // 32-row tiles per ring stage (per barrier)
    static constexpr int PITCH = tile_pitch<D>();
    static constexpr int TILE = 32 * PITCH;           // a tile read row-major
    static constexpr int TPITCH = tr_pitch<D>();
    static constexpr int TRT = 32 * TPITCH;           // a tile read through transposed reads
    // sub-tile: DQ: [K1, read both ways: swizzled layout of sa2_lds.hpp][V1 row-major];  DV: [K1 row-major][V1 transposed-read]
    static constexpr int OFF_TR = DQ ? 0 : TILE;      // the tile read through transposed reads
    static constexpr int OFF_V = TRT;                 // DQ only
    static constexpr int SUB = TILE + TRT;
    static constexpr int STAGE = CT * SUB;
    static constexpr int RING = 2 * STAGE;
    static constexpr int HALO = 31;
    static constexpr int SROWS = 32 + HALO;           // k in [i0-31, i0+31]
    static constexpr int SPITCH = D + 4;              // floats per row of the fp32 rows
    static constexpr int DQS = RING;                  // dq rows [32][SPITCH]            (DQ only)
    static constexpr int SC = RING + (DQ ? 32 * SPITCH * 4 : 0);   // scatter rows [SROWS][SPITCH]
    static constexpr int QS = SC + SROWS * SPITCH * 4;             // q rows   [32][PITCH]
    static constexpr int DOS = QS + TILE;                          // do rows  [32][PITCH]
    static constexpr int K2S = DOS + TILE;                         // k2 rows  [SROWS][PITCH]
    static constexpr int V2S = K2S + SROWS * PITCH;                // v2 rows  [SROWS][PITCH]  (DQ only)
    static constexpr int LDS = DQ ? V2S + SROWS * PITCH : V2S;
    static constexpr int PIECES = 32 * D / 8;         // 16-byte pieces per tile
};

template <int NS, typename F>
__device__ __forceinline__ void with_slice(int s, F &&f) {
    static_assert(NS == 4 || NS == 8, "slice count");
    if constexpr (NS == 8) {
        switch (s & 7) {
            case 0: f(std::integral_constant<int, 0>{}); break;
            case 1: f(std::integral_constant<int, 1>{}); break;
            case 2: f(std::integral_constant<int, 2>{}); break;
            case 3: f(std::integral_constant<int, 3>{}); break;
            case 4: f(std::integral_constant<int, 4>{}); break;
            case 5: f(std::integral_constant<int, 5>{}); break;
            case 6: f(std::integral_constant<int, 6>{}); break;
            default: f(std::integral_constant<int, 7>{}); break;
        }
    } else {
        switch (s & 3) {
            case 0: f(std::integral_constant<int, 0>{}); break;
            case 1: f(std::integral_constant<int, 1>{}); break;
            case 2: f(std::integral_constant<int, 2>{}); break;
            default: f(std::integral_constant<int, 3>{}); break;
        }
    }
}

template <int D, bool DQ>
__global__ __launch_bounds__(512) void bwd_q8_kernel(KParams p, float *ws) {
    using C = Q8Cfg<D, DQ>;
    constexpr int KS = C::KS, DT = C::DT, CT = C::CT, PPR = D / 8, PITCH = C::PITCH;
    __shared__ __attribute__((aligned(16))) char lds[C::LDS];

    const int N = p.N;
    const int ntile = (N + 31) / 32;
    const int item = xcd_contiguous(blockIdx.x, gridDim.x);
    const int tile = ntile - 1 - item % ntile;
    const int bh = item / ntile;
    const int h = bh % p.H, b = bh / p.H;
    const int hk = h / p.G;

    const int tid = threadIdx.x;
    const int wave = wave_index(), lane = tid & 63;
    const int c = lane & 31, hf = lane >> 5;
    const int i0 = tile * 32;
    const int i = i0 + c;
    const bool row_ok = i < N;
    const int ic = row_ok ? i : N - 1;

    const char *k1g = p.k1.ptr + b * p.k1.sb + hk * p.k1.sh;
    const char *v1g = p.v1.ptr + b * p.v1.sb + hk * p.v1.sh;
    const float lse2 = p.lse[((int64_t)b * p.H + h) * N + ic] * kLog2e;
    float dl = 0.f;
    if constexpr (DQ) dl = p.delta[((int64_t)b * p.H + h) * N + ic];

    const int t_lo = (i0 - p.w1 + 1 > 0 ? i0 - p.w1 + 1 : 0) / 32;
    const int t_hi = i0 / 32;
    const int NT = t_hi - t_lo + 1;
    const int NC = (NT + CT - 1) / CT;
    const int nd = p.w2 < i0 + 32 ? p.w2 : i0 + 32;
    const int R = (nd + 7) / 8;                       // <= 4: offsets stay below 32
    const int U = R * NC;
    const float c2 = p.scale_log2e;

    // ---- ring staging: the first PIECES threads move one 16-byte piece of K1 and of V1 per tile
    const bool stager = tid < C::PIECES;
    const int st_row = tid / PPR, st_col = (tid % PPR) * 16;
    const int st_off = DQ ? swz_store_off<D>(st_row, st_col) : st_row * PITCH + st_col;
    const int st_off_tr = C::OFF_TR + st_row * C::TPITCH + st_col;                  // DV only
    const int st_off_v = C::OFF_V + st_row * PITCH + st_col;
    u32x4 st_k[CT], st_v[CT];
#pragma unroll
    for (int x = 0; x < CT; ++x) st_k[x] = st_v[x] = (u32x4){0u, 0u, 0u, 0u};
    int c_load = 0, u_load = 0;
    auto issue_loads = [&]() {
        if (stager) {
#pragma unroll
            for (int x = 0; x < CT; ++x) {
                int t = t_lo + CT * c_load + x;
                t = t < t_hi ? t : t_hi;
                int j = 32 * t + st_row;
                j = j < N ? j : N - 1;
                st_k[x] = ld_global16(k1g + (int64_t)j * p.k1.sn + st_col);
                st_v[x] = ld_global16(v1g + (int64_t)j * p.v1.sn + st_col);
            }
        }
        ++u_load;
        c_load = (c_load == NC - 1) ? 0 : c_load + 1;
    };
    auto write_stage = [&](int buf) {
        if (stager) {
            char *stage = lds + buf * C::STAGE;
#pragma unroll
            for (int x = 0; x < CT; ++x) {
                *reinterpret_cast<u32x4 *>(stage + x * C::SUB + st_off) = st_k[x];
                if constexpr (DQ) {
                    *reinterpret_cast<u32x4 *>(stage + x * C::SUB + st_off_v) = st_v[x];
                } else {
                    *reinterpret_cast<u32x4 *>(stage + x * C::SUB + st_off_tr) = st_v[x];
                }
            }
        }
    };
    const int r_lane = c * PITCH + 16 * hf;                              // row-major fragment: row c, pieces 2*kk + hf
    const int t_lane = C::OFF_TR + tr_lane_off<D, C::TPITCH>(lane);      // transposed fragment, per-lane part
    const SwzLane<D> swz_lane(lane);                                      // DQ: fragments of the swizzled K1 tile

    // ---- fp32 rows shared by the workgroup, zeroed; q/do/k2/v2 rows staged once
    float *dqs = reinterpret_cast<float *>(lds + C::DQS);
    float *sc = reinterpret_cast<float *>(lds + C::SC);
    {
        float4 *z = reinterpret_cast<float4 *>(lds + C::RING);
        constexpr int NZ = (C::QS - C::RING) / 16;
        for (int x = tid; x < NZ; x += 512) z[x] = make_float4(0.f, 0.f, 0.f, 0.f);
        const char *qg = p.q.ptr + b * p.q.sb + h * p.q.sh;
        const char *dog = p.dout.ptr + b * p.dout.sb + h * p.dout.sh;
        const char *k2g = p.k2.ptr + b * p.k2.sb + hk * p.k2.sh;
        const char *v2g = p.v2.ptr + b * p.v2.sb + hk * p.v2.sh;
        for (int x = tid; x < 32 * PPR; x += 512) {
            const int row = x / PPR, col = (x % PPR) * 16;
            int ii = i0 + row;
            ii = ii < N ? ii : N - 1;
            *reinterpret_cast<u32x4 *>(lds + C::QS + row * PITCH + col) = ld_global16(qg + (int64_t)ii * p.q.sn + col);
            *reinterpret_cast<u32x4 *>(lds + C::DOS + row * PITCH + col) = ld_global16(dog + (int64_t)ii * p.dout.sn + col);
        }
        for (int x = tid; x < C::SROWS * PPR; x += 512) {
            const int row = x / PPR, col = (x % PPR) * 16;
            int kk2 = i0 - C::HALO + row;
            kk2 = kk2 < 0 ? 0 : (kk2 < N ? kk2 : N - 1);
            *reinterpret_cast<u32x4 *>(lds + C::K2S + row * PITCH + col) = ld_global16(k2g + (int64_t)kk2 * p.k2.sn + col);
            if constexpr (DQ)
                *reinterpret_cast<u32x4 *>(lds + C::V2S + row * PITCH + col) = ld_global16(v2g + (int64_t)kk2 * p.v2.sn + col);
        }
    }

    issue_loads();
    write_stage(0);
    if (U > 1) issue_loads();
    int u = 0;

    f32x16 neg_delta;          // DQ: -delta_i in every element (one query row per lane column)
#pragma unroll
    for (int rr = 0; rr < 16; ++rr) neg_delta[rr] = -dl;
    f32x16 acc[DT];            // G^T (DQ) or T^T (DV) of the running offset
    u32x4 A[KS];
    u32x4 Bv[DQ ? KS : 1];

    __syncthreads();
    for (int r = 0; r < R; ++r) {
        const int dlt = 8 * r + wave;
        const int kr = i - dlt;
        const bool col_ok = row_ok && kr >= 0 && dlt < p.w2;
        const bool any_bad = wave_any(!col_ok);
        const bool wave_on = wave_any(col_ok);
        const int srow = c - dlt + C::HALO;           // row of k = i - dlt inside the staged / scatter rows
        {
            const char *qr = lds + C::QS + c * PITCH + 16 * hf;
            const char *k2r = lds + C::K2S + srow * PITCH + 16 * hf;
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) A[kk] = mul_bf16x8(ld_lds16(qr + 32 * kk), ld_lds16(k2r + 32 * kk));
            if constexpr (DQ) {
                const char *dor = lds + C::DOS + c * PITCH + 16 * hf;
                const char *v2r = lds + C::V2S + srow * PITCH + 16 * hf;
#pragma unroll
                for (int kk = 0; kk < KS; ++kk) Bv[kk] = mul_bf16x8(ld_lds16(dor + 32 * kk), ld_lds16(v2r + 32 * kk));
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) acc[dt] = zero16();
        }

        const char *stage = lds;
        auto sync_stage = [&]() {
            // stage u goes into its buffer (last read in step u-2) before the barrier that publishes it
            if (u >= 1 && u_load - 1 >= u) {
                write_stage(u & 1);
                if (u_load < U) issue_loads();
            }
            __syncthreads();
            stage = lds + (u & 1) * C::STAGE;
            ++u;
        };
        auto tile_body = [&](int x, int t, auto masked_tag) {
            constexpr bool MASKED = decltype(masked_tag)::value;
            const char *sub = stage + x * C::SUB;
            f32x16 X = zero16();
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) X = mfma32(DQ ? swz_lane.row_frag(sub, kk) : ld_lds16(sub + r_lane + 32 * kk), A[kk], X);
            f32x16 dP;
            if constexpr (DQ) {
                // the chain starts from a register set that holds -delta_i: dP - delta costs no VALU work
                dP = mfma32(ld_lds16(sub + C::OFF_V + r_lane), Bv[0], neg_delta);
#pragma unroll
                for (int kk = 1; kk < KS; ++kk) dP = mfma32(ld_lds16(sub + C::OFF_V + r_lane + 32 * kk), Bv[kk], dP);
            }
#pragma unroll
            for (int rr = 0; rr < 16; ++rr) X[rr] = X[rr] * c2 - lse2;
            if constexpr (MASKED) {
                // row j = 32 t + 4 hf + e (e = 8 (rr / 4) + rr % 4) is attended iff 0 <= i - j < w1;
                // lanes without a valid k2 row get a distance no e can bring into range
                const int rel = col_ok ? i - 32 * t - 4 * hf : -(1 << 30);
#pragma unroll
                for (int rr = 0; rr < 16; ++rr) {
                    const bool ok = (unsigned)(rel - (8 * (rr >> 2) + (rr & 3))) < (unsigned)p.w1;
                    X[rr] = ok ? X[rr] : -INFINITY;
                }
            }
            u32x4 pb[2];
#pragma unroll
            for (int rr = 0; rr < 16; rr += 2) {
                float p0 = fast_exp2(X[rr]);
                float p1 = fast_exp2(X[rr + 1]);
                if constexpr (DQ) {
                    p0 *= dP[rr];
                    p1 *= dP[rr + 1];
                }
                pb[rr >> 3][(rr & 7) >> 1] = pack_bf16(p0, p1);
            }
#pragma unroll
            for (int k2s = 0; k2s < 2; ++k2s)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    u32x4 fr;
                    if constexpr (DQ) {
                        fr = swz_lane.tr_frag(sub, k2s, dt);
                    } else {
                        const u32x2 lo = lds_read_tr<D, C::TPITCH>(sub + t_lane, 16 * k2s, 32 * dt);
                        const u32x2 hi = lds_read_tr<D, C::TPITCH>(sub + t_lane, 16 * k2s + 8, 32 * dt);
                        fr = (u32x4){lo[0], lo[1], hi[0], hi[1]};
                    }
                    acc[dt] = mfma32(fr, pb[k2s], acc[dt]);
                }
        };
        auto run_chunks = [&](int &cc, int cc_end, auto masked_tag) {
            constexpr bool MASKED = decltype(masked_tag)::value;
            for (; cc <= cc_end; ++cc) {
                sync_stage();
                if (!wave_on) continue;
#pragma nounroll
                for (int x = 0; x < CT; ++x) {
                    const int t = t_lo + CT * cc + x;
                    if (MASKED && t > t_hi) break;
                    tile_body(x, t, masked_tag);
                }
            }
        };
        int mid_lo = (i0 + 31 - p.w1 >= 0) ? (i0 + 31 - p.w1) / 32 + 1 : t_lo;   // first unmasked tile
        if (any_bad) mid_lo = t_hi;
        mid_lo = mid_lo > t_hi ? t_hi : mid_lo;
        const int c_mid_lo = (mid_lo - t_lo + CT - 1) / CT;
        const int c_mid_hi = (t_hi - t_lo) / CT - 1;
        int cc = 0;
        run_chunks(cc, c_mid_lo - 1, std::true_type{});
        run_chunks(cc, c_mid_hi, std::false_type{});
        run_chunks(cc, NC - 1, std::true_type{});

        // ---- round end: add into the shared fp32 rows, one d-slice per wave and phase
        {
            const char *qr = lds + (DQ ? C::QS : C::DOS) + c * PITCH + 16 * hf * 2;   // factor of the scattered rows
            const char *k2r = lds + C::K2S + srow * PITCH + 16 * hf * 2;
            float *srow_p = sc + srow * C::SPITCH + 16 * hf;
            float *drow_p = dqs + c * C::SPITCH + 16 * hf;
            auto add_slice = [&](auto slice_tag) {
                constexpr int S = decltype(slice_tag)::value;     // slice: dt = S / 2, registers 8*(S%2) .. +7
                constexpr int dt = S >> 1, r0 = 8 * (S & 1);
                const u32x4 xq = ld_lds16(qr + dt * 64 + r0 * 2);
                float *dst = srow_p + 32 * dt + r0;
                float4 a0 = *reinterpret_cast<float4 *>(dst), a1 = *reinterpret_cast<float4 *>(dst + 4);
                a0.x += bf16_lo(xq[0]) * acc[dt][r0];
                a0.y += bf16_hi(xq[0]) * acc[dt][r0 + 1];
                a0.z += bf16_lo(xq[1]) * acc[dt][r0 + 2];
                a0.w += bf16_hi(xq[1]) * acc[dt][r0 + 3];
                a1.x += bf16_lo(xq[2]) * acc[dt][r0 + 4];
                a1.y += bf16_hi(xq[2]) * acc[dt][r0 + 5];
                a1.z += bf16_lo(xq[3]) * acc[dt][r0 + 6];
                a1.w += bf16_hi(xq[3]) * acc[dt][r0 + 7];
                *reinterpret_cast<float4 *>(dst) = a0;
                *reinterpret_cast<float4 *>(dst + 4) = a1;
                if constexpr (DQ) {
                    const u32x4 xk = ld_lds16(k2r + dt * 64 + r0 * 2);
                    float *dd = drow_p + 32 * dt + r0;
                    float4 b0 = *reinterpret_cast<float4 *>(dd), b1 = *reinterpret_cast<float4 *>(dd + 4);
                    b0.x += bf16_lo(xk[0]) * acc[dt][r0];
                    b0.y += bf16_hi(xk[0]) * acc[dt][r0 + 1];
                    b0.z += bf16_lo(xk[1]) * acc[dt][r0 + 2];
                    b0.w += bf16_hi(xk[1]) * acc[dt][r0 + 3];
                    b1.x += bf16_lo(xk[2]) * acc[dt][r0 + 4];
                    b1.y += bf16_hi(xk[2]) * acc[dt][r0 + 5];
                    b1.z += bf16_lo(xk[3]) * acc[dt][r0 + 6];
                    b1.w += bf16_hi(xk[3]) * acc[dt][r0 + 7];
                    *reinterpret_cast<float4 *>(dd) = b0;
                    *reinterpret_cast<float4 *>(dd + 4) = b1;
                }
            };
            for (int ph = 0; ph < 8; ++ph) {
                // D = 128: eight slices.  D = 64: four slices; waves 0-3 use phases 0-3, waves 4-7 phases 4-7
                if (DT == 4 || (ph >> 2) == (wave >> 2)) with_slice<2 * DT>(wave + ph, add_slice);
                __syncthreads();
            }
        }
    }

    // ---- dq rows to global memory (bf16, scaled)
    if constexpr (DQ) {
        constexpr int SEG = D / 16;
        const int row = tid >> 4, seg = tid & 15;
        const int ir = i0 + row;
        if (ir < N) {
            const float *src = dqs + row * C::SPITCH + seg * SEG;
            char *orow = p.dq.ptr + b * p.dq.sb + (int64_t)ir * p.dq.sn + h * p.dq.sh + seg * SEG * 2;
            float4 a = *reinterpret_cast<const float4 *>(src);
            if constexpr (SEG == 8) {
                float4 bq = *reinterpret_cast<const float4 *>(src + 4);
                u32x4 ov = {pack_bf16(a.x * p.scale, a.y * p.scale), pack_bf16(a.z * p.scale, a.w * p.scale),
                            pack_bf16(bq.x * p.scale, bq.y * p.scale), pack_bf16(bq.z * p.scale, bq.w * p.scale)};
                st_global16(orow, ov);
            } else {
                u32x2 ov = {pack_bf16(a.x * p.scale, a.y * p.scale), pack_bf16(a.z * p.scale, a.w * p.scale)};
                *reinterpret_cast<u32x2 *>(orow) = ov;
            }
        }
    }
    // ---- scattered rows to the workspace: [tensor 0: dk2, 1: dv2][b][h][tile][63][D]
    {
        const int64_t per_tensor = (int64_t)p.B * p.H * ntile * C::SROWS * D;
        float *wk = ws + (DQ ? 0 : per_tensor) + (((int64_t)b * p.H + h) * ntile + tile) * C::SROWS * D;
        for (int x = tid; x < C::SROWS * D / 4; x += 512) {
            const int row = x / (D / 4), col = (x % (D / 4)) * 4;
            *reinterpret_cast<float4 *>(wk + row * D + col) = *reinterpret_cast<const float4 *>(sc + row * C::SPITCH + col);
        }
    }
}

// dV2 from the forward's saved per-offset T:
//     dv2[b,k,hk,:] = sum_g sum_dlt do[b,k+dlt,h,:] * T[b,h,dlt,k+dlt,:] * 2^(m[b,h,dlt,k+dlt] - lse2[b,h,k+dlt])
// (h = hk*G + g).  Streams T once from HBM; a thread owns 8 d of one row k.
template <int D>
__global__ __launch_bounds__(256) void dv2_from_saved_kernel(KParams p) {
    constexpr int LP = D / 8;                 // threads per row
    constexpr int RPB = 256 / LP;             // rows per block
    const int N = p.N;
    const int nblk = (N + RPB - 1) / RPB;
    const int blk = blockIdx.x % nblk;
    const int bh = blockIdx.x / nblk;
    const int hk = bh % p.HK, b = bh / p.HK;
    const int k = blk * RPB + threadIdx.x / LP;
    const int col = (threadIdx.x % LP) * 16;  // byte offset inside a row
    if (k >= N) return;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const int nd = p.w2 < N - k ? p.w2 : N - k;
    for (int g = 0; g < p.G; ++g) {
        const int h = hk * p.G + g;
        const int64_t bh_row = ((int64_t)b * p.H + h);
        const char *dog = p.dout.ptr + b * p.dout.sb + h * p.dout.sh + col;
        const float *lse = p.lse + bh_row * N;
#pragma unroll 8
        for (int dlt = 0; dlt < nd; ++dlt) {
            const int i = k + dlt;
            const int64_t srow = (bh_row * p.w2 + dlt) * N + i;
            const u32x4 t = ld_global16(p.t_save + srow * (D * 2) + col);
            const u32x4 o = ld_global16(dog + (int64_t)i * p.dout.sn);
            const float w = fast_exp2(p.m_save[srow] - lse[i] * kLog2e);
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                acc[2 * x] += bf16_lo(o[x]) * bf16_lo(t[x]) * w;
                acc[2 * x + 1] += bf16_hi(o[x]) * bf16_hi(t[x]) * w;
            }
        }
    }
    u32x4 r = {pack_bf16(acc[0], acc[1]), pack_bf16(acc[2], acc[3]), pack_bf16(acc[4], acc[5]), pack_bf16(acc[6], acc[7])};
    st_global16(p.dv2.ptr + b * p.dv2.sb + (int64_t)k * p.dv2.sn + hk * p.dv2.sh + col, r);
}

}  // namespace sa2
