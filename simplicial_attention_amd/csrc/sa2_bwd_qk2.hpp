// Backward kernel for dQ, dK2 and dV2 (offset-split / tile-streaming).
//
// One workgroup (4 waves) owns 32 query rows i of one (batch, head); the w2 offsets
// dlt = i - k are dealt to the waves (round r: wave w handles dlt = 4r + w) and all
// waves stream the same 32-row K1/V1 tiles through an LDS ring, as in the forward.
// Per (offset, tile) a wave evaluates, with A = q_i * k2_{i-dlt}, B = do_i * v2_{i-dlt}:
//     S^T = K1 A^T,  dP^T = V1 B^T                       (row-major fragments)
//     P = exp2(S scale log2e - lse_i),  dS = P (dP - delta_i)
//     T^T += V1^T P^T,  G^T += K1^T dS^T                 (ds_read_b64_tr_b16 fragments)
// and at the end of the offset
//     dq_i       += k2_{i-dlt} * G_i                     (registers, summed over waves at the end)
//     dk2_{i-dlt} += q_i * G_i,   dv2_{i-dlt} += do_i * T_i
// The two K2/V2 gradients land on rows k = i - dlt in [i0-31, i0+31]; they are added
// into an fp32 LDS buffer shared by the workgroup.  Different waves hit the same rows,
// so a round's additions run in four barrier-separated phases in which wave w touches
// only rows with k mod 4 == (w + phase) mod 4: disjoint rows, fixed order, no atomics,
// bitwise reproducible.  Rows k >= i0 ("own") and rows k < i0 ("halo", which the
// previous workgroup also feeds) go to an fp32 workspace; dk2_dv2_combine_kernel adds
// own + halo of the next tile, sums the query heads of a group and rounds to bf16.
#pragma once

#include <type_traits>

#include "sa2_common.hpp"
#include "sa2_lds.hpp"

namespace sa2 {

template <int D, int W2MAX>
struct Qk2Cfg {
    static constexpr int KS = D / 16;
    static constexpr int DT = D / 32;
    static constexpr int TILE = 32 * tile_pitch<D>();
    static constexpr int NBUF = 3;
    static constexpr int STAGE = 2 * TILE;          // K1 tile + V1 tile
    static constexpr int RING = NBUF * STAGE;
    static constexpr int SPITCH = D + 4;            // floats per row of the scatter buffers
    static constexpr int HALO = W2MAX - 1;          // rows k < i0 a tile can reach
    static constexpr int SROWS = 32 + HALO;         // k in [i0-HALO, i0+31]
    static constexpr int SCAT = SROWS * SPITCH * 4; // one scatter buffer (dk2 or dv2)
    static constexpr int LDS = RING + 2 * SCAT;
    static constexpr int LPT = 32 * D / 8 / 256;    // 16-byte pieces per thread, tile and tensor
};

// workspace layout (floats): [tensor 0: dk2, 1: dv2][b][h][tile][srows][D], srows = 31 + W2MAX
__host__ __device__ inline int64_t qk2_ws_floats(int B, int H, int N, int D, int srows) {
    return 2ll * B * H * ((N + 31) / 32) * srows * D;
}

template <int D, int W2MAX>
__global__ __launch_bounds__(256, 1) void bwd_qk2_kernel(KParams p, float *ws) {
    using C = Qk2Cfg<D, W2MAX>;
    constexpr int KS = C::KS, DT = C::DT, PPR = D / 8, PITCH = tile_pitch<D>();
    __shared__ __attribute__((aligned(16))) char lds[C::LDS];

    const int N = p.N;
    const int ntile = (N + 31) / 32;
    const int item = xcd_contiguous(blockIdx.x, gridDim.x);
    const int tile = ntile - 1 - item % ntile;
    const int bh = item / ntile;
    const int h = bh % p.H, b = bh / p.H;
    const int hk = h / p.G;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int c = lane & 31, hf = lane >> 5;
    const int i0 = tile * 32;
    const int i = i0 + c;
    const bool row_ok = i < N;
    const int ic = row_ok ? i : N - 1;

    const char *qrow = p.q.ptr + b * p.q.sb + (int64_t)ic * p.q.sn + h * p.q.sh;
    const char *dorow = p.dout.ptr + b * p.dout.sb + (int64_t)ic * p.dout.sn + h * p.dout.sh;
    const char *k1g = p.k1.ptr + b * p.k1.sb + hk * p.k1.sh;
    const char *v1g = p.v1.ptr + b * p.v1.sb + hk * p.v1.sh;
    const char *k2g = p.k2.ptr + b * p.k2.sb + hk * p.k2.sh;
    const char *v2g = p.v2.ptr + b * p.v2.sb + hk * p.v2.sh;
    const float lse2 = p.lse[((int64_t)b * p.H + h) * N + ic] * kLog2e;
    const float dl = p.delta[((int64_t)b * p.H + h) * N + ic];

    const int t_lo = (i0 - p.w1 + 1 > 0 ? i0 - p.w1 + 1 : 0) / 32;
    const int t_hi = i0 / 32;
    const int NT = t_hi - t_lo + 1;
    const int nd = p.w2 < i0 + 32 ? p.w2 : i0 + 32;
    const int R = (nd + 3) / 4;
    const int U = R * NT;
    const float c2 = p.scale_log2e;

    // ---- zero the scatter buffers
    float *sk = reinterpret_cast<float *>(lds + C::RING);
    float *sv = sk + C::SROWS * C::SPITCH;
    for (int x = tid; x < 2 * C::SROWS * C::SPITCH / 4; x += 256) reinterpret_cast<float4 *>(sk)[x] = make_float4(0.f, 0.f, 0.f, 0.f);

    // ---- tile staging (same ring as the forward)
    u32x4 st[2 * C::LPT];
    int st_off[C::LPT];
#pragma unroll
    for (int x = 0; x < C::LPT; ++x) st_off[x] = ((x * 256 + tid) / PPR) * PITCH + ((x * 256 + tid) % PPR) * 16;
    auto issue_loads = [&](int t) {
#pragma unroll
        for (int x = 0; x < C::LPT; ++x) {
            const int pc = x * 256 + tid;
            int j = 32 * t + pc / PPR;
            j = j < N ? j : N - 1;
            st[x] = ld_global16(k1g + (int64_t)j * p.k1.sn + (pc % PPR) * 16);
            st[C::LPT + x] = ld_global16(v1g + (int64_t)j * p.v1.sn + (pc % PPR) * 16);
        }
    };
    auto write_stage = [&](int buf) {
        char *stage = lds + buf * C::STAGE;
#pragma unroll
        for (int x = 0; x < C::LPT; ++x) {
            *reinterpret_cast<u32x4 *>(stage + st_off[x]) = st[x];
            *reinterpret_cast<u32x4 *>(stage + C::TILE + st_off[x]) = st[C::LPT + x];
        }
    };
    const int r_lane = c * PITCH + 16 * hf;       // row-major fragment: row c, pieces 2*kk + hf
    const int t_lane = tr_lane_off<D>(lane);      // transposed fragment, per-lane part

    int t_load = t_lo, buf_fill = 0, buf_use = 0, u_load = 0;
    auto advance_load = [&]() {
        ++u_load;
        t_load = (t_load == t_hi) ? t_lo : t_load + 1;
    };
    issue_loads(t_load);
    advance_load();
    write_stage(0);
    buf_fill = 1;
    if (U > 1) {
        issue_loads(t_load);
        advance_load();
    }

    f32x16 dq[DT], G[DT], T[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) dq[dt] = zero16();

    for (int r = 0; r < R; ++r) {
        const int dlt = 4 * r + wave;
        const int kr = i - dlt;
        const bool col_ok = row_ok && kr >= 0 && dlt < p.w2;
        const bool any_bad = wave_any(!col_ok);
        const bool wave_on = wave_any(col_ok);
        const int krc = kr < 0 ? 0 : (kr > N - 1 ? N - 1 : kr);
        const char *k2row = k2g + (int64_t)krc * p.k2.sn;
        const char *v2row = v2g + (int64_t)krc * p.v2.sn;
        u32x4 A[KS], Bv[KS];
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            A[kk] = mul_bf16x8(ld_global16(qrow + (16 * kk + 8 * hf) * 2), ld_global16(k2row + (16 * kk + 8 * hf) * 2));
            Bv[kk] = mul_bf16x8(ld_global16(dorow + (16 * kk + 8 * hf) * 2), ld_global16(v2row + (16 * kk + 8 * hf) * 2));
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            G[dt] = zero16();
            T[dt] = zero16();
        }

        auto run_tiles = [&](int t, int t_end, auto masked_tag) {
            constexpr bool MASKED = decltype(masked_tag)::value;
            for (; t <= t_end; ++t) {
                __syncthreads();
                if (u_load - 1 > r * NT + (t - t_lo)) {
                    write_stage(buf_fill);
                    buf_fill = buf_fill == C::NBUF - 1 ? 0 : buf_fill + 1;
                }
                if (u_load < U) {
                    issue_loads(t_load);
                    advance_load();
                }
                const char *kt = lds + buf_use * C::STAGE;
                const char *vt = kt + C::TILE;
                buf_use = buf_use == C::NBUF - 1 ? 0 : buf_use + 1;
                if (!wave_on) continue;

                f32x16 X = zero16(), dP = zero16();
#pragma unroll
                for (int kk = 0; kk < KS; ++kk) {
                    X = mfma32(ld_lds16(kt + r_lane + 32 * kk), A[kk], X);
                    dP = mfma32(ld_lds16(vt + r_lane + 32 * kk), Bv[kk], dP);
                }
#pragma unroll
                for (int rr = 0; rr < 16; ++rr) X[rr] = X[rr] * c2 - lse2;
                if constexpr (MASKED) {
#pragma unroll
                    for (int rr = 0; rr < 16; ++rr) {
                        int j = 32 * t + 8 * (rr >> 2) + 4 * hf + (rr & 3);
                        bool ok = col_ok && (j <= i) && (j + p.w1 > i);
                        X[rr] = ok ? X[rr] : -INFINITY;
                    }
                }
                u32x4 pb[2], dsb[2];
#pragma unroll
                for (int rr = 0; rr < 16; rr += 2) {
                    float p0 = fast_exp2(X[rr]);
                    float p1 = fast_exp2(X[rr + 1]);
                    pb[rr >> 3][(rr & 7) >> 1] = pack_bf16(p0, p1);
                    dsb[rr >> 3][(rr & 7) >> 1] = pack_bf16(p0 * (dP[rr] - dl), p1 * (dP[rr + 1] - dl));
                }
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int k2s = 0; k2s < 2; ++k2s) {
                        u32x2 vlo = lds_read_tr<D>(vt + t_lane, 16 * k2s, 32 * dt);
                        u32x2 vhi = lds_read_tr<D>(vt + t_lane, 16 * k2s + 8, 32 * dt);
                        u32x2 klo = lds_read_tr<D>(kt + t_lane, 16 * k2s, 32 * dt);
                        u32x2 khi = lds_read_tr<D>(kt + t_lane, 16 * k2s + 8, 32 * dt);
                        u32x4 vfr = {vlo[0], vlo[1], vhi[0], vhi[1]};
                        u32x4 kfr = {klo[0], klo[1], khi[0], khi[1]};
                        T[dt] = mfma32(vfr, pb[k2s], T[dt]);
                        G[dt] = mfma32(kfr, dsb[k2s], G[dt]);
                    }
            }
        };
        int mid_lo = (i0 + 31 - p.w1 >= 0) ? (i0 + 31 - p.w1) / 32 + 1 : t_lo;
        if (any_bad) mid_lo = t_hi;
        mid_lo = mid_lo > t_hi ? t_hi : mid_lo;
        run_tiles(t_lo, mid_lo - 1, std::true_type{});
        run_tiles(mid_lo, t_hi - 1, std::false_type{});
        run_tiles(t_hi, t_hi, std::true_type{});

        // ---- end of the offset: dq in registers, dk2/dv2 into the shared scatter rows
        fma_row<DT>(dq, G, k2row + 16 * hf * 2);
        {
            // q_i * G_i and do_i * T_i in place (lane holds d = 32*dt + 16*hf + rr)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const u32x4 qa = ld_global16(qrow + 16 * hf * 2 + dt * 64), qb = ld_global16(qrow + 16 * hf * 2 + dt * 64 + 16);
                const u32x4 oa = ld_global16(dorow + 16 * hf * 2 + dt * 64), ob = ld_global16(dorow + 16 * hf * 2 + dt * 64 + 16);
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    G[dt][2 * w] *= bf16_lo(qa[w]);
                    G[dt][2 * w + 1] *= bf16_hi(qa[w]);
                    G[dt][8 + 2 * w] *= bf16_lo(qb[w]);
                    G[dt][8 + 2 * w + 1] *= bf16_hi(qb[w]);
                    T[dt][2 * w] *= bf16_lo(oa[w]);
                    T[dt][2 * w + 1] *= bf16_hi(oa[w]);
                    T[dt][8 + 2 * w] *= bf16_lo(ob[w]);
                    T[dt][8 + 2 * w + 1] *= bf16_hi(ob[w]);
                }
            }
            const int srow = c - dlt + C::HALO;       // row of k = i - dlt inside [i0-HALO, i0+31]
            float *dk = sk + srow * C::SPITCH + 16 * hf;
            float *dv = sv + srow * C::SPITCH + 16 * hf;
            for (int ph = 0; ph < 4; ++ph) {
                // wave w touches rows with k mod 4 == (w + ph) mod 4, i.e. columns
                // c == 2*w + ph (mod 4): disjoint rows across the four waves
                if (col_ok && ((c - 2 * wave - ph) & 3) == 0) {
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int r4 = 0; r4 < 4; ++r4) {
                            float4 a = *reinterpret_cast<float4 *>(dk + 32 * dt + 4 * r4);
                            float4 bq = *reinterpret_cast<float4 *>(dv + 32 * dt + 4 * r4);
                            a.x += G[dt][4 * r4];
                            a.y += G[dt][4 * r4 + 1];
                            a.z += G[dt][4 * r4 + 2];
                            a.w += G[dt][4 * r4 + 3];
                            bq.x += T[dt][4 * r4];
                            bq.y += T[dt][4 * r4 + 1];
                            bq.z += T[dt][4 * r4 + 2];
                            bq.w += T[dt][4 * r4 + 3];
                            *reinterpret_cast<float4 *>(dk + 32 * dt + 4 * r4) = a;
                            *reinterpret_cast<float4 *>(dv + 32 * dt + 4 * r4) = bq;
                        }
                }
                __syncthreads();
            }
        }
    }

    // ---- dq: ordered sum of the four waves through LDS (ring area is free now)
    __syncthreads();
    float *dqs = reinterpret_cast<float *>(lds);      // [32][SPITCH]
    for (int w = 0; w < 4; ++w) {
        if (wave == w) {
            float *dst = dqs + c * C::SPITCH + 16 * hf;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (w > 0) a = *reinterpret_cast<float4 *>(dst + 32 * dt + 4 * r4);
                    a.x += dq[dt][4 * r4];
                    a.y += dq[dt][4 * r4 + 1];
                    a.z += dq[dt][4 * r4 + 2];
                    a.w += dq[dt][4 * r4 + 3];
                    *reinterpret_cast<float4 *>(dst + 32 * dt + 4 * r4) = a;
                }
        }
        __syncthreads();
    }
    {
        constexpr int SEG = D / 8;
        const int row = tid >> 3, seg = tid & 7;
        const int ir = i0 + row;
        if (ir < N) {
            const float *src = dqs + row * C::SPITCH + seg * SEG;
            char *orow = p.dq.ptr + b * p.dq.sb + (int64_t)ir * p.dq.sn + h * p.dq.sh + seg * SEG * 2;
#pragma unroll
            for (int x = 0; x < SEG; x += 8) {
                float4 a = *reinterpret_cast<const float4 *>(src + x), bq = *reinterpret_cast<const float4 *>(src + x + 4);
                u32x4 ov = {pack_bf16(a.x * p.scale, a.y * p.scale), pack_bf16(a.z * p.scale, a.w * p.scale),
                            pack_bf16(bq.x * p.scale, bq.y * p.scale), pack_bf16(bq.z * p.scale, bq.w * p.scale)};
                st_global16(orow + x * 2, ov);
            }
        }
    }
    // ---- dk2/dv2 partial rows to the workspace: [tensor][b][h][tile][63][D]
    {
        const int64_t per_tensor = (int64_t)p.B * p.H * ntile * C::SROWS * D;
        float *wk = ws + (((int64_t)b * p.H + h) * ntile + tile) * C::SROWS * D;
        for (int x = tid; x < C::SROWS * D / 4; x += 256) {
            const int row = x / (D / 4), col = (x % (D / 4)) * 4;
            *reinterpret_cast<float4 *>(wk + row * D + col) = *reinterpret_cast<const float4 *>(sk + row * C::SPITCH + col);
            *reinterpret_cast<float4 *>(wk + per_tensor + row * D + col) = *reinterpret_cast<const float4 *>(sv + row * C::SPITCH + col);
        }
    }
}

// dk2[b,k,hk,:] = scale * sum_g sum_tiles partial rows of k,  dv2 likewise (no scale;
// left out if with_dv2 == 0: dv2 then comes from the forward's saved partials).
// Workspace rows of a tile with first query row i0: index x <-> k = i0 - halo + x, so
// rows 0..halo-1 are the halo below the tile and rows halo..halo+31 its own rows.
template <int D>
__global__ __launch_bounds__(256) void dk2_dv2_combine_kernel(KParams p, const float *ws, int srows, int with_dv2) {
    constexpr int LP = D / 8;   // threads per row, 8 d each
    const int N = p.N, ntile = (N + 31) / 32;
    const int halo = srows - 32;
    const int64_t rows = (int64_t)p.B * p.HK * N;
    const int64_t row = (int64_t)blockIdx.x * (256 / LP) + threadIdx.x / LP;
    if (row >= rows) return;
    const int piece = threadIdx.x % LP;
    const int k = (int)(row % N);
    const int hk = (int)((row / N) % p.HK);
    const int b = (int)(row / ((int64_t)N * p.HK));
    const int tile = k / 32, kl = k % 32;
    const int64_t per_tensor = (int64_t)p.B * p.H * ntile * srows * D;
    float ak[8], av[8];
#pragma unroll
    for (int x = 0; x < 8; ++x) ak[x] = av[x] = 0.f;
    for (int g = 0; g < p.G; ++g) {
        const int h = hk * p.G + g;
        const float *base = ws + (((int64_t)b * p.H + h) * ntile) * srows * D;
        for (int m = 0; tile + m < ntile && kl + halo - 32 * m >= 0; ++m) {
            const float *src = base + ((int64_t)(tile + m) * srows + (kl + halo - 32 * m)) * D + piece * 8;
#pragma unroll
            for (int x = 0; x < 8; ++x) {
                ak[x] += src[x];
                if (with_dv2) av[x] += src[per_tensor + x];
            }
        }
    }
    u32x4 ok, ov;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        ok[w] = pack_bf16(ak[2 * w] * p.scale, ak[2 * w + 1] * p.scale);
        ov[w] = pack_bf16(av[2 * w], av[2 * w + 1]);
    }
    st_global16(p.dk2.ptr + b * p.dk2.sb + (int64_t)k * p.dk2.sn + hk * p.dk2.sh + piece * 16, ok);
    if (with_dv2) st_global16(p.dv2.ptr + b * p.dv2.sb + (int64_t)k * p.dv2.sn + hk * p.dv2.sh + piece * 16, ov);
}

}  // namespace sa2
