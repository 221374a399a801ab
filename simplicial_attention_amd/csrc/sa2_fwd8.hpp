// Forward kernel, eight-wave variant (two waves per SIMD).
//
// Measured on MI355X: one wave cannot overlap its own MFMA and VALU instructions (one
// 32x32x16 MFMA followed by n independent VALU instructions costs about 28 + 4.8 n
// cycles), two waves on one SIMD can.  So the kernel is shaped for two waves per SIMD:
// at most 256 registers per wave, eight waves per workgroup.
//
// One workgroup owns 32 query rows of one (batch, head).  In round r wave w handles the
// offset dlt = i - k = 8r + w; all eight waves walk the same 32-row K1/V1 tiles, which
// stream through a double-buffered LDS ring two tiles at a time (one barrier per 64 rows).  Per (offset, tile):
//     S^T = K1 A^T          A = q_i * k2_{i-dlt}   (bf16, built once per offset)
//     P^T = exp2(S^T scale log2e - M_i)
//     T^T += V1^T P^T       (V1 fragments through ds_read_b64_tr_b16)
// Every wave keeps a private softmax reference M and row sum l.  M stays fixed while an
// offset runs (no per-tile rescale of T inside the hot loop); a tile whose logits leave the
// safe exponent range [-32, 64] relative to M takes a slow path outside the loop that
// moves M and rescales T and l.  The output accumulator is shared: an fp32 [32][D]
// LDS buffer relative to a common reference Mc.  At the end of a round the waves
// publish their references, agree on Mc = max, and add v2_{i-dlt} * T * 2^(M - Mc) in
// eight barrier-separated phases; in phase ph wave w owns the d-slice (w + ph) mod 8,
// so concurrent waves never touch the same element and every element sees its eight
// additions in a fixed order (bitwise reproducible, no atomics).
#pragma once

#include <type_traits>

#include "sa2_common.hpp"
#include "sa2_lds.hpp"

namespace sa2 {

template <int D, int W2MAX_>
struct Fwd8 {
    static constexpr int KS = D / 16;
    static constexpr int DT = D / 32;
    static constexpr int CT = 2;                      // 32-row tiles per ring stage (per barrier)
    static constexpr int TILE = 32 * tile_pitch<D>(); // K1 tile, read row-major
    static constexpr int VPITCH = tr_pitch<D>();
    static constexpr int VTILE = 32 * VPITCH;         // V1 tile, read through transposed reads only
    static constexpr int SUB = TILE + VTILE;          // one K1 tile + one V1 tile
    static constexpr int STAGE = CT * SUB;
    static constexpr int NBUF = 2;
    static constexpr int RING = NBUF * STAGE;
    static constexpr int APITCH = D + 4;              // floats per row of the shared accumulator
    static constexpr int ACC = 32 * APITCH * 4;
    static constexpr int EXCH = 8 * 32 * 4;           // one float per (wave, row)
    static constexpr int W2MAX = W2MAX_;              // largest second window this instance accepts (32 or 64)
    static constexpr int SROWS = 32 + W2MAX - 1;      // rows k in [i0-(W2MAX-1), i0+31]
    static constexpr int QS = RING + ACC + 2 * EXCH;  // q rows of the tile      [32][pitch]
    static constexpr int K2S = QS + TILE;             // k2 rows                 [SROWS][pitch]
    static constexpr int V2S = K2S + SROWS * tile_pitch<D>();   // v2 rows      [SROWS][pitch]
    static constexpr int LDS = V2S + SROWS * tile_pitch<D>();
    static constexpr int PIECES = 32 * D / 8;         // 16-byte pieces per tile
};

template <int D, int W2MAX>
__global__ __launch_bounds__(512, (D == 64 && W2MAX == 32) ? 4 : 1) void fwd8_kernel(KParams p) {
    using C = Fwd8<D, W2MAX>;
    constexpr int KS = C::KS, DT = C::DT, CT = C::CT, PPR = D / 8, PITCH = tile_pitch<D>();
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

    const char *k1g = p.k1.ptr + b * p.k1.sb + hk * p.k1.sh;
    const char *v1g = p.v1.ptr + b * p.v1.sb + hk * p.v1.sh;
    const char *k2g = p.k2.ptr + b * p.k2.sb + hk * p.k2.sh;
    const char *v2g = p.v2.ptr + b * p.v2.sb + hk * p.v2.sh;

    const int t_lo = (i0 - p.w1 + 1 > 0 ? i0 - p.w1 + 1 : 0) / 32;
    const int t_hi = i0 / 32;
    const int NT = t_hi - t_lo + 1;
    const int NC = (NT + CT - 1) / CT;                // ring stages (chunks of CT tiles) per round
    const int nd = p.w2 < i0 + 32 ? p.w2 : i0 + 32;   // offsets that meet at least one valid k
    const int R = (nd + 7) / 8;
    const int U = R * NC;
    const float c2 = p.scale_log2e;

    // ---- ring staging: the first PIECES threads move one 16-byte piece of K1 and of V1 per tile
    const bool stager = tid < C::PIECES;
    const int st_row = tid / PPR, st_col = (tid % PPR) * 16;
    const int st_off = st_row * PITCH + st_col;
    const int st_off_v = C::TILE + st_row * C::VPITCH + st_col;
    u32x4 st_k[CT], st_v[CT];
#pragma unroll
    for (int x = 0; x < CT; ++x) st_k[x] = st_v[x] = (u32x4){0u, 0u, 0u, 0u};
    int c_load = 0, u_load = 0;                       // chunk (within the round) / running count of the next load
    auto issue_loads = [&]() {
        if (stager) {
#pragma unroll
            for (int x = 0; x < CT; ++x) {
                int t = t_lo + CT * c_load + x;
                t = t < t_hi ? t : t_hi;              // a missing second tile reloads the diagonal one
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
                *reinterpret_cast<u32x4 *>(stage + x * C::SUB + st_off_v) = st_v[x];
            }
        }
    };
    const int k_lane = c * PITCH + 16 * hf;          // K1 fragment: row c, pieces 2*kk + hf
    const int v_lane = C::TILE + tr_lane_off<D, C::VPITCH>(lane);

    // ---- shared output accumulator and exchange areas
    float *acc_sh = reinterpret_cast<float *>(lds + C::RING);              // [32][APITCH]
    float *xm = reinterpret_cast<float *>(lds + C::RING + C::ACC);         // [8][32] references
    float *xl = xm + 8 * 32;                                               // [8][32] row sums
    for (int x = tid; x < 32 * C::APITCH / 4; x += 512) reinterpret_cast<float4 *>(acc_sh)[x] = make_float4(0.f, 0.f, 0.f, 0.f);
    float Mc = -INFINITY;      // common reference of acc_sh (same value in every wave)

    // ---- the q rows of the tile and the k2/v2 rows every offset can reach, staged once:
    // all per-offset operand builds then read LDS instead of waiting for global memory
    {
        const char *qg = p.q.ptr + b * p.q.sb + h * p.q.sh;
        for (int x = tid; x < 32 * PPR; x += 512) {
            const int row = x / PPR, col = (x % PPR) * 16;
            int ii = i0 + row;
            ii = ii < N ? ii : N - 1;
            *reinterpret_cast<u32x4 *>(lds + C::QS + row * PITCH + col) = ld_global16(qg + (int64_t)ii * p.q.sn + col);
        }
        for (int x = tid; x < C::SROWS * PPR; x += 512) {
            const int row = x / PPR, col = (x % PPR) * 16;
            int kk2 = i0 - (C::W2MAX - 1) + row;
            kk2 = kk2 < 0 ? 0 : (kk2 < N ? kk2 : N - 1);
            *reinterpret_cast<u32x4 *>(lds + C::K2S + row * PITCH + col) = ld_global16(k2g + (int64_t)kk2 * p.k2.sn + col);
            *reinterpret_cast<u32x4 *>(lds + C::V2S + row * PITCH + col) = ld_global16(v2g + (int64_t)kk2 * p.v2.sn + col);
        }
    }

    f32x16 T[DT];
    u32x4 A[KS];
    float M = 0.f;             // private reference (log2 domain); meaningless while `seen` is -inf
    float seen = -INFINITY;    // running maximum of x relative to M; -inf: no valid entry yet
    float l = 0.f;

    // ring protocol: stage u is written right before the barrier of step u (its buffer was last
    // read in step u-2), from registers loaded right before the barrier of step u-1
    issue_loads();
    write_stage(0);
    if (U > 1) issue_loads();
    int u = 0;                 // running step counter

    __syncthreads();           // staged q/k2/v2 rows and the zeroed accumulator are visible
    for (int r = 0; r < R; ++r) {
        const int dlt = 8 * r + wave;
        const int kr = i - dlt;
        const bool col_ok = row_ok && kr >= 0 && dlt < p.w2;
        const bool any_bad = wave_any(!col_ok);
        const bool wave_on = wave_any(col_ok);
        // row of k = i - dlt inside the staged k2/v2 rows (clamped for dead offsets)
        const int srow = (dlt < C::W2MAX ? c - dlt : c) + C::W2MAX - 1;
        {
            const char *k2row = lds + C::K2S + srow * PITCH + 16 * hf;
            const char *qr = lds + C::QS + c * PITCH + 16 * hf;
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) A[kk] = mul_bf16x8(ld_lds16(qr + 32 * kk), ld_lds16(k2row + 32 * kk));
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) T[dt] = zero16();
        }

        f32x16 X;
        float tmax = 0.f;
        u32x2 vf[DT][2][2];
        const char *stage = lds;
        // exponentials, row sums and T^T += V1^T P^T for the tile whose logits are in X
        auto finish_tile = [&]() {
            u32x4 pb[2];
#pragma unroll
            for (int rr = 0; rr < 16; rr += 2) {
                const uint32_t pp = pack_bf16(fast_exp2(X[rr]), fast_exp2(X[rr + 1]));
                l = add_bf16x2(pp, l);            // row sum of the rounded weights the MFMA consumes
                pb[rr >> 3][(rr & 7) >> 1] = pp;
            }
#pragma unroll
            for (int k2s = 0; k2s < 2; ++k2s)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    u32x4 v = {vf[dt][k2s][0][0], vf[dt][k2s][0][1], vf[dt][k2s][1][0], vf[dt][k2s][1][1]};
                    T[dt] = mfma32(v, pb[k2s], T[dt]);
                }
        };
        // logits of sub-tile x of the current stage -> X (scaled, referenced, masked), tmax;
        // returns true if some row left the safe exponent range
        auto logits = [&](int x, int t, auto masked_tag) -> bool {
            constexpr bool MASKED = decltype(masked_tag)::value;
            const char *kbase = stage + x * C::SUB + k_lane;
            const char *vbase = stage + x * C::SUB + v_lane;
            X = zero16();
            u32x4 kf[KS];
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) kf[kk] = ld_lds16(kbase + 32 * kk);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) X = mfma32(kf[kk], A[kk], X);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int k2s = 0; k2s < 2; ++k2s) {
                    vf[dt][k2s][0] = lds_read_tr<D, C::VPITCH>(vbase, 16 * k2s, 32 * dt);
                    vf[dt][k2s][1] = lds_read_tr<D, C::VPITCH>(vbase, 16 * k2s + 8, 32 * dt);
                }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int rr = 0; rr < 16; ++rr) X[rr] = X[rr] * c2 - M;
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
            tmax = X[0];
#pragma unroll
            for (int rr = 1; rr < 16; ++rr) tmax = fmaxf(tmax, X[rr]);
            auto sw = __builtin_amdgcn_permlane32_swap(as_u32(tmax), as_u32(tmax), false, false);
            tmax = fmaxf(as_f32(sw[0]), as_f32(sw[1]));
            return wave_any(tmax > 64.f || (seen == -INFINITY && tmax < -32.f && tmax > -INFINITY));
        };
        // slow path (kept outside the hot loop on purpose): move the reference of the rows
        // that left the safe range and rescale what T and l already hold
        auto move_reference = [&]() {
            const bool fresh = seen == -INFINITY;
            const bool move = tmax > 64.f || (fresh && tmax < -32.f && tmax > -INFINITY);
            const float shift = move ? tmax : 0.f;
            const float alpha = fresh ? 1.f : fast_exp2(-shift);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int rr = 0; rr < 16; ++rr) T[dt][rr] *= alpha;
#pragma unroll
            for (int rr = 0; rr < 16; ++rr) X[rr] -= shift;
            l *= alpha;
            M += shift;
            seen -= shift;
            tmax -= shift;
        };
        // barrier + refill of the ring behind the stage that becomes current
        auto sync_stage = [&]() {
            // stage u goes into its buffer (last read in step u-2) BEFORE the barrier that
            // publishes it: the writes fall into the time a wave would otherwise wait for the others
            if (u >= 1 && u_load - 1 >= u) {
                write_stage(u & 1);
                if (u_load < U) issue_loads();
            }
            __syncthreads();
            stage = lds + (u & 1) * C::STAGE;
            ++u;
        };
        // Runs chunks cc .. cc_end.  Returns true if it stopped inside chunk cc at sub-tile
        // `stop_x` because the logits in X left the safe range (nothing of that sub-tile
        // has been accumulated yet).
        int stop_x = 0;
        auto run_chunks = [&](int &cc, int cc_end, auto masked_tag) -> bool {
            constexpr bool MASKED = decltype(masked_tag)::value;
            for (; cc <= cc_end; ++cc) {
                sync_stage();
                if (!wave_on) continue;
#pragma nounroll
                for (int x = 0; x < CT; ++x) {
                    const int t = t_lo + CT * cc + x;
                    if (MASKED && t > t_hi) break;
                    if (logits(x, t, masked_tag)) {
                        stop_x = x;
                        return true;
                    }
                    seen = fmaxf(seen, tmax);
                    finish_tile();
                }
            }
            return false;
        };

        // chunks of the window: masked head | unmasked middle | masked tail (holds the diagonal)
        int mid_lo = (i0 + 31 - p.w1 >= 0) ? (i0 + 31 - p.w1) / 32 + 1 : t_lo;   // first unmasked tile
        if (any_bad) mid_lo = t_hi;
        mid_lo = mid_lo > t_hi ? t_hi : mid_lo;
        const int c_mid_lo = (mid_lo - t_lo + CT - 1) / CT;         // first chunk made of unmasked tiles only
        const int c_mid_hi = (t_hi - t_lo) / CT - 1;                // last chunk that ends before the diagonal tile
        const int seg_end[3] = {c_mid_lo - 1, c_mid_hi, NC - 1};
        int cc = 0;
#pragma unroll
        for (int seg = 0; seg < 3; ++seg) {
            while (cc <= seg_end[seg]) {
                const bool stopped = (seg == 1) ? run_chunks(cc, seg_end[seg], std::false_type{})
                                                : run_chunks(cc, seg_end[seg], std::true_type{});
                if (!stopped) break;
                // finish chunk cc on the slow path
                move_reference();
                seen = fmaxf(seen, tmax);
                finish_tile();
                for (int x = stop_x + 1; x < CT; ++x) {
                    const int t = t_lo + CT * cc + x;
                    if (t > t_hi) break;
                    if (logits(x, t, std::true_type{})) move_reference();
                    seen = fmaxf(seen, tmax);
                    finish_tile();
                }
                ++cc;
            }
        }

        // ---- round end: agree on the common reference, add v2 * T into the shared rows
        {
            const bool fresh = seen == -INFINITY;
            if (hf == 0) xm[wave * 32 + c] = fresh ? -INFINITY : M + seen;
            __syncthreads();
            float Mn = Mc;
#pragma unroll
            for (int w = 0; w < 8; ++w) Mn = fmaxf(Mn, xm[w * 32 + c]);
            const float fo = (Mc == -INFINITY) ? 0.f : fast_exp2(Mc - Mn);   // rescale of the old content
            const float g = fresh ? 0.f : fast_exp2(M - Mn);                 // weight of this wave's T
            // by-product for the backward: this offset's T and its reference
            if (p.t_save && row_ok && dlt < p.w2) {
                const int64_t srow_g = (((int64_t)b * p.H + h) * p.w2 + dlt) * N + i;
                char *trow = p.t_save + srow_g * (D * 2) + 16 * hf * 2;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    u32x4 lo4, hi4;
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        lo4[w] = pack_bf16(T[dt][2 * w], T[dt][2 * w + 1]);
                        hi4[w] = pack_bf16(T[dt][8 + 2 * w], T[dt][8 + 2 * w + 1]);
                    }
                    st_global16(trow + dt * 64, lo4);
                    st_global16(trow + dt * 64 + 16, hi4);
                }
                if (hf == 0) p.m_save[srow_g] = fresh ? 0.f : M;
            }
            // re-centre the private reference on what this wave has seen
            if (!fresh) {
                l *= fast_exp2(-seen);
                M += seen;
                seen = 0.f;
            }
            Mc = Mn;
            const char *v2row = lds + C::V2S + srow * PITCH + 16 * hf * 2;
            float *arow = acc_sh + c * C::APITCH + 16 * hf;
            auto add_slice = [&](auto slice_tag, bool first) {
                constexpr int S = decltype(slice_tag)::value;     // slice: dt = S / 2, registers 8*(S%2) .. +7
                constexpr int dt = S >> 1, r0 = 8 * (S & 1);
                const u32x4 xv = ld_lds16(v2row + dt * 64 + r0 * 2);
                float *dst = arow + 32 * dt + r0;
                float4 a0 = *reinterpret_cast<float4 *>(dst), a1 = *reinterpret_cast<float4 *>(dst + 4);
                if (first) {
                    a0.x *= fo; a0.y *= fo; a0.z *= fo; a0.w *= fo;
                    a1.x *= fo; a1.y *= fo; a1.z *= fo; a1.w *= fo;
                }
                a0.x += bf16_lo(xv[0]) * T[dt][r0] * g;
                a0.y += bf16_hi(xv[0]) * T[dt][r0 + 1] * g;
                a0.z += bf16_lo(xv[1]) * T[dt][r0 + 2] * g;
                a0.w += bf16_hi(xv[1]) * T[dt][r0 + 3] * g;
                a1.x += bf16_lo(xv[2]) * T[dt][r0 + 4] * g;
                a1.y += bf16_hi(xv[2]) * T[dt][r0 + 5] * g;
                a1.z += bf16_lo(xv[3]) * T[dt][r0 + 6] * g;
                a1.w += bf16_hi(xv[3]) * T[dt][r0 + 7] * g;
                *reinterpret_cast<float4 *>(dst) = a0;
                *reinterpret_cast<float4 *>(dst + 4) = a1;
            };
            for (int ph = 0; ph < 8; ++ph) {
                if constexpr (DT == 4) {
                    switch ((wave + ph) & 7) {
                        case 0: add_slice(std::integral_constant<int, 0>{}, ph == 0); break;
                        case 1: add_slice(std::integral_constant<int, 1>{}, ph == 0); break;
                        case 2: add_slice(std::integral_constant<int, 2>{}, ph == 0); break;
                        case 3: add_slice(std::integral_constant<int, 3>{}, ph == 0); break;
                        case 4: add_slice(std::integral_constant<int, 4>{}, ph == 0); break;
                        case 5: add_slice(std::integral_constant<int, 5>{}, ph == 0); break;
                        case 6: add_slice(std::integral_constant<int, 6>{}, ph == 0); break;
                        default: add_slice(std::integral_constant<int, 7>{}, ph == 0); break;
                    }
                } else {
                    // D = 64: four slices; waves 0-3 use phases 0-3, waves 4-7 phases 4-7
                    if ((ph >> 2) == (wave >> 2)) {
                        switch ((wave + ph) & 3) {
                            case 0: add_slice(std::integral_constant<int, 0>{}, ph == 0); break;
                            case 1: add_slice(std::integral_constant<int, 1>{}, ph == 0); break;
                            case 2: add_slice(std::integral_constant<int, 2>{}, ph == 0); break;
                            default: add_slice(std::integral_constant<int, 3>{}, ph == 0); break;
                        }
                    }
                }
                __syncthreads();
            }
        }
    }

    // ---- output: O = acc_sh / L with L = sum_w l_w 2^(M_w - Mc)
    {
        auto sw = __builtin_amdgcn_permlane32_swap(as_u32(l), as_u32(l), false, false);
        const float l_tot = as_f32(sw[0]) + as_f32(sw[1]);
        const bool fresh = seen == -INFINITY;
        if (hf == 0) {
            xl[wave * 32 + c] = fresh ? 0.f : l_tot * fast_exp2(M - Mc);
            if (wave == 0) xm[c] = Mc;
        }
    }
    __syncthreads();
    {
        constexpr int SEG = D / 16;             // d values per thread (512 threads, 32 rows)
        const int row = tid >> 4, seg = tid & 15;
        const int ir = i0 + row;
        if (ir >= N) return;
        float L = 0.f;
#pragma unroll
        for (int w = 0; w < 8; ++w) L += xl[w * 32 + row];
        const float inv = 1.f / L;
        const float *src = acc_sh + row * C::APITCH + seg * SEG;
        char *orow = p.o.ptr + b * p.o.sb + (int64_t)ir * p.o.sn + h * p.o.sh + seg * SEG * 2;
        char *rrow = p.o_lo.ptr ? p.o_lo.ptr + b * p.o_lo.sb + (int64_t)ir * p.o_lo.sn + h * p.o_lo.sh + seg * SEG * 2 : nullptr;
        float o[SEG];
#pragma unroll
        for (int x = 0; x < SEG; x += 4) {
            float4 v = *reinterpret_cast<const float4 *>(src + x);
            o[x] = v.x * inv;
            o[x + 1] = v.y * inv;
            o[x + 2] = v.z * inv;
            o[x + 3] = v.w * inv;
        }
        if constexpr (SEG == 8) {
            u32x4 ov, rv;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                ov[w] = pack_bf16(o[2 * w], o[2 * w + 1]);
                rv[w] = pack_bf16(o[2 * w] - bf16_lo(ov[w]), o[2 * w + 1] - bf16_hi(ov[w]));
            }
            st_global16(orow, ov);
            if (rrow) st_global16(rrow, rv);
        } else {
            u32x2 ov, rv;
#pragma unroll
            for (int w = 0; w < 2; ++w) {
                ov[w] = pack_bf16(o[2 * w], o[2 * w + 1]);
                rv[w] = pack_bf16(o[2 * w] - bf16_lo(ov[w]), o[2 * w + 1] - bf16_hi(ov[w]));
            }
            *reinterpret_cast<u32x2 *>(orow) = ov;
            if (rrow) *reinterpret_cast<u32x2 *>(rrow) = rv;
        }
        if (seg == 0) p.lse[((int64_t)b * p.H + h) * N + ir] = (xm[row] + __builtin_amdgcn_logf(L)) * kLn2;
    }
}

}  // namespace sa2
