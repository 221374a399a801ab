// Forward kernel, offset-split / tile-streaming variant (the production forward).
//
// One workgroup (4 waves, one per SIMD, up to 512 registers each) owns 32 query rows
// of one (batch, head).  The w2 offsets dlt = i - k are dealt round-robin to the waves,
// two at a time per wave ("streams"): in round r wave w handles dlt = 8r + 2w + {0,1}.
// All four waves therefore walk the SAME sequence of 32-row K1/V1 tiles, which is
// streamed through a small LDS ring once per round and shared by the 8 offsets in
// flight; A = q * k2_{i-dlt} is built once per (offset) instead of once per
// (offset, chunk), and each LDS operand fragment feeds two MFMAs (one per stream).
// Every wave keeps its own online-softmax state (m, l, acc) over its offsets; the four
// partial states are merged through LDS at the end (the usual split-softmax merge).
//
// LDS tiles are row-major [32 rows][D] bf16 with a padded pitch; K1 fragments are read
// with ds_read_b128, V1 fragments (needed transposed: rows = d, k-slots = j) with
// ds_read_b64_tr_b16.
#pragma once

#include <type_traits>

#include "sa2_common.hpp"

#ifndef SA2_SCHED
#define SA2_SCHED 1
#endif

namespace sa2 {

typedef short s16x4 __attribute__((ext_vector_type(4)));

// LDS tile: row-major [32 rows][D] bf16 with a padded pitch of D*2 + 16 bytes, so that
// the 32 rows a fragment read touches start 4 banks apart and every fragment address
// is one per-lane base register plus an immediate.
template <int D>
__host__ __device__ constexpr int tile_pitch() { return D * 2 + 16; }

// Transposed fragment read.  After the call, lane (c, hf) holds for w = 0..3 the
// element  tile[row_base + 4*hf + w][d_base + dmap_row(c)]  in result element w.
// ds_read_b64_tr_b16 works on groups of 16 lanes: result element w of lane 4a+col is
// element `col` of the 8-byte chunk addressed by lane 4w+a of the same group.
// `lane_base` = tile + tr_lane_off<D>(lane) carries the per-lane part of the address.
// Pitch of a tile that is only read through transposed reads: rows 16 banks (64 B)
// apart, so the 4 rows x 8 chunks of 8 bytes that 32 lanes read hit 64 distinct banks.
template <int D>
__host__ __device__ constexpr int tr_pitch() { return D * 2 + 64; }

template <int D, int P = tile_pitch<D>()>
__device__ __forceinline__ int tr_lane_off(int lane) {
    const int row = 4 * (lane >> 5) + ((lane & 15) >> 2);
    const int d = 16 * (lane & 1) + 8 * ((lane >> 4) & 1) + 4 * ((lane & 3) >> 1);
    return row * P + d * 2;
}
template <int D, int P = tile_pitch<D>()>
__device__ __forceinline__ u32x2 lds_read_tr(const char *lane_base, int row_base, int d_base) {
    const char *addr = lane_base + row_base * P + d_base * 2;
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(addr));
    return __builtin_bit_cast(u32x2, v);
}

template <int D>
struct FwdDs {
    static constexpr int KS = D / 16;
    static constexpr int DT = D / 32;
    static constexpr int TILE = 32 * tile_pitch<D>();  // bytes of one padded [32][D] bf16 tile
    static constexpr int NBUF = 4;
    static constexpr int STAGE = 2 * TILE;            // K1 tile + V1 tile
    static constexpr int RING = NBUF * STAGE;
    static constexpr int APITCH = D + 4;              // floats per row of a parked accumulator
    static constexpr int ACCS = 4 * 32 * APITCH * 4;  // per-wave output accumulators, fp32
    static constexpr int LDS = RING + ACCS + 4 * 32 * 4 * 2;
    static constexpr int PIECES = 32 * D / 8;         // 16-byte pieces per tile
    static constexpr int LPT = PIECES / 256;          // loads per thread per tile and tensor
};

template <int D>
__global__ __launch_bounds__(256, 1) void fwd_ds_kernel(KParams p) {
    using C = FwdDs<D>;
    constexpr int KS = C::KS, DT = C::DT, PPR = D / 8;
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
    const char *k1g = p.k1.ptr + b * p.k1.sb + hk * p.k1.sh;
    const char *v1g = p.v1.ptr + b * p.v1.sb + hk * p.v1.sh;
    const char *k2g = p.k2.ptr + b * p.k2.sb + hk * p.k2.sh;
    const char *v2g = p.v2.ptr + b * p.v2.sb + hk * p.v2.sh;

    const int t_lo = (i0 - p.w1 + 1 > 0 ? i0 - p.w1 + 1 : 0) / 32;
    const int t_hi = i0 / 32;
    const int NT = t_hi - t_lo + 1;
    const int nd = p.w2 < i0 + 32 ? p.w2 : i0 + 32;   // offsets that meet at least one valid k
    const int R = (nd + 7) / 8;
    const int U = R * NT;
    const float c2 = p.scale_log2e;
    constexpr int PITCH = tile_pitch<D>();

    // ---- tile staging: each thread moves LPT pieces of K1 and of V1 per tile
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
    const int k_lane = c * PITCH + 16 * hf;          // K1 fragment: row c, pieces 2*kk + hf
    const int v_lane = C::TILE + tr_lane_off<D>(lane);

    // The output accumulator of a wave is touched once per round only, so it is parked
    // in LDS (each lane reads and writes its own 16-d segments: no synchronisation).
    float *macc = reinterpret_cast<float *>(lds + C::RING);                 // [4][32][APITCH]
    float *my_acc = macc + (wave * 32 + c) * C::APITCH + 16 * hf;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) *reinterpret_cast<float4 *>(my_acc + 32 * dt + 4 * r4) = make_float4(0.f, 0.f, 0.f, 0.f);

    f32x16 T[2][DT];
    u32x4 A[2][KS];
    // Softmax state of this wave.  Exponentials are taken relative to a per-row
    // reference M that is FIXED while a round runs, so the hot loop never has to
    // rescale the T accumulators: x = s*scale*log2e - M may drift above 0, which costs
    // no precision in floating point.  M is re-centred on the running maximum between
    // rounds (when T is empty); only if x leaves [-32, 64] inside a round does the loop
    // drop to a slow path that rescales T.
    float M = 0.f;            // reference (log2 domain); meaningless while `seen` is -inf
    float seen = -INFINITY;   // running maximum of x relative to M; -inf: no valid entry yet
    float l = 0.f, acc_scale = 1.f;

    // ---- LDS ring of NBUF = 4 stages, indexed by the running tile counter u (tiles of
    // successive rounds follow each other).  Invariant at the top of the step that
    // consumes tile u: tiles u .. u+2 are in LDS, the data of tile u+3 sits in the
    // staging registers, the K1 fragments of tile u+1 are already in registers.
    int t_load = t_lo;                       // tile index (within the window) of the next global load
    auto advance_load = [&]() { t_load = (t_load == t_hi) ? t_lo : t_load + 1; };
    int buf_fill = 0, buf_use = 0;
    auto next_buf = [&](int b) { return b == C::NBUF - 1 ? 0 : b + 1; };
#pragma unroll
    for (int x = 0; x < 3; ++x) {
        issue_loads(t_load);
        advance_load();
        write_stage(buf_fill);
        buf_fill = next_buf(buf_fill);
    }
    issue_loads(t_load);
    advance_load();
    __syncthreads();

    u32x4 kf[KS];                            // K1 fragments of the tile whose logits are computed next
    auto load_kf = [&](int buf) {
        const char *kbase = lds + buf * C::STAGE + k_lane;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) kf[kk] = ld_lds16(kbase + 32 * kk);
    };
    load_kf(0);
    int buf_k = 1;                           // stage holding the tile after the one in kf

    f32x16 Xc[2];                            // processed logits (relative to M, log2 domain) of the current tile
    float tmax = 0.f;

    for (int r = 0; r < R; ++r) {
        bool col_ok[2], any_bad[2];
        int krc[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int dlt = 8 * r + 2 * wave + s;
            const int kr = i - dlt;
            col_ok[s] = row_ok && kr >= 0 && dlt < p.w2;
            any_bad[s] = wave_any(!col_ok[s]);
            krc[s] = kr < 0 ? 0 : (kr > N - 1 ? N - 1 : kr);
            const char *k2row = k2g + (int64_t)krc[s] * p.k2.sn;
#pragma unroll
            for (int kk = 0; kk < KS; ++kk)
                A[s][kk] = mul_bf16x8(ld_global16(qrow + (16 * kk + 8 * hf) * 2), ld_global16(k2row + (16 * kk + 8 * hf) * 2));
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) T[s][dt] = zero16();
        }

        float lp[4] = {0.f, 0.f, 0.f, 0.f};     // partial row sums of this round
        // logits of a tile from the fragments in kf: every fragment feeds both streams
        auto s_gemm = [&](f32x16 (&X)[2]) {
            X[0] = zero16();
            X[1] = zero16();
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) {
                X[0] = mfma32(kf[kk], A[0][kk], X[0]);
                X[1] = mfma32(kf[kk], A[1][kk], X[1]);
            }
        };
        // raw logits of tile t -> Xc (scaled, referenced, masked) and their row maximum
        auto post_s = [&](const f32x16 (&X)[2], int t, auto masked_tag) {
            constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int rr = 0; rr < 16; ++rr) Xc[s][rr] = X[s][rr] * c2 - M;
            if constexpr (MASKED) {
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int rr = 0; rr < 16; ++rr) {
                        int j = 32 * t + 8 * (rr >> 2) + 4 * hf + (rr & 3);
                        bool ok = col_ok[s] && (j <= i) && (j + p.w1 > i);
                        Xc[s][rr] = ok ? Xc[s][rr] : -INFINITY;
                    }
            }
            tmax = fmaxf(Xc[0][0], Xc[1][0]);
#pragma unroll
            for (int rr = 1; rr < 16; ++rr) tmax = fmaxf(tmax, fmaxf(Xc[0][rr], Xc[1][rr]));
            auto sw = __builtin_amdgcn_permlane32_swap(as_u32(tmax), as_u32(tmax), false, false);
            tmax = fmaxf(as_f32(sw[0]), as_f32(sw[1]));
        };
        // x must stay inside the safe exponent range.  The rare slow path moves the reference
        // of the rows that left it and rescales what the accumulators already hold; it is
        // kept OUT of the pipelined loop (the loop returns to it), because VALU code that
        // touches T inside the loop makes the compiler copy T out of the accumulation
        // registers on every iteration.
        auto out_of_range = [&]() {
            return wave_any(tmax > 64.f || (seen == -INFINITY && tmax < -32.f && tmax > -INFINITY));
        };
        auto slow_path = [&]() {
            const bool fresh = seen == -INFINITY;
            const bool move = tmax > 64.f || (fresh && tmax < -32.f && tmax > -INFINITY);
            const float shift = move ? tmax : 0.f;
            const float alpha = fresh ? 1.f : fast_exp2(-shift);   // fresh rows hold T = l = 0
#pragma unroll
            for (int s = 0; s < 2; ++s) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int rr = 0; rr < 16; ++rr) T[s][dt][rr] *= alpha;
#pragma unroll
                for (int rr = 0; rr < 16; ++rr) Xc[s][rr] -= shift;
            }
            l *= alpha;
#pragma unroll
            for (int x = 0; x < 4; ++x) lp[x] *= alpha;
            acc_scale *= alpha;
            M += shift;
            seen = fmaxf(seen - shift, tmax - shift);
        };
        // exponentials of the current tile -> packed bf16 B operands, row sums into l
        u32x4 pb[2][2];
        auto exps = [&]() {
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int rr = 0; rr < 16; rr += 2) {
                    float p0 = fast_exp2(Xc[s][rr]);
                    float p1 = fast_exp2(Xc[s][rr + 1]);
                    lp[(rr >> 1) & 3] += p0 + p1;
                    pb[s][rr >> 3][(rr & 7) >> 1] = pack_bf16(p0, p1);
                }
        };
        u32x2 vf[DT][2][2];
        auto load_vf = [&](int buf) {
            const char *vbase = lds + buf * C::STAGE + v_lane;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int k2s = 0; k2s < 2; ++k2s) {
                    vf[dt][k2s][0] = lds_read_tr<D>(vbase, 16 * k2s, 32 * dt);
                    vf[dt][k2s][1] = lds_read_tr<D>(vbase, 16 * k2s + 8, 32 * dt);
                }
        };
        auto t_gemm = [&]() {
#pragma unroll
            for (int k2s = 0; k2s < 2; ++k2s)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    u32x4 v = {vf[dt][k2s][0][0], vf[dt][k2s][0][1], vf[dt][k2s][1][0], vf[dt][k2s][1][1]};
                    T[0][dt] = mfma32(v, pb[0][k2s], T[0][dt]);
                    T[1][dt] = mfma32(v, pb[1][k2s], T[1][dt]);
                }
        };
        // barrier + refill of the ring: stage u+3 is written, the loads of tile u+4 issued
        auto sync_and_refill = [&]() {
            __syncthreads();
            write_stage(buf_fill);
            buf_fill = next_buf(buf_fill);
            issue_loads(t_load);
            advance_load();
        };

        // ---- round prologue: logits of the first tile (its K1 fragments are in kf)
        {
            f32x16 Xn[2];
            s_gemm(Xn);
            load_kf(buf_k);
            buf_k = next_buf(buf_k);
            post_s(Xn, t_lo, std::true_type{});
            if (out_of_range()) slow_path();
            else seen = fmaxf(seen, tmax);
        }
        // ---- pipelined steps: exponentials and T-GEMM of tile t overlap with the logit
        // GEMM and the logit post-processing of tile t+1
        int mid_lo = (i0 + 31 - p.w1 >= 0) ? (i0 + 31 - p.w1) / 32 + 1 : t_lo;
        if (any_bad[0] || any_bad[1]) mid_lo = t_hi;
        mid_lo = mid_lo > t_hi ? t_hi : mid_lo;
        // runs steps t .. t_end; returns true if it stopped early (t already advanced)
        // because the logits just produced left the safe range
        auto steps = [&](int &t, int t_end, auto masked_tag) -> bool {
            while (t <= t_end) {                 // consumes tile t, produces the logits of tile t+1
                sync_and_refill();
                load_vf(buf_use);
                buf_use = next_buf(buf_use);
                f32x16 Xn[2];
                s_gemm(Xn);
                exps();
                load_kf(buf_k);
                buf_k = next_buf(buf_k);
                t_gemm();
                post_s(Xn, t + 1, masked_tag);
#if SA2_SCHED
                // phase 1: 16 logit MFMAs, each followed by a share of the exponential work
                // and one of the 16 transposed V1 fragment reads
#pragma unroll
                for (int x = 0; x < 16; ++x) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
                }
                // phase 2: 16 value MFMAs, each followed by a share of the post-processing
                // of the next logits; the first 8 also by one K1 fragment read
#pragma unroll
                for (int x = 0; x < 16; ++x) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (x < 8) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
                }
#endif
                ++t;
                if (out_of_range()) return true;
                seen = fmaxf(seen, tmax);
            }
            return false;
        };
        auto run_segment = [&](int t, int t_end, auto masked_tag) {
            while (t <= t_end && steps(t, t_end, masked_tag)) slow_path();
        };
        run_segment(t_lo, mid_lo - 2, std::true_type{});                    // tile t+1 in the masked head
        run_segment(mid_lo - 1 > t_lo ? mid_lo - 1 : t_lo, t_hi - 2, std::false_type{});   // t+1 unmasked
        if (t_hi > t_lo) run_segment(t_hi - 1, t_hi - 1, std::true_type{});  // t+1 = diagonal tile
        // ---- last tile of the round: nothing to overlap with
        sync_and_refill();
        load_vf(buf_use);
        buf_use = next_buf(buf_use);
        exps();
        t_gemm();
        l += (lp[0] + lp[1]) + (lp[2] + lp[3]);

        // ---- round end: O_i = (O_i * acc_scale + v2_{i-dlt} * T_i) re-centred on the
        // running maximum, so that the next round starts with x <= 0 for what was seen
        {
            const bool fresh = seen == -INFINITY;
            const float shift = fresh ? 0.f : seen;
            const float f = fast_exp2(-shift);
            const float fs = acc_scale * f;
            const char *va = v2g + (int64_t)krc[0] * p.v2.sn + 16 * hf * 2;
            const char *vb = v2g + (int64_t)krc[1] * p.v2.sn + 16 * hf * 2;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const u32x4 xa = ld_global16(va + dt * 64 + half * 16);
                    const u32x4 xb = ld_global16(vb + dt * 64 + half * 16);
#pragma unroll
                    for (int q4 = 0; q4 < 2; ++q4) {
                        float *dst = my_acc + 32 * dt + 8 * half + 4 * q4;
                        float4 a = *reinterpret_cast<float4 *>(dst);
                        const int rr = 8 * half + 4 * q4;
                        a.x = a.x * fs + (bf16_lo(xa[2 * q4]) * T[0][dt][rr] + bf16_lo(xb[2 * q4]) * T[1][dt][rr]) * f;
                        a.y = a.y * fs + (bf16_hi(xa[2 * q4]) * T[0][dt][rr + 1] + bf16_hi(xb[2 * q4]) * T[1][dt][rr + 1]) * f;
                        a.z = a.z * fs + (bf16_lo(xa[2 * q4 + 1]) * T[0][dt][rr + 2] + bf16_lo(xb[2 * q4 + 1]) * T[1][dt][rr + 2]) * f;
                        a.w = a.w * fs + (bf16_hi(xa[2 * q4 + 1]) * T[0][dt][rr + 3] + bf16_hi(xb[2 * q4 + 1]) * T[1][dt][rr + 3]) * f;
                        *reinterpret_cast<float4 *>(dst) = a;
                    }
                }
            l *= f;
            M += shift;
            seen = fresh ? -INFINITY : 0.f;
            acc_scale = 1.f;
        }
    }
    const float m = (seen == -INFINITY) ? -INFINITY : M;

    // ---- merge the four per-wave softmax states
    float *mm = reinterpret_cast<float *>(lds + C::RING + C::ACCS);    // [4][32]
    float *ml = mm + 4 * 32;                                            // [4][32]
    {
        auto sw = __builtin_amdgcn_permlane32_swap(as_u32(l), as_u32(l), false, false);
        const float l_tot = as_f32(sw[0]) + as_f32(sw[1]);
        if (hf == 0) {
            mm[wave * 32 + c] = m;
            ml[wave * 32 + c] = l_tot;
        }
    }
    __syncthreads();
    {
        constexpr int SEG = D / 8;              // d values per thread
        const int row = tid >> 3, seg = tid & 7;
        const int ir = i0 + row;
        if (ir >= N) return;
        float mw[4], M = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            mw[w] = mm[w * 32 + row];
            M = fmaxf(M, mw[w]);
        }
        float f[4], L = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            f[w] = (mw[w] == -INFINITY) ? 0.f : fast_exp2(mw[w] - M);
            L += f[w] * ml[w * 32 + row];
        }
        const float inv = 1.f / L;
        float o[SEG];
#pragma unroll
        for (int x = 0; x < SEG; ++x) o[x] = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float *src = macc + (w * 32 + row) * C::APITCH + seg * SEG;
#pragma unroll
            for (int x = 0; x < SEG; x += 4) {
                float4 v = *reinterpret_cast<const float4 *>(src + x);
                o[x] += f[w] * v.x;
                o[x + 1] += f[w] * v.y;
                o[x + 2] += f[w] * v.z;
                o[x + 3] += f[w] * v.w;
            }
        }
        char *orow = p.o.ptr + b * p.o.sb + (int64_t)ir * p.o.sn + h * p.o.sh + seg * SEG * 2;
        char *rrow = p.o_lo.ptr ? p.o_lo.ptr + b * p.o_lo.sb + (int64_t)ir * p.o_lo.sn + h * p.o_lo.sh + seg * SEG * 2 : nullptr;
#pragma unroll
        for (int x = 0; x < SEG; x += 8) {
            u32x4 ov, rv;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float x0 = o[x + 2 * w] * inv, x1 = o[x + 2 * w + 1] * inv;
                ov[w] = pack_bf16(x0, x1);
                rv[w] = pack_bf16(x0 - bf16_lo(ov[w]), x1 - bf16_hi(ov[w]));
            }
            st_global16(orow + x * 2, ov);
            if (rrow) st_global16(rrow + x * 2, rv);
        }
        if (seg == 0) p.lse[((int64_t)b * p.H + h) * N + ir] = (M + __builtin_amdgcn_logf(L)) * kLn2;
    }
}

}  // namespace sa2
