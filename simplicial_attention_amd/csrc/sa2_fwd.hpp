// Forward kernel (eight waves, two per SIMD).
//
// One workgroup owns 32 query rows of one (batch, head).  In round r wave w handles the
// offset dlt = i - k = 8r + w (any second window: ceil(w2 / 8) rounds); all eight waves walk
// the same 32-row K1/V1 tiles, which stream through a four-buffer LDS ring (direct-to-LDS loads,
// layout DmaTile of sa2_lds.hpp), one tile and one barrier per step.  Per (offset, tile):
//     S^T = K1 A^T          A = q_i * k2_{i-dlt} * scale * log2(e)   (bf16, built once per offset)
//     P^T = exp2(S^T - M_i)                 (the MFMA chain starts from -M_i: no VALU subtraction)
//     T^T += V1^T P^T       (V1 fragments through ds_read_b64_tr_b16)
// Measured on MI355X: a 32x32x16 MFMA occupies the SIMD's issue port for about 15 of its 36-38
// cycles and every other VALU instruction for about 4.9, from either wave of the SIMD: four to five
// VALU instructions per MFMA hide behind it and none beyond that.
// So the per-tile VALU work is kept to the exponentials, the bf16 packing and the row sums:
//   - the softmax reference M of a row is fixed by the first tile of the wave's first offset
//     (the diagonal tile, which every valid row attends) and moves only when a row sum says
//     that weights grew beyond 2^90 (a branch that is almost never taken);
//   - masks are applied on the diagonal tile and on the (at most two) tiles that the window's
//     lower edge crosses; the tiles in between run without mask code;
//   - fragment reads are spread between the MFMAs (a scheduling fence behind every MFMA and its reads):
//     the V1 fragments of a tile along its logit chain, the K1 fragments of the next tile along the
//     value chain.
// The output accumulator is shared: an fp32 [32][D] LDS buffer relative to a common reference
// Mc.  At the end of a round the waves publish their references, agree on Mc = max, and add
// v2_{i-dlt} * T * 2^(M - Mc) (formed in place in T first) in eight barrier-separated phases; in phase ph wave w owns the
// d-slice (w + ph) mod 8, so concurrent waves never touch the same element and every element
// sees its additions in a fixed order (bitwise reproducible, no atomics).
// The k2/v2 rows live in a 64-row circular LDS buffer (row k in slot (k - i0) mod 64), filled before the first round
// with the rows k - i0 = -32 .. 31, which is all that second windows up to 32 ever read; a round needs 39 rows, and
// from the fourth round on the 8 rows that the next round adds are fetched while the round's results are added to
// the shared accumulator.
#pragma once

#include <type_traits>

#include "sa2_common.hpp"
#include "sa2_lds.hpp"

namespace sa2 {

template <int D>
struct FwdCfg {
    static constexpr int KS = D / 16;
    static constexpr int DT = D / 32;
    static constexpr int PITCH = tile_pitch<D>();     // staged q / k2 / v2 rows
    static constexpr int TILE = 32 * PITCH;
    // K1 / V1 ring tiles are written by direct-to-LDS loads (layout: DmaTile)
    using RT = DmaTile<D>;
    static constexpr int RPC = RT::RPC, NCH = RT::NCH, CP = RT::CP;
    static constexpr int DTILE = RT::BYTES;
    static constexpr int BUF = 2 * DTILE;             // one ring buffer: a K1 tile and a V1 tile
    static constexpr int NBUF = 4;
    static constexpr int RING = NBUF * BUF;
    static constexpr int APITCH = D + 4;              // floats per row of the shared accumulator
    static constexpr int ACC = 32 * APITCH * 4;
    static constexpr int EXCH = 8 * 32 * 4;           // one float per (wave, row)
    // q rows of the tile [32][QPITCH bytes]: fp32 times scale log2(e); at D = 64 bf16 (the instance then fits 80 KiB of
    // LDS and 128 registers: two workgroups per CU)
    static constexpr bool QF = D != 64;
    // waves per SIMD the instance is compiled for: D = 128 needs 236 registers (one workgroup per CU); D = 64 is held
    // to 128 registers (a few spills outside the step's MFMA blocks) so that two workgroups share a CU, which is worth
    // 20 % at D = 64; D = 32 fits by itself
    static constexpr int WPE = D == 128 ? 2 : 4;
    // fragments in flight per operand and chain: a rolling window of four of the eight at D = 128; two of the four at
    // D = 64, where four waves per SIMD cover the latency and the registers are the scarcer resource
    static constexpr int FW = D == 64 ? 2 : (KS < 4 ? KS : 4);
    static constexpr int QS = RING + ACC + 2 * EXCH;
    static constexpr int QPITCH = QF ? D * 4 + 16 : tile_pitch<D>();
    static constexpr int KSLOTS = 64;                 // circular k2 / v2 rows
    static constexpr int K2S = QS + 32 * QPITCH;
    static constexpr int V2S = K2S + KSLOTS * PITCH;
    static constexpr int MASKS = V2S + KSLOTS * PITCH; // additive masks (0 / -inf) of the diagonal tile and of up to two lower-edge tiles
    static constexpr int MASK = 16 * 64 * 4;          // one table: [4 quarters][64 lanes][4 floats]
    static constexpr int LDS = MASKS + 3 * MASK;
    static_assert(D == 128 || 2 * LDS <= 160 * 1024, "two workgroups per CU need half the LDS each");
    static_assert(RING - CP < 65536, "the LDS address of a direct load travels in 16 bits of M0");
    static constexpr int PPR = D / 8;                 // 16-byte pieces per row
    static constexpr int PIECES = 32 * PPR;           // ... per tile
};

template <int D>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(FwdCfg<D>::WPE, FwdCfg<D>::WPE))) void fwd_kernel(KParams p) {
    using C = FwdCfg<D>;
    constexpr int KS = C::KS, DT = C::DT, PPR = C::PPR, PITCH = C::PITCH;
    constexpr float kBig = 1.2379400392853803e27f;    // 2^90: row sums beyond it move the reference
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

    // tiles of the first window; sequence of a round: the diagonal tile first, then t_lo .. t_hi - 1
    const int t_lo = (i0 - p.w1 + 1 > 0 ? i0 - p.w1 + 1 : 0) / 32;
    const int t_hi = i0 / 32;
    const int NT = t_hi - t_lo + 1;
    int mid_lo = (i0 + 31 - p.w1 >= 0) ? (i0 + 31 - p.w1) / 32 + 1 : t_lo;   // first tile below the diagonal that no row masks
    mid_lo = mid_lo > t_hi ? t_hi : mid_lo;
    const int n_masked = 1 + (mid_lo - t_lo);         // leading steps of a round that need a mask (at most 3)
    const int nd = p.w2 < i0 + 32 ? p.w2 : i0 + 32;   // offsets that meet at least one valid k
    const int R = (nd + 7) / 8;
    const int U = R * NT;
    auto tile_of = [&](int n) { return n == 0 ? t_hi : t_lo + n - 1; };

    // ---- ring staging: direct-to-LDS loads, wave w moves chunk(s) w of the K1 tile and of the V1 tile.  Lane p of a
    // chunk load fetches row (p / 4) % RPC, segment p / (4 RPC), piece p % 4 of the segment
    const bool stager = C::NCH >= 8 || wave < C::NCH;            // D = 64: four chunks per tile, waves 0-3 stage
    const int st_row = C::RT::st_row(wave % C::NCH, lane), st_col = C::RT::st_col(lane);
    int n_load = 0;                                   // sequence index (within the round) of the next load
    int b_load = 0;                                   // ring buffer of the next load
    // address = tile base (uniform, on the scalar unit) + this lane's row and column (32 bits); only
    // the diagonal tile can reach past the last row, so only it needs a clamped row
    const int st_row_diag = i0 + st_row < N ? st_row : N - 1 - i0;
    const uint32_t so_k = (uint32_t)(st_row * (int)p.k1.sn + st_col), so_v = (uint32_t)(st_row * (int)p.v1.sn + st_col);
    const uint32_t so_k_diag = (uint32_t)(st_row_diag * (int)p.k1.sn + st_col), so_v_diag = (uint32_t)(st_row_diag * (int)p.v1.sn + st_col);
    const uint32_t lds_chunk = (uint32_t)(uintptr_t)lds + (wave % C::NCH) * C::CP;
    // tile bases as running pointers: the diagonal tile, then t_lo, t_lo + 1, ... (no multiplications in the step)
    const char *const k_diag = k1g + (int64_t)(32 * t_hi) * p.k1.sn, *const v_diag = v1g + (int64_t)(32 * t_hi) * p.v1.sn;
    const char *const k_low = k1g + (int64_t)(32 * t_lo) * p.k1.sn, *const v_low = v1g + (int64_t)(32 * t_lo) * p.v1.sn;
    const int64_t k_step = 32 * p.k1.sn, v_step = 32 * p.v1.sn;
    const char *kb = k_diag, *vb = v_diag;
    // Loads are issued at every step, also behind the last tile a round needs (the sequence of tiles simply runs
    // on, into buffers that no wave reads any more): every step then waits for the same number of transfers and
    // the step has no branch on the position in the sequence.  The kernel waits for the last ones before it ends.
    auto issue_loads = [&]() {
        if (stager) {
            load_to_lds16(kb, n_load == 0 ? so_k_diag : so_k, lds_chunk + b_load);
            load_to_lds16(vb, n_load == 0 ? so_v_diag : so_v, lds_chunk + b_load + C::DTILE);
        }
        const bool wrap = n_load == NT - 1;
        kb = wrap ? k_diag : (n_load == 0 ? k_low : kb + k_step);
        vb = wrap ? v_diag : (n_load == 0 ? v_low : vb + v_step);
        n_load = wrap ? 0 : n_load + 1;
        b_load = (b_load == (C::NBUF - 1) * C::BUF) ? 0 : b_load + C::BUF;
    };
    // K1 fragment kk of row c: segment kk / 2, pieces 2 (kk % 2) + hf
    const int k_lane = C::RT::row_lane(lane);
    // V1 transposed read: the lane's 8 bytes of row 4 hf + (lane % 16) / 4, d = 16 (lane & 1) + 8 (lane / 16 % 2) + 4 (lane % 4 / 2)
    const int v_lane = C::DTILE + C::RT::tr_lane(lane);

    // ---- shared output accumulator and exchange areas
    float *acc_sh = reinterpret_cast<float *>(lds + C::RING);              // [32][APITCH]
    float *xm = reinterpret_cast<float *>(lds + C::RING + C::ACC);         // [8][32] references
    float *xl = xm + 8 * 32;                                               // [8][32] row sums
    for (int x = tid; x < 32 * C::APITCH / 4; x += 512) reinterpret_cast<float4 *>(acc_sh)[x] = make_float4(0.f, 0.f, 0.f, 0.f);
    float Mc = -INFINITY;      // common reference of acc_sh (same value in every wave)

    // ---- the q rows of the tile and the k2/v2 rows of the first round, staged before the loop
    {
        const char *qg = p.q.ptr + b * p.q.sb + h * p.q.sh;
        for (int x = tid; x < 32 * PPR; x += 512) {
            const int row = x / PPR, col = (x % PPR) * 16;
            int ii = i0 + row;
            ii = ii < N ? ii : N - 1;
            const u32x4 fq = ld_global16(qg + (int64_t)ii * p.q.sn + col);
            if constexpr (C::QF) {
                // unpacked and scaled once per workgroup: the operand build of every offset then multiplies without
                // unpacking or scaling q again
                const float c2 = p.scale_log2e;
                float4 *dst = reinterpret_cast<float4 *>(lds + C::QS + row * C::QPITCH + col * 2);
                dst[0] = make_float4(bf16_lo(fq[0]) * c2, bf16_hi(fq[0]) * c2, bf16_lo(fq[1]) * c2, bf16_hi(fq[1]) * c2);
                dst[1] = make_float4(bf16_lo(fq[2]) * c2, bf16_hi(fq[2]) * c2, bf16_lo(fq[3]) * c2, bf16_hi(fq[3]) * c2);
            } else {
                *reinterpret_cast<u32x4 *>(lds + C::QS + row * C::QPITCH + col) = fq;
            }
        }
        // rows k - i0 = -32 .. 31 fill the 64 slots: the first four rounds find their rows here
        for (int x = tid; x < 64 * PPR; x += 512) {
            const int row = x / PPR, col = (x % PPR) * 16;
            int kk2 = i0 - 32 + row;
            kk2 = kk2 < 0 ? 0 : (kk2 < N ? kk2 : N - 1);
            const int slot = (row - 32) & 63;
            *reinterpret_cast<u32x4 *>(lds + C::K2S + slot * PITCH + col) = ld_global16(k2g + (int64_t)kk2 * p.k2.sn + col);
            *reinterpret_cast<u32x4 *>(lds + C::V2S + slot * PITCH + col) = ld_global16(v2g + (int64_t)kk2 * p.v2.sn + col);
        }
    }
    // additive masks: table 0 for the diagonal tile, tables 1, 2 for the tiles the lower window edge
    // crosses.  Entry (lane, rr) is 0 if query row i0 + c attends key row 32 t + 4 hf + e(rr), else -inf
    for (int x = tid; x < 3 * 256; x += 512) {
        const int tab = x >> 8, qq = (x >> 6) & 3, ln = x & 63;
        const int t = tab == 0 ? t_hi : t_lo + tab - 1;
        const int rel = (ln & 31) + 32 * (t_hi - t) - 4 * (ln >> 5);
        float4 m4;
        float *mp = &m4.x;
#pragma unroll
        for (int e = 0; e < 4; ++e) mp[e] = ((unsigned)(rel - (8 * qq + e)) < (unsigned)p.w1) ? 0.f : -INFINITY;
        *reinterpret_cast<float4 *>(lds + C::MASKS + tab * C::MASK + qq * 1024 + ln * 16) = m4;
    }
    // the 8 rows that round r + 1 adds (k - i0 = -8r - 15 .. -8r - 8), one 16-byte piece per thread; only rounds
    // beyond the fourth add rows that the prologue has not staged
    auto adds_rows = [&](int r) { return r + 1 < R && r + 1 >= 4; };
    const bool row_stager = tid < 2 * 8 * PPR;
    const int rs_sel = tid / (8 * PPR), rs_row = (tid / PPR) % 8, rs_col = (tid % PPR) * 16;
    u32x4 st_r = {0u, 0u, 0u, 0u};
    auto issue_rows = [&](int r) {
        if (row_stager) {
            int kk2 = i0 - 8 * r - 15 + rs_row;
            kk2 = kk2 < 0 ? 0 : (kk2 < N ? kk2 : N - 1);
            st_r = ld_global16((rs_sel ? v2g + (int64_t)kk2 * p.v2.sn : k2g + (int64_t)kk2 * p.k2.sn) + rs_col);
        }
    };
    auto write_rows = [&](int r) {
        if (row_stager) {
            const int slot = (-8 * r - 15 + rs_row) & 63;
            *reinterpret_cast<u32x4 *>(lds + (rs_sel ? C::V2S : C::K2S) + slot * PITCH + rs_col) = st_r;
        }
    };

    // accumulator clears: as 64-bit moves where registers are plentiful (at four waves per SIMD the register pairs
    // they need cost more in spilled registers than the moves save)
    auto clear16 = [] {
        if constexpr (C::WPE == 2) return zero16_pairs();
        else return zero16();
    };
    f32x16 T[DT];
    u32x4 A[KS];
    // Fragments travel through rolling windows of FW register sets: fragment f of a chain sits in set f % FW and is
    // requested FW MFMAs before its use, the first FW fragments of a chain along the tail of the chain before
    constexpr int FW = C::FW;
    u32x4 kf[FW];              // K1 fragments (row fragments)
    u32x2 vf[FW][2];           // V1 fragments (two transposed reads each)
    float M = 0.f;             // softmax reference of the row (log2 domain); meaningless while `fresh`
    bool fresh = true;         // the row has not met an attended entry yet
    float l = 0.f;             // this lane's part of the row sum, relative to M

    // ring protocol: step u lives in buffer u % 4.  Its transfer starts behind the barrier of step u - 3 (every wave
    // has then finished step u - 4, the last reader of that buffer) and must have landed before the barrier of step
    // u - 1, in which its K1 fragments are read: two steps of time for the memory latency.
    int b_cur = 0, b_nxt = C::BUF;
    issue_loads();
    issue_loads();
    issue_loads();
    int u = 0;
    wait_loads<0>();
    // start of step u: the tile of step u + 1 has landed (at most the transfers of step u + 2 are still in flight),
    // everything is published, the transfer of step u + 3 starts
    // (work placed right behind a barrier runs with an empty MFMA pipe: the steps issue their loads behind the first
    // MFMA of the logit chain and prepare the chain's start value ahead of the barrier)
    auto open_step_barrier = [&]() {
        if (stager) wait_loads<2>();
        __syncthreads();
    };
    auto open_step = [&]() {
        open_step_barrier();
        issue_loads();
    };
    auto close_step = [&]() {
        b_cur = b_nxt;
        b_nxt = (b_nxt == (C::NBUF - 1) * C::BUF) ? 0 : b_nxt + C::BUF;
        ++u;
    };
    __syncthreads();           // the staged rows, the mask tables and the zeroed accumulator are visible

    for (int r = 0; r < R; ++r) {
        const int dlt = 8 * r + wave;
        const int kr = i - dlt;
        const bool col_ok = row_ok && kr >= 0 && dlt < p.w2;
        const bool wave_on = wave_any(col_ok);
        const int slot = (c - dlt) & 63;              // slot of row k = i - dlt in the circular k2/v2 rows
        {
            const char *k2row = lds + C::K2S + slot * PITCH + 16 * hf;
            if constexpr (C::QF) {
                const char *qr = lds + C::QS + c * C::QPITCH + 32 * hf;
#pragma unroll
                for (int kk = 0; kk < KS; ++kk) {
                    const float4 qa = *reinterpret_cast<const float4 *>(qr + 64 * kk), qb = *reinterpret_cast<const float4 *>(qr + 64 * kk + 16);
                    const u32x4 fk = ld_lds16(k2row + 32 * kk);
                    A[kk][0] = pack_bf16(qa.x * bf16_lo(fk[0]), qa.y * bf16_hi(fk[0]));
                    A[kk][1] = pack_bf16(qa.z * bf16_lo(fk[1]), qa.w * bf16_hi(fk[1]));
                    A[kk][2] = pack_bf16(qb.x * bf16_lo(fk[2]), qb.y * bf16_hi(fk[2]));
                    A[kk][3] = pack_bf16(qb.z * bf16_lo(fk[3]), qb.w * bf16_hi(fk[3]));
                }
            } else {
                const char *qr = lds + C::QS + c * C::QPITCH + 16 * hf;
                const float c2 = p.scale_log2e;
#pragma unroll
                for (int kk = 0; kk < KS; ++kk) {
                    const u32x4 fq = ld_lds16(qr + 32 * kk), fk = ld_lds16(k2row + 32 * kk);
#pragma unroll
                    for (int w = 0; w < 4; ++w)
                        A[kk][w] = pack_bf16(bf16_lo(fq[w]) * c2 * bf16_lo(fk[w]), bf16_hi(fq[w]) * c2 * bf16_hi(fk[w]));
                }
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) T[dt] = clear16();
        }

        // exponentials and row sums of the tile whose referenced logits are in X
        auto exponentials = [&](const f32x16 &X, u32x4 (&pb)[2]) {
            // (the row sum takes the unrounded weights: v_dot2c_f32_bf16 on the packed pairs would be exact
            // for what the MFMA consumes, but dot instructions share the MFMA pipe and stall the other
            // wave's chains; the two sums differ by the mean of bf16 rounding errors, far below bf16 eps)
            float ls = l;
#pragma unroll
            for (int rr = 0; rr < 16; rr += 2) {
                const float e0 = fast_exp2(X[rr]), e1 = fast_exp2(X[rr + 1]);
                ls += e0 + e1;
                pb[rr >> 3][(rr & 7) >> 1] = pack_bf16(e0, e1);
            }
            l = ls;
        };
        // fragment reads of a step: the V1 fragments of the tile behind its logit chain, the K1 fragments of
        // the next tile in front of the value chain (they arrive behind it and the barrier)
        auto load_kf = [&](int buf_off) {
            const char *kbase = lds + buf_off + k_lane;
#pragma unroll
            for (int kk = 0; kk < FW; ++kk) kf[kk] = ld_lds16(kbase + C::RT::row_imm(kk));
        };
        // The fragment reads of a step sit between its MFMAs, a scheduling fence behind every MFMA and its reads
        // keeps them there: the V1 fragments of the tile along its logit chain, the K1 fragments of the next tile
        // along the value chain.
        // (the K1 fragments behind the round's last tile are those of the next round's first tile: the ring runs on)
        auto read_vf = [&](const char *vbase, int f) {
            const int k2s = f / DT, dt = f % DT;
            vf[f % FW][0] = lds_read_tr<D, 0>(vbase + C::RT::tr_imm(16 * k2s, 32 * dt), 0, 0);
            vf[f % FW][1] = lds_read_tr<D, 0>(vbase + C::RT::tr_imm(16 * k2s + 8, 32 * dt), 0, 0);
        };
        auto value_products = [&](const u32x4 (&pb)[2]) {
            const char *kbase = lds + b_nxt + k_lane;
            const char *vbase = lds + b_cur + v_lane;
#pragma unroll
            for (int m = 0; m < KS; ++m) {
                const int k2s = m / DT, dt = m % DT;
                u32x4 v = {vf[m % FW][0][0], vf[m % FW][0][1], vf[m % FW][1][0], vf[m % FW][1][1]};
                T[dt] = mfma32(v, pb[k2s], T[dt]);
                if (m + FW < KS) read_vf(vbase, m + FW);
                if (m >= KS - FW) kf[m - (KS - FW)] = ld_lds16(kbase + C::RT::row_imm(m - (KS - FW)));
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        auto logit_chain = [&](f32x16 &X, auto loads_tag) {
            const char *kbase = lds + b_cur + k_lane;
            const char *vbase = lds + b_cur + v_lane;
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) {
                X = mfma32(kf[kk % FW], A[kk], X);
                if constexpr (decltype(loads_tag)::value) {
                    if (kk == 0) issue_loads();
                }
                if (kk + FW < KS) kf[kk % FW] = ld_lds16(kbase + C::RT::row_imm(kk + FW));
                if (kk >= KS - FW) read_vf(vbase, kk - (KS - FW));
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // moves the reference of this lane's row up by `shift` (log2 units): what T and l hold is rescaled
        // (alpha = 2^-shift, or 1 for a row that holds nothing yet)
        auto shift_reference = [&](float shift, float alpha, f32x16 &X) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int rr = 0; rr < 16; ++rr) T[dt][rr] *= alpha;
#pragma unroll
            for (int rr = 0; rr < 16; ++rr) X[rr] -= shift;
            l *= alpha;
            M += shift;
        };
        auto row_max = [&](const f32x16 &X) {
            float tmax = X[0];
#pragma unroll
            for (int rr = 1; rr < 16; ++rr) tmax = fmaxf(tmax, X[rr]);
            auto sw = __builtin_amdgcn_permlane32_swap(as_u32(tmax), as_u32(tmax), false, false);
            return fmaxf(as_f32(sw[0]), as_f32(sw[1]));
        };

        if (wave_on) load_kf(b_cur);    // the round's first tile (its buffer was published at least one barrier ago)
        if (!wave_on) {
            // no valid (row, offset) in this wave: it only keeps the ring going
            // (a wave that is off stays off: later rounds only have larger offsets, so its fragment
            // registers need not follow the ring)
            for (int n = 0; n < NT; ++n) {
                open_step();
                close_step();
            }
        } else {
            int n = 0;
            if (r == 0) {
                // ---- the wave's very first step, the diagonal tile of its first offset: every valid row
                // attends an entry of it, so this is where the rows get their softmax reference M
                open_step();
                f32x16 X = clear16();
                logit_chain(X, std::false_type{});
                {
                    // row j = 32 t + 4 hf + e (e = 8 (rr / 4) + rr % 4) is attended iff 0 <= i - j < w1;
                    // lanes without a valid k2 row get a distance no e can bring into range
                    const int rel = col_ok ? c - 4 * hf : -(1 << 30);
#pragma unroll
                    for (int rr = 0; rr < 16; ++rr) {
                        const bool ok = (unsigned)(rel - (8 * (rr >> 2) + (rr & 3))) < (unsigned)p.w1;
                        X[rr] = ok ? X[rr] : -INFINITY;
                    }
                }
                const float tmax = row_max(X);
                if (tmax > -INFINITY) {
                    M = tmax;
                    fresh = false;
#pragma unroll
                    for (int rr = 0; rr < 16; ++rr) X[rr] -= tmax;
                }
                u32x4 pb[2];
                exponentials(X, pb);
                value_products(pb);
                close_step();
                n = 1;
            }
            // ---- all other steps.  The logit chain starts from -M (from -inf in lanes without a valid
            // (row, offset)), plus an additive 0 / -inf mask from an LDS table on the diagonal tile and on the
            // tiles that the window's lower edge crosses, so its result is the exponent and no mask or
            // subtraction code follows it.  A row's reference moves only if its row sum says that weights
            // outgrew the safe range.
            float nm = col_ok ? -M : -INFINITY;
            // the chains' start value, kept in registers where they are plentiful (eight moves per step instead of sixteen)
            f32x16 NMv;
            if constexpr (C::WPE == 2) NMv = splat16(nm);
            u32x4 pb[2];
            for (; n < NT; ++n) {
                f32x16 X;
                if constexpr (C::WPE == 2) X = NMv;
                else X = splat16(nm);
                if (n < n_masked) {
                    const char *mk = lds + C::MASKS + n * C::MASK + lane * 16;
#pragma unroll
                    for (int qq = 0; qq < 4; ++qq) {
                        const float4 m4 = *reinterpret_cast<const float4 *>(mk + qq * 1024);
                        X[4 * qq] += m4.x;
                        X[4 * qq + 1] += m4.y;
                        X[4 * qq + 2] += m4.z;
                        X[4 * qq + 3] += m4.w;
                    }
                }
                open_step_barrier();
                logit_chain(X, std::true_type{});
                const float l_before = l;
                exponentials(X, pb);
                if (__builtin_expect(wave_any(!(l < kBig)), 0)) {
                    // rare: some row's weights outgrew the safe range; move its reference and redo the tile's weights
                    const float tmax = row_max(X);
                    auto sw = __builtin_amdgcn_permlane32_swap(as_u32(l), as_u32(l), false, false);
                    const float l_row = fmaxf(as_f32(sw[0]), as_f32(sw[1]));
                    const bool over = !(l_row < kBig);
                    l = l_before;
                    const float lb = fmaxf(l_before, 1.f);
                    auto sw2 = __builtin_amdgcn_permlane32_swap(as_u32(lb), as_u32(lb), false, false);
                    const float e_old = (float)(__builtin_amdgcn_frexp_expf(fmaxf(as_f32(sw2[0]), as_f32(sw2[1]))) - 32);
                    const float shift = over ? fmaxf(fmaxf(tmax, e_old), 0.f) : 0.f;
                    shift_reference(shift, fast_exp2(-shift), X);
                    nm = col_ok ? -M : -INFINITY;
                    if constexpr (C::WPE == 2) NMv = splat16(nm);
                    exponentials(X, pb);
                }
                value_products(pb);
                close_step();
            }
        }

        // ---- round end: agree on the common reference, add v2 * T into the shared rows
        {
            if (adds_rows(r)) issue_rows(r);   // the rows that the next round adds arrive behind the phases below
            if (hf == 0) xm[wave * 32 + c] = fresh ? -INFINITY : M;
            __syncthreads();
            float Mn = Mc;
#pragma unroll
            for (int w = 0; w < 8; ++w) Mn = fmaxf(Mn, xm[w * 32 + c]);
            const float fo = (Mc == -INFINITY) ? 0.f : fast_exp2(Mc - Mn);   // rescale of the old content
            const float g = (fresh || !wave_on) ? 0.f : fast_exp2(M - Mn);   // weight of this wave's T
            // by-product for the backward: this offset's T (packed and stored slice by slice in the phases below: a
            // wave's stores issued in one go block it for thousands of cycles in front of a barrier) and its reference
            const bool save = p.t_save && row_ok && dlt < p.w2;
            // (T goes to one block of 32 rows per offset and tile, in the order the lanes hold it: a store of the wave
            // covers 1 KiB of consecutive bytes)
            const int64_t sbh = ((int64_t)b * p.H + h) * p.w2 + dlt;
            const int64_t srow_g = sbh * N + i;
            char *trow = p.t_save + (sbh * ntile + tile) * saved_t_block<D>() + saved_t_offset(c, hf, 0, 0);
            if (save && hf == 0) p.m_save[srow_g] = fresh ? 0.f : M;
            Mc = Mn;
            // the round's contribution of this wave is v2_{i-dlt} * T * g, formed slice by slice inside the phases (the
            // products then ride on the latency of the phase's LDS reads)
            const char *v2row = lds + C::V2S + slot * PITCH + 16 * hf * 2;
            float *arow = acc_sh + c * C::APITCH + 16 * hf;
            auto add_slice = [&](auto slice_tag, bool first) {
                constexpr int S = decltype(slice_tag)::value;     // slice: dt = S / 2, registers 8*(S%2) .. +7
                constexpr int dt = S >> 1, r0 = 8 * (S & 1);
                float *dst = arow + 32 * dt + r0;
                float4 a0 = *reinterpret_cast<float4 *>(dst), a1 = *reinterpret_cast<float4 *>(dst + 4);
                const u32x4 xv = ld_lds16(v2row + dt * 64 + (S & 1) * 16);
                if (save) {
                    u32x4 pk;
#pragma unroll
                    for (int w = 0; w < 4; ++w) pk[w] = pack_bf16(T[dt][r0 + 2 * w], T[dt][r0 + 2 * w + 1]);
                    st_global16(trow + saved_t_offset(0, 0, dt, S & 1), pk);
                }
                if (first) {
                    a0.x *= fo; a0.y *= fo; a0.z *= fo; a0.w *= fo;
                    a1.x *= fo; a1.y *= fo; a1.z *= fo; a1.w *= fo;
                }
                a0.x += T[dt][r0] * bf16_lo(xv[0]) * g;
                a0.y += T[dt][r0 + 1] * bf16_hi(xv[0]) * g;
                a0.z += T[dt][r0 + 2] * bf16_lo(xv[1]) * g;
                a0.w += T[dt][r0 + 3] * bf16_hi(xv[1]) * g;
                a1.x += T[dt][r0 + 4] * bf16_lo(xv[2]) * g;
                a1.y += T[dt][r0 + 5] * bf16_hi(xv[2]) * g;
                a1.z += T[dt][r0 + 6] * bf16_lo(xv[3]) * g;
                a1.w += T[dt][r0 + 7] * bf16_hi(xv[3]) * g;
                *reinterpret_cast<float4 *>(dst) = a0;
                *reinterpret_cast<float4 *>(dst + 4) = a1;
            };
            // 2 DT slices of eight registers: the waves form 8 / (2 DT) groups that take turns, group g owns the
            // phases 2 DT g .. 2 DT g + 2 DT - 1 and its wave w the slice (w + ph) mod 2 DT in phase ph
            for (int ph = 0; ph < 8; ++ph) {
                constexpr int NS = 2 * DT;
                if (NS == 8 || ph / NS == wave / NS) with_slice<NS>(wave + ph, [&](auto tag) { add_slice(tag, ph % NS == 0 && (NS == 8 || wave / NS == 0)); });
                if (ph == 7 && adds_rows(r)) write_rows(r);  // (their slots are not in use in this round)
                __syncthreads();
            }
        }
    }

    wait_loads<0>();           // (transfers issued behind the last tile still write into the ring)
    // ---- output: O = acc_sh / L with L = sum_w l_w 2^(M_w - Mc)
    {
        auto sw = __builtin_amdgcn_permlane32_swap(as_u32(l), as_u32(l), false, false);
        const float l_tot = as_f32(sw[0]) + as_f32(sw[1]);
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
        for (int x = 0; x < SEG; x += 2) {
            float2 v = *reinterpret_cast<const float2 *>(src + x);
            o[x] = v.x * inv;
            o[x + 1] = v.y * inv;
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
        } else if constexpr (SEG == 4) {
            u32x2 ov, rv;
#pragma unroll
            for (int w = 0; w < 2; ++w) {
                ov[w] = pack_bf16(o[2 * w], o[2 * w + 1]);
                rv[w] = pack_bf16(o[2 * w] - bf16_lo(ov[w]), o[2 * w + 1] - bf16_hi(ov[w]));
            }
            *reinterpret_cast<u32x2 *>(orow) = ov;
            if (rrow) *reinterpret_cast<u32x2 *>(rrow) = rv;
        } else {
            static_assert(SEG == 2, "head dimension 32, 64 or 128");
            const uint32_t ov = pack_bf16(o[0], o[1]);
            *reinterpret_cast<uint32_t *>(orow) = ov;
            if (rrow) *reinterpret_cast<uint32_t *>(rrow) = pack_bf16(o[0] - bf16_lo(ov), o[1] - bf16_hi(ov));
        }
        if (seg == 0) p.lse[((int64_t)b * p.H + h) * N + ir] = (xm[row] + __builtin_amdgcn_logf(L)) * kLn2;
    }
}

}  // namespace sa2
