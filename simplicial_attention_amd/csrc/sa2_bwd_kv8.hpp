// Backward kernels for dK1 and dV1, eight-wave variant (two waves per SIMD).
//
// Workgroup = 128 rows j of one (batch, kv head): four 32-row slabs of j, two waves per
// slab.  The workgroup walks pairs of "steps" (query head of the group, 32-row query tile,
// offset dlt); a pair holds the offsets 2m and 2m+1 of one query tile.  The q/do rows of a
// query tile and the 63 k2/v2 rows its offsets (at most 32) can reach are staged in LDS
// once per tile; from them the 512 threads build A = q*k2 and B = do*v2 of both steps
// once per pair (A carries scale log2(e), so S is the exponent's variable part and dK1 comes out
// times scale log2(e): it is stored times ln 2).  With P = exp2(S - lse log2(e)):
//   S = A K1^T,  dP = B V1^T,  dS = P (dP - delta),  dK1^T += A^T dS,  dV1^T += B^T P.
// One wave cannot overlap its own MFMA and VALU work, so every variant keeps two waves per
// SIMD (at most 256 registers per wave):
//   MODE kKvBoth  (D = 64):  both accumulators fit one wave.  The two waves of a slab take
//                  one offset of the pair each and form all four products from one S, one
//                  dP and one set of exponentials; their partial sums are added once,
//                  through LDS, at the end.
//   MODE kKvSplit (D = 128): one wave cannot hold both accumulators, so the two waves of a
//                  slab split the work instead of the offsets.  Wave "P" holds the K1 rows
//                  and the dV1 accumulator: S, P and dV1^T += B^T P for both offsets of the
//                  pair, and it leaves the packed P in LDS.  Wave "S" holds the V1 rows and
//                  the dK1 accumulator: dP - delta meanwhile, then (one barrier later)
//                  dS = P dP and dK1^T += A^T dS.  Two contractions per wave and offset,
//                  one operand build per pair, no final reduction.  Both roles are software
//                  pipelines: the VALU work (exponentials of one offset, dS of the next, the
//                  quarters of the next pair's operand tiles) is cut into eight pieces that
//                  are issued behind the eight MFMAs of a chain that does not depend on them.
//                  The P waves build three quarters of the tiles, the S waves one (the S waves
//                  are the busier ones behind the barrier).
// Every MFMA chain requests its LDS fragments three places ahead (mfma_stream).
// S and dP read row fragments of the A and B tiles (ds_read_b128), the accumulating
// products read transposed fragments (ds_read_b64_tr_b16).  A tile that is read both ways
// is stored once, in the swizzled layout of sa2_lds.hpp.
#pragma once

#include <type_traits>

#include "sa2_common.hpp"
#include "sa2_lds.hpp"

namespace sa2 {

constexpr int kKvBoth = 2, kKvSplit = 3;

template <int D, int MODE>
struct Kv8Cfg {
    static_assert(MODE == kKvBoth || MODE == kKvSplit, "the two forms of the kernel");
    static constexpr int TPITCH = tr_pitch<D>();
    // step buffer: [A swizzled][B swizzled][lse][delta]  (both tiles are read both ways: see sa2_lds.hpp)
    static constexpr int AS = 0;
    static constexpr int BS = 32 * TPITCH;
    static constexpr int LSE = BS + 32 * TPITCH;
    static constexpr int DEL = LSE + 32 * 4;
    static constexpr int STEP = DEL + 32 * 4;
    static constexpr int PAIR = 2 * STEP;
    static constexpr int TILES = 2 * PAIR;            // double-buffered pairs
    // staged rows of the current query tile (unpadded, read lane-linear by the builders)
    static constexpr int HALO = 31;
    static constexpr int KROWS = 32 + HALO;           // k in [32 it - 31, 32 it + 31]
    static constexpr int RP = 2 * D;                  // bytes per staged row
    static constexpr int QS = TILES;
    static constexpr int DOS = QS + 32 * RP;
    static constexpr int K2S = DOS + 32 * RP;
    static constexpr int V2S = K2S + KROWS * RP;
    static constexpr int LSES = V2S + KROWS * RP;     // 32 floats lse * log2e, 32 floats delta
    static constexpr int PX = LSES + 64 * 4;          // kKvSplit: packed P of [slab][offset of the pair], 2 KiB each
    static constexpr int LDS = PX + (MODE == kKvSplit ? 4 * 2 * 2048 : 0);
    static constexpr int NROWP = (64 + 2 * KROWS) * (D / 8);        // 16-byte pieces of the staged rows
    static constexpr int RPT = (NROWP + 511) / 512;                 // ... per thread
    static constexpr int RPITCH = D + 4;              // floats per row of the final reduction
    static constexpr int LPT = 32 * D / 8 / 256;      // 16-byte pieces per thread and tensor
    static constexpr int RED = 128 * RPITCH * 4;      // bytes of one output's final reduction
    static_assert((MODE == kKvBoth ? 2 : 1) * RED <= LDS, "final reduction must fit (everything else is dead by then)");
};

// PARTS: two workgroups per key slab, each walks half of the slab's query tiles and leaves fp32 partial rows in
// p.kv_parts (for grids that would otherwise put one or two long workgroups on every CU and end on a ragged tail)
template <int D, int MODE, bool PARTS = false>
__global__ __launch_bounds__(512) void bwd_kv8_kernel(KParams p) {
    constexpr int KS = D / 16, DT = D / 32, PPR = D / 8;
    using L = Kv8Cfg<D, MODE>;
    constexpr bool TWO = MODE == kKvBoth, SPLIT = MODE == kKvSplit;
    static_assert(!TWO || D <= 64, "both accumulators fit two waves per SIMD up to D = 64 only");
    __shared__ __attribute__((aligned(16))) char lds[L::LDS];

    const int N = p.N;
    const int ntile = (N + 127) / 128;
    const int item_all = xcd_contiguous(blockIdx.x, gridDim.x);
    const int part = PARTS ? item_all & 1 : 0;
    const int item = PARTS ? item_all >> 1 : item_all;
    const int tile = item % ntile;
    const int bh = item / ntile;
    const int hk = bh % p.HK, b = bh / p.HK;

    const int tid = threadIdx.x;
    const int wave = wave_index(), lane = tid & 63;
    // The two waves of a slab sit on different SIMDs (wave w runs on SIMD w % 4): in the query tiles at both ends of a
    // workgroup's walk, which only one or two of its slabs reach, the active waves then have a SIMD each instead of
    // sharing one while others idle.  In the other tiles every SIMD still holds one wave of each group.
    const int pg = wave >> 2, slab = ((wave & 3) + 2 * pg) & 3;
    const int c = lane & 31, hf = lane >> 5;
    const int j0 = tile * 128;
    const int jw = j0 + 32 * slab;
    const int j = jw + c;
    const bool j_ok = j < N;
    const int jc = j_ok ? j : N - 1;

    const char *k2g = p.k2.ptr + b * p.k2.sb + hk * p.k2.sh;
    const char *v2g = p.v2.ptr + b * p.v2.sb + hk * p.v2.sh;

    u32x4 k1f[KS];                        // kKvSplit: the K1 rows in the P waves, the V1 rows in the S waves
    u32x4 v1f[SPLIT ? 1 : KS];
    {
        const char *k1row = p.k1.ptr + b * p.k1.sb + (int64_t)jc * p.k1.sn + hk * p.k1.sh;
        const char *v1row = p.v1.ptr + b * p.v1.sb + (int64_t)jc * p.v1.sn + hk * p.v1.sh;
        const char *own = (SPLIT && pg == 1) ? v1row : k1row;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            k1f[kk] = ld_global16(own + (16 * kk + 8 * hf) * 2);
            if constexpr (!SPLIT) v1f[kk] = ld_global16(v1row + (16 * kk + 8 * hf) * 2);
        }
    }
    f32x16 acc[DT];              // kKvBoth: dK1; kKvSplit: dV1 in the P waves, dK1 in the S waves
    f32x16 acc2[TWO ? DT : 1];   // kKvBoth: dV1
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = zero16();
#pragma unroll
    for (int dt = 0; dt < (TWO ? DT : 1); ++dt) acc2[dt] = zero16();

    const int last_i = (j0 + 127 + p.w1 - 1 < N - 1) ? j0 + 127 + p.w1 - 1 : N - 1;
    const int it_first = j0 / 32, it_last = last_i / 32;          // the query tiles that reach the slab
    const int it_half = (it_last - it_first + 2) / 2;             // PARTS: the first part takes the larger half
    const int it_begin = PARTS && part ? it_first + it_half : it_first;
    const int it_end = PARTS && !part ? it_first + it_half - 1 : it_last;
    // where a lane's row of a partial result goes (PARTS)
    auto part_row = [&](int which) {
        const int64_t rows = (int64_t)p.B * p.HK * N;
        return p.kv_parts + ((int64_t)(2 * part + which) * rows + ((int64_t)b * p.HK + hk) * N + j) * D + 16 * hf;
    };
    if constexpr (PARTS) {
        if (it_begin > it_end) {
            // (a slab with a single query tile: nothing for the second part but its zeros)
            f32x16 z[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) z[dt] = zero16();
            if (j_ok && wave < 4) {
                store_row_f32<DT>(part_row(0), z, 0.f);
                store_row_f32<DT>(part_row(1), z, 0.f);
            }
            return;
        }
    }
    const bool wave_active = jw < N;
    const int wit_lo = jw / 32;
    const int wit_hi = ((jw + 31 + p.w1 - 1 < N - 1) ? jw + 31 + p.w1 - 1 : N - 1) / 32;
    const float c2 = p.scale_log2e;
    // per-lane parts of the fragment addresses of the swizzled tiles
    const SwzLane<D> swz_lane(lane);

    // ---- pair iterator (g, it, blk, m): offsets 32 blk + 2m and 32 blk + 2m + 1 of query tile `it`, query head g
    // of the group.  (it, blk) is the staging unit: the q/do rows of the tile and the 63 k2/v2 rows that the 32
    // offsets of the block reach.
    struct Pair {
        int g, it, blk, m;
    };
    auto dtop_of = [&](int it) { return (p.w2 - 1 < 32 * it + 31) ? p.w2 - 1 : 32 * it + 31; };   // largest offset of a tile
    auto dmax_of = [&](int it, int blk) {                 // largest offset of a block, relative to the block
        const int d = dtop_of(it) - 32 * blk;
        return d < 31 ? d : 31;
    };
    auto next_unit = [&](Pair &s) {      // first pair of the next (query head, query tile, offset block)
        s.m = 0;
        if (32 * (++s.blk) > dtop_of(s.it)) {
            s.blk = 0;
            if (++s.it > it_end) {
                s.it = it_begin;
                ++s.g;
            }
        }
    };
    auto next_pair = [&](Pair &s) {
        if (2 * (++s.m) > dmax_of(s.it, s.blk)) next_unit(s);
    };
    int npairs = 0;
    for (int it = it_begin; it <= it_end; ++it)
        for (int blk = 0; 32 * blk <= dtop_of(it); ++blk) npairs += dmax_of(it, blk) / 2 + 1;
    npairs *= p.G;

    // ---- row staging: per (query head, query tile) the q/do rows and the k2/v2 rows go
    // global -> registers (a whole tile ahead) -> LDS
    u32x4 rows[L::RPT];
    float r_lse = 0.f, r_del = 0.f;
    auto issue_rows = [&](const Pair &s) {
        const int h = hk * p.G + s.g;
        const char *qg = p.q.ptr + b * p.q.sb + h * p.q.sh;
        const char *dog = p.dout.ptr + b * p.dout.sb + h * p.dout.sh;
#pragma unroll
        for (int x = 0; x < L::RPT; ++x) {
            const int pc = x * 512 + tid;
            if (pc >= L::NROWP) break;
            const int row = pc / PPR, col = (pc % PPR) * 16;
            const char *src;
            if (row < 64) {
                int i = 32 * s.it + (row & 31);
                i = i < N ? i : N - 1;
                src = (row < 32 ? qg + (int64_t)i * p.q.sn : dog + (int64_t)i * p.dout.sn);
            } else {
                const int rk = row - 64;
                int kr = 32 * (s.it - s.blk) - L::HALO + (rk < L::KROWS ? rk : rk - L::KROWS);
                kr = kr < 0 ? 0 : (kr < N ? kr : N - 1);
                src = (rk < L::KROWS ? k2g + (int64_t)kr * p.k2.sn : v2g + (int64_t)kr * p.v2.sn);
            }
            rows[x] = ld_global16(src + col);
        }
        if (tid < 32) {
            const int i = 32 * s.it + tid;
            const int icl = i < N ? i : N - 1;
            r_lse = p.lse[((int64_t)b * p.H + h) * N + icl] * kLog2e;
            r_del = p.delta[((int64_t)b * p.H + h) * N + icl];
        }
    };
    auto write_rows = [&]() {
#pragma unroll
        for (int x = 0; x < L::RPT; ++x) {
            const int pc = x * 512 + tid;
            if (pc >= L::NROWP) break;
            *reinterpret_cast<u32x4 *>(lds + L::QS + pc * 16) = rows[x];     // q, do, k2, v2 rows are contiguous
        }
        if (tid < 32) {
            reinterpret_cast<float *>(lds + L::LSES)[tid] = r_lse;
            reinterpret_cast<float *>(lds + L::LSES)[32 + tid] = r_del;
        }
    };

    // ---- operand build.  A tile has 32 * D/8 pieces of 16 bytes: 512 at D = 128, one per
    // thread, and a thread builds its piece of A and of B; 256 at D = 64, where threads 0-255
    // build A and threads 256-511 build B.  Either way a thread builds ITS piece for both steps
    // of the pair, so the q (dO) piece is read and unpacked once for two products.
    constexpr int PIECES = 32 * PPR;
    constexpr bool BOTH = PIECES == 512;
    const int b_row = (tid % PIECES) / PPR, b_col = (tid % PPR) * 16;
    auto build = [&](const Pair &s, int buf) {
        const int row = b_row, col = b_col;
        const int dmax = dmax_of(s.it, s.blk);
        char *stage = lds + buf * L::PAIR;
        const int dl0 = 2 * s.m;                                   // never dead
        const bool dead1 = dl0 + 1 > dmax;
        const int dl1 = dead1 ? dl0 : dl0 + 1;
        auto product = [&](const float (&xv)[8], int bs, auto is_a) {   // xv: q (times scale log2 e) or dO piece, bs: k2 or v2 rows
            constexpr bool IS_A = decltype(is_a)::value;
            u32x4 r0, r1;
            const u32x4 f0 = ld_lds16(lds + bs + (row - dl0 + L::HALO) * L::RP + col);
            const u32x4 f1 = ld_lds16(lds + bs + (row - dl1 + L::HALO) * L::RP + col);
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                r0[w] = pack_bf16(xv[2 * w] * bf16_lo(f0[w]), xv[2 * w + 1] * bf16_hi(f0[w]));
                r1[w] = pack_bf16(xv[2 * w] * bf16_lo(f1[w]), xv[2 * w + 1] * bf16_hi(f1[w]));
            }
            const int o = (IS_A ? L::AS : L::BS) + swz_store_off<D>(row, col);
            *reinterpret_cast<u32x4 *>(stage + o) = r0;
            *reinterpret_cast<u32x4 *>(stage + L::STEP + o) = r1;
        };
        float xv[8];
        auto unpack = [&](int xs, float f) {
            const u32x4 fx = ld_lds16(lds + xs + row * L::RP + col);
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                xv[2 * w] = bf16_lo(fx[w]) * f;
                xv[2 * w + 1] = bf16_hi(fx[w]) * f;
            }
        };
        if (BOTH || tid < PIECES) {
            unpack(L::QS, c2);
            product(xv, L::K2S, std::true_type{});
        }
        if constexpr (BOTH) __builtin_amdgcn_sched_barrier(0);   // one product at a time: no registers for both
        if (BOTH || (tid >= PIECES && tid < 2 * PIECES)) {
            unpack(L::DOS, 1.f);
            product(xv, L::V2S, std::false_type{});
        }
        if (tid < 64) {
            const int e = tid >> 5, r = tid & 31;
            const int i = 32 * s.it + r;
            const int dlt = dl0 + e;
            const bool valid = dlt <= dmax && i < N && i - 32 * s.blk - dlt >= 0;
            char *st = stage + e * L::STEP;
            // (negated: the logit chains start from it)
            reinterpret_cast<float *>(st + L::LSE)[r] = valid ? -reinterpret_cast<const float *>(lds + L::LSES)[r] : -INFINITY;
            reinterpret_cast<float *>(st + L::DEL)[r] = valid ? -reinterpret_cast<const float *>(lds + L::LSES)[32 + r] : 0.f;
        }
    };
    // the -lse / -delta start values of the pair's chains (64 threads of the P group)
    auto build_tables = [&](const Pair &s, int buf) {
        if (tid < 64) {
            const int dmax = dmax_of(s.it, s.blk);
            const int e = tid >> 5, r = tid & 31;
            const int i = 32 * s.it + r;
            const int dlt = 2 * s.m + e;
            const bool valid = dlt <= dmax && i < N && i - 32 * s.blk - dlt >= 0;
            char *st = lds + buf * L::PAIR + e * L::STEP;
            reinterpret_cast<float *>(st + L::LSE)[r] = valid ? -reinterpret_cast<const float *>(lds + L::LSES)[r] : -INFINITY;
            reinterpret_cast<float *>(st + L::DEL)[r] = valid ? -reinterpret_cast<const float *>(lds + L::LSES)[32 + r] : 0.f;
        }
    };
    Pair nb = {0, it_begin, 0, 0};   // next pair to build
    Pair cur = {0, it_begin, 0, 0};  // pair being computed
    Pair rw = {0, it_begin, 0, 0};   // staging unit whose rows are loaded next
    issue_rows(rw);
    next_unit(rw);
    write_rows();
    if (rw.g < p.G) issue_rows(rw);
    __syncthreads();
    build(nb, 0);
    next_pair(nb);

    // A chain of N MFMAs whose LDS operand fragments are requested W places ahead: behind every MFMA the
    // fragment W places further down is read (a scheduling fence keeps it there), so the chain waits for
    // LDS once, at its start, instead of before every MFMA.  frag(integral_constant<s>) reads fragment s,
    // step(integral_constant<s>, fragment) issues MFMA s.
    auto mfma_stream2 = [&](auto n_tag, auto frag, auto step, auto side) {
        constexpr int NF = decltype(n_tag)::value;
        constexpr int W = 3;
        u32x4 f[W];
        static_for<0, (W < NF ? W : NF)>([&](auto s_) { f[s_] = frag(s_); });
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, NF>([&](auto s_) {
            constexpr int x = decltype(s_)::value;
            step(s_, f[x % W]);
            if constexpr (x + W < NF) f[x % W] = frag(std::integral_constant<int, x + W>{});
            side(s_);                    // independent VALU work issued behind MFMA s
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto mfma_stream = [&](auto n_tag, auto frag, auto step) { mfma_stream2(n_tag, frag, step, [](auto) {}); };
    using NChain = std::integral_constant<int, KS>;
    using NProd = std::integral_constant<int, 2 * DT>;

    if constexpr (SPLIT) {
        // The two roles run separate loops with the same barrier sequence (per pair: tiles
        // complete; [new query tile: rows replaced]; P in LDS), so that neither loop carries
        // the other role's registers.
        char *px = lds + L::PX + slab * 4096 + lane * 16;       // [offset of the pair][half] 1 KiB each
        auto open_pair = [&](bool more) {
            __syncthreads();                                    // the tiles of the pair are complete
            if (more && nb.m == 0) {
                write_rows();
                next_unit(rw);
                if (rw.g < p.G) issue_rows(rw);
                __syncthreads();
            }
        };
        // A quarter of the next pair's operand tiles as eight pieces of VALU work that ride behind the MFMAs of a chain:
        // load (three 16-byte LDS reads), piece 2w (q or dO pair w unpacked, product with the first offset's row),
        // piece 2w + 1 (product with the second offset's row), store.
        struct QB {
            u32x4 fx, f0, f1, r0, r1;
            float xl, xh;
            char *dst;
        };
        auto qb_load = [&](QB &qb, const Pair &s, int buf, auto is_a, int half) {
            constexpr bool IS_A = decltype(is_a)::value;
            const int pc = half * 256 + (tid & 255);
            const int row = pc / PPR, col = (pc % PPR) * 16;
            const int dmax = dmax_of(s.it, s.blk);
            const int dl0 = 2 * s.m;                                   // never dead
            const int dl1 = dl0 + 1 > dmax ? dl0 : dl0 + 1;
            const int bs = IS_A ? L::K2S : L::V2S;
            qb.fx = ld_lds16(lds + (IS_A ? L::QS : L::DOS) + row * L::RP + col);
            qb.f0 = ld_lds16(lds + bs + (row - dl0 + L::HALO) * L::RP + col);
            qb.f1 = ld_lds16(lds + bs + (row - dl1 + L::HALO) * L::RP + col);
            qb.dst = lds + buf * L::PAIR + (IS_A ? L::AS : L::BS) + swz_store_off<D>(row, col);
        };
        auto qb_piece = [&](QB &qb, auto k_, float f) {
            constexpr int k = decltype(k_)::value, w = k >> 1;
            if constexpr ((k & 1) == 0) {
                qb.xl = bf16_lo(qb.fx[w]) * f;
                qb.xh = bf16_hi(qb.fx[w]) * f;
                qb.r0[w] = pack_bf16(qb.xl * bf16_lo(qb.f0[w]), qb.xh * bf16_hi(qb.f0[w]));
            } else {
                qb.r1[w] = pack_bf16(qb.xl * bf16_lo(qb.f1[w]), qb.xh * bf16_hi(qb.f1[w]));
            }
        };
        auto qb_store = [&](QB &qb) {
            *reinterpret_cast<u32x4 *>(qb.dst) = qb.r0;
            *reinterpret_cast<u32x4 *>(qb.dst + L::STEP) = qb.r1;
        };
        static_assert(KS == 8 && 2 * DT == 8, "the pipelines pair eight pieces of VALU work with the eight MFMAs of a chain");
        auto start_from = [&](f32x16 &X, const char *table) {
#pragma unroll
            for (int a4 = 0; a4 < 4; ++a4) {
                const float4 l4 = *reinterpret_cast<const float4 *>(table + (8 * a4 + 4 * hf) * 4);
                X[4 * a4] = l4.x;
                X[4 * a4 + 1] = l4.y;
                X[4 * a4 + 2] = l4.z;
                X[4 * a4 + 3] = l4.w;
            }
        };
        if (pg == 0) {
            // ---- P waves: S, P (left in LDS for the other wave of the slab), dV1^T += B^T P, three quarters of the build.
            // Software pipeline: build quarter beside the first logit chain, the exponentials of the first offset beside the
            // second logit chain, those of the second beside the first offset's dV1 products, two build quarters beside
            // the second offset's dV1 products.
            for (int s = 0; s < npairs; ++s) {
                const bool more = s + 1 < npairs;
                open_pair(more);
                const char *buf0 = lds + (s & 1) * L::PAIR, *buf1 = buf0 + L::STEP;
                const int nbuf = (s + 1) & 1;
                const int it = cur.it;
                next_pair(cur);
                const bool on = wave_active && it >= wit_lo && it <= wit_hi;
                const bool full = (jw + 31 <= 32 * it) && (jw + p.w1 > 32 * it + 31);
                auto edge = [&](f32x16 &X) {
                    if (__builtin_expect(!full, 0)) {
                        // (the tile reaches over an edge of the first window; the distance is made opaque so that
                        // none of this is computed ahead of the branch)
                        int base = 32 * it + 4 * hf - j;         // i - j for register 0
                        asm volatile("" : "+v"(base));
#pragma unroll
                        for (int rr = 0; rr < 16; ++rr) {
                            const bool ok = (unsigned)(base + 8 * (rr >> 2) + (rr & 3)) < (unsigned)p.w1;
                            X[rr] = ok ? X[rr] : -INFINITY;
                        }
                    }
                };
                u32x4 pb[2], pb_late[2];
                QB qa;
                qb_load(qa, nb, nbuf, std::true_type{}, 0);
                if (on) {
                    f32x16 X0, X1;
                    start_from(X0, buf0 + L::LSE);
                    start_from(X1, buf1 + L::LSE);
                    mfma_stream2(NChain{}, [&](auto kk) { return swz_lane.row_frag(buf0 + L::AS, kk); },
                                 [&](auto kk, const u32x4 &fr) { X0 = mfma32(fr, k1f[kk], X0); },
                                 [&](auto x_) { qb_piece(qa, x_, c2); });
                    qb_store(qa);
                    edge(X0);
                    mfma_stream2(NChain{}, [&](auto kk) { return swz_lane.row_frag(buf1 + L::AS, kk); },
                                 [&](auto kk, const u32x4 &fr) { X1 = mfma32(fr, k1f[kk], X1); },
                                 [&](auto x_) {
                                     constexpr int x = decltype(x_)::value;
                                     pb[x >> 2][x & 3] = pack_bf16(fast_exp2(X0[2 * x]), fast_exp2(X0[2 * x + 1]));
                                 });
                    *reinterpret_cast<u32x4 *>(px) = pb[0];
                    *reinterpret_cast<u32x4 *>(px + 1024) = pb[1];
                    edge(X1);
                    mfma_stream2(NProd{}, [&](auto x) { return swz_lane.tr_frag(buf0 + L::BS, x / DT, x % DT); },
                                 [&](auto x, const u32x4 &fr) { acc[x % DT] = mfma32(fr, pb[x / DT], acc[x % DT]); },
                                 [&](auto x_) {
                                     constexpr int x = decltype(x_)::value;
                                     pb_late[x >> 2][x & 3] = pack_bf16(fast_exp2(X1[2 * x]), fast_exp2(X1[2 * x + 1]));
                                 });
                    *reinterpret_cast<u32x4 *>(px + 2048) = pb_late[0];
                    *reinterpret_cast<u32x4 *>(px + 2048 + 1024) = pb_late[1];
                } else {
                    static_for<0, 8>([&](auto x_) { qb_piece(qa, x_, c2); });
                    qb_store(qa);
                }
                __syncthreads();                                // P of the pair is in LDS
                QB qb0, qb1;
                qb_load(qb0, nb, nbuf, std::false_type{}, 0);
                qb_load(qb1, nb, nbuf, std::false_type{}, 1);
                if (on) {
                    mfma_stream2(NProd{}, [&](auto x) { return swz_lane.tr_frag(buf1 + L::BS, x / DT, x % DT); },
                                 [&](auto x, const u32x4 &fr) { acc[x % DT] = mfma32(fr, pb_late[x / DT], acc[x % DT]); },
                                 [&](auto x_) {
                                     qb_piece(qb0, x_, 1.f);
                                     qb_piece(qb1, x_, 1.f);
                                 });
                } else {
                    static_for<0, 8>([&](auto x_) {
                        qb_piece(qb0, x_, 1.f);
                        qb_piece(qb1, x_, 1.f);
                    });
                }
                qb_store(qb0);
                qb_store(qb1);
                build_tables(nb, nbuf);
                next_pair(nb);
            }
            if constexpr (PARTS) {
                if (j_ok) store_row_f32<DT>(part_row(1), acc, 1.f);
            } else {
                if (j_ok) store_row<DT>(p.dv1.ptr + b * p.dv1.sb + (int64_t)j * p.dv1.sn + hk * p.dv1.sh + 16 * hf * 2, acc, 1.f);
            }
        } else {
            // ---- S waves: dP - delta for both offsets with a build quarter beside the first chain; after the barrier
            // dS = P (dP - delta) and dK1^T += A^T dS, the second offset's dS formed beside the first offset's products
            for (int s = 0; s < npairs; ++s) {
                const bool more = s + 1 < npairs;
                open_pair(more);
                const char *buf0 = lds + (s & 1) * L::PAIR, *buf1 = buf0 + L::STEP;
                const int nbuf = (s + 1) & 1;
                const int it = cur.it;
                next_pair(cur);
                const bool on = wave_active && it >= wit_lo && it <= wit_hi;
                f32x16 dP0, dP1;
                QB qa;
                qb_load(qa, nb, nbuf, std::true_type{}, 1);
                if (on) {
                    start_from(dP0, buf0 + L::DEL);
                    start_from(dP1, buf1 + L::DEL);
                    mfma_stream2(NChain{}, [&](auto kk) { return swz_lane.row_frag(buf0 + L::BS, kk); },
                                 [&](auto kk, const u32x4 &fr) { dP0 = mfma32(fr, k1f[kk], dP0); },
                                 [&](auto x_) { qb_piece(qa, x_, c2); });
                    qb_store(qa);
                    mfma_stream(NChain{}, [&](auto kk) { return swz_lane.row_frag(buf1 + L::BS, kk); },
                                [&](auto kk, const u32x4 &fr) { dP1 = mfma32(fr, k1f[kk], dP1); });
                } else {
                    static_for<0, 8>([&](auto x_) { qb_piece(qa, x_, c2); });
                    qb_store(qa);
                }
                next_pair(nb);
                __syncthreads();                                // P of the pair is in LDS
                if (on) {
                    u32x4 pq0[2], pq1[2], pb0[2], pb1[2];
#pragma unroll
                    for (int hh = 0; hh < 2; ++hh) {
                        pq0[hh] = ld_lds16(px + hh * 1024);
                        pq1[hh] = ld_lds16(px + 2048 + hh * 1024);
                    }
#pragma unroll
                    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
                        for (int w = 0; w < 4; ++w)
                            pb0[hh][w] = pack_bf16(bf16_lo(pq0[hh][w]) * dP0[8 * hh + 2 * w], bf16_hi(pq0[hh][w]) * dP0[8 * hh + 2 * w + 1]);
                    mfma_stream2(NProd{}, [&](auto x) { return swz_lane.tr_frag(buf0 + L::AS, x / DT, x % DT); },
                                 [&](auto x, const u32x4 &fr) { acc[x % DT] = mfma32(fr, pb0[x / DT], acc[x % DT]); },
                                 [&](auto x_) {
                                     constexpr int x = decltype(x_)::value, hh = x >> 2, w = x & 3;
                                     pb1[hh][w] = pack_bf16(bf16_lo(pq1[hh][w]) * dP1[8 * hh + 2 * w], bf16_hi(pq1[hh][w]) * dP1[8 * hh + 2 * w + 1]);
                                 });
                    mfma_stream(NProd{}, [&](auto x) { return swz_lane.tr_frag(buf1 + L::AS, x / DT, x % DT); },
                                [&](auto x, const u32x4 &fr) { acc[x % DT] = mfma32(fr, pb1[x / DT], acc[x % DT]); });
                }
            }
            if constexpr (PARTS) {
                if (j_ok) store_row_f32<DT>(part_row(0), acc, kLn2);
            } else {
                if (j_ok) store_row<DT>(p.dk1.ptr + b * p.dk1.sb + (int64_t)j * p.dk1.sn + hk * p.dk1.sh + 16 * hf * 2, acc, kLn2);   // A carried scale log2(e)
            }
        }
        return;
    }

    if constexpr (TWO) {
    for (int s = 0; s < npairs; ++s) {
        __syncthreads();
        if (s + 1 < npairs) {
            if (nb.m == 0) {
                // the next pair opens a new query tile: its rows replace the staged ones
                // (all builds from the old rows ended before the barrier above)
                write_rows();
                next_unit(rw);
                if (rw.g < p.G) issue_rows(rw);
                __syncthreads();
            }
            build(nb, (s + 1) & 1);
            next_pair(nb);
        }
        const char *buf = lds + (s & 1) * L::PAIR + pg * L::STEP;
        const int it = cur.it;
        next_pair(cur);
        if (!wave_active || it < wit_lo || it > wit_hi) continue;

        // ---- S[i,j] and dP[i,j]: rows = query rows of the tile, column = j
        // the chain starts from -lse_i log2(e) (stored negated by the build; -inf for dead rows), and A carries
        // scale * log2(e): the result is the exponent
        f32x16 X;
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            const float4 l4 = *reinterpret_cast<const float4 *>(buf + L::LSE + (8 * a4 + 4 * hf) * 4);
            X[4 * a4] = l4.x;
            X[4 * a4 + 1] = l4.y;
            X[4 * a4 + 2] = l4.z;
            X[4 * a4 + 3] = l4.w;
        }
        mfma_stream(NChain{}, [&](auto kk) { return swz_lane.row_frag(buf + L::AS, kk); },
                    [&](auto kk, const u32x4 &fr) { X = mfma32(fr, k1f[kk], X); });
        // the accumulator starts at -delta_i (stored negated by the build): dP - delta costs no VALU work
        f32x16 dP;
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
            const float4 d4 = *reinterpret_cast<const float4 *>(buf + L::DEL + (8 * a4 + 4 * hf) * 4);
            dP[4 * a4] = d4.x;
            dP[4 * a4 + 1] = d4.y;
            dP[4 * a4 + 2] = d4.z;
            dP[4 * a4 + 3] = d4.w;
        }
        const bool full = (jw + 31 <= 32 * it) && (jw + p.w1 > 32 * it + 31);
        if (__builtin_expect(!full, 0)) {
            int base = 32 * it + 4 * hf - j;         // i - j for register 0
            asm volatile("" : "+v"(base));           // (keeps the edge-tile code behind the branch)
#pragma unroll
            for (int rr = 0; rr < 16; ++rr) {
                const bool ok = (unsigned)(base + 8 * (rr >> 2) + (rr & 3)) < (unsigned)p.w1;
                X[rr] = ok ? X[rr] : -INFINITY;
            }
        }
        // The VALU work rides behind MFMAs that do not depend on it: the exponentials of S behind the dP chain, dS = P dP
        // behind the dV1 products (which take P), and the dK1 products last.
        constexpr int NPER = 16 / KS;              // logits per MFMA of a chain (KS = 2 DT MFMAs per chain and per product)
        u32x4 pb[2];                 // dS
        u32x4 pv[2];                 // P
        mfma_stream2(NChain{}, [&](auto kk) { return swz_lane.row_frag(buf + L::BS, kk); },
                     [&](auto kk, const u32x4 &fr) { dP = mfma32(fr, v1f[kk], dP); },
                     [&](auto x_) {
                         constexpr int x = decltype(x_)::value;
#pragma unroll
                         for (int rr = NPER * x; rr < NPER * (x + 1); rr += 2) {
                             X[rr] = fast_exp2(X[rr]);
                             X[rr + 1] = fast_exp2(X[rr + 1]);
                             pv[rr >> 3][(rr & 7) >> 1] = pack_bf16(X[rr], X[rr + 1]);
                         }
                     });
        mfma_stream2(NProd{}, [&](auto x) { return swz_lane.tr_frag(buf + L::BS, x / DT, x % DT); },
                     [&](auto x, const u32x4 &fr) { acc2[x % DT] = mfma32(fr, pv[x / DT], acc2[x % DT]); },
                     [&](auto x_) {
                         constexpr int x = decltype(x_)::value;
#pragma unroll
                         for (int rr = NPER * x; rr < NPER * (x + 1); rr += 2)
                             pb[rr >> 3][(rr & 7) >> 1] = pack_bf16(X[rr] * dP[rr], X[rr + 1] * dP[rr + 1]);
                     });
        mfma_stream(NProd{}, [&](auto x) { return swz_lane.tr_frag(buf + L::AS, x / DT, x % DT); },
                    [&](auto x, const u32x4 &fr) { acc[x % DT] = mfma32(fr, pb[x / DT], acc[x % DT]); });
    }

    // ---- add the two groups of every slab and store
    __syncthreads();
    float *red = reinterpret_cast<float *>(lds) + (32 * slab + c) * L::RPITCH + 16 * hf;
    auto publish = [&](const f32x16 (&a)[DT], float *dst) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4)
                *reinterpret_cast<float4 *>(dst + 32 * dt + 4 * r4) =
                    make_float4(a[dt][4 * r4], a[dt][4 * r4 + 1], a[dt][4 * r4 + 2], a[dt][4 * r4 + 3]);
    };
    auto collect = [&](f32x16 (&a)[DT], const float *src) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const float4 v = *reinterpret_cast<const float4 *>(src + 32 * dt + 4 * r4);
                a[dt][4 * r4] += v.x;
                a[dt][4 * r4 + 1] += v.y;
                a[dt][4 * r4 + 2] += v.z;
                a[dt][4 * r4 + 3] += v.w;
            }
    };
    if (pg == 1) {
        publish(acc, red);
        publish(acc2, red + L::RED / 4);
    }
    __syncthreads();
    if (pg == 1 || !j_ok) return;
    collect(acc, red);
    char *dk1row = p.dk1.ptr + b * p.dk1.sb + (int64_t)j * p.dk1.sn + hk * p.dk1.sh + 16 * hf * 2;
    char *dv1row = p.dv1.ptr + b * p.dv1.sb + (int64_t)j * p.dv1.sn + hk * p.dv1.sh + 16 * hf * 2;
    if constexpr (PARTS) {
        store_row_f32<DT>(part_row(0), acc, kLn2);   // A carried scale log2(e)
        collect(acc2, red + L::RED / 4);
        store_row_f32<DT>(part_row(1), acc2, 1.f);
    } else {
        store_row<DT>(dk1row, acc, kLn2);
        collect(acc2, red + L::RED / 4);
        store_row<DT>(dv1row, acc2, 1.f);
    }
    }
}

// dK1 and dV1 from the two partial results of the split slabs: a thread sums 8 d of one row
template <int D>
__global__ __launch_bounds__(256) void dkv1_parts_combine_kernel(KParams p) {
    constexpr int LP = D / 8;
    const int64_t rows = (int64_t)p.B * p.HK * p.N;
    const int64_t row = (int64_t)blockIdx.x * (256 / LP) + threadIdx.x / LP;
    if (row >= rows) return;
    const int piece = threadIdx.x % LP;
    const int j = (int)(row % p.N);
    const int hk = (int)((row / p.N) % p.HK);
    const int b = (int)(row / ((int64_t)p.N * p.HK));
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const float *a = p.kv_parts + ((int64_t)which * rows + row) * D + piece * 8;
        const float *c = a + 2 * rows * D;
        const float4 a0 = *reinterpret_cast<const float4 *>(a), a1 = *reinterpret_cast<const float4 *>(a + 4);
        const float4 c0 = *reinterpret_cast<const float4 *>(c), c1 = *reinterpret_cast<const float4 *>(c + 4);
        const u32x4 o = {pack_bf16(a0.x + c0.x, a0.y + c0.y), pack_bf16(a0.z + c0.z, a0.w + c0.w),
                         pack_bf16(a1.x + c1.x, a1.y + c1.y), pack_bf16(a1.z + c1.z, a1.w + c1.w)};
        const DevTensor &t = which ? p.dv1 : p.dk1;
        st_global16(t.ptr + b * t.sb + (int64_t)j * t.sn + hk * t.sh + piece * 16, o);
    }
}

}  // namespace sa2
