// Kernels for head dimension 256: forward, dQ/dK2/dV2 and dK1/dV1.
//
// At D = 256 neither the logit operand (64 registers) nor a [32][D] fp32 accumulator (128 registers) leaves room
// for the two-waves-per-SIMD, register-resident designs of the other head dimensions.
//
//   fwd_wide_kernel     one wave per SIMD with all 512 registers: a workgroup of four waves owns four consecutive
//                       query tiles, one per wave; a wave keeps the logit operand, the value accumulator T of the
//                       running offset and the output sum O in registers and shares only the K1 / V1 tiles (LDS)
//                       with the other waves.  For every offset dlt = i - k, for every tile: S^T = K1 A^T, running
//                       softmax over all (offset, tile) pairs, T^T += V1^T P^T; at the end of an offset
//                       O += v2_{i-dlt} * T                                      (reference: TT:58-228)
// The backward kernels hold two accumulators per output row set and split the head dimension over the four waves of
// a workgroup instead: wave w owns the columns d = 64 w .. 64 w + 63.  Every 32 x 32 logit tile is the sum of four
// partial contractions (one per wave, four MFMAs each) that meet in an fp32 exchange area of LDS; every wave then
// holds the complete tile in the MFMA's C layout, forms the same weights, and multiplies them into its own 64
// columns of the accumulators.  No MFMA is issued twice.
//   bwd_wide_q_kernel   owns 32 query rows: S, dP, dS = P (dP - delta), G^T += K1^T dS^T, T^T += V1^T P^T;
//                       dq += k2 * G in registers, dk2 / dv2 partial rows (q * G, do * T) added to the fp32
//                       workspace block of the tile, which dk2_dv2_combine_kernel sums (TT:515-712)
//   bwd_wide_kv_kernel  owns 32 rows j of K1/V1: for every query tile and offset that reaches them
//                       dV1^T += B^T P, dK1^T += A^T dS                              (TT:298-503)
// (TT = simplicial_attention/triton_two_simplicial_attention.py of the reference.)
// Operand tiles live in LDS in the swizzled layout of SwzLane (written once, read as row fragments and as
// transposed fragments); tiles and rows are fetched one step ahead through registers.
// Every sum has a fixed order: results are bitwise reproducible, there are no atomics.
#pragma once

#include "sa2_common.hpp"
#include "sa2_lds.hpp"

namespace sa2 {

template <int D>
struct WideCfg {
    static constexpr int NW = 4;              // waves per workgroup
    static constexpr int DQ = D / NW;         // columns of a wave
    static constexpr int DB = DQ / 32;        // 32-wide column blocks of a wave
    static constexpr int KQ = DQ / 16;        // k-slices of a wave's part of a logit contraction
    static constexpr int P = tr_pitch<D>();
    static constexpr int TILE = 32 * P;
    static constexpr int XCH = NW * 4096;     // one 32 x 32 fp32 partial per wave
    static constexpr int PPR = D / 8;         // 16-byte pieces per row
    static constexpr int NP = 32 * PPR / 256; // pieces per thread and tile
    static_assert(DQ % 32 == 0 && NP * 256 == 32 * PPR, "head dimension must be a multiple of 128");
};

// row and byte column of piece n of thread tid in a [32][D] tile
template <int D>
__device__ __forceinline__ void wide_piece(int tid, int n, int &row, int &col) {
    const int x = tid + 256 * n;
    row = x / WideCfg<D>::PPR;
    col = (x % WideCfg<D>::PPR) * 16;
}

// this thread's pieces into a swizzled LDS tile
template <int D>
__device__ __forceinline__ void wide_store(char *tile, const u32x4 (&src)[WideCfg<D>::NP], int tid) {
#pragma unroll
    for (int n = 0; n < WideCfg<D>::NP; ++n) {
        int row, col;
        wide_piece<D>(tid, n, row, col);
        *reinterpret_cast<u32x4 *>(tile + swz_store_off<D>(row, col)) = src[n];
    }
}

// this thread's pieces of rows row0 .. row0 + 31 of a (seq, dim) matrix, into registers (rows outside the sequence
// are replaced by the nearest row inside: whatever they meet is masked).  The kernels fetch a tile one step ahead,
// so that the memory latency passes behind the step's MFMAs.
template <int D>
__device__ __forceinline__ void wide_pieces(u32x4 (&dst)[WideCfg<D>::NP], const char *g, int64_t sn, int row0, int N, int tid) {
#pragma unroll
    for (int n = 0; n < WideCfg<D>::NP; ++n) {
        int row, col;
        wide_piece<D>(tid, n, row, col);
        int rr = row0 + row;
        rr = rr < 0 ? 0 : (rr < N ? rr : N - 1);
        dst[n] = ld_global16(g + (int64_t)rr * sn + col);
    }
}

// operand tile: piece = bf16(x * y * c), x and y from registers (y: the pieces of rows row0 - dlt .. row0 - dlt + 31)
template <int D>
__device__ __forceinline__ void wide_build(char *tile, const u32x4 (&x)[WideCfg<D>::NP], const u32x4 (&y)[WideCfg<D>::NP], float c, int tid) {
#pragma unroll
    for (int n = 0; n < WideCfg<D>::NP; ++n) {
        int row, col;
        wide_piece<D>(tid, n, row, col);
        u32x4 a;
#pragma unroll
        for (int w = 0; w < 4; ++w) a[w] = pack_bf16(bf16_lo(x[n][w]) * c * bf16_lo(y[n][w]), bf16_hi(x[n][w]) * c * bf16_hi(y[n][w]));
        *reinterpret_cast<u32x4 *>(tile + swz_store_off<D>(row, col)) = a;
    }
}

__device__ __forceinline__ void wide_put(char *xch, int wave, int lane, const f32x16 &X) {
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4)
        *reinterpret_cast<float4 *>(xch + wave * 4096 + r4 * 1024 + lane * 16) = make_float4(X[4 * r4], X[4 * r4 + 1], X[4 * r4 + 2], X[4 * r4 + 3]);
}
// The backward kernels share the elementwise work on a summed tile: wave w sums, weighs and packs the registers
// 4 w .. 4 w + 3 of every lane (a quarter of the tile) and leaves them in LDS as the bytes (w % 2) * 8 .. + 7 of
// [half w / 2][lane][16 bytes], where every wave then reads the packed operand of its products with two 16-byte reads.
__device__ __forceinline__ float4 wide_sum_quarter(const char *xch, int wave, int lane) {
    float4 s = *reinterpret_cast<const float4 *>(xch + wave * 1024 + lane * 16);
#pragma unroll
    for (int w = 1; w < 4; ++w) {
        const float4 v = *reinterpret_cast<const float4 *>(xch + w * 4096 + wave * 1024 + lane * 16);
        s.x += v.x;
        s.y += v.y;
        s.z += v.z;
        s.w += v.w;
    }
    return s;
}
__device__ __forceinline__ void wide_put_packed(char *pex, int wave, int lane, float a0, float a1, float a2, float a3) {
    const u32x2 v = {pack_bf16(a0, a1), pack_bf16(a2, a3)};
    *reinterpret_cast<u32x2 *>(pex + (wave >> 1) * 1024 + lane * 16 + (wave & 1) * 8) = v;
}
__device__ __forceinline__ void wide_get_packed(u32x4 (&pb)[2], const char *pex, int lane) {
    pb[0] = ld_lds16(pex + lane * 16);
    pb[1] = ld_lds16(pex + 1024 + lane * 16);
}

// ------------------------------------------------------------------------------------------------------------------
// Forward, one wave per SIMD: a workgroup of four waves owns four consecutive 32-row query tiles, one per wave, and a
// wave keeps everything of its tile in its 512 registers: the logit operand A (64), the value accumulator T of the
// running offset (128) and the output sum O over the offsets (128).  Nothing is exchanged between waves: the
// workgroup only shares the K1 / V1 tiles, which go through two LDS buffers (one barrier per tile step).  The waves'
// first windows differ by one tile each: the workgroup walks the union and a wave skips what lies outside its own.
template <int D>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void fwd_wide_kernel(KParams p) {
    using C = WideCfg<D>;
    constexpr int KS = D / 16, DT = D / 32;
    __shared__ __attribute__((aligned(16))) char lds[4 * C::TILE];

    const int N = p.N;
    const int ntile = (N + 31) / 32, ngroup = (ntile + 3) / 4;
    const int item = xcd_contiguous(blockIdx.x, gridDim.x);
    const int grp = ngroup - 1 - item % ngroup;
    const int bh = item / ngroup;
    const int h = bh % p.H, b = bh / p.H;
    const int hk = h / p.G;
    const int tid = threadIdx.x;
    const int wave = wave_index(), lane = tid & 63;
    const int c = lane & 31, hf = lane >> 5;
    const int tile = 4 * grp + wave;
    const bool tile_ok = tile < ntile;
    const int i0 = tile * 32, i = i0 + c;
    const bool row_ok = i < N;
    const int ic = row_ok ? i : N - 1;

    const char *qrow = p.q.ptr + b * p.q.sb + h * p.q.sh + (int64_t)ic * p.q.sn + 16 * hf;
    const char *k1g = p.k1.ptr + b * p.k1.sb + hk * p.k1.sh;
    const char *v1g = p.v1.ptr + b * p.v1.sb + hk * p.v1.sh;
    const char *k2g = p.k2.ptr + b * p.k2.sb + hk * p.k2.sh;
    const char *v2g = p.v2.ptr + b * p.v2.sb + hk * p.v2.sh;
    const SwzLane<D> sw(lane);

    // this wave's tiles of the first window and offsets; the workgroup's union
    const int t_lo = (i0 - p.w1 + 1 > 0 ? i0 - p.w1 + 1 : 0) / 32, t_hi = tile;
    const int nd = p.w2 < i0 + 32 ? p.w2 : i0 + 32;
    const int last = (4 * grp + 3 < ntile ? 4 * grp + 3 : ntile - 1);                 // last valid tile of the group
    const int g_lo = (128 * grp - p.w1 + 1 > 0 ? 128 * grp - p.w1 + 1 : 0) / 32, g_hi = last;
    const int g_nd = p.w2 < 32 * last + 32 ? p.w2 : 32 * last + 32;

    float M = -INFINITY, l = 0.f;            // softmax reference of the row (log2 domain; moves only when a tile's maximum
                                             // exceeds it by more than 2^8) and this lane's part of the row sum
    f32x16 O[DT], T[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) O[dt] = zero16();

    u32x4 nk[C::NP], nv[C::NP];
    wide_pieces<D>(nk, k1g, p.k1.sn, 32 * g_lo, N, tid);
    wide_pieces<D>(nv, v1g, p.v1.sn, 32 * g_lo, N, tid);
    int buf = 0;

    for (int dlt = 0; dlt < g_nd; ++dlt) {
        const bool off_on = tile_ok && dlt < nd;
        const bool col_ok = off_on && row_ok && i - dlt >= 0;
        u32x4 A[KS];
        {
            int kr = i - dlt;
            kr = kr < 0 ? 0 : (kr < N ? kr : N - 1);
            const char *k2row = k2g + (int64_t)kr * p.k2.sn + 16 * hf;
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) {
                const u32x4 fq = ld_global16(qrow + 32 * kk), fk = ld_global16(k2row + 32 * kk);
#pragma unroll
                for (int w = 0; w < 4; ++w)
                    A[kk][w] = pack_bf16(bf16_lo(fq[w]) * p.scale_log2e * bf16_lo(fk[w]), bf16_hi(fq[w]) * p.scale_log2e * bf16_hi(fk[w]));
            }
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) T[dt] = zero16();

        for (int t = g_lo; t <= g_hi; ++t) {
            char *tK = lds + buf * 2 * C::TILE, *tV = tK + C::TILE;
            wide_store<D>(tK, nk, tid);
            wide_store<D>(tV, nv, tid);
            {
                const int tn = t < g_hi ? t + 1 : g_lo;
                wide_pieces<D>(nk, k1g, p.k1.sn, 32 * tn, N, tid);
                wide_pieces<D>(nv, v1g, p.v1.sn, 32 * tn, N, tid);
            }
            __syncthreads();       // the tile is complete; every wave has left the step before, whose buffer the next store takes
            buf ^= 1;
            if (!(off_on && t >= t_lo && t <= t_hi)) continue;
            // (fragments through a rolling window of four: a scheduling fence behind every MFMA and its read keeps the
            // reads spread along the chain and the live fragments at sixteen registers)
            constexpr int FW = 4;
            f32x16 X = zero16();
            {
                u32x4 f[FW];
#pragma unroll
                for (int kk = 0; kk < FW; ++kk) f[kk] = sw.row_frag(tK, kk);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kk = 0; kk < KS; ++kk) {
                    X = mfma32(f[kk % FW], A[kk], X);
                    if (kk + FW < KS) f[kk % FW] = sw.row_frag(tK, kk + FW);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // register rr of this lane: key row j = 32 t + 8 (rr / 4) + 4 hf + rr % 4, query row i; attended iff 0 <= i - j < w1
            const bool full = 32 * t + 31 <= i0 && 32 * t > i0 + 31 - p.w1 && i0 - dlt >= 0 && i0 + 31 < N;
            if (!full) {
                int rel = col_ok ? i - 32 * t - 4 * hf : -(1 << 30);
                asm volatile("" : "+v"(rel));
#pragma unroll
                for (int rr = 0; rr < 16; ++rr) {
                    const bool ok = (unsigned)(rel - (8 * (rr >> 2) + (rr & 3))) < (unsigned)p.w1;
                    X[rr] = ok ? X[rr] : -INFINITY;
                }
            }
            float tmax = X[0];
#pragma unroll
            for (int rr = 1; rr < 16; ++rr) tmax = fmaxf(tmax, X[rr]);
            {
                auto s2 = __builtin_amdgcn_permlane32_swap(as_u32(tmax), as_u32(tmax), false, false);
                tmax = fmaxf(as_f32(s2[0]), as_f32(s2[1]));
            }
            if (wave_any(tmax > M + 8.f)) {
                // (rare after a row's first tile) the reference follows the maximum; what the row holds is rescaled
                const float mn = fmaxf(M, tmax);
                const float alpha = mn == -INFINITY ? 1.f : fast_exp2(M - mn);      // 0 for a row that held nothing
                M = mn;
                l *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int rr = 0; rr < 16; ++rr) {
                        T[dt][rr] *= alpha;
                        O[dt][rr] *= alpha;
                    }
            }
            const float mref = M == -INFINITY ? 0.f : M;
            float ls = l;
            u32x4 pb[2];
#pragma unroll
            for (int rr = 0; rr < 16; rr += 2) {
                const float e0 = fast_exp2(X[rr] - mref), e1 = fast_exp2(X[rr + 1] - mref);
                ls += e0 + e1;
                pb[rr >> 3][(rr & 7) >> 1] = pack_bf16(e0, e1);
            }
            l = ls;
            {
                u32x4 f[FW];
#pragma unroll
                for (int m = 0; m < FW; ++m) f[m] = sw.tr_frag(tV, m / DT, m % DT);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int m = 0; m < 2 * DT; ++m) {
                    T[m % DT] = mfma32(f[m % FW], pb[m / DT], T[m % DT]);
                    if (m + FW < 2 * DT) f[m % FW] = sw.tr_frag(tV, (m + FW) / DT, (m + FW) % DT);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        // O += v2_{i - dlt} * T (a lane without a valid k holds T = 0)
        if (off_on) {
            int kr = i - dlt;
            kr = kr < 0 ? 0 : (kr < N ? kr : N - 1);
            fma_row<DT>(O, T, v2g + (int64_t)kr * p.v2.sn + 16 * hf * 2);
        }
    }

    auto s2 = __builtin_amdgcn_permlane32_swap(as_u32(l), as_u32(l), false, false);
    const float L = as_f32(s2[0]) + as_f32(s2[1]);
    if (!row_ok || !tile_ok) return;
    const float inv = 1.f / L;
    char *orow = p.o.ptr + b * p.o.sb + (int64_t)i * p.o.sn + h * p.o.sh + 16 * hf * 2;
    char *rrow = p.o_lo.ptr ? p.o_lo.ptr + b * p.o_lo.sb + (int64_t)i * p.o_lo.sn + h * p.o_lo.sh + 16 * hf * 2 : nullptr;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            u32x4 ov, rv;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float a = O[dt][8 * half + 2 * w] * inv, bb = O[dt][8 * half + 2 * w + 1] * inv;
                ov[w] = pack_bf16(a, bb);
                rv[w] = pack_bf16(a - bf16_lo(ov[w]), bb - bf16_hi(ov[w]));
            }
            st_global16(orow + dt * 64 + half * 16, ov);
            if (rrow) st_global16(rrow + dt * 64 + half * 16, rv);
        }
    if (hf == 0) p.lse[((int64_t)b * p.H + h) * N + i] = (M + __builtin_amdgcn_logf(L)) * kLn2;
}

// ------------------------------------------------------------------------------------------------------------------
// Workspace block of a tile: [32 + halo][D] fp32 rows per tensor, row x <-> k = i0 - halo + x (the layout that
// dk2_dv2_combine_kernel reads: the dk2 rows carry q * scale * log2(e), the kernel multiplies by ln 2).
template <int D>
__global__ __launch_bounds__(256) void bwd_wide_q_kernel(KParams p, float *ws, int halo) {
    using C = WideCfg<D>;
    constexpr int DB = C::DB, KQ = C::KQ;
    // operand tiles A, B; two buffers of K1 / V1 tiles; the exchange areas of the partial tiles; the packed weights
    __shared__ __attribute__((aligned(16))) char lds[6 * C::TILE + 2 * C::XCH + 2 * 2048];
    char *tA = lds, *tB = lds + C::TILE;
    char *xs = lds + 6 * C::TILE, *xp = xs + C::XCH, *pexP = xp + C::XCH, *pexS = pexP + 2048;
    int buf = 0;

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
    const int i0 = tile * 32, i = i0 + c;
    const bool row_ok = i < N;

    const char *qg = p.q.ptr + b * p.q.sb + h * p.q.sh;
    const char *dog = p.dout.ptr + b * p.dout.sb + h * p.dout.sh;
    const char *k1g = p.k1.ptr + b * p.k1.sb + hk * p.k1.sh;
    const char *v1g = p.v1.ptr + b * p.v1.sb + hk * p.v1.sh;
    const char *k2g = p.k2.ptr + b * p.k2.sb + hk * p.k2.sh;
    const char *v2g = p.v2.ptr + b * p.v2.sb + hk * p.v2.sh;
    const SwzLane<D> sw(lane);

    u32x4 qp[C::NP], dop[C::NP];
    wide_pieces<D>(qp, qg, p.q.sn, i0, N, tid);
    wide_pieces<D>(dop, dog, p.dout.sn, i0, N, tid);
    const int64_t srow = ((int64_t)b * p.H + h) * N + (row_ok ? i : N - 1);
    const float lse2 = p.lse[srow] * kLog2e, dl = p.delta[srow];

    const int srows = 32 + halo;
    const int64_t per_tensor = (int64_t)p.B * p.H * ntile * srows * D;
    float *wk = ws + (((int64_t)b * p.H + h) * ntile + tile) * srows * D, *wv = wk + per_tensor;
    for (int x = tid; x < srows * D / 4; x += 256) {
        reinterpret_cast<float4 *>(wk)[x] = make_float4(0.f, 0.f, 0.f, 0.f);
        reinterpret_cast<float4 *>(wv)[x] = make_float4(0.f, 0.f, 0.f, 0.f);
    }

    const int t_lo = (i0 - p.w1 + 1 > 0 ? i0 - p.w1 + 1 : 0) / 32, t_hi = i0 / 32;
    const int nd = p.w2 < i0 + 32 ? p.w2 : i0 + 32;
    const int col0 = wave * C::DQ + 16 * hf;              // first column of this lane's accumulator registers

    f32x16 dQ[DB], G[DB], T[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) dQ[db] = zero16();

    // fetched one step ahead: the k2 / v2 rows of the next offset, the K1 / V1 rows of the next tile
    u32x4 nyk[C::NP], nyv[C::NP], nk[C::NP], nv[C::NP];
    wide_pieces<D>(nyk, k2g, p.k2.sn, i0, N, tid);
    wide_pieces<D>(nyv, v2g, p.v2.sn, i0, N, tid);
    wide_pieces<D>(nk, k1g, p.k1.sn, 32 * t_lo, N, tid);
    wide_pieces<D>(nv, v1g, p.v1.sn, 32 * t_lo, N, tid);

    for (int dlt = 0; dlt < nd; ++dlt) {
        __syncthreads();      // operand tiles free; the rows this offset adds to were written at least one barrier ago
        wide_build<D>(tA, qp, nyk, p.scale_log2e, tid);
        wide_build<D>(tB, dop, nyv, 1.f, tid);
        wide_pieces<D>(nyk, k2g, p.k2.sn, i0 - dlt - 1, N, tid);
        wide_pieces<D>(nyv, v2g, p.v2.sn, i0 - dlt - 1, N, tid);
#pragma unroll
        for (int db = 0; db < DB; ++db) G[db] = T[db] = zero16();
        const bool col_ok = row_ok && i - dlt >= 0;
        for (int t = t_lo; t <= t_hi; ++t) {
            // (two tile buffers: a store meets no reader, every wave has passed three barriers since the buffer's last use)
            char *tK = lds + 2 * C::TILE + buf * 2 * C::TILE, *tV = tK + C::TILE;
            buf ^= 1;
            wide_store<D>(tK, nk, tid);
            wide_store<D>(tV, nv, tid);
            {
                const int tn = t < t_hi ? t + 1 : t_lo;
                wide_pieces<D>(nk, k1g, p.k1.sn, 32 * tn, N, tid);
                wide_pieces<D>(nv, v1g, p.v1.sn, 32 * tn, N, tid);
            }
            __syncthreads();
            {
                f32x16 X = zero16(), Y = zero16();
#pragma unroll
                for (int kq = 0; kq < KQ; ++kq) {
                    X = mfma32(sw.row_frag(tK, wave * KQ + kq), sw.row_frag(tA, wave * KQ + kq), X);
                    Y = mfma32(sw.row_frag(tV, wave * KQ + kq), sw.row_frag(tB, wave * KQ + kq), Y);
                }
                wide_put(xs, wave, lane, X);
                wide_put(xp, wave, lane, Y);
            }
            __syncthreads();
            {
                // this wave's quarter of the tile: key rows j = 32 t + 8 wave + 4 hf + e
                const float4 x4 = wide_sum_quarter(xs, wave, lane), y4 = wide_sum_quarter(xp, wave, lane);
                const int rel = col_ok ? i - 32 * t - 4 * hf - 8 * wave : -(1 << 30);
                const float xe[4] = {x4.x, x4.y, x4.z, x4.w}, ye[4] = {y4.x, y4.y, y4.z, y4.w};
                float pr[4], ds[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const bool ok = (unsigned)(rel - e) < (unsigned)p.w1;
                    pr[e] = ok ? fast_exp2(xe[e] - lse2) : 0.f;
                    ds[e] = pr[e] * (ye[e] - dl);
                }
                wide_put_packed(pexP, wave, lane, pr[0], pr[1], pr[2], pr[3]);
                wide_put_packed(pexS, wave, lane, ds[0], ds[1], ds[2], ds[3]);
            }
            __syncthreads();
            u32x4 pbP[2], pbS[2];
            wide_get_packed(pbP, pexP, lane);
            wide_get_packed(pbS, pexS, lane);
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int k2s = 0; k2s < 2; ++k2s) {
                    G[db] = mfma32(sw.tr_frag(tK, k2s, wave * DB + db), pbS[k2s], G[db]);
                    T[db] = mfma32(sw.tr_frag(tV, k2s, wave * DB + db), pbP[k2s], T[db]);
                }
        }
        // dq_i += k2_{i-dlt} * G;  row k = i - dlt of the tile's partial rows += (q_i scale log2e) * G and do_i * T
        int kr = i - dlt;
        kr = kr < 0 ? 0 : (kr < N ? kr : N - 1);
        fma_row<DB>(dQ, G, k2g + (int64_t)kr * p.k2.sn + col0 * 2);
        if (col_ok) {
            float *rk = wk + (int64_t)(c - dlt + halo) * D + col0, *rv = wv + (int64_t)(c - dlt + halo) * D + col0;
            const char *qrow = qg + (int64_t)i * p.q.sn + col0 * 2, *dorow = dog + (int64_t)i * p.dout.sn + col0 * 2;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const u32x4 xq = ld_global16(qrow + db * 64 + half * 16), xd = ld_global16(dorow + db * 64 + half * 16);
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        float4 *dk = reinterpret_cast<float4 *>(rk + 32 * db + 8 * half + 4 * e);
                        float4 *dv = reinterpret_cast<float4 *>(rv + 32 * db + 8 * half + 4 * e);
                        float4 a = *dk, bq = *dv;
                        const int r0 = 8 * half + 4 * e;
                        a.x += bf16_lo(xq[2 * e]) * p.scale_log2e * G[db][r0];
                        a.y += bf16_hi(xq[2 * e]) * p.scale_log2e * G[db][r0 + 1];
                        a.z += bf16_lo(xq[2 * e + 1]) * p.scale_log2e * G[db][r0 + 2];
                        a.w += bf16_hi(xq[2 * e + 1]) * p.scale_log2e * G[db][r0 + 3];
                        bq.x += bf16_lo(xd[2 * e]) * T[db][r0];
                        bq.y += bf16_hi(xd[2 * e]) * T[db][r0 + 1];
                        bq.z += bf16_lo(xd[2 * e + 1]) * T[db][r0 + 2];
                        bq.w += bf16_hi(xd[2 * e + 1]) * T[db][r0 + 3];
                        *dk = a;
                        *dv = bq;
                    }
                }
        }
    }
    if (row_ok) store_row<DB>(p.dq.ptr + b * p.dq.sb + (int64_t)i * p.dq.sn + h * p.dq.sh + col0 * 2, dQ, p.scale);
}

// ------------------------------------------------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void bwd_wide_kv_kernel(KParams p) {
    using C = WideCfg<D>;
    constexpr int DB = C::DB, KQ = C::KQ;
    __shared__ __attribute__((aligned(16))) char lds[2 * C::TILE + 2 * C::XCH + 2 * 2048 + 2 * 32 * 4];
    char *tA = lds, *tB = lds + C::TILE, *xs = lds + 2 * C::TILE, *xp = xs + C::XCH, *pexP = xp + C::XCH, *pexS = pexP + 2048;
    float *lse_s = reinterpret_cast<float *>(pexS + 2048), *del_s = lse_s + 32;

    const int N = p.N;
    const int ntile = (N + 31) / 32;
    const int item = xcd_contiguous(blockIdx.x, gridDim.x);
    const int jt = item % ntile;
    const int bhk = item / ntile;
    const int hk = bhk % p.HK, b = bhk / p.HK;
    const int tid = threadIdx.x;
    const int wave = wave_index(), lane = tid & 63;
    const int c = lane & 31, hf = lane >> 5;
    const int j0 = jt * 32, j = j0 + c;

    const char *k2g = p.k2.ptr + b * p.k2.sb + hk * p.k2.sh;
    const char *v2g = p.v2.ptr + b * p.v2.sb + hk * p.v2.sh;
    const SwzLane<D> sw(lane);

    // the K1 and V1 rows of this slab: the row fragments of this wave's columns stay in registers
    u32x4 kfr[KQ], vfr[KQ];
    {
        const int jr = j < N ? j : N - 1;
        const char *krow = p.k1.ptr + b * p.k1.sb + hk * p.k1.sh + (int64_t)jr * p.k1.sn + 16 * hf;
        const char *vrow = p.v1.ptr + b * p.v1.sb + hk * p.v1.sh + (int64_t)jr * p.v1.sn + 16 * hf;
#pragma unroll
        for (int kq = 0; kq < KQ; ++kq) {
            kfr[kq] = ld_global16(krow + 32 * (wave * KQ + kq));
            vfr[kq] = ld_global16(vrow + 32 * (wave * KQ + kq));
        }
    }
    f32x16 dK[DB], dV[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) dK[db] = dV[db] = zero16();

    int it_hi = (j0 + 31 + p.w1 - 1) / 32;               // last query tile that reaches a row of the slab
    it_hi = it_hi < ntile - 1 ? it_hi : ntile - 1;
    for (int g = 0; g < p.G; ++g) {
        const int h = hk * p.G + g;
        const char *qg = p.q.ptr + b * p.q.sb + h * p.q.sh;
        const char *dog = p.dout.ptr + b * p.dout.sb + h * p.dout.sh;
        for (int it = jt; it <= it_hi; ++it) {
            const int i0 = 32 * it;
            const int nd = p.w2 < i0 + 32 ? p.w2 : i0 + 32;
            u32x4 qp[C::NP], dop[C::NP];
            wide_pieces<D>(qp, qg, p.q.sn, i0, N, tid);
            wide_pieces<D>(dop, dog, p.dout.sn, i0, N, tid);
            __syncthreads();                             // the statistics of the tile before are no longer read
            if (tid < 32) {
                const int ii = i0 + tid < N ? i0 + tid : N - 1;
                const int64_t srow = ((int64_t)b * p.H + h) * N + ii;
                lse_s[tid] = p.lse[srow] * kLog2e;
                del_s[tid] = p.delta[srow];
            }
            // (fetched one offset ahead: the k2 / v2 rows of the next offset)
            u32x4 nyk[C::NP], nyv[C::NP];
            wide_pieces<D>(nyk, k2g, p.k2.sn, i0, N, tid);
            wide_pieces<D>(nyv, v2g, p.v2.sn, i0, N, tid);
            for (int dlt = 0; dlt < nd; ++dlt) {
                __syncthreads();                         // operand tiles and exchange areas free
                wide_build<D>(tA, qp, nyk, p.scale_log2e, tid);
                wide_build<D>(tB, dop, nyv, 1.f, tid);
                wide_pieces<D>(nyk, k2g, p.k2.sn, i0 - dlt - 1, N, tid);
                wide_pieces<D>(nyv, v2g, p.v2.sn, i0 - dlt - 1, N, tid);
                __syncthreads();
                // S[i][j], dP[i][j]: register rr of this lane is query row i0 + 8 (rr / 4) + 4 hf + rr % 4, the lane's column is key row j
                {
                    f32x16 X = zero16(), Y = zero16();
#pragma unroll
                    for (int kq = 0; kq < KQ; ++kq) {
                        X = mfma32(sw.row_frag(tA, wave * KQ + kq), kfr[kq], X);
                        Y = mfma32(sw.row_frag(tB, wave * KQ + kq), vfr[kq], Y);
                    }
                    wide_put(xs, wave, lane, X);
                    wide_put(xp, wave, lane, Y);
                }
                __syncthreads();
                {
                    // this wave's quarter of the tile: query rows i0 + 8 wave + 4 hf + e
                    const float4 x4 = wide_sum_quarter(xs, wave, lane), y4 = wide_sum_quarter(xp, wave, lane);
                    const float4 l4 = *reinterpret_cast<const float4 *>(lse_s + 8 * wave + 4 * hf);
                    const float4 d4 = *reinterpret_cast<const float4 *>(del_s + 8 * wave + 4 * hf);
                    const float xe[4] = {x4.x, x4.y, x4.z, x4.w}, ye[4] = {y4.x, y4.y, y4.z, y4.w};
                    const float le[4] = {l4.x, l4.y, l4.z, l4.w}, de[4] = {d4.x, d4.y, d4.z, d4.w};
                    float pr[4], ds[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int ii = i0 + 8 * wave + 4 * hf + e;
                        const bool ok = ii < N && ii - dlt >= 0 && (unsigned)(ii - j) < (unsigned)p.w1;
                        pr[e] = ok ? fast_exp2(xe[e] - le[e]) : 0.f;
                        ds[e] = pr[e] * (ye[e] - de[e]);
                    }
                    wide_put_packed(pexP, wave, lane, pr[0], pr[1], pr[2], pr[3]);
                    wide_put_packed(pexS, wave, lane, ds[0], ds[1], ds[2], ds[3]);
                }
                __syncthreads();
                u32x4 pbP[2], pbS[2];
                wide_get_packed(pbP, pexP, lane);
                wide_get_packed(pbS, pexS, lane);
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int k2s = 0; k2s < 2; ++k2s) {
                        dV[db] = mfma32(sw.tr_frag(tB, k2s, wave * DB + db), pbP[k2s], dV[db]);
                        dK[db] = mfma32(sw.tr_frag(tA, k2s, wave * DB + db), pbS[k2s], dK[db]);
                    }
            }
        }
    }
    if (j < N) {
        const int col0 = (wave * C::DQ + 16 * hf) * 2;
        // (the logit operand carried scale log2(e): times ln 2 gives the softmax scale)
        store_row<DB>(p.dk1.ptr + b * p.dk1.sb + (int64_t)j * p.dk1.sn + hk * p.dk1.sh + col0, dK, kLn2);
        store_row<DB>(p.dv1.ptr + b * p.dv1.sb + (int64_t)j * p.dv1.sn + hk * p.dv1.sh + col0, dV, 1.f);
    }
}

}  // namespace sa2
