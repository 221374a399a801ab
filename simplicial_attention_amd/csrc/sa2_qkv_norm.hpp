// Fused split + per-head RMSNorm of the qkv projection, forward and backward.
//
// The module around the attention core (simplicial_mha.py:116-128 in the reference) splits
// the projection output into q | k | v, unflattens heads with channel order (head, set, d)
// for keys and values, chunks the two sets apart and applies one RMSNorm(dim_head) with a
// learned weight to each of q, k1, k2, v1, v2.  Here one kernel reads a row of the
// projection once and writes the five kernel-ready (batch, seq, heads, dim_head) tensors;
// the backward reads the five gradients and writes the gradient of the projection row.
// HBM-bound: every element is read once and written once.
//
// A "head row" is one (token, tensor, head) vector of D elements.  Head rows of a token:
// [0, H) q heads, then for the keys 2*HK rows in (head, set) order, then 2*HK value rows.
// 8 elements (16 bytes) per thread, D/8 threads per head row, sum of squares by shuffles.
#pragma once

#include "sa2_common.hpp"

namespace sa2 {

struct NormParams {
    const char *qkv;        // bf16 [rows][row_stride bytes]: the projection output
    char *dqkv;             // bf16, same layout (backward)
    int64_t row_stride;     // bytes between tokens
    DevTensor t[5];         // q, k1, k2, v1, v2 (forward: outputs; backward: their gradients)
    const char *w[5];       // bf16 [D] weights (nullptr: no learned weight, i.e. ones)
    float *rstd;            // fp32 [tokens][H + 4 HK]: reciprocal rms of every head row
    float *dw_part;         // fp32 [blocks][5][D] partial weight gradients (backward)
    int B, N, H, HK;
    float eps;
};

// head row r of a token -> tensor index (0..4), head, and byte column in the projection row
template <int D>
__device__ __forceinline__ void head_row_of(int r, int H, int HK, int &tensor, int &head) {
    if (r < H) {
        tensor = 0;
        head = r;
    } else {
        const int x = r - H;
        const int part = x / (2 * HK);          // 0: keys, 1: values
        const int y = x % (2 * HK);
        head = y >> 1;
        tensor = 1 + 2 * part + (y & 1);         // k1, k2, v1, v2
    }
}

template <int D>
__global__ __launch_bounds__(256) void qkv_norm_fwd_kernel(NormParams p) {
    constexpr int LP = D / 8, RPB = 256 / LP;
    const int R = p.H + 4 * p.HK;
    const int64_t nrows = (int64_t)p.B * p.N * R;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LP;
    if (row >= nrows) return;
    const int piece = threadIdx.x % LP;
    const int64_t token = row / R;
    const int r = (int)(row % R);
    int tensor, head;
    head_row_of<D>(r, p.H, p.HK, tensor, head);
    const u32x4 x = ld_global16(p.qkv + token * p.row_stride + (int64_t)r * D * 2 + piece * 16);
    float v[8];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        v[2 * k] = bf16_lo(x[k]);
        v[2 * k + 1] = bf16_hi(x[k]);
        ss += v[2 * k] * v[2 * k] + v[2 * k + 1] * v[2 * k + 1];
    }
#pragma unroll
    for (int m = 1; m < LP; m <<= 1) ss += __shfl_xor(ss, m, LP);
    const float rstd = rsqrtf(ss * (1.f / D) + p.eps);
    if (piece == 0) p.rstd[row] = rstd;
    u32x4 w = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
    if (p.w[tensor]) w = ld_global16(p.w[tensor] + piece * 16);
    u32x4 y;
#pragma unroll
    for (int k = 0; k < 4; ++k)
        y[k] = pack_bf16(v[2 * k] * rstd * bf16_lo(w[k]), v[2 * k + 1] * rstd * bf16_hi(w[k]));
    const int b = (int)(token / p.N), n = (int)(token % p.N);
    const DevTensor &o = p.t[tensor];
    st_global16(o.ptr + b * o.sb + (int64_t)n * o.sn + head * o.sh + piece * 16, y);
}

// dx = rstd * (g - xhat * mean(g * xhat)),  g = dy * w,  xhat = x * rstd;   dw += dy * xhat.
// Weight gradients: a block walks groups of 256 / (D/8) head rows with a grid stride; every
// (row slot, 8-element piece) thread keeps its own LDS accumulators per tensor, the block
// adds the row slots in a fixed order and writes one partial [5][D]; qkv_norm_dw_kernel
// adds the partials of the blocks in a fixed order (bitwise reproducible, no atomics).
template <int D>
__global__ __launch_bounds__(256) void qkv_norm_bwd_kernel(NormParams p, int ngroups) {
    constexpr int LP = D / 8, RPB = 256 / LP;
    __shared__ float dw_sh[RPB][5 * D];
    for (int x = threadIdx.x; x < RPB * 5 * D; x += 256) (&dw_sh[0][0])[x] = 0.f;
    __syncthreads();
    const int R = p.H + 4 * p.HK;
    const int64_t nrows = (int64_t)p.B * p.N * R;
    const int slot = threadIdx.x / LP, piece = threadIdx.x % LP;
    for (int grp = blockIdx.x; grp < ngroups; grp += gridDim.x) {
        const int64_t row = (int64_t)grp * RPB + slot;
        if (row >= nrows) continue;
        const int64_t token = row / R;
        const int r = (int)(row % R);
        int tensor, head;
        head_row_of<D>(r, p.H, p.HK, tensor, head);
        const int64_t col = token * p.row_stride + (int64_t)r * D * 2 + piece * 16;
        const u32x4 x = ld_global16(p.qkv + col);
        const int b = (int)(token / p.N), n = (int)(token % p.N);
        const DevTensor &g = p.t[tensor];
        const u32x4 dy = ld_global16(g.ptr + b * g.sb + (int64_t)n * g.sn + head * g.sh + piece * 16);
        u32x4 w = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
        if (p.w[tensor]) w = ld_global16(p.w[tensor] + piece * 16);
        const float rstd = p.rstd[row];
        float xh[8], gg[8];
        float dot = 0.f;
        float *acc = &dw_sh[slot][tensor * D + piece * 8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            xh[2 * k] = bf16_lo(x[k]) * rstd;
            xh[2 * k + 1] = bf16_hi(x[k]) * rstd;
            const float d0 = bf16_lo(dy[k]), d1 = bf16_hi(dy[k]);
            gg[2 * k] = d0 * bf16_lo(w[k]);
            gg[2 * k + 1] = d1 * bf16_hi(w[k]);
            acc[2 * k] += d0 * xh[2 * k];
            acc[2 * k + 1] += d1 * xh[2 * k + 1];
            dot += gg[2 * k] * xh[2 * k] + gg[2 * k + 1] * xh[2 * k + 1];
        }
#pragma unroll
        for (int m = 1; m < LP; m <<= 1) dot += __shfl_xor(dot, m, LP);
        const float mean = dot * (1.f / D);
        u32x4 dx;
#pragma unroll
        for (int k = 0; k < 4; ++k)
            dx[k] = pack_bf16(rstd * (gg[2 * k] - xh[2 * k] * mean), rstd * (gg[2 * k + 1] - xh[2 * k + 1] * mean));
        st_global16(p.dqkv + col, dx);
    }
    __syncthreads();
    float *dst = p.dw_part + (int64_t)blockIdx.x * 5 * D;
    for (int x = threadIdx.x; x < 5 * D; x += 256) {
        float s = 0.f;
#pragma unroll 4
        for (int rr = 0; rr < RPB; ++rr) s += dw_sh[rr][x];
        dst[x] = s;
    }
}

// dw[tensor][d] = sum over blocks of the partials, in a fixed order.  A block of 256 threads owns 16 consecutive
// outputs x = (tensor, d); thread (x, phase) adds the partials of the blocks phase, phase + 16, ... (the 16 threads of
// a phase read 64 consecutive bytes of one partial), then the 16 phases of an output are added in phase order.
__global__ __launch_bounds__(256) void qkv_norm_dw_kernel(const float *part, float *dw, int nblocks, int n /* 5 * D */) {
    __shared__ float red[16][17];
    const int xl = threadIdx.x & 15, phase = threadIdx.x >> 4;
    const int x = blockIdx.x * 16 + xl;
    float s = 0.f;
    if (x < n)
        for (int b = phase; b < nblocks; b += 16) s += part[(int64_t)b * n + x];
    red[phase][xl] = s;
    __syncthreads();
    if (phase == 0 && x < n) {
        float t = 0.f;
#pragma unroll
        for (int q = 0; q < 16; ++q) t += red[q][xl];
        dw[x] = t;
    }
}

}  // namespace sa2
