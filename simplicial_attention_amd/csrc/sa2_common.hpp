// Shared device helpers for the gfx950 kernels of sliding-window 2-simplicial attention.
//
// Register-fragment conventions used by every kernel (wave64, v_mfma_f32_32x32x16_bf16):
//   lane = 32*hf + c            (c = lane % 32, hf = lane / 32)
//   A operand (32 x 16): lane holds row c,    k-slots 8*hf .. 8*hf+7
//   B operand (16 x 32): lane holds column c, k-slots 8*hf .. 8*hf+7
//   C/D       (32 x 32): register r of lane holds row 8*(r/4) + 4*hf + r%4, column c
// A contraction is invariant under any permutation of its k index applied to both
// operands, so the kernels are free to choose which data index sits in which k-slot.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace sa2 {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// (batch, seq, heads, dim) activation with byte strides (innermost stride = 2 bytes).
struct DevTensor {
    char *ptr;
    int64_t sb, sn, sh;
};

// The forward's per-offset T rows are kept in blocks of 32 query rows (one tile of one offset), laid out as the
// forward's lanes hold them: saved_t_offset is the place of the 16-byte piece d = 32 dt + 16 hf + 8 half + 0..7 of
// row c in its block (a wave's store of one (dt, half) covers 1 KiB of consecutive bytes)
template <int D>
__host__ __device__ constexpr int saved_t_block() { return 32 * D * 2; }
__host__ __device__ constexpr int saved_t_offset(int c, int hf, int dt, int half) { return (2 * dt + half) * 1024 + (32 * hf + c) * 16; }

struct KParams {
    DevTensor q, k1, k2, v1, v2, o, dout, dq, dk1, dk2, dv1, dv2;
    DevTensor o_lo;       // optional bf16 residual out_fp32 - bf16(out); ptr == nullptr if absent
    float *lse;
    float *delta;
    // optional by-products of the forward, reused by the backward (nullptr if absent):
    // t_save bf16 [B][H][w2][ceil(N/32)] blocks of 32 rows (saved_t_offset): T = sum_j 2^(x_ij - m) v1_j per offset,
    // m_save fp32 [B][H][w2][N]: m
    char *t_save;
    float *m_save;
    int B, N, H, HK, G;   // G = H / HK query heads per key/value head
    int w1, w2;
    float scale;          // softmax scale
    float scale_log2e;    // scale * log2(e)
    // dK1/dV1 computed in two parts per key slab (each part walks half of the slab's query tiles): fp32 partial rows
    // [part][dk1, dv1][B][HK][N][D], summed by dkv1_parts_combine_kernel; nullptr when the slabs are not split
    float *kv_parts;
};

// compile-time loop: f(integral_constant<int, B>) ... f(integral_constant<int, E - 1>)
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }

__device__ __forceinline__ float bf16_lo(uint32_t w) { return as_f32(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return as_f32(w & 0xffff0000u); }

// two floats -> packed bf16 pair, round to nearest even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ u32x4 ld_global16(const char *p) { return *reinterpret_cast<const u32x4 *>(p); }
__device__ __forceinline__ void st_global16(char *p, u32x4 v) { *reinterpret_cast<u32x4 *>(p) = v; }
__device__ __forceinline__ u32x4 ld_lds16(const char *p) { return *reinterpret_cast<const u32x4 *>(p); }

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// element-wise product of two packed bf16x8 fragments, rounded back to bf16
__device__ __forceinline__ u32x4 mul_bf16x8(u32x4 a, u32x4 b) {
    u32x4 r;
#pragma unroll
    for (int w = 0; w < 4; ++w) r[w] = pack_bf16(bf16_lo(a[w]) * bf16_lo(b[w]), bf16_hi(a[w]) * bf16_hi(b[w]));
    return r;
}

// c + lo(x) + hi(x) for a packed pair of bf16 (v_dot2c_f32_bf16 against (1, 1))
__device__ __forceinline__ float add_bf16x2(uint32_t x, float c) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, x), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), c, false);
}

// wave index as a scalar: branches on it are uniform and index arithmetic stays on the scalar unit
__device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0);
}

// Keeps an MFMA accumulator in accumulation registers at this point of the program.
// VALU instructions cannot read those registers, so without the pin the compiler may
// decide to hold a rarely VALU-touched accumulator in ordinary registers for a whole
// loop and copy all of it to and from the MFMA's registers on every iteration.
__device__ __forceinline__ void pin_acc(f32x16 &x) { asm volatile("" : "+a"(x)); }

__device__ __forceinline__ f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int r = 0; r < 16; ++r) z[r] = 0.f;
    return z;
}

// sixteen zeros, written as eight 64-bit moves (for accumulators that are cleared inside a kernel's loops)
__device__ __forceinline__ f32x16 zero16_pairs() {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    f32x16 z;
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
        f32x2_t t = {0.f, 0.f};
        asm("" : "+v"(t));
        z[r] = t[0];
        z[r + 1] = t[1];
    }
    return z;
}



__device__ __forceinline__ bool wave_any(bool pred) { return __builtin_amdgcn_ballot_w64(pred) != 0ull; }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// d index (within a 32-wide d tile) handled by MFMA row c of a "transposed output"
// GEMM (output rows = d), chosen so that the 16 accumulator registers of a lane
// cover 16 consecutive d:  register r of half hf  <->  d = 16*hf + r.
__device__ __forceinline__ int dmap_row(int c) { return 16 * ((c >> 2) & 1) + 4 * (c >> 3) + (c & 3); }

// acc[dt][r] += x[32*dt + 16*hf + r] * g[dt][r]; xrow points at element 16*hf of the row
template <int DT>
__device__ __forceinline__ void fma_row(f32x16 (&acc)[DT], const f32x16 (&g)[DT], const char *xrow) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        u32x4 xa = ld_global16(xrow + dt * 64);
        u32x4 xb = ld_global16(xrow + dt * 64 + 16);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            acc[dt][2 * w] += bf16_lo(xa[w]) * g[dt][2 * w];
            acc[dt][2 * w + 1] += bf16_hi(xa[w]) * g[dt][2 * w + 1];
            acc[dt][8 + 2 * w] += bf16_lo(xb[w]) * g[dt][8 + 2 * w];
            acc[dt][8 + 2 * w + 1] += bf16_hi(xb[w]) * g[dt][8 + 2 * w + 1];
        }
    }
}

// store acc[dt][r] * s as bf16 at d = 32*dt + 16*hf + r; orow points at element 16*hf
template <int DT>
__device__ __forceinline__ void store_row(char *orow, const f32x16 (&acc)[DT], float s) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        u32x4 oa, ob;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            oa[w] = pack_bf16(acc[dt][2 * w] * s, acc[dt][2 * w + 1] * s);
            ob[w] = pack_bf16(acc[dt][8 + 2 * w] * s, acc[dt][8 + 2 * w + 1] * s);
        }
        st_global16(orow + dt * 64, oa);
        st_global16(orow + dt * 64 + 16, ob);
    }
}

// the same as fp32 (partial results that another kernel sums): orow points at element 16*hf of the row
template <int DT>
__device__ __forceinline__ void store_row_f32(float *orow, const f32x16 (&acc)[DT], float s) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4)
            *reinterpret_cast<float4 *>(orow + 32 * dt + 4 * r4) =
                make_float4(acc[dt][4 * r4] * s, acc[dt][4 * r4 + 1] * s, acc[dt][4 * r4 + 2] * s, acc[dt][4 * r4 + 3] * s);
}

// f(integral_constant<int, s mod NS>) for a run-time s (NS = 2, 4 or 8)
template <int NS, typename F>
__device__ __forceinline__ void with_slice(int s, F &&f) {
    static_assert(NS == 2 || NS == 4 || NS == 8, "slice count");
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
    } else if constexpr (NS == 4) {
        switch (s & 3) {
            case 0: f(std::integral_constant<int, 0>{}); break;
            case 1: f(std::integral_constant<int, 1>{}); break;
            case 2: f(std::integral_constant<int, 2>{}); break;
            default: f(std::integral_constant<int, 3>{}); break;
        }
    } else {
        if (s & 1) f(std::integral_constant<int, 1>{});
        else f(std::integral_constant<int, 0>{});
    }
}

// Grid index -> logical work item such that the eight XCDs (which receive
// consecutive workgroup ids round-robin) each walk a contiguous range of items.
__device__ __forceinline__ int xcd_contiguous(int wg, int total) {
    return (total % 8 == 0) ? (wg % 8) * (total / 8) + wg / 8 : wg;
}

}  // namespace sa2
