// LDS tile layouts and fragment reads shared by the kernels.
//
// Tiles are row-major [32 rows][D] bf16 with a padded pitch.  Fragments whose k-slots run
// along d (row-major operand) are read with ds_read_b128; fragments needed transposed
// (rows = d, k-slots = tile rows) with ds_read_b64_tr_b16, which transposes 4x4 blocks of
// 16-bit elements inside groups of 16 lanes.
#pragma once

#include "sa2_common.hpp"

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

// A tile that is read both ways (row fragments with ds_read_b128 and transposed fragments
// with ds_read_b64_tr_b16) is stored once: pitch tr_pitch (row starts 64 bytes apart
// modulo 256) and the 16-byte pieces XOR-swizzled inside every aligned group of four,
// piece p of row r at piece p ^ ((r >> 2) & 3).  Transposed reads touch whole 64-byte
// groups, so the swizzle does not change their bank footprint; the sixteen rows that a
// quarter of a row fragment read touches then cover all 64 banks.  One copy instead of two
// matters because LDS writes are the slow direction on this chip (measured: about 75 B/clk
// per CU against 165 B/clk for reads).
template <int D>
__device__ __forceinline__ int swz_store_off(int row, int byte_col) {
    return row * tr_pitch<D>() + (byte_col ^ (((row >> 2) & 3) << 4));
}

// Per-lane parts of the fragment addresses of a swizzled tile.  Row fragment kk = row c,
// pieces 2 kk + hf: the swizzle leaves one base for even kk and one for odd kk.  Transposed
// fragment: the lane's 8-byte chunk of tr_lane_off, one base for the row blocks 16 s and
// one for the row blocks 16 s + 8.
template <int D>
struct SwzLane {
    static constexpr int P = tr_pitch<D>();
    int rs_even, rs_odd, ts_0, ts_8;
    __device__ __forceinline__ explicit SwzLane(int lane) {
        const int c = lane & 31, hf = lane >> 5;
        const int sg = ((c >> 2) & 3) ^ hf;
        rs_even = c * P + 16 * sg;
        rs_odd = c * P + 16 * (sg ^ 2);
        const int row = 4 * (lane >> 5) + ((lane & 15) >> 2);
        const int piece = (2 * (lane & 1) + ((lane >> 4) & 1)) ^ (lane >> 5);
        ts_0 = row * P + 16 * piece + 8 * ((lane & 3) >> 1);
        ts_8 = row * P + 16 * (piece ^ 2) + 8 * ((lane & 3) >> 1);
    }
    // row fragment kk (k-slots d = 16 kk + 8 hf .. + 7 of row c)
    __device__ __forceinline__ u32x4 row_frag(const char *tile, int kk) const {
        return ld_lds16(tile + ((kk & 1) ? rs_odd : rs_even) + 64 * (kk >> 1));
    }
    // transposed fragment: rows 16 k2s .. + 15 of the tile as k-slots, d tile dt as rows
    __device__ __forceinline__ u32x4 tr_frag(const char *tile, int k2s, int dt) const {
        const u32x2 lo = lds_read_tr<D, P>(tile + ts_0, 16 * k2s, 32 * dt);
        const u32x2 hi = lds_read_tr<D, P>(tile + ts_8, 16 * k2s + 8, 32 * dt);
        return (u32x4){lo[0], lo[1], hi[0], hi[1]};
    }
};

// ---- tiles written by direct-to-LDS loads (global_load_lds_dwordx4)
//
// One wave instruction moves 64 pieces of 16 bytes to 1 KiB of consecutive LDS, a "chunk" of RPC rows of a
// [32 rows][D] bf16 tile.  Which piece of global memory a lane fetches is free, so inside a chunk the 64-byte
// segments of the rows are interleaved, [segment][row][64 bytes], and chunks start 1040 bytes apart: the 16 rows
// that a quarter of a row-fragment read (ds_read_b128) touches, and the 4 rows x 64 bytes of a transposed read
// (ds_read_b64_tr_b16), then cover all 64 banks.  The same tile serves both kinds of reads.
template <int D>
struct DmaTile {
    static constexpr int NSEG = D * 2 / 64;           // 64-byte segments per row
    static constexpr int RPC = 16 / NSEG;             // rows per chunk
    static constexpr int NCH = 32 / RPC;              // chunks per tile
    static constexpr int CP = 1040;                   // chunk pitch
    static constexpr int BYTES = NCH * CP;
    // byte offset of element (row, d)
    __host__ __device__ static constexpr int off(int row, int d) {
        return (row / RPC) * CP + (d / 32) * (RPC * 64) + (row % RPC) * 64 + (d % 32) * 2;
    }
    // staging: row and byte column that lane `lane` fetches for chunk `ch`
    __device__ static int st_row(int ch, int lane) { return ch * RPC + (lane >> 2) % RPC; }
    __device__ static int st_col(int lane) { return (lane / (4 * RPC)) * 64 + (lane & 3) * 16; }
    // row fragment kk of row c (k-slots d = 16 kk + 8 hf .. + 7): per-lane part + immediate
    __device__ static int row_lane(int lane) { return off(lane & 31, 0) + 16 * (lane >> 5); }
    __host__ __device__ static constexpr int row_imm(int kk) { return (kk >> 1) * (RPC * 64) + (kk & 1) * 32; }
    // transposed fragment (see lds_read_tr): per-lane part + immediate for (row_base multiple of 8, d_base multiple of 32)
    __device__ static int tr_lane(int lane) {
        return off(4 * (lane >> 5) + ((lane & 15) >> 2), 16 * (lane & 1) + 8 * ((lane >> 4) & 1) + 4 * ((lane & 3) >> 1));
    }
    __host__ __device__ static constexpr int tr_imm(int row_base, int d_base) { return off(row_base, d_base); }
    __device__ static u32x4 row_frag(const char *tile_lane, int kk) { return ld_lds16(tile_lane + row_imm(kk)); }
    __device__ static u32x4 tr_frag(const char *tile_lane, int k2s, int dt) {
        const u32x2 lo = lds_read_tr<D, 0>(tile_lane + tr_imm(16 * k2s, 32 * dt), 0, 0);
        const u32x2 hi = lds_read_tr<D, 0>(tile_lane + tr_imm(16 * k2s + 8, 32 * dt), 0, 0);
        return (u32x4){lo[0], lo[1], hi[0], hi[1]};
    }
};

// One direct-to-LDS load: lane l of the wave fetches the 16 bytes at base + offset_l and they land at LDS address
// lds_addr + 16 l (base and lds_addr are wave-uniform; the LDS address travels in 16 bits of M0).  Counted by
// vmcnt like any global load; written as assembly so that the compiler does not order the kernel's ordinary LDS
// reads behind it - a kernel waits for the transfer itself (wait_loads) before the barrier that publishes the tile.
__device__ __forceinline__ void load_to_lds16(const char *base, uint32_t lane_offset, uint32_t lds_addr) {
    // (m0 is reserved: the compiler keeps nothing in it across statements)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_offset), "s"(base), "s"(lds_addr) : "memory");
}
// waits until at most N_LEFT of this wave's vector-memory operations are in flight
template <int N_LEFT>
__device__ __forceinline__ void wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N_LEFT) : "memory");
}

// sixteen registers holding x (each element is pinned to a register of its own: left to itself the compiler
// copies a whole undefined tuple first and then overwrites fifteen of its registers)
__device__ __forceinline__ f32x16 splat16(float x) {
    f32x16 r;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        float t = x;
        asm("" : "+v"(t));
        r[e] = t;
    }
    return r;
}


// the same from a register pair that already holds (x, x): eight 64-bit moves instead of sixteen 32-bit ones
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ f32x16 splat16_pairs(f32x2 xx) {
    f32x16 r;
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
        f32x2 t = xx;
        asm("" : "+v"(t));
        r[e] = t[0];
        r[e + 1] = t[1];
    }
    return r;
}

}  // namespace sa2
