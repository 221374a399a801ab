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

}  // namespace sa2
