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

}  // namespace sa2
