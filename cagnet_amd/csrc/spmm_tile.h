// Staged tiles of a panel plan, multiplied with the accumulators addressed through the register index.
//
// A workgroup of 16 waves owns a unit (a run of tiles of one panel) and one column slice of the dense
// operands; wave w keeps R rows of the panel (w, w + 16, ...) times the slice in NR registers per row,
// NR * R <= 80 of them, for the whole unit.  A tile's rows of B (16 * TCW of them, TCW per wave) go
// global -> LDS directly, double buffered; the tile's entries are records {column in tile | row slot << 8,
// value} in (tile, wave) order.  A record is multiplied as
//     s_set_gpr_idx_on  slot * NR        ; destination and addend registers are taken relative to it
//     v_fma_f32 v[48 + k], value, b[k], v[48 + k]        k = 0 .. NR - 1
// so one piece of code serves every row slot: the records of a wave need no order, no padding and no
// run lengths, and the number of rows a wave owns is a template parameter instead of an unrolled loop.
// The accumulators are the physical registers v48 .. v127: every asm statement that touches them names
// them as operands tied to those registers, and nothing else in the kernel refers to them, so the
// register allocator leaves them where they are.
//
// Narrow slices make tall panels: a panel of 16 R rows needs 64 R NR accumulator floats per lane column,
// so that NR = 5 (a slice of up to 320 columns) allows 256 rows and NR = 1 (64 columns) 1024, and the
// number of (panel, column) pairs - rows of B that have to be copied - falls with the panel height.  A
// product wider than a slice runs one workgroup per (unit, slice).
//
// Replaces nothing in the reference beyond cusparseSpMM itself
// (sparse-extension/sparse_coo_tensor.cu:215-226); sums are in a fixed order, no atomics on floats.
#pragma once
#include "spmm_panel.h"

namespace cg {

typedef float tile_f32x32 __attribute__((ext_vector_type(32)));
typedef float tile_f32x16 __attribute__((ext_vector_type(16)));

struct TileAcc {  // v[48:79], v[80:111], v[112:127]
  tile_f32x32 a0, a1;
  tile_f32x16 a2;
};
#define CG_TILE_ACC(acc) "+{v[48:79]}"((acc).a0), "+{v[80:111]}"((acc).a1), "+{v[112:127]}"((acc).a2)

// Layout of a slice row over the lanes, by NR (lane l, register k -> column of the slice):
//   1: float   at 4 l                                  col = l
//   2: float2  at 8 l                                  col = 2 l + k
//   4: float4  at 16 l                                 col = 4 l + k
//   5: float4  at 16 l, float at 1024 + 4 l            col = 4 l + k | 256 + l
//   6: float4  at 16 l, float2 at 1024 + 8 l           col = 4 l + k | 256 + 2 l + (k - 4)
//   8: float4  at 16 l, float4 at 1024 + 16 l          col = 4 l + k | 256 + 4 l + (k - 4)
//  10: two float4 as for 8, float2 at 2048 + 8 l       ... | 512 + 2 l + (k - 8)
template <int NR>
__device__ __forceinline__ constexpr int tile_max_width() {
  return NR == 1 ? 64 : NR == 2 ? 128 : NR == 4 ? 256 : NR == 5 ? 320 : NR == 6 ? 384 : NR == 8 ? 512 : 640;
}
template <int NR>
__device__ __forceinline__ int tile_col(int k, int lane) {
  if (NR == 1) return lane;
  if (NR == 2) return 2 * lane + k;
  if (k < 4) return 4 * lane + k;
  if (NR == 5) return 256 + lane;
  if (NR == 6) return 256 + 2 * lane + (k - 4);
  if (k < 8) return 256 + 4 * lane + (k - 4);
  return 512 + 2 * lane + (k - 8);
}

typedef float tile_f2 __attribute__((ext_vector_type(2)));
typedef float tile_f4 __attribute__((ext_vector_type(4)));
template <typename T>
__device__ __forceinline__ T tile_lds_load(uint32_t addr) {  // addr: a byte address in LDS
  return *(const __attribute__((address_space(3))) T *)addr;
}

// The lane's registers of a staged row.  a0: LDS address of the lane's first piece (row + lane * 4, 8 or 16 by the
// layout above); a1: of its piece with the other lane stride (NR 5, 6, 10; unused otherwise).
template <int NR>
__device__ __forceinline__ void tile_row_read(uint32_t a0, uint32_t a1, float (&b)[NR]) {
  if constexpr (NR == 1) {
    b[0] = tile_lds_load<float>(a0);
  } else if constexpr (NR == 2) {
    const tile_f2 v = tile_lds_load<tile_f2>(a0);
    b[0] = v.x;
    b[1] = v.y;
  } else {
    const tile_f4 v = tile_lds_load<tile_f4>(a0);
    b[0] = v.x;
    b[1] = v.y;
    b[2] = v.z;
    b[3] = v.w;
    if constexpr (NR == 5) {
      b[4] = tile_lds_load<float>(a1);
    } else if constexpr (NR == 6) {
      const tile_f2 w = tile_lds_load<tile_f2>(a1);
      b[4] = w.x;
      b[5] = w.y;
    } else if constexpr (NR >= 8) {
      const tile_f4 w = tile_lds_load<tile_f4>(a0 + 1024u);
      b[4] = w.x;
      b[5] = w.y;
      b[6] = w.z;
      b[7] = w.w;
      if constexpr (NR == 10) {
        const tile_f2 u = tile_lds_load<tile_f2>(a1);
        b[8] = u.x;
        b[9] = u.y;
      }
    }
  }
}

// K records in one stretch of index mode: the index register is set for the first record and moved for the others
// (the low 8 bits of pk[k] are the record's first accumulator: row slot * NR); acc[idx_k + r] += v[k] * b[k][r].
template <int NR, int K>
__device__ __forceinline__ void tile_window(TileAcc &acc, const uint32_t (&pk)[K], const float (&v)[K], const float (&b)[K][NR]);
template <>
__device__ __forceinline__ void tile_window<1, 8>(TileAcc &acc, const uint32_t (&pk)[8], const float (&v)[8], const float (&b)[8][1]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\ts_set_gpr_idx_idx %[p1]\n\t"
               "v_fma_f32 v48, %[v1], %[b1_0], v48\n\ts_set_gpr_idx_idx %[p2]\n\tv_fma_f32 v48, %[v2], %[b2_0], v48\n\t"
               "s_set_gpr_idx_idx %[p3]\n\tv_fma_f32 v48, %[v3], %[b3_0], v48\n\ts_set_gpr_idx_idx %[p4]\n\t"
               "v_fma_f32 v48, %[v4], %[b4_0], v48\n\ts_set_gpr_idx_idx %[p5]\n\tv_fma_f32 v48, %[v5], %[b5_0], v48\n\t"
               "s_set_gpr_idx_idx %[p6]\n\tv_fma_f32 v48, %[v6], %[b6_0], v48\n\ts_set_gpr_idx_idx %[p7]\n\t"
               "v_fma_f32 v48, %[v7], %[b7_0], v48\n\ts_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [p1] "s"(pk[1]), [v1] "s"(v[1]), [p2] "s"(pk[2]), [v2] "s"(v[2]),
                 [p3] "s"(pk[3]), [v3] "s"(v[3]), [p4] "s"(pk[4]), [v4] "s"(v[4]), [p5] "s"(pk[5]), [v5] "s"(v[5]),
                 [p6] "s"(pk[6]), [v6] "s"(v[6]), [p7] "s"(pk[7]), [v7] "s"(v[7]), [b0_0] "v"(b[0][0]),
                 [b1_0] "v"(b[1][0]), [b2_0] "v"(b[2][0]), [b3_0] "v"(b[3][0]), [b4_0] "v"(b[4][0]),
                 [b5_0] "v"(b[5][0]), [b6_0] "v"(b[6][0]), [b7_0] "v"(b[7][0])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<2, 4>(TileAcc &acc, const uint32_t (&pk)[4], const float (&v)[4], const float (&b)[4][2]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "s_set_gpr_idx_idx %[p1]\n\tv_fma_f32 v48, %[v1], %[b1_0], v48\n\tv_fma_f32 v49, %[v1], %[b1_1], v49\n\t"
               "s_set_gpr_idx_idx %[p2]\n\tv_fma_f32 v48, %[v2], %[b2_0], v48\n\tv_fma_f32 v49, %[v2], %[b2_1], v49\n\t"
               "s_set_gpr_idx_idx %[p3]\n\tv_fma_f32 v48, %[v3], %[b3_0], v48\n\tv_fma_f32 v49, %[v3], %[b3_1], v49\n\t"
               "s_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [p1] "s"(pk[1]), [v1] "s"(v[1]), [p2] "s"(pk[2]), [v2] "s"(v[2]),
                 [p3] "s"(pk[3]), [v3] "s"(v[3]), [b0_0] "v"(b[0][0]), [b0_1] "v"(b[0][1]), [b1_0] "v"(b[1][0]),
                 [b1_1] "v"(b[1][1]), [b2_0] "v"(b[2][0]), [b2_1] "v"(b[2][1]), [b3_0] "v"(b[3][0]),
                 [b3_1] "v"(b[3][1])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<4, 2>(TileAcc &acc, const uint32_t (&pk)[2], const float (&v)[2], const float (&b)[2][4]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "v_fma_f32 v50, %[v0], %[b0_2], v50\n\tv_fma_f32 v51, %[v0], %[b0_3], v51\n\ts_set_gpr_idx_idx %[p1]\n\t"
               "v_fma_f32 v48, %[v1], %[b1_0], v48\n\tv_fma_f32 v49, %[v1], %[b1_1], v49\n\tv_fma_f32 v50, %[v1], %[b1_2], v50\n\t"
               "v_fma_f32 v51, %[v1], %[b1_3], v51\n\ts_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [p1] "s"(pk[1]), [v1] "s"(v[1]), [b0_0] "v"(b[0][0]),
                 [b0_1] "v"(b[0][1]), [b0_2] "v"(b[0][2]), [b0_3] "v"(b[0][3]), [b1_0] "v"(b[1][0]),
                 [b1_1] "v"(b[1][1]), [b1_2] "v"(b[1][2]), [b1_3] "v"(b[1][3])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<5, 2>(TileAcc &acc, const uint32_t (&pk)[2], const float (&v)[2], const float (&b)[2][5]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "v_fma_f32 v50, %[v0], %[b0_2], v50\n\tv_fma_f32 v51, %[v0], %[b0_3], v51\n\tv_fma_f32 v52, %[v0], %[b0_4], v52\n\t"
               "s_set_gpr_idx_idx %[p1]\n\tv_fma_f32 v48, %[v1], %[b1_0], v48\n\tv_fma_f32 v49, %[v1], %[b1_1], v49\n\t"
               "v_fma_f32 v50, %[v1], %[b1_2], v50\n\tv_fma_f32 v51, %[v1], %[b1_3], v51\n\tv_fma_f32 v52, %[v1], %[b1_4], v52\n\t"
               "s_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [p1] "s"(pk[1]), [v1] "s"(v[1]), [b0_0] "v"(b[0][0]),
                 [b0_1] "v"(b[0][1]), [b0_2] "v"(b[0][2]), [b0_3] "v"(b[0][3]), [b0_4] "v"(b[0][4]),
                 [b1_0] "v"(b[1][0]), [b1_1] "v"(b[1][1]), [b1_2] "v"(b[1][2]), [b1_3] "v"(b[1][3]),
                 [b1_4] "v"(b[1][4])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<6, 2>(TileAcc &acc, const uint32_t (&pk)[2], const float (&v)[2], const float (&b)[2][6]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "v_fma_f32 v50, %[v0], %[b0_2], v50\n\tv_fma_f32 v51, %[v0], %[b0_3], v51\n\tv_fma_f32 v52, %[v0], %[b0_4], v52\n\t"
               "v_fma_f32 v53, %[v0], %[b0_5], v53\n\ts_set_gpr_idx_idx %[p1]\n\tv_fma_f32 v48, %[v1], %[b1_0], v48\n\t"
               "v_fma_f32 v49, %[v1], %[b1_1], v49\n\tv_fma_f32 v50, %[v1], %[b1_2], v50\n\tv_fma_f32 v51, %[v1], %[b1_3], v51\n\t"
               "v_fma_f32 v52, %[v1], %[b1_4], v52\n\tv_fma_f32 v53, %[v1], %[b1_5], v53\n\ts_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [p1] "s"(pk[1]), [v1] "s"(v[1]), [b0_0] "v"(b[0][0]),
                 [b0_1] "v"(b[0][1]), [b0_2] "v"(b[0][2]), [b0_3] "v"(b[0][3]), [b0_4] "v"(b[0][4]),
                 [b0_5] "v"(b[0][5]), [b1_0] "v"(b[1][0]), [b1_1] "v"(b[1][1]), [b1_2] "v"(b[1][2]),
                 [b1_3] "v"(b[1][3]), [b1_4] "v"(b[1][4]), [b1_5] "v"(b[1][5])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<8, 2>(TileAcc &acc, const uint32_t (&pk)[2], const float (&v)[2], const float (&b)[2][8]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "v_fma_f32 v50, %[v0], %[b0_2], v50\n\tv_fma_f32 v51, %[v0], %[b0_3], v51\n\tv_fma_f32 v52, %[v0], %[b0_4], v52\n\t"
               "v_fma_f32 v53, %[v0], %[b0_5], v53\n\tv_fma_f32 v54, %[v0], %[b0_6], v54\n\tv_fma_f32 v55, %[v0], %[b0_7], v55\n\t"
               "s_set_gpr_idx_idx %[p1]\n\tv_fma_f32 v48, %[v1], %[b1_0], v48\n\tv_fma_f32 v49, %[v1], %[b1_1], v49\n\t"
               "v_fma_f32 v50, %[v1], %[b1_2], v50\n\tv_fma_f32 v51, %[v1], %[b1_3], v51\n\tv_fma_f32 v52, %[v1], %[b1_4], v52\n\t"
               "v_fma_f32 v53, %[v1], %[b1_5], v53\n\tv_fma_f32 v54, %[v1], %[b1_6], v54\n\tv_fma_f32 v55, %[v1], %[b1_7], v55\n\t"
               "s_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [p1] "s"(pk[1]), [v1] "s"(v[1]), [b0_0] "v"(b[0][0]),
                 [b0_1] "v"(b[0][1]), [b0_2] "v"(b[0][2]), [b0_3] "v"(b[0][3]), [b0_4] "v"(b[0][4]),
                 [b0_5] "v"(b[0][5]), [b0_6] "v"(b[0][6]), [b0_7] "v"(b[0][7]), [b1_0] "v"(b[1][0]),
                 [b1_1] "v"(b[1][1]), [b1_2] "v"(b[1][2]), [b1_3] "v"(b[1][3]), [b1_4] "v"(b[1][4]),
                 [b1_5] "v"(b[1][5]), [b1_6] "v"(b[1][6]), [b1_7] "v"(b[1][7])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<10, 2>(TileAcc &acc, const uint32_t (&pk)[2], const float (&v)[2], const float (&b)[2][10]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "v_fma_f32 v50, %[v0], %[b0_2], v50\n\tv_fma_f32 v51, %[v0], %[b0_3], v51\n\tv_fma_f32 v52, %[v0], %[b0_4], v52\n\t"
               "v_fma_f32 v53, %[v0], %[b0_5], v53\n\tv_fma_f32 v54, %[v0], %[b0_6], v54\n\tv_fma_f32 v55, %[v0], %[b0_7], v55\n\t"
               "v_fma_f32 v56, %[v0], %[b0_8], v56\n\tv_fma_f32 v57, %[v0], %[b0_9], v57\n\ts_set_gpr_idx_idx %[p1]\n\t"
               "v_fma_f32 v48, %[v1], %[b1_0], v48\n\tv_fma_f32 v49, %[v1], %[b1_1], v49\n\tv_fma_f32 v50, %[v1], %[b1_2], v50\n\t"
               "v_fma_f32 v51, %[v1], %[b1_3], v51\n\tv_fma_f32 v52, %[v1], %[b1_4], v52\n\tv_fma_f32 v53, %[v1], %[b1_5], v53\n\t"
               "v_fma_f32 v54, %[v1], %[b1_6], v54\n\tv_fma_f32 v55, %[v1], %[b1_7], v55\n\tv_fma_f32 v56, %[v1], %[b1_8], v56\n\t"
               "v_fma_f32 v57, %[v1], %[b1_9], v57\n\ts_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [p1] "s"(pk[1]), [v1] "s"(v[1]), [b0_0] "v"(b[0][0]),
                 [b0_1] "v"(b[0][1]), [b0_2] "v"(b[0][2]), [b0_3] "v"(b[0][3]), [b0_4] "v"(b[0][4]),
                 [b0_5] "v"(b[0][5]), [b0_6] "v"(b[0][6]), [b0_7] "v"(b[0][7]), [b0_8] "v"(b[0][8]),
                 [b0_9] "v"(b[0][9]), [b1_0] "v"(b[1][0]), [b1_1] "v"(b[1][1]), [b1_2] "v"(b[1][2]),
                 [b1_3] "v"(b[1][3]), [b1_4] "v"(b[1][4]), [b1_5] "v"(b[1][5]), [b1_6] "v"(b[1][6]),
                 [b1_7] "v"(b[1][7]), [b1_8] "v"(b[1][8]), [b1_9] "v"(b[1][9])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<1, 1>(TileAcc &acc, const uint32_t (&pk)[1], const float (&v)[1], const float (&b)[1][1]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\ts_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [b0_0] "v"(b[0][0])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<2, 1>(TileAcc &acc, const uint32_t (&pk)[1], const float (&v)[1], const float (&b)[1][2]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "s_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [b0_0] "v"(b[0][0]), [b0_1] "v"(b[0][1])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<4, 1>(TileAcc &acc, const uint32_t (&pk)[1], const float (&v)[1], const float (&b)[1][4]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "v_fma_f32 v50, %[v0], %[b0_2], v50\n\tv_fma_f32 v51, %[v0], %[b0_3], v51\n\ts_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [b0_0] "v"(b[0][0]), [b0_1] "v"(b[0][1]), [b0_2] "v"(b[0][2]),
                 [b0_3] "v"(b[0][3])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<5, 1>(TileAcc &acc, const uint32_t (&pk)[1], const float (&v)[1], const float (&b)[1][5]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "v_fma_f32 v50, %[v0], %[b0_2], v50\n\tv_fma_f32 v51, %[v0], %[b0_3], v51\n\tv_fma_f32 v52, %[v0], %[b0_4], v52\n\t"
               "s_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [b0_0] "v"(b[0][0]), [b0_1] "v"(b[0][1]), [b0_2] "v"(b[0][2]),
                 [b0_3] "v"(b[0][3]), [b0_4] "v"(b[0][4])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<6, 1>(TileAcc &acc, const uint32_t (&pk)[1], const float (&v)[1], const float (&b)[1][6]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "v_fma_f32 v50, %[v0], %[b0_2], v50\n\tv_fma_f32 v51, %[v0], %[b0_3], v51\n\tv_fma_f32 v52, %[v0], %[b0_4], v52\n\t"
               "v_fma_f32 v53, %[v0], %[b0_5], v53\n\ts_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [b0_0] "v"(b[0][0]), [b0_1] "v"(b[0][1]), [b0_2] "v"(b[0][2]),
                 [b0_3] "v"(b[0][3]), [b0_4] "v"(b[0][4]), [b0_5] "v"(b[0][5])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<8, 1>(TileAcc &acc, const uint32_t (&pk)[1], const float (&v)[1], const float (&b)[1][8]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "v_fma_f32 v50, %[v0], %[b0_2], v50\n\tv_fma_f32 v51, %[v0], %[b0_3], v51\n\tv_fma_f32 v52, %[v0], %[b0_4], v52\n\t"
               "v_fma_f32 v53, %[v0], %[b0_5], v53\n\tv_fma_f32 v54, %[v0], %[b0_6], v54\n\tv_fma_f32 v55, %[v0], %[b0_7], v55\n\t"
               "s_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [b0_0] "v"(b[0][0]), [b0_1] "v"(b[0][1]), [b0_2] "v"(b[0][2]),
                 [b0_3] "v"(b[0][3]), [b0_4] "v"(b[0][4]), [b0_5] "v"(b[0][5]), [b0_6] "v"(b[0][6]),
                 [b0_7] "v"(b[0][7])
               : "m0");
}
template <>
__device__ __forceinline__ void tile_window<10, 1>(TileAcc &acc, const uint32_t (&pk)[1], const float (&v)[1], const float (&b)[1][10]) {
  asm volatile("s_set_gpr_idx_on %[p0], 0xc\n\ts_nop 0\n\tv_fma_f32 v48, %[v0], %[b0_0], v48\n\tv_fma_f32 v49, %[v0], %[b0_1], v49\n\t"
               "v_fma_f32 v50, %[v0], %[b0_2], v50\n\tv_fma_f32 v51, %[v0], %[b0_3], v51\n\tv_fma_f32 v52, %[v0], %[b0_4], v52\n\t"
               "v_fma_f32 v53, %[v0], %[b0_5], v53\n\tv_fma_f32 v54, %[v0], %[b0_6], v54\n\tv_fma_f32 v55, %[v0], %[b0_7], v55\n\t"
               "v_fma_f32 v56, %[v0], %[b0_8], v56\n\tv_fma_f32 v57, %[v0], %[b0_9], v57\n\ts_set_gpr_idx_off"
               : CG_TILE_ACC(acc)
               : [p0] "s"(pk[0]), [v0] "s"(v[0]), [b0_0] "v"(b[0][0]), [b0_1] "v"(b[0][1]), [b0_2] "v"(b[0][2]),
                 [b0_3] "v"(b[0][3]), [b0_4] "v"(b[0][4]), [b0_5] "v"(b[0][5]), [b0_6] "v"(b[0][6]),
                 [b0_7] "v"(b[0][7]), [b0_8] "v"(b[0][8]), [b0_9] "v"(b[0][9])
               : "m0");
}

// All 80 accumulators = 0, by moves of their own: a zero vector assigned in C++ is a loop-invariant value of 32
// registers that the register allocator keeps alive (and spills) across the kernel's loop over units.
#define CG_TILE_Z4(a, b, c, d) "v_mov_b32 v" #a ", 0\n\tv_mov_b32 v" #b ", 0\n\tv_mov_b32 v" #c ", 0\n\tv_mov_b32 v" #d ", 0\n\t"
__device__ __forceinline__ void tile_acc_zero(TileAcc &acc) {
  asm volatile(CG_TILE_Z4(48, 49, 50, 51) CG_TILE_Z4(52, 53, 54, 55) CG_TILE_Z4(56, 57, 58, 59) CG_TILE_Z4(60, 61, 62, 63)
                   CG_TILE_Z4(64, 65, 66, 67) CG_TILE_Z4(68, 69, 70, 71) CG_TILE_Z4(72, 73, 74, 75) CG_TILE_Z4(76, 77, 78, 79)
                       CG_TILE_Z4(80, 81, 82, 83) CG_TILE_Z4(84, 85, 86, 87) CG_TILE_Z4(88, 89, 90, 91) CG_TILE_Z4(92, 93, 94, 95)
                           CG_TILE_Z4(96, 97, 98, 99) CG_TILE_Z4(100, 101, 102, 103) CG_TILE_Z4(104, 105, 106, 107)
                               CG_TILE_Z4(108, 109, 110, 111) CG_TILE_Z4(112, 113, 114, 115) CG_TILE_Z4(116, 117, 118, 119)
                                   CG_TILE_Z4(120, 121, 122, 123) CG_TILE_Z4(124, 125, 126, 127)
               : "={v[48:79]}"(acc.a0), "={v[80:111]}"(acc.a1), "={v[112:127]}"(acc.a2));
}
#undef CG_TILE_Z4

// accumulator e (a constant after unrolling) of the 80
__device__ __forceinline__ float tile_acc_get(const TileAcc &acc, int e) {
  return e < 32 ? acc.a0[e] : e < 64 ? acc.a1[e - 32] : acc.a2[e - 64];
}

// A row of a wide slice, global -> LDS, in PPR pieces of 64 x 16 bytes from one wave-uniform base: M0 is set once and the
// pieces differ in the instruction's immediate offset, which moves the global and the LDS address alike.  The last piece
// runs under `mask` (the lanes that start inside the row), the others with every lane.
template <int PPR>
__device__ __forceinline__ void tile_copy_row(uint32_t lds_addr, const float *base, uint32_t lane16, uint64_t mask) {
  static_assert(PPR >= 1 && PPR <= 3, "pieces of a row");
  uint64_t saved;
  if constexpr (PPR == 3)
    asm volatile(
        "s_mov_b32 m0, %1\n\t"
        "s_mov_b64 %0, exec\n\t"
        "global_load_lds_dwordx4 %2, %3\n\t"
        "global_load_lds_dwordx4 %2, %3 offset:1024\n\t"
        "s_mov_b64 exec, %4\n\t"
        "global_load_lds_dwordx4 %2, %3 offset:2048\n\t"
        "s_mov_b64 exec, %0"
        : "=&s"(saved)
        : "s"(lds_addr), "v"(lane16), "s"(base), "s"(mask)
        : "m0", "memory");
  else if constexpr (PPR == 2)
    asm volatile(
        "s_mov_b32 m0, %1\n\t"
        "s_mov_b64 %0, exec\n\t"
        "global_load_lds_dwordx4 %2, %3\n\t"
        "s_mov_b64 exec, %4\n\t"
        "global_load_lds_dwordx4 %2, %3 offset:1024\n\t"
        "s_mov_b64 exec, %0"
        : "=&s"(saved)
        : "s"(lds_addr), "v"(lane16), "s"(base), "s"(mask)
        : "m0", "memory");
  else
    asm volatile(
        "s_mov_b32 m0, %1\n\t"
        "s_mov_b64 %0, exec\n\t"
        "s_mov_b64 exec, %4\n\t"
        "global_load_lds_dwordx4 %2, %3\n\t"
        "s_mov_b64 exec, %0"
        : "=&s"(saved)
        : "s"(lds_addr), "v"(lane16), "s"(base), "s"(mask)
        : "m0", "memory");
}

struct TileArgs {
  const int32_t *unit_tile, *unit_order, *unit_qstart;
  int32_t *qhead;
  const int32_t *unit_block, *hdr;
  const uint2 *ent;
  const float *B;
  int64_t ldb;
  float *P;
  int32_t f;        // columns of the product
  int32_t fsw;      // columns of a slice (a multiple of 4); slice s covers [s fsw, min(f, (s + 1) fsw))
  int32_t nsl;      // slices
  int32_t m;        // rows of B
  const int32_t *unit_row0, *rank_row;
  float *C;         // nullable: units that are their panel's only block write C = beta C + their rows themselves
  int64_t ldc;
  int32_t rows;
  float beta;
};

// The next (unit, slice) of the queue of the XCD the workgroup runs on, or of the next queue that is not empty:
// unit * nsl + slice, -1 when all queues are empty.  qhead: eight counters, zero at launch.
__device__ __forceinline__ int tile_take_item(const int32_t *__restrict__ unit_queue, const int32_t *__restrict__ qstart,
                                              int32_t *__restrict__ qhead, int nsl) {
  __shared__ int taken;
  if (threadIdx.x == 0) {
    const int xcd = (int)__builtin_amdgcn_s_getreg((3 << 11) | 20) & 7;  // hardware register XCC_ID, bits 0..3
    int item = -1;
    for (int k = 0; k < 8 && item < 0; ++k) {
      const int q = (xcd + k) & 7;
      const int first = qstart[q], count = (qstart[q + 1] - first) * nsl;
      if (count <= 0) continue;
      const int pos = atomicAdd(&qhead[q], 1);
      if (pos < count) item = unit_queue[first + pos / nsl] * nsl + pos % nsl;
    }
    taken = item;
  }
  __syncthreads();
  const int item = __builtin_amdgcn_readfirstlane(taken);
  __syncthreads();  // `taken` is free for the next round
  return item;
}

// NR registers per row, R rows per wave (the panel has 16 R rows), TCW rows of B per wave and tile (the tile has
// 16 TCW columns).  hdr[(tile * 16 + wave) * (TCW + 2) ..]: the TCW rows of B the wave stages, then the range of
// the wave's records.  Place c of a tile is staged by wave c % 16 as its row c / 16 and sits in row c / 16 of
// that wave's staging area of the tile's buffer.
template <int NR, int R, int TCW>
__global__ __launch_bounds__(kPanelThreads) void spmm_tile_kernel(const TileArgs a) {
  static_assert(NR * R <= 80, "80 accumulator registers");
  extern __shared__ __align__(1024) char panel_lds[];  // (the staged rows of narrow slices start on multiples of their stride)
  constexpr int HS = TCW + 2;
  // Slices of up to 256 columns keep a staged row in a fixed stride of 256, 512 or 1024 bytes, whatever the slice's
  // width: the row's offset is then a multiple of it, the record's accumulator index fits below it in the same
  // word, and a lane's LDS address is (word & mask) | the lane's own offset: one instruction.
  constexpr int LROW = NR == 1 ? 256 : NR == 2 ? 512 : NR == 4 ? 1024 : 0;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int32_t *__restrict__ hdr = a.hdr;
  const uint2 *__restrict__ ent = a.ent;
  for (;;) {
    const int item = tile_take_item(a.unit_order, a.unit_qstart, a.qhead, a.nsl);
    if (item < 0) return;
    const int unit = item / a.nsl, slice = item - unit * a.nsl;
    const int col0 = slice * a.fsw;
    const int fs = a.f - col0 < a.fsw ? a.f - col0 : a.fsw;  // columns of this slice
    const float *__restrict__ Bs = a.B + col0;
    const int t0 = a.unit_tile[unit], t1 = a.unit_tile[unit + 1];
    const int c16 = (a.fsw + 3) >> 2;                 // 16-byte pieces of a staged row (every slice alike)
    const int rs = LROW ? LROW : c16 * 16;            // bytes from one staged row to the next
    const uint32_t lim = (uint32_t)fs * 4u;              // bytes of a slice row
    // The last piece of a row may reach up to 12 bytes beyond the slice: into the next slice or the next row of B,
    // which is harmless (those columns of the accumulators are never stored) except behind the last row of B in
    // the last slice, where the bytes may not exist: that one piece is copied float by float instead.
    const bool tail = (fs & 3) != 0 && slice == a.nsl - 1;
    const uint32_t clast = (uint32_t)fs >> 2;
    TileAcc acc;
    tile_acc_zero(acc);

    // Copies of a tile's rows of B.  Slices of at least 256 columns (NR >= 4): row by row, a row in pieces of
    // 64 x 16 bytes from a wave-uniform base address (scalar arithmetic only; the lanes beyond the row's end are
    // switched off inside the copy).  The state below names the next piece; a tile has TCW * ppr of them.
    const int ppr = (c16 + kWave - 1) / kWave;  // pieces of a row
    const int npieces = NR >= 4 ? TCW * ppr : TCW * (LROW / 16) / kWave;  // (narrow slices: 4)
    const int bufsz = kPanelWaves * TCW * rs;  // bytes of a tile's buffer
    const uint32_t lane16 = (uint32_t)lane * 16u;
    const uint32_t ldb32 = (uint32_t)a.ldb;  // the launch refuses leading dimensions of 2^31 and more
    const uint32_t ldb_bytes = ldb32 * 4u;
    const bool b_small = (uint64_t)(uint32_t)a.m * ldb32 * 4u + 4096u < ((uint64_t)1 << 31);  // (offsets that are positive as int32 too)
    int st_r = 0, st_j = 0;
    const float *st_base = Bs;
    uint32_t st_lim = 0;
    auto stage_row = [&](int hrows, int r) {
      const int ridx = __builtin_amdgcn_readlane(hrows, r);
      st_base = Bs + (uint64_t)(uint32_t)ridx * ldb32;
      st_lim = tail && ridx == a.m - 1 ? (lim & ~15u) : lim;
    };
    auto stage_begin = [&](int hrows) {
      st_r = 0;
      st_j = 0;
      stage_row(hrows, 0);
    };
    auto stage_next = [&](int hrows, uint32_t dst_wave) {
      const uint32_t off = lane16 + (uint32_t)st_j * (kWave * 16u);
      panel_copy16_if(dst_wave + (uint32_t)(st_r * rs) + (uint32_t)st_j * (kWave * 16u), st_base, off, st_lim);
      if (++st_j == ppr) {
        st_j = 0;
        if (++st_r < TCW) stage_row(hrows, st_r);
      }
    };
    // The usual case: every row of the slice is as long as the slice's width says (all but the last row of B in a last
    // slice that does not end on a 16-byte piece) and long enough to fill all but the last of its PPR pieces.
    constexpr int PPR = NR == 10 ? 3 : NR >= 5 ? 2 : 1;
    const bool whole_rows = NR >= 4 && lim > (uint32_t)(PPR - 1) * 1024u;
    const uint32_t last_lanes = (lim - (uint32_t)(PPR - 1) * 1024u + 15u) >> 4;  // lanes of the last piece that start inside the row
    const uint64_t last_mask = last_lanes >= 64u ? ~0ull : (1ull << (last_lanes & 63u)) - 1ull;
    auto stage_wide = [&](int hrows, uint32_t dst_wave) {  // all rows of a tile
      if (whole_rows && !tail && b_small) {  // every byte of B within 2 GB of its start: 32-bit offsets from one base
#pragma unroll
        for (int r = 0; r < TCW; ++r) {
          const uint32_t ridx = (uint32_t)__builtin_amdgcn_readlane(hrows, r);
          tile_copy_row<PPR>(dst_wave + (uint32_t)(r * rs), Bs, ridx * ldb_bytes + lane16, last_mask);
        }
      } else if (whole_rows && !tail) {
#pragma unroll
        for (int r = 0; r < TCW; ++r) {
          const uint32_t ridx = (uint32_t)__builtin_amdgcn_readlane(hrows, r);
          tile_copy_row<PPR>(dst_wave + (uint32_t)(r * rs), Bs + (uint64_t)ridx * ldb32, lane16, last_mask);
        }
      } else if (whole_rows) {
#pragma unroll
        for (int r = 0; r < TCW; ++r) {
          const int ridx = __builtin_amdgcn_readlane(hrows, r);
          const float *base = Bs + (uint64_t)(uint32_t)ridx * ldb32;
          if (tail && ridx == a.m - 1) {  // the short row: piece by piece, its last piece is left to stage_tail
            for (int j = 0; j < ppr; ++j)
              panel_copy16_if(dst_wave + (uint32_t)(r * rs) + (uint32_t)j * (kWave * 16u), base, lane16 + (uint32_t)j * (kWave * 16u),
                              lim & ~15u);
          } else {
            tile_copy_row<PPR>(dst_wave + (uint32_t)(r * rs), base, lane16, last_mask);
          }
        }
      } else {
        stage_begin(hrows);
        for (int pc = 0; pc < npieces; ++pc) stage_next(hrows, dst_wave);
      }
    };
    // Narrower slices (NR < 4): a copy instruction covers several rows of B, so every lane has an offset of its own
    // (32 bits from the slice's base: the launch makes sure that B fits).  A staged row takes LROW bytes, and piece
    // q = pc * 64 + lane of the wave's staging area is row q / (LROW / 16), position q % (LROW / 16).  Nothing is
    // switched off: positions behind the row's end copy the row's last piece once more, into places nobody reads.
    // (The launch hands narrow products to this kernel only when f is a multiple of 4, so that every row of B ends
    // with a whole piece.)
    constexpr int NPN = NR >= 4 ? 1 : 4;  // pieces of a tile: 16 rows of 256 bytes, 8 of 512
    int nsel[NPN];
    uint32_t noff[NPN];
    if constexpr (NR < 4) {
      constexpr uint32_t C16L = LROW / 16;
      const uint32_t cmax = (lim - 1u) >> 4;  // the last piece that starts inside a row
#pragma unroll
      for (int pc = 0; pc < NPN; ++pc) {
        const uint32_t q = (uint32_t)(pc * kWave + lane);
        const uint32_t row = q / C16L, c = q % C16L;
        nsel[pc] = (int)(row << 2);
        noff[pc] = (c < cmax ? c : cmax) * 16u;
      }
    }
    auto stage_narrow = [&](int hrows, uint32_t dst_wave) {
#pragma unroll
      for (int pc = 0; pc < NPN; ++pc) {
        if (pc < npieces) {
          const uint32_t ridx = (uint32_t)__builtin_amdgcn_ds_bpermute(nsel[pc], hrows);
          panel_copy16_at(dst_wave + (uint32_t)pc * (kWave * 16u), Bs, ridx * ldb_bytes + noff[pc]);
        }
      }
    };
    auto stage_tail = [&](int hrows, char *dst_wave) {  // the piece left out above
      if (!tail) return;
      const unsigned long long last = __ballot(lane < TCW && hrows == a.m - 1);
      if (last == 0ull) return;
      const int j = __builtin_ctzll(last);
      if (lane < (fs & 3))
        *reinterpret_cast<float *>(dst_wave + j * rs + clast * 16u + lane * 4) =
            Bs[(int64_t)(a.m - 1) * a.ldb + clast * 4u + lane];
    };
    // the wave's header of a tile: lanes 0 .. HS - 1 (the plan keeps two tiles' worth of zero headers behind the last)
    const int32_t *hdr_lane = hdr + ((int64_t)t0 * kPanelWaves + wave) * HS + (lane < HS ? lane : HS - 1);
    auto hdr_load = [&](int dt) { return hdr_lane[(int64_t)dt * (kPanelWaves * HS)]; };  // dt tiles behind the current one
    // 64 records from `first` on, one per lane (the plan keeps 64 records of room behind the last one)
    auto rec_load = [&](int first, int, int) { return ent[(uint32_t)(first + lane)]; };
    const int area = TCW * rs;  // bytes of a wave's staging area in a buffer
    char *const wave_area = panel_lds + wave * area;
    const uint32_t wave_area32 = (uint32_t)(uintptr_t)wave_area;

    uint2 rec = make_uint2(0u, 0u);
    int e0 = 0, e1 = 0, hn = 0;
    if (t1 > t0) {
      const int h0 = hdr_load(0);
      hn = hdr_load(1);
      if constexpr (NR >= 4) {
        stage_wide(h0, wave_area32);
      } else {
        stage_narrow(h0, wave_area32);
      }
      if constexpr (NR >= 4) stage_tail(h0, wave_area);
      e0 = __builtin_amdgcn_readlane(h0, TCW);
      e1 = __builtin_amdgcn_readlane(h0, TCW + 1);
      rec = rec_load(e0, e0, e1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    uint32_t cur_off = 0u, nxt_off = (uint32_t)bufsz;  // the buffer of the tile in use, of the tile on its way
    for (int t = t0; t < t1; ++t) {
      const char *lbase = panel_lds + cur_off;
      // The records of this tile and the header of the next arrived before the last barrier.  Touching them
      // here puts the compiler's wait for them ahead of the copies it cannot see.
      asm volatile("" ::"v"(rec.x), "v"(rec.y), "v"(hn));
      const int e0n = __builtin_amdgcn_readlane(hn, TCW), e1n = __builtin_amdgcn_readlane(hn, TCW + 1);
      const int hn2 = hdr_load(2);
      hdr_lane += kPanelWaves * HS;
      const uint2 recn = rec_load(e0n, e0n, e1n);
      const uint32_t dst32 = wave_area32 + nxt_off;
      // The next tile's copies (behind the unit's last tile: the tile after it, whatever it is, into the free buffer).
      // A wave cannot go on before the memory pipeline has taken its copy instructions, and that pipeline takes one
      // (1 KiB) in about 17 cycles: with all 16 waves issuing their copies at the start of a tile nobody multiplied
      // until the tile's 96 copies were nearly through (cycle counters: 800 cycles per wave in the six copies).  So two
      // of a SIMD's four waves issue theirs behind their records: they multiply while the other two's copies are
      // taken, and the other way round.  (Four different points instead of two: no better.)
      const bool copies_first = ((wave >> 2) & 1) == 0;  // (waves w, w + 4, w + 8, w + 12 share a SIMD)
      if constexpr (NR >= 4) {
        if (copies_first) stage_wide(hn, dst32);
      } else {
        if (copies_first) stage_narrow(hn, dst32);
      }

      // cnt records in the lanes of r.  K records at a time: their rows of B are read from LDS, then one stretch of
      // index mode multiplies them (while a wave waits for its reads the other waves of the SIMD multiply).  A
      // record becomes one word: the LDS offset of its row of B and, in the low 8 bits, its first accumulator.
      const uint32_t lane_off = (uint32_t)lane * (NR == 1 ? 4u : NR == 2 ? 8u : 16u);
      // the lane's second piece of a row: behind the first 1024 (2048) bytes, 4 (8) bytes per lane
      const uint32_t lane_off2 = NR == 5 ? 1024u + (uint32_t)lane * 4u : NR == 6 ? 1024u + (uint32_t)lane * 8u
                                                                                  : 2048u + (uint32_t)lane * 8u;
      const uint32_t lbase32 = (uint32_t)(uintptr_t)lbase;
      auto process = [&](const uint2 r, int cnt) {
        const uint32_t c = r.x & 0xffu;
        const uint32_t rowoff = lbase32 + (c & 15u) * (uint32_t)area + (c >> 4) * (uint32_t)rs;
        const uint32_t idx = (r.x >> 8) * (uint32_t)NR;
        const uint32_t packed = LROW ? (rowoff | idx) : ((rowoff << 8) | idx);
        constexpr int K = NR == 1 ? 8 : NR == 2 ? 4 : 2;
        auto read = [&](uint32_t pk, float (&b)[NR]) {
          if constexpr (LROW != 0) {
            uint32_t addr;  // (pk & ~(LROW - 1)) | lane_off: the row's address is a multiple of LROW, the index lies below it
            asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(addr) : "s"(pk), "v"(~(uint32_t)(LROW - 1)), "v"(lane_off));
            tile_row_read<NR>(addr, 0u, b);
          } else {
            const uint32_t row = pk >> 8;
            tile_row_read<NR>(row + lane_off, row + lane_off2, b);
          }
        };
        auto step = [&](int first) {  // K records from lane `first` on
          uint32_t pk[K];
          float v[K], b[K][NR];
#pragma unroll
          for (int k = 0; k < K; ++k) {
            pk[k] = __builtin_amdgcn_readlane(packed, first + k);
            v[k] = __uint_as_float(__builtin_amdgcn_readlane(r.y, first + k));
            read(pk[k], b[k]);
          }
          tile_window<NR, K>(acc, pk, v, b);
          __builtin_amdgcn_sched_barrier(0);  // the next K records' reads stay behind this stretch (registers)
        };
        int i = 0;
        for (; i + K <= cnt; i += K) step(i);
        for (; i < cnt; ++i) {
          uint32_t pk[1];
          float v[1], b[1][NR];
          pk[0] = __builtin_amdgcn_readlane(packed, i);
          v[0] = __uint_as_float(__builtin_amdgcn_readlane(r.y, i));
          read(pk[0], b[0]);
          tile_window<NR, 1>(acc, pk, v, b);
        }
      };
      // the first 64 records came with the last tile; a (tile, wave) with more loads the others here (few tiles have
      // that many: the fullest ones are the dense tiles of the panel plan)
      if (e1 > e0) process(rec, e1 - e0 < kWave ? e1 - e0 : kWave);
      for (int base = e0 + kWave; base < e1; base += kWave) {
        const uint2 more = rec_load(base, e0, e1);
        process(more, e1 - base < kWave ? e1 - base : kWave);
      }
      if constexpr (NR >= 4) {
        if (!copies_first) stage_wide(hn, dst32);
      } else {
        if (!copies_first) stage_narrow(hn, dst32);
      }
      if constexpr (NR >= 4) stage_tail(hn, wave_area + nxt_off);
      rec = recn;
      e0 = e0n;
      e1 = e1n;
      hn = hn2;
      {
        const uint32_t o = cur_off;
        cur_off = nxt_off;
        nxt_off = o;
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }

    // C[row, slice] = beta C[row, slice] + the sums (the unit is the only block of its panel), or the unit's block
    // of partial rows: P[block][slot * 16 + wave][:], position in the block = rank of the row inside its panel.
    const int row0 = a.C ? a.unit_row0[unit] : -1;
    const int block = a.unit_block[unit];
#pragma unroll
    for (int s = 0; s < R; ++s) {
      float *out;
      float beta = 0.f;
      if (row0 >= 0) {
        const int rank = row0 + s * kPanelWaves + wave;
        if (rank >= a.rows) continue;
        out = a.C + (int64_t)a.rank_row[rank] * a.ldc + col0;
        beta = a.beta;
      } else {
        out = a.P + ((int64_t)block * (kPanelWaves * R) + s * kPanelWaves + wave) * a.f + col0;
      }
#pragma unroll
      for (int k = 0; k < NR; ++k) {
        const int col = tile_col<NR>(k, lane);
        if (col < fs) {
          float v = tile_acc_get(acc, s * NR + k);
          if (beta != 0.f) v += beta * out[col];
          out[col] = v;
        }
      }
    }
  }  // the next (unit, slice)
}

}  // namespace cg
