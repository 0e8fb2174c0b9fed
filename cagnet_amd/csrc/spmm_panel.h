// Panel plan of the wide CSR SpMM: a matrix whose rows share columns is multiplied out of LDS, tile by tile.
//
// A row-wise SpMM gathers one row of B per stored entry (2408 bytes at f = 602); on a matrix with a
// few hundred entries per row nearly all of that traffic is re-reading rows of B that other rows of A
// also use.  Here rows are ranked by their entry counts and taken in panels of 128 consecutive ranks;
// inside a panel the columns the panel uses are ranked (those with several entries in these 128 rows
// first, each group in the order of the columns' entry counts over the whole matrix) and taken in blocks
// of 32 consecutive ranks: every panel has its own blocks, and all panels walk the columns in the same
// order.  A (panel, block) tile has its 32 rows of B copied into LDS once (global -> LDS directly, no
// registers in between) and all of the tile's entries read them from there, at LDS bandwidth instead
// of through the vector memory path.  A workgroup of 16 waves owns a unit = a run of tiles of one
// panel; wave w holds the accumulators of the 8 rows {w, w + 16, ...} of the panel in registers for the
// whole unit and writes them out once as partial rows.  Tiles with many entries ("dense" tiles) are
// stored as full 128 x 32 blocks instead and multiplied on the fp32 matrix cores
// (v_mfma_f32_16x16x4_f32: exact fp32 products, fp32 accumulation) by a second kernel, in units of
// their own; the zeros of such a block are multiplied too, so a row of B that holds an infinity or a
// NaN reaches every row of the block (the row-wise kernels and cusparseSpMM would only touch the rows
// that reference it).  By default every tile is multiplied by one of the two kernels; a unit that is
// the only one of its panel writes C = beta C + its rows itself, and a last pass writes the other rows
// as C = beta C + the sum of their panel's partial rows.  Tiles that a threshold leaves out keep their
// entries in a second CSR matrix (the "rest") that the row-wise kernels multiply, and their finished
// rows add the partial rows in.  The staged-tile kernel runs one workgroup per compute unit; the units
// wait in one queue per XCD (neighbouring panels' units, which walk the same rows of B, one behind the
// other, so that they share that XCD's L2) and a workgroup takes units until all queues are empty.  Replaces nothing in the reference beyond cusparseSpMM itself
// (sparse-extension/sparse_coo_tensor.cu:215-226); sums are in a fixed order, no atomics on floats.
#pragma once
#include "spmm_tables.h"
#include <algorithm>
#include <vector>

namespace cg {

constexpr int kPanelRows = 128;   // rows of a panel
constexpr int kPanelWaves = 16;   // waves of a workgroup; wave w owns rows w, w + 16, ... of the panel
constexpr int kPanelSlots = kPanelRows / kPanelWaves;  // rows per wave
constexpr int kPanelCols = 32;    // columns of a block = rows of B staged per tile
constexpr int kPanelThreads = kPanelWaves * kWave;
constexpr int32_t kPanelMinF = 258, kPanelMaxF = 636;  // widths the kernel is instantiated for (even)

constexpr int kDenseWaves = 8;    // waves of a workgroup of the dense-tile kernel; wave w owns rows 16 w .. 16 w + 15
constexpr int kDenseThreads = kDenseWaves * kWave;
constexpr int kDenseTileFloats = kPanelRows * kPanelCols;

static std::atomic<int> g_tune_panel{0}, g_tune_panel_emin{0}, g_tune_panel_cols{0}, g_tune_panel_unit{0};
static std::atomic<int> g_tune_panel_dmin{0}, g_tune_panel_dwg{0}, g_tune_panel_share{0}, g_tune_tile{0}, g_tune_strict{0};
static std::atomic<int> g_tune_panel_costcap{0};  // microseconds of modelled cost from which a unit is cut at the latest (0: 100)
static std::atomic<int> g_tune_panel_legacy{0};  // > 0: the panel plan's staged tiles through spmm_panel_kernel (padded records)
static std::atomic<int> g_tune_panel_qskip{0}, g_tune_panel_qcap{0};  // measuring aid: a launch takes units qskip .. qcap - 1 of every queue only

struct CsrSide;

struct PanelPlan {
  bool valid = false, declined = false, failed = false;  // failed: declined because the build ran out of memory
  int32_t emin = 0, hot_cols = 0, unit_entries = 0, dmin = 0, dwg = 0;  // what the plan was built with
  bool share = true;
  int32_t prows = 128, tcols = 32;  // rows of a panel (a multiple of 16) and columns of a tile (a multiple of 16, at most
                                    // 256); the matrix-core kernels and spmm_panel_kernel need 128 x 32
  bool padded = true;               // odd (tile, wave, slot) runs of records are padded (spmm_panel_kernel needs that)
  int64_t covered = 0;      // entries the panel kernel multiplies
  int64_t dcovered = 0;     // entries in dense tiles (the matrix-core kernel)
  int32_t ntiles = 0, nunits = 0, nsplit = 0;
  int32_t bcols = 0;               // columns of the matrix = rows of B
  int32_t ndtiles = 0, ndunits = 0;
  int32_t nblocks = 0;             // blocks of 128 partial rows, one per unit of either kind
  int32_t *unit_tile = nullptr;    // [nunits + 1] tiles of a unit (units never span panels)
  int32_t *unit_order = nullptr;   // [nunits] the units in eight queues, one per XCD, each in launch order
  int32_t *unit_qstart = nullptr;  // [9] where the queues start in unit_order
  int32_t *unit_block = nullptr;   // [nunits] block of partial rows a unit writes
  int32_t ndwg = 0;                // workgroups of the dense-tile kernel: equal shares of the list of dense tiles
  int32_t *dwg_unit = nullptr;     // [ndwg + 1] units of a workgroup (runs of tiles of one panel inside its share)
  int32_t *dunit_tile = nullptr;   // [ndunits + 1] dense tiles of a unit
  int32_t *dunit_block = nullptr;  // [ndunits] block of partial rows a unit writes
  int32_t *dhdr = nullptr;         // [ndtiles * 32] row of B of every column of a dense tile
  float *dA = nullptr;             // [ndtiles * 4096] dense tiles in the operand layout of the matrix instruction
  int32_t *hdr = nullptr;          // [ntiles * 16 * 4] per (tile, wave): two rows of B to stage, record range
  int64_t nrec = 0;                // records: the covered entries and the zeros that pad odd runs
  uint2 *ent = nullptr;            // [nrec] {column in block | slot << 8, value bits}, by (tile, wave, slot); every
                                   // (tile, wave, slot) run has an even number of records
  int32_t *dslot = nullptr;        // [rows] partial row of a row of A: block * 128 + position, or -1
  int32_t *split = nullptr;        // [2 * nsplit] (first block, blocks) of panels that have several units
  int32_t *bcount = nullptr;       // [nblocks] blocks of the panel whose first block this is (0 for its other blocks);
                                   // -1: one block, of a staged unit, which can write its rows of C itself
  int32_t *unit_row0 = nullptr;    // [nunits] rank of the first row of the unit's panel if the unit is its only block, else -1
  int32_t *rank_row = nullptr;     // [rows] the row of every rank (rows by descending length)
  int32_t *finish_rows = nullptr;  // [nfinish] the rows that the pass over the partial rows writes: all but those of panels
                                   // whose only block is a staged unit's
  int32_t nfinish = 0;
  CsrSide *rest = nullptr;         // entries outside active tiles, same rows and columns
  void release();
};

// -------------------------------------------------------------------------------------------------
// the product kernel
// -------------------------------------------------------------------------------------------------
// One 16-byte (or 4-byte) piece per lane from global memory straight into LDS at lds_addr + lane * size (the
// instruction takes the LDS address from m0, one wait state after the move that sets it).
// The compiler does not see these loads: it would otherwise wait for them before every LDS read (it
// cannot tell the two LDS buffers apart); the kernel waits for them itself before the barrier.
__device__ __forceinline__ void panel_copy16(uint32_t lds_addr, const float *src) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(src) : "m0", "memory");
}
__device__ __forceinline__ void panel_copy4(uint32_t lds_addr, const float *src) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_addr), "v"(src) : "m0", "memory");
}
// The same with the source as a wave-uniform base and a 32-bit byte offset per lane (no 64-bit address per lane).
__device__ __forceinline__ void panel_copy16_at(uint32_t lds_addr, const float *base, uint32_t byte_off) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(byte_off), "s"(base) : "m0", "memory");
}
__device__ __forceinline__ void panel_copy4_at(uint32_t lds_addr, const float *base, uint32_t byte_off) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_addr), "v"(byte_off), "s"(base) : "m0", "memory");
}

// Lanes with byte_off < limit copy 16 (4) bytes from base + byte_off to LDS at lds_addr + lane * 16 (4).
__device__ __forceinline__ void panel_copy16_if(uint32_t lds_addr, const float *base, uint32_t byte_off, uint32_t limit) {
  uint64_t saved;
  asm volatile(
      "s_mov_b64 %0, exec\n\t"
      "v_cmp_gt_u32 vcc, %4, %2\n\t"
      "s_and_b64 exec, exec, vcc\n\t"
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %2, %3\n\t"
      "s_mov_b64 exec, %0"
      : "=&s"(saved)
      : "s"(lds_addr), "v"(byte_off), "s"(base), "s"(limit)
      : "vcc", "scc", "m0", "memory");  // s_and writes scc
}
__device__ __forceinline__ void panel_copy4_if(uint32_t lds_addr, const float *base, uint32_t byte_off, uint32_t limit) {
  uint64_t saved;
  asm volatile(
      "s_mov_b64 %0, exec\n\t"
      "v_cmp_gt_u32 vcc, %4, %2\n\t"
      "s_and_b64 exec, exec, vcc\n\t"
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dword %2, %3\n\t"
      "s_mov_b64 exec, %0"
      : "=&s"(saved)
      : "s"(lds_addr), "v"(byte_off), "s"(base), "s"(limit)
      : "vcc", "scc", "m0", "memory");  // s_and writes scc
}

// hdr[(tile * 16 + wave) * 4 ..]: the two rows of B the wave stages for the tile and the range of its records.
// It is read two tiles ahead and the records one tile ahead, so that no load of a tile depends on another
// load of the same tile: the copies of the next tile go out as soon as the barrier has been passed.
//
// A wave walks its records of a tile two at a time and has the row of B of the record behind the current one on
// its way from LDS while the current one is multiplied: a record costs 2408 bytes of LDS reads (f = 602)
// whose latency four waves per SIMD do not hide by themselves.
// A workgroup takes the next unit from the queue of the XCD it runs on (the plan fills the queues so that the
// workgroups of an XCD walk the same rows of B at the same time, and evenly by its estimate of the units' costs) and,
// once that queue is empty, from the next XCD's that is not: what an XCD is short of by the estimate's error the
// others make up.  Returns -1 when every queue is empty.  qhead: eight counters, zero at launch.
__device__ __forceinline__ int panel_take_unit(const int32_t *__restrict__ unit_queue, const int32_t *__restrict__ qstart,
                                               int32_t *__restrict__ qhead, int32_t qcap) {
  __shared__ int taken;
  if (threadIdx.x == 0) {
    const int xcd = (int)__builtin_amdgcn_s_getreg((3 << 11) | 20) & 7;  // hardware register XCC_ID, bits 0..3
    int unit = -1;
    for (int k = 0; k < 8 && unit < 0; ++k) {
      const int q = (xcd + k) & 7;
      const int first = qstart[q];
      int count = qstart[q + 1] - first;
      if (qcap > 0 && count > qcap) count = qcap;  // measuring aid (spmm_panel_qcap): only the queue's first units
      if (count <= 0) continue;
      const int pos = atomicAdd(&qhead[q], 1);
      if (pos < count) unit = unit_queue[first + pos];
    }
    taken = unit;
  }
  __syncthreads();
  return __builtin_amdgcn_readfirstlane(taken);
}

template <int CHUNKS>
__global__ __launch_bounds__(kPanelThreads) void spmm_panel_kernel(
    const int32_t *__restrict__ unit_tile, const int32_t *__restrict__ unit_order, const int32_t *__restrict__ unit_qstart,
    int32_t *__restrict__ qhead, const int32_t *__restrict__ unit_block,
    const int32_t *__restrict__ hdr, const uint2 *__restrict__ ent, const float *__restrict__ B, int64_t ldb,
    float *__restrict__ P, int32_t f, const int32_t *__restrict__ unit_row0, const int32_t *__restrict__ rank_row,
    float *__restrict__ C, int64_t ldc, int32_t rows, float beta, int32_t qcap) {
  extern __shared__ __align__(16) char panel_lds[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  // One workgroup per compute unit, each taking units until the queues are empty (no workgroup waits for another).
  for (;;) {
  const int unit = panel_take_unit(unit_order, unit_qstart, qhead, qcap);
  if (unit < 0) return;
  const int t0 = unit_tile[unit], t1 = unit_tile[unit + 1];
  const int npair = f >> 1;
  const int rs = (f * 4 + 15) & ~15;  // bytes of a staged row: 16-byte aligned for the direct copies
  const int bufsz = kPanelCols * rs;
  constexpr int RPW = kPanelCols / kPanelWaves;  // rows of B a wave stages per tile
  static_assert(RPW == 2, "the header holds two staged rows per wave");
  float2 acc[kPanelSlots][CHUNKS];
#pragma unroll
  for (int s = 0; s < kPanelSlots; ++s)
#pragma unroll
    for (int ch = 0; ch < CHUNKS; ++ch) acc[s][ch] = make_float2(0.f, 0.f);

  // A wave stages two rows of B per tile, in pieces of one copy instruction each: per row NX4 of 64 x 16
  // bytes and one of 4-byte words (for widths that are not a multiple of 4; lanes without a piece are switched
  // off inside the copy).  One copy instruction keeps the CU's vector memory path busy for 16 cycles, and a
  // wave that issues its copies back to back sits behind those of the 15 other waves: the pieces of the next
  // tile are therefore issued one at a time, piece s ahead of the records of slot s.  Which piece that is
  // (row, position, kind) is known when the slot loop is unrolled, so that no address arithmetic is left.
  constexpr int NX4 = CHUNKS == 5 ? 3 : 2;  // 16-byte pieces of a row at the widest f of the class (636 / 512 / 384)
  constexpr int PPR = NX4 + 1, NPIECES = RPW * PPR;
  static_assert(NPIECES <= kPanelSlots, "one piece per slot");
  const int nq = f >> 2;
  const uint32_t lim16 = (uint32_t)nq * 16u, lim4 = (uint32_t)f * 4u;
  const uint32_t lane16 = (uint32_t)lane * 16u, tail_off = lim16 + (uint32_t)lane * 4u;
  const uint32_t lds_wave = (uint32_t)(uintptr_t)panel_lds + (uint32_t)(wave * rs);  // the wave's first row in buffer 0
  const uint32_t lds_row1 = (uint32_t)(kPanelWaves * rs);                             // its second row behind it
  const uint32_t ldb32 = (uint32_t)ldb;                                               // ldb < 2^31 (launch_panel refuses larger ones)
  auto stage_piece = [&](int pc, const float *srca, const float *srcb, uint32_t dst0) {  // pc: a constant after unrolling
    const int r = pc / PPR, j = pc % PPR;
    const uint32_t dst = dst0 + (r ? lds_row1 : 0u);
    const float *src = r ? srcb : srca;
    if (j < NX4 - 1)  // every width of the class fills these pieces: no lane to switch off
      panel_copy16_at(dst + j * (kWave * 16), src, lane16 + (uint32_t)(j * kWave * 16));
    else if (j < NX4)
      panel_copy16_if(dst + j * (kWave * 16), src, lane16 + (uint32_t)(j * kWave * 16), lim16);
    else
      panel_copy4_if(dst + lim16, src, tail_off, lim4);
  };
  // lanes 0..3 of a wave fetch the four words of its header (a vector load: its wait is the one at the
  // end of the tile, with the copies, not the LDS counter)
  auto hdr_load = [&](int t) { return hdr[((int64_t)t * kPanelWaves + wave) * 4 + (lane & 3)]; };
  // records of a (tile, wave), 64 of them from `first`: one per lane, clamped to the range
  auto rec_load = [&](int first, int b0, int b1) {
    int idx = first + lane;
    idx = idx < b1 ? idx : (b1 > b0 ? b1 - 1 : 0);
    return ent[idx];
  };
  uint2 rec = make_uint2(0u, 0u);
  int e0 = 0, e1 = 0, hn = 0;
  if (t1 > t0) {
    const int h0 = hdr_load(t0);
    hn = hdr_load(t0 + 1 < t1 ? t0 + 1 : t0);
    const float *srca = B + (int64_t)__builtin_amdgcn_readlane(h0, 0) * ldb;
    const float *srcb = B + (int64_t)__builtin_amdgcn_readlane(h0, 1) * ldb;
#pragma unroll
    for (int pc = 0; pc < NPIECES; ++pc) stage_piece(pc, srca, srcb, lds_wave);
    e0 = __builtin_amdgcn_readlane(h0, 2);
    e1 = __builtin_amdgcn_readlane(h0, 3);
    rec = rec_load(e0, e0, e1);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  for (int t = t0; t < t1; ++t) {
    const int buf = (t - t0) & 1;
    const char *lbase = panel_lds + buf * bufsz + lane * 8;
    // The records of this tile and the header of the next arrived before the last barrier.  Touching them
    // here puts the compiler's wait for them ahead of the copies it cannot see, so that nothing below
    // waits for those.
    asm volatile("" ::"v"(rec.x), "v"(rec.y), "v"(hn));
    // the next tile (the last tile names itself and is staged once more)
    const int q0 = __builtin_amdgcn_readlane(hn, 0), q1 = __builtin_amdgcn_readlane(hn, 1);
    const int e0n = __builtin_amdgcn_readlane(hn, 2), e1n = __builtin_amdgcn_readlane(hn, 3);
    const int hn2 = hdr_load(t + 2 < t1 ? t + 2 : t1 - 1);
    const uint2 recn = rec_load(e0n, e0n, e1n);
    const float *srca = B + (uint64_t)(uint32_t)q0 * ldb32, *srcb = B + (uint64_t)(uint32_t)q1 * ldb32;  // unsigned 32 x 32 -> 64
    const uint32_t dst0 = lds_wave + (uint32_t)((buf ^ 1) * bufsz);

    // cnt >= 2 records in the lanes of r, sorted by slot, every slot's run of even length (the plan pads odd
    // runs with a record of value 0): the lanes' ballots give the length of every slot's run, and a run adds
    // into that slot's registers (static register indices), two records per step.  While a record is
    // multiplied the row of B of the record behind it (whatever its slot) is on its way from LDS into the
    // other of two sets of registers.
    auto process = [&](const uint2 r, int cnt, bool stage) {
      float2 ba[CHUNKS], bb[CHUNKS];
      const uint32_t myslot = (r.x >> 8) & 0x7u;
      const uint32_t row_off = (r.x & 0xffu) * (uint32_t)rs;  // of every record of the batch at once
      auto row_read = [&](int idx, float2 (&b)[CHUNKS]) {
        const char *src = lbase + __builtin_amdgcn_readlane(row_off, idx);
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch) b[ch] = *reinterpret_cast<const float2 *>(src + ch * 512);
      };
      row_read(0, ba);
      int i = 0;
#pragma unroll
      for (int s = 0; s < kPanelSlots; ++s) {
        if (s < NPIECES && stage) stage_piece(s, srca, srcb, dst0);
        const int end = i + __builtin_popcountll(__ballot(lane < cnt && myslot == (uint32_t)s));
        for (; i < end; i += 2) {
          const float v0 = __uint_as_float(__builtin_amdgcn_readlane(r.y, i));
          const float v1 = __uint_as_float(__builtin_amdgcn_readlane(r.y, i + 1));
          row_read(i + 1, bb);
          __builtin_amdgcn_sched_barrier(0);  // the reads stay ahead of the multiplies they overlap with
#pragma unroll
          for (int ch = 0; ch < CHUNKS; ++ch) {
            acc[s][ch].x = fmaf(v0, ba[ch].x, acc[s][ch].x);
            acc[s][ch].y = fmaf(v0, ba[ch].y, acc[s][ch].y);
          }
          row_read((i + 2) & (kWave - 1), ba);  // behind the last record: a lane that holds a copy of it (rec_load)
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int ch = 0; ch < CHUNKS; ++ch) {
            acc[s][ch].x = fmaf(v1, bb[ch].x, acc[s][ch].x);
            acc[s][ch].y = fmaf(v1, bb[ch].y, acc[s][ch].y);
          }
        }
      }
    };
    // 64 records at a time; a dense tile's further records are fetched while the batch before them is multiplied
    uint2 cur = rec;
    for (int base = e0; base < e1; base += kWave) {
      const int left = e1 - base;
      uint2 nxt = cur;
      if (left > kWave) nxt = rec_load(base + kWave, e0, e1);
      process(cur, left > kWave ? kWave : left, base == e0);
      cur = nxt;
    }
    if (e0 >= e1) {  // a wave without records in this tile
#pragma unroll
      for (int pc = 0; pc < NPIECES; ++pc) stage_piece(pc, srca, srcb, dst0);
    }
    rec = recn;
    e0 = e0n;
    e1 = e1n;
    hn = hn2;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }
  // The only block of its panel (C given): C[row, :] = beta C[row, :] + the sums, nothing left to add up.
  const int row0 = C ? unit_row0[unit] : -1;
  if (row0 >= 0) {
#pragma unroll
    for (int s = 0; s < kPanelSlots; ++s) {
      const int rank = row0 + s * kPanelWaves + wave;  // position in the panel = rank of the row inside it
      if (rank < rows) {
        float *crow = C + (int64_t)rank_row[rank] * ldc;
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch) {
          const int p = lane + kWave * ch;
          if (p < npair) {
            float2 v = acc[s][ch];
            if (beta != 0.f) {
              v.x += beta * crow[2 * p];
              v.y += beta * crow[2 * p + 1];
            }
            crow[2 * p] = v.x;
            crow[2 * p + 1] = v.y;
          }
        }
      }
    }
    continue;
  }
  // P[block][slot * 16 + wave][:]: position in the block = rank of the row inside its panel
  const int block = unit_block[unit];
#pragma unroll
  for (int s = 0; s < kPanelSlots; ++s) {
    float *prow = P + ((int64_t)block * kPanelRows + s * kPanelWaves + wave) * f;
#pragma unroll
    for (int ch = 0; ch < CHUNKS; ++ch) {
      const int p = lane + kWave * ch;
      if (p < npair) *reinterpret_cast<float2 *>(prow + 2 * p) = acc[s][ch];
    }
  }
  }  // the next unit
}

// -------------------------------------------------------------------------------------------------
// dense tiles on the fp32 matrix cores
// -------------------------------------------------------------------------------------------------
// A dense tile is a full 128 x 32 block of A.  Wave w of 8 owns rows 16 w .. 16 w + 15 of the panel and all
// columns of the result: per tile 8 reduction steps of 4 columns of A (= 4 staged rows of B), each one
// v_mfma_f32_16x16x4_f32 per 16 result columns.  Register layout of the instruction (lane l):
//   A (16 x 4): lane holds A[l % 16][l / 16]      B (4 x 16): lane holds B[l / 16][l % 16]
//   D (16 x 16) in 4 registers: register v holds D[4 (l / 16) + v][l % 16]
// The 16 columns of one instruction are taken 4 apart: lane (q, c) = (l / 16, l % 16) reads the 16 bytes
// B[4 ks + q][64 g + 4 c .. + 3] from LDS and feeds its four floats to four instructions, so that the lane ends
// up with four consecutive result columns per group g of 64 columns.
// dA[((tile * 8 + wave) * 2 + ks / 4) * 256 + lane * 4 + ks % 4] = A[16 wave + lane % 16][4 ks + lane / 16].
//
// All dense tiles cost the same, so every workgroup takes an equal share of the list of dense tiles (in
// (panel, column block) order) and walks it in one pipeline.  A unit is a run of tiles of one panel inside one
// share; after a unit's last tile the accumulators go out as that unit's block of partial rows.
//
// The loop over the tiles of a unit has no branch in it: the accumulators of the matrix instructions are
// live across it, and a loop body of many basic blocks makes the register allocator move them from register
// to register between the instructions (and spill).  The copies of the next tile are therefore predicated
// inside their asm statement (exec is narrowed to the lanes that have a piece and put back).
typedef float panel_f4 __attribute__((ext_vector_type(4)));

template <int NG>  // groups of 64 result columns: ceil(f / 64)
__global__ __launch_bounds__(kDenseThreads) void spmm_panel_dense_kernel(
    const int32_t *__restrict__ wg_unit, const int32_t *__restrict__ unit_tile, const int32_t *__restrict__ unit_block,
    const int32_t *__restrict__ dhdr, const float *__restrict__ dA, const float *__restrict__ B, int64_t ldb,
    float *__restrict__ P, int32_t f) {
  extern __shared__ __align__(16) char panel_lds[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int c16 = lane & 15, q = lane >> 4;
  const int u0 = wg_unit[blockIdx.x], u1 = wg_unit[blockIdx.x + 1];
  if (u0 >= u1) return;
  const int t_first = unit_tile[u0], t_end = unit_tile[u1];  // the units of a workgroup are consecutive, and so are their tiles
  const int rs = (f * 4 + 15) & ~15;  // bytes of a staged row
  const int bufsz = kPanelCols * rs;
  constexpr int RPW = kPanelCols / kDenseWaves;  // rows of B a wave stages per tile
  static_assert(RPW == 4, "a wave reads the four rows it stages from lanes 0..3 of its header");
  // A row is staged in NX4 pieces of 64 x 16 bytes and one of up to 3 x 4 bytes behind the last whole 16 bytes
  // (widths that are not a multiple of 4); which lanes of a piece have something to copy depends on f.
  constexpr int NX4 = (NG + 3) / 4, PPR = NX4 + 1, NPIECES = RPW * PPR;
  static_assert(NPIECES <= 4 * NG, "one copy per two groups of a tile's 8 NG group steps must cover all pieces");
  const uint32_t lim16 = (uint32_t)(f >> 2) * 16u, lim4 = (uint32_t)f * 4u;
  const uint32_t tail_off = lim16 + (uint32_t)lane * 4u;  // byte offset of the lane's 4-byte piece
  auto stage_piece = [&](int pc, const float *const (&src4)[RPW], int buf) {  // pc is a constant after unrolling
    const int r = pc / PPR, j = pc % PPR;
    const uint32_t dst = (uint32_t)(uintptr_t)(panel_lds + buf * bufsz + (wave + r * kDenseWaves) * rs);
    if (j < NX4)
      panel_copy16_if(dst + j * (kWave * 16), src4[r], (uint32_t)(j * kWave + lane) * 16u, lim16);
    else
      panel_copy4_if(dst + lim16, src4[r], tail_off, lim4);
  };
  auto hdr_load = [&](int t) { return dhdr[(int64_t)t * kPanelCols + wave + kDenseWaves * (lane & 3)]; };
  auto a_load = [&](int t, float4 (&a)[2]) {
    const float4 *src = reinterpret_cast<const float4 *>(dA) + ((int64_t)t * kDenseWaves + wave) * 2 * kWave + lane;
    a[0] = src[0];
    a[1] = src[kWave];
  };
  // byte offset of the lane's piece of group g inside a staged buffer at reduction step 0: off_main + 256 g,
  // except that the last group's pieces beyond the row end are clamped to the row's last piece (their result
  // columns are never stored)
  const int off_main = q * rs + 16 * c16;
  int last_col = (NG - 1) * 64 + 4 * c16;
  last_col = last_col < rs / 4 - 4 ? last_col : rs / 4 - 4;
  const int off_last = q * rs + last_col * 4;
  auto b_read = [&](const char *lb, int ks, int g) {
    return *reinterpret_cast<const float4 *>(lb + ks * 4 * rs + (g < NG - 1 ? off_main + g * 256 : off_last));
  };

  float4 a_cur[2];
  int hn;
  {
    const int h0 = hdr_load(t_first);
    hn = hdr_load(t_first + 1 < t_end ? t_first + 1 : t_first);
    const float *src4[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) src4[r] = B + (int64_t)__builtin_amdgcn_readlane(h0, r) * ldb;
#pragma unroll
    for (int pc = 0; pc < NPIECES; ++pc) stage_piece(pc, src4, 0);
    a_load(t_first, a_cur);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  int buf = 0;
  for (int u = u0; u < u1; ++u) {
    panel_f4 acc[NG][4];
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[g][j] = (panel_f4){0.f, 0.f, 0.f, 0.f};
    const int ut1 = unit_tile[u + 1];
    for (int t = unit_tile[u]; t < ut1; ++t) {
      // the operands of this tile and the header of the next arrived before the last barrier: naming them here
      // puts the compiler's wait for them ahead of the copies it cannot see
      asm volatile("" ::"v"(a_cur[0].x), "v"(a_cur[1].x), "v"(hn));
      const float *src4[RPW];  // the next tile (the last tile of the share names itself and is staged once more)
#pragma unroll
      for (int r = 0; r < RPW; ++r) src4[r] = B + (int64_t)__builtin_amdgcn_readlane(hn, r) * ldb;
      int hn2 = 0;
      float4 a_nxt[2];
      const float a8[8] = {a_cur[0].x, a_cur[0].y, a_cur[0].z, a_cur[0].w, a_cur[1].x, a_cur[1].y, a_cur[1].z, a_cur[1].w};
      const char *lb = panel_lds + buf * bufsz;
      float4 b[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) b[g] = b_read(lb, 0, g);
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        if (ks == 6) {  // operands of the next tile and the header of the one after it: late, when most of a8 is dead
          hn2 = hdr_load(t + 2 < t_end ? t + 2 : t_end - 1);
          a_load(t + 1 < t_end ? t + 1 : t, a_nxt);
        }
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          acc[g][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a8[ks], b[g].x, acc[g][0], 0, 0, 0);
          acc[g][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a8[ks], b[g].y, acc[g][1], 0, 0, 0);
          acc[g][2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a8[ks], b[g].z, acc[g][2], 0, 0, 0);
          acc[g][3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a8[ks], b[g].w, acc[g][3], 0, 0, 0);
          // the piece of the next reduction step replaces the one just used, NG - 1 groups ahead of its use
          if (ks + 1 < 8) b[g] = b_read(lb, ks + 1, g);
          // the next tile's copies, spread over this tile's steps
          if ((ks * NG + g) % 2 == 0 && (ks * NG + g) / 2 < NPIECES) stage_piece((ks * NG + g) / 2, src4, buf ^ 1);
          __builtin_amdgcn_sched_barrier(0);  // keeps the read where it is: NG - 1 groups of instructions ahead of its use
        }
      }
      a_cur[0] = a_nxt[0];
      a_cur[1] = a_nxt[1];
      hn = hn2;
      buf ^= 1;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
    // register v of acc[g][j] is row 16 w + 4 q + v, column 64 g + 4 c + j of the unit's block
    const int block = unit_block[u];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      float *prow = P + ((int64_t)block * kPanelRows + wave * 16 + 4 * q + v) * f;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int col = g * 64 + 4 * c16;
        if (col + 1 < f) *reinterpret_cast<float2 *>(prow + col) = make_float2(acc[g][0][v], acc[g][1][v]);
        if (col + 3 < f) *reinterpret_cast<float2 *>(prow + col + 2) = make_float2(acc[g][2][v], acc[g][3][v]);
      }
    }
  }
}

// Panels with several units: the blocks of the later units are added to the first one's, in unit order.
__global__ __launch_bounds__(kSpmmThreads) void panel_reduce_kernel(const int32_t *__restrict__ split, float *__restrict__ P,
                                                                    int32_t f, int32_t prows) {
  const int32_t first = split[2 * blockIdx.y], count = split[2 * blockIdx.y + 1];
  const int64_t block = (int64_t)prows * f;
  const int64_t idx = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (idx >= block) return;
  float *p = P + (int64_t)first * block + idx;
  float s = p[0];
  int32_t u = 1;
  for (; u + 4 <= count; u += 4) {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = p[(int64_t)(u + k) * block];
#pragma unroll
    for (int k = 0; k < 4; ++k) s += v[k];
  }
  for (; u < count; ++u) s += p[(int64_t)u * block];
  p[0] = s;
}

// C[r, :] = beta C[r, :] + the row's partial rows, one per block of its panel and added in block order, for a plan
// whose tiles hold every entry (the rest matrix is empty); f is even, a thread takes two columns; beta == 0 does
// not read C.  list: the rows to write (the rows of a panel whose only block is a staged unit's are in C already).
__global__ __launch_bounds__(kSpmmThreads) void panel_finish_kernel(float *__restrict__ C, int64_t ldc,
                                                                     const float *__restrict__ P,
                                                                     const int32_t *__restrict__ dslot,
                                                                     const int32_t *__restrict__ bcount,
                                                                     const int32_t *__restrict__ list, int32_t count,
                                                                     int32_t f, float beta, int32_t prows) {
  const int32_t half = f >> 1;
  const int64_t idx = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  const int64_t i = idx / half;
  if (i >= count) return;
  const int64_t r = list[i];
  const int32_t c = (int32_t)(idx - i * half) * 2;
  const int32_t d = dslot[r];
  float2 v = make_float2(0.f, 0.f);
  if (d >= 0) {
    const int32_t blocks = bcount[d / prows];
    const float *p = P + (int64_t)d * f + c;
    v = *reinterpret_cast<const float2 *>(p);
    for (int32_t k = 1; k < blocks; ++k) {
      const float2 w = *reinterpret_cast<const float2 *>(p + (int64_t)k * prows * f);
      v.x += w.x;
      v.y += w.y;
    }
  }
  float *out = C + r * ldc + c;
  if (beta != 0.f) {
    v.x += beta * out[0];
    v.y += beta * out[1];
  }
  out[0] = v.x;
  out[1] = v.y;
}

// The same for an odd f: a thread takes one column.
__global__ __launch_bounds__(kSpmmThreads) void panel_finish1_kernel(float *__restrict__ C, int64_t ldc,
                                                                      const float *__restrict__ P,
                                                                      const int32_t *__restrict__ dslot,
                                                                      const int32_t *__restrict__ bcount,
                                                                      const int32_t *__restrict__ list, int32_t count,
                                                                      int32_t f, float beta, int32_t prows) {
  const int64_t idx = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  const int64_t i = idx / f;
  if (i >= count) return;
  const int64_t r = list[i];
  const int32_t c = (int32_t)(idx - i * f);
  const int32_t d = dslot[r];
  float v = 0.f;
  if (d >= 0) {
    const int32_t blocks = bcount[d / prows];
    const float *p = P + (int64_t)d * f + c;
    v = p[0];
    for (int32_t k = 1; k < blocks; ++k) v += p[(int64_t)k * prows * f];
  }
  float *out = C + r * ldc + c;
  if (beta != 0.f) v += beta * out[0];
  out[0] = v;
}

// Entries in (panel, column) pairs that hold at least two entries: every thread walks a stretch of the pairs, a
// workgroup adds its threads' sums in LDS and makes one 64-bit integer add
__global__ __launch_bounds__(kSpmmThreads) void panel_pair_reuse_kernel(const uint32_t *__restrict__ pair_first, int64_t npairs,
                                                                        unsigned long long *__restrict__ reuse) {
  __shared__ unsigned long long part[kSpmmThreads / kWave];
  unsigned long long v = 0;
  for (int64_t p = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x; p < npairs; p += (int64_t)gridDim.x * kSpmmThreads) {
    const uint32_t len = pair_first[p + 1] - pair_first[p];
    v += len >= 2u ? len : 0u;
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) part[threadIdx.x / kWave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long t = 0;
    for (int w = 0; w < kSpmmThreads / kWave; ++w) t += part[w];
    if (t) atomicAdd(reuse, t);
  }
}

// -------------------------------------------------------------------------------------------------
// plan construction kernels
// -------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kSpmmThreads) void panel_degree_key_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                        int32_t maxdeg, int32_t *__restrict__ key,
                                                                        int32_t *__restrict__ id) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (r < n) {
    key[r] = maxdeg - (rowptr[r + 1] - rowptr[r]);  // ascending key = descending degree, ties by row (stable sort)
    id[r] = (int32_t)r;
  }
}

// count[column] = its entries in the whole matrix, added up pair by pair (a pair = the entries of one column in one
// panel, a run of the entries sorted by (panel, column): one atomic per pair instead of one per entry)
__global__ __launch_bounds__(kSpmmThreads) void panel_col_count_kernel(const uint32_t *__restrict__ pair_first, int64_t npairs,
                                                                       const int32_t *__restrict__ kcol_sorted,
                                                                       uint32_t *__restrict__ count) {
  const int64_t p = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (p >= npairs) return;
  const uint32_t first = pair_first[p];
  atomicAdd(&count[kcol_sorted[first]], pair_first[p + 1] - first);  // integer count: order independent
}

__global__ __launch_bounds__(kSpmmThreads) void panel_count_key_kernel(const uint32_t *__restrict__ count, int32_t m,
                                                                       uint32_t maxcount, int32_t *__restrict__ key,
                                                                       int32_t *__restrict__ id) {
  const int64_t j = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (j < m) {
    key[j] = (int32_t)(maxcount - count[j]);
    id[j] = (int32_t)j;
  }
}

// rank_of[ranked[k]] = k
__global__ __launch_bounds__(kSpmmThreads) void panel_invert_kernel(const int32_t *__restrict__ ranked, int32_t count,
                                                                    int32_t *__restrict__ rank_of) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k < count) rank_of[ranked[k]] = (int32_t)k;
}

// Tiles are numbered panel by panel: panel p has tbase[p + 1] - tbase[p] of them, one per 32 column ranks it uses
// (at most `hot` ranks).  Tile of an entry from its row rank and its column's rank in the row's panel, -1 for a
// column rank from `hot` on.
__device__ __forceinline__ int64_t panel_tile_of(int32_t rrank, int32_t crank, int32_t hot, const int32_t *__restrict__ tbase,
                                                 int32_t prows, int32_t tcols) {
  if (crank >= hot) return -1;
  return (int64_t)tbase[rrank / prows] + crank / tcols;
}

// blocks[p] = tiles of panel p = ceil(min(column ranks of the panel, hot) / 32); blocks[npanels] = 0 (slot of the scan's total)
__global__ __launch_bounds__(kSpmmThreads) void panel_tile_base_kernel(const int32_t *__restrict__ pstart, int32_t npanels,
                                                                       int32_t hot, int32_t tcols, uint32_t *__restrict__ blocks) {
  const int64_t p = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (p > npanels) return;
  uint32_t b = 0;
  if (p < npanels) {
    const int32_t ranks = pstart[p + 1] - pstart[p];
    b = (uint32_t)(((ranks < hot ? ranks : hot) + tcols - 1) / tcols);
  }
  blocks[p] = b;
}

// Tiles with emin .. dmin - 1 entries are staged ("active"), tiles with at least dmin entries are dense
// (dmin == 0: none).
__device__ __forceinline__ int panel_tile_kind(uint32_t count, uint32_t emin, uint32_t dmin) {
  if (dmin > 0 && count >= dmin) return 2;
  return count >= emin ? 1 : 0;
}

// Column ranks inside the panels.  The entries are sorted by (panel, column); a run of equal keys is a
// (panel, column) pair, and the pairs of a panel are ranked by descending length (ties: by column).
// Entries of rows behind the ranked panels get the panel number `npanels`, which sorts them last.
__global__ __launch_bounds__(kSpmmThreads) void panel_pair_key_kernel(const int32_t *__restrict__ erow,
                                                                      const int32_t *__restrict__ colind, int64_t nnz,
                                                                      const int32_t *__restrict__ row_rank, int32_t ranked_rows,
                                                                      int32_t npanels, int32_t prows, int32_t *__restrict__ kpanel,
                                                                      int32_t *__restrict__ kcol, int32_t *__restrict__ pos) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k >= nnz) return;
  const int32_t rr = row_rank[erow[k]];
  kpanel[k] = rr < ranked_rows ? rr / prows : npanels;
  kcol[k] = colind[k];
  pos[k] = (int32_t)k;
}

// sort keys of the pairs: (panel, 255 - min(entries, 255)), payload the pair's number; pair_col[pair] = its column.
// pair_first[npairs] = number of entries.
// With col_rank (the columns' ranks by entry count over the whole matrix) the minor key is that rank for the pairs
// with at least cmin entries and m + rank for the others: a panel's blocks then hold the columns that are worth
// staging in the same order in every panel, so that workgroups on different panels walk the rows of B alike.
__global__ __launch_bounds__(kSpmmThreads) void panel_pair_count_key_kernel(
    const uint32_t *__restrict__ pair_first, int64_t npairs, const int32_t *__restrict__ kpanel_sorted,
    const int32_t *__restrict__ kcol_sorted, const int32_t *__restrict__ col_rank, uint32_t cmin, int32_t m,
    int32_t *__restrict__ pk_panel, int32_t *__restrict__ pk_count, int32_t *__restrict__ pk_pair,
    int32_t *__restrict__ pair_col) {
  const int64_t p = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (p >= npairs) return;
  const uint32_t first = pair_first[p], count = pair_first[p + 1] - first;
  const int32_t col = kcol_sorted[first];
  pk_panel[p] = kpanel_sorted[first];
  pk_count[p] = col_rank ? col_rank[col] + (count >= cmin ? 0 : m) : 255 - (int32_t)(count < 255u ? count : 255u);
  pk_pair[p] = (int32_t)p;
  pair_col[p] = col;
}

// pair_lr[pair] = rank of the pair's column inside its panel, `hot` for ranks from `hot` on and for the rows
// behind the panels (hot = the ranks that can be part of a tile); the pair's entries are counted into its tile
// (integer counts: order independent)
__global__ __launch_bounds__(kSpmmThreads) void panel_pair_rank_kernel(const int32_t *__restrict__ spanel,
                                                                       const int32_t *__restrict__ spair, int64_t npairs,
                                                                       const int32_t *__restrict__ pstart, int32_t npanels,
                                                                       int32_t hot, int32_t tcols, const int32_t *__restrict__ tbase,
                                                                       const uint32_t *__restrict__ pair_first,
                                                                       int32_t *__restrict__ pair_lr,
                                                                       uint32_t *__restrict__ tcount) {
  const int64_t j = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (j >= npairs) return;
  const int32_t panel = spanel[j], pair = spair[j];
  int64_t lr = hot;
  if (panel < npanels) {
    lr = j - pstart[panel];
    if (lr >= hot)
      lr = hot;
    else
      atomicAdd(&tcount[(int64_t)tbase[panel] + lr / tcols], pair_first[pair + 1] - pair_first[pair]);
  }
  pair_lr[pair] = (int32_t)lr;
}

// ecr[entry] = rank of the entry's column inside the entry's panel (start / runs_before: the run starts of the
// sorted entries and their exclusive scan; pos_sorted: the entry at a sorted position)
__global__ __launch_bounds__(kSpmmThreads) void panel_entry_rank_kernel(const uint32_t *__restrict__ start,
                                                                        const uint32_t *__restrict__ runs_before,
                                                                        const int32_t *__restrict__ pos_sorted, int64_t nnz,
                                                                        const int32_t *__restrict__ pair_lr,
                                                                        int32_t *__restrict__ ecr) {
  const int64_t i = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (i >= nnz) return;
  ecr[pos_sorted[i]] = pair_lr[runs_before[i] + start[i] - 1u];
}

// The column of every place of the active and of the dense tiles, from the ranked pairs: place c of an active
// tile is staged by wave c % 16 as its row c / 16 (hdr[(tile * 16 + wave) * 4 + c / 16]), place c of a dense
// tile is dhdr[tile * 32 + c] (a header of an active tile has tcols / 16 + 2 ints: 4 for tiles of 32 columns).  Both arrays hold -1 beforehand; a panel's last block can have fewer than 32
// columns, and its empty places are then given the block's first column (panel_hdr_kernel,
// panel_dense_hdr_fill_kernel): no entry refers to them, a dense tile holds zeros there.
__global__ __launch_bounds__(kSpmmThreads) void panel_pair_hdr_kernel(
    const int32_t *__restrict__ spanel, const int32_t *__restrict__ spair, int64_t npairs, const int32_t *__restrict__ pstart,
    int32_t npanels, int32_t hot, const int32_t *__restrict__ tbase, const int32_t *__restrict__ pair_col,
    const uint32_t *__restrict__ tcount,
    const uint32_t *__restrict__ tindex, const uint32_t *__restrict__ dindex, uint32_t emin, uint32_t dmin, int32_t tcols,
    int32_t *__restrict__ hdr, int32_t *__restrict__ dhdr) {
  const int64_t j = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (j >= npairs) return;
  const int32_t panel = spanel[j];
  if (panel >= npanels) return;
  const int64_t lr = j - pstart[panel];
  if (lr >= hot) return;
  const int64_t t = (int64_t)tbase[panel] + lr / tcols;
  const int c = (int)(lr % tcols);
  const int kind = panel_tile_kind(tcount[t], emin, dmin);
  const int32_t col = pair_col[spair[j]];
  const int hs = tcols / kPanelWaves + 2;  // ints of a (tile, wave) header: its rows of B, then its record range
  if (kind == 1)
    hdr[((int64_t)tindex[t] * kPanelWaves + c % kPanelWaves) * hs + c / kPanelWaves] = col;
  else if (kind == 2)
    dhdr[(int64_t)dindex[t] * kPanelCols + c] = col;
}

__global__ __launch_bounds__(kSpmmThreads) void panel_dense_hdr_fill_kernel(int32_t *__restrict__ dhdr, int64_t ndtiles) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k >= ndtiles * kPanelCols || k % kPanelCols == 0) return;  // place 0 of a tile is always taken
  if (dhdr[k] < 0) dhdr[k] = dhdr[k / kPanelCols * kPanelCols];
}

// flag[t] = 1 and kept[t] = tcount[t] for active tiles, dflag / dkept the same for dense ones, else 0 (the four
// arrays are then scanned).

__global__ __launch_bounds__(kSpmmThreads) void panel_tile_select_kernel(const uint32_t *__restrict__ tcount, int64_t tiles,
                                                                         uint32_t emin, uint32_t dmin,
                                                                         uint32_t *__restrict__ flag, uint32_t *__restrict__ kept,
                                                                         uint32_t *__restrict__ dflag,
                                                                         uint32_t *__restrict__ dkept) {
  const int64_t t = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (t > tiles) return;
  const int kind = t < tiles ? panel_tile_kind(tcount[t], emin, dmin) : 0;  // entry `tiles` is the slot the scans leave their totals in
  flag[t] = kind == 1 ? 1u : 0u;
  kept[t] = kind == 1 ? tcount[t] : 0u;
  dflag[t] = kind == 2 ? 1u : 0u;
  dkept[t] = kind == 2 ? tcount[t] : 0u;
}

// panel (and block number inside it) of every tile of one kind (1: active, 2: dense), in the compacted numbering
__global__ __launch_bounds__(kSpmmThreads) void panel_tile_tables_kernel(const uint32_t *__restrict__ tcount,
                                                                         const uint32_t *__restrict__ tindex, int64_t tiles,
                                                                         uint32_t emin, uint32_t dmin, int kind,
                                                                         const int32_t *__restrict__ tbase, int32_t npanels,
                                                                         int32_t *__restrict__ tile_panel,
                                                                         int32_t *__restrict__ tile_kb) {
  const int64_t t = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (t >= tiles || panel_tile_kind(tcount[t], emin, dmin) != kind) return;
  int32_t lo = 0, hi = npanels;  // the panel with tbase[panel] <= t < tbase[panel + 1]
  while (hi - lo > 1) {
    const int32_t mid = lo + (hi - lo) / 2;
    if ((int64_t)tbase[mid] <= t)
      lo = mid;
    else
      hi = mid;
  }
  tile_panel[tindex[t]] = lo;
  if (tile_kb) tile_kb[tindex[t]] = (int32_t)(t - tbase[lo]);
}

// sort keys: entries of active tiles get (active tile * 16 + wave) as major and the slot as minor key, entries of
// no tile the sentinel `ntiles * 16`, which a stable sort leaves behind the first ones in their (row, col)
// order, and entries of dense tiles sentinel + 1: those are written into their place of the dense tile right
// here and take no further part.  Two entries of one (row, column) pair would land in the same place: the
// exchange finds the second one (unless one of them is +0, which changes nothing) and raises *collision,
// after which the caller builds the plan again without dense tiles.
__global__ __launch_bounds__(kSpmmThreads) void panel_entry_key_kernel(
    const int32_t *__restrict__ erow, const int32_t *__restrict__ ecr, const float *__restrict__ val, int64_t nnz,
    const int32_t *__restrict__ row_rank, int32_t hot, const int32_t *__restrict__ tbase,
    const uint32_t *__restrict__ tcount, const uint32_t *__restrict__ tindex, const uint32_t *__restrict__ dindex,
    uint32_t emin, uint32_t dmin, int32_t sentinel, int32_t prows, int32_t tcols, int32_t *__restrict__ key,
    int32_t *__restrict__ slot, int32_t *__restrict__ pos, uint32_t *__restrict__ dA_bits, uint32_t *__restrict__ collision) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k >= nnz) return;
  const int32_t rr = row_rank[erow[k]];
  const int32_t cr = ecr[k];
  const int64_t t = panel_tile_of(rr, cr, hot, tbase, prows, tcols);
  int32_t ky = sentinel, sl = 0;
  const int kind = t >= 0 ? panel_tile_kind(tcount[t], emin, dmin) : 0;
  if (kind == 1) {
    const int32_t p = rr % prows;
    ky = (int32_t)tindex[t] * kPanelWaves + p % kPanelWaves;
    sl = p / kPanelWaves;
  } else if (kind == 2) {
    const int32_t p = rr % kPanelRows, c = cr % kPanelCols;
    const int32_t w = p / 16, ks = c / 4, lane = (c % 4) * 16 + p % 16;
    const int64_t at = (((int64_t)dindex[t] * kDenseWaves + w) * 2 + ks / 4) * 256 + lane * 4 + ks % 4;
    const uint32_t old = atomicExch(&dA_bits[at], __float_as_uint(val[k]));  // integer exchange of the value's bits
    if (old != 0u) atomicOr(collision, 1u);
    ky = sentinel + 1;
  }
  key[k] = ky;
  slot[k] = sl;
  pos[k] = (int32_t)k;
}

// after the sort: records of the covered entries, and the arrays of the rest
__global__ __launch_bounds__(kSpmmThreads) void panel_entry_finish_kernel(
    const int32_t *__restrict__ slot_sorted, const int32_t *__restrict__ pos, int64_t count, int64_t covered,
    const int32_t *__restrict__ erow, const int32_t *__restrict__ colind, const float *__restrict__ val,
    const int32_t *__restrict__ ecr, int32_t tcols, uint2 *__restrict__ ent, int32_t *__restrict__ rest_row,
    int32_t *__restrict__ rest_col, float *__restrict__ rest_val) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k >= count) return;  // count = entries of active tiles + rest; the entries of dense tiles lie behind them
  const int32_t p = pos[k];
  if (k < covered) {
    ent[k] = make_uint2((uint32_t)(ecr[p] % tcols) | ((uint32_t)slot_sorted[k] << 8), __float_as_uint(val[p]));
  } else {
    rest_row[k - covered] = erow[p];
    rest_col[k - covered] = colind[p];
    rest_val[k - covered] = val[p];
  }
}

// Runs of records = maximal stretches of equal (key, slot) in the sorted order.  The product kernel takes the
// records of a run two at a time, so a run of odd length gets one more record behind its last one: the same
// column and slot with the value +0 (which adds nothing as long as that row of B is finite).
__global__ __launch_bounds__(kSpmmThreads) void panel_run_start_kernel(const int32_t *__restrict__ key,
                                                                        const int32_t *__restrict__ slot, int64_t count,
                                                                        uint32_t *__restrict__ start) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k > count) return;
  start[k] = k < count && (k == 0 || key[k] != key[k - 1] || slot[k] != slot[k - 1]) ? 1u : 0u;  // entry `count`: slot of the scan's total
}

// run_first[run] = first record of the run; runs_before[k] is the exclusive scan of start[]
__global__ __launch_bounds__(kSpmmThreads) void panel_run_first_kernel(const uint32_t *__restrict__ start,
                                                                        const uint32_t *__restrict__ runs_before,
                                                                        int64_t count, uint32_t *__restrict__ run_first) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k < count && start[k]) run_first[runs_before[k]] = (uint32_t)k;
}

// pad[k] = 1 when record k is the last of a run of odd length (entry `count` is the slot of the scan's total)
__global__ __launch_bounds__(kSpmmThreads) void panel_run_pad_kernel(const uint32_t *__restrict__ start,
                                                                      const uint32_t *__restrict__ runs_before,
                                                                      const uint32_t *__restrict__ run_first, int64_t count,
                                                                      uint32_t *__restrict__ pad) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k > count) return;
  uint32_t p = 0;
  if (k < count && (k + 1 == count || start[k + 1])) {
    const uint32_t run = runs_before[k] + start[k] - 1u;  // runs_before counts the starts ahead of k
    p = ((uint32_t)k - run_first[run] + 1u) & 1u;
  }
  pad[k] = p;
}

// shift[k] = exclusive scan of pad[]: record k moves to k + shift[k], its padding record (if any) behind it
__global__ __launch_bounds__(kSpmmThreads) void panel_pad_write_kernel(const uint2 *__restrict__ in,
                                                                        const uint32_t *__restrict__ pad,
                                                                        const uint32_t *__restrict__ shift, int64_t count,
                                                                        uint2 *__restrict__ out) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k >= count) return;
  const uint2 r = in[k];
  const int64_t at = k + shift[k];
  out[at] = r;
  if (pad[k]) out[at + 1] = make_uint2(r.x, 0u);
}

// flag[r] = 1 for the rows the pass over the partial rows writes: rows without a partial row (C = beta C) and rows
// of panels with several blocks or a dense one
__global__ __launch_bounds__(kSpmmThreads) void panel_finish_flag_kernel(const int32_t *__restrict__ dslot,
                                                                         const int32_t *__restrict__ bcount, int32_t rows,
                                                                         int32_t prows, uint32_t *__restrict__ flag) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (r > rows) return;
  uint32_t fl = 0;
  if (r < rows) {
    const int32_t d = dslot[r];
    fl = d < 0 || bcount[d / prows] >= 0 ? 1u : 0u;
  }
  flag[r] = fl;  // flag[rows] = 0: the place of the scan's total
}

__global__ __launch_bounds__(kSpmmThreads) void panel_finish_list_kernel(const uint32_t *__restrict__ flag,
                                                                         const uint32_t *__restrict__ pos, int32_t rows,
                                                                         int32_t *__restrict__ list) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (r < rows && flag[r]) list[pos[r]] = (int32_t)r;
}

// first[k] = wptr[16 k]: the first record of tile k (k = tiles: all records)
__global__ __launch_bounds__(kSpmmThreads) void panel_tile_first_kernel(const int32_t *__restrict__ wptr, int64_t count,
                                                                        int32_t *__restrict__ first) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k < count) first[k] = wptr[k * kPanelWaves];
}

// wptr[j] += shift[wptr[j]] (shift[count] = all padding records)
__global__ __launch_bounds__(kSpmmThreads) void panel_pad_wptr_kernel(int32_t *__restrict__ wptr, int64_t entries,
                                                                       const uint32_t *__restrict__ shift) {
  const int64_t j = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (j < entries) wptr[j] += (int32_t)shift[wptr[j]];
}

// hdr[(t * 16 + w) * hs ..] = {rows of B of places w, w + 16, ... of the tile, first record, end}, hs = tcols / 16 + 2:
// the rows are there already (panel_pair_hdr_kernel) except for empty places, which get the row of the tile's place 0
__global__ __launch_bounds__(kSpmmThreads) void panel_hdr_kernel(const int32_t *__restrict__ tile_wptr, int64_t ntiles,
                                                                  int32_t tcols, int32_t *__restrict__ hdr) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k >= ntiles * kPanelWaves) return;
  const int tcw = tcols / kPanelWaves, hs = tcw + 2;
  const int64_t t = k / kPanelWaves;
  const int32_t first = hdr[t * kPanelWaves * hs];  // place 0 of a tile is always taken, and nobody writes it here
  for (int j = 0; j < tcw; ++j)
    if ((j > 0 || k % kPanelWaves != 0) && hdr[k * hs + j] < 0) hdr[k * hs + j] = first;
  hdr[k * hs + tcw] = tile_wptr[k];
  hdr[k * hs + tcw + 1] = tile_wptr[k + 1];
}

__global__ __launch_bounds__(kSpmmThreads) void panel_dslot_kernel(const int32_t *__restrict__ row_rank, int32_t n,
                                                                   const int32_t *__restrict__ panel_unit, int32_t npanels,
                                                                   int32_t prows, int32_t *__restrict__ dslot) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (r >= n) return;
  const int32_t rr = row_rank[r];
  const int32_t panel = rr / prows;
  const int32_t u = panel < npanels ? panel_unit[panel] : -1;
  dslot[r] = u < 0 ? -1 : u * prows + rr % prows;
}

__global__ __launch_bounds__(kSpmmThreads) void panel_expand_rows_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                         int32_t *__restrict__ row_out) {
  const int64_t wave = ((int64_t)blockIdx.x * kSpmmThreads + threadIdx.x) / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (wave >= n) return;
  const int32_t s = rowptr[wave], e = rowptr[wave + 1];
  for (int32_t k = s + lane; k < e; k += kWave) row_out[k] = (int32_t)wave;
}

}  // namespace cg
