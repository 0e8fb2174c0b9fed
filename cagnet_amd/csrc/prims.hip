// Device-wide primitives written for 64-wide wavefronts: exclusive scan (reduce-then-scan over
// 2048-element tiles) and a stable LSD radix sort (digits of up to 8 bits, balanced over the
// passes; per-wave match ranking in LDS).
// Both are integer-only and order-preserving, so results are run-to-run identical.
#include "common.h"

namespace cg {

// ---------------------------------------------------------------------------------------------
// scan
// ---------------------------------------------------------------------------------------------
constexpr int kScanThreads = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanThreads * kScanItems;  // 2048

__device__ inline uint32_t wave_inclusive_scan(uint32_t v, int lane) {
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    uint32_t t = __shfl_up(v, d, kWave);
    if (lane >= d) v += t;
  }
  return v;
}

// Exclusive scan of one value per thread across a 256-thread block; *block_total gets the sum.
__device__ inline uint32_t block_exclusive_scan(uint32_t v, uint32_t *block_total) {
  __shared__ uint32_t wave_sum[kScanThreads / kWave];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  uint32_t incl = wave_inclusive_scan(v, lane);
  if (lane == kWave - 1) wave_sum[wave] = incl;
  __syncthreads();
  uint32_t offset = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kScanThreads / kWave; ++w) {
    uint32_t s = wave_sum[w];
    if (w < wave) offset += s;
    total += s;
  }
  __syncthreads();
  *block_total = total;
  return offset + incl - v;
}

__global__ __launch_bounds__(kScanThreads) void scan_tile_sums_kernel(const uint32_t *__restrict__ in,
                                                                      uint32_t *__restrict__ sums, int64_t count) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  uint32_t s = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    int64_t idx = base + i;
    if (idx < count) s += in[idx];
  }
  uint32_t total;
  (void)block_exclusive_scan(s, &total);
  if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// out[i] = offsets[tile] + exclusive prefix inside the tile.  in and out may alias: every thread
// reads all of its own items before it writes them.
__global__ __launch_bounds__(kScanThreads) void scan_tile_apply_kernel(const uint32_t *in, uint32_t *out,
                                                                       const uint32_t *__restrict__ offsets,
                                                                       int64_t count, uint32_t *total_out) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  uint32_t item[kScanItems];
  uint32_t s = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    int64_t idx = base + i;
    item[i] = idx < count ? in[idx] : 0u;
    s += item[i];
  }
  uint32_t total;
  uint32_t run = block_exclusive_scan(s, &total);
  run += offsets ? offsets[blockIdx.x] : 0u;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    int64_t idx = base + i;
    if (idx < count) out[idx] = run;
    run += item[i];
  }
  if (total_out && blockIdx.x == gridDim.x - 1 && threadIdx.x == kScanThreads - 1) *total_out = run;
}

static int scan_level(const uint32_t *d_in, uint32_t *d_out, int64_t count, uint32_t *d_total, uint32_t *d_sums,
                      hipStream_t stream) {
  const int64_t tiles = ceil_div64(count, kScanTile);
  if (tiles <= 1) {
    scan_tile_apply_kernel<<<1, kScanThreads, 0, stream>>>(d_in, d_out, nullptr, count, d_total);
    CG_LAUNCH_CHECK();
    return CG_OK;
  }
  scan_tile_sums_kernel<<<(unsigned)tiles, kScanThreads, 0, stream>>>(d_in, d_sums, count);
  CG_LAUNCH_CHECK();
  // the tile sums are scanned in place; the next level's sums live right behind them
  CG_TRY(scan_level(d_sums, d_sums, tiles, nullptr, d_sums + tiles, stream));
  scan_tile_apply_kernel<<<(unsigned)tiles, kScanThreads, 0, stream>>>(d_in, d_out, d_sums, count, d_total);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

int exclusive_scan_u32(const uint32_t *d_in, uint32_t *d_out, int64_t count, uint32_t *d_total, hipStream_t stream) {
  if (count < 0) CG_FAIL(CG_ERR_SIZE, "scan: negative count");
  if (count == 0) {
    if (d_total) CG_HIP(hipMemsetAsync(d_total, 0, sizeof(uint32_t), stream));
    return CG_OK;
  }
  if (ceil_div64(count, kScanTile) > 0x7fffffffLL) CG_FAIL(CG_ERR_OVERFLOW, "scan: too many tiles");
  size_t sums = 0;
  for (int64_t t = ceil_div64(count, kScanTile); t > 1; t = ceil_div64(t, kScanTile)) sums += (size_t)t;
  sums += 1;
  void *d_sums = nullptr;
  CG_TRY(scratch_get(stream, kSlotD, sums * sizeof(uint32_t), &d_sums));
  return scan_level(d_in, d_out, count, d_total, (uint32_t *)d_sums, stream);
}

// ---------------------------------------------------------------------------------------------
// radix sort
// ---------------------------------------------------------------------------------------------
constexpr int kSortThreads = 256;
constexpr int kSortWaves = kSortThreads / kWave;         // 4
constexpr int kSortRounds = 16;                          // keys per lane
constexpr int kSortWaveTile = kSortRounds * kWave;       // 1024 consecutive keys per wave
constexpr int kSortTile = kSortWaves * kSortWaveTile;    // 4096 keys per workgroup
constexpr int kRadix = 256;
constexpr int kXcds = 8;

// hist[digit * tiles + tile] = number of keys of this tile with that digit
__global__ __launch_bounds__(kSortThreads) void radix_hist_kernel(const int32_t *__restrict__ key, int64_t count,
                                                                  int shift, int dbits, uint32_t *__restrict__ hist,
                                                                  int64_t tiles) {
  __shared__ uint32_t lh[kRadix];
  lh[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kSortTile;
  // every load is issued before the first count (unconditional, clamped index: a load behind a branch
  // would make each of the 16 steps wait for its own round trip)
  uint32_t k[kSortTile / kSortThreads];
#pragma unroll
  for (int i = 0; i < kSortTile / kSortThreads; ++i) {
    const int64_t idx = base + (int64_t)i * kSortThreads + threadIdx.x;
    k[i] = (uint32_t)key[idx < count ? idx : count - 1];
  }
#pragma unroll
  for (int i = 0; i < kSortTile / kSortThreads; ++i) {
    const int64_t idx = base + (int64_t)i * kSortThreads + threadIdx.x;
    if (idx < count) atomicAdd(&lh[(k[i] >> shift) & ((1u << dbits) - 1u)], 1u);  // integer LDS atomic: order independent
  }
  __syncthreads();
  if ((int)threadIdx.x < (1 << dbits)) hist[(int64_t)threadIdx.x * tiles + blockIdx.x] = lh[threadIdx.x];
}

// Stable scatter.  Wave w of a workgroup owns keys [tile + 1024 w, tile + 1024 (w+1)) and ranks
// them 64 at a time: lanes holding equal digits find each other with 8 ballots, their rank is the
// number of lower lanes in that peer set plus the wave's running count of the digit.  The records
// are then ordered by digit inside LDS and written out from there, so that the records of one
// digit leave as one contiguous run instead of one 4-byte store each.
// in_p == nullptr: the payload of a record is its position in the input.  Outputs that are nullptr
// are not written.
__global__ __launch_bounds__(kSortThreads) void radix_scatter_kernel(
    int key_is_a, int shift, int dbits, const int32_t *__restrict__ in_a, const int32_t *__restrict__ in_b,
    const int32_t *__restrict__ in_p, int32_t *__restrict__ out_a, int32_t *__restrict__ out_b,
    int32_t *__restrict__ out_p, int64_t count, const uint32_t *__restrict__ scanned_hist, int64_t tiles) {
  __shared__ uint32_t cnt[kSortWaves][kRadix];
  __shared__ uint32_t goff[kRadix];        // global position of a record = goff[digit] + its position in the tile
  __shared__ uint32_t wave_total[kSortWaves];
  __shared__ int32_t sa[kSortTile], sb[kSortTile], sp[kSortTile];
  for (int i = threadIdx.x; i < kSortWaves * kRadix; i += kSortThreads) (&cnt[0][0])[i] = 0;
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint64_t lt_mask = (1ull << lane) - 1ull;
  const int64_t per_xcd = (tiles + kXcds - 1) / kXcds;
  const int64_t tile = (int64_t)(blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
  if (tile >= tiles) return;  // whole workgroup
  const int64_t tile_base = tile * kSortTile;
  const int64_t base = tile_base + (int64_t)wave * kSortWaveTile;
  const uint32_t dmask = (1u << dbits) - 1u;

  int32_t ra[kSortRounds], rb[kSortRounds], rp[kSortRounds];
  uint32_t packed[kSortRounds];  // digit | rank among the wave's records of that digit << 8

  // All loads of the tile are issued before the first record is ranked: keys first, payload last.
  // They are unconditional (index clamped to the last record, dead lanes are masked where the value
  // is used), because a load behind a branch makes the compiler wait for all outstanding loads and
  // each of the 16 rounds would then pay a full memory round trip.
  const int64_t last = count - 1;
  const int32_t *__restrict__ src_p = in_p ? in_p : in_a;  // no payload array: the position is the payload
#pragma unroll
  for (int r = 0; r < kSortRounds; ++r) {
    const int64_t idx = base + (int64_t)r * kWave + lane;
    const int64_t cidx = idx < last ? idx : last;
    ra[r] = in_a[cidx];
    rb[r] = in_b[cidx];
  }
#pragma unroll
  for (int r = 0; r < kSortRounds; ++r) {
    const int64_t idx = base + (int64_t)r * kWave + lane;
    const int64_t cidx = idx < last ? idx : last;
    const int32_t v = src_p[cidx];
    rp[r] = in_p ? v : (int32_t)idx;
  }
  __builtin_amdgcn_sched_barrier(0);

#pragma unroll
  for (int r = 0; r < kSortRounds; ++r) {
    const int64_t idx = base + (int64_t)r * kWave + lane;
    const bool valid = idx < count;
    uint32_t d = 0;
    if (valid) d = ((uint32_t)(key_is_a ? ra[r] : rb[r]) >> shift) & dmask;
    uint64_t peers = __ballot(valid);
#pragma unroll
    for (int bit = 0; bit < 8; ++bit) {
      if (bit < dbits) {  // wave-uniform
        const bool one = (d >> bit) & 1u;
        const uint64_t bal = __ballot(one);
        peers &= one ? bal : ~bal;
      }
    }
    const uint32_t rank = (uint32_t)__popcll(peers & lt_mask);
    uint32_t pre = 0;
    if (valid) pre = cnt[wave][d];
    // the peer set's lowest lane publishes the new running count; its value depends on `pre`, so
    // the LDS read above completes before this write issues, and LDS serves a wave in order
    if (valid && rank == 0) cnt[wave][d] = pre + (uint32_t)__popcll(peers);
    packed[r] = d | ((pre + rank) << 8);
  }
  __syncthreads();

  {  // thread t owns digit t: exclusive scan of the tile's digit counts, then per-wave offsets
    const int t = threadIdx.x;
    uint32_t c[kSortWaves], total = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
      c[w] = cnt[w][t];
      total += c[w];
    }
    uint32_t inc = total;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const uint32_t up = __shfl_up(inc, off, kWave);
      if (lane >= off) inc += up;
    }
    if (lane == kWave - 1) wave_total[wave] = inc;
    __syncthreads();
    uint32_t excl = inc - total;
    for (int w = 0; w < wave; ++w) excl += wave_total[w];
    // modulo 2^32, undone by the addition below; digits beyond the pass's range have no records
    goff[t] = t <= (int)dmask ? scanned_hist[(int64_t)t * tiles + tile] - excl : 0u;
    uint32_t run = excl;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
      cnt[w][t] = run;
      run += c[w];
    }
  }
  __syncthreads();

#pragma unroll
  for (int r = 0; r < kSortRounds; ++r) {
    const int64_t idx = base + (int64_t)r * kWave + lane;
    if (idx < count) {
      const uint32_t d = packed[r] & (kRadix - 1);
      const uint32_t lpos = cnt[wave][d] + (packed[r] >> 8);
      sa[lpos] = ra[r];
      sb[lpos] = rb[r];
      sp[lpos] = rp[r];
    }
  }
  __syncthreads();

  const int64_t left = count - tile_base;
  const int32_t here = (int32_t)(left < kSortTile ? left : kSortTile);
  for (int32_t i = threadIdx.x; i < here; i += kSortThreads) {
    const int32_t va = sa[i], vb = sb[i];
    const uint32_t d = ((uint32_t)(key_is_a ? va : vb) >> shift) & dmask;
    const uint32_t pos = goff[d] + (uint32_t)i;
    if (out_a) out_a[pos] = va;
    if (out_b) out_b[pos] = vb;
    if (out_p) out_p[pos] = sp[i];
  }
}

struct SortPass {
  int which, shift, dbits;  // which 0: digit of key_b (minor key), 1: of key_a (major key)
};

// Balanced digits: the fewest 8-bit passes, each as narrow as that allows (18 bits: 3 x 6), so the
// records of one digit leave a tile as longer runs.
static int plan_passes(int bits_a, int bits_b, SortPass out[16]) {
  int count = 0;
  for (int which = 0; which < 2; ++which) {
    const int bits = which == 0 ? bits_b : bits_a;
    if (bits <= 0) continue;
    const int passes = (bits + 7) / 8;
    const int dbits = (bits + passes - 1) / passes;
    for (int shift = 0; shift < bits; shift += dbits) out[count++] = SortPass{which, shift, dbits};
  }
  return count;
}

static int sort_pass(const SortPass &ps, const int32_t *in_a, const int32_t *in_b, const int32_t *in_p, int32_t *out_a,
                     int32_t *out_b, int32_t *out_p, int64_t count, uint32_t *hist, int64_t tiles, hipStream_t stream) {
  radix_hist_kernel<<<(unsigned)tiles, kSortThreads, 0, stream>>>(ps.which == 0 ? in_b : in_a, count, ps.shift, ps.dbits,
                                                                  hist, tiles);
  CG_LAUNCH_CHECK();
  CG_TRY(exclusive_scan_u32(hist, hist, tiles << ps.dbits, nullptr, stream));
  const int64_t grid = (tiles + kXcds - 1) / kXcds * kXcds;
  radix_scatter_kernel<<<(unsigned)grid, kSortThreads, 0, stream>>>(ps.which, ps.shift, ps.dbits, in_a, in_b, in_p, out_a,
                                                                     out_b, out_p, count, hist, tiles);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

static int sort_hist(int64_t count, uint32_t **hist, int64_t *tiles, hipStream_t stream) {
  if (count > 0x7fffffffLL) CG_FAIL(CG_ERR_OVERFLOW, "radix sort: count %lld >= 2^31", (long long)count);
  *tiles = ceil_div64(count, kSortTile);
  void *d_hist = nullptr;
  CG_TRY(scratch_get(stream, kSlotC, (size_t)*tiles * kRadix * sizeof(uint32_t), &d_hist));
  *hist = (uint32_t *)d_hist;
  return CG_OK;
}

int radix_sort_pairs(SortBuffers &buf, int64_t count, int bits_a, int bits_b, int *result_set, hipStream_t stream) {
  int cur = 0;
  *result_set = 0;
  if (count <= 1) return CG_OK;
  uint32_t *hist = nullptr;
  int64_t tiles = 0;
  CG_TRY(sort_hist(count, &hist, &tiles, stream));
  SortPass passes[16];
  const int np = plan_passes(bits_a, bits_b, passes);
  for (int i = 0; i < np; ++i) {
    CG_TRY(sort_pass(passes[i], buf.key_a[cur], buf.key_b[cur], buf.payload[cur], buf.key_a[cur ^ 1], buf.key_b[cur ^ 1],
                     buf.payload[cur ^ 1], count, hist, tiles, stream));
    cur ^= 1;
  }
  *result_set = cur;
  return CG_OK;
}

int radix_sort_records(const SortIo &io, SortBuffers &tmp, int64_t count, int bits_a, int bits_b, hipStream_t stream) {
  if (count <= 0) return CG_OK;
  uint32_t *hist = nullptr;
  int64_t tiles = 0;
  CG_TRY(sort_hist(count, &hist, &tiles, stream));
  SortPass passes[16];
  int np = plan_passes(bits_a, bits_b, passes);
  if (np == 0) passes[np++] = SortPass{1, 0, 0};  // nothing to sort on: one pass with a single digit copies the records
  if (np == 1) {
    // a single pass would write the outputs while other tiles still read the inputs: when they overlap,
    // a copying pass through `tmp` comes first
    const size_t bytes = (size_t)count * sizeof(int32_t);
    const int32_t *ins[3] = {io.in_a, io.in_b, io.in_p};
    const int32_t *outs[3] = {io.out_a, io.out_b, io.payload ? io.out_p : nullptr};
    bool overlap = false;
    for (const int32_t *i : ins)
      for (const int32_t *o : outs)
        if (i && o && (const char *)i < (const char *)o + bytes && (const char *)o < (const char *)i + bytes) overlap = true;
    if (overlap) {
      passes[1] = passes[0];
      passes[0] = SortPass{1, 0, 0};
      np = 2;
    }
  }
  for (int i = 0; i < np; ++i) {
    const bool first = i == 0, last = i == np - 1;
    const int from = (i - 1) & 1, to = i & 1;
    const int32_t *in_a = first ? io.in_a : tmp.key_a[from];
    const int32_t *in_b = first ? io.in_b : tmp.key_b[from];
    const int32_t *in_p = first ? io.in_p : (io.payload ? tmp.payload[from] : nullptr);
    int32_t *out_a = last ? io.out_a : tmp.key_a[to];
    int32_t *out_b = last ? io.out_b : tmp.key_b[to];
    int32_t *out_p = !io.payload ? nullptr : (last ? io.out_p : tmp.payload[to]);
    CG_TRY(sort_pass(passes[i], in_a, in_b, in_p, out_a, out_b, out_p, count, hist, tiles, stream));
  }
  return CG_OK;
}

}  // namespace cg
