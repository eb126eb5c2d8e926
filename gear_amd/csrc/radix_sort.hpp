// Stable least-significant-digit radix sort (8-bit digits) for key/value pairs, gfx950.
//
// Per digit every tile re-reads its keys, ranks them in LDS (wave ballots give the rank among equal
// digits inside a wave, a small LDS table the rank across the waves of the tile) and scatters keys
// and payloads to their final place for this digit.  Ranks follow element order, so the sort is
// stable.  Where a key lands depends on a table of (tile, digit) counts:
//  * up to kFusedTiles tiles (the candidate lists of top-k, index batches): two launches per digit.
//    A count launch fills a tile-major table; every scatter workgroup sums the counts of the tiles
//    before it and scans the digit totals itself.  (Counting the next digit from inside the
//    scatter launch with global atomics, one launch per digit, was measured too: 65 536 atomics
//    cost 6.9 us per digit, the count launch 4.6 us.)
//  * more tiles: count launch, one workgroup per digit scans its row of the digit-major table,
//    scatter launch.
#pragma once
#include "wave.hpp"

namespace gearhip {
namespace radix {
namespace {  // every translation unit gets its own copy of the kernels

constexpr int kBlock = 256;
constexpr int kBins = 256;
constexpr int kWaves = kBlock / kWave;
constexpr int kFusedTiles = 128;

struct Plan {
  int rounds;      // elements per thread and tile
  int64_t ntiles;  // tiles of kBlock * rounds elements
  bool fused;      // the scatter workgroups sum the count table themselves
};

inline Plan plan(int64_t num) {
  Plan p;
  int64_t r = ceil_div64(num, (int64_t)kBlock * 1024);
  if (r < 4) r = 4;
  if (r > 64) r = 64;
  p.rounds = (int)r;
  p.ntiles = num <= 0 ? 0 : ceil_div64(num, (int64_t)kBlock * r);
  p.fused = p.ntiles <= kFusedTiles;
  return p;
}

inline size_t table_bytes(const Plan &p) { return (size_t)p.ntiles * kBins * sizeof(uint32_t); }

// digit totals (1 KiB) followed by the count table
inline size_t hist_bytes(int64_t num) {
  const Plan p = plan(num);
  return align_up(kBins * sizeof(uint32_t) + table_bytes(p) + 256, 256);
}

// Counts the digit of every key of a tile.  TILE_MAJOR: hist[tile][digit], else hist[digit][tile].
template <typename K, bool TILE_MAJOR>
__global__ __launch_bounds__(kBlock) void hist_kernel(const K *__restrict__ keys, int64_t num,
                                                      int shift, uint32_t dmask, int rounds,
                                                      int64_t ntiles, uint32_t *__restrict__ hist) {
  __shared__ uint32_t h[kBins];
  const int tid = threadIdx.x;
  h[tid] = 0;
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * kBlock * rounds;
  for (int r0 = 0; r0 < rounds; r0 += 4) {  // four loads in flight before the first LDS atomic
    K k[4];
    bool ok[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int64_t i = base + (int64_t)(r0 + q) * kBlock + tid;
      ok[q] = r0 + q < rounds && i < num;
      k[q] = ok[q] ? keys[i] : (K)0;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (ok[q]) atomicAdd(&h[(uint32_t)(k[q] >> shift) & dmask], 1u);
  }
  __syncthreads();
  if (TILE_MAJOR) {
    hist[(int64_t)blockIdx.x * kBins + tid] = h[tid];
  } else {
    hist[(int64_t)tid * ntiles + blockIdx.x] = h[tid];
  }
}

// Workgroup d turns row d of the digit-major table into exclusive prefixes over the tiles and
// records the row's total.
__global__ __launch_bounds__(kBlock) void digit_scan_kernel(uint32_t *__restrict__ table,
                                                            int64_t ntiles,
                                                            uint32_t *__restrict__ totals) {
  __shared__ uint32_t wsum[kWaves];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t *row = table + (int64_t)blockIdx.x * ntiles;
  uint32_t carry = 0;
  for (int64_t base = 0; base < ntiles; base += kBlock) {
    const int64_t i = base + tid;
    const int v = i < ntiles ? (int)row[i] : 0;
    const int inc = wave_inclusive_sum(v);
    if (lane == 63) wsum[wave] = (uint32_t)inc;
    __syncthreads();
    uint32_t before = carry, total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      if (w < wave) before += wsum[w];
      total += wsum[w];
    }
    if (i < ntiles) row[i] = before + (uint32_t)(inc - v);
    carry += total;
    __syncthreads();
  }
  if (tid == 0) totals[blockIdx.x] = carry;
}

// FUSED: `table` holds this digit's raw tile-major counts.  Otherwise `table` holds the
// digit-major row prefixes and `totals` the digit totals.
// What the LAST digit's scatter does with a sorted pair instead of storing it to kout/vout: a
// caller may pass its own functor (kActive = true, operator()(position, key, value)) to fuse the
// kernel that would otherwise read the sorted arrays once more.
struct StoreSorted {
  static constexpr bool kActive = false;
  template <typename K, typename V>
  __device__ __forceinline__ void operator()(uint32_t, K, V) const {}
};

template <typename K, typename V, bool HAS_V, bool FUSED, typename Final>
__global__ __launch_bounds__(kBlock) void scatter_kernel(
    const K *__restrict__ kin, const V *__restrict__ vin, K *__restrict__ kout,
    V *__restrict__ vout, int64_t num, int shift, uint32_t dmask, int rounds, int64_t ntiles,
    const uint32_t *__restrict__ table, const uint32_t *__restrict__ totals, Final fin,
    int last) {
  constexpr int kSub = 4;                  // rounds ranked together: independent ballot chains
  constexpr int kSlots = kSub * kWaves;    // (round, wave) slots of the count table
  __shared__ uint32_t base[kBins];
  __shared__ uint32_t wcnt[kSlots][kBins];  // keys of digit d seen by slot s (kept zero between uses)
  __shared__ uint32_t wpre[kSlots][kBins];  // where slot s starts writing digit d
  __shared__ uint32_t wsum[kWaves];
  __shared__ uint32_t part[FUSED ? kWaves : 1][2][kBins];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t tile = blockIdx.x;
  // keys of the first rounds are loaded before the offsets are worked out
  const int64_t tile0 = tile * kBlock * rounds;
  K key[kSub];
  V val[kSub];
  auto load_rounds = [&](int r0) {
#pragma unroll
    for (int q = 0; q < kSub; ++q) {
      const int64_t i = tile0 + (int64_t)(r0 + q) * kBlock + tid;
      const bool ok = r0 + q < rounds && i < num;
      key[q] = ok ? kin[i] : (K)0;
      val[q] = V();
      if (HAS_V && ok) val[q] = vin[i];
    }
  };
  load_rounds(0);
  {
    uint32_t before = 0, total = 0;  // of digit tid: in the tiles before this one, in all tiles
    if (FUSED) {
      // lane q of wave g sums digits 4q..4q+3 over the tiles g, g + 4, g + 8, ...: sixteen
      // 16-byte loads in flight per lane; the four waves' parts meet in LDS
      uint32_t bef[4] = {0u, 0u, 0u, 0u}, tot[4] = {0u, 0u, 0u, 0u};
      for (int64_t t0 = wave; t0 < ntiles; t0 += kWaves * 16) {
        u32x4 c[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int64_t t = t0 + (int64_t)j * kWaves;
          c[j] = u32x4{0u, 0u, 0u, 0u};
          if (t < ntiles) c[j] = *reinterpret_cast<const u32x4 *>(table + t * kBins + 4 * lane);
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const bool earlier = t0 + (int64_t)j * kWaves < tile;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            tot[i] += c[j][i];
            if (earlier) bef[i] += c[j][i];
          }
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        part[wave][0][4 * lane + i] = bef[i];
        part[wave][1][4 * lane + i] = tot[i];
      }
      __syncthreads();
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        before += part[w][0][tid];
        total += part[w][1][tid];
      }
    } else {
      before = table[(int64_t)tid * ntiles + tile];
      total = totals[tid];
    }
    const int inc = wave_inclusive_sum((int)total);
    if (lane == 63) wsum[wave] = (uint32_t)inc;
#pragma unroll
    for (int w = 0; w < kSlots; ++w) wcnt[w][tid] = 0;
    __syncthreads();
    uint32_t lower = (uint32_t)inc - total;  // keys with a smaller digit
    for (int w = 0; w < wave; ++w) lower += wsum[w];
    base[tid] = lower + before;
  }
  __syncthreads();
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  for (int r0 = 0; r0 < rounds; r0 += kSub) {
    bool valid[kSub];
    uint32_t d[kSub];
    int rank[kSub];
#pragma unroll
    for (int q = 0; q < kSub; ++q) {
      const int64_t i = tile0 + (int64_t)(r0 + q) * kBlock + tid;
      valid[q] = r0 + q < rounds && i < num;
      d[q] = (uint32_t)(key[q] >> shift) & dmask;
      uint64_t peers = wave_ballot(valid[q]);
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const bool bit = (d[q] >> b) & 1u;
        const uint64_t bal = wave_ballot(bit);
        peers &= bit ? bal : ~bal;
      }
      rank[q] = __popcll(peers & lt_mask);
      if (valid[q] && rank[q] == 0) wcnt[q * kWaves + wave][d[q]] = (uint32_t)__popcll(peers);
    }
    __syncthreads();
    {
      // thread tid owns digit tid: running start over the slots in element order; the counts
      // are cleared for the next use on the way
      uint32_t run = base[tid];
#pragma unroll
      for (int sl = 0; sl < kSlots; ++sl) {
        const uint32_t c = wcnt[sl][tid];
        wcnt[sl][tid] = 0;
        wpre[sl][tid] = run;
        run += c;
      }
      base[tid] = run;
    }
    __syncthreads();
    K kcur[kSub];
    V vcur[kSub];
#pragma unroll
    for (int q = 0; q < kSub; ++q) {
      kcur[q] = key[q];
      vcur[q] = val[q];
    }
    if (r0 + kSub < rounds) load_rounds(r0 + kSub);  // in flight during the scatter
#pragma unroll
    for (int q = 0; q < kSub; ++q) {
      if (valid[q]) {
        const uint32_t pos = wpre[q * kWaves + wave][d[q]] + (uint32_t)rank[q];
        if (Final::kActive && last) {
          fin(pos, kcur[q], vcur[q]);
        } else {
          kout[pos] = kcur[q];
          if (HAS_V) vout[pos] = vcur[q];
        }
      }
    }
    // the next use of wpre is ordered behind this scatter by the barrier after the next ballots
  }
}

// ---- ranking sort for small batches (a sampled batch of indices, a batch of updates) ----------
// Every workgroup keeps ALL keys of the batch (at most kRankMax) in LDS and ranks 64 of them:
// rank(e) = number of smaller keys + equal keys at smaller positions, the position of e after a
// stable sort.  The sixteen waves of a workgroup each count over a sixteenth of the keys (a lone
// wave per SIMD issues a dependent instruction only every ~8 clocks, so the CU wants several); a key
// read from LDS is broadcast to the 64 lanes and costs a compare and an add per lane.  num / 64
// workgroups run side by side: O(num^2) compares spread over that many CUs beat a one-workgroup
// LDS radix sort, which is bound by the instruction issue of its single CU (2048 20-bit keys:
// 13.8 us, against 6.7 us for the ranking sort).
constexpr int kRankBlock = 1024;
constexpr int kRankWaves = kRankBlock / kWave;
constexpr int kRankMax = 4096;

template <typename C>
struct RankSmem {
  C keys[kRankMax];
  uint32_t part[kRankWaves][kWave];
};

// All threads of the workgroup call this.  load(j) gives the compare key of element j < num.
// Returns the rank of element e = blockIdx.x * 64 + lane (meaningless for e >= num); *mine_out is
// that element's compare key.
template <typename C, typename Load>
__device__ __forceinline__ uint32_t block_rank(RankSmem<C> &sm, int num, Load load, C *mine_out) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // wave shares are multiples of 16 keys; the padding keys are larger than or equal to any key
  // and sit behind every real position, so they are never counted
  const int padded = (num + 16 * kRankWaves - 1) & ~(16 * kRankWaves - 1);
  {
    // all of a thread's loads are issued before the first LDS write (one memory round trip)
    constexpr int kPerThread = kRankMax / kRankBlock;
    C mykeys[kPerThread];
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int j = tid + i * kRankBlock;
      mykeys[i] = j < num ? load(j) : (C) ~(C)0;
    }
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int j = tid + i * kRankBlock;
      if (j < padded) sm.keys[j] = mykeys[i];
    }
  }
  __syncthreads();
  const int e0 = (int)blockIdx.x * kWave, e = e0 + lane;
  const C mine = sm.keys[e < num ? e : 0];
  const int share = padded / kRankWaves;
  const int jb = wave * share, je = jb + share;
  uint32_t c = 0;
  // three stretches with a uniform rule each, sixteen keys (four LDS reads in flight) per step
  const int before_end = je < e0 ? je : (e0 > jb ? e0 : jb);
  for (int j = jb; j < before_end; j += 16) {  // positions before this workgroup's keys
    C k[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) k[i] = sm.keys[j + i];
#pragma unroll
    for (int i = 0; i < 16; ++i) c += k[i] <= mine;  // equal keys at smaller positions rank first
  }
  const int in_begin = jb > e0 ? jb : e0, in_end = je < e0 + kWave ? je : e0 + kWave;
  for (int j = in_begin; j < in_end; j += 16) {
    C k[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) k[i] = sm.keys[j + i];
#pragma unroll
    for (int i = 0; i < 16; ++i) c += (k[i] < mine) || (k[i] == mine && j + i < e);
  }
  const int after_begin = jb > e0 + kWave ? jb : (e0 + kWave < je ? e0 + kWave : je);
  for (int j = after_begin; j < je; j += 16) {
    C k[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) k[i] = sm.keys[j + i];
#pragma unroll
    for (int i = 0; i < 16; ++i) c += k[i] < mine;
  }
  sm.part[wave][lane] = c;
  __syncthreads();
  uint32_t rank = 0;
#pragma unroll
  for (int w = 0; w < kRankWaves; ++w) rank += sm.part[w][lane];
  *mine_out = mine;
  return rank;
}

// Stable sort of bits [begin_bit, end_bit) of num <= kRankMax keys (and payloads): grid = num / 64
// workgroups.  C is the compare type: uint32_t where end_bit - begin_bit <= 32.  A padding key
// equal to the largest real key is harmless because it sits behind every real position.
template <typename K, typename V, typename C, bool HAS_V>
__global__ __launch_bounds__(kRankBlock) void rank_sort_kernel(const K *__restrict__ kin,
                                                               K *__restrict__ kout,
                                                               const V *__restrict__ vin,
                                                               V *__restrict__ vout, int num,
                                                               int begin_bit, int end_bit) {
  __shared__ RankSmem<C> sm;
  const int width = end_bit - begin_bit;
  const K mask = width >= (int)(8 * sizeof(K)) ? (K) ~(K)0 : (K)(((K)1 << width) - 1);
  C mine;
  const uint32_t rank =
      block_rank<C>(sm, num, [&](int j) { return (C)((kin[j] >> begin_bit) & mask); }, &mine);
  const int e = (int)blockIdx.x * kWave + (threadIdx.x & 63);
  if (threadIdx.x >= kWave || e >= num) return;
  kout[rank] = kin[e];
  if (HAS_V) vout[rank] = vin[e];
}

template <typename T>
__global__ void copy_kernel(const T *__restrict__ in, T *__restrict__ out, int64_t num) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < num) out[i] = in[i];
}

// Sorts bits [begin_bit, end_bit) of the keys ascending, stable.  kin/vin are not modified; the
// result lands in kout/vout; ktmp/vtmp are scratch of the same size; hist has hist_bytes(num).
// vin == nullptr sorts keys only.  num < 2^32.
// `fin` (see StoreSorted) replaces the stores of the last digit on the radix path; batches of at
// most kRankMax keys take the ranking sort, which ignores it (the caller checks num).
template <typename K, typename V, typename Final = StoreSorted>
int sort_pairs(const K *kin, K *kout, const V *vin, V *vout, K *ktmp, V *vtmp, int64_t num,
               int begin_bit, int end_bit, uint32_t *hist, hipStream_t st, Final fin = Final()) {
  if (num <= 0) return 0;
  if (num >= (1ll << 32)) return GEAR_HIP_ERANGE;
  const Plan p = plan(num);
  const int passes = end_bit > begin_bit ? (end_bit - begin_bit + 7) / 8 : 0;
  const bool has_v = vin != nullptr;
  if (num <= kRankMax && passes > 0) {
    const dim3 grid((unsigned)ceil_div64(num, kWave)), block(kRankBlock);
    const bool narrow = end_bit - begin_bit <= 32;
#define GEARHIP_RANK_SORT(C, HV) \
  rank_sort_kernel<K, V, C, HV><<<grid, block, 0, st>>>(kin, kout, vin, vout, (int)num, begin_bit, end_bit)
    if (narrow) {
      if (has_v) GEARHIP_RANK_SORT(uint32_t, true); else GEARHIP_RANK_SORT(uint32_t, false);
    } else {
      if (has_v) GEARHIP_RANK_SORT(K, true); else GEARHIP_RANK_SORT(K, false);
    }
#undef GEARHIP_RANK_SORT
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  if (passes == 0) {
    const unsigned g = (unsigned)ceil_div64(num, 256);
    copy_kernel<K><<<dim3(g), dim3(256), 0, st>>>(kin, kout, num);
    if (has_v) copy_kernel<V><<<dim3(g), dim3(256), 0, st>>>(vin, vout, num);
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  const K *ksrc = kin;
  const V *vsrc = vin;
  bool to_out = (passes & 1) != 0;  // alternate so that the last pass writes kout/vout
  uint32_t *totals = hist;
  uint32_t *table = hist + kBins;
  const dim3 grid((unsigned)p.ntiles), block(kBlock);
  for (int pass = 0; pass < passes; ++pass) {
    const int shift = begin_bit + 8 * pass;
    const uint32_t dmask = end_bit - shift >= 8 ? 255u : ((1u << (end_bit - shift)) - 1u);
    K *kdst = to_out ? kout : ktmp;
    V *vdst = to_out ? vout : vtmp;
    const int last = pass + 1 == passes ? 1 : 0;
    if (p.fused) {
      hist_kernel<K, true><<<grid, block, 0, st>>>(ksrc, num, shift, dmask, p.rounds, p.ntiles,
                                                   table);
      if (has_v)
        scatter_kernel<K, V, true, true, Final><<<grid, block, 0, st>>>(
            ksrc, vsrc, kdst, vdst, num, shift, dmask, p.rounds, p.ntiles, table, nullptr, fin,
            last);
      else
        scatter_kernel<K, V, false, true, Final><<<grid, block, 0, st>>>(
            ksrc, vsrc, kdst, vdst, num, shift, dmask, p.rounds, p.ntiles, table, nullptr, fin,
            last);
    } else {
      hist_kernel<K, false><<<grid, block, 0, st>>>(ksrc, num, shift, dmask, p.rounds, p.ntiles,
                                                    table);
      digit_scan_kernel<<<dim3(kBins), block, 0, st>>>(table, p.ntiles, totals);
      if (has_v)
        scatter_kernel<K, V, true, false, Final><<<grid, block, 0, st>>>(
            ksrc, vsrc, kdst, vdst, num, shift, dmask, p.rounds, p.ntiles, table, totals, fin,
            last);
      else
        scatter_kernel<K, V, false, false, Final><<<grid, block, 0, st>>>(
            ksrc, vsrc, kdst, vdst, num, shift, dmask, p.rounds, p.ntiles, table, totals, fin,
            last);
    }
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
    ksrc = kdst;
    vsrc = vdst;
    to_out = !to_out;
  }
  return 0;
}

}  // namespace
}  // namespace radix
}  // namespace gearhip
