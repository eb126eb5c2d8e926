// Top-k of fp32 priorities by radix select + ordered compaction + segmented ordering, gfx950.
//
// fp32 priorities map to order-preserving uint32 keys, selected top-down in three levels: 16384
// level-0 bins, then up to 11 and up to 10 bits inside the picked bin.  The launches of one call:
//   prep      one workgroup draws 2048 to 32768 samples and lays out the level-0 bins around them (coarse
//             below the bin that safely lies under the k-th largest priority -- the hint --, fine
//             from there to the largest sample, the rest above); the others clear the histograms.
//   level 0   ONE read of the priorities: per wave a list of every candidate (key | index) at or
//             above the hint, in index order, and the level-0 histogram of the candidates (the
//             entries below the hint cost one compare each and are not counted).  Without a
//             hint every entry is counted (and listed, when the lists hold whole ranges).
//   level 1   picks the level-0 bin that holds the k-th largest key; histogram of the top bits
//             inside that bin over its members;   level 2   the same for the remaining bits.
//   count     picks the last digit: threshold key T and the number of entries equal to T still
//             needed; counts (greater, equal) per wave and workgroup.
//   write     sums the counts of the waves before it and places the selected entries in index
//             order: every entry above T and the first `need` entries equal to T (ties go to the
//             smaller index).
// Levels 1, 2, count and write walk the candidate lists (about 2 % of the input) when the hint
// held; a wave whose list overflowed (clustered maxima, masses of equal priorities) reads its own
// range of the priorities again instead, in each of them (count then rebuilds its list with the
// exact threshold, write re-reads if that overflows too).
// When the hint fails (fewer than k candidates: the k-th largest priority lies below it; only a
// sample that misleads does that) the entries below the hint -- which level 0 does not even
// count, that is what makes it fast -- are searched by the same launches in another way: level 1
// and level 2 stream the priorities and count the upper and the lower 16 bits of the keys below
// the hint (65536-bin histograms, 16-bit counters packed in LDS and flushed before they can
// overflow), count picks the threshold from the second one and streams as for an overflowed
// list.  The hint only decides which way it is, never the result.
// Value order (k <= 131072): write leaves the selection as (key, index, segment) in index order
// and puts the entries equal to T straight at the tail of the output; the level-0 histogram says
// where every bin starts in value order, bins that start in the same stretch of output places
// form the segment of one workgroup of a last launch, which collects its entries, sorts them
// (most-significant-digit radix sort in LDS; a segment of more than 8192 entries -- thousands of
// equal priorities -- is first cut by counting-sort levels in global memory) and writes its
// stretch of values and indices.
// Larger k take the stable LSD radix sort on the inverted key.
// The streaming loops are sensitive to their instruction count, so they compare floats (one
// instruction, same order as the keys for non-NaN values) wherever a key is not needed.
#include <type_traits>

#include "radix_sort.hpp"

namespace gearhip {
namespace {

constexpr int kThreads = 1024;               // every kernel of the selection
constexpr int kWavesPerBlock = kThreads / kWave;
constexpr int kMaxBlocks = 256;              // one workgroup per CU
constexpr int kBins0 = 16384;  // level-0 bins
constexpr int kBinsR = 2048;   // bins of a refinement level (up to 11 bits)
constexpr int kBinsF = 65536;  // bins of the two levels that run after a failed hint (16 bits)
constexpr int kUniformShift = 18;  // level-0 bins without a sample: the top 14 bits of the key
// with a sample: keys below the hint at 12 bits (numbered, never counted), a middle stretch up to
// the sample's top in up to kMidBins (value order: even segments for the sort) or kMidBinsCoarse
// bins of its own resolution, the rest above in at most kTopBins bins: at most kHintedBins bins
// from the hint upwards, which are the ones that are counted
constexpr int kLowShift = 20, kMidBins = 2048, kMidBinsCoarse = 256, kTopBins = 2046;
constexpr int kHintedBins = 4096;
// Keys of one level-0 bin differ in at most this many low bits, whichever stretch it lies in:
// level 1 resolves the top 11 of them, level 2 the rest.
constexpr int kMaxBinBits = 21;
static_assert(kLowShift <= kMaxBinBits && kUniformShift <= kMaxBinBits, "coarse bins within the levels' reach");
// (a stretch too wide for its bins at 2^kMaxBinBits keys apiece gets more of them: no more than
// 2^11 + 3 for both stretches together when both are that wide.  1023 + 1022 bins, which would
// let value order keep eight copies too, were measured: level 0 0.8 us faster, the sort 0.7 us
// slower.)
static_assert(kMidBins + 1 + kTopBins + 1 <= kHintedBins &&
                  (1ll << (32 - kMaxBinBits)) + 3 <= kHintedBins &&
                  (1ll << (32 - kMaxBinBits)) <= kMidBins && (1ll << (32 - kMaxBinBits)) <= kTopBins + 2,
              "the bins from the hint upwards fit one copy of the histogram");
static_assert((1ll << 32 >> kLowShift) + kHintedBins <= kBins0, "every bin has a number below kBins0");
// The sample: 2, 8 or 32 priorities per thread of one workgroup (2048, 8192 or 32768).  One CU
// sustains about one random miss per 1.2 ns, so the sample is as small as keeps the candidate
// lists from overflowing: a loose bound lists too much, and after an overflow every later level
// reads the whole input again.
constexpr int kMaxSamplesPerThread = 32;
constexpr uint32_t kNoLists = 0xffffffffu;   // hint_bin: level 0 writes no candidate lists
constexpr uint32_t kListFull = 0xffffffffu;  // wave_listed: the wave's list overflowed, the wave reads its range instead
constexpr int64_t kBucketMaxK = 131072;      // value order by buckets up to this k
constexpr int kSortThreads = 1024;           // segment sort workgroup
constexpr int kSmallGroup = 256;             // groups up to this size are ranked directly
constexpr int kNoSegment = 255;              // segment id of an entry that no sort workgroup takes

// Level-0 bins: three stretches of keys with a resolution each, so that the stretch in which the
// selection ends -- known roughly from the sample -- is cut finely (a bin holds few entries: the
// later levels and the value-order sort then have little to do per bin) while 16384 bins still
// cover every key.  Without a sample: one stretch, bin = key >> kUniformShift.
struct BinMap {
  uint32_t uniform;  // 1: no sample
  uint32_t a_end;    // keys below:              bin = key >> kLowShift
  uint32_t b_last;   // a_end <= key <= b_last:  bin = nb0 + ((key - a_end) >> b_shift)
  uint32_t nb0, nc0;  // first bin of the middle / of the top stretch
  uint32_t b_shift, c_shift;  // keys above b_last: bin = nc0 + ((key - b_last - 1) >> c_shift)
};

__device__ __forceinline__ uint32_t bin_of(const BinMap &m, uint32_t key) {
  if (m.uniform) return key >> kUniformShift;
  uint32_t bin = key >> kLowShift;
  if (key >= m.a_end) {  // about one key in a hundred
    bin = key <= m.b_last ? m.nb0 + ((key - m.a_end) >> m.b_shift)
                          : m.nc0 + ((key - m.b_last - 1u) >> m.c_shift);
  }
  return bin;
}
// smallest key of a bin; for one past the last bin of the map the result wraps to 0
__device__ __forceinline__ uint32_t bin_lo_key(const BinMap &m, uint32_t bin) {
  if (m.uniform) return bin << kUniformShift;
  if (bin < m.nb0) return bin << kLowShift;
  if (bin < m.nc0) return m.a_end + ((bin - m.nb0) << m.b_shift);
  return m.b_last + 1u + ((bin - m.nc0) << m.c_shift);
}
__device__ __forceinline__ uint32_t bin_hi_key(const BinMap &m, uint32_t bin) {
  return bin_lo_key(m, bin + 1u) - 1u;
}

// The map around a hint: keys below a_end (a multiple of 2^kLowShift) in coarse bins, the stretch
// a_end .. b_last in up to mid_bins bins of its own resolution, the keys above in at most
// kTopBins bins (top_coarse: as coarsely as the levels below allow).  A bin never spans more
// than 2^kMaxBinBits keys -- the two levels below resolve 11 and 10 bits --: a stretch too wide
// for its bins at that size gets more of them; the two stretches together then still stay below
// 2^(32 - kMaxBinBits) + 3 bins.
__device__ __forceinline__ BinMap make_map(uint32_t a_end, uint32_t b_last, int mid_bins,
                                           bool top_coarse) {
  BinMap map;
  map.uniform = 0u;
  map.a_end = a_end;
  map.b_last = b_last < a_end ? a_end : b_last;
  map.b_shift = map.c_shift = 0u;
  const uint32_t span = map.b_last - map.a_end;
  while (map.b_shift < (uint32_t)kMaxBinBits && (span >> map.b_shift) >= (uint32_t)mid_bins)
    ++map.b_shift;
  map.nb0 = map.a_end >> kLowShift;
  map.nc0 = map.nb0 + (span >> map.b_shift) + 1u;
  const uint32_t rest = 0xffffffffu - map.b_last;  // keys above the middle stretch
  while (rest != 0u && map.c_shift < (uint32_t)kMaxBinBits &&
         ((rest - 1u) >> map.c_shift) >= (uint32_t)kTopBins)
    ++map.c_shift;
  if (top_coarse && rest != 0u) map.c_shift = (uint32_t)kMaxBinBits;
  return map;
}

// The level-0 histogram of a map with a hint holds the bins from the hint upwards only (at most
// kHintedBins; bin b is counted at b - nb0), in several copies.  Every workgroup of level 0 adds
// its counts to the histogram in memory at the end, all of them at about the same time and to
// the same cache lines, and atomics on one line are served one after the other (about 16 ns
// apiece: 245 workgroups, 4 us; more with more lines).  With 8 copies (4 when the histogram has
// more than 2048 bins: value order) workgroup b adds to copy b mod 8, and level 1 adds the
// copies up when it picks: 3 us less for level 0.
struct Copies {
  uint32_t used;    // bins from the hint upwards: bin b is counted at b - nb0
  uint32_t copies;  // 8 or 4
  uint32_t pitch;   // words from one copy to the next
};
__device__ __forceinline__ Copies copies_of(const BinMap &m) {
  Copies c;
  const uint32_t rest = 0xffffffffu - m.b_last;
  c.used = (m.nc0 - m.nb0) + (rest != 0u ? ((rest - 1u) >> m.c_shift) + 1u : 0u);
  c.copies = c.used <= (uint32_t)kBins0 / 8u ? 8u : 4u;
  c.pitch = (uint32_t)kBins0 / c.copies;  // (used <= kHintedBins = kBins0 / 4)
  return c;
}

// The mark a call leaves with the hint for the next one: the hint is taken up again only by a
// call of the same shape (and never from a workspace that holds anything else).
__host__ __device__ __forceinline__ uint64_t next_mark(int64_t n, int64_t k, int mid_bins) {
  uint64_t x = 0x9e3779b97f4a7c15ull ^ (uint64_t)n;
  x = (x ^ (x >> 31)) * 0xbf58476d1ce4e5b9ull + (uint64_t)k;
  x = (x ^ (x >> 29)) * 0x94d049bb133111ebull + (uint64_t)mid_bins;
  x ^= x >> 32;
  return x | 1ull;  // never zero: zero says "no hint"
}

struct State {
  uint32_t prefix[3];  // level-0 bin, level-1 digit, threshold key
  uint32_t k_rem[3];   // entries still to take from the bin picked at that level
  uint32_t overflow;   // no lists were asked for: every level reads the priorities
  uint32_t fail;       // the hint was too high (fewer than k candidates): see "when the hint fails"
  uint32_t hint_bin;   // candidates are the entries whose level-0 bin is >= this
  uint32_t full;       // levels 1, 2, count stream the priorities instead of the lists
  uint32_t lo0, hi0;   // smallest and largest key of the picked level-0 bin
  BinMap map;
  // what the next call may start from instead of a sample (the warm form): the bound below which
  // nothing is listed and the largest key of the finely cut stretch, valid when next_magic holds
  // the mark of a call with the same n, k and bin resolution
  uint64_t next_magic;
  uint32_t next_a_end, next_b_last;
  uint32_t low_seg;  // after a failed hint, value order: the segment of the entries below the hint
  uint32_t pad[39];
};
static_assert(sizeof(State) == 256, "State is the 256-byte header of the workspace");

__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t b = __float_as_uint(f);
  // positive: set the sign bit; negative: flip every bit
  uint32_t key = b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);
  key += key == 0x7fffffffu ? 1u : 0u;  // -0.0 ranks with +0.0
  return key;
}

// the priority whose order_key is `key` (for +-0.0: +0.0)
__device__ __forceinline__ float key_to_float(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

// Float bounds of a range of keys: float order = key order for non-NaN values.  The keys beyond
// the infinities decode to NaN, with which every compare is false, and the key just below
// +-0.0's does not exist (-0.0 ranks with +0.0), so the bounds stop short of them.
constexpr uint32_t kKeyPosInf = 0xff800000u, kKeyNegInf = 0x007fffffu;
__device__ __forceinline__ float lower_bound_float(uint32_t lo_key) {
  if (lo_key < kKeyNegInf) lo_key = kKeyNegInf;
  if (lo_key > kKeyPosInf) lo_key = kKeyPosInf;
  return key_to_float(lo_key);
}
__device__ __forceinline__ float upper_bound_float(uint32_t hi_key) {
  if (hi_key == 0x7fffffffu) hi_key = 0x7ffffffeu;
  if (hi_key > kKeyPosInf) hi_key = kKeyPosInf;
  if (hi_key < kKeyNegInf) hi_key = kKeyNegInf;
  return key_to_float(hi_key);
}

constexpr int kStep = kWave * 4;  // elements one wave handles per step (one float4 per lane)
constexpr int kAhead = 4;         // steps whose loads are in flight together

// Every wave owns wave_len consecutive elements (a multiple of kStep) and a candidate list of
// list_cap entries; `blocks` workgroups of 16 waves cover the input.
struct Geom {
  int64_t blocks, wave_len, list_cap;
};

Geom geom(int64_t n, int64_t k) {
  Geom g;
  const int64_t nn = n > 0 ? n : 1;
  g.wave_len = ceil_div64(ceil_div64(nn, (int64_t)kMaxBlocks * kWavesPerBlock), kStep) * kStep;
  g.blocks = ceil_div64(nn, g.wave_len * kWavesPerBlock);
  // eight times a wave's fair share of k, between 256 and 1024 entries, never more than the wave
  // has elements; clustered maxima or masses of ties overflow it and take the streaming path
  const int64_t waves = g.blocks * kWavesPerBlock;
  int64_t cap = ceil_div64(8 * ceil_div64(k > 0 ? k : 1, waves), 64) * 64;
  if (cap < 256) cap = 256;
  if (cap > 1024) cap = 1024;  // (level 0 itself lists at most kQueueCap = 512 per wave)
  if (cap > g.wave_len) cap = g.wave_len;
  g.list_cap = cap;
  return g;
}

struct Layout {
  size_t hist0, hist1, hist2, wg_bins, histf1, histf2, boff, wave_listed, wave_ge, block_ge, lists, cidx,
      cand, cand2, cseg, ckey, skey, sidx, tkey, tidx, shist, zero_begin, zero_end, total;
};

Layout layout(int64_t n, int64_t k) {
  Layout l;
  const Geom g = geom(n, k);
  const size_t kk = k > 0 ? (size_t)k : 1;
  size_t o = sizeof(State);
  l.zero_begin = o;
  l.hist0 = o;  o += kBins0 * sizeof(uint32_t);
  l.hist1 = o;  o += kBinsR * sizeof(uint32_t);
  l.hist2 = o;  o += kBinsR * sizeof(uint32_t);
  l.wg_bins = o; o += 4 * kMaxBlocks * sizeof(uint32_t);
  l.histf1 = o; o += kBinsF * sizeof(uint32_t);  // after a failed hint: upper / lower 16 key bits
  l.histf2 = o; o += kBinsF * sizeof(uint32_t);
  l.zero_end = o;
  l.boff = o;   o += kBins0 * sizeof(uint32_t);
  l.wave_listed = o; o += (size_t)kMaxBlocks * kWavesPerBlock * sizeof(uint32_t);
  l.wave_ge = o;     o += (size_t)kMaxBlocks * kWavesPerBlock * sizeof(uint64_t);
  l.block_ge = o;    o += (size_t)kMaxBlocks * sizeof(uint64_t);
  l.lists = o;  o += align_up((size_t)(g.blocks * kWavesPerBlock * g.list_cap) * 8, 256);
  l.cidx = o;   o += align_up(kk * 4, 256);
  l.cand = l.cand2 = l.cseg = l.ckey = l.skey = l.sidx = l.tkey = l.tidx = l.shist = 0;
  if (k <= kBucketMaxK) {
    l.ckey = o;  o += align_up(kk * 4, 256);
    l.cand = o;  o += align_up(kk * 8, 256);
    l.cand2 = o; o += align_up(kk * 8, 256);
    l.cseg = o;  o += align_up(kk, 256);
  } else {
    const size_t k4 = align_up(kk * 4, 256);
    l.ckey = o; o += k4;
    l.skey = o; o += k4;
    l.sidx = o; o += k4;
    l.tkey = o; o += k4;
    l.tidx = o; o += k4;
    l.shist = o; o += radix::hist_bytes(k);
  }
  l.total = o;
  return l;
}

// Every thread of a kThreads workgroup calls this: walk a histogram of BINS bins from the top
// bin down and stop at the bin that holds the k_rem-th largest remaining key.  Returns the bin
// and the number of entries still needed inside it to all threads.  When boff is not null the
// number of entries above every bin at or above the picked one is stored there (where the bin
// starts in value order), and every non-empty one of those bins is entered into the segment
// whose stretch of 2^seg_shift output places it starts in (wg_bins, four words per segment:
// highest bin + 1, BINS - lowest bin, ~(entries above the segment), entries above it + its own;
// 0 = none; zeroed by the caller): the workgroups of the launch share
// that work, every one of them has to call with the same arguments.
// With no such bin (the histogram holds fewer than k_rem entries: the candidates of a hint that
// was too high, or NaN priorities, which nothing counts) the lowest bin is returned, nothing is
// taken off k_rem and `found` is 0; `total` is the number of entries in the histogram.
struct Pick {
  uint32_t bin, k_rem, found, total;
};
template <int BINS>
__device__ __forceinline__ Pick pick_bin(uint32_t k_rem, const uint32_t *hist, uint32_t *boff,
                                         uint32_t *wg_bins = nullptr, int seg_shift = 0,
                                         uint32_t rank2 = 0u, uint32_t *bin2 = nullptr) {
  constexpr int kPerThread = BINS / kThreads > 0 ? BINS / kThreads : 1;
  constexpr int kActive = BINS / kPerThread;  // threads that own bins
  __shared__ uint32_t wsum[kWavesPerBlock];
  __shared__ Pick s_pick;
  __shared__ uint32_t s_bin2;  // the bin that holds the rank2-th largest key (rank2 > 0)
  __shared__ uint32_t s_base[BINS / kWave];  // entries above every 64th bin from the top
  const int tid = threadIdx.x;
  // this workgroup's share of the bins whose place in value order is stored (boff): ranks
  // [r_begin, r_begin + per) from the top; the counts of the first 64 are asked for right away
  const int per = (((BINS + (int)gridDim.x - 1) / (int)gridDim.x) + kWave - 1) & ~(kWave - 1);
  const int r_begin = (int)blockIdx.x * per;
  uint32_t cb0 = 0u;
  if (boff && tid < kWave && r_begin + tid < BINS) cb0 = hist[BINS - 1 - (r_begin + tid)];
  uint32_t c[kPerThread];  // c[j] = count of bin BINS-1 - tid*kPerThread - j (top down)
  int tsum = 0;
  if (kPerThread % 4 == 0) {
    // the thread's bins are one contiguous run: 16-byte loads, reversed into top-down order
#pragma unroll
    for (int v = 0; v < kPerThread / 4; ++v) {
      const u32x4 q = *reinterpret_cast<const u32x4 *>(hist + BINS - (tid + 1) * kPerThread + v * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) c[kPerThread - 1 - (v * 4 + e)] = q[e];
    }
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) tsum += (int)c[j];
  } else {
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      c[j] = tid < kActive ? hist[BINS - 1 - tid * kPerThread - j] : 0u;
      tsum += (int)c[j];
    }
  }
  const int inc = wave_inclusive_sum(tsum);
  if ((tid & 63) == 63) wsum[tid >> 6] = (uint32_t)inc;
  if (tid == 0) {
    s_pick.bin = 0u;
    s_pick.k_rem = k_rem;
    s_pick.found = 0u;
    s_bin2 = 0u;
  }
  __syncthreads();
  // the sums of the waves before this one: one LDS read per lane and a wave sum (a loop over
  // them would be a chain of dependent LDS reads)
  const int lane = tid & 63;
  const uint32_t before =
      (uint32_t)wave_sum((int)(lane < (tid >> 6) && lane < kWavesPerBlock ? wsum[lane] : 0u));
  const uint32_t running0 = before + (uint32_t)(inc - tsum);  // entries above the thread's bins
  const bool active = tid < kActive;
  // The picked bin is the first one that takes the count up to k_rem: it lies in the ONE thread
  // whose bins do that, and only that thread walks its bins (16 waves that all walk 16 bins
  // are bound by instruction issue: 1.5 us).
  auto find = [&](uint32_t rank, uint32_t *bin_out, uint32_t *rem_out) {
    if (active && running0 < rank && running0 + (uint32_t)tsum >= rank) {
      uint32_t r = running0, pb = 0u, pk = 0u;
      bool found = false;
#pragma unroll
      for (int j = 0; j < kPerThread; ++j) {
        const bool here = !found && r + c[j] >= rank;
        pb = here ? (uint32_t)(BINS - 1 - tid * kPerThread - j) : pb;
        pk = here ? rank - r : pk;
        found = found || here;
        r += c[j];
      }
      *bin_out = pb;
      if (rem_out) {
        *rem_out = pk;
        s_pick.found = 1u;
      }
    }
  };
  find(k_rem, &s_pick.bin, &s_pick.k_rem);
  if (rank2 != 0u) find(rank2, &s_bin2, nullptr);
  if (tid == kActive - 1) s_pick.total = running0 + (uint32_t)tsum;
  if (boff && (tid * kPerThread) % kWave == 0 && active) s_base[tid * kPerThread / kWave] = running0;
  __syncthreads();
  // Where the bins at or above the picked one start in value order (the entries above them),
  // and the segment table.  The workgroups of the launch share the bins, `per` each in runs of
  // 64: one bin per lane of a wave, after the pick is out, while the other waves go on.  (The
  // thread that owns 16 bins walking them for this took a microsecond, in workgroup 0 alone
  // three.)  Bins of one segment are neighbours: the table (zeroed before the launch) hears of
  // the first and the last non-empty one of a segment in the wave.
  if (boff) {
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    const uint64_t gt_mask = lane == 63 ? 0ull : (~0ull << (lane + 1));
    for (int ch = tid >> 6; ch * kWave < per && r_begin + ch * kWave < BINS; ch += kWavesPerBlock) {
      const int r = r_begin + ch * kWave + lane;  // the bin's rank from the top
      const uint32_t bin = (uint32_t)(BINS - 1 - r);
      const uint32_t cnt = ch == 0 ? cb0 : hist[bin];
      const uint32_t inc_b = (uint32_t)wave_inclusive_sum((int)cnt);
      const uint32_t above = s_base[(r_begin + ch * kWave) / kWave] + inc_b - cnt;
      const bool sel = above < k_rem;
      if (sel) boff[bin] = above;
      const bool ne = sel && cnt != 0u;
      const uint32_t w = above >> seg_shift;
      const uint64_t nem = wave_ballot(ne);
      const uint64_t lower = nem & lt_mask, upper = nem & gt_mask;
      const int prev = lower ? 63 - __builtin_clzll(lower) : lane;
      const int next = upper ? __builtin_ctzll(upper) : lane;
      const uint32_t w_prev = (uint32_t)__shfl((int)w, prev), w_next = (uint32_t)__shfl((int)w, next);
      // highest bin and start of the stretch from the segment's first bin in the wave, lowest
      // bin and end of the stretch from its last one (the start as its complement: all four are
      // maxima over the waves that see bins of the segment)
      if (ne && (lower == 0ull || w_prev != w)) {
        atomicMax(&wg_bins[4 * w], bin + 1u);
        atomicMax(&wg_bins[4 * w + 2], ~above);
      }
      if (ne && (upper == 0ull || w_next != w)) {
        atomicMax(&wg_bins[4 * w + 1], (uint32_t)BINS - bin);
        atomicMax(&wg_bins[4 * w + 3], above + cnt);
      }
    }
  }
  if (bin2) *bin2 = s_bin2;
  return s_pick;  // a kernel calls this once: nothing here is written again
}

typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));

__device__ __forceinline__ void load_quad(const float *__restrict__ p, int64_t e0, int64_t end,
                                          float q[4]) {
  if (e0 + 4 <= end) {
    const f4 v = *reinterpret_cast<const f4 *>(p + e0);
    q[0] = v[0]; q[1] = v[1]; q[2] = v[2]; q[3] = v[3];
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = (e0 + j < end) ? p[e0 + j] : 0.0f;
  }
}

// A wave streams its range [begin, end): kAhead steps of one float4 per lane are in flight while
// the previous kAhead are handed to f(e0, q) -- e0 the index of the lane's first element, q its
// four values; elements at or beyond `end` hold 0 and must be skipped (e0 + j < end).  Every
// lane of the wave calls f the same number of times, so f may ballot.
// The loads of the steps that lie inside the range carry no test and no branch: the compiler
// waits for every load that a branch goes around where the paths meet, one round trip to memory
// per step instead of one per kAhead steps.  A step beyond the last whole one is loaded from the
// last one's place and not looked at; what is left of the range after its whole steps (the end
// of the input: the last wave) is loaded element by element, once.
__device__ const float g_zero_step[kStep] = {};  // something to load where a range has no whole step
__device__ __forceinline__ f4 load_whole_step(const float *lane_base, int step, int last) {
  const int st = step < last ? step : last;
  return *reinterpret_cast<const f4 *>(lane_base + (int64_t)st * kStep);
}
template <typename F>
__device__ __forceinline__ void stream_range(const float *__restrict__ p, int64_t begin,
                                             int64_t end, int lane, F f) {
  if (begin >= end) return;
  const int whole = (int)((end - begin) / kStep);
  if (whole > 0) {
    const float *lane_base = p + begin + lane * 4;
    f4 q[kAhead];
#pragma unroll
    for (int a = 0; a < kAhead; ++a) q[a] = load_whole_step(lane_base, a, whole - 1);
    for (int s = 0; s < whole; s += kAhead) {
      f4 qn[kAhead];
#pragma unroll
      for (int a = 0; a < kAhead; ++a) qn[a] = load_whole_step(lane_base, s + kAhead + a, whole - 1);
#pragma unroll
      for (int a = 0; a < kAhead; ++a) {
        if (s + a < whole) {
          const float v[4] = {q[a][0], q[a][1], q[a][2], q[a][3]};
          f(begin + (int64_t)(s + a) * kStep + lane * 4, v);
        }
      }
#pragma unroll
      for (int a = 0; a < kAhead; ++a) q[a] = qn[a];
    }
  }
  const int64_t t0 = begin + (int64_t)whole * kStep;
  if (t0 < end) {
    float v[4];
    load_quad(p, t0 + lane * 4, end, v);
    f(t0 + lane * 4, v);
  }
}

// The same for callers that pay for the test of every element against `end`: f(e0, q, whole) with
// whole = std::true_type when no element of the wave's step lies at or beyond `end`.
// The caller asks for the first kAhead steps itself (stream_first), ahead of work that does
// not depend on them.
__device__ __forceinline__ void stream_first(const float *__restrict__ p, int64_t begin, int64_t end,
                                             int lane, f4 (&q)[kAhead]) {
  // (a wave without a whole step loads zeros that it does not look at: no branch here either)
  const int whole = begin < end ? (int)((end - begin) / kStep) : 0;
  const float *lane_base = (whole > 0 ? p + begin : g_zero_step) + lane * 4;
#pragma unroll
  for (int a = 0; a < kAhead; ++a) q[a] = load_whole_step(lane_base, a, whole > 0 ? whole - 1 : 0);
}
template <typename F>
__device__ __forceinline__ void stream_range_tagged(const float *__restrict__ p, int64_t begin,
                                                    int64_t end, int lane, f4 (&q)[kAhead], F f) {
  if (begin >= end) return;
  const int whole = (int)((end - begin) / kStep);
  if (whole > 0) {
    const float *lane_base = p + begin + lane * 4;
    for (int s = 0; s < whole; s += kAhead) {
      f4 qn[kAhead];
#pragma unroll
      for (int a = 0; a < kAhead; ++a) qn[a] = load_whole_step(lane_base, s + kAhead + a, whole - 1);
#pragma unroll
      for (int a = 0; a < kAhead; ++a) {
        if (s + a < whole) {
          const float v[4] = {q[a][0], q[a][1], q[a][2], q[a][3]};
          f(begin + (int64_t)(s + a) * kStep + lane * 4, v, std::true_type{});
        }
      }
#pragma unroll
      for (int a = 0; a < kAhead; ++a) q[a] = qn[a];
    }
  }
  const int64_t t0 = begin + (int64_t)whole * kStep;
  if (t0 < end) {
    float v[4];
    load_quad(p, t0 + lane * 4, end, v);
    f(t0 + lane * 4, v, std::false_type{});
  }
}

// The same range as rows of 64 consecutive elements, one per lane: f(i, v, valid) for the lane's
// element i of every row (all lanes call), rows in index order.  For a wave that stores something
// per element: the lanes' stores then fall side by side.
template <typename F>
__device__ __forceinline__ void stream_rows(const float *__restrict__ p, int64_t begin, int64_t end,
                                            int lane, F f) {
  if (begin >= end) return;
  const int whole = (int)((end - begin) / kStep);  // steps of four whole rows
  if (whole > 0) {
    const float *lane_base = p + begin + lane;
    auto load_step = [&](int step, float (&q)[4]) {
      const int st = step < whole - 1 ? step : whole - 1;
#pragma unroll
      for (int j = 0; j < 4; ++j) q[j] = lane_base[(int64_t)st * kStep + j * kWave];
    };
    float q[kAhead][4];
#pragma unroll
    for (int a = 0; a < kAhead; ++a) load_step(a, q[a]);
    for (int s = 0; s < whole; s += kAhead) {
      float qn[kAhead][4];
#pragma unroll
      for (int a = 0; a < kAhead; ++a) load_step(s + kAhead + a, qn[a]);
#pragma unroll
      for (int a = 0; a < kAhead; ++a) {
        if (s + a < whole) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            f(begin + (int64_t)(s + a) * kStep + j * kWave + lane, q[a][j], true);
        }
      }
#pragma unroll
      for (int a = 0; a < kAhead; ++a)
#pragma unroll
        for (int j = 0; j < 4; ++j) q[a][j] = qn[a][j];
    }
  }
  // what is left after the whole steps: up to four rows, the last one ragged
  for (int64_t r0 = begin + (int64_t)whole * kStep; r0 < end; r0 += kWave) {
    const int64_t i = r0 + lane;
    f(i, i < end ? p[i] : 0.0f, i < end);
  }
}

// Appends the lane's selected entries (sel[j], in element order) to the wave's list in index
// order.  `listed` counts every candidate seen, also the ones that no longer fit (wave-uniform).
__device__ __forceinline__ void list_append(uint64_t *list, int list_cap, int &listed,
                                            bool &overflow, const bool sel[4],
                                            const uint32_t key[4], int64_t e0, uint64_t lt_mask) {
  int off[4], nc = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    off[j] = nc;
    nc += sel[j] ? 1 : 0;
  }
  if (wave_ballot(nc != 0) == 0ull) return;
  // candidates in the lanes before this one: nc <= 4 is three bits, one ballot per bit
  // (independent instructions; a DPP scan is a chain of a dozen dependent ones)
  const uint64_t b0 = wave_ballot((nc & 1) != 0), b1 = wave_ballot((nc & 2) != 0),
                 b2 = wave_ballot((nc & 4) != 0);
  const int before = __popcll(b0 & lt_mask) + 2 * __popcll(b1 & lt_mask) + 4 * __popcll(b2 & lt_mask);
  const int total = __popcll(b0) + 2 * __popcll(b1) + 4 * __popcll(b2);
  if (listed + total > list_cap) {
    overflow = true;
  } else {
    const int at = listed + before;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (sel[j]) list[at + off[j]] = ((uint64_t)key[j] << 32) | (uint32_t)(e0 + j);
  }
  listed += total;
}

// ---- prep: the sample, the bin map and the zeros ------------------------------------------------------
// Workgroup 0 looks at kPer * 1024 priorities spread over the input (one per stride, at a hashed
// offset inside it) and lays out the level-0 bins around them: the keys below the bin of the
// `rank`-th largest sample (the hint; bins of the top 14 key bits) are binned coarsely, the
// stretch from there to the largest sample as finely as kMidBins bins allow, the keys above with
// what is left of the 16384 bins.  rank is set a few standard deviations beyond the sample's
// share of k, so that the k-th largest priority of the whole input lies in the fine stretch
// unless the sample misleads -- which costs time (the later levels stream the input again),
// never correctness.  rank = 0: no sample, uniform bins; every entry is listed when list_all is
// set (the lists are as long as the waves' ranges), none otherwise.
// warm != 0: when the workspace holds the hint that the last call of the same shape left for this
// one (the bound derived from its exact counts), the map is laid out around that and no sample
// is drawn; otherwise as above.  The other workgroups clear the histograms.
template <int kPer>  // samples per thread
__global__ __launch_bounds__(kThreads) void prep_kernel(const float *__restrict__ p, int64_t n,
                                                        int64_t k, uint32_t rank, int list_all,
                                                        int mid_bins, int warm, State *state,
                                                        uint32_t *zero, int64_t zero_words) {
  __shared__ __align__(16) uint32_t h[kBins0];
  const int tid = threadIdx.x;
  if (blockIdx.x > 0) {
    const int64_t i = ((int64_t)(blockIdx.x - 1) * kThreads + tid) * 4;
    if (i + 4 <= zero_words) {
      *reinterpret_cast<u32x4 *>(zero + i) = u32x4{0u, 0u, 0u, 0u};
    } else {
      for (int64_t j = i; j < zero_words; ++j) zero[j] = 0u;
    }
    return;
  }
  // the hint of the last call, read by one thread before anything of the state is written
  __shared__ uint32_t s_warm[3];
  bool reuse = false;
  uint32_t warm_a_end = 0u, warm_b_last = 0u;
  if (warm && rank != 0u) {
    if (tid == 0) {
      s_warm[0] = state->next_magic == next_mark(n, k, mid_bins) ? 1u : 0u;
      s_warm[1] = state->next_a_end & ~((1u << kLowShift) - 1u);
      s_warm[2] = state->next_b_last;
    }
    __syncthreads();
    reuse = s_warm[0] != 0u;
    warm_a_end = s_warm[1];
    warm_b_last = s_warm[2];
  }
  float v[kPer];
  if (rank != 0u && !reuse) {
    const int64_t stride = n / (kPer * kThreads);  // >= 128 (the caller's condition), < 2^20
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const uint32_t s = (uint32_t)(tid + j * kThreads);
      // a hashed offset inside the sample's stride: high half of hash * stride, no division
      v[j] = p[(int64_t)s * stride + __umulhi(s * 2654435761u, (uint32_t)stride)];
    }
  }
  if (tid < 3) state->prefix[tid] = 0u;
  if (tid >= 3 && tid < 6) state->k_rem[tid - 3] = 0u;
  if (tid == 6) state->fail = 0u;
  if (tid == 7) state->full = 0u;
  if (tid == 8) state->overflow = (rank == 0u && !list_all) ? 1u : 0u;
  if (tid == 9) state->next_magic = 0ull;  // level 1 of this call leaves the next hint, if any
  BinMap map;
  map.uniform = 1u;
  map.a_end = map.b_last = map.nb0 = map.nc0 = map.b_shift = map.c_shift = 0u;
  uint32_t hint = (rank == 0u && !list_all) ? kNoLists : 0u;
  if (rank != 0u && reuse) {
    map = make_map(warm_a_end, warm_b_last, mid_bins, mid_bins == kMidBinsCoarse);
    hint = map.nb0;
  } else if (rank != 0u) {
    for (int i = tid; i < kBins0; i += kThreads) h[i] = 0u;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kPer; ++j) atomicAdd(&h[order_key(v[j]) >> kUniformShift], 1u);
    __syncthreads();
    uint32_t top14 = 0u;
    const uint32_t hint14 = pick_bin<kBins0>(rank, h, nullptr, nullptr, 0, 1u, &top14).bin;
    // (the last key of the top bin: the shift wraps to 0 there)
    map = make_map((hint14 << kUniformShift) & ~((1u << kLowShift) - 1u),
                   ((top14 + 1u) << kUniformShift) - 1u, mid_bins, mid_bins == kMidBinsCoarse);
    hint = map.nb0;  // the candidates: everything from the middle stretch upwards
  }
  if (tid == 0) {
    state->hint_bin = hint;
    state->map = map;
  }
}

// Adds 1 to cnt[d] for every valid lane; lanes of the wave that share a counter take one atomic
// (defined with the segment sort).  Called by all lanes of the wave.
__device__ __forceinline__ void count_add(uint32_t *cnt, uint32_t d, bool valid);

// ---- level 0: ONE read of the priorities --------------------------------------------------------------
constexpr int kQueueCap = 512;  // candidates per wave held in LDS; longer lists overflow

// With a hint.  The loop over the priorities is bound by the instructions a CU can issue, not
// by memory, so an entry below the hint -- forty-nine in fifty -- costs ONE compare and nothing
// else: it is not counted anywhere (if the hint turns out too high, levels 1 and 2 look for
// the threshold among those entries themselves, see the top of the file).  The candidates of a
// step enter the wave's queue in LDS as value | index at their place in index order: the
// compares of the wave leave four lane masks, the candidates of the lanes before a lane are four
// masked bit counts.  After the stream the wave turns its queue into its list (key | index),
// all lanes busy, and counts the candidates in the workgroup's level-0 histogram in LDS, noting
// which runs of 64 bins it touched; once every wave is through, only those runs are added to the
// histogram in memory (a sweep over all 16384 bins by every workgroup cost 4 us of a 16 us
// launch).  A wave whose candidates outgrow the queue gives its list up (the later launches read
// its range again) and counts the candidates of its range straight into the histogram.
// Where a candidate's bin is counted: from the hint's bin upwards.  (A map laid out around NaN
// samples -- NaN is not a valid priority -- can take an infinity for a candidate whose bin lies
// below the hint's: whatever the result then is, the count stays inside the histogram.)
__device__ __forceinline__ uint32_t counted_bin(uint32_t bin, uint32_t bin_base) {
  const uint32_t at = bin >= bin_base ? bin - bin_base : 0u;
  return at < (uint32_t)kHintedBins ? at : (uint32_t)kHintedBins - 1u;
}

__device__ __forceinline__ uint32_t lanes_before(uint64_t mask, uint32_t acc) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo((uint32_t)mask, acc));
}

__global__ __launch_bounds__(kThreads) void level0_hinted_kernel(
    const float *__restrict__ p, int64_t n, const State *state, uint32_t *__restrict__ hist0,
    int64_t wave_len, uint32_t *__restrict__ wave_listed, uint64_t *__restrict__ lists,
    int list_cap) {
  __shared__ __align__(16) uint32_t h[kHintedBins];  // the bins from the hint upwards
  __shared__ uint64_t queue[kWavesPerBlock][kQueueCap];
  __shared__ uint32_t s_touched[kHintedBins / kWave];  // runs of 64 bins that hold a count
  const int tid = threadIdx.x, lane = tid & 63;
  // (the same in every lane of a wave: said so, everything that follows from it -- the wave's
  // range, the number of its steps -- stays in scalar registers and branches on it are taken by
  // whole waves, without copies of the loaded values where the paths meet)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t gw = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t begin = gw * wave_len;
  const int64_t end = begin + wave_len < n ? begin + wave_len : n;
  const int len = end > begin ? (int)(end - begin) : 0;  // (a wave's range is far below 2^31)
  const int whole = len / kStep;  // steps of one float4 per lane that lie inside the range
  const float *base = p + (len > 0 ? begin : 0);
  // Loads of whole steps carry no test and no branch (a branch around a load makes the compiler
  // wait for every load where the paths meet); a step beyond the last whole one is loaded from
  // the last one's place and not looked at.
  // (a wave without a whole step loads the first steps of the input, which exist, and does not
  // look at them: the first loads then need no branch either)
  const float *lbase = whole > 0 ? base : p;
  const int last = whole > 0 ? whole - 1 : 0;
  auto load_step = [&](int step, f4 &v) {
    const int st = step < last ? step : last;
    v = *reinterpret_cast<const f4 *>(lbase + (int64_t)st * kStep + lane * 4);
  };
  // the first loads go out before the histogram is cleared
  f4 qa[kAhead], qb[kAhead];
#pragma unroll
  for (int a = 0; a < kAhead; ++a) load_step(a, qa[a]);
  static_assert(kHintedBins == kThreads * 4, "one 16-byte store per thread clears the histogram");
  *reinterpret_cast<u32x4 *>(&h[tid * 4]) = u32x4{0u, 0u, 0u, 0u};
  if (tid < kHintedBins / kWave) s_touched[tid] = 0u;
  const BinMap map = state->map;
  const float lo_f = lower_bound_float(map.a_end);
  const uint32_t bin_base = map.nb0;  // candidates' bins are counted from here
  const uint32_t cap = (uint32_t)(list_cap < kQueueCap ? list_cap : kQueueCap);
  const uint32_t first_index = (uint32_t)begin + (uint32_t)lane * 4u;
  uint64_t *wq = queue[wave];
  uint32_t queued = 0;    // candidates of the wave so far, all in the queue (the same in every lane)
  bool given_up = false;  // ... until they outgrow it
  __syncthreads();
  // v: the lane's four entries of the step at offset s of the range
  auto take = [&](int s, const f4 &v) {
    const uint64_t m0 = wave_ballot(v[0] >= lo_f), m1 = wave_ballot(v[1] >= lo_f),
                   m2 = wave_ballot(v[2] >= lo_f), m3 = wave_ballot(v[3] >= lo_f);
    if ((m0 | m1 | m2 | m3) == 0ull) return;
    // (wave-wide counts: said so, the branch on them is taken by the whole wave)
    const uint32_t total = (uint32_t)__builtin_amdgcn_readfirstlane(
        __popcll(m0) + __popcll(m1) + __popcll(m2) + __popcll(m3));
    if (queued + total > cap) {
      given_up = true;
      return;
    }
    uint32_t at = lanes_before(m3, lanes_before(m2, lanes_before(m1, lanes_before(m0, queued))));
    const uint32_t i0 = first_index + (uint32_t)s;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (v[j] >= lo_f) {
        wq[at] = ((uint64_t)__float_as_uint(v[j]) << 32) | (i0 + (uint32_t)j);
        ++at;
      }
    }
    queued = (uint32_t)__builtin_amdgcn_readfirstlane((int)(queued + total));
  };
  // Two groups of kAhead steps take turns: while one is looked at, the loads of the other are
  // under way.  Inside the loop the next group lies wholly inside the range, so its loads carry
  // no test (a branch around a load makes the compiler copy the loaded registers where the
  // paths meet, and wait for the load there); the last one or two groups are handled after it,
  // with loads past the range redirected to the last step and not looked at.
  int st = 0;  // qa holds the steps st .. st + kAhead - 1
  while (!given_up && st + 2 * kAhead <= whole) {
#pragma unroll
    for (int a = 0; a < kAhead; ++a)
      qb[a] = *reinterpret_cast<const f4 *>(lbase + (int64_t)(st + kAhead + a) * kStep + lane * 4);
#pragma unroll
    for (int a = 0; a < kAhead; ++a)
      if (!given_up) take((st + a) * kStep, qa[a]);
    st += kAhead;
    if (given_up || st + 2 * kAhead > whole) {
#pragma unroll
      for (int a = 0; a < kAhead; ++a) qa[a] = qb[a];
      break;
    }
#pragma unroll
    for (int a = 0; a < kAhead; ++a)
      qa[a] = *reinterpret_cast<const f4 *>(lbase + (int64_t)(st + kAhead + a) * kStep + lane * 4);
#pragma unroll
    for (int a = 0; a < kAhead; ++a)
      if (!given_up) take((st + a) * kStep, qb[a]);
    st += kAhead;
  }
  if (!given_up && st < whole) {
#pragma unroll
    for (int a = 0; a < kAhead; ++a) load_step(st + kAhead + a, qb[a]);
#pragma unroll
    for (int a = 0; a < kAhead; ++a)
      if (st + a < whole && !given_up) take((st + a) * kStep, qa[a]);
#pragma unroll
    for (int a = 0; a < kAhead; ++a)
      if (st + kAhead + a < whole && !given_up) take((st + kAhead + a) * kStep, qb[a]);
  }
  if (!given_up && whole * kStep < len) {
    // the ragged end of the input, in the one wave that holds it; what lies beyond reads as
    // NaN, which no compare takes for a candidate
    f4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = whole * kStep + lane * 4 + j;
      v[j] = e < len ? base[e] : __uint_as_float(0x7fc00000u);
    }
    take(whole * kStep, v);
  }
  if (given_up) {
    // Masses of equal priorities or clustered maxima: more candidates than the queue holds.  The
    // wave gives its list up and counts the candidates of its whole range straight into the
    // histogram, lanes that share a bin by one atomic (the range is read again: it is in the
    // caches, and the later launches read it again anyway).
    queued = 0;
    stream_range(p, begin, end, lane, [&](int64_t e0, const float q[4]) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool cand = e0 + j < end && q[j] >= lo_f;
        if (wave_ballot(cand) == 0ull) continue;
        const uint32_t bin = counted_bin(bin_of(map, order_key(q[j])), bin_base);
        count_add(h, bin, cand);
        if (cand) s_touched[bin / kWave] = 1u;
      }
    });
  }
  // the queue, in index order, becomes the wave's list and is counted
  uint64_t *list = lists + gw * list_cap;
  for (uint32_t i = (uint32_t)lane; i < queued; i += kWave) {
    const uint64_t ent = wq[i];
    const uint32_t key = order_key(__uint_as_float((uint32_t)(ent >> 32)));
    const uint32_t bin = counted_bin(bin_of(map, key), bin_base);
    atomicAdd(&h[bin], 1u);
    s_touched[bin / kWave] = 1u;
    list[i] = ((uint64_t)key << 32) | (uint32_t)ent;
  }
  // a wave whose list overflowed says so: the later launches read its range of the priorities
  // again, its range only
  if (lane == 0) wave_listed[gw] = given_up ? kListFull : queued;
  __syncthreads();
  // The counts go to memory by runs of 64 bins, a lane per bin, and only the runs that hold
  // any: atomics of a wave that fall into one cache line travel as one request, and requests to
  // a line are served one after the other -- candidates that each added their own bin's count
  // sent some 50 000 requests to the eight lines of 256 coarse bins, 20 to 35 us.  Wave w looks
  // after the runs w, w + 16, w + 32 and w + 48, in this workgroup's copy of the histogram.
  static_assert(kHintedBins / kWave == kWavesPerBlock * 4, "four runs of bins per wave");
  const Copies cp = copies_of(map);
  uint32_t *mine = hist0 + (blockIdx.x % cp.copies) * cp.pitch;
  const uint32_t flag = lane < 4 ? s_touched[wave + kWavesPerBlock * lane] : 0u;
  for (uint64_t todo = wave_ballot(flag != 0u); todo != 0ull; todo &= todo - 1ull) {
    const int run = wave + kWavesPerBlock * (__ffsll((unsigned long long)todo) - 1);
    const uint32_t c = h[run * kWave + lane];
    if (c != 0u) atomicAdd(&mine[run * kWave + lane], c);
  }
}

// Without a hint: every entry is counted in its level-0 bin (uniform bins of the top 14 key
// bits; LDS histogram, flushed with atomics).  Short inputs, whose lists hold whole ranges, also
// list every entry at its own place in the wave's range -- nothing to queue or order; otherwise
// nothing is listed and the later levels stream the priorities.
__global__ __launch_bounds__(kThreads) void level0_kernel(const float *__restrict__ p, int64_t n,
                                                          const State *state,
                                                          uint32_t *__restrict__ hist0,
                                                          int64_t wave_len,
                                                          uint32_t *__restrict__ wave_listed,
                                                          uint64_t *__restrict__ lists, int list_cap) {
  __shared__ __align__(16) uint32_t h[kBins0];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // the first loads of the wave's range go out before the histogram is cleared
  const int64_t gw = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t begin = gw * wave_len;
  const int64_t end = begin + wave_len < n ? begin + wave_len : n;
  f4 q0[kAhead];
  stream_first(p, begin, end, lane, q0);
  for (int i = tid; i < kBins0; i += kThreads) h[i] = 0u;
  const bool whole_ranges = state->hint_bin != kNoLists;
  const BinMap map = state->map;
  __syncthreads();
  uint64_t *list = lists + gw * list_cap;
  stream_range_tagged(p, begin, end, lane, q0, [&](int64_t e0, const float q[4], auto whole) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (decltype(whole)::value || e0 + j < end) {
        const uint32_t key = order_key(q[j]);
        atomicAdd(&h[bin_of(map, key)], 1u);
        if (whole_ranges && e0 + j - begin < list_cap)
          list[e0 + j - begin] = ((uint64_t)key << 32) | (uint32_t)(e0 + j);
      }
    }
  });
  if (whole_ranges && lane == 0) wave_listed[gw] = begin < end ? (uint32_t)(end - begin) : 0u;
  __syncthreads();
  for (int i = tid; i < kBins0; i += kThreads)
    if (h[i]) atomicAdd(&hist0[i], h[i]);
}

// pick_bin for the level-0 histogram of a map with a hint (see Copies): the bins from the hint
// upwards, at most kHintedBins, kept in several copies that are added up here into `sums` (LDS,
// kHintedBins words).  Returns the picked bin under its number in the map; boff, wg_bins and
// seg_shift as for pick_bin.  Every thread of the workgroup calls.
__device__ __forceinline__ Pick pick_copies(uint32_t k_rem, const uint32_t *hist, const BinMap &map,
                                            uint32_t rank2, uint32_t *bin2, uint32_t *sums,
                                            uint32_t *boff, uint32_t *wg_bins, int seg_shift) {
  constexpr int kPer = 4;  // bins per thread, top down: thread 0 owns the top four
  static_assert(kPer * kThreads == kHintedBins, "every bin of a copy has its thread");
  __shared__ uint32_t wsum[kWavesPerBlock];
  __shared__ Pick s_pick;
  __shared__ uint32_t s_bin2;
  __shared__ uint32_t s_base[kHintedBins / kWave];  // entries above every 64th bin from the top
  const Copies cp = copies_of(map);
  const int tid = threadIdx.x, lane = tid & 63;
  // the copies are added up into `sums` (LDS, 4096 words): neighbouring threads take neighbouring
  // bins, and a thread's loads of the copies of its bin are all under way together
  for (uint32_t at = (uint32_t)tid; at < cp.used; at += kThreads) {
    uint32_t v[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) v[r] = (uint32_t)r < cp.copies ? hist[(uint32_t)r * cp.pitch + at] : 0u;
    sums[at] = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
  }
  __syncthreads();
  uint32_t c[kPer];
  uint32_t tsum = 0u;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const uint32_t from_top = (uint32_t)(tid * kPer + j);
    c[j] = from_top < cp.used ? sums[cp.used - 1u - from_top] : 0u;
    tsum += c[j];
  }
  const int inc = wave_inclusive_sum((int)tsum);
  if (lane == 63) wsum[tid >> 6] = (uint32_t)inc;
  if (tid == 0) {
    s_pick.bin = map.nb0;
    s_pick.k_rem = k_rem;
    s_pick.found = 0u;
    s_bin2 = 0u;
  }
  __syncthreads();
  const uint32_t before =
      (uint32_t)wave_sum((int)(lane < (tid >> 6) && lane < kWavesPerBlock ? wsum[lane] : 0u));
  const uint32_t running0 = before + (uint32_t)inc - tsum;  // entries above the thread's bins
  auto find = [&](uint32_t rank, uint32_t *bin_out, uint32_t *rem_out) {
    if (running0 < rank && running0 + tsum >= rank) {  // one thread
      uint32_t r = running0, pb = 0u, pk = 0u;
      bool found = false;
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const bool here = !found && r + c[j] >= rank;
        pb = here ? map.nb0 + cp.used - 1u - (uint32_t)(tid * kPer + j) : pb;
        pk = here ? rank - r : pk;
        found = found || here;
        r += c[j];
      }
      *bin_out = pb;
      if (rem_out) {
        *rem_out = pk;
        s_pick.found = 1u;
      }
    }
  };
  find(k_rem, &s_pick.bin, &s_pick.k_rem);
  if (rank2 != 0u) find(rank2, &s_bin2, nullptr);
  if (tid == kThreads - 1) s_pick.total = running0 + tsum;
  if (boff && (tid * kPer) % kWave == 0) s_base[tid * kPer / kWave] = running0;
  __syncthreads();
  // Where the bins at or above the picked one start in value order, and the segment table: as
  // in pick_bin (the workgroups of the launch share the bins in runs of 64, a bin per lane),
  // with the counts taken from the sums in LDS.
  if (boff) {
    const uint32_t used = cp.used;
    const int per = (int)((((used + gridDim.x - 1u) / gridDim.x) + kWave - 1u) & ~(uint32_t)(kWave - 1));
    const int r_begin = (int)blockIdx.x * per;
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    const uint64_t gt_mask = lane == 63 ? 0ull : (~0ull << (lane + 1));
    for (int ch = tid >> 6; ch * kWave < per && r_begin + ch * kWave < (int)used; ch += kWavesPerBlock) {
      const int r = r_begin + ch * kWave + lane;  // the bin's rank from the top
      const bool real = r < (int)used;
      const uint32_t bin = map.nb0 + used - 1u - (uint32_t)(real ? r : 0);
      const uint32_t cnt = real ? sums[used - 1u - (uint32_t)r] : 0u;
      const uint32_t inc_b = (uint32_t)wave_inclusive_sum((int)cnt);
      const uint32_t above = s_base[(r_begin + ch * kWave) / kWave] + inc_b - cnt;
      const bool sel = real && above < k_rem;
      if (sel) boff[bin] = above;
      const bool ne = sel && cnt != 0u;
      const uint32_t w = above >> seg_shift;
      const uint64_t nem = wave_ballot(ne);
      const uint64_t lower = nem & lt_mask, upper = nem & gt_mask;
      const int prev = lower ? 63 - __builtin_clzll(lower) : lane;
      const int next = upper ? __builtin_ctzll(upper) : lane;
      const uint32_t w_prev = (uint32_t)__shfl((int)w, prev), w_next = (uint32_t)__shfl((int)w, next);
      if (ne && (lower == 0ull || w_prev != w)) {
        atomicMax(&wg_bins[4 * w], bin + 1u);
        atomicMax(&wg_bins[4 * w + 2], ~above);
      }
      if (ne && (upper == 0ull || w_next != w)) {
        atomicMax(&wg_bins[4 * w + 1], (uint32_t)kBins0 - bin);
        atomicMax(&wg_bins[4 * w + 3], above + cnt);
      }
    }
  }
  if (bin2) *bin2 = s_bin2;
  return s_pick;
}

// ---- when the hint fails: 65536-bin histograms over the entries below it -----------------------------
// pick_bin for a histogram of 65536 bins in memory: every thread of the workgroup calls.
__device__ __forceinline__ Pick pick_wide(uint32_t rank, const uint32_t *hist) {
  constexpr int kPer = kBinsF / kThreads;  // 64 bins per thread, thread 0 the top ones
  __shared__ uint32_t wsum[kWavesPerBlock];
  __shared__ Pick s_pick;
  const int tid = threadIdx.x, lane = tid & 63;
  const uint32_t *mine = hist + kBinsF - (tid + 1) * kPer;
  uint32_t tsum = 0u;
#pragma unroll 4
  for (int v = 0; v < kPer / 4; ++v) {
    const u32x4 q = *reinterpret_cast<const u32x4 *>(mine + v * 4);
    tsum += q[0] + q[1] + q[2] + q[3];
  }
  const int inc = wave_inclusive_sum((int)tsum);
  if (lane == 63) wsum[tid >> 6] = (uint32_t)inc;
  if (tid == 0) {
    s_pick.bin = 0u;
    s_pick.k_rem = rank;
    s_pick.found = 0u;
  }
  __syncthreads();
  const uint32_t before =
      (uint32_t)wave_sum((int)(lane < (tid >> 6) && lane < kWavesPerBlock ? wsum[lane] : 0u));
  const uint32_t running0 = before + (uint32_t)inc - tsum;  // entries above the thread's bins
  if (running0 < rank && running0 + tsum >= rank) {  // one thread
    uint32_t r = running0;
    for (int j = kPer - 1; j >= 0; --j) {
      const uint32_t c = mine[j];
      if (r + c >= rank) {
        s_pick.bin = (uint32_t)(kBinsF - (tid + 1) * kPer + j);
        s_pick.k_rem = rank - r;
        s_pick.found = 1u;
        break;
      }
      r += c;
    }
  }
  if (tid == kThreads - 1) s_pick.total = running0 + tsum;
  __syncthreads();
  return s_pick;
}

// Every wave streams its range and counts digit(q) for the entries that member(q) takes, in a
// histogram of kBinsF 16-bit counters packed two to a word in LDS (hp, kBinsF / 2 words), which
// the workgroup adds to hist_out in memory before a counter can overflow: after every 15 steps
// of its 16 waves (61440 entries).  Called by every thread of the workgroup.
constexpr int kFlushSteps = 15;
static_assert(kFlushSteps * kStep * kWavesPerBlock < 65536, "a 16-bit counter holds a period's entries");
template <typename F>
__device__ __forceinline__ void wide_hist(const float *__restrict__ p, int64_t n, int64_t wave_len,
                                          int64_t gw, uint32_t *hp, uint32_t *__restrict__ hist_out,
                                          F digit_of) {
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < kBinsF / 2; i += kThreads) hp[i] = 0u;
  __syncthreads();
  const int64_t begin = gw * wave_len;
  const int64_t end = begin + wave_len < n ? begin + wave_len : n;
  // (the same number of periods in every wave of the workgroup: each ends at a barrier)
  for (int64_t o = 0; o < wave_len; o += (int64_t)kFlushSteps * kStep) {
    const int64_t a = begin + o;
    const int64_t b = a + (int64_t)kFlushSteps * kStep < end ? a + (int64_t)kFlushSteps * kStep : end;
    stream_range(p, a, b, lane, [&](int64_t e0, const float q[4]) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t d = 0u;
        if (e0 + j < b && digit_of(q[j], &d)) atomicAdd(&hp[d >> 1], 1u << (16 * (d & 1u)));
      }
    });
    __syncthreads();
    for (int i = tid; i < kBinsF / 2; i += kThreads) {
      const uint32_t w = hp[i];
      if (w != 0u) {
        if (w & 0xffffu) atomicAdd(&hist_out[2 * i], w & 0xffffu);
        if (w >> 16) atomicAdd(&hist_out[2 * i + 1], w >> 16);
        hp[i] = 0u;
      }
    }
    __syncthreads();
  }
}

// ---- levels 1 and 2: histograms inside the picked bin ------------------------------------------------
// The keys of the picked level-0 bin are lo0 .. hi0; in `bits0` bits they can differ (at most 21).
// LEVEL 1: picks the level-0 bin from hist0 (with a hint the histogram holds the candidates only:
// when they are fewer than k the hint has failed); counts the top min(bits0, 11) of those bits
// over the members of the bin; leaves the next call's hint.  LEVEL 2: picks the level-1 digit
// from hist1; counts the remaining bits (at most 10) over the keys that share bin and digit.
// After a failed hint: LEVEL 1 counts the upper 16 key bits of the entries below the hint
// (histf1), LEVEL 2 picks from that and counts the lower 16 bits of the keys that share the
// upper ones (histf2).
__device__ __forceinline__ int bits_of(uint32_t span) { return span ? 32 - __builtin_clz(span) : 0; }
__device__ __forceinline__ int level1_shift(int bits0) { return bits0 > 11 ? bits0 - 11 : 0; }

template <int LEVEL>
__global__ __launch_bounds__(kThreads) void member_hist_kernel(
    const float *__restrict__ p, int64_t n, int64_t k, int mid_bins, State *state,
    const uint32_t *hist_prev, uint32_t *__restrict__ hist_out, const uint32_t *histf_prev,
    uint32_t *__restrict__ histf_out, uint32_t *boff, uint32_t *wg_bins, int seg_shift,
    int64_t wave_len, const uint32_t *__restrict__ wave_listed,
    const uint64_t *__restrict__ lists, int list_cap) {
  __shared__ uint32_t hp[kBinsF / 2];  // packed counters after a failed hint; else h, below
  uint32_t *h = hp;
  static_assert(kBinsR + kHintedBins <= kBinsF / 2,
                "the level's histogram and the sums of the level-0 copies fit the same LDS");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < kBinsR; i += kThreads) h[i] = 0u;
  // the wave's list does not depend on the pick: its length and first stretch are asked for
  // before the histogram is walked (used only when the lists are in use)
  const int64_t gw = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const uint64_t *list = lists + gw * list_cap;
  // (the same word in every lane: said so, the branches on it are taken by whole waves)
  const uint32_t m_raw = (uint32_t)__builtin_amdgcn_readfirstlane((int)wave_listed[gw]);
  const int m_pre = (int)m_raw;
  const uint64_t ent_pre = list[lane];
  uint32_t lo, hi;  // the keys that are counted
  int shift;        // digit = (key - lo) >> shift
  bool full, fail;
  uint32_t a_end = 0u, upper16 = 0u;
  // what earlier launches left in the state is asked for before the histogram is walked, not
  // after it (a round trip to memory each time)
  if (LEVEL == 1) {
    const BinMap map = state->map;
    const uint32_t overflow = state->overflow, hint_bin = state->hint_bin;
    const bool hinted = map.uniform == 0u && hint_bin != kNoLists;
    // (the 2k-th largest key, where the histogram holds that many: the next call's hint)
    uint32_t bin2 = 0u;
    // (with a hint the histogram holds the bins from the hint upwards, in copies, which are added
    // up in the part of the LDS that only a failed hint uses, later)
    const Pick r = hinted ? pick_copies((uint32_t)k, hist_prev, map, 2u * (uint32_t)k, &bin2,
                                        hp + kBinsR, boff, wg_bins, seg_shift)
                          : pick_bin<kBins0>((uint32_t)k, hist_prev, boff, wg_bins, seg_shift);
    fail = hinted && r.found == 0u;
    lo = bin_lo_key(map, r.bin);
    hi = bin_hi_key(map, r.bin);
    shift = level1_shift(bits_of(hi - lo));
    full = overflow != 0u || fail;
    a_end = map.a_end;
    if (blockIdx.x == 0 && tid == 0) {
      state->prefix[0] = r.bin;
      state->k_rem[0] = fail ? (uint32_t)k - r.total : r.k_rem;
      state->full = full ? 1u : 0u;
      state->fail = fail ? 1u : 0u;
      state->lo0 = lo;
      state->hi0 = hi;
      if (hinted && !fail) {
        // The next call's hint, from exact counts: the coarse-bin boundary at or below the 2k-th
        // largest key; with fewer than 2k candidates one coarse bin below this call's.
        const uint32_t step = 1u << kLowShift;
        uint32_t next = bin2 >= map.nb0 && bin2 != 0u ? bin_lo_key(map, bin2) & ~(step - 1u)
                                                      : (map.a_end >= step ? map.a_end - step : 0u);
        state->next_a_end = next;
        state->next_b_last = map.b_last;
        state->next_magic = next_mark(n, k, mid_bins);
      }
      if (fail && boff != nullptr) {
        // Value order: the entries below the hint that end up selected follow the r.total
        // candidates in the output.  They go to the segment in whose stretch of the output place
        // r.total lies (write finds it in the state); that segment's table entry is widened to
        // the coarse bins [0, nb0) and to the rest of the output.
        const uint32_t w = r.total >> seg_shift;
        state->low_seg = w;
        atomicMax(&wg_bins[4 * w], map.nb0);
        atomicMax(&wg_bins[4 * w + 1], (uint32_t)kBins0);
        atomicMax(&wg_bins[4 * w + 2], ~r.total);
        atomicMax(&wg_bins[4 * w + 3], (uint32_t)k);
      }
    }
  } else {
    const uint32_t lo0 = state->lo0, hi0 = state->hi0, full0 = state->full;
    fail = state->fail != 0u;
    a_end = state->map.a_end;
    const uint32_t k_rem0 = state->k_rem[0];
    Pick r;
    if (!fail) {
      r = pick_bin<kBinsR>(k_rem0, hist_prev, nullptr);
    } else {
      r = pick_wide(k_rem0, histf_prev);
      upper16 = r.bin;
    }
    const int shift1 = level1_shift(bits_of(hi0 - lo0));
    lo = lo0 + (r.bin << shift1);
    hi = lo + ((1u << shift1) - 1u);
    if (hi > hi0 || hi < lo) hi = hi0;
    shift = 0;
    full = full0 != 0u;
    if (blockIdx.x == 0 && tid == 0) {
      state->prefix[1] = r.bin;
      state->k_rem[1] = r.k_rem;
    }
  }
  __syncthreads();
  if (fail) {
    // the entries below the hint: exactly the ones level 0 did not take for candidates
    const float lo_f = lower_bound_float(a_end);
    if (LEVEL == 1) {
      wide_hist(p, n, wave_len, gw, hp, histf_out, [&](float q, uint32_t *d) {
        *d = order_key(q) >> 16;
        return q < lo_f;
      });
    } else {
      wide_hist(p, n, wave_len, gw, hp, histf_out, [&](float q, uint32_t *d) {
        const uint32_t key = order_key(q);
        *d = key & 0xffffu;
        return q < lo_f && (key >> 16) == upper16;
      });
    }
    return;
  }
  // a wave whose list overflowed reads its own range again, the others walk their lists
  if (!full && m_raw != kListFull) {
    const int m = m_pre;
    for (int c0 = 0; c0 < m; c0 += kWave) {
      if (c0 + lane < m) {
        const uint32_t key = (uint32_t)((c0 == 0 ? ent_pre : list[c0 + lane]) >> 32);
        if (key >= lo && key <= hi) atomicAdd(&h[(key - lo) >> shift], 1u);
      }
    }
  } else {
    // membership by two float compares against the bounds of the key range; the key itself is
    // worked out only for the members
    const float lo_f = lower_bound_float(lo);
    const float hi_f = upper_bound_float(hi);
    const int64_t begin = gw * wave_len;
    const int64_t end = begin + wave_len < n ? begin + wave_len : n;
    stream_range(p, begin, end, lane, [&](int64_t e0, const float q[4]) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool near = e0 + j < end && q[j] >= lo_f && q[j] <= hi_f;
        if (wave_ballot(near) == 0ull) continue;
        // masses of equal priorities share a digit: one atomic per wave then
        const uint32_t key = order_key(q[j]);
        count_add(h, (key - lo) >> shift, near && key >= lo && key <= hi);
      }
    });
  }
  __syncthreads();
  for (int i = tid; i < kBinsR; i += kThreads)
    if (h[i]) atomicAdd(&hist_out[i], h[i]);
}

// ---- count: threshold, then (greater, equal) per wave and workgroup ---------------------------------
// Packed counts: greater << 32 | equal.  When the levels before streamed the priorities, this
// launch does too and lists every wave's entries at or above the threshold on the way.
__global__ __launch_bounds__(kThreads) void count_kernel(
    const float *__restrict__ p, int64_t n, State *state, const uint32_t *hist2,
    const uint32_t *histf2, int64_t wave_len, uint32_t *__restrict__ wave_listed, uint64_t *__restrict__ lists, int list_cap,
    uint64_t *__restrict__ wave_ge, uint64_t *__restrict__ block_ge) {
  __shared__ uint64_t red[kWavesPerBlock];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t gw = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  uint64_t *list = lists + gw * list_cap;
  // (the same word in every lane: said so, the branches on it are taken by whole waves)
  const uint32_t m_raw = (uint32_t)__builtin_amdgcn_readfirstlane((int)wave_listed[gw]);
  const int m_pre = (int)m_raw;
  const uint64_t ent_pre = list[lane];
  const uint32_t lo0 = state->lo0, hi0 = state->hi0, digit1 = state->prefix[1];
  const bool full = state->full != 0u || m_raw == kListFull;  // this wave reads its range
  const bool fail = state->fail != 0u;  // digit1: the upper 16 bits, histf2: the lower ones
  const uint32_t k_rem1 = state->k_rem[1];
  Pick r;
  if (!fail)
    r = pick_bin<kBinsR>(k_rem1, hist2, nullptr);
  else
    r = pick_wide(k_rem1, histf2);
  const uint32_t thr = fail ? ((digit1 << 16) | r.bin)
                            : lo0 + (digit1 << level1_shift(bits_of(hi0 - lo0))) + r.bin;
  if (blockIdx.x == 0 && tid == 0) {
    state->prefix[2] = thr;
    state->k_rem[2] = r.k_rem;
  }
  uint32_t gt = 0, eq = 0;
  if (!full) {
    const int m = m_pre;
    for (int c0 = 0; c0 < m; c0 += kWave) {
      if (c0 + lane < m) {
        const uint32_t key = (uint32_t)((c0 == 0 ? ent_pre : list[c0 + lane]) >> 32);
        gt += key > thr;
        eq += key == thr;
      }
    }
  } else {
    const float thr_f = key_to_float(thr);
    const int64_t begin = gw * wave_len;
    const int64_t end = begin + wave_len < n ? begin + wave_len : n;
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    int listed = 0;
    bool overflow = false;
    stream_range(p, begin, end, lane, [&](int64_t e0, const float q[4]) {
      bool sel[4];
      uint32_t key[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // float compares order non-NaN priorities exactly like their keys (-0.0 == +0.0)
        const bool above = q[j] > thr_f;
        sel[j] = e0 + j < end && q[j] >= thr_f;
        gt += sel[j] && above;
        eq += sel[j] && !above;
        key[j] = above ? order_key(q[j]) : thr;
      }
      list_append(list, list_cap, listed, overflow, sel, key, e0, lt_mask);
    });
    if (lane == 0) wave_listed[gw] = overflow ? kListFull : (uint32_t)listed;
  }
  const int64_t w = wave_sum((int64_t)(((uint64_t)gt << 32) | (uint64_t)eq));
  if (lane == 0) {
    wave_ge[gw] = (uint64_t)w;
    red[wave] = (uint64_t)w;
  }
  __syncthreads();
  if (tid == 0) {
    uint64_t t = 0;
#pragma unroll
    for (int i = 0; i < kWavesPerBlock; ++i) t += red[i];
    block_ge[blockIdx.x] = t;
  }
}

// ---- write: ordered compaction -----------------------------------------------------------------------
enum Flavour {
  kDirect,  // indices_out / values_out in index order
  kPairs,   // (inverted key, index) in index order for the LSD radix sort
  kBucket   // (key, index) in index order for the bucket sort; ties at T go straight to the output's tail
};

template <int FLAVOUR>
__global__ __launch_bounds__(kThreads) void write_kernel(
    const float *__restrict__ p, int64_t n, int64_t k, const State *state, int64_t wave_len,
    const uint32_t *__restrict__ wave_listed, const uint64_t *__restrict__ lists, int list_cap,
    const uint64_t *__restrict__ wave_ge, const uint64_t *__restrict__ block_ge,
    uint32_t *__restrict__ ckey, uint32_t *__restrict__ cidx, const uint32_t *__restrict__ boff,
    int seg_shift, uint8_t *__restrict__ cseg, float *__restrict__ values_out,
    int64_t *__restrict__ indices_out) {
  __shared__ uint64_t red[kWavesPerBlock];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t gw = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const uint64_t *list = lists + gw * list_cap;
  // (the same word in every lane: said so, the branch on it is taken by whole waves)
  const uint32_t m_raw = (uint32_t)__builtin_amdgcn_readfirstlane((int)wave_listed[gw]);
  const int m_pre = (int)m_raw;
  const uint64_t ent_pre = list[lane];
  const uint32_t thr = state->prefix[2];
  const uint32_t need_eq = state->k_rem[2];
  const bool reread = m_raw == kListFull;
  const BinMap map = state->map;
  const uint32_t low_seg = state->low_seg;
  const uint32_t low_end = state->fail != 0u ? map.a_end : 0u;  // keys below: under a failed hint

  // counts of the workgroups before this one (at most kMaxBlocks), then of the waves before
  // this one in its own workgroup
  uint64_t part = 0;
  if (tid < (int)blockIdx.x) part = block_ge[tid];
  const int64_t pw = wave_sum((int64_t)part);
  if (lane == 0) red[wave] = (uint64_t)pw;
  __syncthreads();
  uint64_t excl = 0;
#pragma unroll
  for (int i = 0; i < kWavesPerBlock; ++i) excl += red[i];
  uint64_t own = 0;
  if (lane < wave) own = wave_ge[(int64_t)blockIdx.x * kWavesPerBlock + lane];
  excl += (uint64_t)wave_sum((int64_t)own);
  uint32_t gt_run = (uint32_t)(excl >> 32), eq_run = (uint32_t)excl;
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  const uint32_t ties_at = (uint32_t)k - need_eq;  // where the ties at T start in value order

  // pos = the entry's place in index order among the selected, e = its rank among the entries
  // equal to T.
  // `have` says that `value` is the entry's priority (the streaming path has it at hand; from a
  // list it is read from the input: the key does not tell the two zeros apart).
  auto emit = [&](bool selected, bool is_eq, uint32_t pos, uint32_t e, uint32_t index, uint32_t key,
                  auto have, float value) {
    selected = selected && pos < (uint32_t)k;  // out of step only with NaN priorities
    // (a listed entry's priority follows from its key, except for the two zeros, which share
    // one: only those are read from the input -- a gather of every selected value costs 8 MB of
    // cache lines for 65536 entries)
    auto value_of = [&]() {
      return decltype(have)::value ? value : (key != 0x80000000u ? key_to_float(key) : p[index]);
    };
    if (FLAVOUR == kDirect) {
      if (selected) {
        indices_out[pos] = (int64_t)index;
        if (values_out) values_out[pos] = value_of();
      }
    } else if (FLAVOUR == kPairs) {
      if (selected) {
        ckey[pos] = ~key;
        cidx[pos] = index;
      }
    } else {
      // ties at T are the smallest selected keys: they close the output, in index order; the
      // bucket sort skips them (it takes keys above T only)
      if (selected && is_eq && ties_at + e < (uint32_t)k) {
        indices_out[ties_at + e] = (int64_t)index;
        if (values_out) values_out[ties_at + e] = value_of();
      }
      if (selected) {
        ckey[pos] = key;
        cidx[pos] = index;
        // the segment of the sort that takes the entry: the one in whose stretch of the
        // output the entry's level-0 bin starts (ties at T belong to none)
        // (entries below a failed hint have no counted bin: their segment is in the state)
        cseg[pos] = is_eq ? (uint8_t)kNoSegment
                          : (uint8_t)(key < low_end ? low_seg : boff[bin_of(map, key)] >> seg_shift);
      }
    }
  };

  if (!reread) {
    const int m = m_pre;
    for (int c0 = 0; c0 < m; c0 += kWave) {
      const bool valid = c0 + lane < m;
      const uint64_t ent = valid ? (c0 == 0 ? ent_pre : list[c0 + lane]) : 0ull;
      const uint32_t key = (uint32_t)(ent >> 32);
      const bool is_gt = valid && key > thr, is_eq = valid && key == thr;
      const uint64_t bg = wave_ballot(is_gt), be = wave_ballot(is_eq);
      const uint32_t g = gt_run + (uint32_t)__popcll(bg & lt_mask);
      const uint32_t e = eq_run + (uint32_t)__popcll(be & lt_mask);
      const bool selected = is_gt || (is_eq && e < need_eq);
      emit(selected, is_eq, g + (e < need_eq ? e : need_eq), e, (uint32_t)ent, key,
           std::false_type{}, 0.0f);
      gt_run += (uint32_t)__popcll(bg);
      eq_run += (uint32_t)__popcll(be);
    }
    return;
  }

  const float thr_f = key_to_float(thr);
  const int64_t begin = gw * wave_len;
  const int64_t end = begin + wave_len < n ? begin + wave_len : n;
  // (rows of 64: the stores of a row's selected entries fall side by side -- a wave that comes
  // here is one whose list overflowed, and such a wave often selects most of its range)
  stream_rows(p, begin, end, lane, [&](int64_t i, float v, bool valid) {
    const bool is_gt = valid && v > thr_f, is_eq = valid && v == thr_f;
    const uint64_t bg = wave_ballot(is_gt), be = wave_ballot(is_eq);
    // nothing of the row is selected once the ties needed are placed and no entry is above T
    if (bg == 0ull && (be == 0ull || eq_run >= need_eq)) return;
    const uint32_t g = gt_run + (uint32_t)__popcll(bg & lt_mask);
    const uint32_t e = eq_run + (uint32_t)__popcll(be & lt_mask);
    const bool selected = is_gt || (is_eq && e < need_eq);
    emit(selected, is_eq, g + (e < need_eq ? e : need_eq), e, (uint32_t)i,
         is_gt ? order_key(v) : thr, std::true_type{}, v);
    gt_run += (uint32_t)__popcll(bg);
    eq_run += (uint32_t)__popcll(be);
  });
}

// ---- value order: segments gathered and sorted --------------------------------------------------------
// The selected entries arrive in index order as (key, index).  The level-0 histogram says where
// every level-0 bin starts in the value-ordered output; bins whose start falls into the same
// stretch of 2^seg_shift output places form the segment of one workgroup (a run of neighbouring
// bins: workgroup w owns the bins wg_bins[w]).  The workgroup reads all k keys once, keeps the
// entries above T inside its key range -- in LDS when they fit, else in its stretch of a
// global buffer; the places come from a cursor of its own in LDS (global atomics that meet on an
// address are served one after the other by the memory side) --, sorts them, and writes its
// stretch of the output.  An entry is (key - smallest key of the segment's bins) << 32 | ~index, so a larger entry comes earlier in
// value order (ties: smaller index first) and no two are equal.  The sort is a most-significant-
// digit radix sort from the highest bit in which the segment's keys can differ: counting sort on
// 9 bits, groups of up to kSmallGroup entries are ranked directly (every entry counts the larger
// ones), larger groups (equal or nearly equal keys) go down another 9 bits from a stack.
constexpr int kLdsEntries = 8192;  // entries per LDS buffer of the segment sort
constexpr int kStack = 1024;

constexpr int kSortBins = 512;  // 9-bit digits
constexpr int kNarrowFrom = 2048;  // groups from this size on first look for the bits that differ
struct SortShared {
  uint32_t cnt[kSortBins + 1];
  uint32_t start[kSortBins + 1];
  uint32_t wsum[kSortThreads / kWave];
  uint32_t stk_off[kStack], stk_len[kStack];
  uint8_t stk_bits[kStack];   // low bits of the entries still undecided inside the group
  uint8_t stk_flip[kStack];   // the group sits in the second buffer
  int stk_top;
  uint32_t bits_or_and[4];    // OR (two words) and AND (two words) of a long group's entries
};

// Where a sorted entry goes: place i of the segment's stretch of the output.  The value follows
// from the key (the map is one to one) except for the two zeros, which share a key: those are
// read from the input.  (A gather of every value would be bound by the misses one CU can have in
// flight.)
struct SegmentOut {
  const float *p;
  int64_t n;
  float *values;
  int64_t *indices;
  uint32_t base;
  uint32_t key_base;  // entries hold key - key_base
  __device__ __forceinline__ void operator()(uint32_t i, uint64_t ent) const {
    const uint32_t index = ~(uint32_t)ent, key = (uint32_t)(ent >> 32) + key_base;
    indices[base + i] = (int64_t)index;
    if (values)
      values[base + i] =
          key != 0x80000000u ? key_to_float(key) : ((int64_t)index < n ? p[index] : 0.0f);
  }
  __device__ __forceinline__ SegmentOut shifted(uint32_t by) const {
    return SegmentOut{p, n, values, indices, base + by, key_base};
  }
};

// number of entries of src[lo, hi) larger than `mine`
__device__ __forceinline__ uint32_t larger_in(const uint64_t *src, uint32_t lo, uint32_t hi,
                                              uint64_t mine) {
  uint32_t r = 0;
  uint32_t j = lo;
  for (; j + 4 <= hi; j += 4) {
    const uint64_t x0 = src[j], x1 = src[j + 1], x2 = src[j + 2], x3 = src[j + 3];
    r += (x0 > mine) + (x1 > mine) + (x2 > mine) + (x3 > mine);
  }
  for (; j < hi; ++j) r += src[j] > mine;
  return r;
}

// Counting-sort bookkeeping in LDS with the lanes of a wave that share a digit served by ONE
// atomic: thousands of equal priorities put every entry of a group on the same counter, and LDS
// atomics on one address are served one lane after the other.  Two rounds peel off the digits
// of the wave's first unserved lanes when at least eight lanes share them; the rest take plain
// atomics.  cursor_take returns the old value of cursor[d] for each valid lane (distinct places
// for the lanes of a digit); count_add only adds.  Called by all lanes of the wave.
__device__ __forceinline__ uint32_t cursor_take(uint32_t *cursor, uint32_t d, bool valid) {
  const int lane = (int)(threadIdx.x & 63);
  const uint64_t lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  uint64_t todo = wave_ballot(valid);
  uint32_t pos = 0;
  for (int round = 0; round < 2 && todo != 0ull; ++round) {
    const int leader = __ffsll((unsigned long long)todo) - 1;
    const uint32_t dl = (uint32_t)__builtin_amdgcn_readlane((int)d, leader);
    const uint64_t match = wave_ballot(valid && d == dl) & todo;
    if (__popcll(match) < 8) break;
    uint32_t base = 0;
    if (lane == leader) base = atomicAdd(&cursor[dl], (uint32_t)__popcll(match));
    base = (uint32_t)__builtin_amdgcn_readlane((int)base, leader);
    if ((match >> lane) & 1ull) pos = base + (uint32_t)__popcll(match & lt);
    todo &= ~match;
  }
  if ((todo >> lane) & 1ull) pos = atomicAdd(&cursor[d], 1u);
  return pos;
}
__device__ __forceinline__ void count_add(uint32_t *cnt, uint32_t d, bool valid) {
  const int lane = (int)(threadIdx.x & 63);
  uint64_t todo = wave_ballot(valid);
  for (int round = 0; round < 2 && todo != 0ull; ++round) {
    const int leader = __ffsll((unsigned long long)todo) - 1;
    const uint32_t dl = (uint32_t)__builtin_amdgcn_readlane((int)d, leader);
    const uint64_t match = wave_ballot(valid && d == dl) & todo;
    if (__popcll(match) < 8) break;
    if (lane == leader) atomicAdd(&cnt[dl], (uint32_t)__popcll(match));
    todo &= ~match;
  }
  if ((todo >> lane) & 1ull) atomicAdd(&cnt[d], 1u);
}

// A long group often shares most of its remaining bits (thousands of equal priorities: only the
// index bits differ), and a digit that all entries share would send every one of them to the same
// LDS counter, one after the other.  Returns how many low bits of src[off, off+len) can still
// differ (at most rem): the position of the highest bit in which two entries differ, plus one.
// Called by every thread of the workgroup.
// (the second half of it: o and a are the OR and the AND of the entries this thread looked at)
__device__ __forceinline__ int differing_bits_of(uint64_t o, uint64_t a, int rem, SortShared &sh) {
  const int tid = threadIdx.x;
  if (tid < 4) sh.bits_or_and[tid] = tid < 2 ? 0u : 0xffffffffu;
  __syncthreads();
  for (int d = 32; d >= 1; d >>= 1) {  // the wave's lanes, then one atomic per wave and word
    o |= (uint64_t)__shfl_xor((unsigned long long)o, d, kWave);
    a &= (uint64_t)__shfl_xor((unsigned long long)a, d, kWave);
  }
  if ((tid & 63) == 0) {
    atomicOr(&sh.bits_or_and[0], (uint32_t)o);
    atomicOr(&sh.bits_or_and[1], (uint32_t)(o >> 32));
    atomicAnd(&sh.bits_or_and[2], (uint32_t)a);
    atomicAnd(&sh.bits_or_and[3], (uint32_t)(a >> 32));
  }
  __syncthreads();
  uint64_t diff = (((uint64_t)sh.bits_or_and[1] << 32) | sh.bits_or_and[0]) ^
                  (((uint64_t)sh.bits_or_and[3] << 32) | sh.bits_or_and[2]);
  __syncthreads();
  if (rem < 64) diff &= (1ull << rem) - 1ull;
  return diff ? 64 - __builtin_clzll(diff) : 0;
}
__device__ __forceinline__ int differing_bits(const uint64_t *src, uint32_t off, uint32_t len,
                                              int rem, SortShared &sh) {
  uint64_t o = 0ull, a = ~0ull;
  // (several loads under way per thread: out of global memory one at a time is a round trip each)
  constexpr int kLoadsAhead = 8;
  for (uint32_t i0 = threadIdx.x; i0 < len; i0 += kSortThreads * kLoadsAhead) {
    uint64_t x[kLoadsAhead];
#pragma unroll
    for (int u = 0; u < kLoadsAhead; ++u) {
      const uint32_t i = i0 + (uint32_t)u * kSortThreads;
      x[u] = src[off + (i < len ? i : 0u)];  // (beyond the end: the first entry once more)
    }
#pragma unroll
    for (int u = 0; u < kLoadsAhead; ++u) {
      o |= x[u];
      a &= x[u];
    }
  }
  return differing_bits_of(o, a, rem, sh);
}

// Sorts the m entries a[0, m) (descending; only their low `bits` bits can differ) with b as the
// second buffer and hands them to fin(place, entry); called by every thread of the workgroup.  The two
// callers pass either the LDS buffers or global ones, so that after inlining every access has a
// known address space.
__device__ __forceinline__ void sort_segment(uint64_t *a, uint64_t *b, uint32_t m, int bits,
                                             const SegmentOut &fin, SortShared &sh) {
  const int tid = threadIdx.x;
  if (tid == 0) {
    sh.stk_off[0] = 0u;
    sh.stk_len[0] = m;
    sh.stk_bits[0] = (uint8_t)bits;
    sh.stk_flip[0] = 0;
    sh.stk_top = 1;
  }
  __syncthreads();
  while (true) {
    const int top = sh.stk_top;
    if (top == 0) break;
    const uint32_t off = sh.stk_off[top - 1], len = sh.stk_len[top - 1];
    int rem = sh.stk_bits[top - 1];
    const bool flip = sh.stk_flip[top - 1] != 0;
    __syncthreads();
    if (tid == 0) sh.stk_top = top - 1;
    const uint64_t *src = flip ? b : a;
    uint64_t *dst = flip ? a : b;
    if (len <= (uint32_t)kSmallGroup || rem == 0) {
      for (uint32_t i = tid; i < len; i += kSortThreads) {
        const uint64_t mine = src[off + i];
        fin(off + larger_in(src, off, off + len, mine), mine);
      }
      __syncthreads();
      continue;
    }
    if (len >= (uint32_t)kNarrowFrom) {
      rem = differing_bits(src, off, len, rem, sh);
      if (rem == 0) {  // all entries equal: cannot happen (the indices differ), kept for safety
        for (uint32_t i = tid; i < len; i += kSortThreads) fin(off + i, src[off + i]);
        __syncthreads();
        continue;
      }
    }
    const int nb = rem < 9 ? rem : 9;
    const int shift = rem - nb;
    const uint32_t mask = (1u << nb) - 1u;
    // counting sort of src[off, off+len) by the digit, largest digit first
    for (int i = tid; i <= kSortBins; i += kSortThreads) sh.cnt[i] = 0u;
    __syncthreads();
#pragma unroll 4
    for (uint32_t i = tid; i < len; i += kSortThreads)
      atomicAdd(&sh.cnt[mask - (uint32_t)((src[off + i] >> shift) & mask)], 1u);
    __syncthreads();
    {
      const uint32_t c = tid < kSortBins ? sh.cnt[tid] : 0u;  // the first kSortBins threads own a digit each
      const int inc = wave_inclusive_sum((int)c);
      if ((tid & 63) == 63) sh.wsum[tid >> 6] = (uint32_t)inc;
      __syncthreads();
      // sums of the waves before this one: one LDS read per lane and a wave sum, not a chain of
      // dependent LDS reads
      const int ln = tid & 63;
      const uint32_t before =
          (uint32_t)inc - c +
          (uint32_t)wave_sum((int)(ln < (tid >> 6) && ln < kSortThreads / kWave ? sh.wsum[ln] : 0u));
      if (tid < kSortBins) {
        sh.start[tid] = before;
        sh.cnt[tid] = before;  // cursors
      }
      if (tid == kSortBins - 1) sh.start[kSortBins] = before + c;
      __syncthreads();
    }
#pragma unroll 4
    for (uint32_t i = tid; i < len; i += kSortThreads) {
      const uint64_t ent = src[off + i];
      const uint32_t d = mask - (uint32_t)((ent >> shift) & mask);
      dst[off + atomicAdd(&sh.cnt[d], 1u)] = ent;
    }
    __syncthreads();
    // groups: small ones are ranked and stored, large ones go down a level
    for (uint32_t i = tid; i < len; i += kSortThreads) {
      const uint64_t mine = dst[off + i];
      const uint32_t d = mask - (uint32_t)((mine >> shift) & mask);
      const uint32_t gs = sh.start[d], ge = sh.start[d + 1];
      if (ge - gs <= (uint32_t)kSmallGroup || shift == 0) {
        fin(off + gs + larger_in(dst, off + gs, off + ge, mine), mine);
      } else if (i == gs) {
        const int at = atomicAdd(&sh.stk_top, 1);
        if (at < kStack) {
          sh.stk_off[at] = off + gs;
          sh.stk_len[at] = ge - gs;
          sh.stk_bits[at] = (uint8_t)shift;
          sh.stk_flip[at] = flip ? 0 : 1;
        }
      }
    }
    __syncthreads();
  }
}

// The same for a segment that does not fit LDS (thousands of equal or nearly equal priorities
// among the selected): g0 holds the entries, g1 is the second buffer, both in global memory.
// Ranking small groups out of global memory would cost a CU one load per pair of entries, so only
// the counting-sort levels run there: a level cuts its group by 11 bits (ranking a subgroup costs
// a compare per pair of its members, and all of it is the work of ONE workgroup: short subgroups
// matter), then runs of whole subgroups that fit LDS are loaded and finished there (small
// subgroups ranked, longer ones sorted by sort_segment); a subgroup that still exceeds LDS goes
// down another level.  The level's counters live in the second LDS buffer, which is idle then.
constexpr int kBigStack = 32;
constexpr int kBigBits = 11, kBigBins = 1 << kBigBits;
constexpr int kBigSubgroups = 16;
struct BigShared {
  uint32_t gstart[kBigBins + 1];
  uint32_t off[kBigStack], len[kBigStack];
  uint8_t bits[kBigStack], flip[kBigStack];
  uint8_t ord[kBigStack];  // the group's entries are still in the order they were collected in
  int top;
  int nmid;                  // subgroups of the level that fit LDS but are too long to rank
  uint16_t mid[kBigBins];
  int nbig;                  // subgroups of the level that exceed LDS (a group in index order only)
  uint16_t big[kBigSubgroups];
};
static_assert((kBucketMaxK + kLdsEntries - 1) / kLdsEntries <= kBigSubgroups,
              "every subgroup of a segment that exceeds LDS has a slot");
static_assert(kBigBins * 4 <= kLdsEntries * 8, "the counters fit the second LDS buffer");
static_assert(kBigBins == 2 * kSortThreads, "two counters per thread in the level's scan");

// The entries of src[0, len) for which pred holds go to dst[0, ...) in the order they have in
// src: a wave takes a stretch of src, counts its hits, and once the counts of the waves before
// it are known, copies them -- a lane an entry of every 64, so that loads and stores fall side
// by side.  Returns nothing; wcnt: a word per wave in LDS.  Called by every thread of the workgroup.
template <typename P>
__device__ __forceinline__ void ordered_compact(const uint64_t *src, uint32_t len, uint64_t *dst,
                                                P pred, uint32_t *wcnt) {
  constexpr int kWaves = kSortThreads / kWave;
  constexpr int kLoadsAhead = 8;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t per_wave = (len + kWaves * kWave - 1) / (kWaves * kWave) * kWave;
  const uint32_t w_begin = (uint32_t)wave * per_wave < len ? (uint32_t)wave * per_wave : len;
  const uint32_t w_end = w_begin + per_wave < len ? w_begin + per_wave : len;
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  uint32_t run = 0;
  for (int pass = 0; pass < 2; ++pass) {
    for (uint32_t c0 = w_begin; c0 < w_end; c0 += kWave * kLoadsAhead) {
      uint64_t ent[kLoadsAhead];
#pragma unroll
      for (int u = 0; u < kLoadsAhead; ++u) {
        // (no test around the load; beyond the stretch its last entry, not looked at)
        const uint32_t c = c0 + (uint32_t)u * kWave + lane;
        ent[u] = src[c < w_end ? c : w_end - 1u];
      }
#pragma unroll
      for (int u = 0; u < kLoadsAhead; ++u) {
        const bool hit = c0 + (uint32_t)u * kWave + lane < w_end && pred(ent[u]);
        const uint64_t b = wave_ballot(hit);
        if (pass == 1 && hit) dst[run + (uint32_t)__popcll(b & lt_mask)] = ent[u];
        run += (uint32_t)__popcll(b);
      }
    }
    if (pass == 0) {
      if (lane == 0) wcnt[wave] = run;
      __syncthreads();
      run = (uint32_t)wave_sum((int)(lane < wave ? wcnt[lane] : 0u));
    }
  }
  __syncthreads();
}

// `bits` of the whole segment is already what differing_bits would find (the caller looked at
// the entries when it collected them, in index order).
__device__ __forceinline__ void sort_big_segment(uint64_t *g0, uint64_t *g1, uint32_t m, int bits,
                                                 const SegmentOut &fin, SortShared &sh,
                                                 BigShared &bg, uint64_t *lds_a, uint64_t *lds_b) {
  const int tid = threadIdx.x;
  uint32_t *cnt = reinterpret_cast<uint32_t *>(lds_b);
  constexpr int kInFlight = 8;  // entries a thread has under way in the passes over global memory
  if (tid == 0) {
    bg.off[0] = 0u;
    bg.len[0] = m;
    bg.bits[0] = (uint8_t)bits;
    bg.flip[0] = 0;
    bg.ord[0] = 1;
    bg.top = 1;
  }
  __syncthreads();
  bool first = true;  // the whole segment: its differing bits are known
  while (true) {
    const int top = bg.top;
    if (top == 0) break;
    const uint32_t off = bg.off[top - 1], len = bg.len[top - 1];
    int rem = bg.bits[top - 1];
    const bool flip = bg.flip[top - 1] != 0;
    const bool ordered = bg.ord[top - 1] != 0;
    __syncthreads();
    if (tid == 0) bg.top = top - 1;
    const uint64_t *src = flip ? g1 : g0;
    uint64_t *dst = flip ? g0 : g1;
    if (!first) rem = differing_bits(src, off, len, rem, sh);
    first = false;
    // Entries that differ in their indices only -- equal priorities -- are in place when they
    // are still in index order, as collected.  (The cursors of a level hand out places in the
    // order the waves come by: the order is lost there, except for the subgroups that exceed
    // LDS -- they are few, and they are where thousands of equal priorities end up when other
    // keys share their segment --, which a group in index order hands on in index order.)
    if (rem == 0 || (ordered && rem <= 32)) {
      for (uint32_t i0 = tid; i0 < len; i0 += kSortThreads * kInFlight) {
        uint64_t ent[kInFlight];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) {
          const uint32_t i = i0 + (uint32_t)u * kSortThreads;
          ent[u] = src[off + (i < len ? i : 0u)];
        }
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) {
          const uint32_t i = i0 + (uint32_t)u * kSortThreads;
          if (i < len) fin(off + i, ent[u]);
        }
      }
      __syncthreads();
      continue;
    }
    const int nb = rem < kBigBits ? rem : kBigBits;
    const int shift = rem - nb;
    const uint32_t mask = (1u << nb) - 1u;
    cnt[tid] = 0u;
    cnt[tid + kSortThreads] = 0u;
    __syncthreads();
    for (uint32_t i0 = 0; i0 < len; i0 += kSortThreads * kInFlight) {
      uint64_t ent[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const uint32_t i = i0 + (uint32_t)u * kSortThreads + tid;
        ent[u] = src[off + (i < len ? i : 0u)];  // (no test around the load; not looked at beyond the end)
      }
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const bool valid = i0 + (uint32_t)u * kSortThreads + tid < len;
        count_add(cnt, mask - (uint32_t)((ent[u] >> shift) & mask), valid);
      }
    }
    __syncthreads();
    {
      // exclusive scan of the 2048 counters: thread t owns counters 2t and 2t+1
      const uint32_t c0 = cnt[2 * tid], c1 = cnt[2 * tid + 1];
      const int inc = wave_inclusive_sum((int)(c0 + c1));
      if ((tid & 63) == 63) sh.wsum[tid >> 6] = (uint32_t)inc;
      __syncthreads();
      const int ln = tid & 63;
      const uint32_t before =
          (uint32_t)inc - (c0 + c1) +
          (uint32_t)wave_sum((int)(ln < (tid >> 6) && ln < kSortThreads / kWave ? sh.wsum[ln] : 0u));
      bg.gstart[2 * tid] = before;
      bg.gstart[2 * tid + 1] = before + c0;
      if (tid == kSortThreads - 1) bg.gstart[kBigBins] = before + c0 + c1;
      if (tid == 0) bg.nmid = bg.nbig = 0;
      __syncthreads();
      cnt[2 * tid] = before;  // cursors
      cnt[2 * tid + 1] = before + c0;
      // subgroups that fit LDS but are too long to rank (one entry of the list per digit at most)
      if (shift != 0) {
        if (c0 > (uint32_t)kSmallGroup && c0 <= (uint32_t)kLdsEntries)
          bg.mid[atomicAdd(&bg.nmid, 1)] = (uint16_t)(2 * tid);
        if (c1 > (uint32_t)kSmallGroup && c1 <= (uint32_t)kLdsEntries)
          bg.mid[atomicAdd(&bg.nmid, 1)] = (uint16_t)(2 * tid + 1);
        if (ordered && c0 > (uint32_t)kLdsEntries) bg.big[atomicAdd(&bg.nbig, 1)] = (uint16_t)(2 * tid);
        if (ordered && c1 > (uint32_t)kLdsEntries)
          bg.big[atomicAdd(&bg.nbig, 1)] = (uint16_t)(2 * tid + 1);
      }
      __syncthreads();
    }
    // the subgroups that exceed LDS, in the order the group has them
    const int nbig = bg.nbig;
    for (int qb = 0; qb < nbig; ++qb) {
      const uint32_t b = bg.big[qb];
      ordered_compact(
          src + off, len, dst + off + bg.gstart[b],
          [&](uint64_t e) { return mask - (uint32_t)((e >> shift) & mask) == b; }, sh.wsum);
    }
    for (uint32_t i0 = 0; i0 < len; i0 += kSortThreads * kInFlight) {
      uint64_t ent[kInFlight];
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const uint32_t i = i0 + (uint32_t)u * kSortThreads + tid;
        ent[u] = src[off + (i < len ? i : 0u)];  // (no test around the load; not looked at beyond the end)
      }
#pragma unroll
      for (int u = 0; u < kInFlight; ++u) {
        const uint32_t d = mask - (uint32_t)((ent[u] >> shift) & mask);
        bool valid = i0 + (uint32_t)u * kSortThreads + tid < len;
        for (int qb = 0; qb < nbig; ++qb) valid = valid && d != bg.big[qb];  // (those are in place)
        const uint32_t at = cursor_take(cnt, d, valid);
        if (valid) dst[off + at] = ent[u];
      }
    }
    __syncthreads();
    // runs of whole subgroups that fit LDS
    int d0 = 0;
    while (d0 < kBigBins) {
      const uint32_t cs = bg.gstart[d0];
      int d1 = d0;  // the last d with gstart[d] - cs <= kLdsEntries (binary search: gstart ascends)
      for (int step = kBigBins / 2; step >= 1; step >>= 1)
        if (d1 + step <= kBigBins && bg.gstart[d1 + step] - cs <= (uint32_t)kLdsEntries) d1 += step;
      if (d1 + 1 <= kBigBins && bg.gstart[d1 + 1] - cs <= (uint32_t)kLdsEntries) ++d1;
      if (d1 == d0) {  // subgroup d0 alone exceeds LDS: another level in global memory
        // (at most m / kLdsEntries such groups exist at a time, far fewer than the stack holds;
        // with no bits left to cut by, the entries are equal and stay as they are)
        const int at = bg.top;
        const bool push = shift != 0 && at < kBigStack;
        __syncthreads();
        if (push) {
          if (tid == 0) {
            bg.off[at] = off + cs;
            bg.len[at] = bg.gstart[d0 + 1] - cs;
            bg.bits[at] = (uint8_t)shift;
            bg.flip[at] = flip ? 0 : 1;
            bg.ord[at] = ordered ? 1 : 0;
            bg.top = at + 1;
          }
        } else {
          const uint32_t ge = bg.gstart[d0 + 1];
          for (uint32_t i = cs + tid; i < ge; i += kSortThreads) fin(off + i, dst[off + i]);
        }
        ++d0;
        __syncthreads();
        continue;
      }
      const uint32_t ce = bg.gstart[d1], cn = ce - cs;
      if (cn != 0u) {
        for (uint32_t i = tid; i < cn; i += kSortThreads) lds_a[i] = dst[off + cs + i];
        __syncthreads();
        for (uint32_t i = tid; i < cn; i += kSortThreads) {
          const uint64_t mine = lds_a[i];
          const uint32_t d = mask - (uint32_t)((mine >> shift) & mask);
          const uint32_t gs = bg.gstart[d] - cs, ge = bg.gstart[d + 1] - cs;
          if (ge - gs <= (uint32_t)kSmallGroup || shift == 0)
            fin(off + cs + gs + larger_in(lds_a, gs, ge, mine), mine);
        }
        __syncthreads();
        // the few subgroups too long to rank (listed when the level was cut) are sorted in place
        for (int q = 0; q < bg.nmid; ++q) {
          const int d = bg.mid[q];
          if (d < d0 || d >= d1) continue;
          const uint32_t gs = bg.gstart[d] - cs, sz = bg.gstart[d + 1] - bg.gstart[d];
          sort_segment(lds_a + gs, lds_b, sz, shift, fin.shifted(off + cs + gs), sh);
        }
        __syncthreads();
      }
      d0 = d1;
    }
  }
}

// A segment that exceeds LDS is most often thousands of EQUAL priorities (fresh transitions at the
// maximum priority, integer returns): its entries then only have to go to the output in index
// order, which is the order of the candidate arrays, and the workgroups that own no segment in
// such a call -- its output stretches lie inside the long segment's -- can share that: workgroup
// `slot` of `parts` stores the entries whose place among the segment's lies in its part.  Every
// one of them works out alone whether the keys are equal (one pass over the segment's ids and
// keys: nobody waits for anybody), so they all decide alike.  Returns false, with nothing
// stored, when the keys differ.  Called by every thread of the workgroup.
__device__ __forceinline__ bool store_equal_segment(uint32_t seg_id, uint32_t m, uint32_t slot,
                                                    uint32_t parts, uint32_t kk,
                                                    const uint32_t *__restrict__ ckey,
                                                    const uint32_t *__restrict__ cidx,
                                                    const uint8_t *__restrict__ cseg,
                                                    const SegmentOut &out, SortShared &sh) {
  constexpr int kWaves = kSortThreads / kWave;
  constexpr int kLoadsAhead = 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint8_t seg = (uint8_t)seg_id;
  const uint32_t per_wave = (kk + kWaves * kWave - 1) / (kWaves * kWave) * kWave;
  const uint32_t w_begin = (uint32_t)wave * per_wave < kk ? (uint32_t)wave * per_wave : kk;
  const uint32_t w_end = w_begin + per_wave < kk ? w_begin + per_wave : kk;
  if (tid < 4) sh.bits_or_and[tid] = tid < 2 ? 0u : 0xffffffffu;
  __syncthreads();
  // (bits_or_and[1] is raised by the first wave that sees two keys: the others stop looking)
  volatile uint32_t *differ = &sh.bits_or_and[1];
  uint32_t cnt = 0, k_or = 0u, k_and = 0xffffffffu;
  for (uint32_t c0 = w_begin; c0 < w_end && *differ == 0u; c0 += kWave * kLoadsAhead) {
    uint8_t id[kLoadsAhead];
    uint32_t key[kLoadsAhead];
#pragma unroll
    for (int u = 0; u < kLoadsAhead; ++u) {
      // (no test around the loads; beyond the stretch its last id once more, not looked at)
      const uint32_t c = c0 + (uint32_t)u * kWave + lane;
      const uint32_t at = c < w_end ? c : w_end - 1u;
      id[u] = cseg[at];
      key[u] = ckey[at];
    }
#pragma unroll
    for (int u = 0; u < kLoadsAhead; ++u) {
      const bool hit = c0 + (uint32_t)u * kWave + lane < w_end && id[u] == seg;
      cnt += hit ? 1u : 0u;
      k_or |= hit ? key[u] : 0u;
      k_and &= hit ? key[u] : 0xffffffffu;
    }
    // (a lane's own keys, or two lanes' -- the wave's first hit against every other one)
    const uint64_t has = wave_ballot(cnt != 0u);
    const uint32_t first = (uint32_t)__builtin_amdgcn_readlane((int)k_or, has ? __builtin_ctzll(has) : 0);
    if (wave_ballot(cnt != 0u && (k_or != k_and || k_or != first)) != 0ull && lane == 0) *differ = 1u;
  }
  cnt = (uint32_t)wave_sum((int)cnt);
  for (int d = 32; d >= 1; d >>= 1) {
    k_or |= (uint32_t)__shfl_xor((int)k_or, d, kWave);
    k_and &= (uint32_t)__shfl_xor((int)k_and, d, kWave);
  }
  if (lane == 0) {
    sh.wsum[wave] = cnt;
    atomicOr(&sh.bits_or_and[0], k_or);
    atomicAnd(&sh.bits_or_and[2], k_and);
  }
  __syncthreads();
  const uint32_t key = sh.bits_or_and[0];
  const bool equal = key == sh.bits_or_and[2] && sh.bits_or_and[1] == 0u;
  uint32_t run = (uint32_t)wave_sum((int)(lane < wave ? sh.wsum[lane] : 0u));
  __syncthreads();  // (sh is used again by whoever goes on)
  if (!equal) return false;
  const uint32_t part_lo = (uint32_t)((uint64_t)m * slot / parts);
  const uint32_t part_hi = (uint32_t)((uint64_t)m * (slot + 1u) / parts);
  if (run + cnt <= part_lo || run >= part_hi) return true;  // none of the wave's entries
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  const uint64_t key_part = (uint64_t)(key - out.key_base) << 32;
  for (uint32_t c0 = w_begin; c0 < w_end; c0 += kWave * kLoadsAhead) {
    uint8_t id[kLoadsAhead];
    uint32_t idx[kLoadsAhead];
#pragma unroll
    for (int u = 0; u < kLoadsAhead; ++u) {
      const uint32_t c = c0 + (uint32_t)u * kWave + lane;
      const uint32_t at = c < w_end ? c : w_end - 1u;
      id[u] = cseg[at];
      idx[u] = cidx[at];
    }
#pragma unroll
    for (int u = 0; u < kLoadsAhead; ++u) {
      const bool hit = c0 + (uint32_t)u * kWave + lane < w_end && id[u] == seg;
      const uint64_t b = wave_ballot(hit);
      const uint32_t place = run + (uint32_t)__popcll(b & lt_mask);
      if (hit && place >= part_lo && place < part_hi) out(place, key_part | (uint32_t)~idx[u]);
      run += (uint32_t)__popcll(b);
    }
  }
  return true;
}

__global__ __launch_bounds__(kSortThreads) void segment_sort_kernel(
    const float *__restrict__ p, int64_t n, int64_t k, const State *state,
    const uint32_t *__restrict__ seg_table, const uint32_t *__restrict__ ckey,
    const uint32_t *__restrict__ cidx, const uint8_t *__restrict__ cseg, uint64_t *buf0,
    uint64_t *buf1, float *__restrict__ values_out, int64_t *__restrict__ indices_out) {
  __shared__ uint64_t lds_a[kLdsEntries], lds_b[kLdsEntries];
  __shared__ uint32_t s_cur;
  __shared__ SortShared sh;
  __shared__ BigShared bg;
  const int tid = threadIdx.x, lane = tid & 63;
  // The segment ids of the selected entries (a byte each; every workgroup reads them all) do
  // not depend on what this workgroup owns: their loads go out first, sixteen ids per load.
  const uint32_t kk = (uint32_t)k;
  const uint32_t pattern = blockIdx.x * 0x01010101u;
  constexpr int kLoads = 8;  // covers kBucketMaxK ids
  static_assert((int64_t)kLoads * kSortThreads * 16 >= kBucketMaxK, "one batch of loads reads every id");
  u32x4 q[kLoads];
#pragma unroll
  for (int u = 0; u < kLoads; ++u) {
    const uint32_t i0 = ((uint32_t)u * kSortThreads + tid) * 16;
    q[u] = u32x4{~pattern, ~pattern, ~pattern, ~pattern};  // no byte matches
    if (i0 + 16 <= kk) q[u] = *reinterpret_cast<const u32x4 *>(cseg + i0);
  }
  // this workgroup's segment: its bins (highest + 1, kBins0 - lowest; 0 = none) and its stretch
  // of the output, one load; the entries equal to the threshold are not part of any segment
  u32x4 mine4 = *reinterpret_cast<const u32x4 *>(seg_table + 4 * blockIdx.x);
  const uint32_t need_eq = state->k_rem[2];
  const BinMap map = state->map;
  if (tid == 0) s_cur = 0u;
  // How long a segment's stretch of the output is (0: the workgroup owns none).
  const auto stretch = [&](const u32x4 &e, uint32_t *lo) {
    uint32_t hi = e[3] > kk - need_eq ? kk - need_eq : e[3];
    *lo = ~e[2];
    return (e[0] != 0u && e[1] != 0u && *lo < hi) ? hi - *lo : 0u;
  };
  uint32_t out_lo;
  uint32_t m = stretch(mine4, &out_lo);
  uint32_t seg_id = blockIdx.x, slot = 0u, parts = 1u;
  // The workgroups that own no segment, and the owners of segments that exceed LDS, look at the
  // whole table: which segments are long, which workgroups idle.  The idle ones are dealt out to
  // the long segments (see store_equal_segment).  (The others have no use for it: a barrier and a
  // walk over the table cost them a microsecond.)
  static_assert(kMaxBlocks <= kSortThreads && kMaxBlocks % kWave == 0, "a thread per table entry");
  __shared__ uint64_t s_long[kMaxBlocks / kWave], s_idle[kMaxBlocks / kWave];
  if (m == 0u || m > (uint32_t)kLdsEntries) {
    if (tid < kMaxBlocks) {
      const u32x4 e = *reinterpret_cast<const u32x4 *>(seg_table + 4 * tid);
      uint32_t lo;
      const uint32_t mt = tid < (int)gridDim.x ? stretch(e, &lo) : 0u;
      const uint64_t lm = wave_ballot(mt > (uint32_t)kLdsEntries), im = wave_ballot(mt == 0u);
      if (lane == 0) {
        s_long[tid >> 6] = lm;
        s_idle[tid >> 6] = im;
      }
    }
    __syncthreads();
    uint32_t nlong = 0u, nidle = 0u, long_before = 0u, idle_before = 0u;
#pragma unroll
    for (int w = 0; w < kMaxBlocks / kWave; ++w) {
      const uint64_t lm = s_long[w], im = s_idle[w];
      nlong += (uint32_t)__popcll(lm);
      nidle += (uint32_t)__popcll(im);
      if (w * kWave < (int)blockIdx.x) {
        const int below = (int)blockIdx.x - w * kWave;
        const uint64_t mask = below >= kWave ? ~0ull : ((1ull << below) - 1ull);
        long_before += (uint32_t)__popcll(lm & mask);
        idle_before += (uint32_t)__popcll(im & mask);
      }
    }
    if (m == 0u) {
      if (nlong == 0u) return;
      // the idle workgroup's long segment: number idle_before mod nlong of them
      const uint32_t which = idle_before % nlong;
      slot = 1u + idle_before / nlong;
      uint32_t seen = 0u;
#pragma unroll
      for (int w = 0; w < kMaxBlocks / kWave; ++w) {
        uint64_t lm = s_long[w];
        while (lm != 0ull) {
          const int bit = __builtin_ctzll(lm);
          lm &= lm - 1ull;
          if (seen == which) seg_id = (uint32_t)(w * kWave + bit);
          ++seen;
        }
      }
      long_before = which;
      mine4 = *reinterpret_cast<const u32x4 *>(seg_table + 4 * seg_id);
      m = stretch(mine4, &out_lo);
    }
    if (m > (uint32_t)kLdsEntries)  // the segment's owner and the idle workgroups dealt to it
      parts = 1u + (nidle > long_before ? (nidle - 1u - long_before) / nlong + 1u : 0u);
  }
  const uint32_t hi_bin = mine4[0] - 1u, lo_bin = (uint32_t)kBins0 - mine4[1];
  // keys of the segment lie inside the bins' key range
  const uint32_t lo_key = bin_lo_key(map, lo_bin);
  const uint32_t hi_key = bin_hi_key(map, hi_bin);
  const bool in_lds = m <= (uint32_t)kLdsEntries;
  int big_bits = 0;  // of a segment that does not fit LDS: the low bits in which its entries differ
  if (!in_lds) {
    const SegmentOut whole{p, n, values_out, indices_out, out_lo, lo_key};
    const bool stored = store_equal_segment(seg_id, m, slot, parts, kk, ckey, cidx, cseg, whole, sh);
    if (stored || slot != 0u) return;  // (keys that differ: the owner sorts, alone)
  }
  __syncthreads();

  // One pass over the segment ids, then the segment's entries (key, inverted index) are fetched
  // and kept: in LDS when they fit, else in the segment's stretch of the first global buffer.
  // All of it is bound by the instructions a CU can issue (1024 threads: 100 instructions per
  // thread are 0.8 us), so: the ids of a word are compared without branches (exact zero-byte
  // flags of id ^ own id, gathered into a nibble by a multiplication); the order in which the
  // entries are collected does not matter (they are sorted next), so a thread counts the hits
  // of all its loads and the wave takes its places with ONE scan and one LDS atomic; the
  // fetches of up to eight hits per lane are under way together.
  {
    uint64_t hits[kLoads / 4];  // bit 16 * (u % 4) + e: id e of load u is this segment's
#pragma unroll
    for (int g = 0; g < kLoads / 4; ++g) {
      hits[g] = 0ull;
      if ((uint32_t)g * 4u * kSortThreads * 16u >= kk) continue;  // loads beyond the ids
#pragma unroll
      for (int uu = 0; uu < 4; ++uu) {
        const int u = g * 4 + uu;
        const uint32_t i0 = ((uint32_t)u * kSortThreads + tid) * 16;
        if ((kk & 15u) != 0u && i0 < kk && i0 + 16 > kk) {  // the ragged end: at most one thread
          for (int e = 0; e < 16; ++e)
            if (i0 + e < kk)
              q[u][e >> 2] = (q[u][e >> 2] & ~(0xffu << (8 * (e & 3)))) |
                             ((uint32_t)cseg[i0 + e] << (8 * (e & 3)));
        }
        uint32_t h16 = 0u;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t t = q[u][w] ^ pattern;
          // 0x80 in every byte of t that is zero (exact: no borrow between the bytes)
          const uint32_t z = ~(((t & 0x7f7f7f7fu) + 0x7f7f7f7fu) | t | 0x7f7f7f7fu);
          // bits 7, 15, 23, 31 -> bits 0..3
          h16 |= ((((z >> 7) * 0x00204081u) >> 21) & 0xfu) << (4 * w);
        }
        hits[g] |= (uint64_t)h16 << (16 * uu);
      }
    }
    int nc = 0;
#pragma unroll
    for (int g = 0; g < kLoads / 4; ++g) nc += __popcll(hits[g]);
    if (in_lds && wave_ballot(nc != 0) != 0ull) {
      const int inc = wave_inclusive_sum(nc);
      uint32_t base = 0;
      if (lane == kWave - 1) base = atomicAdd(&s_cur, (uint32_t)inc);
      base = (uint32_t)__builtin_amdgcn_readlane((int)base, kWave - 1) + (uint32_t)(inc - nc);
      {  // (the entries' order in LDS does not matter: they are sorted next)
#pragma unroll
        for (int g = 0; g < kLoads / 4; ++g) {
          uint64_t h = hits[g];
          while (wave_ballot(h != 0ull) != 0ull) {
            constexpr int kFetch = 8;
            uint32_t pos[kFetch], key[kFetch], idx[kFetch];
#pragma unroll
            for (int f = 0; f < kFetch; ++f) {
              pos[f] = kk;
              if (h != 0ull) {
                const int bit = __builtin_ctzll(h);
                h &= h - 1ull;
                pos[f] = ((uint32_t)(g * 4 + (bit >> 4)) * kSortThreads + tid) * 16 + (uint32_t)(bit & 15);
              }
            }
#pragma unroll
            for (int f = 0; f < kFetch; ++f) {
              // (no test around the loads -- the compiler would wait for each one where the paths
              // meet --: a slot without a hit loads the first entry and does not look at it)
              const uint32_t at = pos[f] < kk ? pos[f] : 0u;
              key[f] = ckey[at];
              idx[f] = cidx[at];
            }
#pragma unroll
            for (int f = 0; f < kFetch; ++f) {
              if (pos[f] < kk) {
                if (base < m) lds_a[base] = ((uint64_t)(key[f] - lo_key) << 32) | (uint32_t)~idx[f];
                ++base;
              }
            }
          }
        }
      }
    }
  }
  __syncthreads();
  if (!in_lds) {
    // A long segment (thousands of equal priorities, or a crowd in a narrow range): most ids are
    // hits.  A wave takes a stretch of the ids, a lane an id of every 64: the loads of the keys
    // and indices and the stores of the entries fall side by side, and the entries end up in the
    // order of the candidate arrays -- index order --, which lets a segment of equal priorities
    // go to the output as it is.
    constexpr int kWaves = kSortThreads / kWave;
    __shared__ uint32_t s_wcnt[kWaves];
    const int wave = tid >> 6;
    const uint8_t seg = (uint8_t)blockIdx.x;
    const uint32_t per_wave = (kk + kWaves * kWave - 1) / (kWaves * kWave) * kWave;
    const uint32_t w_begin = (uint32_t)wave * per_wave < kk ? (uint32_t)wave * per_wave : kk;
    const uint32_t w_end = w_begin + per_wave < kk ? w_begin + per_wave : kk;
    // how many of the wave's ids are hits: sixteen ids per load, the zero bytes of id ^ own id
    uint32_t cnt = 0;
    for (uint32_t c = w_begin + (uint32_t)lane * 16u; c < w_end; c += kWave * 16u) {
      if (c + 16u <= w_end) {
        const u32x4 ids = *reinterpret_cast<const u32x4 *>(cseg + c);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t t = ids[w] ^ pattern;
          cnt += (uint32_t)__popc(~(((t & 0x7f7f7f7fu) + 0x7f7f7f7fu) | t | 0x7f7f7f7fu));
        }
      } else {
        for (uint32_t e = c; e < w_end; ++e) cnt += cseg[e] == seg ? 1u : 0u;
      }
    }
    cnt = (uint32_t)wave_sum((int)cnt);
    if (lane == 0) s_wcnt[wave] = cnt;
    __syncthreads();
    uint32_t run = (uint32_t)wave_sum((int)(lane < wave ? s_wcnt[lane] : 0u));
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    constexpr int kGathers = 16;
    uint64_t bits_or = 0ull, bits_and = ~0ull;  // of the entries: which bits differ among them
    for (uint32_t c0 = w_begin; c0 < w_end; c0 += kWave * kGathers) {
      uint32_t key[kGathers], idx[kGathers];
      uint8_t id[kGathers];
#pragma unroll
      for (int u = 0; u < kGathers; ++u) {
        // (loads without a test around them, see above: beyond the stretch's end its last id
        // is loaded once more and not looked at)
        const uint32_t c = c0 + (uint32_t)u * kWave + lane;
        const uint32_t at = c < w_end ? c : w_end - 1u;
        id[u] = cseg[at];
        key[u] = ckey[at];
        idx[u] = cidx[at];
      }
#pragma unroll
      for (int u = 0; u < kGathers; ++u) {
        const bool hit = c0 + (uint32_t)u * kWave + lane < w_end && id[u] == seg;
        const uint64_t b = wave_ballot(hit);
        const uint32_t place = run + (uint32_t)__popcll(b & lt_mask);
        if (hit && place < m) {
          const uint64_t ent = ((uint64_t)(key[u] - lo_key) << 32) | (uint32_t)~idx[u];
          buf0[out_lo + place] = ent;
          bits_or |= ent;
          bits_and &= ent;
        }
        run += (uint32_t)__popcll(b);
      }
    }
    big_bits = differing_bits_of(bits_or, bits_and, 64, sh);  // (ends with a barrier)
  }

  // An entry holds its key as the distance from the segment's smallest possible key: the bits
  // in which entries can differ are the index and as many bits as that distance takes for the
  // largest key, and the digits of the sort cut the key range evenly wherever it lies (the bits
  // in which the smallest and the largest key themselves differ would be all 24 of them for a
  // range around a power of two, with every entry in one of two digits).
  const int bits = 32 + bits_of(hi_key - lo_key);
  // the sorted entries go straight to the segment's stretch of values and indices
  const SegmentOut out{p, n, values_out, indices_out, out_lo, lo_key};
  if (in_lds)
    sort_segment(lds_a, lds_b, m, bits, out, sh);
  else
    sort_big_segment(buf0 + out_lo, buf1 + out_lo, m, big_bits < bits ? big_bits : bits, out, sh, bg,
                     lds_a, lds_b);
}
static_assert(kSortThreads >= kSortBins, "a thread per digit in the segment sort's scan");

// Final store of the value-ordered form for k > kBucketMaxK, fused into the last digit of the
// candidate sort.
struct EmitSorted {
  static constexpr bool kActive = true;
  const float *p;
  float *values;
  int64_t *indices;
  uint32_t n;
  __device__ __forceinline__ void operator()(uint32_t pos, uint32_t, uint32_t index) const {
    // index < n always holds for valid input; with NaN priorities fewer than k candidates are
    // written and the rest of the candidate arrays is whatever the workspace held
    indices[pos] = (int64_t)index;
    if (values) values[pos] = index < n ? p[index] : 0.0f;
  }
};

}  // namespace
}  // namespace gearhip

using namespace gearhip;

extern "C" size_t gear_hip_topk_workspace_bytes(int64_t n, int64_t k) { return layout(n, k).total; }

namespace gearhip {
namespace {
int topk_launch(const float *priorities, int64_t n, int64_t k, int sorted_by_value, int warm,
                float *values_out, int64_t *indices_out, void *workspace, size_t workspace_bytes,
                void *stream) {
  if (n < 0 || k < 0) return GEAR_HIP_EINVAL;
  if (k == 0) return 0;
  if (k > n || !priorities || !indices_out) return GEAR_HIP_EINVAL;
  if (n >= (1ll << 31)) return GEAR_HIP_ERANGE;
  if (reinterpret_cast<uintptr_t>(priorities) & 3) return GEAR_HIP_EALIGN;
  const Layout l = layout(n, k);
  if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 255))
    return GEAR_HIP_EWORKSPACE;
  char *ws = static_cast<char *>(workspace);
  State *state = reinterpret_cast<State *>(ws);
  uint32_t *hist0 = reinterpret_cast<uint32_t *>(ws + l.hist0);
  uint32_t *hist1 = reinterpret_cast<uint32_t *>(ws + l.hist1);
  uint32_t *hist2 = reinterpret_cast<uint32_t *>(ws + l.hist2);
  uint32_t *histf1 = reinterpret_cast<uint32_t *>(ws + l.histf1);
  uint32_t *histf2 = reinterpret_cast<uint32_t *>(ws + l.histf2);
  uint32_t *boff = reinterpret_cast<uint32_t *>(ws + l.boff);
  uint32_t *wave_listed = reinterpret_cast<uint32_t *>(ws + l.wave_listed);
  uint64_t *wave_ge = reinterpret_cast<uint64_t *>(ws + l.wave_ge);
  uint64_t *block_ge = reinterpret_cast<uint64_t *>(ws + l.block_ge);
  uint64_t *lists = reinterpret_cast<uint64_t *>(ws + l.lists);
  uint32_t *cidx = reinterpret_cast<uint32_t *>(ws + l.cidx);
  hipStream_t st = as_stream(stream);
  const Geom g = geom(n, k);

  // The hint: rank of the sample that safely lies below the k-th largest priority -- the sample's
  // expected share of k plus six standard deviations and a little.  No sample when the input is
  // small or when k is a large part of it (the lists would hold most of the input: the levels
  // stream instead).  (Lists that hold whole ranges cannot overflow; with a sample they hold the
  // candidates only, and the launches after level 0 walk a tenth of the input instead of all.)
  const int list_all = g.list_cap >= g.wave_len ? 1 : 0;
  uint32_t rank = 0;
  // Samples per thread: the fewest with which the entries above the hint fit a wave's list with
  // six standard deviations to spare (a small sample of a long input gives a loose bound: the
  // rank below cannot go under ~9, whatever the sample's share of k).  No sample at all when even
  // the largest one would overflow the lists: the levels then stream the input anyway.
  const auto hint_rank = [&](int per) {
    const double samples = (double)per * kThreads;
    const double mu = samples * (double)k / (double)n;
    return mu + 6.0 * __builtin_sqrt(mu) + 8.0;
  };
  const int cap_used = g.list_cap < kQueueCap ? (int)g.list_cap : kQueueCap;
  const auto lists_hold = [&](int per) {
    // (the hint is rounded down to a boundary of the coarse bins, up to an eighth of an octave
    // lower: half as many entries again, and a little, lie above it)
    const double e = 1.6 * hint_rank(per) / ((double)per * kThreads) * (double)g.wave_len;
    return e + 6.0 * __builtin_sqrt(e) <= (double)cap_used;
  };
  int per = 2;
  while (per < kMaxSamplesPerThread && !lists_hold(per)) per *= 4;
  while (per > 2 && n < 128 * (int64_t)per * kThreads) per /= 4;  // strides of 128 elements or more
  if ((list_all || lists_hold(per)) && n >= 128 * (int64_t)per * kThreads && k <= n / 8 &&
      env_int("GEAR_HIP_TOPK_HINT", 1) != 0) {
    const double r = hint_rank(per);
    if (r < (double)per * kThreads / 4) rank = (uint32_t)r + 1u;
  }
  const int64_t zero_words = (int64_t)((l.zero_end - l.zero_begin) / 4);
  const unsigned zero_blocks = (unsigned)ceil_div64(zero_words, (int64_t)kThreads * 4);
  const dim3 block(kThreads), grid((unsigned)g.blocks);
  // Finer bins pay off in the value-order sort (small, even segments) but cost level 0 more
  // cache lines to add its counts to; the index-ordered selection takes coarse ones.
  const int mid_bins = (sorted_by_value && k <= kBucketMaxK) ? kMidBins : kMidBinsCoarse;
  {
    uint32_t *zero = reinterpret_cast<uint32_t *>(ws + l.zero_begin);
    const dim3 pgrid(1 + zero_blocks);
    if (per == 2)
      prep_kernel<2><<<pgrid, block, 0, st>>>(priorities, n, k, rank, list_all, mid_bins, warm, state,
                                              zero, zero_words);
    else if (per == 8)
      prep_kernel<8><<<pgrid, block, 0, st>>>(priorities, n, k, rank, list_all, mid_bins, warm, state,
                                              zero, zero_words);
    else
      prep_kernel<32><<<pgrid, block, 0, st>>>(priorities, n, k, rank, list_all, mid_bins, warm, state,
                                               zero, zero_words);
  }
  if (rank != 0u)
    level0_hinted_kernel<<<grid, block, 0, st>>>(priorities, n, state, hist0, g.wave_len,
                                                 wave_listed, lists, (int)g.list_cap);
  else
    level0_kernel<<<grid, block, 0, st>>>(priorities, n, state, hist0, g.wave_len, wave_listed,
                                          lists, (int)g.list_cap);
  // value order by segments: workgroup w of the sort owns the bins that start in the output
  // places [w << seg_shift, (w + 1) << seg_shift)
  const bool by_segments = sorted_by_value && k <= kBucketMaxK;
  int seg_shift = 0;
  while ((k >> seg_shift) >= kNoSegment) ++seg_shift;  // segment ids stay below kNoSegment
  uint32_t *wg_bins = reinterpret_cast<uint32_t *>(ws + l.wg_bins);
  member_hist_kernel<1><<<grid, block, 0, st>>>(priorities, n, k, mid_bins, state, hist0, hist1,
                                                nullptr, histf1, by_segments ? boff : nullptr,
                                                wg_bins, seg_shift, g.wave_len, wave_listed, lists,
                                                (int)g.list_cap);
  member_hist_kernel<2><<<grid, block, 0, st>>>(priorities, n, k, mid_bins, state, hist1, hist2,
                                                histf1, histf2, nullptr, nullptr, 0, g.wave_len,
                                                wave_listed, lists, (int)g.list_cap);
  count_kernel<<<grid, block, 0, st>>>(priorities, n, state, hist2, histf2, g.wave_len,
                                       wave_listed, lists, (int)g.list_cap, wave_ge, block_ge);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  uint8_t *cseg = reinterpret_cast<uint8_t *>(ws + l.cseg);
#define GEARHIP_WRITE(F, CKEY)                                                                     \
  write_kernel<F><<<grid, block, 0, st>>>(priorities, n, k, state, g.wave_len, wave_listed, lists,  \
                                          (int)g.list_cap, wave_ge, block_ge, CKEY, cidx, boff,     \
                                          seg_shift, cseg, values_out, indices_out)
  if (!sorted_by_value) {
    GEARHIP_WRITE(kDirect, nullptr);
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  if (k <= kBucketMaxK) {
    uint64_t *cand = reinterpret_cast<uint64_t *>(ws + l.cand);
    uint64_t *cand2 = reinterpret_cast<uint64_t *>(ws + l.cand2);
    uint32_t *bkey = reinterpret_cast<uint32_t *>(ws + l.ckey);
    GEARHIP_WRITE(kBucket, bkey);
    segment_sort_kernel<<<dim3(kMaxBlocks), dim3(kSortThreads), 0, st>>>(
        priorities, n, k, state, wg_bins, bkey, cidx, cseg, cand, cand2, values_out, indices_out);
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  uint32_t *ckey = reinterpret_cast<uint32_t *>(ws + l.ckey);
  GEARHIP_WRITE(kPairs, ckey);
#undef GEARHIP_WRITE
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  uint32_t *skey = reinterpret_cast<uint32_t *>(ws + l.skey);
  uint32_t *sidx = reinterpret_cast<uint32_t *>(ws + l.sidx);
  uint32_t *tkey = reinterpret_cast<uint32_t *>(ws + l.tkey);
  uint32_t *tidx = reinterpret_cast<uint32_t *>(ws + l.tidx);
  uint32_t *shist = reinterpret_cast<uint32_t *>(ws + l.shist);
  // the last digit's scatter writes values_out / indices_out itself
  const EmitSorted fin{priorities, values_out, indices_out, (uint32_t)n};
  return radix::sort_pairs<uint32_t, uint32_t, EmitSorted>(ckey, skey, cidx, sidx, tkey, tidx, k, 0,
                                                           32, shist, st, fin);
}
}  // namespace
}  // namespace gearhip

extern "C" int gear_hip_topk_f32(const float *priorities, int64_t n, int64_t k,
                                 int sorted_by_value, float *values_out, int64_t *indices_out,
                                 void *workspace, size_t workspace_bytes, void *stream) {
  return topk_launch(priorities, n, k, sorted_by_value, 0, values_out, indices_out, workspace,
                     workspace_bytes, stream);
}

extern "C" int gear_hip_topk_f32_warm(const float *priorities, int64_t n, int64_t k,
                                      int sorted_by_value, float *values_out,
                                      int64_t *indices_out, void *workspace,
                                      size_t workspace_bytes, void *stream) {
  return topk_launch(priorities, n, k, sorted_by_value, 1, values_out, indices_out, workspace,
                     workspace_bytes, stream);
}
