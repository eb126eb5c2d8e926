// Inclusive prefix sums and a deterministic sum, gfx950.  fp32 inputs are accumulated in fp64.
//
// The range kernels work on blocked ranges: thread t of a workgroup owns G consecutive 16-byte
// granules of its range, adds them up in order, and one DPP wave scan per range joins the
// threads (a wave-private LDS row turns the row-major order of the memory instructions, 1 KiB of
// consecutive addresses per wave and instruction, into that blocked order and back):
//  * chained single pass, up to 4096 ranges (of up to 16384 fp32 elements: 67 M):
//    scan_ranges_kernel<kChained>.  A workgroup
//    keeps its range in registers, publishes the range's sum and adds the sums of ALL earlier
//    ranges (fixed order: bit-reproducible), then writes the prefix: the input is read once.
//    Range r belongs to workgroup r (no ticket).  A published sum travels as three 64-bit words
//    that each carry 42 bits of the call's tag next to 21 or 22 bits of payload, so a word is valid
//    on its own: no fence, no flag, nothing to clear before a call (a host counter hands every
//    call a fresh tag; what an earlier call or an uninitialised workspace left never matches).
//    The wait for a predecessor is bounded: when it runs out, the workgroup sums that
//    predecessor's range itself, with the same reduction tree, and publishes it on the
//    predecessor's behalf, so no kernel can spin forever and the result does not change.
//  * two launches, up to 16384 ranges (n <= 134 M fp32): range_sum_kernel writes the sum of every
//    range; scan_ranges_kernel<kTwoLaunches> re-reads its range (now in L2 / MALL), adds the
//    sums of all earlier ranges and writes the prefix.  No workgroup waits for another one.  Used
//    for long inputs, under stream capture (a captured launch would replay its tag) and for the
//    incremental rescan of a suffix.
//  * beyond that: three launches -- range_sum_kernel, range_prefix_kernel (ONE workgroup scans the
//    range sums in a fixed order) and scan_ranges_kernel<kPrefixed>, which finds the sum of all
//    earlier ranges in one word.  Same bits on every run, and for the rescan of a suffix.
#include <atomic>
#include <chrono>
#include <mutex>
#include <random>
#include <type_traits>

#include "wave.hpp"

namespace gearhip {
namespace {

constexpr int kBlock = 256;
constexpr int kMinRange = 2048;  // elements of the smallest range (fp32, 2 granules per thread)
constexpr size_t kHeaderBytes = 256;

template <typename Acc> struct Bits;
template <> struct Bits<double> {
  static __device__ __forceinline__ uint64_t to(double v) { return (uint64_t)__double_as_longlong(v); }
  static __device__ __forceinline__ double from(uint64_t b) { return __longlong_as_double((long long)b); }
};
template <> struct Bits<int64_t> {
  static __device__ __forceinline__ uint64_t to(int64_t v) { return (uint64_t)v; }
  static __device__ __forceinline__ int64_t from(uint64_t b) { return (int64_t)b; }
};

// Results that fit the caches are stored normally (the search that follows reads them back);
// larger ones stream past the caches with non-temporal stores.
template <typename V>
__device__ __forceinline__ void store_vec(V *p, V v, bool nt) {
  if (nt)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}

// ---- range variant -------------------------------------------------------------------------------
// A workgroup owns NR rows of 256 vectors kept in registers and takes its exclusive prefix as the
// sum of ALL earlier ranges' sums (each thread adds its share of them, fixed summation order).
// Nobody waits for an inclusive value, so there is no serial chain across the XCDs, and the result
// is bit-reproducible from run to run.
constexpr int kMaxRanges = 4096;      // chained: every thread polls up to 16 range sums
constexpr int kMaxRangesTwo = 16384;  // two launches: every thread adds up to 64 range sums

// A range sum in flight between workgroups of one launch: three self-validating words.
constexpr int kTagBits = 42;
constexpr uint64_t kTagMask = (1ull << kTagBits) - 1ull;
struct Slot {
  uint64_t w[3];
};
__device__ __forceinline__ void publish(Slot *s, uint64_t tag, uint64_t v) {
  store_agent(&s->w[0], (tag << 22) | (v & 0x3fffffull));
  store_agent(&s->w[1], (tag << 22) | ((v >> 22) & 0x1fffffull));
  store_agent(&s->w[2], (tag << 22) | (v >> 43));
}
__device__ __forceinline__ bool try_read(const Slot *s, uint64_t tag, uint64_t *v) {
  const uint64_t a = load_agent(&s->w[0]), b = load_agent(&s->w[1]), c = load_agent(&s->w[2]);
  *v = (a & 0x3fffffull) | ((b & 0x1fffffull) << 22) | ((c & 0x1fffffull) << 43);
  return (a >> 22) == tag && (b >> 22) == tag && (c >> 22) == tag;
}

// ---- blocked ranges -------------------------------------------------------------------------------
// A range is 256 threads x G granules of 16 bytes; thread t owns the G consecutive granules
// [t*G, t*G + G) of its range (EPT = G * 16 / sizeof(In) consecutive elements), so that one serial
// pass over registers and ONE wave scan per range replace a wave scan per row.  Global loads and
// stores stay contiguous per instruction (1 KiB per wave): a wave-private LDS row turns the
// row-major order of the memory instructions into the blocked order of the arithmetic and back.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <typename T> struct Gran {  // one 16-byte granule of T
  static constexpr int kN = 16 / (int)sizeof(T);
  typedef T type __attribute__((ext_vector_type(kN)));
  typedef T loose __attribute__((ext_vector_type(kN), aligned(sizeof(T))));
};

template <typename In, typename Out, int G> struct Geo {
  static constexpr int kVE = Gran<In>::kN;
  static constexpr int kEPT = G * kVE;                       // elements per thread
  static constexpr int kRange = kBlock * kEPT;               // elements per range
  static constexpr int kWaveElems = kWave * kEPT;
  static constexpr int kOE = Gran<Out>::kN;
  static constexpr int kOG = kEPT / kOE;                     // result granules per thread
  static constexpr int kPiece = kOG <= G ? kWave : kWave * G / kOG;  // lanes per store piece
  static constexpr int kPitchIn = G + 1, kPitchOut = kOG + 1;  // odd pitches: no bank conflicts
  static constexpr int kStage = kWave * kPitchIn;            // granules of LDS per wave
  static_assert(kPiece * kPitchOut <= kStage, "result piece fits the staging row");
  static_assert((G & (G - 1)) == 0 && (kOG & (kOG - 1)) == 0, "powers of two");
};

// The wave's kWaveElems elements starting at wbase, in blocked order: f[] of lane l holds elements
// [wbase + l*EPT, wbase + (l+1)*EPT); elements at or beyond n read as 0.
// Inputs of up to 64 MB are loaded normally: priorities are read again and again (by the next
// scan, by the top-k before it) and such an array stays in the 256 MB memory-side cache; longer
// ones stream past the caches with non-temporal loads.
__host__ __device__ __forceinline__ bool streams_in(int64_t n, size_t elem) {
  return n * (int64_t)elem > (64ll << 20);
}

template <typename In, typename Out, int G>
__device__ __forceinline__ void load_blocked(const In *__restrict__ in, int64_t n, int64_t wbase,
                                             u32x4 *stage, int lane,
                                             In (&f)[Geo<In, Out, G>::kEPT]) {
  typedef Geo<In, Out, G> geo;
  typedef typename Gran<In>::loose in_vec;
  typedef typename Gran<In>::type in_gran;
  if (wbase + geo::kWaveElems <= n) {
    in_vec v[G];
    const in_vec *src = reinterpret_cast<const in_vec *>(in + wbase + (int64_t)lane * geo::kVE);
    if (streams_in(n, sizeof(In))) {
#pragma unroll
      for (int r = 0; r < G; ++r) v[r] = __builtin_nontemporal_load(src + r * kWave);
    } else {
#pragma unroll
      for (int r = 0; r < G; ++r) v[r] = src[r * kWave];
    }
#pragma unroll
    for (int r = 0; r < G; ++r) {
      const int g = r * kWave + lane;
      in_gran q;
#pragma unroll
      for (int k = 0; k < geo::kVE; ++k) q[k] = v[r][k];
      stage[(g / G) * geo::kPitchIn + (g % G)] = __builtin_bit_cast(u32x4, q);
    }
  } else {
#pragma unroll
    for (int r = 0; r < G; ++r) {
      const int g = r * kWave + lane;
      const int64_t e0 = wbase + (int64_t)g * geo::kVE;
      in_gran q;
#pragma unroll
      for (int k = 0; k < geo::kVE; ++k) q[k] = (e0 + k < n) ? in[e0 + k] : (In)0;
      stage[(g / G) * geo::kPitchIn + (g % G)] = __builtin_bit_cast(u32x4, q);
    }
  }
  wave_lds_sync();
#pragma unroll
  for (int j = 0; j < G; ++j) {
    const in_gran q = __builtin_bit_cast(in_gran, stage[lane * geo::kPitchIn + j]);
#pragma unroll
    for (int k = 0; k < geo::kVE; ++k) f[j * geo::kVE + k] = q[k];
  }
  wave_lds_sync();
}

// Sum of a thread's elements in order, then the wave's inclusive scan of those sums.
template <typename In, typename Acc, int EPT>
__device__ __forceinline__ Acc thread_total(const In (&f)[EPT]) {
  Acc t = (Acc)f[0];
#pragma unroll
  for (int e = 1; e < EPT; ++e) t += (Acc)f[e];
  return t;
}

// The sum of one range with the reduction tree every kernel here uses for it (thread: its
// elements in order; wave: the DPP scan's last lane; workgroup: (w0 + w1) + (w2 + w3)), returned
// to every thread.  `red` is LDS for the four wave sums; the caller separates calls with a barrier.
template <typename In, typename Acc, typename Out, int G>
__device__ __forceinline__ Acc range_total(const In *__restrict__ in, int64_t n, int64_t range,
                                           u32x4 *stage, Acc *red) {
  typedef Geo<In, Out, G> geo;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  In f[geo::kEPT];
  load_blocked<In, Out, G>(in, n, range * geo::kRange + (int64_t)wave * geo::kWaveElems, stage, lane,
                           f);
  const Acc inc = wave_inclusive_sum(thread_total<In, Acc, geo::kEPT>(f));
  if (lane == kWave - 1) red[wave] = inc;
  __syncthreads();
  const Acc total = (red[0] + red[1]) + (red[2] + red[3]);
  __syncthreads();
  return total;
}

// The same sum with the same tree, read straight from memory (a lane's elements are consecutive,
// so its loads do not share lines with its neighbours': slow, and light on registers).  For the
// rare workgroup that has to add up a predecessor's range while its own is in registers.
template <typename In, typename Acc, typename Out, int G>
__device__ __noinline__ Acc range_total_direct(const In *__restrict__ in, int64_t n, int64_t range,
                                               Acc *red) {
  typedef Geo<In, Out, G> geo;
  typedef typename Gran<In>::loose in_vec;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  const int64_t e0 = range * geo::kRange + (int64_t)tid * geo::kEPT;
  Acc t = (Acc)0;
#pragma unroll 1
  for (int j = 0; j < G; ++j) {
    const int64_t e = e0 + (int64_t)j * geo::kVE;
    In q[geo::kVE];
    if (e + geo::kVE <= n) {
      const in_vec v = *reinterpret_cast<const in_vec *>(in + e);
#pragma unroll
      for (int k = 0; k < geo::kVE; ++k) q[k] = v[k];
    } else {
#pragma unroll
      for (int k = 0; k < geo::kVE; ++k) q[k] = (e + k < n) ? in[e + k] : (In)0;
    }
#pragma unroll
    for (int k = 0; k < geo::kVE; ++k) t = (j == 0 && k == 0) ? (Acc)q[0] : t + (Acc)q[k];
  }
  const Acc inc = wave_inclusive_sum(t);
  if (lane == kWave - 1) red[wave] = inc;
  __syncthreads();
  const Acc total = (red[0] + red[1]) + (red[2] + red[3]);
  __syncthreads();
  return total;
}

// Sum of every range, one workgroup per range: the first launch of the two-launch variant, in
// which the scan launch below finds all sums ready (no publishing, no polling).
template <typename In, typename Acc, typename Out, int G>
__global__ __launch_bounds__(kBlock) void range_sum_kernel(const In *__restrict__ in, int64_t n,
                                                           uint64_t *__restrict__ sums,
                                                           int64_t first_range) {
  __shared__ u32x4 stage[kBlock / kWave][Geo<In, Out, G>::kStage];
  __shared__ Acc red[kBlock / kWave];
  const int64_t range = first_range + blockIdx.x;
  const Acc total = range_total<In, Acc, Out, G>(in, n, range, stage[threadIdx.x >> 6], red);
  if (threadIdx.x == 0) sums[range] = Bits<Acc>::to(total);
}

// Exclusive prefix of the range sums by ONE workgroup, in an order that depends on nothing but
// the number of ranges (thread t adds its stretch of the sums one after the other, the stretches'
// totals are scanned, the stretch is walked again): the third launch between the two above for
// inputs of more ranges than a workgroup can add up by itself.
constexpr int kPrefixThreads = 1024;
template <typename Acc>
__global__ __launch_bounds__(kPrefixThreads) void range_prefix_kernel(
    const uint64_t *__restrict__ sums, uint64_t *__restrict__ prefix, int64_t ranges) {
  __shared__ Acc wtot[kPrefixThreads / kWave];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  const int64_t per = ceil_div64(ranges, kPrefixThreads);
  const int64_t lo = (int64_t)tid * per, hi = lo + per < ranges ? lo + per : ranges;
  Acc mine = (Acc)0;
  for (int64_t i = lo; i < hi; ++i) mine += Bits<Acc>::from(sums[i]);
  const Acc inc = wave_inclusive_sum(mine);
  if (lane == kWave - 1) wtot[wave] = inc;
  __syncthreads();
  Acc run = (Acc)0;
  for (int w = 0; w < wave; ++w) run += wtot[w];
  run += wave_shift_up1(inc);
  for (int64_t i = lo; i < hi; ++i) {
    prefix[i] = Bits<Acc>::to(run);
    run += Bits<Acc>::from(sums[i]);
  }
}

// sums[r]   plain range sums (kept between calls: the incremental rescan reuses the ones before
//           its first range)
// slots[r]  chained: the same sums as tagged words, for the workgroups of this launch; prefixed:
//           8-byte words, the sum of all ranges before r
// spin_limit  chained only: polls of a missing predecessor before the workgroup sums that range
//           itself
enum RangeMode {
  kTwoLaunches = 0,  // every workgroup adds up the sums of the ranges before its own
  kChained = 1,      // ... and the sums of this launch's ranges arrive while it runs
  kPrefixed = 2      // the sum of all earlier ranges is ready: slots holds one word per range
};
template <typename In, typename Acc, typename Out, int G, int MODE>
__global__ __launch_bounds__(kBlock) void scan_ranges_kernel(const In *__restrict__ in,
                                                             Out *__restrict__ out, int64_t n,
                                                             uint64_t *__restrict__ sums,
                                                             Slot *__restrict__ slots,
                                                             int64_t first_range, uint64_t tag,
                                                             int spin_limit, int stagger,
                                                             int first_wave) {
  typedef Geo<In, Out, G> geo;
  typedef typename Gran<Out>::type out_gran;
  constexpr bool CHAINED = MODE == kChained;
  constexpr int kWaves = kBlock / kWave;
  constexpr int kPolls = MODE == kPrefixed ? 0 : (CHAINED ? kMaxRanges : kMaxRangesTwo) / kBlock;
  constexpr int kBatch = 4;
  __shared__ u32x4 stage_all[kWaves][geo::kStage];
  __shared__ Acc wtot[kWaves];
  __shared__ Acc red[kWaves];
  __shared__ uint32_t s_missing[CHAINED ? kMaxRanges / 32 : 1];  // one bit per unpublished range

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  const int64_t tile = first_range + (int64_t)blockIdx.x;
  const int64_t wbase = tile * geo::kRange + (int64_t)wave * geo::kWaveElems;
  u32x4 *stage = stage_all[wave];

  if (CHAINED) {
    if (tid < kMaxRanges / 32) s_missing[tid] = 0u;
    // All workgroups that fit the GPU at once start within a microsecond.  Left alone, their loads
    // queue up together and come back in no particular order, every workgroup then waits for the
    // slowest load of ALL its predecessors, and the whole GPU first reads and then writes.  Starting
    // workgroup r a little later than r-1 (stagger/1024 clock ticks apiece, the pace at which
    // memory delivers ranges anyway) makes the ranges arrive in order: early ranges are being
    // written while late ones are still being read.  The wait is bounded by first_wave * stagger.
    if (stagger > 0 && blockIdx.x < (unsigned)first_wave) {
      const unsigned long long until = (unsigned long long)wall_clock64() +
                                       (((unsigned long long)blockIdx.x * (unsigned)stagger) >> 10);
      while ((unsigned long long)wall_clock64() < until) __builtin_amdgcn_s_sleep(1);
    }
  }
  In f[geo::kEPT];
  load_blocked<In, Out, G>(in, n, wbase, stage, lane, f);
  const Acc inc = wave_inclusive_sum(thread_total<In, Acc, geo::kEPT>(f));
  const Acc wexcl = wave_shift_up1(inc);
  if (lane == kWave - 1) wtot[wave] = inc;
  __syncthreads();
  const Acc w0 = wtot[0], w1 = wtot[1], w2 = wtot[2], w3 = wtot[3];
  // the range's sum goes out first
  if (CHAINED && tid == 0) {
    const uint64_t bits = Bits<Acc>::to((w0 + w1) + (w2 + w3));
    publish(&slots[tile], tag, bits);
    sums[tile] = bits;
  }
  // Sum of every earlier range: thread t adds ranges t, t+256, ... in that order.  The ones
  // before this launch's first range are plain words from an earlier call, the others are
  // published by the workgroups of this launch.  They are read kBatch at a time (all polls of a
  // batch are issued together, only the unpublished ones are repeated).  What is still missing
  // after the bounded wait is summed by this workgroup from the input, with the tree its own
  // workgroup uses, and published on its behalf (same bits): the kernel ends whatever the others
  // do, and the next pass over the words finds everything.
  Acc part = (Acc)0;
  bool failed = CHAINED;
  for (int attempt = 0; attempt < (CHAINED ? 3 : 1); ++attempt) {
    part = (Acc)0;
    bool miss = false;
#pragma unroll 1
    for (int b = 0; b < kPolls; b += kBatch) {
      if ((int64_t)b * kBlock >= tile) break;
      uint64_t pv[kBatch];
      bool have[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        const int64_t j = tid + (int64_t)(b + i) * kBlock;
        pv[i] = 0ull;
        have[i] = true;
        if (j < tile) {
          if (!CHAINED || j < first_range)
            pv[i] = sums[j];
          else
            have[i] = try_read(&slots[j], tag, &pv[i]);
        }
      }
      if (CHAINED) {
        bool pending = true;
        for (int spin = 0; pending && spin < spin_limit; ++spin) {
          pending = false;
#pragma unroll
          for (int i = 0; i < kBatch; ++i) {
            if (!have[i]) {
              have[i] = try_read(&slots[tid + (int64_t)(b + i) * kBlock], tag, &pv[i]);
              pending |= !have[i];
            }
          }
          if (pending) __builtin_amdgcn_s_sleep(1);
        }
      }
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        const int j = tid + (b + i) * kBlock;
        if (CHAINED && !have[i]) {
          atomicOr(&s_missing[j >> 5], 1u << (j & 31));
          miss = true;
        } else if (j < tile) {
          part += Bits<Acc>::from(pv[i]);
        }
      }
    }
    if (!CHAINED) break;
    if (!__syncthreads_or(miss)) {
      failed = false;
      break;
    }
    for (int word = 0; word < kMaxRanges / 32; ++word) {
      uint32_t bits = s_missing[word];
      while (bits) {
        const int j = word * 32 + (__ffs((int)bits) - 1);
        bits &= bits - 1u;
        const Acc total = range_total_direct<In, Acc, Out, G>(in, n, j, red);
        if (tid == 0) publish(&slots[j], tag, Bits<Acc>::to(total));
      }
    }
    __syncthreads();
    if (tid < kMaxRanges / 32) s_missing[tid] = 0u;
    __syncthreads();
  }
  const Acc pw = wave_sum(part);
  if (lane == 0) red[wave] = pw;
  __syncthreads();
  Acc excl = (red[0] + red[1]) + (red[2] + red[3]);
  if (MODE == kPrefixed) excl = Bits<Acc>::from(reinterpret_cast<const uint64_t *>(slots)[tile]);
  // Three passes cannot fail (the second one reads what this workgroup published itself); should
  // they -- two launches that share one workspace at the same time --, the range is marked rather
  // than silently wrong: NaN for the fp64 sums, the most negative integer for int64 ones (the
  // prefixes of that range then come out negative where the inputs are not).
  if (CHAINED && failed)
    excl = Bits<Acc>::from(std::is_same<Acc, double>::value ? 0x7ff8dead00000000ull
                                                            : 0x8000000000000000ull);
  const Acc wavebase = wave == 0 ? (Acc)0 : wave == 1 ? w0 : wave == 2 ? w0 + w1 : (w0 + w1) + w2;
  Acc run = (excl + wavebase) + wexcl;

  // Results leave through the staging row so that every store instruction of the wave writes
  // whole 128-byte lines.  Results that fit the caches are stored normally (the search that
  // follows reads them back); larger ones stream past the caches with non-temporal stores.
  const bool nt = n * (int64_t)sizeof(Out) > (32ll << 20);
  constexpr bool kByRun = geo::kOG > G && G * 16 >= 128;  // pieces of G granules of every lane
  constexpr int kPG = geo::kOG <= G ? geo::kOG : (kByRun ? G : geo::kOG);  // granules per lane and piece
  constexpr int kPL = (geo::kOG <= G || kByRun) ? kWave : geo::kPiece;   // lanes per piece
  constexpr int kPieces = (geo::kOG / kPG) * (kWave / kPL);
  constexpr int kPitch = kPG + 1;
  static_assert(kPL * kPitch <= geo::kStage, "piece fits the staging row");
  out_gran o[kPL == kWave ? kPG : geo::kOG];
  if (kPL != kWave) {
#pragma unroll
    for (int j = 0; j < geo::kOG; ++j)
#pragma unroll
      for (int k = 0; k < geo::kOE; ++k) {
        run += (Acc)f[j * geo::kOE + k];
        o[j][k] = (Out)run;
      }
  }
#pragma unroll
  for (int p = 0; p < kPieces; ++p) {
    if (kPL == kWave) {
      // piece p = granules [p*kPG, (p+1)*kPG) of every lane
#pragma unroll
      for (int j = 0; j < kPG; ++j) {
#pragma unroll
        for (int k = 0; k < geo::kOE; ++k) {
          run += (Acc)f[(p * kPG + j) * geo::kOE + k];
          o[j][k] = (Out)run;
        }
        stage[lane * kPitch + j] = __builtin_bit_cast(u32x4, o[j]);
      }
    } else if (lane / kPL == p) {
      // piece p = all granules of lanes [p*kPL, (p+1)*kPL)
      const int l = lane - p * kPL;
#pragma unroll
      for (int j = 0; j < geo::kOG; ++j) stage[l * kPitch + j] = __builtin_bit_cast(u32x4, o[j]);
    }
    wave_lds_sync();
    constexpr int kStores = kPG * kPL / kWave;
    const bool whole = wbase + geo::kWaveElems <= n;
#pragma unroll
    for (int i = 0; i < kStores; ++i) {
      const int q = i * kWave + lane;
      const int l2 = q / kPG, j = q % kPG;
      const out_gran v = __builtin_bit_cast(out_gran, stage[l2 * kPitch + j]);
      const int64_t e0 = kPL == kWave
                             ? wbase + (int64_t)l2 * geo::kEPT + (int64_t)(p * kPG + j) * geo::kOE
                             : wbase + (int64_t)(p * kPL + l2) * geo::kEPT + (int64_t)j * geo::kOE;
      if (whole) {
        store_vec(reinterpret_cast<out_gran *>(out + e0), v, nt);
      } else {  // ragged end of the input
#pragma unroll
        for (int k = 0; k < geo::kOE; ++k)
          if (e0 + k < n) out[e0 + k] = v[k];
      }
    }
    wave_lds_sync();
  }
}

// ---- deterministic sum: fixed grid, fixed tree ------------------------------------------------
constexpr int kSumMaxBlocks = 1024;

__global__ __launch_bounds__(kBlock) void sum_partial_kernel(const float *__restrict__ in,
                                                             int64_t n, double *partial) {
  __shared__ double wtot[kBlock / kWave];
  typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));
  const int tid = threadIdx.x;
  double acc = 0.0;
  const int64_t nvec = n >> 2;
  for (int64_t v = (int64_t)blockIdx.x * kBlock + tid; v < nvec; v += (int64_t)gridDim.x * kBlock) {
    const f4 q = *reinterpret_cast<const f4 *>(in + (v << 2));
    acc += ((double)q[0] + (double)q[1]) + ((double)q[2] + (double)q[3]);
  }
  if (blockIdx.x == 0 && tid < (int)(n & 3)) acc += (double)in[(nvec << 2) + tid];
  const double w = wave_sum(acc);
  if ((tid & 63) == 0) wtot[tid >> 6] = w;
  __syncthreads();
  if (tid == 0) partial[blockIdx.x] = (wtot[0] + wtot[1]) + (wtot[2] + wtot[3]);
}

__global__ __launch_bounds__(kBlock) void sum_final_kernel(const double *partial, int nblocks,
                                                           float *out, double *out_f64) {
  __shared__ double wtot[kBlock / kWave];
  const int tid = threadIdx.x;
  double acc = 0.0;
  for (int i = tid; i < nblocks; i += kBlock) acc += partial[i];
  const double w = wave_sum(acc);
  if ((tid & 63) == 0) wtot[tid >> 6] = w;
  __syncthreads();
  if (tid == 0) {
    const double t = (wtot[0] + wtot[1]) + (wtot[2] + wtot[3]);
    if (out) *out = (float)t;
    if (out_f64) *out_f64 = t;
  }
}

int64_t scan_tiles(int64_t n, int tile_elems) { return n <= 0 ? 0 : ceil_div64(n, tile_elems); }

// Workspace: a 256-byte header (unused), then per smallest range (2048 elements, so that both
// element types fit) one 8-byte plain sum and one 24-byte tagged slot.
size_t scan_ws_bytes(int64_t n) {
  const int64_t tiles = scan_tiles(n, kMinRange);
  return kHeaderBytes + align_up((size_t)tiles * (8 + sizeof(Slot)), 256);
}

// Every chained launch of the process gets a tag of its own, and one that nothing else is likely
// to have left in memory: a workspace need not be initialised, and what it holds is rarely
// random -- small integers (indices, counts, sums of them) are common, and so would be the tags
// 1, 2, 3 ... of an earlier process whose memory this one was given.  The launch counter
// therefore starts at a random place and goes through a bijection of the 42-bit tags that
// scatters neighbouring counts (multiplications by odd numbers and xor-shifts).
std::atomic<uint64_t> g_scan_epoch{0};
uint64_t next_tag() {
  static const uint64_t seed = [] {
    std::random_device rd;
    uint64_t s = ((uint64_t)rd() << 32) ^ (uint64_t)rd();
    s ^= (uint64_t)std::chrono::steady_clock::now().time_since_epoch().count();
    return s;
  }();
  for (;;) {
    uint64_t x = (g_scan_epoch.fetch_add(1, std::memory_order_relaxed) + seed) & kTagMask;
    x = (x * 0x2545F4914F5ull) & kTagMask;
    x ^= x >> 21;
    x = (x * 0x1B03738712Full) & kTagMask;
    x ^= x >> 19;
    if (x != 0ull && x != kTagMask) return x;  // all-zero and all-one words are common too
  }
}

// How many workgroups of a kernel the current GPU holds at once, and the rate of wall_clock64().
struct Residency {
  int workgroups;
  int64_t clock_khz;
};
Residency residency(const void *kernel) {
  Residency r{0, 100000};
  int dev = 0, per_cu = 0, cus = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess) return r;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kBlock, 0) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
    (void)hipGetLastError();
    return r;
  }
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) == hipSuccess && khz > 0)
    r.clock_khz = khz;
  else
    (void)hipGetLastError();
  r.workgroups = per_cu * cus;
  return r;
}

// first_changed > 0: the sums of the ranges before the one that holds element first_changed are
// still in the workspace from the last scan of this array, and `out` still holds the prefix up to
// there; only the later ranges are summed and scanned again.
template <typename In, typename Acc, typename Out, int VE, int G>
int launch_ranges(const In *in, Out *out, int64_t n, void *ws, hipStream_t st, bool chained,
                  int64_t first_changed) {
  const int64_t range_elems = (int64_t)G * kBlock * VE;
  const int64_t ranges = ceil_div64(n, range_elems);
  const int64_t max_ranges = scan_tiles(n, kMinRange);
  uint64_t *sums = reinterpret_cast<uint64_t *>(static_cast<char *>(ws) + kHeaderBytes);
  Slot *slots = reinterpret_cast<Slot *>(sums + max_ranges);
  const int64_t first = first_changed > 0 ? first_changed / range_elems : 0;
  const dim3 grid((unsigned)(ranges - first)), block(kBlock);
  if (!chained) {
    range_sum_kernel<In, Acc, Out, G><<<grid, block, 0, st>>>(in, n, sums, first);
    if (ranges <= kMaxRangesTwo) {
      scan_ranges_kernel<In, Acc, Out, G, kTwoLaunches><<<grid, block, 0, st>>>(
          in, out, n, sums, slots, first, 0ull, 0, 0, 0);
    } else {
      // more ranges than a workgroup adds up by itself: their prefix comes from a launch in
      // between (into the words that the chained variant uses for its slots)
      range_prefix_kernel<Acc><<<dim3(1), dim3(kPrefixThreads), 0, st>>>(
          sums, reinterpret_cast<uint64_t *>(slots), ranges);
      scan_ranges_kernel<In, Acc, Out, G, kPrefixed><<<grid, block, 0, st>>>(
          in, out, n, sums, slots, first, 0ull, 0, 0, 0);
    }
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  const uint64_t tag = next_tag();
  const int spin_limit = env_int("GEAR_HIP_SCAN_SPIN_LIMIT", 1 << 14);
  // Staggered starts pay once several workgroups share a CU (measured: from ~5e6 fp32 elements
  // on; below that they only delay the launch): 5 ns per range of 8192 fp32 elements.
  int stagger = 0, first_wave = 0;
  if (ranges - first > 512) {
    static const Residency res = residency((const void *)scan_ranges_kernel<In, Acc, Out, G, kChained>);
    const int64_t ps = env_int("GEAR_HIP_SCAN_STAGGER_PS", 5000) * (int64_t)(G * 16) / 128;
    stagger = (int)(ps * res.clock_khz * 1024 / 1000000000ll);
    first_wave = res.workgroups;
  }
  scan_ranges_kernel<In, Acc, Out, G, kChained><<<grid, block, 0, st>>>(
      in, out, n, sums, slots, first, tag, spin_limit, stagger, first_wave);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

template <typename In, typename Acc, typename Out, int VE>
int launch_scan(const In *in, Out *out, int64_t n, void *ws, size_t ws_bytes, hipStream_t st,
                int64_t first_changed = 0) {
  if (n < 0 || n > (1ll << 40)) return n < 0 ? GEAR_HIP_EINVAL : GEAR_HIP_ERANGE;
  if (n == 0) return 0;
  if (!in || !out) return GEAR_HIP_EINVAL;
  if (!ws || ws_bytes < scan_ws_bytes(n) || (reinterpret_cast<uintptr_t>(ws) & 7))
    return GEAR_HIP_EWORKSPACE;
  if ((reinterpret_cast<uintptr_t>(in) & (sizeof(In) - 1)) ||
      (reinterpret_cast<uintptr_t>(out) & 15))
    return GEAR_HIP_EALIGN;
  // GEAR_HIP_SCAN_SINGLE_PASS: 1 = the chained kernel wherever it applies, 0 = never; unset = the
  // chained kernel for full scans, two launches for the rescan of a suffix.  A launch that is
  // being captured into a graph would replay its tag, so it takes the two launches.
  const int forced = env_int("GEAR_HIP_SCAN_SINGLE_PASS", -1);
  bool chained = forced < 0 ? first_changed <= 0 : forced == 1;
  if (chained) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess) {
      (void)hipGetLastError();
      cap = hipStreamCaptureStatusActive;
    }
    if (cap != hipStreamCaptureStatusNone) chained = false;
  }
  // Ranges of 2, 4, 8 or 16 granules per thread (2048 to 16384 fp32 elements): 2 while that
  // leaves at most 256 ranges, 4 up to 512 ranges, then 8 (a workgroup adds up ALL earlier sums, so
  // more ranges cost more than they gain once every CU has work), and 16 -- 190 registers, two
  // workgroups per CU -- where 8 would need more than 4096 ranges (33.5 to 67 M fp32: one read
  // instead of two, 187 -> 148 us at 6e7).  The chained kernel and the two launches cut the input
  // the same way, so a rescan finds the sums of the last full scan.
  // Beyond 4096 ranges the words to poll outweigh the second read: two launches, up to 16384
  // ranges of 8 granules.  (8-byte elements: ranges of 2 granules would be smaller than the 2048 elements the
  // workspace is laid out for, so they start at 4.)
  constexpr int64_t g1 = (int64_t)kBlock * VE;  // elements per range and granule
  if (VE == 4 && ceil_div64(n, 2 * g1) <= 256)
    return launch_ranges<In, Acc, Out, VE, 2>(in, out, n, ws, st, chained, first_changed);
  else if (ceil_div64(n, 4 * g1) <= 512)
    return launch_ranges<In, Acc, Out, VE, 4>(in, out, n, ws, st, chained, first_changed);
  else if (ceil_div64(n, 8 * g1) <= kMaxRanges)
    return launch_ranges<In, Acc, Out, VE, 8>(in, out, n, ws, st, chained, first_changed);
  else if (ceil_div64(n, 16 * g1) <= kMaxRanges)
    return launch_ranges<In, Acc, Out, VE, 16>(in, out, n, ws, st, chained, first_changed);
  return launch_ranges<In, Acc, Out, VE, 8>(in, out, n, ws, st, false, first_changed);
}

}  // namespace
}  // namespace gearhip

using namespace gearhip;

extern "C" size_t gear_hip_scan_workspace_bytes(int64_t n) { return scan_ws_bytes(n); }

extern "C" int gear_hip_scan_f32_f64(const float *in, double *out, int64_t n, void *workspace,
                                     size_t workspace_bytes, void *stream) {
  return launch_scan<float, double, double, 4>(in, out, n, workspace, workspace_bytes,
                                               as_stream(stream));
}

// ---- the scan with its workspace in a static device array ---------------------------------------
// For callers that cannot allocate device memory (a stream under graph capture, a serving loop
// with a frozen memory pool): the range sums live in a file-scope device array instead of a
// caller-supplied workspace.  In host code the array's name is only a handle for
// hipGetSymbolAddress; the device address it yields (one per GPU, each GPU holds its own copy)
// is what the kernels and every host-side use receive.
namespace gearhip {
namespace {

constexpr int64_t kStaticMaxN = 1ll << 27;  // 134 217 728 priorities
constexpr size_t kStaticBytes =
    kHeaderBytes + (size_t)(kStaticMaxN / (kMinRange)) * (8 + sizeof(Slot));
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kStaticBytes];

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];

// One static call at a time per device: calls that overlapped (two streams, two host threads)
// would overwrite each other's range sums.  The event marks the end of the last static call's
// kernels on its stream; the next call's stream waits for it before its own kernels start.
struct StaticOrder {
  std::mutex lock;
  hipEvent_t done = nullptr;
  bool recorded = false;
};
StaticOrder g_static_order[kMaxDevices];

bool stream_is_capturing(hipStream_t st) {
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &cap) != hipSuccess) {
    (void)hipGetLastError();
    return true;  // unknown: treat as capturing, the careful side
  }
  return cap != hipStreamCaptureStatusNone;
}

// Device address of `scratch` on device `dev` (the current one), looked up once per device.
// may_look_up = false (the stream is being captured): only an address found earlier is returned.
int static_scratch(int dev, bool may_look_up, void **ptr) {
  void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (!may_look_up) return GEAR_HIP_ENOTREADY;
    GEARHIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (p == nullptr) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // every thread finds the same address
  }
  *ptr = p;
  return 0;
}

int current_device(int *dev) {
  GEARHIP_CHECK(hipGetDevice(dev));
  if (*dev < 0 || *dev >= kMaxDevices) return GEAR_HIP_ERANGE;
  return 0;
}

}  // namespace

// Set-up for the static form on the current device: the array's address and the event that
// orders its calls.  What fails here is reported again by the entry point itself.
int scan_static_init() {
  int dev = -1;
  int rc = current_device(&dev);
  if (rc) return rc;
  void *p = nullptr;
  rc = static_scratch(dev, true, &p);
  if (rc) return rc;
  StaticOrder &order = g_static_order[dev];
  std::lock_guard<std::mutex> guard(order.lock);
  if (order.done == nullptr)
    GEARHIP_CHECK(hipEventCreateWithFlags(&order.done, hipEventDisableTiming));
  return 0;
}

}  // namespace gearhip

extern "C" int64_t gear_hip_scan_static_max_n(void) { return kStaticMaxN; }

extern "C" int gear_hip_scan_f32_f64_static(const float *in, double *out, int64_t n,
                                            void *stream) {
  if (n < 0) return GEAR_HIP_EINVAL;
  if (n > kStaticMaxN) return GEAR_HIP_ERANGE;
  if (n == 0) return 0;
  static_assert(kStaticBytes >= kHeaderBytes + 16, "scratch holds at least one range");
  if (kStaticBytes < scan_ws_bytes(n)) return GEAR_HIP_ERANGE;
  int dev = -1;
  int rc = current_device(&dev);
  if (rc) return rc;
  hipStream_t st = as_stream(stream);
  const bool capturing = stream_is_capturing(st);
  void *ws = nullptr;
  rc = static_scratch(dev, !capturing, &ws);
  if (rc) return rc;
  if (capturing)  // the graph's own order is the caller's; events of this kind are not captured
    return launch_scan<float, double, double, 4>(in, out, n, ws, kStaticBytes, st);
  StaticOrder &order = g_static_order[dev];
  std::lock_guard<std::mutex> guard(order.lock);
  if (order.done == nullptr)
    GEARHIP_CHECK(hipEventCreateWithFlags(&order.done, hipEventDisableTiming));
  if (order.recorded) GEARHIP_CHECK(hipStreamWaitEvent(st, order.done, 0));
  rc = launch_scan<float, double, double, 4>(in, out, n, ws, kStaticBytes, st);
  if (rc) return rc;
  GEARHIP_CHECK(hipEventRecord(order.done, st));
  order.recorded = true;
  return 0;
}

extern "C" int gear_hip_rescan_f32_f64(const float *in, double *out, int64_t n,
                                       int64_t first_changed, void *workspace,
                                       size_t workspace_bytes, void *stream) {
  if (first_changed < 0) return GEAR_HIP_EINVAL;
  if (first_changed >= n && n >= 0) return 0;  // nothing changed
  return launch_scan<float, double, double, 4>(in, out, n, workspace, workspace_bytes,
                                               as_stream(stream), first_changed);
}

extern "C" int gear_hip_scan_i64(const int64_t *in, int64_t *out, int64_t n, void *workspace,
                                 size_t workspace_bytes, void *stream) {
  return launch_scan<int64_t, int64_t, int64_t, 2>(in, out, n, workspace, workspace_bytes,
                                                   as_stream(stream));
}

extern "C" int gear_hip_scan_f32_f32(const float *in, float *out, int64_t n, void *workspace,
                                     size_t workspace_bytes, void *stream) {
  return launch_scan<float, double, float, 4>(in, out, n, workspace, workspace_bytes,
                                              as_stream(stream));
}

extern "C" size_t gear_hip_sum_workspace_bytes(int64_t n) {
  (void)n;
  return kSumMaxBlocks * sizeof(double);
}

extern "C" int gear_hip_sum_f32(const float *in, int64_t n, float *out, double *out_f64,
                                void *workspace, size_t workspace_bytes, void *stream) {
  if (n < 0 || (!out && !out_f64)) return GEAR_HIP_EINVAL;
  if (n > 0 && !in) return GEAR_HIP_EINVAL;
  if (!workspace || workspace_bytes < kSumMaxBlocks * sizeof(double)) return GEAR_HIP_EWORKSPACE;
  if (reinterpret_cast<uintptr_t>(in) & 3) return GEAR_HIP_EALIGN;
  int64_t blocks = ceil_div64(n, (int64_t)kBlock * 16);
  if (blocks < 1) blocks = 1;
  if (blocks > kSumMaxBlocks) blocks = kSumMaxBlocks;
  double *partial = static_cast<double *>(workspace);
  hipStream_t st = as_stream(stream);
  sum_partial_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(in, n, partial);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  sum_final_kernel<<<dim3(1), dim3(kBlock), 0, st>>>(partial, (int)blocks, out, out_f64);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}
