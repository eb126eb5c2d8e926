// Inclusive prefix sums and a deterministic sum, gfx950.  fp32 inputs are accumulated in fp64.
//
// Three kernels share the inner scan (each thread scans inside its 16-byte input vectors, row sums
// go through a DPP wave scan, wave totals meet in LDS, results leave through LDS so that every store
// instruction writes whole lines):
//  * default, up to 8192 ranges (n <= 134 M fp32): two launches.  range_sum_kernel writes the sum
//    of every range; scan_ranges_kernel<TWO = true> re-reads its range (now in L2 / MALL), adds
//    the sums of all earlier ranges in a fixed order and writes the prefix.  No workgroup waits for
//    another one.  On this multi-XCD part that is faster than the one-pass kernels: a ticket per
//    workgroup on one address costs ~19 ns each across the XCDs, and every agent-scope round trip
//    of a look-back 1-2 us.
//  * GEAR_HIP_SCAN_SINGLE_PASS=1: scan_ranges_kernel<TWO = false>, one pass over the data.  Tile
//    numbers are handed out by an atomic ticket in launch order (every awaited predecessor is
//    already running); a workgroup publishes the sum of its range in one agent-scope 64-bit store
//    (kEmpty = not published, so no fence pairs) and sums ALL earlier ranges' words.
//  * beyond that (and beyond 2048 ranges in the single-pass mode): scan_kernel, the tiled decoupled look-back (aggr[t] = sum of tile t alone,
//    incl[t] = sum of tiles 0..t; wave 0 looks back 64 predecessors at a time, ballots pick the
//    nearest published inclusive value).
#include <atomic>
#include <type_traits>

#include "wave.hpp"

namespace gearhip {
namespace {

constexpr int kBlock = 256;
constexpr int kRows = 4;
constexpr uint64_t kEmpty = ~0ull;  // no fp64 sum of fp32 values has this bit pattern (fp64 scans only)
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

template <typename In, int VE> struct InVec;
template <> struct InVec<float, 4> {
  typedef float type __attribute__((ext_vector_type(4), aligned(4)));
};
template <> struct InVec<int64_t, 2> {
  typedef int64_t type __attribute__((ext_vector_type(2), aligned(8)));
};
template <typename Acc> struct OutVec2;
// result vectors are stored with their natural alignment (the launcher checks the pointer)
template <> struct OutVec2<double> {
  typedef double type __attribute__((ext_vector_type(2)));
};
template <> struct OutVec2<int64_t> {
  typedef int64_t type __attribute__((ext_vector_type(2)));
};
template <> struct OutVec2<float> {
  typedef float type __attribute__((ext_vector_type(2)));
};

// Writes the VE consecutive results of every lane of a wave (a contiguous slice of 64*VE
// elements starting at e_wave) so that each store instruction covers one contiguous run:
// non-temporal stores only reach full bandwidth when a wave writes whole cache lines.  With
// 16 bytes per lane the lanes already do; with 32 bytes per lane (fp64 results of a float4) the
// slice takes a detour through a wave-private LDS row.
// Results that fit the caches are stored normally (the search that follows reads them back);
// larger ones stream past the caches with non-temporal stores.
template <typename V>
__device__ __forceinline__ void store_vec(V *p, V v, bool nt) {
  if (nt)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}

template <typename Out, int VE>
__device__ __forceinline__ void store_slice(Out *__restrict__ out, int64_t e_wave, int64_t n,
                                            const Out (&v)[VE], Out *stage_row, int lane) {
  const bool nt = n * (int64_t)sizeof(Out) > (32ll << 20);
  typedef typename OutVec2<Out>::type out_vec2;
  constexpr int kLaneBytes = VE * (int)sizeof(Out);
  const int64_t e0 = e_wave + (int64_t)lane * VE;
  if (e_wave + (int64_t)kWave * VE > n) {  // ragged end of the input
#pragma unroll
    for (int j = 0; j < VE; ++j)
      if (e0 + j < n) out[e0 + j] = v[j];
    return;
  }
  if (kLaneBytes <= 16) {
#pragma unroll
    for (int j = 0; j < VE; j += 2) {
      out_vec2 o;
      o[0] = v[j];
      o[1] = v[j + 1];
      store_vec(reinterpret_cast<out_vec2 *>(out + e0 + j), o, nt);
    }
  } else {
#pragma unroll
    for (int j = 0; j < VE; ++j) stage_row[lane * VE + j] = v[j];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int h = 0; h < VE / 2; ++h) {
      out_vec2 o;
      o[0] = stage_row[h * 2 * kWave + 2 * lane];
      o[1] = stage_row[h * 2 * kWave + 2 * lane + 1];
      store_vec(reinterpret_cast<out_vec2 *>(out + e_wave + (int64_t)h * 2 * kWave + 2 * lane), o,
                nt);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

__global__ void scan_init_kernel(uint32_t *ticket, uint64_t *desc, int64_t words) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i == 0) *ticket = 0u;
  if (i < words) desc[i] = kEmpty;
}

template <typename In, typename Acc, typename Out, int VE>
__global__ __launch_bounds__(kBlock) void scan_kernel(const In *__restrict__ in,
                                                      Out *__restrict__ out, int64_t n,
                                                      uint32_t *ticket, uint64_t *aggr,
                                                      uint64_t *incl) {
  constexpr int kTileElems = kRows * kBlock * VE;
  constexpr int kWaves = kBlock / kWave;
  typedef typename InVec<In, VE>::type in_vec;
  __shared__ Acc wtot[kRows][kWaves];
  __shared__ Out stage[kWaves][kWave * VE];
  __shared__ Acc s_excl;
  __shared__ uint32_t s_tile;

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  if (tid == 0) s_tile = atomicAdd(ticket, 1u);
  __syncthreads();
  const int64_t tile = s_tile;
  const int64_t base = tile * kTileElems;

  Acc x[kRows][VE];
  Acc s[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int64_t e0 = base + ((int64_t)r * kBlock + tid) * VE;
    if (e0 + VE <= n) {
      const in_vec v = *reinterpret_cast<const in_vec *>(in + e0);
#pragma unroll
      for (int j = 0; j < VE; ++j) x[r][j] = (Acc)v[j];
    } else {
#pragma unroll
      for (int j = 0; j < VE; ++j) x[r][j] = (e0 + j < n) ? (Acc)in[e0 + j] : (Acc)0;
    }
#pragma unroll
    for (int j = 1; j < VE; ++j) x[r][j] += x[r][j - 1];
    s[r] = x[r][VE - 1];
  }

  Acc wexcl[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const Acc inc = wave_inclusive_sum(s[r]);
    wexcl[r] = wave_shift_up1(inc);
    if (lane == kWave - 1) wtot[r][wave] = inc;
  }
  __syncthreads();

  Acc tile_total = (Acc)0;
  Acc mybase[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    Acc acc = tile_total;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      if (w == wave) mybase[r] = acc + wexcl[r];
      acc += wtot[r][w];
    }
    tile_total = acc;
  }

  if (wave == 0) {
    Acc excl = (Acc)0;
    if (tile == 0) {
      if (lane == 0) store_agent(&incl[0], Bits<Acc>::to(tile_total));
    } else {
      if (lane == 0) store_agent(&aggr[tile], Bits<Acc>::to(tile_total));
      int64_t look = tile - 1;
      while (true) {
        const int64_t idx = look - lane;
        uint64_t vi = kEmpty, va = kEmpty;
        if (idx >= 0) {
          vi = load_agent(&incl[idx]);
          if (vi == kEmpty) va = load_agent(&aggr[idx]);
        }
        const bool has_incl = (idx < 0) || (vi != kEmpty);
        const bool ready = has_incl || (va != kEmpty);
        const uint64_t bi = wave_ballot(has_incl), br = wave_ballot(ready);
        const int first = bi ? (__ffsll((unsigned long long)bi) - 1) : kWave;
        const uint64_t need = first >= 63 ? ~0ull : ((2ull << first) - 1ull);
        if ((br & need) != need) {
          __builtin_amdgcn_s_sleep(1);
          continue;
        }
        Acc c = (Acc)0;
        if (lane < first)
          c = Bits<Acc>::from(va);
        else if (lane == first && idx >= 0)
          c = Bits<Acc>::from(vi);
        excl += wave_sum(c);
        if (first < kWave) break;
        look -= kWave;
      }
      if (lane == 0) store_agent(&incl[tile], Bits<Acc>::to(excl + tile_total));
    }
    if (lane == 0) s_excl = excl;
  }
  __syncthreads();
  const Acc excl = s_excl;

#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const Acc b = excl + mybase[r];
    Out o[VE];
#pragma unroll
    for (int j = 0; j < VE; ++j) o[j] = (Out)(b + x[r][j]);
    store_slice<Out, VE>(out, base + ((int64_t)r * kBlock + wave * kWave) * VE, n, o, stage[wave],
                         lane);
  }
}

// ---- range variant -------------------------------------------------------------------------------
// For up to kMaxRanges workgroups the look-back chain is not needed at all: a workgroup owns NR
// rows of 256 vectors kept in registers, publishes the sum of its range as soon as it has loaded
// it, and takes its exclusive prefix as the sum of ALL earlier ranges' aggregates (each thread
// polls its share of them, fixed summation order).  Nobody waits for an inclusive value, so there
// is no serial chain across the XCDs, and the result is bit-reproducible from run to run.
constexpr int kMaxRanges = 2048;     // single-pass variant: every thread polls 8 range sums
constexpr int kMaxRangesTwo = 8192;  // two launches: every thread adds up to 32 range sums

// Sum of every range, one workgroup per range: the first launch of the two-launch variant, in
// which the scan launch below finds all aggregates ready (no ticket, no publishing, no polling).
template <typename In, typename Acc, int VE, int NR>
__global__ __launch_bounds__(kBlock) void range_sum_kernel(const In *__restrict__ in, int64_t n,
                                                           uint64_t *__restrict__ aggr,
                                                           int64_t first_range) {
  constexpr int kElems = NR * kBlock * VE;
  constexpr int kWaves = kBlock / kWave;
  typedef typename InVec<In, VE>::type in_vec;
  __shared__ Acc red[kWaves];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  const int64_t range = first_range + blockIdx.x;
  const int64_t base = range * kElems;
  In raw[NR][VE];
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int64_t e0 = base + ((int64_t)r * kBlock + tid) * VE;
    if (e0 + VE <= n) {
      const in_vec v = *reinterpret_cast<const in_vec *>(in + e0);
#pragma unroll
      for (int j = 0; j < VE; ++j) raw[r][j] = v[j];
    } else {
#pragma unroll
      for (int j = 0; j < VE; ++j) raw[r][j] = (e0 + j < n) ? in[e0 + j] : (In)0;
    }
  }
  Acc tsum = (Acc)0;
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    Acc a = (Acc)raw[r][0];
#pragma unroll
    for (int j = 1; j < VE; ++j) a += (Acc)raw[r][j];
    tsum += a;
  }
  const Acc w = wave_sum(tsum);
  if (lane == 0) red[wave] = w;
  __syncthreads();
  if (tid == 0) aggr[range] = Bits<Acc>::to((red[0] + red[1]) + (red[2] + red[3]));
}

template <typename In, typename Acc, typename Out, int VE, int NR, bool TWO>
__global__ __launch_bounds__(kBlock) void scan_ranges_kernel(const In *__restrict__ in,
                                                             Out *__restrict__ out, int64_t n,
                                                             uint32_t *ticket, uint64_t *aggr,
                                                             int64_t first_range) {
  constexpr int kElems = NR * kBlock * VE;
  constexpr int kWaves = kBlock / kWave;
  typedef typename InVec<In, VE>::type in_vec;
  __shared__ Acc wtot[NR][kWaves];
  __shared__ Out stage[kWaves][kWave * VE];
  __shared__ Acc red[kWaves];
  __shared__ uint32_t s_tile;

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  if (!TWO) {
    if (tid == 0) s_tile = atomicAdd(ticket, 1u);
    __syncthreads();
  }
  const int64_t tile = TWO ? first_range + (int64_t)blockIdx.x : (int64_t)s_tile;
  const int64_t base = tile * kElems;

  In raw[NR][VE];
  Acc s[NR];
  Acc tsum = (Acc)0;
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int64_t e0 = base + ((int64_t)r * kBlock + tid) * VE;
    if (e0 + VE <= n) {
      const in_vec v = __builtin_nontemporal_load(reinterpret_cast<const in_vec *>(in + e0));
#pragma unroll
      for (int j = 0; j < VE; ++j) raw[r][j] = v[j];
    } else {
#pragma unroll
      for (int j = 0; j < VE; ++j) raw[r][j] = (e0 + j < n) ? in[e0 + j] : (In)0;
    }
  }
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    Acc a = (Acc)raw[r][0];
#pragma unroll
    for (int j = 1; j < VE; ++j) a += (Acc)raw[r][j];
    s[r] = a;
    tsum += a;
  }
  // the range's aggregate goes out before the detailed scan
  if (!TWO) {
    const Acc w = wave_sum(tsum);
    if (lane == 0) red[wave] = w;
    __syncthreads();
    if (tid == 0) store_agent(&aggr[tile], Bits<Acc>::to((red[0] + red[1]) + (red[2] + red[3])));
  }
  Acc wexcl[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const Acc inc = wave_inclusive_sum(s[r]);
    wexcl[r] = wave_shift_up1(inc);
    if (lane == kWave - 1) wtot[r][wave] = inc;
  }
  // sum of every earlier range (thread t takes ranges t, t+256, ...)
  // all of a thread's polls are issued together; only the ones not yet published are repeated
  constexpr int kPolls = (TWO ? kMaxRangesTwo : kMaxRanges) / kBlock;
  uint64_t pv[kPolls];
#pragma unroll
  for (int i = 0; i < kPolls; ++i) {
    const int64_t j = tid + (int64_t)i * kBlock;
    pv[i] = j < tile ? (TWO ? aggr[j] : load_agent(&aggr[j])) : 0ull;
  }
  bool pending = !TWO;
  while (pending) {
    pending = false;
#pragma unroll
    for (int i = 0; i < kPolls; ++i) {
      const int64_t j = tid + (int64_t)i * kBlock;
      if (j < tile && pv[i] == kEmpty) {
        pv[i] = load_agent(&aggr[j]);
        pending |= pv[i] == kEmpty;
      }
    }
    if (pending) __builtin_amdgcn_s_sleep(1);
  }
  Acc part = (Acc)0;
#pragma unroll
  for (int i = 0; i < kPolls; ++i)
    if (tid + (int64_t)i * kBlock < tile) part += Bits<Acc>::from(pv[i]);
  const Acc pw = wave_sum(part);
  __syncthreads();  // wtot complete; everybody is done reading red
  if (lane == 0) red[wave] = pw;
  __syncthreads();
  const Acc excl = (red[0] + red[1]) + (red[2] + red[3]);

  Acc rowbase = excl;
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    Acc acc = rowbase, mine = rowbase;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      if (w == wave) mine = acc + wexcl[r];
      acc += wtot[r][w];
    }
    rowbase = acc;
    Acc run = mine;
    Out o[VE];
#pragma unroll
    for (int j = 0; j < VE; ++j) {
      run += (Acc)raw[r][j];
      o[j] = (Out)run;
    }
    store_slice<Out, VE>(out, base + ((int64_t)r * kBlock + wave * kWave) * VE, n, o, stage[wave],
                         lane);
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

// the workspace is sized for the smaller tile (int64: 2048 elements) so both scans fit
size_t scan_ws_bytes(int64_t n) {
  const int64_t tiles = scan_tiles(n, kRows * kBlock * 2);
  return kHeaderBytes + align_up((size_t)tiles * 16, 256);
}

// first_changed > 0 (two-launch variant only): the range sums of the ranges before the one that
// holds element first_changed are still in the workspace from the last scan of this array, and
// `out` still holds the prefix up to there; only the later ranges are summed and scanned again.
template <typename In, typename Acc, typename Out, int VE, int NR>
int launch_ranges(const In *in, Out *out, int64_t n, void *ws, hipStream_t st, bool single_pass,
                  int64_t first_changed) {
  const int64_t range_elems = (int64_t)NR * kBlock * VE;
  const int64_t ranges = ceil_div64(n, range_elems);
  uint32_t *ticket = static_cast<uint32_t *>(ws);
  uint64_t *aggr = reinterpret_cast<uint64_t *>(static_cast<char *>(ws) + kHeaderBytes);
  if (!single_pass) {
    const int64_t first = first_changed > 0 ? first_changed / range_elems : 0;
    const dim3 grid((unsigned)(ranges - first)), block(kBlock);
    range_sum_kernel<In, Acc, VE, NR><<<grid, block, 0, st>>>(in, n, aggr, first);
    scan_ranges_kernel<In, Acc, Out, VE, NR, true><<<grid, block, 0, st>>>(in, out, n, ticket, aggr,
                                                                          first);
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  scan_init_kernel<<<dim3((unsigned)ceil_div64(ranges, kBlock)), dim3(kBlock), 0, st>>>(ticket, aggr,
                                                                                      ranges);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  scan_ranges_kernel<In, Acc, Out, VE, NR, false><<<dim3((unsigned)ranges), dim3(kBlock), 0, st>>>(
      in, out, n, ticket, aggr, 0);
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
  const int64_t row = (int64_t)kBlock * VE;
  // Up to 8192 ranges of 2, 4, 8 or 16 rows of 256 vectors.  Default: two launches (range sums,
  // then the scan with every aggregate ready).  GEAR_HIP_SCAN_SINGLE_PASS=1 selects the one-pass
  // kernel with tickets and published aggregates instead (larger ranges, so that all workgroups
  // are resident together).
  // The kernels in which a workgroup waits for another one mark "not published yet" with the
  // word kEmpty, which no fp64 sum of fp32 values can equal but an int64 sum can (-1): int64
  // scans therefore always take the two launches, in which nobody waits, and stop at their limit.
  constexpr bool kMayWait = std::is_same<Acc, double>::value;
  const bool single_pass = kMayWait && env_int("GEAR_HIP_SCAN_SINGLE_PASS", 0) != 0;
  const int64_t cap = single_pass ? 1024 : kMaxRanges;  // the largest ranges may be up to 8192
  if (!single_pass && ceil_div64(n, 2 * row) <= cap)
    return launch_ranges<In, Acc, Out, VE, 2>(in, out, n, ws, st, single_pass, first_changed);
  if (ceil_div64(n, 4 * row) <= cap)
    return launch_ranges<In, Acc, Out, VE, 4>(in, out, n, ws, st, single_pass, first_changed);
  if (ceil_div64(n, 8 * row) <= cap)
    return launch_ranges<In, Acc, Out, VE, 8>(in, out, n, ws, st, single_pass, first_changed);
  if (ceil_div64(n, 16 * row) <= (single_pass ? kMaxRanges : kMaxRangesTwo))
    return launch_ranges<In, Acc, Out, VE, 16>(in, out, n, ws, st, single_pass, first_changed);
  if (!kMayWait) return GEAR_HIP_ERANGE;
  const int64_t tiles = scan_tiles(n, kRows * kBlock * VE);
  uint32_t *ticket = static_cast<uint32_t *>(ws);
  uint64_t *aggr = reinterpret_cast<uint64_t *>(static_cast<char *>(ws) + kHeaderBytes);
  uint64_t *incl = aggr + tiles;
  const int64_t words = 2 * tiles;
  scan_init_kernel<<<dim3((unsigned)ceil_div64(words, kBlock)), dim3(kBlock), 0, st>>>(ticket, aggr,
                                                                                     words);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  scan_kernel<In, Acc, Out, VE><<<dim3((unsigned)tiles), dim3(kBlock), 0, st>>>(in, out, n, ticket,
                                                                              aggr, incl);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
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
constexpr size_t kStaticBytes = kHeaderBytes + (size_t)(kStaticMaxN / (kRows * kBlock * 2)) * 16;
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kStaticBytes];

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch(void **ptr) {
  int dev = -1;
  GEARHIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return GEAR_HIP_ERANGE;
  void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    GEARHIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (p == nullptr) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // every thread finds the same address
  }
  *ptr = p;
  return 0;
}

}  // namespace

int scan_static_init() {
  void *p = nullptr;
  return static_scratch(&p);
}

}  // namespace gearhip

extern "C" int64_t gear_hip_scan_static_max_n(void) { return kStaticMaxN; }

extern "C" int gear_hip_scan_f32_f64_static(const float *in, double *out, int64_t n,
                                            void *stream) {
  if (n < 0) return GEAR_HIP_EINVAL;
  if (n > kStaticMaxN) return GEAR_HIP_ERANGE;
  if (n == 0) return 0;
  void *ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc) return rc;
  static_assert(kStaticBytes >= kHeaderBytes + 16, "scratch holds at least one range");
  if (kStaticBytes < scan_ws_bytes(n)) return GEAR_HIP_ERANGE;
  return launch_scan<float, double, double, 4>(in, out, n, ws, kStaticBytes, as_stream(stream));
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
