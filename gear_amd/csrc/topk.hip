// Top-k of fp32 priorities by radix select + ordered compaction + radix sort, gfx950.
//
// fp32 priorities map to order-preserving uint32 keys.  Three histogram passes (11 + 11 + 10
// bits, LDS histograms, last finished workgroup picks the bin) find the key T of the k-th
// largest priority and how many entries equal to T are still needed.  One compaction pass with a
// decoupled look-back over packed (greater, equal) counts writes the selected entries in index
// order: every entry above T, and the first need_eq entries equal to T -- ties go to the smaller
// index.  For value order the k candidates then go through the stable LSD radix sort on the
// inverted key.
#include "radix_sort.hpp"

namespace gearhip {
namespace {

constexpr int kBlock = 256;
constexpr int kRows = 4;
constexpr int kTile = kBlock * kRows * 4;  // elements per compaction tile
constexpr int kHistBins = 2048;
constexpr int kMaxHistBlocks = 512;

struct State {
  uint32_t prefix[3];  // key bits decided after pass 0, 1, 2 (right-aligned)
  uint32_t k_rem[3];   // entries still to take from the bin picked in that pass
  uint32_t ticket;     // tile ticket of the compaction pass
  uint32_t pad[57];
};
static_assert(sizeof(State) == 256, "State is the 256-byte header of the workspace");

__device__ __forceinline__ uint32_t order_key(float f) {
  uint32_t b = __float_as_uint(f);
  if (b == 0x80000000u) b = 0u;  // -0.0 ranks with +0.0
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

struct Layout {
  size_t hist, desc, ckey, cidx, skey, sidx, tkey, tidx, shist, total;
};

Layout layout(int64_t n, int64_t k) {
  Layout l;
  const int64_t tiles = n > 0 ? ceil_div64(n, kTile) : 0;
  const size_t kk = align_up((size_t)(k > 0 ? k : 1) * 4, 256);
  size_t o = sizeof(State);
  l.hist = o;  o += 3 * kHistBins * sizeof(uint32_t);
  l.desc = o;  o += align_up((size_t)tiles * 8, 256);
  l.ckey = o;  o += kk;
  l.cidx = o;  o += kk;
  l.skey = o;  o += kk;
  l.sidx = o;  o += kk;
  l.tkey = o;  o += kk;
  l.tidx = o;  o += kk;
  l.shist = o; o += radix::hist_bytes(k);
  l.total = o;
  return l;
}

__global__ void zero_kernel(uint32_t *p, int64_t words) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < words) p[i] = 0u;
}

// Every thread of a 256-thread workgroup calls this: walk the histogram of pass PASS from the top
// bin down and stop at the bin that holds the k_rem-th largest remaining key.  The result
// (key prefix after this pass, entries still needed inside that bin) is returned to all threads.
// The kernel that needs the result computes it itself instead of waiting for a launch of its own;
// workgroup 0 also records it in `state` for the kernels after it.
struct Pick {
  uint32_t prefix, k_rem;
};
template <int PASS>
__device__ __forceinline__ Pick pick_bin(int64_t k, State *state, const uint32_t *hist) {
  constexpr int kBinsHere = PASS == 2 ? 1024 : 2048;
  constexpr int kPerThread = kBinsHere / kBlock;
  __shared__ uint32_t wsum[kBlock / kWave];
  __shared__ Pick s_pick;
  const int tid = threadIdx.x;
  const uint32_t prefix = PASS == 0 ? 0u : state->prefix[PASS == 0 ? 0 : PASS - 1];
  const uint32_t k_rem = PASS == 0 ? (uint32_t)k : state->k_rem[PASS == 0 ? 0 : PASS - 1];
  // thread t owns bins top-down: kBinsHere-1 - t*kPerThread - j
  uint32_t c[kPerThread];
  int tsum = 0;
#pragma unroll
  for (int j = 0; j < kPerThread; ++j) {
    c[j] = hist[kBinsHere - 1 - tid * kPerThread - j];
    tsum += (int)c[j];
  }
  const int inc = wave_inclusive_sum(tsum);
  if ((tid & 63) == 63) wsum[tid >> 6] = (uint32_t)inc;
  __syncthreads();
  uint32_t running = (uint32_t)(inc - tsum);
  for (int w = 0; w < (tid >> 6); ++w) running += wsum[w];
#pragma unroll
  for (int j = 0; j < kPerThread; ++j) {
    if (running < k_rem && running + c[j] >= k_rem) {
      const uint32_t bin = (uint32_t)(kBinsHere - 1 - tid * kPerThread - j);
      s_pick.prefix = PASS == 0 ? bin : (PASS == 1 ? ((prefix << 11) | bin) : ((prefix << 10) | bin));
      s_pick.k_rem = k_rem - running;
    }
    running += c[j];
  }
  __syncthreads();
  const Pick r = s_pick;
  if (blockIdx.x == 0 && tid == 0) {
    state->prefix[PASS] = r.prefix;
    state->k_rem[PASS] = r.k_rem;
  }
  return r;
}

// PASS 0: bits 31..21, PASS 1: bits 20..10 of keys whose top 11 bits equal state->prefix,
// PASS 2: bits 9..0 of keys whose top 22 bits equal state->prefix.  Workgroups count into LDS and
// add their non-empty bins to the global histogram of this pass (hist; the previous pass's is
// at hist - kHistBins); the bin of the previous pass is picked by every workgroup for itself.
template <int PASS>
__global__ __launch_bounds__(kBlock) void select_hist_kernel(const float *__restrict__ p,
                                                             int64_t n, int64_t k, State *state,
                                                             uint32_t *hist) {
  constexpr int kBinsHere = PASS == 2 ? 1024 : 2048;
  typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));
  __shared__ uint32_t h[kBinsHere];
  const int tid = threadIdx.x;
  for (int i = tid; i < kBinsHere; i += kBlock) h[i] = 0;
  uint32_t prefix = 0u;
  if (PASS == 1) prefix = pick_bin<0>(k, state, hist - kHistBins).prefix;
  if (PASS == 2) prefix = pick_bin<1>(k, state, hist - kHistBins).prefix;
  __syncthreads();

  auto count = [&](float f) {
    const uint32_t key = order_key(f);
    if (PASS == 0) {
      atomicAdd(&h[key >> 21], 1u);
    } else if (PASS == 1) {
      if ((key >> 21) == prefix) atomicAdd(&h[(key >> 10) & 0x7ffu], 1u);
    } else {
      if ((key >> 10) == prefix) atomicAdd(&h[key & 0x3ffu], 1u);
    }
  };
  const int64_t nvec = n >> 2;
  for (int64_t v = (int64_t)blockIdx.x * kBlock + tid; v < nvec; v += (int64_t)gridDim.x * kBlock) {
    const f4 q = *reinterpret_cast<const f4 *>(p + (v << 2));
    count(q[0]);
    count(q[1]);
    count(q[2]);
    count(q[3]);
  }
  if (blockIdx.x == 0 && tid < (int)(n & 3)) count(p[(nvec << 2) + tid]);
  __syncthreads();
  for (int i = tid; i < kBinsHere; i += kBlock)
    if (h[i]) atomicAdd(&hist[i], h[i]);
}

// packed per-tile descriptor: status (2 bits) | greater (31 bits) | equal (31 bits)
constexpr uint64_t kStatusAggregate = 1ull << 62;
constexpr uint64_t kStatusInclusive = 2ull << 62;
constexpr uint64_t kCountMask = (1ull << 62) - 1;

template <bool DIRECT>
__global__ __launch_bounds__(kBlock) void compact_kernel(
    const float *__restrict__ p, int64_t n, int64_t k, State *state, const uint32_t *hist2,
    uint64_t *desc,
    uint32_t *__restrict__ ckey, uint32_t *__restrict__ cidx, float *__restrict__ values_out,
    int64_t *__restrict__ indices_out) {
  typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));
  constexpr int kWaves = kBlock / kWave;
  __shared__ int wtot[kRows][kWaves];
  __shared__ uint64_t s_excl;
  __shared__ uint32_t s_tile;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) s_tile = atomicAdd(&state->ticket, 1u);
  __syncthreads();
  const int64_t tile = s_tile;
  const int64_t base = tile * kTile;
  const Pick pk = pick_bin<2>(k, state, hist2);
  const uint32_t thr = pk.prefix;
  const uint32_t need_eq = pk.k_rem;

  uint32_t key[kRows][4];
  int s[kRows];  // packed counts of the thread's vector: greater << 16 | equal
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int64_t e0 = base + ((int64_t)r * kBlock + tid) * 4;
    float q[4];
    if (e0 + 4 <= n) {
      const f4 v = *reinterpret_cast<const f4 *>(p + e0);
      q[0] = v[0]; q[1] = v[1]; q[2] = v[2]; q[3] = v[3];
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) q[j] = (e0 + j < n) ? p[e0 + j] : 0.0f;
    }
    s[r] = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      key[r][j] = order_key(q[j]);
      if (e0 + j < n) s[r] += key[r][j] > thr ? (1 << 16) : (key[r][j] == thr ? 1 : 0);
    }
  }
  int wexcl[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int inc = wave_inclusive_sum(s[r]);
    wexcl[r] = wave_shift_up1(inc);
    if (lane == kWave - 1) wtot[r][wave] = inc;
  }
  __syncthreads();
  int tile_total = 0;
  int mybase[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    int acc = tile_total;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      if (w == wave) mybase[r] = acc + wexcl[r];
      acc += wtot[r][w];
    }
    tile_total = acc;
  }
  const uint64_t tile_packed =
      ((uint64_t)((uint32_t)tile_total >> 16) << 31) | (uint64_t)((uint32_t)tile_total & 0xffffu);

  if (wave == 0) {
    uint64_t excl = 0;
    if (tile == 0) {
      if (lane == 0) store_agent(&desc[0], kStatusInclusive | tile_packed);
    } else {
      if (lane == 0) store_agent(&desc[tile], kStatusAggregate | tile_packed);
      int64_t look = tile - 1;
      while (true) {
        const int64_t idx = look - lane;
        uint64_t v = kStatusInclusive;  // tiles before the first one: inclusive, zero counts
        if (idx >= 0) v = load_agent(&desc[idx]);
        const bool has_incl = (v >> 62) == 2;
        const bool ready = (v >> 62) != 0;
        const uint64_t bi = wave_ballot(has_incl), br = wave_ballot(ready);
        const int first = bi ? (__ffsll((unsigned long long)bi) - 1) : kWave;
        const uint64_t need = first >= 63 ? ~0ull : ((2ull << first) - 1ull);
        if ((br & need) != need) {
          __builtin_amdgcn_s_sleep(1);
          continue;
        }
        const int64_t c = lane <= first ? (int64_t)(v & kCountMask) : 0;
        excl += (uint64_t)wave_sum(c);
        if (first < kWave) break;
        look -= kWave;
      }
      if (lane == 0) store_agent(&desc[tile], kStatusInclusive | (excl + tile_packed));
    }
    if (lane == 0) s_excl = excl;
  }
  __syncthreads();
  const uint32_t gt0 = (uint32_t)(s_excl >> 31);
  const uint32_t eq0 = (uint32_t)(s_excl & 0x7fffffffu);

#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int64_t e0 = base + ((int64_t)r * kBlock + tid) * 4;
    uint32_t gt = gt0 + ((uint32_t)mybase[r] >> 16);
    uint32_t eq = eq0 + ((uint32_t)mybase[r] & 0xffffu);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (e0 + j < n) {
        const bool is_gt = key[r][j] > thr, is_eq = key[r][j] == thr;
        if (is_gt || (is_eq && eq < need_eq)) {
          const uint32_t pos = gt + (eq < need_eq ? eq : need_eq);
          if (DIRECT) {
            indices_out[pos] = e0 + j;
            if (values_out) values_out[pos] = p[e0 + j];
          } else {
            ckey[pos] = ~key[r][j];
            cidx[pos] = (uint32_t)(e0 + j);
          }
        }
        gt += is_gt;
        eq += is_eq;
      }
    }
  }
}

// Range variant of the compaction (cf. the range variant of the prefix sum): with at most
// kMaxRanges workgroups every workgroup publishes its packed (greater, equal) count and takes the
// sum of all earlier ranges' counts; no chain of inclusive values across the XCDs.
constexpr int kMaxRanges = 2048;
constexpr uint64_t kRangeReady = 1ull << 63;

template <bool DIRECT, int NR>
__global__ __launch_bounds__(kBlock) void compact_ranges_kernel(
    const float *__restrict__ p, int64_t n, int64_t k, State *state, const uint32_t *hist2,
    uint64_t *desc,
    uint32_t *__restrict__ ckey, uint32_t *__restrict__ cidx, float *__restrict__ values_out,
    int64_t *__restrict__ indices_out) {
  typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));
  constexpr int kWaves = kBlock / kWave;
  constexpr int kElems = NR * kBlock * 4;
  __shared__ int wtot[NR][kWaves];
  __shared__ int64_t red[kWaves];
  __shared__ uint32_t s_tile;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) s_tile = atomicAdd(&state->ticket, 1u);
  __syncthreads();
  const int64_t tile = s_tile;
  const int64_t base = tile * kElems;
  const Pick pk = pick_bin<2>(k, state, hist2);
  const uint32_t thr = pk.prefix;
  const uint32_t need_eq = pk.k_rem;

  float q[NR][4];
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int64_t e0 = base + ((int64_t)r * kBlock + tid) * 4;
    if (e0 + 4 <= n) {
      const f4 v = *reinterpret_cast<const f4 *>(p + e0);
      q[r][0] = v[0]; q[r][1] = v[1]; q[r][2] = v[2]; q[r][3] = v[3];
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) q[r][j] = (e0 + j < n) ? p[e0 + j] : 0.0f;
    }
  }
  int s[NR];  // packed counts of the thread's vector: greater << 16 | equal
  int64_t tsum = 0;  // greater << 31 | equal over the thread's vectors
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int64_t e0 = base + ((int64_t)r * kBlock + tid) * 4;
    s[r] = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t key = order_key(q[r][j]);
      if (e0 + j < n) s[r] += key > thr ? (1 << 16) : (key == thr ? 1 : 0);
    }
    tsum += ((int64_t)(s[r] >> 16) << 31) | (int64_t)(s[r] & 0xffff);
  }
  {
    const int64_t w = wave_sum(tsum);
    if (lane == 0) red[wave] = w;
    __syncthreads();
    if (tid == 0)
      store_agent(&desc[tile], kRangeReady | (uint64_t)(red[0] + red[1] + red[2] + red[3]));
  }
  int wexcl[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int inc = wave_inclusive_sum(s[r]);
    wexcl[r] = wave_shift_up1(inc);
    if (lane == kWave - 1) wtot[r][wave] = inc;
  }
  int64_t part = 0;
  for (int64_t j = tid; j < tile; j += kBlock) {
    uint64_t v = load_agent(&desc[j]);
    while (!(v & kRangeReady)) {
      __builtin_amdgcn_s_sleep(1);
      v = load_agent(&desc[j]);
    }
    part += (int64_t)(v & ~kRangeReady);
  }
  const int64_t pw = wave_sum(part);
  __syncthreads();
  if (lane == 0) red[wave] = pw;
  __syncthreads();
  const int64_t excl = red[0] + red[1] + red[2] + red[3];
  uint32_t gt_row = (uint32_t)(excl >> 31), eq_row = (uint32_t)(excl & 0x7fffffff);

#pragma unroll
  for (int r = 0; r < NR; ++r) {
    int before = 0, mine = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      if (w == wave) mine = before + wexcl[r];
      before += wtot[r][w];
    }
    const int64_t e0 = base + ((int64_t)r * kBlock + tid) * 4;
    uint32_t gt = gt_row + ((uint32_t)mine >> 16);
    uint32_t eq = eq_row + ((uint32_t)mine & 0xffffu);
    gt_row += (uint32_t)before >> 16;
    eq_row += (uint32_t)before & 0xffffu;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (e0 + j < n) {
        const uint32_t key = order_key(q[r][j]);
        const bool is_gt = key > thr, is_eq = key == thr;
        if (is_gt || (is_eq && eq < need_eq)) {
          const uint32_t pos = gt + (eq < need_eq ? eq : need_eq);
          if (DIRECT) {
            indices_out[pos] = e0 + j;
            if (values_out) values_out[pos] = q[r][j];
          } else {
            ckey[pos] = ~key;
            cidx[pos] = (uint32_t)(e0 + j);
          }
        }
        gt += is_gt;
        eq += is_eq;
      }
    }
  }
}

__global__ __launch_bounds__(kBlock) void emit_kernel(const float *__restrict__ p,
                                                      const uint32_t *__restrict__ sidx, int64_t k,
                                                      float *__restrict__ values_out,
                                                      int64_t *__restrict__ indices_out) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= k) return;
  const uint32_t i = sidx[j];
  indices_out[j] = (int64_t)i;
  if (values_out) values_out[j] = p[i];
}

}  // namespace
}  // namespace gearhip

using namespace gearhip;

extern "C" size_t gear_hip_topk_workspace_bytes(int64_t n, int64_t k) { return layout(n, k).total; }

extern "C" int gear_hip_topk_f32(const float *priorities, int64_t n, int64_t k,
                                 int sorted_by_value, float *values_out, int64_t *indices_out,
                                 void *workspace, size_t workspace_bytes, void *stream) {
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
  uint32_t *hist = reinterpret_cast<uint32_t *>(ws + l.hist);
  uint64_t *desc = reinterpret_cast<uint64_t *>(ws + l.desc);
  hipStream_t st = as_stream(stream);

  const int64_t zero_words = (int64_t)(l.ckey / 4);  // header + histograms + descriptors
  zero_kernel<<<dim3((unsigned)ceil_div64(zero_words, 256)), dim3(256), 0, st>>>(
      reinterpret_cast<uint32_t *>(ws), zero_words);
  int64_t hblocks = ceil_div64(n, (int64_t)kBlock * 4 * 4);
  if (hblocks < 1) hblocks = 1;
  if (hblocks > kMaxHistBlocks) hblocks = kMaxHistBlocks;
  const dim3 hgrid((unsigned)hblocks), block(kBlock);
  select_hist_kernel<0><<<hgrid, block, 0, st>>>(priorities, n, k, state, hist);
  select_hist_kernel<1><<<hgrid, block, 0, st>>>(priorities, n, k, state, hist + kHistBins);
  select_hist_kernel<2><<<hgrid, block, 0, st>>>(priorities, n, k, state, hist + 2 * kHistBins);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();

  uint32_t *ckey = reinterpret_cast<uint32_t *>(ws + l.ckey);
  uint32_t *cidx = reinterpret_cast<uint32_t *>(ws + l.cidx);
  const bool direct = !sorted_by_value;
  const int64_t row = (int64_t)kBlock * 4;
#define GEARHIP_COMPACT_RANGES(NR)                                                              \
  do {                                                                                          \
    const unsigned g = (unsigned)ceil_div64(n, (NR) * row);                                     \
    if (direct)                                                                                 \
      compact_ranges_kernel<true, NR><<<dim3(g), block, 0, st>>>(priorities, n, k, state, hist + 2 * kHistBins, desc,    \
                                                                 ckey, cidx, values_out,        \
                                                                 indices_out);                  \
    else                                                                                        \
      compact_ranges_kernel<false, NR><<<dim3(g), block, 0, st>>>(priorities, n, k, state, hist + 2 * kHistBins, desc,   \
                                                                  ckey, cidx, values_out,       \
                                                                  indices_out);                 \
  } while (0)
  if (ceil_div64(n, 4 * row) <= 1024) {
    GEARHIP_COMPACT_RANGES(4);
  } else if (ceil_div64(n, 8 * row) <= 1024) {
    GEARHIP_COMPACT_RANGES(8);
  } else if (ceil_div64(n, 16 * row) <= kMaxRanges) {
    GEARHIP_COMPACT_RANGES(16);
  } else {
    const int64_t tiles = ceil_div64(n, kTile);
    if (direct)
      compact_kernel<true><<<dim3((unsigned)tiles), block, 0, st>>>(priorities, n, k, state, hist + 2 * kHistBins, desc, ckey,
                                                                    cidx, values_out, indices_out);
    else
      compact_kernel<false><<<dim3((unsigned)tiles), block, 0, st>>>(priorities, n, k, state, hist + 2 * kHistBins, desc,
                                                                     ckey, cidx, values_out,
                                                                     indices_out);
  }
#undef GEARHIP_COMPACT_RANGES
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  if (direct) return 0;
  uint32_t *skey = reinterpret_cast<uint32_t *>(ws + l.skey);
  uint32_t *sidx = reinterpret_cast<uint32_t *>(ws + l.sidx);
  int rc = radix::sort_pairs<uint32_t, uint32_t>(
      ckey, skey, cidx, sidx, reinterpret_cast<uint32_t *>(ws + l.tkey),
      reinterpret_cast<uint32_t *>(ws + l.tidx), k, 0, 32,
      reinterpret_cast<uint32_t *>(ws + l.shist), st);
  if (rc) return rc;
  emit_kernel<<<dim3((unsigned)ceil_div64(k, kBlock)), block, 0, st>>>(priorities, sidx, k,
                                                                      values_out, indices_out);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}
